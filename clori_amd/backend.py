"""Thin object wrapper over the C ABI, shaped like the reference's backend API so a
test reads like the reference's own (open -> tensor_alloc/write -> operation -> read).

Every numerical operation is executed by libyvex_rocm.so on the GPU; nothing here
computes attention and nothing here falls back to the host.
"""
import ctypes as C

import numpy as np

from . import binding as B


class YvexError(RuntimeError):
    """A refused call: carries the reference status code, the stage and the message."""

    def __init__(self, code, where, message):
        super().__init__("%s at %s: %s" % (B_status_name(code), where, message))
        self.code = code
        self.where = where
        self.message = message


_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        _LIB = B.load()
    return _LIB


def B_status_name(code):
    return lib().yvex_status_name(code).decode()


def _check(rc, err):
    if rc != B.YVEX_OK:
        raise YvexError(rc, err.where.decode(errors="replace"), err.message.decode(errors="replace"))


_NP_DTYPE = {B.DTYPE_F32: np.float32, B.DTYPE_BF16: np.uint16, B.DTYPE_F16: np.float16,
             B.DTYPE_I32: np.int32, B.DTYPE_I8: np.int8, B.DTYPE_I64: np.int64}


class Tensor:
    """One backend-owned device tensor (struct yvex_device_tensor)."""

    def __init__(self, backend, handle, dtype, shape):
        self.backend = backend
        self.handle = handle
        self.dtype = dtype
        self.shape = tuple(shape)

    @property
    def nbytes(self):
        return int(lib().yvex_device_tensor_bytes(self.handle))

    @property
    def is_written(self):
        return bool(lib().yvex_device_tensor_is_written(self.handle))

    def write(self, array):
        array = np.ascontiguousarray(array)
        err = B.Error()
        _check(lib().yvex_backend_tensor_write(self.backend.handle, self.handle,
                                               array.ctypes.data, array.nbytes, C.byref(err)), err)
        self._keep = None
        return self

    def read(self, np_dtype=None, shape=None):
        np_dtype = np_dtype or _NP_DTYPE[self.dtype]
        out = np.empty(self.nbytes // np.dtype(np_dtype).itemsize, dtype=np_dtype)
        err = B.Error()
        _check(lib().yvex_backend_tensor_read(self.backend.handle, self.handle, out.ctypes.data,
                                              out.nbytes, C.byref(err)), err)
        return out.reshape(shape or self.shape)

    def zero(self):
        err = B.Error()
        _check(lib().yvex_backend_tensor_zero(self.backend.handle, self.handle, C.byref(err)), err)

    def copy_from_async(self, source):
        """The same copy put on the backend's stream and not waited for
        (yvex_backend_tensor_copy_async)."""
        err = B.Error()
        _check(lib().yvex_backend_tensor_copy_async(self.backend.handle, self.handle, source.handle,
                                                    C.byref(err)), err)

    def copy_from_shared_async(self, source):
        """Copy from a tensor of another backend with the same physical owner, ordered by
        events between the two streams (yvex_backend_tensor_copy_shared_async)."""
        err = B.Error()
        _check(lib().yvex_backend_tensor_copy_shared_async(self.backend.handle, self.handle,
                                                           source.handle, C.byref(err)), err)

    def copy_from(self, source):
        """Device-to-device copy of a tensor with the same descriptor."""
        err = B.Error()
        _check(lib().yvex_backend_tensor_copy(self.backend.handle, self.handle, source.handle,
                                              C.byref(err)), err)

    # -- tensors over a reserved address range -----------------------------
    @property
    def resident_bytes(self):
        return int(self.handle.contents.resident_bytes)

    def commit(self, byte_offset, nbytes):
        """Backs the granules under [byte_offset, byte_offset + nbytes) that are not backed
        yet (zero-filled) and returns how many bytes that added."""
        delta, err = C.c_ulonglong(0), B.Error()
        _check(lib().yvex_backend_tensor_commit_range(self.backend.handle, self.handle, byte_offset,
                                                      nbytes, C.byref(delta), C.byref(err)), err)
        return delta.value

    def decommit(self):
        """Returns every committed page, keeps the address range; returns the bytes released."""
        released, err = C.c_ulonglong(0), B.Error()
        _check(lib().yvex_backend_tensor_decommit(self.backend.handle, self.handle,
                                                  C.byref(released), C.byref(err)), err)
        return released.value

    def release(self):
        if self.handle:
            err = B.Error()
            ptr = B.TensorP(self.handle.contents)
            rc = lib().yvex_backend_tensor_release(self.backend.handle, C.byref(ptr), C.byref(err))
            _check(rc, err)
            self.handle = None

    def view(self, byte_offset, dtype, shape):
        """Sub-view made the way the reference does it: copy the struct, offset `data`
        (src/backend/core.c:1763-1778).  The view borrows this tensor's storage."""
        view = B.DeviceTensor()
        C.memmove(C.byref(view), self.handle, C.sizeof(B.DeviceTensor))
        count = int(np.prod(shape))
        view.dtype = dtype
        view.rank = len(shape)
        for i in range(4):
            view.dims[i] = shape[i] if i < len(shape) else 0
        view.bytes = count * B.DTYPE_BYTES[dtype]
        view.data = self.handle.contents.data + byte_offset
        tensor = Tensor(self.backend, C.pointer(view), dtype, shape)
        tensor._parent = self
        return tensor


class Backend:
    """struct yvex_backend of kind ROCM."""

    def __init__(self, device=None, memory_limit_bytes=0, kind=B.KIND_ROCM, shared_with=None):
        """shared_with: a primary Backend; the new one is a session backend on its device
        (yvex_backend_open_shared_rocm)."""
        self.handle = C.c_void_p()
        err = B.Error()
        if shared_with is not None:
            _check(lib().yvex_backend_open_shared_rocm(C.byref(self.handle), shared_with.handle,
                                                       memory_limit_bytes, C.byref(err)), err)
        else:
            options = B.BackendOptions(kind, device.encode() if device else None, memory_limit_bytes)
            _check(lib().yvex_backend_open(C.byref(self.handle), C.byref(options), C.byref(err)), err)
        self.tensors = []

    # -- lifecycle --------------------------------------------------------
    def close(self):
        if self.handle:
            for tensor in self.tensors:
                if tensor.handle:
                    lib().yvex_backend_tensor_free(self.handle, tensor.handle)
                    tensor.handle = None
            err = B.Error()
            rc = lib().yvex_backend_close_checked(C.byref(self.handle), C.byref(err))
            _check(rc, err)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def status(self):
        return int(lib().yvex_backend_status_of(self.handle))

    def sync(self):
        err = B.Error()
        _check(lib().yvex_backend_sync(self.handle, C.byref(err)), err)

    def memory_stats(self):
        out, err = B.MemoryStats(), B.Error()
        _check(lib().yvex_backend_get_memory_stats(self.handle, C.byref(out), C.byref(err)), err)
        return out

    def device_info(self):
        out, err = B.DeviceInfo(), B.Error()
        _check(lib().yvex_backend_get_device_info(self.handle, C.byref(out), C.byref(err)), err)
        return out

    def report(self):
        out, err = B.RocmReport(), B.Error()
        _check(lib().yvex_backend_rocm_report_get(self.handle, C.byref(out), C.byref(err)), err)
        return out

    def query_capability(self, variant):
        out, err = B.CapabilityResult(), B.Error()
        _check(lib().yvex_backend_query_capability(self.handle, variant, C.byref(out),
                                                   C.byref(err)), err)
        return out

    def supports(self, capability):
        return bool(lib().yvex_backend_supports(self.handle, capability))

    def set_completion_mode(self, mode):
        err = B.Error()
        _check(lib().yvex_backend_rocm_completion_mode_set(self.handle, mode, C.byref(err)), err)

    def timing_begin(self):
        err = B.Error()
        _check(lib().yvex_backend_rocm_timing_begin(self.handle, C.byref(err)), err)

    def timing_end(self):
        ms, err = C.c_double(0.0), B.Error()
        _check(lib().yvex_backend_rocm_timing_end(self.handle, C.byref(ms), C.byref(err)), err)
        return ms.value

    def bandwidth_probe(self):
        """Measured streaming-read and copy rates of the device (kept after the first call)."""
        evidence, err = B.BandwidthEvidence(), B.Error()
        _check(lib().yvex_backend_bandwidth_probe(self.handle, C.byref(evidence), C.byref(err)), err)
        return evidence

    # -- recorded launch sequences -------------------------------------
    def graph_begin(self):
        err = B.Error()
        _check(lib().yvex_backend_rocm_graph_begin(self.handle, C.byref(err)), err)

    def graph_end(self):
        """Ends the recording and returns the handle of the recorded sequence."""
        graph, err = C.c_void_p(), B.Error()
        _check(lib().yvex_backend_rocm_graph_end(self.handle, C.byref(graph), C.byref(err)), err)
        return graph

    def graph_launch(self, graph):
        facts, err = B.OperationFacts(), B.Error()
        _check(lib().yvex_backend_rocm_graph_launch(self.handle, graph, C.byref(facts),
                                                    C.byref(err)), err)
        return facts

    def graph_release(self, graph):
        err = B.Error()
        _check(lib().yvex_backend_rocm_graph_release(self.handle, C.byref(graph), C.byref(err)), err)

    def kernel_probe_begin(self, kernel):
        """Brackets every launch of the named bundle kernel with its own event pair."""
        err = B.Error()
        _check(lib().yvex_backend_rocm_kernel_probe_begin(self.handle, kernel.encode(),
                                                          C.byref(err)), err)

    def kernel_probe_end(self):
        """Returns (measured launches, summed device milliseconds)."""
        count, ms, err = C.c_uint(0), C.c_double(0.0), B.Error()
        _check(lib().yvex_backend_rocm_kernel_probe_end(self.handle, C.byref(count), C.byref(ms),
                                                        C.byref(err)), err)
        return count.value, ms.value

    # -- tensors ----------------------------------------------------------
    def tensor(self, name, dtype, shape, data=None, nbytes=None):
        desc = B.TensorDesc()
        desc.name = name.encode()
        desc.dtype = dtype
        desc.rank = len(shape)
        for i, dim in enumerate(shape):
            desc.dims[i] = dim
        desc.bytes = nbytes if nbytes is not None else int(np.prod(shape)) * B.DTYPE_BYTES[dtype]
        handle, err = B.TensorP(), B.Error()
        _check(lib().yvex_backend_tensor_alloc(self.handle, C.byref(desc), C.byref(handle),
                                               C.byref(err)), err)
        tensor = Tensor(self, handle, dtype, shape)
        self.tensors.append(tensor)
        if data is not None:
            tensor.write(data)
        return tensor

    def reserve(self, name, dtype, shape, nbytes=None):
        """A tensor that owns a device address range and no memory yet (Tensor.commit backs
        parts of it).  The granule size is kept as `tensor.granularity`."""
        desc = B.TensorDesc()
        desc.name = name.encode()
        desc.dtype = dtype
        desc.rank = len(shape)
        for i, dim in enumerate(shape):
            desc.dims[i] = dim
        desc.bytes = nbytes if nbytes is not None else int(np.prod(shape)) * B.DTYPE_BYTES[dtype]
        handle, granularity, err = B.TensorP(), C.c_ulonglong(0), B.Error()
        _check(lib().yvex_backend_tensor_reserve(self.handle, C.byref(desc), C.byref(handle),
                                                 C.byref(granularity), C.byref(err)), err)
        tensor = Tensor(self, handle, dtype, shape)
        tensor.granularity = granularity.value
        self.tensors.append(tensor)
        return tensor

    def workspace_attach(self, tensor, generation=1):
        err = B.Error()
        _check(lib().yvex_backend_workspace_attach(self.handle, tensor.handle, generation,
                                                   C.byref(err)), err)

    def workspace_detach(self):
        lib().yvex_backend_workspace_detach(self.handle)

    # -- operations ---------------------------------------------------------
    def op_attention(self, query, keys, values, seq_len, position, scale, causal, score, prob, out):
        err = B.Error()
        _check(lib().yvex_backend_op_attention(self.handle, query.handle, keys.handle,
                                               values.handle, seq_len, position, scale,
                                               int(causal), score.handle, prob.handle, out.handle,
                                               C.byref(err)), err)

    def transformer_operations(self):
        ops = lib().yvex_backend_transformer_operations_get(self.handle)
        return ops.contents if ops else None

    def rocm_attention_operations(self):
        ops = lib().yvex_backend_rocm_attention_operations_get(self.handle)
        return ops.contents if ops else None

    @staticmethod
    def attention_requirement(query_tokens, kv_tokens, query_heads, kv_heads, head_dim,
                              causal=True, query_start=0, dtype=B.DTYPE_F32,
                              contract=B.NUMERIC_EXACT_F32, q_stride=0, k_stride=0, v_stride=0,
                              deterministic=1):
        r = B.AttentionRequirement()
        r.query_tokens, r.key_value_tokens, r.query_start = query_tokens, kv_tokens, query_start
        r.query_heads, r.key_value_heads, r.head_dimension = query_heads, kv_heads, head_dim
        r.query_token_stride, r.key_token_stride, r.value_token_stride = q_stride, k_stride, v_stride
        r.query_dtype = r.key_dtype = r.value_dtype = r.output_dtype = dtype
        r.layout = B.LAYOUT_TOKEN_HEAD_DIM
        r.mask = B.MASK_CAUSAL if causal else B.MASK_FULL
        r.numeric_contract = contract
        r.deterministic = deterministic
        return r

    def attention_workspace_required(self, requirement):
        ops = self.transformer_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "transformer_operations", "not published")
        out, err = B.ull(0), B.Error()
        _check(ops.attention_workspace_required(C.byref(requirement), C.byref(out), C.byref(err)),
               err)
        return out.value

    def attention_execute(self, requirement, query, key, value, output, lse=None, gate=None):
        ops = self.transformer_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "transformer_operations", "not published")
        request = B.AttentionRequest(requirement, query.handle, key.handle, value.handle,
                                     output.handle)
        facts, err = B.OperationFacts(), B.Error()
        if gate is not None:
            epilogue = B.AttentionEpilogue(gate.handle)
            rc = self.rocm_attention_operations().attention_execute_fused(
                self.handle, C.byref(request), C.byref(epilogue), lse.handle if lse else None,
                C.byref(facts), C.byref(err))
        elif lse is None:
            rc = ops.attention_execute(self.handle, C.byref(request), C.byref(facts), C.byref(err))
        else:
            rocm = self.rocm_attention_operations()
            rc = rocm.attention_execute_lse(self.handle, C.byref(request), lse.handle,
                                            C.byref(facts), C.byref(err))
        _check(rc, err)
        return facts

    def _elementwise(self, slot, *arguments):
        ops = self.transformer_operations()
        if ops is None or not getattr(ops, slot):
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "transformer_operations", "not published")
        facts, err = B.OperationFacts(), B.Error()
        _check(getattr(ops, slot)(self.handle, *arguments, C.byref(facts), C.byref(err)), err)
        return facts

    def rotary_half_f32(self, values, cosines, sines, tokens, heads, head_dim, rotary_dim):
        """The reference's rotary_half_f32 slot: plain F32 rotate-half of `values` in place."""
        return self._elementwise("rotary_half_f32", values.handle, cosines.handle, sines.handle,
                                 tokens, heads, head_dim, rotary_dim)

    def split_interleaved_two_f32(self, source, first, second, rows, heads, head_dim):
        return self._elementwise("split_interleaved_two_f32", source.handle, first.handle,
                                 second.handle, rows, heads, head_dim)

    def sigmoid_product_bf16(self, values, gate, output, count):
        return self._elementwise("sigmoid_product_bf16", values.handle, gate.handle, output.handle,
                                 count)

    def bf16_round(self, values, count):
        return self._elementwise("bf16_round", values.handle, count)

    @staticmethod
    def paged_requirement(sessions, query_heads, kv_heads, head_dim, page_tokens, pool_pages,
                          table_stride, max_context, storage=B.KV_BF16,
                          contract=B.NUMERIC_BF16_F32_ACCUMULATE, deterministic=1):
        r = B.PagedDecodeRequirement()
        r.sessions, r.query_heads, r.key_value_heads = sessions, query_heads, kv_heads
        r.head_dimension, r.page_tokens, r.pool_pages = head_dim, page_tokens, pool_pages
        r.page_table_stride, r.max_context_tokens = table_stride, max_context
        r.kv_storage, r.numeric_contract, r.deterministic = storage, contract, deterministic
        return r

    def paged_decode_workspace_required(self, requirement):
        out, err = B.ull(0), B.Error()
        ops = self.rocm_attention_operations()
        _check(ops.paged_decode_workspace_required(C.byref(requirement), C.byref(out),
                                                   C.byref(err)), err)
        return out.value

    def paged_decode_execute(self, requirement, query, key_pages, value_pages, page_table,
                             context, output, lse=None, gate=None):
        ops = self.rocm_attention_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "rocm_attention_operations", "not published")
        request = B.PagedDecodeRequest(requirement, query.handle, key_pages.handle,
                                       value_pages.handle, page_table.handle, context.handle,
                                       output.handle, lse.handle if lse else None)
        facts, err = B.OperationFacts(), B.Error()
        if gate is not None:
            epilogue = B.AttentionEpilogue(gate.handle)
            rc = ops.paged_decode_execute_fused(self.handle, C.byref(request), C.byref(epilogue),
                                                C.byref(facts), C.byref(err))
        else:
            rc = ops.paged_decode_execute(self.handle, C.byref(request), C.byref(facts),
                                          C.byref(err))
        _check(rc, err)
        return facts

    def paged_decode_execute_static(self, requirement, query, key_pages, value_pages, page_table,
                                    context, output, lse=None):
        """paged_decode_execute through the exported entry point that allocates nothing."""
        request = B.PagedDecodeRequest(requirement, query.handle, key_pages.handle,
                                       value_pages.handle, page_table.handle, context.handle,
                                       output.handle, lse.handle if lse else None)
        facts, err = B.OperationFacts(), B.Error()
        _check(lib().yvex_backend_rocm_paged_decode_execute_static(
            self.handle, C.byref(request), C.byref(facts), C.byref(err)), err)
        return facts

    @staticmethod
    def mla_requirement(batch, heads, key_dim, value_dim, page_tokens, pool_pages, table_stride,
                        max_context, contract=B.NUMERIC_BF16_F32_ACCUMULATE, deterministic=1,
                        sliding_window=0, compressed_pool_pages=0, compressed_table_stride=0,
                        max_compressed_tokens=0, compressed_selected_stride=0,
                        output_inverse_rope=None, scale=0.0):
        """output_inverse_rope: optional dict(rope_dimensions, theta[, scaling_factor,
        original_context, beta_fast, beta_slow]) rotating the published rows back by the query
        token's position; scale: softmax scale, 0 = 1 / sqrt(key_dim)."""
        r = B.MlaDecodeRequirement()
        r.batch, r.heads, r.key_dimension, r.value_dimension = batch, heads, key_dim, value_dim
        r.page_tokens, r.pool_pages, r.page_table_stride = page_tokens, pool_pages, table_stride
        r.max_context_tokens, r.numeric_contract, r.deterministic = max_context, contract, deterministic
        r.sliding_window = sliding_window
        r.compressed_pool_pages = compressed_pool_pages
        r.compressed_page_table_stride = compressed_table_stride
        r.max_compressed_tokens = max_compressed_tokens
        r.compressed_selected_stride = compressed_selected_stride
        for name, value in (output_inverse_rope or {}).items():
            setattr(r.output_inverse_rope, name, value)
        r.scale = scale
        return r

    def mla_decode_workspace_required(self, requirement):
        out, err = B.ull(0), B.Error()
        ops = self.rocm_attention_operations()
        _check(ops.mla_decode_workspace_required(C.byref(requirement), C.byref(out),
                                                 C.byref(err)), err)
        return out.value

    def mla_decode_execute(self, requirement, query, latent_pages, page_table, context, output,
                           lse=None, sinks=None, compressed=None, output_positions=None):
        """compressed: optional (pages, page table, row counts[, selected row lists]) device
        tensors; output_positions: optional I64 [batch] query token positions for the output
        rotation."""
        ops = self.rocm_attention_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "rocm_attention_operations", "not published")
        request = B.MlaDecodeRequest(requirement, query.handle, latent_pages.handle,
                                     page_table.handle, context.handle, output.handle,
                                     lse.handle if lse else None,
                                     sinks.handle if sinks else None,
                                     *(x.handle for x in (compressed or (None, None, None))
                                       if x is not None))
        if output_positions is not None:
            request.output_positions = output_positions.handle
        facts, err = B.OperationFacts(), B.Error()
        _check(ops.mla_decode_execute(self.handle, C.byref(request), C.byref(facts),
                                      C.byref(err)), err)
        return facts


    # -- KV page writer ---------------------------------------------------
    def kv_append_execute(self, key, value, row_start, position_start, token_count, page_table,
                          k_pool, v_pool, kv_heads, pool_pages, max_tokens_per_session,
                          storage=B.KV_BF16, cosine=None, sine=None, rotary_dimension=0,
                          head_dimension=128, page_tokens=16, rotary_mode=B.ROTARY_BF16_STAGED):
        """Writes the new rows into the paged pools; all arguments are device tensors."""
        ops = self.rocm_attention_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "rocm_attention_operations", "not published")
        r = B.KvAppendRequirement()
        r.sessions = row_start.shape[0]
        r.total_tokens = key.shape[0]
        r.max_tokens_per_session = max_tokens_per_session
        r.key_value_heads, r.head_dimension, r.page_tokens = kv_heads, head_dimension, page_tokens
        r.pool_pages, r.page_table_stride = pool_pages, page_table.shape[1]
        r.rotary_dimension, r.storage, r.rotary_mode = rotary_dimension, storage, rotary_mode
        request = B.KvAppendRequest(r, key.handle, value.handle,
                                    cosine.handle if cosine else None,
                                    sine.handle if sine else None, row_start.handle,
                                    position_start.handle, token_count.handle, page_table.handle,
                                    k_pool.handle, v_pool.handle)
        facts, err = B.OperationFacts(), B.Error()
        _check(ops.kv_append_execute(self.handle, C.byref(request), C.byref(facts), C.byref(err)),
               err)
        return facts


    def history_append_execute(self, key, value, key_history, value_history, first_row, kv_heads,
                               head_dimension=128, cosine=None, sine=None, rotary_dimension=0,
                               key_token_stride=0, value_token_stride=0,
                               rotary_mode=B.ROTARY_BF16_STAGED, query=None, query_heads=0):
        """Writes the new rows (keys rotated) into rows first_row.. of the token-major K and V
        history views; all tensor arguments are device tensors.  With query and query_heads
        the same launch rotates the [tokens][query_heads][d] query tensor where it lies."""
        ops = self.rocm_attention_operations()
        if ops is None:
            raise YvexError(B.YVEX_ERR_UNSUPPORTED, "rocm_attention_operations", "not published")
        r = B.HistoryAppendRequirement()
        r.tokens, r.first_row = key.shape[0], first_row
        r.key_value_heads, r.head_dimension = kv_heads, head_dimension
        r.rotary_dimension = rotary_dimension
        r.key_token_stride, r.value_token_stride = key_token_stride, value_token_stride
        r.rotary_mode = rotary_mode
        r.query_heads = query_heads
        request = B.HistoryAppendRequest(r, key.handle, value.handle,
                                         cosine.handle if cosine else None,
                                         sine.handle if sine else None, key_history.handle,
                                         value_history.handle, query.handle if query else None)
        facts, err = B.OperationFacts(), B.Error()
        _check(ops.history_append_execute(self.handle, C.byref(request), C.byref(facts),
                                          C.byref(err)), err)
        return facts


# -- host helpers that are part of the product (layout + codecs, no attention math) --

def kv_pack_pages(rows, storage, is_value, kv_heads, head_dim=128, page_tokens=16):
    """rows: token-major [pool_pages][page_tokens][kv_heads][row] (uint16 for BF16, uint8
    canonical blocks for Q8_0) -> packed device layout as a flat uint8 array."""
    rows = np.ascontiguousarray(rows)
    pool_pages = rows.shape[0]
    block = int(lib().yvex_rocm_kv_page_block_bytes(storage, head_dim, page_tokens))
    packed = np.empty(pool_pages * kv_heads * block, dtype=np.uint8)
    err = B.Error()
    _check(lib().yvex_rocm_kv_pack_pages(storage, int(is_value), rows.ctypes.data, pool_pages,
                                         page_tokens, kv_heads, head_dim, packed.ctypes.data,
                                         C.byref(err)), err)
    return packed


def kv_unpack_pages(packed, storage, is_value, pool_pages, kv_heads, head_dim=128, page_tokens=16):
    packed = np.ascontiguousarray(packed).reshape(-1).view(np.uint8)
    if storage == B.KV_BF16:
        rows = np.empty((pool_pages, page_tokens, kv_heads, head_dim), dtype=np.uint16)
    else:
        rows = np.empty((pool_pages, page_tokens, kv_heads, head_dim // 32 * 34), dtype=np.uint8)
    err = B.Error()
    _check(lib().yvex_rocm_kv_unpack_pages(storage, int(is_value), packed.ctypes.data, pool_pages,
                                           page_tokens, kv_heads, head_dim, rows.ctypes.data,
                                           C.byref(err)), err)
    return rows


def q8_0_encode_rows(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.shape[-1]
    out = np.empty(x.shape[:-1] + (n // 32 * 34,), dtype=np.uint8)
    err = B.Error()
    _check(lib().yvex_rocm_q8_0_encode_row(x.ctypes.data, x.size, out.ctypes.data, C.byref(err)),
           err)
    return out


def q8_0_decode_rows(b, n):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape[:-1] + (n,), dtype=np.float32)
    err = B.Error()
    _check(lib().yvex_rocm_q8_0_decode_row(b.ctypes.data, out.size, out.ctypes.data, C.byref(err)),
           err)
    return out


def benchmark_summarize(seconds, prefix=""):
    """Distribution fields of a benchmark record from per-iteration samples in seconds
    (src/runtime/benchmark.c:421-447): {"minimum_ns": ..., "p50_ns": ..., ...}, each name
    prefixed with `prefix` ("device_" for device timing).  Raises YvexError on samples that are
    not finite and positive."""
    samples = np.ascontiguousarray(seconds, dtype=np.float64).copy()
    out, err = B.TimingDistribution(), B.Error()
    _check(lib().yvex_runtime_benchmark_samples_summarize(
        samples.ctypes.data_as(C.POINTER(C.c_double)), samples.size, C.byref(out), C.byref(err)), err)
    return {prefix + lib().yvex_runtime_benchmark_statistic_name(i).decode(): int(out.values[i])
            for i in range(B.BENCHMARK_STATISTIC_COUNT)}

"""ctypes access to the CPU oracle (test infrastructure) and, when it has been
built, to the compiled reference operator in oracle/_ref.

Only tests, the smoke check and the benchmark's CPU leg may import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libyvex_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libyvex_ref.so")

u64 = C.c_uint64
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
u16p = C.POINTER(C.c_uint16)
u8p = C.POINTER(C.c_ubyte)
i32p = C.POINTER(C.c_int32)


class PositionPolicy(C.Structure):
    """yvo_position_policy (the fields of include/yvex/internal/backend.h:51-54)."""
    _fields_ = [("theta", u64), ("scaling_factor", u64), ("original_context", u64),
                ("beta_fast", u64), ("beta_slow", u64), ("rope_dimensions", u64)]


def _ptr(a, typ):
    if a is None:
        return C.cast(None, typ)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(typ)


def load_oracle():
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "all"])
    lib = C.CDLL(ORACLE_SO)
    lib.yvo_exp.restype = C.c_double
    lib.yvo_exp.argtypes = [C.c_double]
    lib.yvo_f16_decode.restype = C.c_float
    lib.yvo_f16_decode.argtypes = [C.c_uint16]
    lib.yvo_f16_encode.restype = C.c_uint16
    lib.yvo_f16_encode.argtypes = [C.c_float]
    lib.yvo_bf16_decode.restype = C.c_float
    lib.yvo_bf16_decode.argtypes = [C.c_uint16]
    lib.yvo_bf16_encode.restype = C.c_uint16
    lib.yvo_bf16_encode.argtypes = [C.c_float]
    lib.yvo_bf16_decode_n.argtypes = [u16p, f32p, C.c_size_t]
    lib.yvo_bf16_encode_n.argtypes = [f32p, u16p, C.c_size_t]
    lib.yvo_q8_0_encode_block.argtypes = [f32p, u8p]
    lib.yvo_q8_0_decode_block.argtypes = [u8p, f32p]
    lib.yvo_q8_0_encode_row.argtypes = [f32p, C.c_size_t, u8p]
    lib.yvo_q8_0_decode_row.argtypes = [u8p, C.c_size_t, f32p]
    lib.yvo_attention_head.argtypes = [f32p, f32p, C.c_size_t, f32p, C.c_size_t, u64, u64, u64,
                                       C.c_float, C.c_int, f32p, f32p, f32p, f64p]
    lib.yvo_gqa_attention.argtypes = [f32p, f32p, f32p, f32p, f64p] + [u64] * 9 + [C.c_int, C.c_int]
    lib.yvo_gqa_attention_bf16.argtypes = [u16p, u16p, u16p, f32p, u16p, f64p] + [u64] * 6 + [C.c_int, C.c_int]
    paged = [i32p, i32p, f32p, u16p, f64p] + [u64] * 7 + [C.c_int]
    lib.yvo_paged_decode_bf16.argtypes = [u16p, u16p, u16p] + paged
    lib.yvo_paged_decode_q8_0.argtypes = [u16p, u8p, u8p] + paged
    lib.yvo_shared_kv_head.argtypes = [f32p, f32p, C.c_size_t, u64, u64, u64, C.c_double, f32p, f32p, f64p]
    lib.yvo_rotary_half_bf16.argtypes = [u16p, f32p, f32p] + [u64] * 4
    lib.yvo_rotary_half_f32.argtypes = [f32p, f32p, f32p] + [u64] * 4
    lib.yvo_rotary_half_f32_rounded.argtypes = [f32p, f32p, f32p] + [u64] * 4
    lib.yvo_rotary_half_plain_f32.argtypes = [f32p, f32p, f32p] + [u64] * 4
    lib.yvo_sigmoid_gate_bf16.argtypes = [f32p, f32p, u64, f32p]
    lib.yvo_mla_decode_bf16.argtypes = [u16p, u16p, i32p, i32p, f32p, u16p, f64p] + [u64] * 7 + [f32p, u64, u16p, i32p, i32p, u64, u64, i32p, u64, C.c_int]
    lib.yvo_yarn_frequency.restype = C.c_double
    lib.yvo_yarn_frequency.argtypes = [C.POINTER(PositionPolicy), u64, u64]
    lib.yvo_rope_apply.argtypes = [f32p, u64, u64, u64, C.POINTER(PositionPolicy), C.c_int]
    lib.yvo_reduce_output_finish.argtypes = [f32p, u64, u64, u64, C.POINTER(PositionPolicy)]
    lib.yvo_lse_merge.argtypes = [f32p, f64p, u64, u64, f32p, f64p]
    return lib


REF_REDUCE_SO = os.path.join(os.path.dirname(REF_SO), "libyvex_ref_reduce.so")


def load_reference_reduce():
    """The compiled reference shared-KV reduce, or None when oracle/_ref was not built."""
    if not os.path.exists(REF_REDUCE_SO):
        return None
    lib = C.CDLL(REF_REDUCE_SO)
    u64p = C.POINTER(C.c_ulonglong)
    lib.yvref_attention_reduce.argtypes = [f32p, f32p, u64p, u64, f32p, u64p, u64, f32p, u64, u64,
                                           u64, u64, C.c_uint, u64, u64, u64, u64, u64, u64, u64, f32p]
    return lib


def reference_reduce(lib, query, local, local_positions, compressed, compressed_positions, sinks,
                     sliding_window, compression_ratio, attention_class, position,
                     rope_dims=2, theta=10000, scaling_factor=0, original_context=0, beta_fast=0,
                     beta_slow=0):
    """One query token through the reference reduce; returns (status, out [heads][dim])."""
    query = np.ascontiguousarray(query, dtype=np.float32)
    local = np.ascontiguousarray(local, dtype=np.float32)
    local_positions = np.ascontiguousarray(local_positions, dtype=np.uint64)
    compressed = np.ascontiguousarray(compressed, dtype=np.float32).reshape(-1, query.shape[1])
    compressed_positions = np.ascontiguousarray(compressed_positions, dtype=np.uint64)
    sinks = np.ascontiguousarray(sinks, dtype=np.float32)
    out = np.zeros_like(query)
    u64p = C.POINTER(C.c_ulonglong)
    rc = lib.yvref_attention_reduce(
        _ptr(query, f32p), _ptr(local, f32p), _ptr(local_positions, u64p), local.shape[0],
        _ptr(compressed, f32p) if len(compressed) else None,
        _ptr(compressed_positions, u64p) if len(compressed) else None, compressed.shape[0],
        _ptr(sinks, f32p), query.shape[0], query.shape[1], sliding_window, compression_ratio,
        attention_class, position, rope_dims, theta, scaling_factor, original_context, beta_fast,
        beta_slow, _ptr(out, f32p))
    return rc, out


def load_reference():
    """The compiled reference operator, or None when oracle/_ref was not built."""
    if not os.path.exists(REF_SO):
        return None
    lib = C.CDLL(REF_SO)
    lib.yvref_op_attention.argtypes = [f32p, f32p, f32p, C.c_ulonglong, C.c_ulonglong,
                                       C.c_ulonglong, C.c_float, C.c_int, f32p, f32p, f32p]
    lib.yvref_f16_decode.restype = C.c_float
    lib.yvref_f16_decode.argtypes = [C.c_ushort]
    lib.yvref_f16_encode.restype = C.c_ushort
    lib.yvref_f16_encode.argtypes = [C.c_float]
    lib.yvref_bf16_decode.restype = C.c_float
    lib.yvref_bf16_decode.argtypes = [C.c_ushort]
    lib.yvref_bf16_encode.restype = C.c_ushort
    lib.yvref_bf16_encode.argtypes = [C.c_float]
    lib.yvref_bf16_encode_n.argtypes = [f32p, u16p, C.c_size_t]
    lib.yvref_f16_encode_n.argtypes = [f32p, u16p, C.c_size_t]
    lib.yvref_f16_decode_n.argtypes = [u16p, f32p, C.c_size_t]
    if hasattr(lib, "yvref_q8_0_encode_block"):
        lib.yvref_q8_0_encode_block.argtypes = [f32p, u8p]
        lib.yvref_q8_0_decode_block.argtypes = [u8p, f32p]
    return lib


class Oracle:
    """numpy-facing wrapper over the oracle library."""

    def __init__(self):
        self.lib = load_oracle()
        self.threads = int(self.lib.yvo_hardware_threads())

    # -- codecs -----------------------------------------------------------
    def bf16_encode(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.uint16)
        self.lib.yvo_bf16_encode_n(_ptr(x, f32p), _ptr(out, u16p), x.size)
        return out

    def bf16_decode(self, b):
        b = np.ascontiguousarray(b, dtype=np.uint16)
        out = np.empty(b.shape, dtype=np.float32)
        self.lib.yvo_bf16_decode_n(_ptr(b, u16p), _ptr(out, f32p), b.size)
        return out

    def q8_0_encode_rows(self, x):
        """x float32 [..., n] (n % 32 == 0) -> uint8 [..., n/32*34]."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        n = x.shape[-1]
        rows = x.reshape(-1, n)
        out = np.empty((rows.shape[0], n // 32 * 34), dtype=np.uint8)
        rc = self.lib.yvo_q8_0_encode_row(_ptr(rows, f32p), rows.size, _ptr(out, u8p))
        assert rc == 0, rc
        return out.reshape(x.shape[:-1] + (n // 32 * 34,))

    def q8_0_decode_rows(self, b, n):
        b = np.ascontiguousarray(b, dtype=np.uint8)
        rows = b.reshape(-1, n // 32 * 34)
        out = np.empty((rows.shape[0], n), dtype=np.float32)
        rc = self.lib.yvo_q8_0_decode_row(_ptr(rows, u8p), out.size, _ptr(out, f32p))
        assert rc == 0, rc
        return out.reshape(b.shape[:-1] + (n,))

    # -- attention ----------------------------------------------------------
    def attention_head(self, q, k, v, position, scale, causal=True):
        q = np.ascontiguousarray(q, dtype=np.float32)
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        n, d = k.shape
        score = np.zeros(n, dtype=np.float32)
        prob = np.zeros(n, dtype=np.float32)
        out = np.zeros(d, dtype=np.float32)
        lse = C.c_double(0.0)
        rc = self.lib.yvo_attention_head(_ptr(q, f32p), _ptr(k, f32p), d, _ptr(v, f32p), d, n,
                                         position, d, scale, int(causal), _ptr(score, f32p),
                                         _ptr(prob, f32p), _ptr(out, f32p), C.byref(lse))
        return rc, out, score, prob, lse.value

    def gqa(self, q, k, v, query_start=0, causal=True, q_stride=0, k_stride=0, v_stride=0,
            query_tokens=None, kv_tokens=None, query_heads=None, kv_heads=None, head_dim=None,
            threads=None):
        """q/k/v float32; when strides are 0 shapes are [T,H,d]."""
        q = np.ascontiguousarray(q, dtype=np.float32)
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        if query_tokens is None:
            query_tokens, query_heads, head_dim = q.shape
            kv_tokens, kv_heads, _ = k.shape
        out = np.zeros((query_tokens, query_heads, head_dim), dtype=np.float32)
        lse = np.zeros((query_tokens, query_heads), dtype=np.float64)
        rc = self.lib.yvo_gqa_attention(_ptr(q, f32p), _ptr(k, f32p), _ptr(v, f32p),
                                        _ptr(out, f32p), _ptr(lse, f64p), query_tokens,
                                        kv_tokens, query_start, query_heads, kv_heads, head_dim,
                                        q_stride, k_stride, v_stride, int(causal),
                                        threads or self.threads)
        return rc, out, lse

    def gqa_bf16(self, q, k, v, query_start=0, causal=True, threads=None):
        """q uint16 [Tq,Hq,d], k/v uint16 [Tk,Hkv,d] -> (rc, out_f32, out_bf16, lse)."""
        tq, hq, d = q.shape
        tk, hkv, _ = k.shape
        out = np.zeros((tq, hq, d), dtype=np.float32)
        outb = np.zeros((tq, hq, d), dtype=np.uint16)
        lse = np.zeros((tq, hq), dtype=np.float64)
        rc = self.lib.yvo_gqa_attention_bf16(_ptr(q, u16p), _ptr(k, u16p), _ptr(v, u16p),
                                             _ptr(out, f32p), _ptr(outb, u16p), _ptr(lse, f64p),
                                             tq, tk, query_start, hq, hkv, d, int(causal),
                                             threads or self.threads)
        return rc, out, outb, lse

    def paged_decode(self, q, k_pool, v_pool, page_table, context, kv_heads, page_tokens,
                     q8=False, threads=None):
        """q uint16 [S,Hq,d]; canonical pools (see the oracle header)."""
        s, hq, d = q.shape
        pool_pages = k_pool.shape[0]
        page_table = np.ascontiguousarray(page_table, dtype=np.int32)
        context = np.ascontiguousarray(context, dtype=np.int32)
        out = np.zeros((s, hq, d), dtype=np.float32)
        outb = np.zeros((s, hq, d), dtype=np.uint16)
        lse = np.zeros((s, hq), dtype=np.float64)
        fn = self.lib.yvo_paged_decode_q8_0 if q8 else self.lib.yvo_paged_decode_bf16
        pt = u8p if q8 else u16p
        rc = fn(_ptr(q, u16p), _ptr(k_pool, pt), _ptr(v_pool, pt), _ptr(page_table, i32p),
                _ptr(context, i32p), _ptr(out, f32p), _ptr(outb, u16p), _ptr(lse, f64p), s, hq,
                kv_heads, d, page_tokens, pool_pages, page_table.shape[1],
                threads or self.threads)
        return rc, out, outb, lse

    def shared_kv_head(self, q, rows, key_dim, value_dim, scale, sink=None):
        q = np.ascontiguousarray(q, dtype=np.float32)
        rows = np.ascontiguousarray(rows, dtype=np.float32)
        out = np.zeros(value_dim, dtype=np.float32)
        lse = C.c_double(0.0)
        sink_arr = None if sink is None else np.array([sink], dtype=np.float32)
        rc = self.lib.yvo_shared_kv_head(_ptr(q, f32p), _ptr(rows, f32p), rows.shape[1],
                                         rows.shape[0], key_dim, value_dim, scale,
                                         _ptr(sink_arr, f32p), _ptr(out, f32p), C.byref(lse))
        return rc, out, lse.value

    def rotary_half_bf16(self, values, cosines, sines, rotary_dim):
        """values uint16 [tokens, heads, d] -> rotated copy (rotate-half, bf16 roundings)."""
        out = np.ascontiguousarray(values).copy()
        tokens, heads, d = out.shape
        cosines = np.ascontiguousarray(cosines, dtype=np.float32)
        sines = np.ascontiguousarray(sines, dtype=np.float32)
        rc = self.lib.yvo_rotary_half_bf16(_ptr(out, u16p), _ptr(cosines, f32p), _ptr(sines, f32p),
                                           tokens, heads, d, rotary_dim)
        assert rc == 0
        return out

    def rotary_half_f32(self, values, cosines, sines, rotary_dim):
        """values float32 [tokens, heads, d] -> rotated copy (products and sums rounded to bf16)."""
        out = np.ascontiguousarray(values, dtype=np.float32).copy()
        tokens, heads, d = out.shape
        cosines = np.ascontiguousarray(cosines, dtype=np.float32)
        sines = np.ascontiguousarray(sines, dtype=np.float32)
        rc = self.lib.yvo_rotary_half_f32(_ptr(out, f32p), _ptr(cosines, f32p), _ptr(sines, f32p),
                                          tokens, heads, d, rotary_dim)
        assert rc == 0
        return out

    def rotary_half_f32_rounded(self, values, cosines, sines, rotary_dim):
        """values float32 [tokens, heads, d] -> plain F32 rotation, then every lane rounded to
        bf16 (the decoder's order)."""
        out = np.ascontiguousarray(values, dtype=np.float32).copy()
        tokens, heads, d = out.shape
        cosines = np.ascontiguousarray(cosines, dtype=np.float32)
        sines = np.ascontiguousarray(sines, dtype=np.float32)
        rc = self.lib.yvo_rotary_half_f32_rounded(_ptr(out, f32p), _ptr(cosines, f32p),
                                                  _ptr(sines, f32p), tokens, heads, d, rotary_dim)
        assert rc == 0
        return out

    def rotary_half_plain_f32(self, values, cosines, sines, rotary_dim):
        """values float32 [tokens, heads, d] -> plain F32 rotation, nothing rounded to bf16."""
        out = np.ascontiguousarray(values, dtype=np.float32).copy()
        tokens, heads, d = out.shape
        cosines = np.ascontiguousarray(cosines, dtype=np.float32)
        sines = np.ascontiguousarray(sines, dtype=np.float32)
        rc = self.lib.yvo_rotary_half_plain_f32(_ptr(out, f32p), _ptr(cosines, f32p),
                                                _ptr(sines, f32p), tokens, heads, d, rotary_dim)
        assert rc == 0
        return out

    def sigmoid_gate_bf16(self, values, gate):
        """F32 values (bf16-representable) times sigmoid(gate), rounded to bf16; F32 out."""
        values = np.ascontiguousarray(values, dtype=np.float32)
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        out = np.zeros_like(values)
        rc = self.lib.yvo_sigmoid_gate_bf16(_ptr(values, f32p), _ptr(gate, f32p), values.size,
                                            _ptr(out, f32p))
        assert rc == 0
        return out

    def mla_decode(self, q, pool, page_table, context, value_dim, page_tokens, threads=None,
                   sinks=None, sliding_window=0, compressed=None, selected=None):
        """compressed: optional (pool uint16 [pages][page_tokens][kd], table int32 [b][stride],
        counts int32 [b]) second row set; selected: optional int32 [b][capacity] row lists."""
        b, h, kd = q.shape
        page_table = np.ascontiguousarray(page_table, dtype=np.int32)
        context = np.ascontiguousarray(context, dtype=np.int32)
        out = np.zeros((b, h, value_dim), dtype=np.float32)
        outb = np.zeros((b, h, value_dim), dtype=np.uint16)
        lse = np.zeros((b, h), dtype=np.float64)
        if sinks is not None:
            sinks = np.ascontiguousarray(sinks, dtype=np.float32)
        extra = (None, None, None, 0, 0, None, 0)
        if compressed is not None:
            cpool = np.ascontiguousarray(compressed[0], dtype=np.uint16)
            ctable = np.ascontiguousarray(compressed[1], dtype=np.int32)
            ccount = np.ascontiguousarray(compressed[2], dtype=np.int32)
            chosen = np.ascontiguousarray(selected, dtype=np.int32) if selected is not None else None
            extra = (_ptr(cpool, u16p), _ptr(ctable, i32p), _ptr(ccount, i32p), cpool.shape[0],
                     ctable.shape[1], _ptr(chosen, i32p) if chosen is not None else None,
                     chosen.shape[1] if chosen is not None else 0)
        rc = self.lib.yvo_mla_decode_bf16(_ptr(q, u16p), _ptr(pool, u16p), _ptr(page_table, i32p),
                                          _ptr(context, i32p), _ptr(out, f32p), _ptr(outb, u16p),
                                          _ptr(lse, f64p), b, h, kd, value_dim, page_tokens,
                                          pool.shape[0], page_table.shape[1],
                                          _ptr(sinks, f32p) if sinks is not None else None,
                                          sliding_window, *extra, threads or self.threads)
        return rc, out, outb, lse

    @staticmethod
    def position_policy(rope_dims, theta=10000, scaling_factor=0, original_context=0, beta_fast=0,
                        beta_slow=0):
        return PositionPolicy(theta, scaling_factor, original_context, beta_fast, beta_slow, rope_dims)

    def rope_apply(self, row, position, policy, inverse=False):
        out = np.ascontiguousarray(row, dtype=np.float32).copy()
        rc = self.lib.yvo_rope_apply(_ptr(out, f32p), out.size, policy.rope_dimensions, position,
                                     C.byref(policy), int(inverse))
        return rc, out

    def reduce_output_finish(self, rows, position, policy):
        """rows float [heads][dim] -> bf16 round, inverse rotation of the rope lanes, bf16 round."""
        out = np.ascontiguousarray(rows, dtype=np.float32).copy()
        rc = self.lib.yvo_reduce_output_finish(_ptr(out, f32p), out.shape[0], out.shape[1], position,
                                               C.byref(policy))
        return rc, out

    def lse_merge(self, part_out, part_lse):
        part_out = np.ascontiguousarray(part_out, dtype=np.float32)
        part_lse = np.ascontiguousarray(part_lse, dtype=np.float64)
        parts, dim = part_out.shape
        out = np.zeros(dim, dtype=np.float32)
        lse = C.c_double(0.0)
        rc = self.lib.yvo_lse_merge(_ptr(part_out, f32p), _ptr(part_lse, f64p), parts, dim,
                                    _ptr(out, f32p), C.byref(lse))
        return rc, out, lse.value

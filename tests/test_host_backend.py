"""Host-side behaviour of the C backend on a machine without a GPU: symbol export,
fail-closed admission, argument-check order, bookkeeping, failure transitions and
checked cleanup.  A stand-in HIP runtime (tests/fake_hip) is injected through
YVEX_TEST_ROCM_DRIVER_LIBRARY; its kernel launches do nothing, so no numerics are
tested here (those are the GPU tests)."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import (Backend, YvexError, kv_pack_pages, kv_unpack_pages, lib,
                               q8_0_decode_rows, q8_0_encode_rows)
from oracle_binding import Oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE_DIR = os.path.join(ROOT, "tests", "fake_hip")
FAKE_SO = os.path.join(FAKE_DIR, "libfakehip.so")
ORACLE = Oracle()


@pytest.fixture(scope="module", autouse=True)
def fake_runtime():
    subprocess.check_call(["gcc", "-std=c11", "-O1", "-fPIC", "-shared", "-I/opt/rocm/include",
                           "-o", FAKE_SO, os.path.join(FAKE_DIR, "fake_hip.c")])
    os.environ["YVEX_TEST_ROCM_DRIVER_LIBRARY"] = FAKE_SO
    yield C.CDLL(FAKE_SO)
    for name in list(os.environ):
        if name.startswith(("YVEX_TEST_ROCM_", "FAKE_HIP_")):
            del os.environ[name]


@pytest.fixture
def env():
    """Sets variables for one test and restores them afterwards."""
    touched = []

    def setter(name, value):
        touched.append((name, os.environ.get(name)))
        if value is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = value
    yield setter
    for name, old in reversed(touched):
        if old is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = old


def f32(backend, name, shape, data=None):
    return backend.tensor(name, B.DTYPE_F32, shape,
                          None if data is None else np.asarray(data, dtype=np.float32))


def written(backend, name, dtype, shape):
    t = backend.tensor(name, dtype, shape)
    t.zero()
    return t


# ------------------------------------------------------------------ exports ----

def test_library_exports_every_declared_symbol():
    library = lib()
    for name in B.EXPORTED_SYMBOLS:
        assert hasattr(library, name), name
    header = "".join(open(os.path.join(ROOT, "include", name)).read()
                     for name in ("yvex_rocm.h", "yvex_rocm_operations.h"))
    for name in B.EXPORTED_SYMBOLS:
        assert name + "(" in header, "declared in binding but not in the header: " + name


def test_names_match_the_reference_vocabulary():
    library = lib()
    assert library.yvex_status_name(B.YVEX_ERR_BOUNDS) == b"YVEX_ERR_BOUNDS"
    assert library.yvex_backend_kind_name(B.KIND_ROCM) == b"rocm"
    assert library.yvex_backend_status_name(B.STATUS_CONTEXT_READY) == b"context-ready"
    assert library.yvex_backend_operation_variant_name(13) == b"attention-causal-f32"
    assert library.yvex_backend_operation_variant_name(16) == b"encoded-attention"
    assert library.yvex_backend_capability_reason_name(4) == b"kernel-bundle-absent"
    assert library.yvex_backend_capability_reason_name(6) == b"required-function-missing"
    assert library.yvex_backend_capability_name(B.CAP_OP_ATTENTION) == b"op_attention"
    kind, err = C.c_int(-1), B.Error()
    assert library.yvex_backend_kind_parse(b"rocm", C.byref(kind), C.byref(err)) == 0
    assert kind.value == B.KIND_ROCM
    assert library.yvex_backend_kind_parse(b"vulkan", C.byref(kind), C.byref(err)) == \
        B.YVEX_ERR_INVALID_ARG and b"unknown backend kind: vulkan" in err.message


def test_other_kinds_are_not_implemented_here():
    for kind in (B.KIND_CPU, B.KIND_CUDA, B.KIND_METAL):
        with pytest.raises(YvexError) as e:
            Backend(kind=kind)
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED and "is not implemented" in e.value.message


def test_open_without_a_device_fails_closed(env):
    env("FAKE_HIP_DEVICES", "0")
    with pytest.raises(YvexError) as e:
        Backend()
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    env("FAKE_HIP_DEVICES", None)
    env("FAKE_HIP_INIT", "fail")
    with pytest.raises(YvexError) as e:
        Backend()
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    env("FAKE_HIP_INIT", None)
    env("YVEX_TEST_ROCM_DRIVER_LIBRARY", "/nonexistent/libhip.so")
    with pytest.raises(YvexError) as e:
        Backend()
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED and "unavailable" in e.value.message
    assert lib().yvex_backend_rocm_available() == 0


# ---------------------------------------------------------- admission ----

def test_ready_backend_publishes_attention_only():
    with Backend() as b:
        report = b.report()
        assert b.status == B.STATUS_READY and report.bundle_admitted and report.bundle_built
        assert report.architecture == b"gfx950" and report.function_count >= 9
        assert report.device_name == b"fake-gfx950"
        for variant in (B.VARIANT_TENSOR_ALLOC, B.VARIANT_TENSOR_COPY,
                        B.VARIANT_ATTENTION_CAUSAL_F32, B.VARIANT_ATTENTION_NONCAUSAL_F32,
                        B.VARIANT_ROCM_GQA_F32, B.VARIANT_ROCM_GQA_BF16, B.VARIANT_ROCM_PAGED_BF16,
                        B.VARIANT_ROCM_PAGED_Q8_0, B.VARIANT_ROCM_MLA_BF16):
            r = b.query_capability(variant)
            assert r.state == B.CAPABILITY_SUPPORTED and r.reason == B.REASON_NONE, variant
            assert r.context_available and r.kernel_bundle_available and r.function_available
        for variant in (B.VARIANT_MATMUL_F32, B.VARIANT_ATTENTION_ENCODED, 5, 9, 15):
            r = b.query_capability(variant)      # embed, rope, qtype, ... : not this backend's
            assert r.state == B.CAPABILITY_UNSUPPORTED and r.reason == B.REASON_VARIANT_UNSUPPORTED
        assert b.supports(B.CAP_TENSOR_ALLOC) and b.supports(B.CAP_TENSOR_READ_WRITE)
        assert b.supports(B.CAP_OP_ATTENTION) and not b.supports(3)
        r = b.query_capability(B.VARIANT_ROCM_PAGED_Q8_0)
        assert (r.input_dtype, r.weight_dtype, r.output_dtype) == (B.DTYPE_BF16, B.DTYPE_Q8_0,
                                                                   B.DTYPE_BF16)
        with pytest.raises(YvexError) as e:
            b.query_capability(40)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
        assert b.transformer_operations() is not None
        assert b.rocm_attention_operations() is not None
        info = b.device_info()
        assert info.kind == B.KIND_ROCM and info.name == b"fake-gfx950"


def test_encoded_attention_transaction_fails_closed():
    """include/yvex/internal/backend.h:193-198: the symbol exists and refuses; the table the
    backend returns has the reference's slot order with the attention slots and the element-wise slots
    the decoder calls around them published, the rest NULL."""
    library = lib()

    class Failure(C.Structure):
        _fields_ = [("code", C.c_int), ("stage", C.c_char_p), ("expected", C.c_ulonglong),
                    ("actual", C.c_ulonglong)]
    library.yvex_backend_attention_execute.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                                       C.POINTER(Failure), C.POINTER(B.Error)]
    library.yvex_backend_attention_complete.argtypes = [C.c_void_p, C.c_void_p, C.c_int,
                                                        C.POINTER(B.Error)]
    job, output = C.create_string_buffer(4096), C.create_string_buffer(b"\x5a" * 1024, 1024)
    with Backend() as b:
        failure, err = Failure(), B.Error()
        rc = library.yvex_backend_attention_execute(b.handle, job, output, C.byref(failure),
                                                    C.byref(err))
        assert rc == B.YVEX_ERR_UNSUPPORTED and err.code == B.YVEX_ERR_UNSUPPORTED
        assert failure.code == 2 and failure.stage == b"rocm.attention.encoded"   # CAPABILITY
        assert output.raw == b"\x5a" * 1024                       # the output record is untouched
        assert b.query_capability(B.VARIANT_ATTENTION_ENCODED).state == B.CAPABILITY_UNSUPPORTED
        rc = library.yvex_backend_attention_execute(b.handle, None, output, C.byref(failure),
                                                    C.byref(err))
        assert rc == B.YVEX_ERR_INVALID_ARG and failure.code == 1
        rc = library.yvex_backend_attention_complete(b.handle, job, 0, C.byref(err))
        assert rc == B.YVEX_ERR_INVALID_ARG
        ops = b.transformer_operations()
        for name in B.TRANSFORMER_OPERATION_SLOTS:
            published = bool(getattr(ops, name))
            assert published == (name in ("attention_workspace_required", "attention_execute",
                                              "rotary_half_f32", "split_interleaved_two_f32",
                                              "sigmoid_product_bf16", "bf16_round")), name


@pytest.mark.parametrize("injected,reason_for_attention", [
    ("module", B.REASON_KERNEL_BUNDLE_REJECTED),
    ("symbol", B.REASON_FUNCTION_MISSING),
    ("yvex_rocm_decode_merge", B.REASON_KERNEL_BUNDLE_REJECTED),
])
def test_rejected_bundle_publishes_nothing(env, fake_runtime, injected, reason_for_attention):
    env("YVEX_TEST_ROCM_BUNDLE_FAILURE", injected)
    with Backend() as b:
        assert b.status == B.STATUS_CONTEXT_READY
        report = b.report()
        assert not report.bundle_admitted and report.function_count == 0 and report.rejection
        assert fake_runtime.fake_hip_live_modules() == 0          # everything loaded was unloaded
        r = b.query_capability(B.VARIANT_ATTENTION_CAUSAL_F32)
        assert r.state == B.CAPABILITY_FAILED and r.reason == reason_for_attention
        if injected == "yvex_rocm_decode_merge":
            r = b.query_capability(B.VARIANT_ROCM_PAGED_BF16)      # the variant that lost a symbol
            assert r.reason == B.REASON_FUNCTION_MISSING
        assert b.transformer_operations() is None and b.rocm_attention_operations() is None
        assert not b.supports(B.CAP_OP_ATTENTION) and b.supports(B.CAP_TENSOR_ALLOC)
        t = f32(b, "x", (4,), [1, 2, 3, 4])                        # tensor traffic still works
        assert np.array_equal(t.read(), [1, 2, 3, 4])
        q, k = f32(b, "q", (4,), np.ones(4)), f32(b, "k", (3, 4), np.ones((3, 4)))
        s, o = f32(b, "s", (3,)), f32(b, "o", (4,))
        with pytest.raises(YvexError) as e:
            b.op_attention(q, k, k, 3, 0, 0.5, True, s, s, o)
        assert e.value.code == B.YVEX_ERR_BACKEND and "refused" in e.value.message
        assert not o.is_written


def test_missing_function_in_runtime_rejects_the_whole_bundle(env):
    env("FAKE_HIP_MISSING_FUNCTION", "yvex_rocm_prefill_bf16")
    with Backend() as b:
        assert b.status == B.STATUS_CONTEXT_READY
        assert b.query_capability(B.VARIANT_ROCM_GQA_BF16).reason == B.REASON_FUNCTION_MISSING
        assert b.query_capability(B.VARIANT_ROCM_MLA_BF16).reason == \
            B.REASON_KERNEL_BUNDLE_REJECTED
        assert b"yvex_rocm_prefill_bf16" in b.report().rejection


def test_bundle_absent_build_reports_absent_and_refuses(tmp_path):
    out = tmp_path / "libyvex_rocm_nobundle.so"
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "clori_amd", "csrc"), "BUNDLE=0",
                           "BUILD=%s" % (tmp_path / "build"), "OUT=%s" % out])
    script = """
import sys, ctypes as C
sys.path.insert(0, %r)
from clori_amd import binding as B
lib = B.load(%r)
handle, err = C.c_void_p(), B.Error()
opts = B.BackendOptions(B.KIND_ROCM, None, 0)
assert lib.yvex_backend_open(C.byref(handle), C.byref(opts), C.byref(err)) == 0
assert lib.yvex_backend_status_of(handle) == B.STATUS_CONTEXT_READY
res = B.CapabilityResult()
assert lib.yvex_backend_query_capability(handle, B.VARIANT_ATTENTION_CAUSAL_F32, C.byref(res), C.byref(err)) == 0
assert res.state == B.CAPABILITY_UNSUPPORTED and res.reason == B.REASON_KERNEL_BUNDLE_ABSENT
assert lib.yvex_backend_query_capability(handle, B.VARIANT_TENSOR_ALLOC, C.byref(res), C.byref(err)) == 0
assert res.state == B.CAPABILITY_SUPPORTED
assert not lib.yvex_backend_transformer_operations_get(handle)
rep = B.RocmReport()
lib.yvex_backend_rocm_report_get(handle, C.byref(rep), C.byref(err))
assert not rep.bundle_built and rep.image_count == 0
assert lib.yvex_backend_close_checked(C.byref(handle), C.byref(err)) == 0
print("absent-ok")
""" % (ROOT, str(out))
    result = subprocess.run(["python3", "-c", script], capture_output=True, text=True,
                            env=dict(os.environ))
    assert "absent-ok" in result.stdout, result.stderr
    # the inspection command of the same build, with the lines the reference's bundle-less
    # build prints (tests/test_cuda_failclosed.sh:59-80)
    shown = subprocess.run([str(tmp_path / "yvex-rocm"), "inspect", "backend", "rocm"],
                           capture_output=True, text=True, env=dict(os.environ))
    assert shown.returncode == 0, shown.stderr
    for line in ("status: context-ready", "  tensor_alloc: yes", "  tensor_read_write: yes",
                 "  op_attention: no", "context_available: yes", "kernel_bundle: absent",
                 "kernel_bundle_reason: kernel-bundle-absent", "kernel_bundle_native: no",
                 "  attention-noncausal-f32: unsupported (kernel-bundle-absent)",
                 "  encoded-attention: unsupported (kernel-bundle-absent)",
                 "  rocm-attention-paged-bf16: unsupported (kernel-bundle-absent)",
                 "status: backend-capabilities"):
        assert line + "\n" in shown.stdout, line


# ------------------------------------------------------------- tensors ----

def test_tensor_lifecycle_and_accounting(fake_runtime):
    with Backend(memory_limit_bytes=1 << 20) as b:
        base = fake_runtime.fake_hip_live_allocations()
        t = f32(b, "weights", (16, 4))
        assert np.all(t.read() == 0) and not t.is_written          # read before write is zero
        t.write(np.arange(64, dtype=np.float32))
        assert t.is_written and np.array_equal(t.read().ravel(), np.arange(64))
        stats = b.memory_stats()
        assert stats.allocated_bytes == 256 and stats.allocation_count == 1
        assert stats.h2d_bytes == 256 and stats.d2h_bytes == 512 and stats.memory_limit_bytes == 1 << 20
        err = B.Error()
        short = np.zeros(3, np.float32)
        rc = lib().yvex_backend_tensor_write(b.handle, t.handle, short.ctypes.data, 12, C.byref(err))
        assert rc == B.YVEX_ERR_BOUNDS and b"does not match tensor bytes" in err.message
        with pytest.raises(YvexError) as e:
            b.tensor("too-big", B.DTYPE_I8, (1 << 21,))
        assert e.value.code == B.YVEX_ERR_NOMEM and "memory limit" in e.value.message
        with pytest.raises(YvexError) as e:
            b.tensor("zero-dim", B.DTYPE_F32, (0,), nbytes=4)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
        desc, handle = B.TensorDesc(b"rank5", B.DTYPE_F32, 5), B.TensorP()
        desc.bytes = 4
        assert lib().yvex_backend_tensor_alloc(b.handle, C.byref(desc), C.byref(handle),
                                               C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        u = f32(b, "copy", (16, 4))
        rc = lib().yvex_backend_tensor_copy(b.handle, u.handle, t.handle, C.byref(err))
        assert rc == 0 and np.array_equal(u.read(), t.read())
        v = f32(b, "other-shape", (64,))
        assert lib().yvex_backend_tensor_copy(b.handle, v.handle, t.handle, C.byref(err)) == \
            B.YVEX_ERR_BOUNDS
        with Backend() as other:                                     # a foreign tensor is refused
            foreign = f32(other, "foreign", (16, 4))
            assert lib().yvex_backend_tensor_copy(b.handle, foreign.handle, t.handle,
                                                  C.byref(err)) == B.YVEX_ERR_STATE
            assert not lib().yvex_backend_tensor_owned_by(b.handle, foreign.handle)
        t.release()
        assert t.handle is None
        stats = b.memory_stats()
        assert stats.allocation_count == 2 and stats.release_events == 1
        assert stats.peak_allocated_bytes >= 768
        assert fake_runtime.fake_hip_live_allocations() == base + 2


def test_async_copy_refusal_order_and_effect(fake_runtime):
    """yvex_backend_tensor_copy_async (src/backend/core.c:822-840): lifecycle first, then
    ownership (STATE), then descriptors (BOUNDS); the copy itself is not waited for and the
    destination inherits the source's written flag (src/backend/cuda/backend.c:1159-1191)."""
    err = B.Error()
    copy_async = lib().yvex_backend_tensor_copy_async
    with Backend() as b, Backend() as other:
        source, target = f32(b, "source", (8, 4)), f32(b, "target", (8, 4))
        source.write(np.arange(32, dtype=np.float32))
        assert not target.is_written
        assert copy_async(b.handle, target.handle, source.handle, C.byref(err)) == 0
        assert target.is_written and np.array_equal(target.read(), source.read())
        fresh, into = f32(b, "never-written", (8, 4)), f32(b, "into", (8, 4))
        into.write(np.ones(32, np.float32))
        assert copy_async(b.handle, into.handle, fresh.handle, C.byref(err)) == 0
        assert not into.is_written                                   # flag follows the source
        reshaped = f32(b, "reshaped", (32,))
        assert copy_async(b.handle, reshaped.handle, source.handle, C.byref(err)) == B.YVEX_ERR_BOUNDS
        assert b"descriptors differ" in err.message
        foreign = f32(other, "foreign", (8, 4))
        assert copy_async(b.handle, foreign.handle, source.handle, C.byref(err)) == B.YVEX_ERR_STATE
        assert copy_async(b.handle, target.handle, foreign.handle, C.byref(err)) == B.YVEX_ERR_STATE
        assert err.where == b"backend.tensor.copy-async"
        # the session layer's use (src/runtime/stateful_attention.c:183-222): row views of the
        # projections copied into [K | V] rows of the history
        history = f32(b, "history", (4, 2, 16))
        history.zero()
        keys, values = f32(b, "keys", (2, 16)), f32(b, "values", (2, 16))
        keys.write(np.arange(32, dtype=np.float32))
        values.write(-np.arange(32, dtype=np.float32))
        for token in range(2):
            history.view((1 + token) * 128, B.DTYPE_F32, (16,)).copy_from_async(
                keys.view(token * 64, B.DTYPE_F32, (16,)))
            history.view((1 + token) * 128 + 64, B.DTYPE_F32, (16,)).copy_from_async(
                values.view(token * 64, B.DTYPE_F32, (16,)))
        rows = history.read().reshape(4, 32)
        assert np.all(rows[0] == 0) and np.all(rows[3] == 0)
        assert np.array_equal(rows[1], np.concatenate([np.arange(16), -np.arange(16)]))
        assert np.array_equal(rows[2], np.concatenate([np.arange(16, 32), -np.arange(16, 32)]))
    closed = C.c_void_p()
    options = B.BackendOptions(B.KIND_ROCM, None, 0)
    assert lib().yvex_backend_open(C.byref(closed), C.byref(options), C.byref(err)) == 0
    assert copy_async(None, None, None, C.byref(err)) == B.YVEX_ERR_STATE    # lifecycle gate first
    assert lib().yvex_backend_close_checked(C.byref(closed), C.byref(err)) == 0


def test_session_backends_lease_their_primary_and_copy_between_streams(fake_runtime):
    """yvex_backend_open_shared_rocm (src/backend/cuda/backend.c:1795-1879) and
    yvex_backend_tensor_copy_shared_async (src/backend/core.c:842-874): a session backend has
    its own stream and accounting on the primary's device; the primary cannot be discharged
    while a session backend is open; a copy across the two is admitted only for one physical
    owner, equal descriptors and a written source."""
    err = B.Error()
    shared_copy = lib().yvex_backend_tensor_copy_shared_async
    primary = Backend(memory_limit_bytes=1 << 20)
    session = Backend(shared_with=primary, memory_limit_bytes=1 << 16)
    second = Backend(shared_with=primary)
    stranger = Backend()
    assert session.status == B.STATUS_READY
    assert session.memory_stats().memory_limit_bytes == 1 << 16
    source = f32(primary, "weights", (4, 4))
    source.write(np.arange(16, dtype=np.float32))
    target = f32(session, "copy", (4, 4))
    target.copy_from_shared_async(source)                           # primary -> session
    assert target.is_written and np.array_equal(target.read(), source.read())
    sibling = f32(second, "sibling", (4, 4))
    sibling.copy_from_shared_async(target)                          # session -> session
    assert np.array_equal(sibling.read(), source.read())
    back = f32(primary, "back", (4, 4))
    back.copy_from_shared_async(sibling)                            # session -> primary
    assert np.array_equal(back.read(), source.read())
    assert primary.memory_stats().allocated_bytes == 128 and session.memory_stats().allocated_bytes == 64
    # refusals: destination not the executor's, another physical owner, descriptors, unwritten
    assert shared_copy(primary.handle, target.handle, source.handle, C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    outsider = f32(stranger, "outsider", (4, 4))
    outsider.write(np.zeros(16, np.float32))
    assert shared_copy(session.handle, target.handle, outsider.handle, C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    assert shared_copy(session.handle, f32(session, "flat", (16,)).handle, source.handle,
                       C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    assert shared_copy(session.handle, target.handle, f32(primary, "blank", (4, 4)).handle,
                       C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    assert shared_copy(None, target.handle, source.handle, C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    # a session backend cannot be the owner of another one
    nested = C.c_void_p()
    assert lib().yvex_backend_open_shared_rocm(C.byref(nested), session.handle, 0, C.byref(err)) == \
        B.YVEX_ERR_INVALID_ARG and not nested.value
    # the primary is not discharged while session backends are open: the close marks it
    # cleanup-only and keeps the handle; after the sessions are closed it goes
    stranger.close()
    for backend in (primary, session, second):
        for tensor in backend.tensors:
            tensor.release()
    handle = C.c_void_p(primary.handle.value)
    assert lib().yvex_backend_close_checked(C.byref(handle), C.byref(err)) == B.YVEX_ERR_STATE
    assert handle.value and b"live shared children" in err.message
    late = C.c_void_p()
    assert lib().yvex_backend_open_shared_rocm(C.byref(late), handle, 0, C.byref(err)) == B.YVEX_ERR_STATE
    session.close()
    assert lib().yvex_backend_close_checked(C.byref(handle), C.byref(err)) == B.YVEX_ERR_STATE
    second.close()
    assert lib().yvex_backend_close_checked(C.byref(handle), C.byref(err)) == 0 and not handle.value
    primary.handle = None


def test_f32_subview_matches_reference_rules():
    with Backend() as b:
        t = f32(b, "row", (8, 4), np.arange(32))
        view = B.DeviceTensor()
        assert lib().yvex_backend_tensor_f32_subview(t.handle, 4, 8, C.byref(view)) == 1
        assert view.rank == 1 and view.dims[0] == 8 and view.bytes == 32
        assert view.data == t.handle.contents.data + 16
        assert lib().yvex_backend_tensor_f32_subview(t.handle, 30, 8, C.byref(view)) == 0
        assert lib().yvex_backend_tensor_f32_subview(t.handle, 0, 0, C.byref(view)) == 0


# ------------------------------------------------ virtual-range tensors ----

def test_virtual_tensor_sequence_of_the_reference_unit_test(fake_runtime):
    """The steps of tests/unit/cuda/tensor.c:30-89, assertion for assertion."""
    with Backend() as b:
        before = b.memory_stats().allocated_bytes
        t = b.reserve("rocm_virtual_pages", B.DTYPE_I8, (16 << 20,))
        g = t.granularity
        assert g and t.handle.contents.virtual_reserved and t.resident_bytes == 0
        assert b.memory_stats().allocated_bytes == before      # an address range costs no memory
        assert fake_runtime.fake_hip_live_physical() == 0
        assert t.commit(g + 1, 1) == g and t.resident_bytes == g     # exactly one granule
        assert t.commit(g + 2, 1) == 0 and t.resident_bytes == g     # idempotent
        assert t.commit(3 * g, 1) == g and t.resident_bytes == 2 * g  # a disjoint granule
        view = t.view(g + 1, B.DTYPE_I8, (1,))
        view.write(np.array([0x5a], np.int8))
        assert view.read()[0] == 0x5a
        assert b.memory_stats().allocated_bytes == before + 2 * g
        assert t.decommit() == 2 * g and t.resident_bytes == 0 and not t.is_written
        assert b.memory_stats().allocated_bytes == before
        assert fake_runtime.fake_hip_live_physical() == 0 and fake_runtime.fake_hip_mapped_bytes() == 0
        assert fake_runtime.fake_hip_live_ranges() == 1        # the address range is kept
        t.release()
        assert t.handle is None and fake_runtime.fake_hip_live_ranges() == 0


def test_virtual_tensor_commit_is_zero_filled_granule_by_granule_and_checked(fake_runtime):
    with Backend(memory_limit_bytes=32 << 20) as b:
        t = b.reserve("history", B.DTYPE_I8, (64 << 21,))     # 64 granules
        g = t.granularity
        assert g == 2 << 20              # the stand-in runtime reports 64 KiB: 2 MiB is the floor
        # a span that touches five granules backs five, one equal-sized mapping each
        assert t.commit(2 * g + 5, 4 * g) == 5 * g and fake_runtime.fake_hip_live_physical() == 5
        assert np.all(t.view(2 * g, B.DTYPE_I8, (5 * g,)).read() == 0)   # fresh pages read as zero
        # a span around it adds only the missing granules on each side
        assert t.commit(g, 8 * g) == 3 * g and fake_runtime.fake_hip_live_physical() == 8
        assert b.memory_stats().allocated_bytes == 8 * g and t.resident_bytes == 8 * g
        assert fake_runtime.fake_hip_mapped_bytes() == 8 * g
        # the memory limit counts committed bytes: 32 MiB = 16 granules
        with pytest.raises(YvexError) as e:
            t.commit(20 * g, 9 * g)
        assert e.value.code == B.YVEX_ERR_NOMEM and "memory limit" in e.value.message
        assert t.resident_bytes == 8 * g and fake_runtime.fake_hip_live_physical() == 8
        assert t.commit(20 * g, 8 * g) == 8 * g
        # anything handed to the device must lie on committed pages
        for bad in (t.view(0, B.DTYPE_I8, (g + 1,)), t.view(9 * g - 1, B.DTYPE_I8, (2,)), t):
            with pytest.raises(YvexError) as e:
                bad.read()
            assert e.value.code == B.YVEX_ERR_STATE and "not committed" in e.value.message
            with pytest.raises(YvexError) as e:
                bad.zero()
            assert e.value.code == B.YVEX_ERR_STATE
        inside = t.view(g, B.DTYPE_I8, (8 * g,))
        inside.write(np.full(8 * g, 7, np.int8))
        assert np.all(inside.read() == 7)
        # a committed page that is given back and committed again reads as zero again
        assert t.decommit() == 16 * g
        assert t.commit(g, 1) == g and np.all(t.view(g, B.DTYPE_I8, (g,)).read() == 0)
        plain = b.tensor("plain", B.DTYPE_I8, (g + 1,))
        err = B.Error()
        assert lib().yvex_backend_tensor_copy(b.handle, plain.handle,
                                              t.view(0, B.DTYPE_I8, (g + 1,)).handle,
                                              C.byref(err)) == B.YVEX_ERR_STATE
        with pytest.raises(YvexError) as e:                     # not a workspace
            b.workspace_attach(t)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG


def test_virtual_tensor_refusals(env, fake_runtime):
    with Backend() as b:
        err, out, gran, delta = B.Error(), B.TensorP(), C.c_ulonglong(5), C.c_ulonglong(5)
        desc = B.TensorDesc(b"range", B.DTYPE_I8, 1)
        desc.dims[0] = desc.bytes = 1 << 22
        L = lib()
        assert L.yvex_backend_tensor_reserve(b.handle, C.byref(desc), None, C.byref(gran),
                                             C.byref(err)) == B.YVEX_ERR_INVALID_ARG and gran.value == 0
        assert L.yvex_backend_tensor_reserve(b.handle, C.byref(desc), C.byref(out), None,
                                             C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        desc.bytes = 0
        assert L.yvex_backend_tensor_reserve(b.handle, C.byref(desc), C.byref(out), C.byref(gran),
                                             C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        desc.bytes = 1 << 22
        t = b.reserve("range", B.DTYPE_I8, (1 << 22,))
        plain = b.tensor("plain", B.DTYPE_I8, (1 << 22,))
        for tensor, offset, count in ((t, 0, 0), (t, (1 << 22) + 1, 1), (t, 1 << 22, 1),
                                      (t, 5, 1 << 22), (plain, 0, 16)):
            delta.value = 5
            rc = L.yvex_backend_tensor_commit_range(b.handle, tensor.handle, offset, count,
                                                    C.byref(delta), C.byref(err))
            assert rc == B.YVEX_ERR_INVALID_ARG and delta.value == 0, (offset, count)
        assert L.yvex_backend_tensor_commit_range(b.handle, t.handle, 0, 1, None,
                                                  C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        assert L.yvex_backend_tensor_decommit(b.handle, plain.handle, C.byref(delta),
                                              C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        assert L.yvex_backend_tensor_decommit(b.handle, t.handle, None,
                                              C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        t.commit(0, 1)
        assert L.yvex_backend_tensor_decommit(b.handle, t.view(16, B.DTYPE_I8, (16,)).handle,
                                              C.byref(delta), C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        with Backend() as other:                                # a foreign backend's range
            assert L.yvex_backend_tensor_commit_range(other.handle, t.handle, 0, 1, C.byref(delta),
                                                      C.byref(err)) == B.YVEX_ERR_INVALID_ARG
            assert L.yvex_backend_tensor_decommit(other.handle, t.handle, C.byref(delta),
                                                  C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        b.graph_begin()                                         # not while recording
        for call in (lambda: b.reserve("late", B.DTYPE_I8, (1 << 20,)), lambda: t.commit(1 << 21, 1),
                     t.decommit):
            with pytest.raises(YvexError) as e:
                call()
            assert e.value.code == B.YVEX_ERR_STATE
        b.graph_release(b.graph_end())
        assert lib().yvex_backend_virtual_tensor_supported(b.handle) == 1
    assert lib().yvex_backend_virtual_tensor_supported(None) == 0
    env("FAKE_HIP_VIRTUAL_MEMORY", "absent")                    # a device without the feature
    with Backend() as b:
        assert lib().yvex_backend_virtual_tensor_supported(b.handle) == 0
        with pytest.raises(YvexError) as e:
            b.reserve("range", B.DTYPE_I8, (1 << 20,))
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED and "unavailable" in e.value.message
        assert f32(b, "still-works", (4,)).read().sum() == 0


@pytest.mark.parametrize("injected", ["FAKE_HIP_MAP", "FAKE_HIP_ACCESS", "FAKE_HIP_PHYSICAL_LIMIT"])
def test_virtual_tensor_failed_commit_leaves_nothing_behind(env, fake_runtime, injected):
    with Backend() as b:
        t = b.reserve("history", B.DTYPE_I8, (32 << 21,))
        g = t.granularity
        assert t.commit(4 * g, g) == g
        stats = b.memory_stats().allocated_bytes
        # two runs are missing around the committed granule; the limit lets the first through
        env(injected, "2" if injected == "FAKE_HIP_PHYSICAL_LIMIT" else "fail")
        with pytest.raises(YvexError) as e:
            t.commit(2 * g, 6 * g)
        assert e.value.code == B.YVEX_ERR_BACKEND
        assert b.status == B.STATUS_READY                       # rolled back cleanly: still usable
        assert t.resident_bytes == g and b.memory_stats().allocated_bytes == stats
        assert fake_runtime.fake_hip_live_physical() == 1 and fake_runtime.fake_hip_mapped_bytes() == g
        env(injected, None)
        assert t.commit(2 * g, 6 * g) == 5 * g                  # and the same commit then succeeds
        assert np.all(t.view(2 * g, B.DTYPE_I8, (6 * g,)).read() == 0)


def test_virtual_tensor_failed_release_keeps_the_owner(env, fake_runtime):
    b = Backend()
    t = b.reserve("history", B.DTYPE_I8, (8 << 21,))
    t.commit(0, 3 << 21)
    env("FAKE_HIP_UNMAP", "fail")
    with pytest.raises(YvexError) as e:
        t.decommit()
    assert e.value.code == B.YVEX_ERR_BACKEND and t.resident_bytes == 3 << 21
    with pytest.raises(YvexError):
        t.release()                                             # a failed release fails the backend
    assert t.handle is not None and b.status == B.STATUS_FAILED
    assert lib().yvex_backend_virtual_tensor_supported(b.handle) == 0   # a failed backend says no
    env("FAKE_HIP_UNMAP", None)
    t.release()                                                 # cleanup-only release still works
    assert fake_runtime.fake_hip_live_physical() == 0 and fake_runtime.fake_hip_live_ranges() == 0
    b.tensors.clear()
    b.close()


def test_virtual_tensor_views_outlive_nothing_and_count_on_the_owner(env, fake_runtime):
    """A view is a struct copy that carries the range pointer and the owner's id.  Commits
    through a view are counted on the tensor that owns the range; a view kept past the release
    of that tensor is refused everywhere instead of reading freed host state; a granule that a
    failed release left half done is finished by the next commit, not skipped."""
    b = Backend()
    owner = b.reserve("history", B.DTYPE_I8, (8 << 21,))
    view = owner.view(2 << 21, B.DTYPE_I8, (2 << 21,))
    assert view.commit(0, 2 << 21) == 2 << 21                   # granules 2 and 3
    assert owner.resident_bytes == 2 << 21
    assert b.memory_stats().allocated_bytes == 2 << 21
    view.zero()                                                 # backed: accepted
    # half-released granule: the unmap goes through, giving the memory back fails
    env("FAKE_HIP_RELEASE", "fail")
    with pytest.raises(YvexError) as e:
        owner.decommit()
    assert e.value.code == B.YVEX_ERR_BACKEND and b.status == B.STATUS_FAILED
    env("FAKE_HIP_RELEASE", None)
    owner.release()                                             # cleanup-only release finishes it
    assert fake_runtime.fake_hip_live_physical() == 0 and fake_runtime.fake_hip_live_ranges() == 0
    b.tensors.clear()
    b.close()
    # a stale view on a live backend
    b = Backend()
    owner = b.reserve("history", B.DTYPE_I8, (4 << 21,))
    owner.commit(0, 4 << 21)
    stale = owner.view(0, B.DTYPE_I8, (1 << 21,))
    target = b.tensor("target", B.DTYPE_I8, (1 << 21,))
    owner.release()
    again = b.reserve("again", B.DTYPE_I8, (4 << 21,))          # may reuse the freed host block
    again.commit(0, 4 << 21)
    err = B.Error()
    for call in (lambda: lib().yvex_backend_tensor_zero(b.handle, stale.handle, C.byref(err)),
                 lambda: lib().yvex_backend_tensor_copy(b.handle, target.handle, stale.handle, C.byref(err)),
                 lambda: lib().yvex_backend_tensor_copy_async(b.handle, target.handle, stale.handle,
                                                               C.byref(err))):
        assert call() == B.YVEX_ERR_STATE, err.message
    delta = C.c_ulonglong(0)
    assert lib().yvex_backend_tensor_commit_range(b.handle, stale.handle, 0, 1 << 21, C.byref(delta),
                                                  C.byref(err)) == B.YVEX_ERR_INVALID_ARG
    b.close()


# ------------------------------------------------- operation admission ----

def test_bounded_primitive_refusal_order_and_facts(fake_runtime):
    with Backend() as b:
        q, k, v = f32(b, "q", (4,), np.ones(4)), f32(b, "k", (3, 4), np.ones((3, 4))), \
            f32(b, "v", (3, 4), np.ones((3, 4)))
        s, p, o = f32(b, "s", (3,)), f32(b, "p", (3,)), f32(b, "o", (4,))
        before = fake_runtime.fake_hip_launches()
        b.op_attention(q, k, v, 3, 2, 0.5, True, s, p, o)
        assert fake_runtime.fake_hip_launches() == before + 1
        assert o.is_written and s.is_written and p.is_written
        cases = [((0, 0, 0.5), B.YVEX_ERR_INVALID_ARG), ((3, 3, 0.5), B.YVEX_ERR_BOUNDS),
                 ((3, 9, float("nan")), B.YVEX_ERR_BOUNDS),      # position is checked before scale
                 ((3, 0, float("nan")), B.YVEX_ERR_INVALID_ARG), ((3, 0, 0.0), B.YVEX_ERR_INVALID_ARG),
                 ((3, 0, -2.0), B.YVEX_ERR_INVALID_ARG)]
        for (seq, pos, scale), code in cases:
            with pytest.raises(YvexError) as e:
                b.op_attention(q, k, v, seq, pos, scale, True, s, p, o)
            assert e.value.code == code, (seq, pos, scale)
        with pytest.raises(YvexError) as e:                          # dtype before shape
            b.op_attention(q, k, v, 3, 0, 0.5, True, s, p, b.tensor("h", B.DTYPE_BF16, (9,)))
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED
        with pytest.raises(YvexError) as e:
            b.op_attention(q, k, v, 3, 0, 0.5, True, s, p, f32(b, "o5", (5,)))
        assert e.value.code == B.YVEX_ERR_FORMAT and "output must have dims" in e.value.message
        with pytest.raises(YvexError) as e:
            b.op_attention(q, f32(b, "k2", (4, 4)), v, 3, 0, 0.5, True, s, p, o)
        assert e.value.code == B.YVEX_ERR_FORMAT
        with pytest.raises(YvexError) as e:
            b.op_attention(f32(b, "q2", (2, 2)), k, v, 3, 0, 0.5, True, s, p, o)
        assert e.value.code == B.YVEX_ERR_FORMAT
        with Backend() as other:
            with pytest.raises(YvexError) as e:
                b.op_attention(f32(other, "q", (4,)), k, v, 3, 0, 0.5, True, s, p, o)
            assert e.value.code == B.YVEX_ERR_STATE
        err = B.Error()
        rc = lib().yvex_backend_op_attention(b.handle, None, k.handle, v.handle, 3, 0, 0.5, 1,
                                             s.handle, p.handle, o.handle, C.byref(err))
        assert rc == B.YVEX_ERR_INVALID_ARG


def test_attention_execute_contracts_facts_and_workspace(fake_runtime):
    with Backend() as b:
        # exact F32: one launch, one synchronisation, a 4-byte status read-back
        req = b.attention_requirement(3, 5, 4, 2, 64, query_start=2)
        q, k = written(b, "q", B.DTYPE_F32, (3, 4, 64)), written(b, "k", B.DTYPE_F32, (5, 2, 64))
        out = b.tensor("o", B.DTYPE_F32, (3, 4, 64))
        facts = b.attention_execute(req, q, k, k, out)
        assert (facts.kernel_launches, facts.device_synchronizations, facts.d2h_bytes,
                facts.download_count) == (1, 1, 4, 1) and out.is_written
        assert b.attention_workspace_required(req) == 0
        # bf16 decode: one launch (split segments are merged in the kernel), workspace == planned bytes, attached workspace is used
        req = b.attention_requirement(1, 4096, 32, 8, 128, query_start=4095, dtype=B.DTYPE_BF16,
                                      contract=B.NUMERIC_BF16_F32_ACCUMULATE)
        planned = b.attention_workspace_required(req)
        assert planned > 0 and planned % 256 == 0
        qb = written(b, "q", B.DTYPE_BF16, (1, 32, 128))
        kb = written(b, "k", B.DTYPE_BF16, (4096, 8, 128))
        ob = b.tensor("o", B.DTYPE_BF16, (1, 32, 128))
        live = fake_runtime.fake_hip_live_allocations()
        facts = b.attention_execute(req, qb, kb, kb, ob)
        assert facts.kernel_launches == 1 and facts.temporary_bytes == planned
        assert fake_runtime.fake_hip_live_allocations() == live      # temporary released
        work = b.tensor("workspace", B.DTYPE_I8, (planned,))
        b.workspace_attach(work)
        with pytest.raises(YvexError) as e:
            b.workspace_attach(work)
        assert e.value.code == B.YVEX_ERR_STATE
        live = fake_runtime.fake_hip_live_allocations()
        stats_before = b.memory_stats().allocation_events
        facts = b.attention_execute(req, qb, kb, kb, ob)
        assert facts.temporary_bytes == planned
        assert b.memory_stats().allocation_events == stats_before    # no counted temporary
        b.workspace_detach()
        # bf16 prefill: one launch
        req = b.attention_requirement(300, 300, 8, 2, 128, dtype=B.DTYPE_BF16,
                                      contract=B.NUMERIC_BF16_F32_ACCUMULATE)
        qp, kp = written(b, "q", B.DTYPE_BF16, (300, 8, 128)), written(b, "k", B.DTYPE_BF16, (300, 2, 128))
        facts = b.attention_execute(req, qp, kp, kp, b.tensor("o", B.DTYPE_BF16, (300, 8, 128)))
        assert facts.kernel_launches == 1 and facts.accelerated_matrix_launches == 1
        # refusals
        unwritten = b.tensor("k-unwritten", B.DTYPE_BF16, (300, 2, 128))
        with pytest.raises(YvexError) as e:
            b.attention_execute(req, qp, unwritten, kp, b.tensor("o", B.DTYPE_BF16, (300, 8, 128)))
        assert e.value.code == B.YVEX_ERR_FORMAT
        for mutate, code in [(dict(query_heads=9), B.YVEX_ERR_INVALID_ARG),
                             (dict(query_start=1), B.YVEX_ERR_INVALID_ARG),
                             (dict(key_token_stride=255), B.YVEX_ERR_INVALID_ARG),
                             (dict(head_dimension=96), B.YVEX_ERR_UNSUPPORTED),
                             (dict(deterministic=0), B.YVEX_ERR_UNSUPPORTED),
                             (dict(output_dtype=B.DTYPE_F32), B.YVEX_ERR_UNSUPPORTED),
                             (dict(numeric_contract=7), B.YVEX_ERR_UNSUPPORTED),
                             (dict(layout=0), B.YVEX_ERR_UNSUPPORTED)]:
            bad = b.attention_requirement(300, 300, 8, 2, 128, dtype=B.DTYPE_BF16,
                                          contract=B.NUMERIC_BF16_F32_ACCUMULATE)
            for key, value in mutate.items():
                setattr(bad, key, value)
            with pytest.raises(YvexError) as e:
                b.attention_workspace_required(bad)
            assert e.value.code == code, mutate


def test_paged_and_mla_admission():
    with Backend() as b:
        ok = b.paged_requirement(4, 32, 8, 128, 16, 100, 64, 1024)
        assert b.paged_decode_workspace_required(ok) > 0
        for mutate, code in [(dict(head_dimension=96), B.YVEX_ERR_UNSUPPORTED),
                             (dict(page_tokens=32), B.YVEX_ERR_UNSUPPORTED),
                             (dict(kv_storage=9), B.YVEX_ERR_UNSUPPORTED),
                             (dict(numeric_contract=B.NUMERIC_EXACT_F32), B.YVEX_ERR_UNSUPPORTED),
                             (dict(query_heads=33), B.YVEX_ERR_INVALID_ARG),
                             (dict(max_context_tokens=1025), B.YVEX_ERR_INVALID_ARG),
                             (dict(pool_pages=0), B.YVEX_ERR_INVALID_ARG)]:
            bad = b.paged_requirement(4, 32, 8, 128, 16, 100, 64, 1024)
            for key, value in mutate.items():
                setattr(bad, key, value)
            with pytest.raises(YvexError) as e:
                b.paged_decode_workspace_required(bad)
            assert e.value.code == code, mutate
        q = written(b, "q", B.DTYPE_BF16, (4, 32, 128))
        pool = written(b, "pool", B.DTYPE_BF16, (100 * 8 * 2048,))
        table, ctx = written(b, "t", B.DTYPE_I32, (4, 64)), written(b, "c", B.DTYPE_I32, (4,))
        out = b.tensor("o", B.DTYPE_BF16, (4, 32, 128))
        facts = b.paged_decode_execute(ok, q, pool, pool, table, ctx, out)
        assert facts.kernel_launches == 1 and out.is_written
        # the same pool read as 25 pages of 64 tokens (four 16-token blocks each)
        wide = b.paged_requirement(4, 32, 8, 128, 64, 25, 16, 1024)
        assert b.paged_decode_workspace_required(wide) == b.paged_decode_workspace_required(ok)
        wide_table = written(b, "t64", B.DTYPE_I32, (4, 16))
        assert b.paged_decode_execute(wide, q, pool, pool, wide_table, ctx, out).kernel_launches == 1
        small = written(b, "small-pool", B.DTYPE_BF16, (99 * 8 * 2048,))
        with pytest.raises(YvexError) as e:
            b.paged_decode_execute(ok, q, small, pool, table, ctx, out)
        assert e.value.code == B.YVEX_ERR_FORMAT
        mla = b.mla_requirement(16, 128, 576, 512, 64, 2048, 128, 8192)
        assert b.mla_decode_workspace_required(mla) > 0
        windowed = b.mla_requirement(16, 128, 576, 512, 64, 2048, 128, 8192, sliding_window=1024)
        assert 0 < b.mla_decode_workspace_required(windowed) < b.mla_decode_workspace_required(mla)
        mq = written(b, "mq", B.DTYPE_BF16, (16, 128, 576))
        latent = written(b, "latent", B.DTYPE_BF16, (2048, 64, 576))
        mtable, mctx = written(b, "mt", B.DTYPE_I32, (16, 128)), written(b, "mc", B.DTYPE_I32, (16,))
        mout = b.tensor("mo", B.DTYPE_BF16, (16, 128, 512))
        sinks = written(b, "sinks", B.DTYPE_F32, (128,))
        assert b.mla_decode_execute(windowed, mq, latent, mtable, mctx, mout, sinks=sinks).kernel_launches == 2
        both = b.mla_requirement(16, 128, 576, 512, 64, 2048, 128, 8192, compressed_pool_pages=40,
                                 compressed_table_stride=2, max_compressed_tokens=128)
        assert b.mla_decode_workspace_required(both) > b.mla_decode_workspace_required(mla)
        cpool = written(b, "cp", B.DTYPE_BF16, (40, 64, 576))
        ctable, ccount = written(b, "ct", B.DTYPE_I32, (16, 2)), written(b, "cc", B.DTYPE_I32, (16,))
        facts = b.mla_decode_execute(both, mq, latent, mtable, mctx, mout, compressed=[cpool, ctable, ccount])
        assert facts.kernel_launches == 3
        with pytest.raises(YvexError) as e:                 # declared but not passed
            b.mla_decode_execute(both, mq, latent, mtable, mctx, mout)
        assert e.value.code == B.YVEX_ERR_FORMAT
        chosen = b.mla_requirement(16, 128, 576, 512, 64, 2048, 128, 8192, compressed_pool_pages=40,
                                   compressed_table_stride=2, max_compressed_tokens=128,
                                   compressed_selected_stride=96)
        assert b.mla_decode_workspace_required(chosen) > b.mla_decode_workspace_required(both)
        lists = written(b, "sel", B.DTYPE_I32, (16, 96))
        facts = b.mla_decode_execute(chosen, mq, latent, mtable, mctx, mout,
                                     compressed=[cpool, ctable, ccount, lists])
        assert facts.kernel_launches == 4 and facts.accelerated_matrix_launches == 2
        with pytest.raises(YvexError) as e:                 # a list without the class declared on it
            b.mla_decode_execute(chosen, mq, latent, mtable, mctx, mout, compressed=[cpool, ctable, ccount])
        assert e.value.code == B.YVEX_ERR_FORMAT
        with pytest.raises(YvexError) as e:                 # a list needs a compressed set
            b.mla_decode_workspace_required(b.mla_requirement(
                16, 128, 576, 512, 64, 2048, 128, 8192, compressed_selected_stride=96))
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
        with pytest.raises(YvexError) as e:                 # more rows than the table can address
            b.mla_decode_workspace_required(b.mla_requirement(
                16, 128, 576, 512, 64, 2048, 128, 8192, compressed_pool_pages=40,
                compressed_table_stride=2, max_compressed_tokens=129))
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
        for wrong in (written(b, "s1", B.DTYPE_F32, (64,)), written(b, "s2", B.DTYPE_BF16, (128,)),
                      b.tensor("s3", B.DTYPE_F32, (128,))):
            with pytest.raises(YvexError) as e:
                b.mla_decode_execute(mla, mq, latent, mtable, mctx, mout, sinks=wrong)
            assert e.value.code == B.YVEX_ERR_FORMAT
        bad = b.mla_requirement(16, 64, 576, 512, 64, 2048, 128, 8192)
        with pytest.raises(YvexError) as e:
            b.mla_decode_workspace_required(bad)
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED


def test_kv_append_admission():
    """Refusal order of the page writer: arguments, then geometry the kernels do not cover,
    then tensor views; one launch, both pools marked written."""
    with Backend() as b:
        sessions, total, hkv, pages, stride = 3, 10, 8, 12, 4
        key = written(b, "k", B.DTYPE_BF16, (total, hkv, 128))
        value = written(b, "v", B.DTYPE_BF16, (total, hkv, 128))
        cosine, sine = written(b, "cos", B.DTYPE_F32, (total, 64)), written(b, "sin", B.DTYPE_F32, (total, 64))
        rows, starts, counts = (written(b, n, B.DTYPE_I32, (sessions,)) for n in ("r", "s", "c"))
        table = written(b, "t", B.DTYPE_I32, (sessions, stride))
        k_pool = b.tensor("kp", B.DTYPE_BF16, (pages * hkv * 2048,))
        v_pool = b.tensor("vp", B.DTYPE_BF16, (pages * hkv * 2048,))
        args = (key, value, rows, starts, counts, table, k_pool, v_pool, hkv, pages, 8)
        facts = b.kv_append_execute(*args, cosine=cosine, sine=sine, rotary_dimension=64)
        assert facts.kernel_launches == 1 and k_pool.is_written and v_pool.is_written
        # pages of 64 tokens: four 16-token blocks each, so a quarter of the pages hold the same rows
        wide_table = written(b, "t64", B.DTYPE_I32, (sessions, 1))
        assert b.kv_append_execute(key, value, rows, starts, counts, wide_table, k_pool, v_pool, hkv,
                                   pages // 4, 8, page_tokens=64).kernel_launches == 1
        q_pool = b.tensor("qp", B.DTYPE_I8, (pages * hkv * 2176,))
        assert b.kv_append_execute(key, value, rows, starts, counts, table, q_pool, q_pool, hkv,
                                   pages, 8, storage=B.KV_Q8_0).kernel_launches == 1
        for kwargs, code in [(dict(head_dimension=96), B.YVEX_ERR_UNSUPPORTED),
                             (dict(page_tokens=32), B.YVEX_ERR_UNSUPPORTED),
                             (dict(storage=7), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=24, cosine=cosine, sine=sine), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=256, cosine=cosine, sine=sine), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=64), B.YVEX_ERR_INVALID_ARG),        # no tables
                             (dict(rotary_dimension=128, cosine=cosine, sine=sine), B.YVEX_ERR_FORMAT)]:
            with pytest.raises(YvexError) as e:
                b.kv_append_execute(*args, **kwargs)
            assert e.value.code == code, kwargs
        with pytest.raises(YvexError) as e:        # pool one page short
            b.kv_append_execute(key, value, rows, starts, counts, table, k_pool, v_pool, hkv,
                                pages + 1, 8)
        assert e.value.code == B.YVEX_ERR_FORMAT
        with pytest.raises(YvexError) as e:        # a session cannot hold more rows than exist
            b.kv_append_execute(key, value, rows, starts, counts, table, k_pool, v_pool, hkv,
                                pages, total + 1)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
        unwritten = b.tensor("k2", B.DTYPE_BF16, (total, hkv, 128))
        with pytest.raises(YvexError) as e:
            b.kv_append_execute(unwritten, value, rows, starts, counts, table, k_pool, v_pool,
                                hkv, pages, 8)
        assert e.value.code == B.YVEX_ERR_FORMAT


def test_history_append_admission(fake_runtime):
    """Refusal order of the token-major history writer: arguments, geometry, what the kernel
    does not cover, then tensor views (uncommitted rows of a reserved range included)."""
    with Backend() as b:
        tokens, first, hkv, d = 5, 11, 4, 128
        width = hkv * d
        key = written(b, "k", B.DTYPE_BF16, (tokens, hkv, d))
        value = written(b, "v", B.DTYPE_BF16, (tokens, hkv, d))
        cosine, sine = written(b, "cos", B.DTYPE_F32, (tokens, 64)), written(b, "sin", B.DTYPE_F32, (tokens, 64))
        store = b.tensor("history", B.DTYPE_BF16, (first + tokens, 2 * width))
        count = (first + tokens - 1) * 2 * width + width
        kh, vh = store.view(0, B.DTYPE_BF16, (count,)), store.view(2 * width, B.DTYPE_BF16, (count,))
        args = (key, value, kh, vh, first, hkv)
        strides = dict(key_token_stride=2 * width, value_token_stride=2 * width)
        facts = b.history_append_execute(*args, cosine=cosine, sine=sine, rotary_dimension=64, **strides)
        assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
        assert kh.is_written and vh.is_written
        for kwargs, code in [(dict(head_dimension=0), B.YVEX_ERR_INVALID_ARG),
                             (dict(rotary_dimension=64), B.YVEX_ERR_INVALID_ARG),         # no tables
                             (dict(key_token_stride=width - 8), B.YVEX_ERR_INVALID_ARG),
                             (dict(key_token_stride=2 * width + 4), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=24, cosine=cosine, sine=sine), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=256, cosine=cosine, sine=sine), B.YVEX_ERR_UNSUPPORTED),
                             (dict(rotary_dimension=128, cosine=cosine, sine=sine), B.YVEX_ERR_FORMAT),
                             (dict(key_token_stride=width), B.YVEX_ERR_FORMAT)]:           # view too long
            merged = dict(strides)
            merged.update(kwargs)
            with pytest.raises(YvexError) as e:
                b.history_append_execute(*args, **merged)
            assert e.value.code == code, kwargs
        with pytest.raises(YvexError) as e:                         # one row beyond the views
            b.history_append_execute(key, value, kh, vh, first + 1, hkv, **strides)
        assert e.value.code == B.YVEX_ERR_FORMAT
        unwritten = b.tensor("k2", B.DTYPE_BF16, (tokens, hkv, d))
        with pytest.raises(YvexError) as e:
            b.history_append_execute(unwritten, value, kh, vh, first, hkv, **strides)
        assert e.value.code == B.YVEX_ERR_FORMAT
        # F32 rows go into F32 histories (the reference's own element type), not into BF16 ones
        key32 = written(b, "k32", B.DTYPE_F32, (tokens, hkv, d))
        store32 = b.tensor("history32", B.DTYPE_F32, (first + tokens, 2 * width))
        kh32 = store32.view(0, B.DTYPE_F32, (count,))
        vh32 = store32.view(4 * width, B.DTYPE_F32, (count,))
        assert b.history_append_execute(key32, key32, kh32, vh32, first, hkv, cosine=cosine, sine=sine,
                                        rotary_dimension=64, **strides).kernel_launches == 1
        for bad in ((key32, value, kh32, vh32), (key32, key32, kh, vh), (key, value, kh32, vh32)):
            with pytest.raises(YvexError) as e:
                b.history_append_execute(*bad, first, hkv, **strides)
            assert e.value.code == B.YVEX_ERR_FORMAT
        with pytest.raises(YvexError) as e:                         # rotary halves of 4 F32 lanes
            b.history_append_execute(key32, key32, kh32, vh32, first, hkv, cosine=cosine, sine=sine,
                                     rotary_dimension=12, **strides)
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED
        ints = written(b, "ints", B.DTYPE_I32, (tokens, hkv, d))
        with pytest.raises(YvexError) as e:
            b.history_append_execute(ints, ints, kh32, vh32, first, hkv, **strides)
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED
        # a history in a reserved range: the rows must be committed first
        row_bytes = 2 * width * 2
        reserved = b.reserve("reserved-history", B.DTYPE_BF16, (8192, 2 * width))
        rk = reserved.view(0, B.DTYPE_BF16, (count,))
        rv = reserved.view(2 * width, B.DTYPE_BF16, (count,))
        with pytest.raises(YvexError) as e:
            b.history_append_execute(key, value, rk, rv, first, hkv, **strides)
        assert e.value.code == B.YVEX_ERR_STATE and "not committed" in e.value.message
        reserved.commit(0, (first + tokens) * row_bytes)
        assert b.history_append_execute(key, value, rk, rv, first, hkv, **strides).kernel_launches == 1
        # the optional query tensor: its pieces join the launch; it comes with its head count, has
        # the element type and geometry of the new rows and overlaps nothing else
        hq = 12
        query = written(b, "q", B.DTYPE_BF16, (tokens, hq, d))
        assert b.history_append_execute(*args, query=query, query_heads=hq, **strides).kernel_launches == 1
        fake_runtime.fake_hip_last_grid_x.restype = C.c_uint
        assert fake_runtime.fake_hip_last_grid_x() == (tokens * (hkv + hq) * (d // 8) + 255) // 256
        for kwargs, code in [(dict(query=query), B.YVEX_ERR_INVALID_ARG),
                             (dict(query_heads=hq), B.YVEX_ERR_INVALID_ARG),
                             (dict(query=query, query_heads=hq + 1), B.YVEX_ERR_FORMAT),
                             (dict(query=query, query_heads=65536), B.YVEX_ERR_UNSUPPORTED),
                             (dict(query=key32, query_heads=hkv), B.YVEX_ERR_FORMAT),
                             (dict(query=key, query_heads=hkv), B.YVEX_ERR_INVALID_ARG),
                             (dict(query=b.tensor("q2", B.DTYPE_BF16, (tokens, hq, d)), query_heads=hq),
                              B.YVEX_ERR_FORMAT)]:
            with pytest.raises(YvexError) as e:
                b.history_append_execute(*args, **kwargs, **strides)
            assert e.value.code == code, kwargs


def test_fused_gate_admission():
    """The epilogue entry points: an epilogue is required, the gate has the output geometry
    and is a written tensor other than the output, and only the BF16 contract takes one."""
    with Backend() as b:
        ops = b.rocm_attention_operations()
        req = b.attention_requirement(4, 4, 2, 1, 128, dtype=B.DTYPE_BF16,
                                      contract=B.NUMERIC_BF16_F32_ACCUMULATE)
        q = written(b, "q", B.DTYPE_BF16, (4, 2, 128))
        k, v = written(b, "k", B.DTYPE_BF16, (4, 1, 128)), written(b, "v", B.DTYPE_BF16, (4, 1, 128))
        out = b.tensor("o", B.DTYPE_BF16, (4, 2, 128))
        gate = written(b, "g", B.DTYPE_BF16, (4, 2, 128))
        assert b.attention_execute(req, q, k, v, out, gate=gate).kernel_launches == 1
        assert out.is_written
        request = B.AttentionRequest(req, q.handle, k.handle, v.handle, out.handle)
        facts, err = B.OperationFacts(), B.Error()
        assert ops.attention_execute_fused(b.handle, C.byref(request), None, None, C.byref(facts),
                                           C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        empty = B.AttentionEpilogue(None)
        assert ops.attention_execute_fused(b.handle, C.byref(request), C.byref(empty), None,
                                           C.byref(facts), C.byref(err)) == B.YVEX_ERR_INVALID_ARG
        for bad in (written(b, "g1", B.DTYPE_BF16, (4, 2, 64)), written(b, "g2", B.DTYPE_F32, (4, 2, 128)),
                    b.tensor("g3", B.DTYPE_BF16, (4, 2, 128)), out):
            with pytest.raises(YvexError) as e:
                b.attention_execute(req, q, k, v, out, gate=bad)
            assert e.value.code == B.YVEX_ERR_FORMAT
        paged = b.paged_requirement(4, 32, 8, 128, 16, 100, 64, 1024)
        pq = written(b, "pq", B.DTYPE_BF16, (4, 32, 128))
        pool = written(b, "pool", B.DTYPE_BF16, (100 * 8 * 2048,))
        table, ctx = written(b, "t", B.DTYPE_I32, (4, 64)), written(b, "c", B.DTYPE_I32, (4,))
        pout = b.tensor("po", B.DTYPE_BF16, (4, 32, 128))
        pgate = written(b, "pg", B.DTYPE_BF16, (4, 32, 128))
        assert b.paged_decode_execute(paged, pq, pool, pool, table, ctx, pout, gate=pgate).kernel_launches == 1
        with pytest.raises(YvexError) as e:
            b.paged_decode_execute(paged, pq, pool, pool, table, ctx, pout, gate=gate)
        assert e.value.code == B.YVEX_ERR_FORMAT


def test_recorded_sequence_rules(fake_runtime):
    """Recording: operations launch into the sequence, everything that allocates, copies,
    clears or waits is refused, a replay counts the recorded launches."""
    with Backend() as b:
        req = b.attention_requirement(1, 300, 8, 2, 128, query_start=299, dtype=B.DTYPE_BF16,
                                      contract=B.NUMERIC_BF16_F32_ACCUMULATE)
        q = written(b, "q", B.DTYPE_BF16, (1, 8, 128))
        k, v = written(b, "k", B.DTYPE_BF16, (300, 2, 128)), written(b, "v", B.DTYPE_BF16, (300, 2, 128))
        out = b.tensor("o", B.DTYPE_BF16, (1, 8, 128))
        with pytest.raises(YvexError) as e:
            b.graph_end()
        assert e.value.code == B.YVEX_ERR_STATE
        b.graph_begin()
        with pytest.raises(YvexError) as e:                   # no workspace: would allocate
            b.attention_execute(req, q, k, v, out)
        assert e.value.code == B.YVEX_ERR_STATE
        for call in (lambda: b.tensor("x", B.DTYPE_F32, (4,)), lambda: q.zero(), lambda: q.read(),
                     lambda: q.release(), b.sync, b.graph_begin, b.timing_begin,
                     lambda: b.set_completion_mode(B.COMPLETION_DEFERRED)):
            with pytest.raises(YvexError) as e:
                call()
            assert e.value.code == B.YVEX_ERR_STATE
        empty = b.graph_end()                                  # an empty sequence is legal
        assert b.graph_launch(empty).kernel_launches == 0
        b.graph_release(empty)
        work = b.tensor("work", B.DTYPE_I8, (b.attention_workspace_required(req) + (1 << 20),))
        b.workspace_attach(work)
        before = fake_runtime.fake_hip_launches()
        b.graph_begin()
        facts = b.attention_execute(req, q, k, v, out)
        assert facts.kernel_launches == 1 and facts.device_synchronizations == 0
        assert fake_runtime.fake_hip_launches() == before      # recorded, not run
        graph = b.graph_end()
        for n in (1, 2, 3):
            facts = b.graph_launch(graph)
            assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
            assert fake_runtime.fake_hip_launches() == before + n
        b.set_completion_mode(B.COMPLETION_DEFERRED)
        assert b.graph_launch(graph).device_synchronizations == 0
        b.sync()
        b.set_completion_mode(B.COMPLETION_IMMEDIATE)
        # the sequence holds device addresses: nothing it may name can be freed while it lives,
        # and it is not replayed without the workspace it was recorded with
        live = fake_runtime.fake_hip_live_allocations()
        for tensor in (q, out, work):
            with pytest.raises(YvexError) as e:
                tensor.release()
            assert e.value.code == B.YVEX_ERR_STATE and "recorded launch sequence" in e.value.message
        assert fake_runtime.fake_hip_live_allocations() == live
        later = b.tensor("later", B.DTYPE_F32, (16,))         # allocated after the recording:
        later.release()                                        # the sequence cannot name it
        assert fake_runtime.fake_hip_live_allocations() == live
        b.workspace_detach()
        launched = fake_runtime.fake_hip_launches()
        with pytest.raises(YvexError) as e:
            b.graph_launch(graph)
        assert e.value.code == B.YVEX_ERR_STATE and "workspace" in e.value.message
        assert fake_runtime.fake_hip_launches() == launched
        b.workspace_attach(work)
        assert b.graph_launch(graph).kernel_launches == 1
        b.graph_release(graph)
        b.workspace_detach()
        work.release()
        assert fake_runtime.fake_hip_live_allocations() == live - 1


def test_bandwidth_probe_record(env, fake_runtime):
    """Five samples of eight passes each for the read and for the copy, medians published,
    the working set released, the first evidence kept."""
    env("YVEX_TEST_ROCM_BANDWIDTH_BYTES", str(1 << 20))
    with Backend() as b:
        live, launches = fake_runtime.fake_hip_live_allocations(), fake_runtime.fake_hip_launches()
        e = b.bandwidth_probe()
        assert e.schema_version == 1 and e.working_set_bytes == 1 << 20
        assert e.iterations == 8 and e.sample_count == 5
        assert fake_runtime.fake_hip_launches() == launches + 1 + 5 * 8
        assert fake_runtime.fake_hip_live_allocations() == live
        assert all(x > 0 for x in e.stream_elapsed_ns) and all(x > 0 for x in e.copy_elapsed_ns)
        assert e.sustainable_read_bytes_per_second > 0 and e.sustainable_copy_bytes_per_second > 0
        assert list(e.coherent_host_elapsed_ns) == [0] * 5
        again = b.bandwidth_probe()
        assert fake_runtime.fake_hip_launches() == launches + 1 + 5 * 8       # not measured twice
        assert again.sustainable_read_bytes_per_second == e.sustainable_read_bytes_per_second
        b.graph_begin()
        b.graph_release(b.graph_end())


# ------------------------------------------------- failure transitions ----

def test_launch_failure_fails_only_that_variant(env):
    with Backend() as b:
        q, k = f32(b, "q", (4,), np.ones(4)), f32(b, "k", (3, 4), np.ones((3, 4)))
        s, o = f32(b, "s", (3,)), f32(b, "o", (4,))
        env("YVEX_TEST_ROCM_LAUNCH_FAILURE", "attention-causal-f32")
        with pytest.raises(YvexError) as e:
            b.op_attention(q, k, k, 3, 0, 0.5, True, s, s, o)
        assert e.value.code == B.YVEX_ERR_BACKEND and not o.is_written
        env("YVEX_TEST_ROCM_LAUNCH_FAILURE", None)
        r = b.query_capability(B.VARIANT_ATTENTION_CAUSAL_F32)
        assert r.state == B.CAPABILITY_FAILED and r.reason == B.REASON_LAUNCH_FAILED
        assert b.status == B.STATUS_READY                             # backend survives
        assert b.query_capability(B.VARIANT_ROCM_GQA_F32).state == B.CAPABILITY_SUPPORTED
        with pytest.raises(YvexError) as e:                           # the failed variant stays failed
            b.op_attention(q, k, k, 3, 0, 0.5, True, s, s, o)
        assert e.value.code == B.YVEX_ERR_BACKEND
        b.op_attention(q, k, k, 3, 0, 0.5, False, s, s, o)            # non-causal variant unaffected


def test_runtime_launch_error_is_reported(env):
    with Backend() as b:
        req = b.attention_requirement(2, 2, 2, 1, 8)
        q, k = written(b, "q", B.DTYPE_F32, (2, 2, 8)), written(b, "k", B.DTYPE_F32, (2, 1, 8))
        out = b.tensor("o", B.DTYPE_F32, (2, 2, 8))
        env("FAKE_HIP_LAUNCH", "fail")
        with pytest.raises(YvexError) as e:
            b.attention_execute(req, q, k, k, out)
        assert e.value.code == B.YVEX_ERR_BACKEND and "HIP error" in e.value.message
        assert not out.is_written
        assert b.query_capability(B.VARIANT_ROCM_GQA_F32).reason == B.REASON_LAUNCH_FAILED


def test_synchronisation_failure_fails_the_backend(env):
    b = Backend()
    q, k = f32(b, "q", (4,), np.ones(4)), f32(b, "k", (3, 4), np.ones((3, 4)))
    s, o = f32(b, "s", (3,)), f32(b, "o", (4,))
    env("YVEX_TEST_ROCM_SYNC_FAILURE", "all")
    with pytest.raises(YvexError) as e:
        b.op_attention(q, k, k, 3, 0, 0.5, True, s, s, o)
    assert e.value.code == B.YVEX_ERR_BACKEND
    env("YVEX_TEST_ROCM_SYNC_FAILURE", None)
    assert b.status == B.STATUS_FAILED
    r = b.query_capability(B.VARIANT_ATTENTION_CAUSAL_F32)
    assert r.state == B.CAPABILITY_FAILED and r.reason == B.REASON_SYNCHRONIZATION_FAILED
    with pytest.raises(YvexError) as e:
        b.op_attention(q, k, k, 3, 0, 0.5, True, s, s, o)
    assert e.value.code == B.YVEX_ERR_STATE and "cleanup only" in e.value.message
    with pytest.raises(YvexError) as e:
        b.tensor("late", B.DTYPE_F32, (4,))
    assert e.value.code == B.YVEX_ERR_STATE
    b.close()                                                      # checked close still discharges


def test_checked_close_retains_the_owner_until_cleanup_succeeds(env, fake_runtime):
    handle, err = C.c_void_p(), B.Error()
    options = B.BackendOptions(B.KIND_ROCM, None, 0)
    assert lib().yvex_backend_open(C.byref(handle), C.byref(options), C.byref(err)) == 0
    env("YVEX_TEST_ROCM_CLEANUP_FAILURE", "1")
    rc = lib().yvex_backend_close_checked(C.byref(handle), C.byref(err))
    assert rc == B.YVEX_ERR_BACKEND and handle.value                # owner retained for a retry
    result = B.CapabilityResult()
    lib().yvex_backend_query_capability(handle, B.VARIANT_TENSOR_ALLOC, C.byref(result), C.byref(err))
    assert result.state == B.CAPABILITY_FAILED and result.reason == B.REASON_CLEANUP_FAILED
    env("YVEX_TEST_ROCM_CLEANUP_FAILURE", None)
    assert lib().yvex_backend_close_checked(C.byref(handle), C.byref(err)) == 0
    assert not handle.value and fake_runtime.fake_hip_live_modules() == 0
    assert lib().yvex_backend_close_checked(C.byref(handle), C.byref(err)) == 0   # idempotent


def test_deferred_completion_checks_status_at_sync():
    with Backend() as b:
        req = b.attention_requirement(2, 2, 2, 1, 8)
        q, k = written(b, "q", B.DTYPE_F32, (2, 2, 8)), written(b, "k", B.DTYPE_F32, (2, 1, 8))
        out = b.tensor("o", B.DTYPE_F32, (2, 2, 8))
        b.set_completion_mode(B.COMPLETION_DEFERRED)
        d2h = b.memory_stats().d2h_bytes
        facts = b.attention_execute(req, q, k, k, out)
        assert facts.device_synchronizations == 0 and facts.d2h_bytes == 0
        assert b.memory_stats().d2h_bytes == d2h
        b.sync()                                                   # reads the status word once
        assert b.memory_stats().d2h_bytes == d2h + 4
        b.set_completion_mode(B.COMPLETION_IMMEDIATE)
        b.timing_begin()
        assert b.timing_end() == 1.0
        with pytest.raises(YvexError) as e:
            b.timing_end()
        assert e.value.code == B.YVEX_ERR_STATE


# ------------------------------------------------ codecs and page layout ----

def test_host_codecs_match_the_oracle_bit_for_bit():
    library = lib()
    bits = np.arange(1 << 16, dtype=np.uint16)
    for b16 in bits[::7]:
        f = ORACLE.lib.yvo_f16_decode(int(b16))
        g = library.yvex_quant_f16_decode(int(b16))
        assert (np.isnan(f) and np.isnan(g)) or np.float32(f).view(np.uint32) == np.float32(g).view(np.uint32)
        assert np.float32(ORACLE.lib.yvo_bf16_decode(int(b16))).view(np.uint32) == \
            np.float32(library.yvex_quant_bf16_decode(int(b16))).view(np.uint32) or np.isnan(g)
    rng = np.random.default_rng(17)
    x = np.concatenate([rng.standard_normal(6000) * s for s in (1e-8, 3e-8, 1e-5, 1e-3, 1.0, 7e4)])
    x = np.concatenate([x, [0.0, -0.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 6.1e-5,
                            np.inf, -np.inf]]).astype(np.float32)
    for value in x:
        assert library.yvex_quant_f16_encode(float(value)) == ORACLE.lib.yvo_f16_encode(float(value)), value
        assert library.yvex_quant_bf16_encode(float(value)) == ORACLE.lib.yvo_bf16_encode(float(value))
    rows = (rng.standard_normal((300, 128)) * rng.uniform(1e-4, 30, (300, 1))).astype(np.float32)
    rows[0] = 0.0
    enc = q8_0_encode_rows(rows)
    assert np.array_equal(enc, ORACLE.q8_0_encode_rows(rows))
    assert np.array_equal(q8_0_decode_rows(enc, 128).view(np.uint32),
                          ORACLE.q8_0_decode_rows(enc, 128).view(np.uint32))
    golden = np.zeros(32, np.float32)
    golden[:4] = [127.0, -127.0, 0.5, -0.5]
    assert bytes(q8_0_encode_rows(golden)[:6]) == bytes([0x00, 0x3C, 0x7F, 0x81, 0x01, 0xFF])
    with pytest.raises(YvexError) as e:
        q8_0_encode_rows(np.full(32, np.finfo(np.float32).max, np.float32))
    assert e.value.code == B.YVEX_ERR_BOUNDS
    bad = np.zeros(34, np.uint8)
    bad[1] = 0x7C
    with pytest.raises(YvexError) as e:
        q8_0_decode_rows(bad, 32)
    assert e.value.code == B.YVEX_ERR_FORMAT


def test_page_layouts_follow_the_documented_index_formulas():
    rng = np.random.default_rng(23)
    pages, hkv, d = 3, 2, 128
    rows = rng.integers(0, 1 << 16, size=(pages, 16, hkv, d), dtype=np.uint16)
    for is_value in (False, True):
        packed = kv_pack_pages(rows, B.KV_BF16, is_value, hkv).view(np.uint16).reshape(pages, hkv, 2048)
        t, c = np.meshgrid(np.arange(16), np.arange(d), indexing="ij")
        index = c * 16 + t if is_value else ((c // 8) * 16 + t) * 8 + c % 8
        for page in range(pages):
            for head in range(hkv):
                assert np.array_equal(packed[page, head][index], rows[page, :, head, :])
        back = kv_unpack_pages(packed, B.KV_BF16, is_value, pages, hkv)
        assert np.array_equal(back, rows)
    blocks = rng.integers(0, 256, size=(pages, 16, hkv, 4 * 34), dtype=np.uint8)
    for is_value in (False, True):
        packed = kv_pack_pages(blocks, B.KV_Q8_0, is_value, hkv).reshape(pages, hkv, 2176)
        canon = blocks.reshape(pages, 16, hkv, 4, 34)
        t, c = np.meshgrid(np.arange(16), np.arange(d), indexing="ij")
        if is_value:
            lane_byte = (((t // 4) * 16 + c % 16) * 8 + c // 16) * 4 + t % 4
        else:
            lane_byte = ((((c % 32) // 8) * 16 + t) * 4 + c // 32) * 8 + c % 8
        # byte r of the 32 a lane consumes lies at (r // 16) * 1024 + 16 * lane + r % 16
        index = ((lane_byte & 16) << 6) + ((lane_byte >> 5) << 4) + (lane_byte & 15)
        for page in range(pages):
            for head in range(hkv):
                codes = canon[page, :, head, :, 2:].reshape(16, d)
                assert np.array_equal(packed[page, head, :2048][index], codes)
                scales = canon[page, :, head, :, :2].reshape(16 * 4 * 2)
                assert np.array_equal(packed[page, head, 2048:], scales)
        assert np.array_equal(kv_unpack_pages(packed, B.KV_Q8_0, is_value, pages, hkv), blocks)
    # a page of 64 tokens is four 16-token blocks, one behind the other, per (page, kv head)
    for storage, wide, width in ((B.KV_BF16, rng.integers(0, 1 << 16, size=(pages, 64, hkv, d), dtype=np.uint16), 4096),
                                 (B.KV_Q8_0, rng.integers(0, 256, size=(pages, 64, hkv, 4 * 34), dtype=np.uint8), 2176)):
        for is_value in (False, True):
            packed = kv_pack_pages(wide, storage, is_value, hkv, page_tokens=64).reshape(pages, hkv, 4, width)
            as_blocks = wide.reshape((pages * 4, 16) + wide.shape[2:])
            narrow = kv_pack_pages(as_blocks, storage, is_value, hkv).reshape(pages, 4, hkv, width)
            assert np.array_equal(packed, narrow.transpose(0, 2, 1, 3))
            back = kv_unpack_pages(packed, storage, is_value, pages, hkv, page_tokens=64)
            assert np.array_equal(back.reshape(wide.shape), wide)
    assert lib().yvex_rocm_kv_page_block_bytes(B.KV_BF16, 128, 64) == 4 * 4096
    assert lib().yvex_rocm_kv_page_block_bytes(B.KV_Q8_0, 128, 64) == 4 * 2176
    assert lib().yvex_rocm_kv_page_block_bytes(B.KV_BF16, 128, 32) == 0
    with pytest.raises(YvexError) as e:
        kv_pack_pages(rows, B.KV_BF16, False, hkv, head_dim=96)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    with pytest.raises(YvexError) as e:
        kv_pack_pages(rng.integers(0, 256, size=(pages, 16, hkv, 2 * 34), dtype=np.uint8), B.KV_Q8_0, False,
                      hkv, head_dim=64)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    # bf16 pages at head dimension 64 and 256: the same index formulas with other chunk counts
    for width in (64, 256):
        wide_rows = rng.integers(0, 1 << 16, size=(pages, 16, hkv, width), dtype=np.uint16)
        assert lib().yvex_rocm_kv_page_block_bytes(B.KV_BF16, width, 16) == 16 * width * 2
        for is_value in (False, True):
            packed = kv_pack_pages(wide_rows, B.KV_BF16, is_value, hkv, head_dim=width).view(np.uint16)
            packed = packed.reshape(pages, hkv, 16 * width)
            t, c = np.meshgrid(np.arange(16), np.arange(width), indexing="ij")
            index = c * 16 + t if is_value else ((c // 8) * 16 + t) * 8 + c % 8
            for page in range(pages):
                for head in range(hkv):
                    assert np.array_equal(packed[page, head][index], wide_rows[page, :, head, :])
            back = kv_unpack_pages(packed, B.KV_BF16, is_value, pages, hkv, head_dim=width)
            assert np.array_equal(back, wide_rows)


def test_elementwise_slots_validate_like_the_reference():
    """The element-wise slots of the transformer operations table on the stand-in runtime: one
    launch and one synchronisation each, outputs marked written, and YVEX_ERR_FORMAT for anything
    but packed, written F32 tensors of this backend with the declared counts
    (src/backend/cuda/transformer.c:409-441,1356-1372, src/backend/cuda/decoder.c:11-47,75-103);
    a backend that is closing refuses first (YVEX_ERR_STATE)."""
    with Backend() as b, Backend() as other:
        x = written(b, "x", B.DTYPE_F32, (2, 4, 16))
        table = written(b, "t", B.DTYPE_F32, (2, 8))
        out, gate = b.tensor("o", B.DTYPE_F32, (2, 4, 16)), written(b, "g", B.DTYPE_F32, (2, 4, 16))
        first, second = b.tensor("a", B.DTYPE_F32, (64,)), b.tensor("b", B.DTYPE_F32, (64,))
        for facts in (b.rotary_half_f32(x, table, table, 2, 4, 16, 8), b.bf16_round(x, 128),
                      b.sigmoid_product_bf16(x, gate, out, 128),
                      b.split_interleaved_two_f32(x, first, second, 2, 2, 16)):
            assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
        assert out.is_written and first.is_written and second.is_written
        foreign = written(other, "f", B.DTYPE_F32, (2, 4, 16))
        half = written(b, "h", B.DTYPE_BF16, (128,))
        fresh = b.tensor("n", B.DTYPE_F32, (128,))
        for call in (lambda: b.rotary_half_f32(x, table, table, 2, 4, 16, 7),
                     lambda: b.rotary_half_f32(x, table, table, 2, 4, 16, 0),
                     lambda: b.rotary_half_f32(x, table, table, 2, 4, 16, 32),
                     lambda: b.rotary_half_f32(x, table, table, 2, 4, 16, 16),   # tables too short
                     lambda: b.rotary_half_f32(foreign, table, table, 2, 4, 16, 8),
                     lambda: b.rotary_half_f32(fresh, table, table, 2, 4, 16, 8),
                     lambda: b.bf16_round(x, 127), lambda: b.bf16_round(half, 128),
                     lambda: b.bf16_round(fresh, 128),
                     lambda: b.sigmoid_product_bf16(x, fresh, out, 128),
                     lambda: b.sigmoid_product_bf16(x, gate, half, 128),
                     lambda: b.sigmoid_product_bf16(x, gate, out, 0),
                     lambda: b.split_interleaved_two_f32(x, first, first, 2, 2, 16),
                     lambda: b.split_interleaved_two_f32(x, first, second, 2, 4, 16)):
            with pytest.raises(YvexError) as e:
                call()
            assert e.value.code == B.YVEX_ERR_FORMAT


def test_causal_exact_prefill_gets_item_lists_with_equal_work_per_unit(fake_runtime, env):
    """A causal EXACT_F32 prefill geometry that comes twice in a row is launched as 2 x 256 lists
    of items (the stand-in runtime reports 256 compute units): every item exactly once, no list
    longer than a row holds, and every unit (lists u and u + 256) within one item step of the
    mean number of key tiles; the first launch of a geometry, and launches too small to fill
    the units twice, keep one item per workgroup."""
    fake_runtime.fake_hip_last_grid_x.restype = C.c_uint
    fake_runtime.fake_hip_last_params.restype = C.POINTER(C.c_ubyte)
    env("FAKE_HIP_PARAM_BYTES", "176")
    tokens, hq, hkv, d = 2048, 40, 8, 128
    items = hq * (tokens // 128)
    with Backend() as b:
        q = written(b, "q", B.DTYPE_F32, (tokens, hq, d))
        k, v = written(b, "k", B.DTYPE_F32, (tokens, hkv, d)), written(b, "v", B.DTYPE_F32, (tokens, hkv, d))
        out = b.tensor("o", B.DTYPE_F32, (tokens, hq, d))
        req = b.attention_requirement(tokens, tokens, hq, hkv, d, causal=True)

        def launch():
            b.attention_execute(req, q, k, v, out)
            raw = bytes(fake_runtime.fake_hip_last_params()[:176])
            pair_units = int.from_bytes(raw[160:164], "little")
            lists = int.from_bytes(raw[168:176], "little")
            return fake_runtime.fake_hip_last_grid_x(), pair_units, lists

        grid, pair_units, lists = launch()
        assert grid == items and pair_units == 256 and lists == 0     # first time: pairs only
        grid, pair_units, lists = launch()
        assert grid == 512 and pair_units == 0 and lists != 0
        rows = np.ctypeslib.as_array(C.cast(lists, C.POINTER(C.c_uint16)), shape=(512, 8)).copy()
        counts = rows[:, 0].astype(int)
        assert counts.max() <= 7
        seen = np.concatenate([rows[i, 1:1 + counts[i]] for i in range(512)])
        assert sorted(seen.tolist()) == list(range(items))
        steps = lambda item: 4 * (16 - item // hq)                     # key tiles of 32 an item walks
        per_unit = [sum(steps(i) for i in rows[u, 1:1 + counts[u]]) + sum(steps(i) for i in rows[u + 256, 1:1 + counts[u + 256]])
                    for u in range(256)]
        mean = sum(per_unit) / 256.0
        assert max(per_unit) - min(per_unit) <= 8 and max(per_unit) <= mean + 6, (min(per_unit), max(per_unit), mean)
        for u in range(512):                                            # heaviest first within a list
            assert list(rows[u, 1:1 + counts[u]]) == sorted(rows[u, 1:1 + counts[u]])
        assert launch() == (512, 0, lists)                              # kept while the geometry repeats
        # too few items to fill the units twice are never scheduled (and leave the lists alone)
        small = b.attention_requirement(1024, 1024, 8, 8, d, causal=True)
        q2 = written(b, "q2", B.DTYPE_F32, (1024, 8, d))
        k2, v2 = written(b, "k2", B.DTYPE_F32, (1024, 8, d)), written(b, "v2", B.DTYPE_F32, (1024, 8, d))
        out2 = b.tensor("o2", B.DTYPE_F32, (1024, 8, d))
        for _ in range(3):
            b.attention_execute(small, q2, k2, v2, out2)
            assert fake_runtime.fake_hip_last_grid_x() == 64
        assert launch()[0] == 512
        # another geometry that can be scheduled takes the place of the first, which starts over
        other = b.attention_requirement(1024, tokens, hq, hkv, d, causal=True, query_start=1024)
        q3, out3 = written(b, "q3", B.DTYPE_F32, (1024, hq, d)), b.tensor("o3", B.DTYPE_F32, (1024, hq, d))
        b.attention_execute(other, q3, k, v, out3)
        assert fake_runtime.fake_hip_last_grid_x() == 8 * hq
        b.attention_execute(other, q3, k, v, out3)
        assert fake_runtime.fake_hip_last_grid_x() == 512
        assert launch()[0] == items


def test_single_token_bf16_requests_take_the_team_kernels_at_every_head_dimension(fake_runtime):
    """One query token over a token-major bf16 history: teams of waves at head dimension 64,
    128 and 256 for groups of at most eight query heads (grid = teams x kv heads, the
    workspace holds one partial per team), the one-row prefill tile for wider groups at 64
    and 256 (no workspace)."""
    fake_runtime.fake_hip_last_grid_x.restype = C.c_uint
    with Backend() as b:
        for d, hq, hkv, ctx, grid, partials in [(128, 32, 8, 4096, 16, True), (64, 16, 4, 4096, 16, True),
                                                (256, 24, 4, 4096, 16, True), (256, 24, 4, 300, 2, True),
                                                (256, 24, 4, 100000, 32, True), (64, 4, 4, 16, 1, True),
                                                (256, 32, 2, 4096, 32, False), (64, 12, 1, 300, 12, False)]:
            req = b.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1,
                                          dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
            q, out = written(b, "q", B.DTYPE_BF16, (1, hq, d)), b.tensor("o", B.DTYPE_BF16, (1, hq, d))
            k, v = written(b, "k", B.DTYPE_BF16, (ctx, hkv, d)), written(b, "v", B.DTYPE_BF16, (ctx, hkv, d))
            need = b.attention_workspace_required(req)
            facts = b.attention_execute(req, q, k, v, out)
            label = (d, hq, hkv, ctx)
            assert facts.kernel_launches == 1, label
            assert fake_runtime.fake_hip_last_grid_x() == grid, label
            assert (need > 0) == partials and facts.temporary_bytes == need, label
            for t in (q, out, k, v):
                t.release()


def test_status_word_reaches_the_host_through_the_mailbox_or_by_copy(env, fake_runtime):
    """An operation that completes at once hands its status word to the host through a word of
    host memory the device can write (one forward per completion, and per yvex_backend_sync in
    deferred mode); a runtime that gives no such memory leaves the copy of the word, with the
    same facts either way."""
    fake_runtime.fake_hip_status_forwards.restype = C.c_ulonglong
    facts_seen = []
    for pinned in (True, False):
        env("FAKE_HIP_HOST_MALLOC", None if pinned else "fail")
        with Backend() as b:
            x = written(b, "x", B.DTYPE_F32, (128,))
            before = fake_runtime.fake_hip_status_forwards()
            launches = fake_runtime.fake_hip_launches()
            facts = b.bf16_round(x, 128)
            assert fake_runtime.fake_hip_status_forwards() - before == (1 if pinned else 0)
            assert fake_runtime.fake_hip_launches() - launches == 1      # the operation's own kernel
            facts_seen.append((facts.kernel_launches, facts.device_synchronizations, facts.download_count,
                               facts.d2h_bytes))
            b.set_completion_mode(B.COMPLETION_DEFERRED)
            for _ in range(5):
                b.bf16_round(x, 128)
            assert fake_runtime.fake_hip_status_forwards() - before == (1 if pinned else 0)
            b.sync()
            assert fake_runtime.fake_hip_status_forwards() - before == (2 if pinned else 0)
            b.set_completion_mode(B.COMPLETION_IMMEDIATE)
            env("FAKE_HIP_SYNC", "fail")                                  # the runtime's wait fails
            env("YVEX_TEST_ROCM_SYNC_FAILURE", None)
            if not pinned:
                with pytest.raises(YvexError) as e:
                    b.bf16_round(x, 128)
                assert e.value.code == B.YVEX_ERR_BACKEND
            env("FAKE_HIP_SYNC", None)
    assert facts_seen[0] == facts_seen[1] == (1, 1, 1, 4)


def test_small_async_copies_leave_in_batches_in_stream_order(env, fake_runtime):
    """The session layer's per-token copies (src/runtime/stateful_attention.c:183-222) wait in a
    queue and leave as one launch per 128 of them when anything else is asked of the stream; a
    copy that meets what a queued one reads or writes sends the queue off first; large and odd
    sizes go to the runtime behind the queue; a refused batch is issued copy by copy."""
    for name in ("fake_hip_copy_batches", "fake_hip_device_copies", "fake_hip_launches"):
        getattr(fake_runtime, name).restype = C.c_ulonglong
    batches, singles = fake_runtime.fake_hip_copy_batches, fake_runtime.fake_hip_device_copies
    with Backend() as b:
        tokens, width = 300, 64
        keys, values = f32(b, "keys", (tokens, width)), f32(b, "values", (tokens, width))
        rng = np.random.default_rng(5)
        k, v = rng.standard_normal((tokens, width), dtype=np.float32), rng.standard_normal((tokens, width), dtype=np.float32)
        keys.write(k)
        values.write(v)
        history = f32(b, "history", (tokens + 2, 2 * width))
        history.zero()
        b0, s0, l0 = batches(), singles(), fake_runtime.fake_hip_launches()
        for token in range(tokens):
            row = (1 + token) * 2 * width * 4
            history.view(row, B.DTYPE_F32, (width,)).copy_from_async(keys.view(token * width * 4, B.DTYPE_F32, (width,)))
            history.view(row + width * 4, B.DTYPE_F32, (width,)).copy_from_async(
                values.view(token * width * 4, B.DTYPE_F32, (width,)))
        assert batches() - b0 == (2 * tokens) // 128                    # full queues left, the rest waits
        got = history.read().reshape(tokens + 2, 2 * width)              # the read is behind every copy
        assert batches() - b0 == (2 * tokens + 127) // 128 and singles() == s0
        assert fake_runtime.fake_hip_launches() == l0                    # not launches of an operation
        assert np.all(got[0] == 0) and np.all(got[-1] == 0)
        assert np.array_equal(got[1:-1, :width], k) and np.array_equal(got[1:-1, width:], v)
        # a chain through one buffer: each copy reads what the one before wrote
        a, mid, c = f32(b, "a", (64,)), f32(b, "mid", (64,)), f32(b, "c", (64,))
        a.write(np.arange(64, dtype=np.float32))
        mid.zero()
        c.zero()
        b1 = batches()
        mid.copy_from_async(a)
        c.copy_from_async(mid)                                            # reads a queued destination
        mid.copy_from_async(values.view(0, B.DTYPE_F32, (64,)))           # writes a queued source
        assert batches() - b1 == 2
        assert np.array_equal(c.read(), np.arange(64, dtype=np.float32)) and np.array_equal(mid.read(), v[0])
        assert batches() - b1 == 3
        a.copy_from_async(mid)
        # an odd size and a large one are the runtime's, behind what is queued
        odd_from, odd_to = f32(b, "odd-from", (3,)), f32(b, "odd-to", (3,))
        odd_from.write(np.array([1, 2, 3], np.float32))
        big_from, big_to = f32(b, "big-from", (1 << 17,)), f32(b, "big-to", (1 << 17,))
        big_from.zero()
        s1, b2 = singles(), batches()
        mid.copy_from_async(c)
        odd_to.copy_from_async(odd_from)
        assert singles() - s1 == 1 and batches() - b2 == 1
        big_to.copy_from_async(big_from)
        assert singles() - s1 == 2 and batches() - b2 == 1
        assert np.array_equal(odd_to.read(), [1, 2, 3])
        # the batch launch refused: the same copies, one by one
        env("FAKE_HIP_COPY_BATCH", "fail")
        s2 = singles()
        mid.copy_from_async(a)
        c.copy_from_async(keys.view(0, B.DTYPE_F32, (64,)))
        assert np.array_equal(mid.read(), v[0]) and np.array_equal(c.read(), k[0])
        assert singles() - s2 == 2
        env("FAKE_HIP_COPY_BATCH", None)
        # a tensor that queued copies name is not freed under them
        b3 = batches()
        mid.copy_from_async(c)
        mid.release()
        assert batches() - b3 == 1


def test_small_transfers_take_the_kernel_path_and_fall_back(env, fake_runtime):
    """Tensor writes of up to 2048 bytes and reads of up to 16384 go by kernel (no copy of the
    runtime, and for the write no wait); longer ones, and every one when the runtime gives no
    host memory the device can write or a failure of the wait is injected, take the runtime's
    copy and its wait."""
    fake_runtime.fake_hip_small_transfers.restype = C.c_ulonglong
    small = fake_runtime.fake_hip_small_transfers
    with Backend() as b:
        t = b.tensor("t", B.DTYPE_I8, (1 << 16,))
        t.zero()
        for size, by_kernel_write, by_kernel_read in [(1, 1, 1), (7, 1, 1), (2048, 1, 1), (2049, 0, 1),
                                                       (16384, 0, 1), (16385, 0, 0)]:
            data = (np.arange(size) % 251).astype(np.int8)
            view = t.view(3, B.DTYPE_I8, (size,))
            before = small()
            view.write(data)
            assert small() - before == by_kernel_write, size
            before = small()
            assert np.array_equal(view.read(), data)
            assert small() - before == by_kernel_read, size
        stats = b.memory_stats()
        assert stats.h2d_bytes == sum((1, 7, 2048, 2049, 16384, 16385))
        assert stats.d2h_bytes == stats.h2d_bytes
        env("YVEX_TEST_ROCM_SYNC_FAILURE", "tensor-read")
        before = small()
        with pytest.raises(YvexError) as e:
            t.view(0, B.DTYPE_I8, (8,)).read()
        assert e.value.code == B.YVEX_ERR_BACKEND and small() == before   # the injected failure is the wait's
        env("YVEX_TEST_ROCM_SYNC_FAILURE", None)
    env("FAKE_HIP_HOST_MALLOC", "fail")
    with Backend() as b:
        t = b.tensor("t", B.DTYPE_I8, (64,))
        before = small()
        t.write(np.arange(64, dtype=np.int8))
        assert small() - before == 1                                      # the write needs no host memory
        assert np.array_equal(t.read(), np.arange(64, dtype=np.int8))
        assert small() - before == 1                                      # the read does
    env("FAKE_HIP_HOST_MALLOC", None)
    # with a session backend on the device a written tensor may be read from another stream with
    # no event in between: the small write is waited for (a second, empty transfer) on both
    primary = Backend()
    t = primary.tensor("t", B.DTYPE_I8, (64,))
    before = small()
    t.write(np.arange(64, dtype=np.int8))
    assert small() - before == 1
    session = Backend(shared_with=primary)
    u = session.tensor("u", B.DTYPE_I8, (64,))
    for tensor in (t, u):
        before = small()
        tensor.write(np.arange(64, dtype=np.int8))
        assert small() - before == 2
    session.close()
    before = small()
    t.write(np.arange(64, dtype=np.int8))
    assert small() - before == 1                                          # alone again
    primary.close()
    with Backend() as b:                                                  # a device that does not answer
        t = b.tensor("t", B.DTYPE_I8, (64,))
        t.write(np.arange(64, dtype=np.int8))
        env("FAKE_HIP_SYNC", "fail")
        with pytest.raises(YvexError) as e:
            t.read()
        assert e.value.code == B.YVEX_ERR_BACKEND
        env("FAKE_HIP_SYNC", None)

"""GPU parity at the benchmark's full sizes (configs 3, 4 and 5), against the CPU oracle on
the same bytes, through the C ABI.

The oracle is multi-threaded C and finishes these sizes in seconds.  To keep input
generation in seconds as well, the KV pools repeat a seeded block of 2048 distinct pages
(every session still gets its own seeded permutation of page ids, and queries are all
distinct); values are N(0,1) rounded to bf16 as the configurations state.
"""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import kv_pack_pages, q8_0_encode_rows
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu

UNIQUE_PAGES = 2048


def paged_case(seed, lo, hi, sessions=32, hq=32, hkv=8, d=128, page=16, q8=False):
    rng = np.random.default_rng(seed)
    contexts = rng.integers(lo, hi + 1, size=sessions).astype(np.int32)
    need = (contexts + page - 1) // page
    pool_pages = int(need.sum())
    stride = hi // page
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((sessions, stride), dtype=np.int32)
    at = 0
    for s in range(sessions):
        table[s, :need[s]] = perm[at:at + need[s]]
        at += int(need[s])
    pools = []
    for _ in range(2):
        block = bf16_normal(rng, (UNIQUE_PAGES, page, hkv, d))
        if q8:
            block = q8_0_encode_rows(ORACLE.bf16_decode(block))   # [.., d/32, 34] bytes
        reps = (pool_pages + UNIQUE_PAGES - 1) // UNIQUE_PAGES
        pools.append(np.ascontiguousarray(
            np.tile(block, (reps,) + (1,) * (block.ndim - 1))[:pool_pages]))
    q = bf16_normal(rng, (sessions, hq, d))
    return q, pools[0], pools[1], table, contexts, pool_pages, stride


def run_full_paged(backend, q, k_rows, v_rows, table, contexts, pool_pages, stride, hi, storage):
    sessions, hq, d = q.shape
    hkv = 8
    dtype = B.DTYPE_BF16 if storage == B.KV_BF16 else B.DTYPE_I8
    tensors = []

    def tensor(*args):
        t = backend.tensor(*args)
        tensors.append(t)
        return t

    kp = kv_pack_pages(k_rows, storage, False, hkv)
    tkp = tensor("kpool", dtype, (kp.size // B.DTYPE_BYTES[dtype],), kp)
    del kp
    vp = kv_pack_pages(v_rows, storage, True, hkv)
    tvp = tensor("vpool", dtype, (vp.size // B.DTYPE_BYTES[dtype],), vp)
    del vp
    tq = tensor("q", B.DTYPE_BF16, q.shape, q)
    tt = tensor("table", B.DTYPE_I32, table.shape, table)
    tc = tensor("ctx", B.DTYPE_I32, contexts.shape, contexts)
    out = tensor("o", B.DTYPE_BF16, q.shape)
    lse = tensor("lse", B.DTYPE_F32, (sessions, hq))
    req = backend.paged_requirement(sessions, hq, hkv, d, 16, pool_pages, stride, hi,
                                    storage=storage)
    backend.paged_decode_execute(req, tq, tkp, tvp, tt, tc, out, lse)
    result = out.read(), lse.read()
    for t in tensors:
        t.release()
    return result


def test_config3_full_size_matches_cpu_operator(backend):
    """32 sessions, 32/8 heads, d=128, contexts U[512,16384], 16-token bf16 pages, seeded
    permutation page tables: every output row and LSE against the oracle."""
    q, k_rows, v_rows, table, contexts, pool_pages, stride = paged_case(3, 512, 16384)
    got, lse = run_full_paged(backend, q, k_rows, v_rows, table, contexts, pool_pages, stride,
                              16384, B.KV_BF16)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, contexts, 8, 16)
    assert rc == 0
    assert_close_bf16(got, ref, "config3 full")
    assert_lse(lse, ref_lse, "config3 full")


def test_config4_full_size_matches_cpu_operator_on_same_q8_0_bytes(backend):
    """As config 3 with contexts U[4096,32768] and Q8_0 KV blocks quantised on the host."""
    q, k_rows, v_rows, table, contexts, pool_pages, stride = paged_case(4, 4096, 32768, q8=True)
    got, lse = run_full_paged(backend, q, k_rows, v_rows, table, contexts, pool_pages, stride,
                              32768, B.KV_Q8_0)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, contexts, 8, 16, q8=True)
    assert rc == 0
    assert_close_bf16(got, ref, "config4 full")
    assert_lse(lse, ref_lse, "config4 full")


def test_config5_full_size_matches_shared_kv_oracle(backend):
    """Batch 16, 128 heads, latent 512 + rope 64, context 8192 in 64-token pages."""
    batch, heads, kd, vd, page, ctx = 16, 128, 576, 512, 64, 8192
    rng = np.random.default_rng(5)
    pages_each = ctx // page
    pool_pages = batch * pages_each
    table = rng.permutation(pool_pages).astype(np.int32).reshape(batch, pages_each)
    contexts = np.full(batch, ctx, dtype=np.int32)
    pool = bf16_normal(rng, (pool_pages, page, kd))
    q = bf16_normal(rng, (batch, heads, kd))
    tensors = [backend.tensor("latent-pages", B.DTYPE_BF16, pool.shape, pool),
               backend.tensor("q", B.DTYPE_BF16, q.shape, q),
               backend.tensor("table", B.DTYPE_I32, table.shape, table),
               backend.tensor("ctx", B.DTYPE_I32, contexts.shape, contexts),
               backend.tensor("out", B.DTYPE_BF16, (batch, heads, vd)),
               backend.tensor("lse", B.DTYPE_F32, (batch, heads))]
    tp, tq, tt, tc, out, lse = tensors
    req = backend.mla_requirement(batch, heads, kd, vd, page, pool_pages, pages_each, ctx)
    backend.mla_decode_execute(req, tq, tp, tt, tc, out, lse)
    got, got_lse = out.read(), lse.read()
    for t in tensors:
        t.release()
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, contexts, vd, page)
    assert rc == 0
    assert_close_bf16(got, ref, "config5 full")
    assert_lse(got_lse, ref_lse, "config5 full")

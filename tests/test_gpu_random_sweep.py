"""GPU parity: a seeded random sweep over the four kernel families (prefill with and without
the fused gate, paged decode bf16 / Q8_0, MLA decode with sinks, window and compressed rows,
page writer with rotary) at shapes the fixed cases do not list: odd head groups, ragged
contexts around tile and page edges, empty sessions, unaligned spans.  Same bar as the fixed
cases
the page writer is byte-exact."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import kv_pack_pages, kv_unpack_pages, q8_0_encode_rows
from gpu_common import ORACLE as O, MAX_ABS, REL_L2, LSE_ABS, backend  # noqa: F401

pytestmark = pytest.mark.gpu
C = B.NUMERIC_BF16_F32_ACCUMULATE


def close(got_bits, ref, label):
    got = O.bf16_decode(got_bits).astype(np.float64)
    ref = ref.astype(np.float64)
    err = np.abs(got - ref).max()
    rel = np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30)
    assert np.all(np.isfinite(got)) and err <= MAX_ABS and rel <= REL_L2, (label, err, rel)


@pytest.mark.parametrize("seed", [11, 12])
def test_random_sweep(backend, seed):
    b = backend
    rng = np.random.default_rng(seed)

    def bf(shape, scale=1.0):
        return O.bf16_encode((rng.standard_normal(shape) * scale).astype(np.float32))

    counts = dict(prefill=0, paged=0, mla=0, append=0)
    for _ in range(80):
        kind = rng.choice(["prefill", "paged", "mla", "append"])
        tensors = []
        def T(*a):
            t = b.tensor(*a)
            tensors.append(t)
            return t
        if kind == "prefill":
            hkv = int(rng.choice([1, 2, 4, 8]))
            g = int(rng.choice([1, 2, 4, 5, 8]))
            hq = hkv * g
            tq = int(rng.integers(2, 400))
            start = int(rng.choice([0, 0, rng.integers(0, 500)]))
            causal = bool(rng.integers(0, 2))
            tk = start + tq if causal else tq + int(rng.integers(0, 400))
            if not causal: start = 0
            q, k, v = bf((tq, hq, 128), 1.0), bf((tk, hkv, 128)), bf((tk, hkv, 128))
            gate = bf((tq, hq, 128), 2.0) if rng.integers(0, 2) else None
            req = b.attention_requirement(tq, tk, hq, hkv, 128, causal=causal, query_start=start, dtype=B.DTYPE_BF16, contract=C)
            out = T("o", B.DTYPE_BF16, q.shape)
            lse = T("l", B.DTYPE_F32, (tq, hq))
            b.attention_execute(req, T("q", B.DTYPE_BF16, q.shape, q), T("k", B.DTYPE_BF16, k.shape, k), T("v", B.DTYPE_BF16, v.shape, v), out, lse=lse,
                                gate=T("g", B.DTYPE_BF16, gate.shape, gate) if gate is not None else None)
            rc, ref, _, ref_lse = O.gqa_bf16(q, k, v, query_start=start, causal=causal)
            assert rc == 0
            if gate is not None:
                ref = O.sigmoid_gate_bf16(O.bf16_decode(O.bf16_encode(ref)), O.bf16_decode(gate)).reshape(ref.shape)
            label = ("prefill", tq, tk, start, hq, hkv, causal, gate is not None)
            close(out.read(), ref, label)
            assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label
        elif kind == "paged":
            hkv = int(rng.choice([1, 2, 8]))
            g = int(rng.choice([1, 2, 4, 8, 16]))
            hq = hkv * g
            sessions = int(rng.integers(1, 12))
            q8 = bool(rng.integers(0, 2))
            ctx = rng.integers(1, int(rng.choice([40, 600, 6000])), size=sessions).astype(np.int32)
            need = (ctx + 15) // 16
            pool_pages = int(need.sum()) + 3
            stride = int(need.max()) + int(rng.integers(0, 3))
            perm = rng.permutation(pool_pages).astype(np.int32)
            table = np.zeros((sessions, stride), np.int32)
            at = 0
            for s in range(sessions): table[s, :need[s]] = perm[at:at + need[s]]; at += int(need[s])
            kr, vr = bf((pool_pages, 16, hkv, 128)), bf((pool_pages, 16, hkv, 128))
            storage, dt = (B.KV_Q8_0, B.DTYPE_I8) if q8 else (B.KV_BF16, B.DTYPE_BF16)
            if q8: kr, vr = q8_0_encode_rows(O.bf16_decode(kr)), q8_0_encode_rows(O.bf16_decode(vr))
            kp, vp = kv_pack_pages(kr, storage, False, hkv), kv_pack_pages(vr, storage, True, hkv)
            q = bf((sessions, hq, 128))
            gate = bf(q.shape, 2.0) if rng.integers(0, 2) else None
            out = T("o", B.DTYPE_BF16, q.shape)
            lse = T("l", B.DTYPE_F32, (sessions, hq))
            req = b.paged_requirement(sessions, hq, hkv, 128, 16, pool_pages, stride, stride * 16, storage=storage)
            b.paged_decode_execute(req, T("q", B.DTYPE_BF16, q.shape, q), T("kp", dt, (kp.size // B.DTYPE_BYTES[dt],), kp), T("vp", dt, (vp.size // B.DTYPE_BYTES[dt],), vp),
                                   T("t", B.DTYPE_I32, table.shape, table), T("c", B.DTYPE_I32, ctx.shape, ctx), out, lse,
                                   gate=T("g", B.DTYPE_BF16, gate.shape, gate) if gate is not None else None)
            rc, ref, _, ref_lse = O.paged_decode(q, kr, vr, table, ctx, hkv, 16, q8=q8)
            assert rc == 0
            if gate is not None:
                ref = O.sigmoid_gate_bf16(O.bf16_decode(O.bf16_encode(ref)), O.bf16_decode(gate)).reshape(ref.shape)
            label = ("paged", sessions, hq, hkv, q8, ctx.tolist(), gate is not None)
            close(out.read(), ref, label)
            assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label
        elif kind == "mla":
            batch = int(rng.integers(1, 5))
            ctx = rng.integers(1, int(rng.choice([100, 700, 3000])), size=batch).astype(np.int32)
            need = (ctx + 63) // 64
            pool_pages = int(need.sum()) + 2
            stride = int(need.max()) + 1
            perm = rng.permutation(pool_pages).astype(np.int32)
            table = np.zeros((batch, stride), np.int32)
            at = 0
            for s in range(batch): table[s, :need[s]] = perm[at:at + need[s]]; at += int(need[s])
            pool = bf((pool_pages, 64, 576))
            q = bf((batch, 128, 576))
            window = int(rng.choice([0, 0, rng.integers(1, 2000)]))
            sinks = (rng.standard_normal(128) * 2).astype(np.float32) if rng.integers(0, 2) else None
            comp = None
            sel = None
            extra = {}
            if rng.integers(0, 2):
                stored = rng.integers(1, 300, size=batch)
                cneed = (stored + 63) // 64
                cpages = int(cneed.sum()) + 1
                cstride = int(cneed.max())
                cperm = rng.permutation(cpages).astype(np.int32)
                ctable = np.zeros((batch, cstride), np.int32)
                at = 0
                for s in range(batch): ctable[s, :cneed[s]] = cperm[at:at + cneed[s]]; at += int(cneed[s])
                cpool = bf((cpages, 64, 576))
                if rng.integers(0, 2):
                    cap = int(rng.integers(1, 200))
                    sel = np.stack([rng.integers(0, stored[s], cap) for s in range(batch)]).astype(np.int32)
                    ccount = rng.integers(0, cap + 1, size=batch).astype(np.int32)
                else:
                    ccount = np.array([rng.integers(0, stored[s] + 1) for s in range(batch)], np.int32)
                comp = (cpool, ctable, ccount)
                extra = dict(compressed_pool_pages=cpages, compressed_table_stride=cstride, max_compressed_tokens=cstride * 64,
                             compressed_selected_stride=sel.shape[1] if sel is not None else 0)
            req = b.mla_requirement(batch, 128, 576, 512, 64, pool_pages, stride, stride * 64, sliding_window=window, **extra)
            out = T("o", B.DTYPE_BF16, (batch, 128, 512))
            lse = T("l", B.DTYPE_F32, (batch, 128))
            tc = None
            if comp is not None:
                tc = [T("cp", B.DTYPE_BF16, comp[0].shape, comp[0]), T("ct", B.DTYPE_I32, comp[1].shape, comp[1]), T("cc", B.DTYPE_I32, comp[2].shape, comp[2])]
                if sel is not None: tc.append(T("sel", B.DTYPE_I32, sel.shape, sel))
            b.mla_decode_execute(req, T("q", B.DTYPE_BF16, q.shape, q), T("p", B.DTYPE_BF16, pool.shape, pool), T("t", B.DTYPE_I32, table.shape, table),
                                 T("c", B.DTYPE_I32, ctx.shape, ctx), out, lse, sinks=T("s", B.DTYPE_F32, (128,), sinks) if sinks is not None else None, compressed=tc)
            rc, ref, _, ref_lse = O.mla_decode(q, pool, table, ctx, 512, 64, sinks=sinks, sliding_window=window, compressed=comp, selected=sel)
            assert rc == 0
            label = ("mla", batch, ctx.tolist(), window, sinks is not None, comp is not None, sel is not None)
            close(out.read(), ref, label)
            assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label
        else:
            hkv = int(rng.choice([1, 3, 4, 8]))
            sessions = int(rng.integers(1, 6))
            q8 = bool(rng.integers(0, 2))
            rd = int(rng.choice([0, 16, 32, 64, 96, 128]))
            starts = rng.integers(0, 200, size=sessions).astype(np.int32)
            cnt = rng.integers(0, int(rng.choice([2, 40, 150])), size=sessions).astype(np.int32)
            if cnt.sum() == 0: cnt[0] = 1
            stride = int(((starts + cnt + 15) // 16).max()) + 1
            pool_pages = sessions * stride + 2
            table = rng.permutation(pool_pages)[:sessions * stride].astype(np.int32).reshape(sessions, stride)
            total = int(cnt.sum())
            rows0 = np.concatenate([[0], np.cumsum(cnt)[:-1]]).astype(np.int32)
            kn, vn = bf((total, hkv, 128)), bf((total, hkv, 128))
            ang = rng.uniform(-3, 3, (total, max(rd, 16))).astype(np.float32)
            cs, sn = np.cos(ang), np.sin(ang)
            old_k, old_v = bf((pool_pages, 16, hkv, 128)), bf((pool_pages, 16, hkv, 128))
            storage, dt = (B.KV_Q8_0, B.DTYPE_I8) if q8 else (B.KV_BF16, B.DTYPE_BF16)
            enc = (lambda x: q8_0_encode_rows(O.bf16_decode(x))) if q8 else (lambda x: x)
            kr, vr = enc(old_k), enc(old_v)
            kp, vp = kv_pack_pages(kr, storage, False, hkv), kv_pack_pages(vr, storage, True, hkv)
            tk_, tv_ = T("kp", dt, (kp.size // B.DTYPE_BYTES[dt],), kp), T("vp", dt, (vp.size // B.DTYPE_BYTES[dt],), vp)
            b.kv_append_execute(T("k", B.DTYPE_BF16, kn.shape, kn), T("v", B.DTYPE_BF16, vn.shape, vn), T("r", B.DTYPE_I32, (sessions,), rows0),
                                T("s", B.DTYPE_I32, (sessions,), starts), T("c", B.DTYPE_I32, (sessions,), cnt), T("t", B.DTYPE_I32, table.shape, table),
                                tk_, tv_, hkv, pool_pages, int(max(cnt.max(), 1)), storage=storage,
                                cosine=T("cos", B.DTYPE_F32, cs.shape, cs) if rd else None, sine=T("sin", B.DTYPE_F32, sn.shape, sn) if rd else None, rotary_dimension=rd)
            krot = O.rotary_half_bf16(kn, cs[:, :rd], sn[:, :rd], rd) if rd else kn
            wk, wv = kr.copy(), vr.copy()
            for s in range(sessions):
                for i in range(cnt[s]):
                    pos = starts[s] + i
                    pg, sl = table[s, pos // 16], pos % 16
                    wk[pg, sl] = enc(krot[rows0[s] + i][None])[0]
                    wv[pg, sl] = enc(vn[rows0[s] + i][None])[0]
            gk = kv_unpack_pages(tk_.read(np.uint8, (-1,)), storage, False, pool_pages, hkv).reshape(wk.shape)
            gv = kv_unpack_pages(tv_.read(np.uint8, (-1,)), storage, True, pool_pages, hkv).reshape(wv.shape)
            label = ("append", sessions, hkv, q8, rd, starts.tolist(), cnt.tolist())
            assert np.array_equal(gk, wk), label
            assert np.array_equal(gv, wv), label
        counts[kind] += 1
        for t in tensors:
            t.release()
    assert min(counts.values()) > 5, counts

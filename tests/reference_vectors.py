"""Input vectors and expected values held by the reference's own tests for the
attention path, restated as data (the reference generates them with the integer
patterns below; nothing here is reference code).

Citations are relative to the yailabs/clori tree.
"""
import math

import numpy as np


def _pattern(count, mul, add, mod, sub, div):
    i = np.arange(count, dtype=np.int64)
    return (((i * mul + add) % mod) - sub).astype(np.float32) / np.float32(div)


# tests/unit/backend_ops.c:455-467: single head, d=4, 3 rows, scale 0.5
CPU_OP_QUERY = np.array([0.1, 0.2, 0.3, 0.4], dtype=np.float32)
CPU_OP_KEYS = np.array([[0.2, 0.1, 0.0, 0.3], [0.4, 0.3, 0.2, 0.1], [0.1, 0.5, 0.3, 0.2]],
                       dtype=np.float32)
CPU_OP_VALUES = np.array([[1, 2, 3, 4], [10, 20, 30, 40], [5, 6, 7, 8]], dtype=np.float32)
CPU_OP_SCALE = 0.5


def gqa_kat():
    """tests/unit/cuda/quant_qtype.c:1998-2031,2112-2136: 2 tokens, 2 q heads, 1 kv head, d=2.
    Causal row 0 == V[0]; row 1 (and every FULL row) == (e^{1/sqrt2} V0 + V1)/(e^{1/sqrt2}+1)."""
    q = np.zeros((2, 2, 2), dtype=np.float32)
    q[..., 0] = 1.0
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=np.float32)
    v = np.array([[[2.0, 4.0]], [[6.0, 8.0]]], dtype=np.float32)
    p = math.exp(1.0 / math.sqrt(2.0))
    mixed = np.array([(p * 2.0 + 6.0) / (p + 1.0), (p * 4.0 + 8.0) / (p + 1.0)], dtype=np.float64)
    return q, k, v, mixed


def small_5x128():
    """tests/unit/cuda/quant_qtype.c:2293-2296: 5 tokens, 1 head, d=128 (tolerance 2e-5)."""
    n = 5 * 128
    return (_pattern(n, 3, 0, 19, 9, 8).reshape(5, 1, 128),
            _pattern(n, 5, 2, 23, 11, 9).reshape(5, 1, 128),
            _pattern(n, 7, 1, 29, 14, 10).reshape(5, 1, 128))


def qwen_24_4_256():
    """tests/unit/cuda/quant_qtype.c:2413-2418: 3 tokens, 24/4 heads, d=256
    (tolerance 2e-4 * (1+|ref|))."""
    qn, kn = 3 * 24 * 256, 3 * 4 * 256
    return (_pattern(qn, 3, 0, 29, 14, 32).reshape(3, 24, 256),
            _pattern(kn, 5, 1, 31, 15, 32).reshape(3, 4, 256),
            _pattern(kn, 7, 2, 37, 18, 16).reshape(3, 4, 256))


def cached_decode_qwen():
    """tests/unit/cuda/quant_qtype.c:2503-2508: Tq=1, Tk=3, query_start=2, 24/4 heads, d=256."""
    qn, kn = 1 * 24 * 256, 3 * 4 * 256
    return (_pattern(qn, 11, 0, 43, 21, 32).reshape(1, 24, 256),
            _pattern(kn, 13, 1, 47, 23, 32).reshape(3, 4, 256),
            _pattern(kn, 17, 2, 53, 26, 16).reshape(3, 4, 256))


def strided_qwen(query_tokens=2, kv_tokens=4, query_heads=24, kv_heads=4, head_dim=256):
    """tests/unit/cuda/quant_qtype.c:2600-2620: packed values that the test interleaves as
    [Q|gate] rows (stride 2*Hq*d) and [K|V] rows (stride 2*Hkv*d)."""
    qn = query_tokens * query_heads * head_dim
    kn = kv_tokens * kv_heads * head_dim
    return (_pattern(qn, 19, 3, 59, 29, 32).reshape(query_tokens, query_heads, head_dim),
            _pattern(kn, 23, 5, 61, 30, 32).reshape(kv_tokens, kv_heads, head_dim),
            _pattern(kn, 29, 7, 67, 33, 16).reshape(kv_tokens, kv_heads, head_dim))


def tiled_257x128():
    """tests/unit/cuda/quant_qtype.c:2749-2756: 257 tokens, 1 head, d=128, bf16-representable
    values (tolerance 2e-3 relative)."""
    n = 257 * 128
    return (_pattern(n, 3, 0, 31, 15, 16).reshape(257, 1, 128),
            _pattern(n, 5, 2, 37, 18, 16).reshape(257, 1, 128),
            _pattern(n, 7, 1, 41, 20, 8).reshape(257, 1, 128))


def uniform_large(tokens, heads, head_dim=128):
    """tests/unit/cuda/quant_qtype.c:2896-2931: Q=K=0, V[t,h,:] = h+1  =>  out == V."""
    q = np.zeros((tokens, heads, head_dim), dtype=np.float32)
    v = np.broadcast_to((np.arange(heads, dtype=np.float32) + 1.0)[None, :, None],
                        (tokens, heads, head_dim)).copy()
    return q, q.copy(), v


# tests/unit/quant_numeric.c:514-526: Q8_0 golden block
Q8_0_GOLDEN_SOURCE = np.array([127.0, -127.0, 0.5, -0.5] + [0.0] * 28, dtype=np.float32)
Q8_0_GOLDEN_PREFIX = bytes([0x00, 0x3C, 0x7F, 0x81, 0x01, 0xFF])

# tests/reference/deepseek_attention.c:2696-2698: bf16 RNE literals
BF16_LITERALS = [(1.00390625, 0x3F80), (1.01171875, 0x3F82), (-0.0, 0x8000)]

# tests/reference/deepseek_attention.c:2722-2725: sink softmax known answer
SINK_KAT = dict(logits=[0.0, 0.6931471824645996], values=[[1.0, 2.0], [3.0, 4.0]], sink=0.0,
                expected=[1.75, 2.5])


def float_two_pass_gqa(q, k, v, query_start, causal):
    """Independent float32 two-pass softmax in the style of the scalar checkers the
    reference tests carry (tests/unit/cuda/quant_qtype.c:2253-2281,2343-2391): float
    dot, float max, expf, float accumulate.  Used to pin the oracle from a second
    direction, never as the oracle itself."""
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    group = hq // hkv
    scale = np.float32(1.0) / np.sqrt(np.float32(d))
    out = np.zeros((tq, hq, d), dtype=np.float32)
    for t in range(tq):
        visible = query_start + t + 1 if causal else tk
        for h in range(hq):
            kh = h // group
            s = (k[:visible, kh, :].astype(np.float32) @ q[t, h, :].astype(np.float32)) * scale
            p = np.exp((s - s.max()).astype(np.float32)).astype(np.float32)
            out[t, h] = (p[:, None] * v[:visible, kh, :]).sum(axis=0, dtype=np.float32) / p.sum(
                dtype=np.float32)
    return out

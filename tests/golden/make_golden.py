#!/usr/bin/env python3
"""Writes tests/golden/reference_attention.npz: outputs of the REFERENCE's own CPU attention
operator and codecs (compiled from its sources into oracle/_ref by `make -C oracle ref`)
on inputs that the test regenerates from closed-form integer patterns.

Run in a container that has the reference tree:  python tests/golden/make_golden.py
The fixture holds data only (inputs are formulas, outputs are arrays); it lets the oracle
be checked bit for bit where the reference cannot be built.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_binding import (f32p, load_reference, load_reference_reduce, reference_reduce,  # noqa: E402
                            _ptr)

# (name, seq_len, head_dim, position, causal)
CASES = [
    ("one-key", 1, 128, 0, 1),
    ("five-keys", 5, 128, 4, 1),
    ("mid-causal", 64, 128, 37, 1),
    ("odd-257-full", 257, 128, 0, 0),
    ("narrow-d64", 300, 64, 299, 1),
    ("decode-4096", 4096, 128, 4095, 1),
    ("long-16384", 16384, 128, 16383, 1),
]


# Shared-KV reduce of one query token (yvex_attention_reduce_chunk):
# (name, attention class, sliding window, context, stored compressed rows, heads, dim)
REDUCE_CASES = [
    ("reduce-one-row", 0, 128, 1, 0, 2, 64),
    ("reduce-window-16", 0, 16, 90, 0, 4, 64),
    ("reduce-window-wide", 0, 1 << 20, 300, 0, 4, 64),
    ("reduce-compressed-127", 2, 64, 127, 3, 4, 64),
    ("reduce-compressed-128", 2, 64, 128, 3, 4, 64),
    ("reduce-compressed-700", 2, 128, 700, 7, 4, 128),
]
REDUCE_RATIO = 128
# the same reduce with a real rope tail: (name, attention_class, window, context, stored, heads,
# dim, position policy).  Policy = rope lanes, theta and the YaRN fields of the reference's
# position policy; the second one is the DeepSeek-style long-context scaling
# (factor 40 over an original context of 4096, beta 32 / 1).
ROPE_PLAIN = dict(rope_dims=64, theta=10000)
ROPE_YARN = dict(rope_dims=64, theta=10000, scaling_factor=40, original_context=4096, beta_fast=32,
                 beta_slow=1)
REDUCE_ROPE_CASES = [
    ("reduce-rope-plain", 0, 1 << 20, 300, 0, 4, 128, ROPE_PLAIN),
    ("reduce-rope-yarn", 0, 1 << 20, 300, 0, 4, 128, ROPE_YARN),
    ("reduce-rope-yarn-compressed", 2, 64, 700, 7, 4, 128, ROPE_YARN),
    ("reduce-rope-all-lanes", 0, 16, 90, 0, 2, 64, dict(rope_dims=64, theta=500000)),
]


# the reduce at the reference model's own geometry (tests/unit/deepseek_arch_ir.c:110-125:
# 64 heads, 512 lanes, 64 rope lanes inside, window 128, ratio 128), dense compressed class
MODEL_GEOMETRY_CASE = ("reduce-model-geometry", 2, 128, 700, 7, 64, 512, ROPE_YARN)


def reduce_inputs(heads, dim, context, stored):
    """bf16-representable patterns: query, local rows (positions 0 .. context-1), compressed
    rows (positions 0, 128, 256, ...), sink logits."""
    q = pattern(heads * dim, 3, 0, 19, 9, 8).reshape(heads, dim)
    local = pattern(context * dim, 5, 2, 23, 11, 16).reshape(context, dim)
    compressed = pattern(max(stored, 1) * dim, 7, 1, 29, 14, 16).reshape(-1, dim)[:stored]
    sinks = pattern(heads, 1, 0, 5, 2, 2)
    return q, local, compressed, sinks


def pattern(count, mul, add, mod, offset, div):
    """The integer generators of the reference's own tests
    (tests/unit/cuda/quant_qtype.c:2293-2296): ((i * mul + add) % mod - offset) / div."""
    i = np.arange(count, dtype=np.int64)
    return (((i * mul + add) % mod - offset).astype(np.float32) / np.float32(div)).astype(np.float32)


def inputs(seq_len, head_dim):
    q = pattern(head_dim, 3, 0, 19, 9, 8)
    k = pattern(seq_len * head_dim, 5, 2, 23, 11, 9).reshape(seq_len, head_dim)
    v = pattern(seq_len * head_dim, 7, 1, 29, 14, 10).reshape(seq_len, head_dim)
    return q, k, v


def main():
    ref = load_reference()
    if ref is None:
        sys.exit("oracle/_ref/libyvex_ref.so is not built: run `make -C oracle ref`")
    out = {}
    for name, n, d, position, causal in CASES:
        q, k, v = inputs(n, d)
        score = np.zeros(n, np.float32)
        prob = np.zeros(n, np.float32)
        o = np.zeros(d, np.float32)
        rc = ref.yvref_op_attention(_ptr(q, f32p), _ptr(k, f32p), _ptr(v, f32p), n, position, d,
                                    np.float32(1.0 / np.sqrt(d)), causal, _ptr(score, f32p),
                                    _ptr(prob, f32p), _ptr(o, f32p))
        assert rc == 0, (name, rc)
        out[name + "/out"] = o
        # score and prob rows are long: keep both ends and strided samples
        keep = np.unique(np.concatenate([np.arange(min(n, 16)), np.arange(max(n - 16, 0), n),
                                         np.arange(0, n, 97)]))
        out[name + "/index"] = keep.astype(np.int64)
        out[name + "/score"] = score[keep]
        out[name + "/prob"] = prob[keep]
    # codecs: bf16 / f16 encodings of a float sweep, Q8_0 of two blocks
    sweep = np.concatenate([pattern(4096, 37, 5, 1009, 504, 64),
                            np.array([0.0, -0.0, 1.00390625, 1.01171875, 65504.0, 7e-8, -3e38],
                                     np.float32)])
    sweep = np.ascontiguousarray(sweep, np.float32)
    bits = np.zeros(sweep.size, np.uint16)
    ref.yvref_bf16_encode_n(_ptr(sweep, f32p), bits.ctypes.data_as(C.POINTER(C.c_uint16)), sweep.size)
    out["codec/bf16"] = bits.copy()
    ref.yvref_f16_encode_n(_ptr(sweep, f32p), bits.ctypes.data_as(C.POINTER(C.c_uint16)), sweep.size)
    out["codec/f16"] = bits.copy()
    blocks = pattern(64, 11, 3, 61, 30, 7)
    enc = np.zeros(68, np.uint8)
    for b in range(2):
        ref.yvref_q8_0_encode_block(_ptr(np.ascontiguousarray(blocks[32 * b:32 * b + 32]), f32p),
                                    enc[34 * b:].ctypes.data_as(C.POINTER(C.c_ubyte)))
    out["codec/q8_0"] = enc
    reduce = load_reference_reduce()
    if reduce is None:
        sys.exit("oracle/_ref/libyvex_ref_reduce.so is not built: run `make -C oracle ref`")
    for name, attention_class, window, context, stored, heads, dim in REDUCE_CASES:
        q, local, compressed, sinks = reduce_inputs(heads, dim, context, stored)
        rc, o = reference_reduce(reduce, q, local, np.arange(context), compressed,
                                 np.arange(stored) * REDUCE_RATIO, sinks, window,
                                 REDUCE_RATIO if attention_class == 2 else 0, attention_class,
                                 context - 1)
        assert rc == 0, (name, rc)
        out[name + "/out"] = o
    for name, attention_class, window, context, stored, heads, dim, policy in REDUCE_ROPE_CASES + [MODEL_GEOMETRY_CASE]:
        q, local, compressed, sinks = reduce_inputs(heads, dim, context, stored)
        rc, o = reference_reduce(reduce, q, local, np.arange(context), compressed,
                                 np.arange(stored) * REDUCE_RATIO, sinks, window,
                                 REDUCE_RATIO if attention_class == 2 else 0, attention_class,
                                 context - 1, **policy)
        assert rc == 0, (name, rc)
        out[name + "/out"] = o
    np.savez_compressed(os.path.join(HERE, "reference_attention.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()

"""The oracle against committed outputs of the reference's own CPU operator and codecs
(tests/golden/reference_attention.npz, written by tests/golden/make_golden.py from the
reference compiled in place).  Bit-exact: same double accumulation, float score store, own
exp and two float roundings of the probabilities as src/backend/cpu.c:307-399."""
import importlib.util
import os

import numpy as np
import pytest

from oracle_binding import Oracle

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_golden",
                                              os.path.join(HERE, "golden", "make_golden.py"))
make_golden = importlib.util.module_from_spec(spec)
spec.loader.exec_module(make_golden)

GOLDEN = np.load(os.path.join(HERE, "golden", "reference_attention.npz"), allow_pickle=False)
ORACLE = Oracle()


@pytest.mark.parametrize("case", make_golden.CASES, ids=[c[0] for c in make_golden.CASES])
def test_attention_head_matches_reference_output_bits(case):
    name, n, d, position, causal = case
    q, k, v = make_golden.inputs(n, d)
    rc, out, score, prob, _ = ORACLE.attention_head(q, k, v, position, np.float32(1.0 / np.sqrt(d)),
                                                    causal=bool(causal))
    assert rc == 0
    keep = GOLDEN[name + "/index"]
    assert np.array_equal(out.view(np.uint32), GOLDEN[name + "/out"].view(np.uint32))
    assert np.array_equal(score[keep].view(np.uint32), GOLDEN[name + "/score"].view(np.uint32))
    assert np.array_equal(prob[keep].view(np.uint32), GOLDEN[name + "/prob"].view(np.uint32))


def test_codecs_match_reference_bits():
    sweep = np.concatenate([make_golden.pattern(4096, 37, 5, 1009, 504, 64),
                            np.array([0.0, -0.0, 1.00390625, 1.01171875, 65504.0, 7e-8, -3e38],
                                     np.float32)]).astype(np.float32)
    assert np.array_equal(ORACLE.bf16_encode(sweep), GOLDEN["codec/bf16"])
    f16 = np.array([ORACLE.lib.yvo_f16_encode(float(x)) for x in sweep], dtype=np.uint16)
    assert np.array_equal(f16, GOLDEN["codec/f16"])
    blocks = make_golden.pattern(64, 11, 3, 61, 30, 7)
    enc = ORACLE.q8_0_encode_rows(blocks.reshape(2, 32)).reshape(-1)
    assert np.array_equal(enc, GOLDEN["codec/q8_0"])


@pytest.mark.parametrize("case", make_golden.REDUCE_CASES, ids=[c[0] for c in make_golden.REDUCE_CASES])
def test_shared_kv_reduce_matches_reference_output_bits(case):
    """yvo_mla_decode_bf16 (sink logits, sliding window, dense compressed rows; key_dim ==
    value_dim as in the reference) against committed outputs of yvex_attention_reduce_chunk.
    The reference rounds the row to bf16, rotates its last two lanes back by the position
    and rounds again (src/graph/core.c:499-507): the other lanes compare as they are, the last
    two after the same rotation."""
    import math
    name, attention_class, window, context, stored, heads, dim = case
    q, local, compressed, sinks = make_golden.reduce_inputs(heads, dim, context, stored)
    page = 16

    def paged(rows):
        pages = max((len(rows) + page - 1) // page, 1)
        pool = np.zeros((pages, page, dim), np.uint16)
        pool.reshape(-1, dim)[:len(rows)] = ORACLE.bf16_encode(rows)
        return pool, np.arange(pages, dtype=np.int32)[None, :]

    pool, table = paged(local)
    cpool, ctable = paged(compressed)
    visible = np.array([context // make_golden.REDUCE_RATIO if attention_class == 2 else 0], np.int32)
    rc, out, _, _ = ORACLE.mla_decode(ORACLE.bf16_encode(q)[None], pool, table,
                                      np.array([context], np.int32), dim, page, sinks=sinks,
                                      sliding_window=window,
                                      compressed=(cpool, ctable, visible) if attention_class == 2 else None)
    assert rc == 0
    mine = ORACLE.bf16_decode(ORACLE.bf16_encode(out[0]))
    want = GOLDEN[name + "/out"]
    assert np.array_equal(mine[:, :-2].view(np.uint32), want[:, :-2].view(np.uint32))
    c, s = math.cos(float(context - 1)), -math.sin(float(context - 1))
    for h in range(heads):
        x, y = float(mine[h, -2]), float(mine[h, -1])
        tail = ORACLE.bf16_decode(ORACLE.bf16_encode(np.array([x * c - y * s, x * s + y * c], np.float32)))
        assert np.array_equal(tail, want[h, -2:])


@pytest.mark.parametrize("case", make_golden.REDUCE_ROPE_CASES + [make_golden.MODEL_GEOMETRY_CASE],
                         ids=[c[0] for c in make_golden.REDUCE_ROPE_CASES + [make_golden.MODEL_GEOMETRY_CASE]])
def test_reduce_output_rotation_matches_reference_output_bits(case):
    """The whole published row of yvex_attention_reduce_chunk with a real rope tail (64 rope
    lanes, plain and YaRN-scaled frequencies, src/graph/core.c:499-507 and
    src/graph/numeric.c:877-949): yvo_mla_decode_bf16 followed by yvo_reduce_output_finish
    equals the committed reference output on every lane, bit for bit."""
    name, attention_class, window, context, stored, heads, dim, policy = case
    q, local, compressed, sinks = make_golden.reduce_inputs(heads, dim, context, stored)
    page = 16

    def paged(rows):
        pages = max((len(rows) + page - 1) // page, 1)
        pool = np.zeros((pages, page, dim), np.uint16)
        pool.reshape(-1, dim)[:len(rows)] = ORACLE.bf16_encode(rows)
        return pool, np.arange(pages, dtype=np.int32)[None, :]

    pool, table = paged(local)
    cpool, ctable = paged(compressed)
    visible = np.array([context // make_golden.REDUCE_RATIO if attention_class == 2 else 0], np.int32)
    rc, out, _, _ = ORACLE.mla_decode(ORACLE.bf16_encode(q)[None], pool, table,
                                      np.array([context], np.int32), dim, page, sinks=sinks,
                                      sliding_window=window,
                                      compressed=(cpool, ctable, visible) if attention_class == 2 else None)
    assert rc == 0
    rc, mine = ORACLE.reduce_output_finish(out[0], context - 1, ORACLE.position_policy(**policy))
    assert rc == 0
    want = GOLDEN[name + "/out"]
    assert np.array_equal(mine.view(np.uint32), want.view(np.uint32))
    # the rotation did something: the rope lanes differ from the unrotated row
    plain = ORACLE.bf16_decode(ORACLE.bf16_encode(out[0]))
    assert not np.array_equal(plain[:, -policy["rope_dims"]:], want[:, -policy["rope_dims"]:])
    assert np.array_equal(plain[:, :dim - policy["rope_dims"]], want[:, :dim - policy["rope_dims"]])

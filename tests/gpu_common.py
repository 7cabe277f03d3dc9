"""Shared helpers for the GPU parity tests: seeded inputs, the tolerance bar, and one
backend per test session."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import Backend
from oracle_binding import Oracle

ORACLE = Oracle()

# The bar stated by the task for bf16 outputs against the fp32 CPU operator.
MAX_ABS = 2e-2
REL_L2 = 1e-2
LSE_ABS = 1e-3


def bf16_normal(rng, shape, scale=1.0):
    """N(0,1)*scale drawn in f32, rounded to bf16 (RNE): returns uint16 bits."""
    x = rng.standard_normal(shape).astype(np.float32) * np.float32(scale)
    return ORACLE.bf16_encode(x)


def assert_close_bf16(got_bits, ref_f32, label=""):
    got = ORACLE.bf16_decode(got_bits).astype(np.float64)
    ref = ref_f32.astype(np.float64)
    assert np.all(np.isfinite(got)), label
    max_abs = np.abs(got - ref).max()
    rel_l2 = np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30)
    assert max_abs <= MAX_ABS, "%s max-abs %.4g" % (label, max_abs)
    assert rel_l2 <= REL_L2, "%s rel-L2 %.4g" % (label, rel_l2)
    return max_abs, rel_l2


def assert_lse(got, ref, label=""):
    err = np.abs(np.asarray(got, dtype=np.float64) - ref).max()
    assert err <= LSE_ABS, "%s LSE err %.4g" % (label, err)
    return err


@pytest.fixture(scope="session")
def backend():
    b = Backend()
    assert b.status == B.STATUS_READY, b.report().rejection
    yield b
    b.close()

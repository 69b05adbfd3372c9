"""Encode side on the GPU against the oracle encoders (needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, say, t

pytestmark = pytest.mark.gpu


def test_e8_quantize_matches_oracle_indices():
    """Random vectors at several scales, exact ties (the origin, midpoints between table
    rows, lattice points themselves) and the 256-row secondary table: indices bit-equal."""
    from glq_amd import ext
    say("e8 quantize")
    rng = np.random.default_rng(0)
    cb = O.e8_table()
    X = np.concatenate([
        rng.standard_normal((3000, 8)).astype(np.float32),
        (rng.standard_normal((1000, 8)) * 3.0).astype(np.float32),
        (rng.standard_normal((500, 8)) * 0.1).astype(np.float32),
        np.zeros((1, 8), np.float32),
        cb[rng.integers(0, 65536, 300)],
        0.5 * (cb[rng.integers(0, 65536, 300)] + cb[rng.integers(0, 65536, 300)]),
        rng.standard_normal((700, 8)).astype(np.float16).astype(np.float32),
    ])
    dec_ref, idx_ref = O.e8_quantize(X)
    dec, idx = ext.e8_quantize(t(X), t(cb))
    idx = idx.cpu().numpy()
    bad = np.nonzero(idx != idx_ref)[0]
    assert bad.size == 0, (bad[:5], idx[bad[:5]], idx_ref[bad[:5]])
    assert np.array_equal(dec.cpu().numpy(), dec_ref)
    # secondary table of the 3 bpw recipe
    _, i2_ref = O.e8_quantize(X[:1000], cb[:256])
    _, i2 = ext.e8_quantize(t(X[:1000]), t(cb[:256]))
    assert np.array_equal(i2.cpu().numpy(), i2_ref)


def test_e8_quantize_residual_stage_and_size():
    from glq_amd import ext
    say("e8 quantize rvq")
    rng = np.random.default_rng(1)
    cb = O.e8_table()
    X = rng.standard_normal((4099, 8)).astype(np.float32)        # ragged against the launch tiling
    d1, i1 = ext.e8_quantize(t(X), t(cb))
    res = (t(X) - d1) * 3.0
    d2, i2 = ext.e8_quantize(res, t(cb))
    r1, j1 = O.e8_quantize(X)
    r2, j2 = O.e8_quantize((X - r1) * np.float32(3.0))
    assert np.array_equal(i1.cpu().numpy(), j1) and np.array_equal(i2.cpu().numpy(), j2)
    again = ext.e8_quantize(t(X), t(cb))[1]
    assert torch.equal(i1, again)

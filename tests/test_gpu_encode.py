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


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_viterbi_matches_oracle_states(K, golden):
    """Tail-biting Viterbi: the reference's own tiles (golden vectors) and random tiles, state
    sequences and reconstructions bit-equal to the oracle (which is pinned on the reference)."""
    from glq_amd import ext
    say("viterbi", K)
    g = golden("trellis_viterbi")
    rng = np.random.default_rng(K)
    gk = K if f"K{K}_tiles" in g.files else 4           # the reference vectors hold K = 2 and 4
    tiles = np.concatenate([g[f"K{gk}_tiles"].astype(np.float32),
                            rng.standard_normal((5, 256)).astype(np.float32),
                            np.zeros((1, 256), np.float32),
                            (rng.standard_normal((2, 256)) * 3).astype(np.float32)])
    hat_ref, st_ref = O.trellis_quantize_tiles(tiles, K)
    hat, st = ext.trellis_quantize_tiles(t(tiles), K)
    st = st.cpu().numpy()
    bad = np.nonzero((st != st_ref).any(axis=1))[0]
    assert bad.size == 0, ("tiles differ", bad)
    assert np.array_equal(hat.cpu().numpy(), hat_ref)
    if gk == K:                                          # and directly against the reference's states
        assert np.array_equal(st[:6], g[f"K{K}_states"])
    # tail-biting: consecutive states overlap in 16-K bits, also across the wrap
    mask = (1 << (16 - K)) - 1
    assert np.array_equal(st[:, :-1] & mask, st[:, 1:] >> K)
    assert np.array_equal(st[:, -1] & mask, st[:, 0] >> K)
    again = ext.trellis_quantize_tiles(t(tiles), K)[1]
    assert np.array_equal(again.cpu().numpy(), st)


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_pack_states_matches_oracle_layout(K):
    """states -> packed kernel layout, bit-equal to the oracle's packer; the HIP dequantizer
    reads the weights back."""
    from glq_amd import ext
    m, n = 64, 192
    say("pack states", K)
    p0 = O.random_packed(m, n, K, seed=K)
    st = O.trellis_states(p0, m, n).astype(np.int32)            # valid tail-biting sequences
    packed = ext.trellis_pack_states(t(st), m, n, K)
    assert np.array_equal(packed.cpu().numpy(), O.pack_layer_from_states(st, m, n, K))
    assert np.array_equal(packed.cpu().numpy(), p0)


def test_quantize_matrix_round_trip():
    """Whole encode path on the GPU: Gaussian matrix -> tiles -> Viterbi -> pack, then the
    decode kernels: decompress equals the encoder's own reconstruction bit for bit, and the
    quantization error is what 4 bpw gives (relative error ~0.07-0.1)."""
    from glq_amd import ext
    say("quantize matrix")
    m, n, K = 64, 128, 4
    W = torch.randn(m, n, generator=torch.Generator().manual_seed(0)) * 0.8934
    packed, recon = ext.trellis_quantize_matrix(W.to(DEV), K)
    Wd = ext.glq_decompress_trellis_3inst_cuda(packed, m, n)
    assert torch.equal(Wd.float(), recon)
    hat_ref, st_ref = O.trellis_quantize_tiles(O.matrix_to_tiles(W.numpy()), K)
    assert np.array_equal(packed.cpu().numpy(), O.pack_layer_from_states(st_ref, m, n, K))
    err = float(((recon.cpu() - W) ** 2).sum() / (W ** 2).sum())
    assert err < 0.02, err

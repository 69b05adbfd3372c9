"""Pins the oracle's FHT / RHT / E8 functions (CPU only)."""
import hashlib

import numpy as np
import pytest

from oracle import glq_oracle as O


def sylvester(n):
    i = np.arange(n)
    pc = np.array([[bin(a & b).count("1") for b in i] for a in i])
    return ((-1.0) ** pc / np.sqrt(n)).astype(np.float64)


@pytest.mark.parametrize("n", [1, 2, 4, 16, 64])
def test_fht_is_sylvester_matrix(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((3, n)).astype(np.float32)
    want = x.astype(np.float64) @ sylvester(n).T
    assert np.allclose(O.fht(x), want, atol=1e-5)


def test_fht_known_value_involution_parseval():
    assert np.allclose(O.fht(np.array([3.0, 1.0])), np.array([4.0, 2.0]) / np.sqrt(2))
    x = np.random.default_rng(0).standard_normal((4, 512)).astype(np.float32)
    y = O.fht(x)
    assert np.allclose(O.fht(y), x, atol=1e-4)
    assert np.allclose((y ** 2).sum(-1), (x ** 2).sum(-1), rtol=1e-4)


def test_fht_matches_reference_outputs(golden):
    g = golden("rht_fht")
    assert np.array_equal(O.fht(g["fht_x"]), g["fht_y"])
    assert list(g["bd_blocks"]) == O.block_decompose(960) == [512, 256, 128, 64]
    assert np.array_equal(O.block_diag_fht(g["bd_x"], list(g["bd_blocks"])), g["bd_y"])


def test_block_decompose_doctest_values():
    assert O.block_decompose(2688) == [2048, 512, 128]
    assert O.block_decompose(4096) == [4096]
    assert O.block_decompose(5376) == [4096, 1024, 256]
    assert O.block_decompose(48) == [32, 16] and O.block_decompose(10) == [8, 2]
    assert O.block_decompose(11008) == [8192, 2048, 512, 256]
    assert O.block_decompose(14336) == [8192, 4096, 2048]


def test_block_meta_columns():
    meta = O.pack_block_meta([2048, 512, 128])
    assert meta.dtype == np.int32 and meta.shape == (3, 4)
    assert meta[:, 0].tolist() == [0, 2048, 2560]
    assert meta[:, 1].tolist() == [2048, 512, 128]
    assert meta[:, 2].tolist() == [11, 9, 7]
    assert meta[:, 3].tolist() == [0, 0, 0]
    sm = O.pack_shard_meta([[2048], [512, 256]])
    assert sm[:, 0].tolist() == [0, 2048, 2560]
    assert sm[0, 3] == np.array([1.0 / np.sqrt(np.float32(2048))], np.float32).view(np.int32)[0]
    assert sm[1, 3] == 0 and sm[2, 3] == 0


def test_rht_signs_and_transforms_match_reference(golden):
    g = golden("rht_fht")
    su, sv = O.rht_signs(96, 160, 42)
    assert np.array_equal(su, g["rht_su"]) and np.array_equal(sv, g["rht_sv"])
    bm, bn = O.block_decompose(96), O.block_decompose(160)
    Wt = O.rht_transform_weights(g["rht_W"], su, sv, bm, bn)
    assert np.allclose(Wt, g["rht_Wt"], atol=1e-5)
    xh = O.block_diag_fht(g["rht_x"] * sv[None], bn)
    assert np.array_equal(xh, g["rht_xhat"])


# ---------------------------------------------------------------- E8 table
def test_e8_table_identity_and_invariants(golden):
    t = O.e8_table()
    assert t.shape == (65536, 8) and t.dtype == np.float32
    assert hashlib.sha256(t.tobytes()).hexdigest() == \
        "c46821e43e5a573cc3431a06377121bc3b7d694e6ae0d20cb8e765c97b47cff7"
    n2 = (t * t).sum(-1)
    assert np.all(np.diff(n2) >= 0)
    counts = [int((n2 == v).sum()) for v in (0, 2, 4, 6, 8, 10, 12)]
    assert counts == [1, 240, 2160, 6720, 17520, 30240, 8655]
    frac = t - np.floor(t)
    is_int = np.all(frac == 0, axis=1)
    is_half = np.all(frac == 0.5, axis=1)
    assert np.all(is_int | is_half) and int(is_half.sum()) == 36497
    assert np.all(t.sum(-1) % 2 == 0)
    assert len(np.unique(t, axis=0)) == 65536
    # the nibble packing is the reference's codebook_packed
    g = golden("e8_layer")
    assert np.array_equal(O.e8_nibbles().view(np.int32), g["packed_table"])


def test_e8_nearest_matches_reference(golden):
    g = golden("e8_layer")
    _, idx = O.e8_quantize(g["nn_x"])
    assert np.array_equal(idx.astype(np.uint16), g["nn_idx"])
    x = g["nn_x"][:512]
    d1, i1 = O.e8_quantize(x)
    d2, i2 = O.e8_quantize((x - d1) * np.float32(3.0))
    assert np.array_equal(i1.astype(np.uint16), g["rvq_i1"])
    assert np.array_equal(i2.astype(np.uint16), g["rvq_i2"])
    assert np.allclose(d1 + d2 / np.float32(3.0), g["rvq_dec"], atol=1e-6)


def test_e8_nearest_brute_force_small():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 8)).astype(np.float32)
    t = O.e8_table()
    d = ((x[:, None, :].astype(np.float64) - t[None].astype(np.float64)) ** 2).sum(-1)
    _, idx = O.e8_quantize(x)
    assert np.allclose(d[np.arange(64), idx], d.min(-1), atol=1e-5)


def test_e8_dequant_matmul_naive_and_boundaries():
    rng = np.random.default_rng(2)
    t = O.e8_table()
    Q = rng.integers(0, 65536, size=(32, 16)).astype(np.uint16)
    Q[0, 0] = 0
    Q[0, 1] = 65535
    Qi = Q.view(np.int16)
    assert Qi[0, 1] == -1
    x = rng.standard_normal((3, 128)).astype(np.float32)
    W = np.zeros((32, 128), np.float32)
    for i in range(32):
        for j in range(16):
            W[i, 8 * j:8 * j + 8] = t[int(Q[i, j])]
    assert np.array_equal(W[0, 0:8], t[0]) and np.array_equal(W[0, 8:16], t[65535])
    want = x @ W.T * np.float32(0.37)
    got = O.e8_dequant_matmul(x, Qi, 0.37)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    Q2 = rng.integers(0, 65536, size=(32, 16)).astype(np.uint16).view(np.int16)
    assert np.array_equal(O.e8_dequant_matmul(x, Qi, 0.37, Q2, 0.0), got)
    two = O.e8_dequant_matmul(x, Qi, 0.37, Q2, 1.0 / 3.0)
    W2 = O.e8_decode(Q2.reshape(-1)).reshape(32, 128)
    assert np.allclose(two, x @ (W + W2 / 3.0).T * 0.37, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("tag,bpw,bd", [("bd2", 2, True), ("bd4", 4, True),
                                        ("p2", 2, False), ("p4", 4, False)])
def test_e8_layer_quantize_and_forward_match_reference(golden, tag, bpw, bd):
    g = golden("e8_layer")
    W = g[f"{tag}_W"]
    art, hat = O.e8_quantize_layer(W, bpw=bpw, seed=42, block_diagonal=bd)
    assert art["blocks_m"] == list(g[f"{tag}_blocks_m"])
    assert art["blocks_n"] == list(g[f"{tag}_blocks_n"])
    assert np.array_equal(art["SU"], g[f"{tag}_SU"]) and np.array_equal(art["SV"], g[f"{tag}_SV"])
    assert np.isclose(float(art["Wscale"]), float(g[f"{tag}_Wscale"]), rtol=1e-6)
    if tag != "p2":
        # (p2 pads 100 -> 128 columns, which makes the transformed Hessian of the
        # reference non-identity, so its LDLQ feedback is not plain rounding)
        same = (art["Qidxs"] == g[f"{tag}_Qidxs"]).mean()
        assert same > 0.999, same        # fp32 summation order may flip a near-tie
    # forward from the REFERENCE's artifacts must reproduce the reference's output
    ref_art = {"Qidxs": g[f"{tag}_Qidxs"], "SU": g[f"{tag}_SU"], "SV": g[f"{tag}_SV"],
               "Wscale": g[f"{tag}_Wscale"], "blocks_m": list(g[f"{tag}_blocks_m"]),
               "blocks_n": list(g[f"{tag}_blocks_n"])}
    if bpw == 4:
        ref_art["Qidxs2"] = g[f"{tag}_Qidxs2"]
        ref_art["inv_resid_scale"] = g[f"{tag}_inv_resid_scale"]
    m, n = W.shape
    y = O.e8_linear_forward(g[f"{tag}_x"], ref_art, n, m)
    assert O.rel_fro(y, g[f"{tag}_y"]) < 1e-5
    # and equals x @ W_hat^T with the reference's own dequantised weight
    assert O.rel_fro(y, g[f"{tag}_x"] @ g[f"{tag}_W_hat"].T) < 1e-4


def test_embedding_rows_closed_form():
    """Embedding lookup against the Sylvester matrix written out (n = 32) and against the
    linear-layer pieces used row by row."""
    rng = np.random.default_rng(5)
    vocab, n = 11, 32
    tab = O.e8_table()
    q1 = rng.integers(0, 65536, (vocab, n // 8)).astype(np.uint16).view(np.int16)
    q2 = rng.integers(0, 65536, (vocab, n // 8)).astype(np.uint16).view(np.int16)
    sv = rng.choice([-1.0, 1.0], n).astype(np.float32)
    ws = rng.uniform(0.5, 2.0, vocab).astype(np.float32)
    inv = rng.uniform(0.1, 0.5, vocab).astype(np.float32)
    ids = np.array([[3, 0], [10, 3]])
    got = O.e8_embedding_rows(ids, q1, sv, ws, q2, inv, embedding_dim=27, embed_scale=1.5)
    assert got.shape == (2, 2, 27)
    H = sylvester(n)
    for (a, b), i in np.ndenumerate(ids):
        row = np.concatenate([tab[int(c) & 0xFFFF] for c in q1[i].view(np.uint16)]).astype(np.float64)
        row2 = np.concatenate([tab[int(c) & 0xFFFF] for c in q2[i].view(np.uint16)]).astype(np.float64)
        want = (H @ ((row + row2 * inv[i]) * ws[i])) * sv * 1.5
        assert np.allclose(got[a, b], want[:27], atol=1e-5)
    # one stage == the dequantizer of the linear path on the same rows
    one = O.e8_embedding_rows(np.arange(vocab), q1, sv, ws)
    W = O.e8_dequant(q1) * ws[:, None]
    assert np.allclose(one, O.fht(W) * sv, atol=1e-6)


@pytest.mark.parametrize("tag,bpw", [("bd2", 2), ("bd4", 4), ("p2", 2), ("p4", 4)])
def test_dense_weight_matches_reference_dequantize(golden, tag, bpw):
    """The weight-domain matrix against the reference's own `dequantize()` output (stored for the
    power-of-two layers, the only ones its method takes) and against the weight its quantizer
    returned for every layer; a transposed transform, a swapped sign vector or a missing scale
    fails both."""
    g = golden("e8_layer")
    inv = float(g[f"{tag}_inv_resid_scale"]) if bpw == 4 else 0.0
    W_rht = O.e8_dequant(g[f"{tag}_Qidxs"], g[f"{tag}_Qidxs2"] if bpw == 4 else None, inv) \
        * np.float32(g[f"{tag}_Wscale"])
    m, n = g[f"{tag}_W"].shape
    W = O.dense_weight(W_rht, g[f"{tag}_SU"], g[f"{tag}_SV"], list(g[f"{tag}_blocks_m"]),
                       list(g[f"{tag}_blocks_n"]), m, n)
    assert W.shape == (m, n)
    assert O.rel_fro(W, g[f"{tag}_W_hat"]) < 1e-5
    if f"{tag}_dequantize" in g.files:
        assert O.rel_fro(W, g[f"{tag}_dequantize"]) < 1e-6
    # forward(x) == x @ dequantize().T  (tests/test_quantized_linear.py:120-131)
    assert O.rel_fro(g[f"{tag}_x"] @ W.T, g[f"{tag}_y"]) < 1e-5

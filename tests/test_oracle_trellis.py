"""Pins the oracle's trellis-3INST functions (CPU only)."""
import hashlib

import numpy as np
import pytest

from oracle import glq_oracle as O


KNOWN = {0: 0x3a25, 1: 0xbb5b, 2: 0x3b74, 255: 0x3cd1, 32768: 0xb7f8, 65535: 0xb110}


def test_decode_3inst_known_answers_and_lut_hash(golden):
    for s, bits in KNOWN.items():
        assert int(O.decode_3inst(np.array([s])).view(np.uint16)[0]) == bits, s
    lut = O.lut_3inst()
    assert hashlib.sha256(lut.tobytes()).hexdigest() == \
        "ad88de2dcff5bb05fff2faec37cceceb43aa1c2e8203f9d81a6fbd6dd3393eea"
    g = golden("trellis_storage")
    assert np.array_equal(lut.view(np.uint16), g["lut_fp16"].view(np.uint16))
    assert np.isclose(O.trellis_opt_scale(), float(g["opt_scale_K4"]), rtol=1e-9)
    assert np.isclose(O.trellis_opt_scale(), 0.8933837, rtol=1e-6)
    assert not np.isnan(lut.astype(np.float32)).any()


def test_permute_closed_form():
    for t in range(256):
        l, j = t >> 3, t & 7
        row = (l >> 2) + 8 * ((j >> 1) & 1)
        col = 2 * (l & 3) + 8 * (j >> 2) + (j & 1)
        assert O.PERMUTE[t] == 16 * row + col
    assert sorted(O.PERMUTE.tolist()) == list(range(256))


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_decode_layer_matches_reference(golden, K):
    g = golden("trellis_storage")
    packed, want = g[f"K{K}_packed"], g[f"K{K}_decoded"]
    got = O.decode_layer(packed, 64, 128)
    assert np.array_equal(got, want.astype(np.float32))
    # the states themselves, in the reference's (m, n) slab order
    st = O.trellis_states(packed, 64, 128)                       # (tiles, 256)
    q = g[f"K{K}_Qidxs"].astype(np.int64)                        # (m, n) rows of 16 per tile
    q_tiles = q.reshape(4, 16, 8, 16).transpose(0, 2, 1, 3).reshape(32, 256)
    assert np.array_equal(st, q_tiles)
    # repacking the states reproduces the reference's bytes exactly
    assert np.array_equal(O.pack_layer_from_states(st, 64, 128, K), packed)


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_natural_layout_is_big_endian_stream(golden, K):
    """The un-flipped packing holds each tile's stream as big-endian int16 words."""
    g = golden("trellis_storage")
    nat = g[f"K{K}_packed_natural"]
    sb = O.kernel_to_stream_bytes(g[f"K{K}_packed"], 64, 128, K)
    assert np.array_equal(nat.view(np.uint16).byteswap().view(np.uint8).reshape(sb.shape), sb)


# ---- second, independent formulation: per-lane walk over the kernel layout ----
def lane_walk_decode(packed, m, n):
    """Reads the kernel-layout bytes the way a 32-lane group does: lane l of block
    (mp, kp) owns one 4K-byte record holding its 8K-bit chunk of four tiles
    [(k0,m0),(k0,m1),(k1,m0),(k1,m1)], little-endian, and borrows 16 bits from lane
    l+1 (K=1: lanes l+1 and l+2).  Independent of oracle.decode_layer: no bit
    arrays, no PERMUTE table."""
    K = packed.shape[1] // 16
    raw = np.ascontiguousarray(packed).view(np.uint8).reshape(-1)
    lut = O.lut_3inst().astype(np.float32)
    W = np.zeros((m, n), np.float32)
    nkp = n // 32
    for mp in range(m // 32):
        for kp in range(nkp):
            base = (mp * nkp + kp) * 128 * K
            chunk = np.zeros((32, 2, 2), np.int64)               # [lane][ks][ms]
            for l in range(32):
                for ks in range(2):
                    for ms in range(2):
                        o = base + l * 4 * K + (ks * 2 + ms) * K
                        chunk[l, ks, ms] = int.from_bytes(raw[o:o + K].tobytes(), "little")
            for l in range(32):
                for ks in range(2):
                    for ms in range(2):
                        c = int(chunk[l, ks, ms])
                        if K >= 2:
                            cont = (int(chunk[(l + 1) % 32, ks, ms]) >> (8 * K - 16)) & 0xFFFF
                        else:
                            cont = ((int(chunk[(l + 1) % 32, ks, ms]) & 0xFF) << 8) | \
                                   (int(chunk[(l + 2) % 32, ks, ms]) & 0xFF)
                        ext = (c << 16) | cont
                        for j in range(8):
                            s = (ext >> (8 * K - K * j)) & 0xFFFF
                            row = 32 * mp + 16 * ms + (l >> 2) + 8 * ((j >> 1) & 1)
                            col = 32 * kp + 16 * ks + 2 * (l & 3) + 8 * (j >> 2) + (j & 1)
                            W[row, col] = lut[s]
    return W


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_lane_walk_equals_decode_layer(golden, K):
    g = golden("trellis_storage")
    assert np.array_equal(lane_walk_decode(g[f"K{K}_packed"], 64, 128),
                          g[f"K{K}_decoded"].astype(np.float32))
    rnd = O.random_packed(32, 64, K, seed=K)
    assert np.array_equal(lane_walk_decode(rnd, 32, 64), O.decode_layer(rnd, 32, 64))


def test_hand_placed_states_round_trip():
    """A path built by hand: state t+1 = (state t << K | new bits) & 0xFFFF, cyclic."""
    K = 2
    rng = np.random.default_rng(9)
    bits = rng.integers(0, 2, size=(8, 512))
    ext = np.concatenate([bits, bits[:, :16]], axis=1)
    st = np.zeros((8, 256), np.int64)
    for t in range(256):
        for i in range(16):
            st[:, t] |= ext[:, K * t + i].astype(np.int64) << (15 - i)
    packed = O.pack_layer_from_states(st, 64, 32, K)
    assert packed.shape == (8, 32) and packed.dtype == np.int16
    assert np.array_equal(O.trellis_states(packed, 64, 32), st)
    W = O.decode_layer(packed, 64, 32)
    lut = O.lut_3inst().astype(np.float32)
    # tile 3 = rows 16..31, cols 16..31 ; step 8*l+j sits at the closed-form position
    t = 8 * 13 + 5
    assert W[16 + (13 >> 2) + 8 * ((5 >> 1) & 1), 16 + 2 * (13 & 3) + 8 * (5 >> 2) + (5 & 1)] \
        == lut[st[3, t]]
    with pytest.raises(ValueError):
        bad = st.copy()
        bad[0, 5] ^= 1 << 9
        O.pack_states(bad, K)


def test_bits_from_packed_refuses_bad_width():
    assert O.trellis_bits_from_packed(np.zeros((4, 48), np.int16)) == 3
    with pytest.raises(ValueError, match="bits/weight"):
        O.trellis_bits_from_packed(np.zeros((4, 80), np.int16))


@pytest.mark.parametrize("K", [2, 4])
def test_viterbi_matches_reference(golden, K):
    g = golden("trellis_viterbi")
    hat, st = O.trellis_quantize_tiles(g[f"K{K}_tiles"], K)
    assert np.array_equal(st.astype(np.uint16), g[f"K{K}_states"])
    assert np.array_equal(hat, g[f"K{K}_hat"])


@pytest.mark.parametrize("K", [1, 3])
def test_viterbi_matches_reference_layer_states(golden, K):
    """The rates the tile vectors above do not cover, on the states the reference's trellis_ldlq
    (identity Hessian: no feedback, glq/trellis.py:649-688) wrote for a 64 x 128 layer: tile (i, k)
    is rows 16i.., columns 16k.. of W / Wscale in step order, its states the same window of Qidxs."""
    g = golden("trellis_storage")
    W = g[f"K{K}_W"]
    m, n = W.shape
    tiles = O.matrix_to_tiles((W / np.float32(g[f"K{K}_Wscale"])).astype(np.float32))
    want = g[f"K{K}_Qidxs"].reshape(m // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(-1, 256)
    sel = [0, 7, 13, 31] if K == 1 else [0, 5, 9, 14, 22, 31]
    hat, st = O.trellis_quantize_tiles(tiles[sel], K)
    assert np.array_equal(st.astype(np.uint16), want[sel])
    dec = O.matrix_to_tiles(g[f"K{K}_decoded"].astype(np.float32))
    assert np.array_equal(hat, dec[sel])


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_fast_unpack_equals_bit_array_unpack(K):
    p = O.random_packed(64, 128, K, seed=40 + K)
    sb = O.kernel_to_stream_bytes(p, 64, 128, K)
    assert np.array_equal(O.unpack_states_fast(sb, K), O.unpack_states(sb, K))
    big = O.random_packed(512, 192, K, seed=K)
    assert np.array_equal(O.decode_layer(big, 512, 192, fast=True), O.decode_layer(big, 512, 192))


def test_nstage_sum():
    p1 = O.random_packed(32, 64, 4, 1)
    p2 = O.random_packed(32, 64, 2, 2)
    got = O.decode_layer_nstage([p1, p2], [1.0, 0.31], 32, 64)
    want = O.decode_layer(p1, 32, 64) + O.decode_layer(p2, 32, 64) * np.float32(0.31)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("tag", ["k2", "k4", "k4k2"])
def test_trellis_layer_forward_matches_reference(golden, tag):
    g = golden("trellis_layer")
    W = g[f"{tag}_W"]
    m, n = W.shape
    art = {"trellis_packed": g[f"{tag}_trellis_packed"], "SU": g[f"{tag}_SU"],
           "SV": g[f"{tag}_SV"], "Wscale": g[f"{tag}_Wscale"],
           "blocks_m": list(g[f"{tag}_blocks_m"]), "blocks_n": list(g[f"{tag}_blocks_n"])}
    if tag == "k4k2":
        art["trellis_packed2"] = g[f"{tag}_trellis_packed2"]
        art["inv_resid_scale2"] = g[f"{tag}_inv_resid_scale2"]
    y = O.trellis_linear_forward(g[f"{tag}_x"], art, n, m)
    assert O.rel_fro(y, g[f"{tag}_y"]) < 1e-5
    assert O.rel_fro(y, g[f"{tag}_x"] @ g[f"{tag}_W_hat"].T) < 1e-4
    # the oracle's own quantiser reproduces the reference's signs and scale, and its
    # bytes wherever the fp32 transform agrees to the last bit
    K = art["trellis_packed"].shape[1] // 16
    if tag != "k4k2":
        mine, _ = O.trellis_quantize_layer(W, K=K, seed=42)
        assert np.array_equal(mine["SU"], art["SU"]) and np.array_equal(mine["SV"], art["SV"])
        assert np.isclose(float(mine["Wscale"]), float(art["Wscale"]), rtol=1e-6)
        same = (mine["trellis_packed"] == art["trellis_packed"]).mean()
        assert same > 0.95, same

"""E8RHTLinear.dequantize() / dequantize_glq_weight on the HIP path against the reference's stored
`dequantize()` outputs, its quantizer's returned weights, and the oracle (needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t

pytestmark = pytest.mark.gpu


def _shell_layer(g, tag, bpw, bd):
    from glq_amd.quantized_linear import E8RHTLinear
    m, n = g[f"{tag}_W"].shape
    keys = ["Qidxs", "SU", "SV", "Wscale"] + (["Qidxs2", "inv_resid_scale"] if bpw == 4 else [])
    layer = E8RHTLinear(n, m, block_diagonal=bd)
    layer.load_state_dict({k: torch.from_numpy(np.asarray(g[f"{tag}_{k}"])) for k in keys})
    layer.to(DEV)
    cb = e8_table_f16()
    layer.set_codebook(cb, cb if bpw == 4 else None)
    return layer


@pytest.mark.parametrize("tag,bpw,bd", [("bd2", 2, True), ("bd4", 4, True), ("p2", 2, False), ("p4", 4, False)])
def test_shell_dequantize_matches_reference(golden, tag, bpw, bd):
    """fp32 decode + fp32 transforms: the reference's own `dequantize()` output (power-of-two
    layers) and the weight its quantizer returned, to fp32 rounding (1e-5; the transforms sum in
    another order than the reference's butterflies)."""
    g = golden("e8_layer")
    say("dequantize shell", tag)
    layer = _shell_layer(g, tag, bpw, bd)
    W = layer.dequantize()
    m, n = g[f"{tag}_W"].shape
    assert W.shape == (m, n) and W.dtype == torch.float32
    if f"{tag}_dequantize" in g.files:
        assert rel(W, g[f"{tag}_dequantize"]) < 1e-5, rel(W, g[f"{tag}_dequantize"])
    assert rel(W, g[f"{tag}_W_hat"]) < 1e-5, rel(W, g[f"{tag}_W_hat"])
    # forward(x) == x @ dequantize().T (tests/test_quantized_linear.py:120-131), here against the
    # fp16-activation forward path: the 1e-2 bound of the path
    x = torch.from_numpy(g[f"{tag}_x"]).to(DEV)
    assert rel(layer(x.half()), (x @ W.t()).cpu().numpy()) < 1e-2
    assert torch.equal(W, layer.dequantize())
    # the helper with the reference's argument order returns the same matrix in fp16
    from glq_amd.dequant import dequantize_glq_weight
    cb = e8_table_f16()
    Wh = dequantize_glq_weight(layer.Qidxs, layer.SU, layer.SV, layer.Wscale, cb,
                               layer.Qidxs2 if bpw == 4 else None,
                               float(layer.inv_resid_scale) if bpw == 4 else 0.0, cb if bpw == 4 else None,
                               out_features=m, in_features=n)
    assert Wh.dtype == torch.float16 and torch.equal(Wh, W.half())


@pytest.mark.parametrize("stages", [3, 4])
def test_shell_dequantize_three_and_four_stages_against_oracle(stages):
    from glq_amd.quantized_linear import E8RHTLinear
    say("dequantize shell stages", stages)
    m, n = 96, 320
    rng = np.random.default_rng(stages)
    q = [rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16) for _ in range(stages)]
    inv = [1 / 3.0, 1 / 9.0, 1 / 27.0][:stages - 1] + [0.0] * (4 - stages)
    su, sv = O.rht_signs(m, n, 7)
    layer = E8RHTLinear(n, m, block_diagonal=True)
    sd = {"Qidxs": q[0], "Qidxs2": q[1], "Qidxs3": q[2], "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
          "Wscale": np.float32(0.013), "inv_resid_scale": np.float32(inv[0]), "inv_resid_scale2": np.float32(inv[1]),
          "inv_resid_scale3": np.float32(inv[2])}
    if stages == 4:
        sd["Qidxs4"] = q[3]
    layer.load_state_dict({k: torch.from_numpy(np.asarray(v)) for k, v in sd.items()}, strict=False)
    layer.to(DEV)
    cb = e8_table_f16()
    layer.set_codebook(cb, cb)
    W_rht = O.e8_dequant(q[0], q[1], inv[0], q[2], inv[1], q[3] if stages == 4 else None, inv[2]) * np.float32(0.013)
    ref = O.dense_weight(W_rht, su, sv, O.block_decompose(m), O.block_decompose(n), m, n)
    assert rel(layer.dequantize(), ref) < 1e-5


@pytest.mark.parametrize("tag", ["k2", "k4", "k4k2"])
def test_trellis_dequantize_matches_reference_weight(golden, tag):
    """Trellis layers (the reference module has no dequantize for them; its quantizer returns the
    weight): decode_layer_nstage in the transform domain, then the same two inverse transforms."""
    from glq_amd.quantized_linear import E8RHTLinear
    g = golden("trellis_layer")
    say("dequantize trellis", tag)
    m, n = g[f"{tag}_W"].shape
    keys = ["trellis_packed", "SU", "SV", "Wscale"] + (["trellis_packed2", "inv_resid_scale2"] if tag == "k4k2" else [])
    layer = E8RHTLinear(n, m, codebook_type="trellis")
    layer.load_state_dict({k: torch.from_numpy(np.asarray(g[f"{tag}_{k}"])) for k in keys})
    layer.to(DEV)
    W = layer.dequantize()
    assert rel(W, g[f"{tag}_W_hat"]) < 1e-5, rel(W, g[f"{tag}_W_hat"])
    packs = [g[f"{tag}_trellis_packed"]] + ([g[f"{tag}_trellis_packed2"]] if tag == "k4k2" else [])
    cum = [1.0] + ([float(g[f"{tag}_inv_resid_scale2"])] if tag == "k4k2" else [])
    W_rht = O.decode_layer_nstage(packs, cum, m, n) * np.float32(g[f"{tag}_Wscale"])
    ref = O.dense_weight(W_rht, g[f"{tag}_SU"], g[f"{tag}_SV"], list(g[f"{tag}_blocks_m"]),
                         list(g[f"{tag}_blocks_n"]), m, n)
    assert rel(W, ref) < 1e-5
    x = torch.from_numpy(g[f"{tag}_x"]).to(DEV)
    assert rel(layer(x.half()), (x @ W.t()).cpu().numpy()) < 1e-2


def test_dequantize_of_a_full_size_layer_reproduces_the_forward():
    """2048 x 11008 trellis (a down projection of configs[1]): `x @ dequantize().T` against the fused
    forward on the same layer -- the size-independent property, where the oracle would take minutes."""
    from glq_amd.quantized_linear import E8RHTLinear
    say("dequantize 2048x11008")
    m, n = 2048, 11008
    su, sv = O.rht_signs(m, n, 5)
    layer = E8RHTLinear(n, m, codebook_type="trellis")
    layer.load_state_dict({"trellis_packed": torch.from_numpy(O.random_packed(m, n, 4, 9)),
                           "SU": torch.from_numpy(su.astype(np.float16)), "SV": torch.from_numpy(sv.astype(np.float16)),
                           "Wscale": torch.tensor(0.0179)})
    layer.to(DEV)
    W = layer.dequantize()
    assert W.shape == (m, n)
    x = torch.randn(8, n, generator=torch.Generator().manual_seed(0)).to(DEV)
    y = layer(x.to(torch.bfloat16))
    assert rel(y, (x.to(torch.bfloat16).float() @ W.t()).cpu().numpy()) < 1e-2
    # orthogonal transforms keep the Frobenius norm: ||W|| = Wscale * ||decoded||
    from glq_amd import ext
    dec = ext.glq_decompress_trellis_3inst_cuda(layer.trellis_packed, m, n).float()
    assert abs(float(W.norm()) / (0.0179 * float(dec.norm())) - 1.0) < 1e-4

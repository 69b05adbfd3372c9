"""Writes tests/golden/*.npz from the reference implementation.

Run in the development container only (the reference checkout is not present
anywhere else):

    TORCHDYNAMO_DISABLE=1 python tests/golden/make_golden.py /root/reference

It imports the reference's CPU code paths for the functions that nothing else
pins absolutely -- the trellis pack/decode direction conventions, the Viterbi and
nearest-E8 tie-breaks, and the end-to-end CPU forward of E8RHTLinear -- and stores
inputs and expected outputs as small arrays.  No reference source is stored.
"""
import os
import sys

import numpy as np
import torch

os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, ref_root)
OUT = os.path.dirname(os.path.abspath(__file__))

import glq.trellis as gt                      # noqa: E402
from glq.codebook import E8ShellCodebook       # noqa: E402
from glq.quantized_linear import E8RHTLinear   # noqa: E402
from glq.quantize_model import quantize_layer_e8_shell_rht  # noqa: E402
from glq.hadamard import _pytorch_fht, block_diagonal_fht, _block_decompose  # noqa: E402
from glq.rht import RHT                        # noqa: E402


def np16(t):
    return t.detach().cpu().numpy()


def trellis_storage():
    """pack_layer / decode_layer on real Viterbi output, K=1..4, 64x128."""
    out = {}
    m, n = 64, 128
    for K in (1, 2, 3, 4):
        torch.manual_seed(K)
        cb = gt.TrellisCodebook(variant="3inst", K=K, device="cpu")
        W = (torch.randn(m, n) * 0.05).float()
        hatWr, Qidxs, Wscale = gt.trellis_ldlq(W, torch.eye(n), cb, for_kernel=True)
        packed = gt.pack_layer(cb, Qidxs, m, n, has_kernel=True)
        dec = gt.decode_layer(cb, packed, m, n, has_kernel=True)
        assert torch.equal(dec.float(), hatWr.float())
        out[f"K{K}_W"] = np16(W)
        out[f"K{K}_Wscale"] = np.float64(Wscale)
        out[f"K{K}_Qidxs"] = np16(Qidxs).astype(np.uint16)
        out[f"K{K}_packed"] = np16(packed)
        out[f"K{K}_decoded"] = np16(dec).astype(np.float16)
        assert np.array_equal(out[f"K{K}_decoded"].astype(np.float32), np16(dec))
        # natural (un-flipped) packing of the same states, to pin the byte flip alone
        out[f"K{K}_packed_natural"] = np16(gt.pack_layer(cb, Qidxs, m, n, has_kernel=False))
    lut = gt.decode_3inst(torch.arange(1 << 16))
    out["lut_fp16"] = np16(lut).astype(np.float16)
    out["opt_scale_K4"] = np.float64(gt.TrellisCodebook(variant="3inst", K=4).opt_scale)
    np.savez_compressed(os.path.join(OUT, "trellis_storage.npz"), **out)


def trellis_viterbi():
    """bitshift_codebook.quantize on a few tiles: tie-breaks, fp16 cast, tail-biting."""
    out = {}
    for K in (2, 4):
        torch.manual_seed(100 + K)
        cb = gt.TrellisCodebook(variant="3inst", K=K, device="cpu")
        tiles = torch.randn(6, 256) * 1.1
        hat, st = cb.quantize_tiles(tiles)
        out[f"K{K}_tiles"] = np16(tiles)
        out[f"K{K}_hat"] = np16(hat).astype(np.float32)
        out[f"K{K}_states"] = np16(st).astype(np.uint16)
    np.savez_compressed(os.path.join(OUT, "trellis_viterbi.npz"), **out)


def trellis_layer():
    """quantize_layer_trellis_rht + E8RHTLinear CPU forward, 1- and 2-stage."""
    out = {}
    for tag, m, n, ks in (("k2", 64, 128, [2]), ("k4", 96, 192, [4]), ("k4k2", 64, 128, [4, 2])):
        torch.manual_seed(7)
        W = (torch.randn(m, n) * 0.02).float()
        cbs = [gt.TrellisCodebook(variant="3inst", K=k, device="cpu") for k in ks]
        W_hat, art = gt.quantize_layer_trellis_rht(W, torch.eye(n), cbs if len(cbs) > 1 else cbs[0])
        layer = E8RHTLinear(n, m, codebook_type="trellis")
        sd = {k: v for k, v in art.items()}
        layer.load_state_dict(sd, strict=False)
        layer.set_codebook(cbs[0], cbs[1] if len(cbs) > 1 else None)
        x = torch.randn(5, n)
        y = layer(x)
        out[f"{tag}_W"] = np16(W)
        out[f"{tag}_W_hat"] = np16(W_hat)
        out[f"{tag}_x"] = np16(x)
        out[f"{tag}_y"] = np16(y)
        for k, v in art.items():
            out[f"{tag}_{k}"] = np16(v)
        out[f"{tag}_blocks_m"] = np.array(layer.blocks_m)
        out[f"{tag}_blocks_n"] = np.array(layer.blocks_n)
    np.savez_compressed(os.path.join(OUT, "trellis_layer.npz"), **out)


def e8_layer():
    """quantize_layer_e8_shell_rht (H=I) + E8RHTLinear CPU forward at 2 and 4 bpw,
    block-diagonal and legacy pow2-padded."""
    out = {}
    cb = E8ShellCodebook.build(device="cpu", verbose=False)
    for tag, m, n, bpw, bd in (("bd2", 96, 160, 2, True), ("bd4", 96, 160, 4, True),
                               ("p2", 48, 100, 2, False), ("p4", 64, 128, 4, False)):
        torch.manual_seed(11)
        W = (torch.randn(m, n) * 0.02).float()
        W_hat, art, met = quantize_layer_e8_shell_rht(W, torch.eye(n), cb, bpw=bpw,
                                                     block_diagonal=bd)
        layer = E8RHTLinear(n, m, block_diagonal=bd)
        layer.load_state_dict(dict(art), strict=False)
        layer.set_codebook(cb, cb if bpw == 4 else None)
        x = torch.randn(3, n)
        y = layer(x)
        if not bd:                                    # dequantize() is pow2-only
            out[f"{tag}_dequantize"] = np16(layer.dequantize())
        out[f"{tag}_W"] = np16(W)
        out[f"{tag}_W_hat"] = np16(W_hat)
        out[f"{tag}_x"] = np16(x)
        out[f"{tag}_y"] = np16(y)
        for k, v in art.items():
            out[f"{tag}_{k}"] = np16(v)
        out[f"{tag}_blocks_m"] = np.array(layer.blocks_m)
        out[f"{tag}_blocks_n"] = np.array(layer.blocks_n)
    # nearest-neighbour search on raw vectors (ties, overload region)
    torch.manual_seed(3)
    v = torch.randn(4000, 8) * 1.3
    v[:200] = torch.round(v[:200] * 2) / 2            # exact half-grid points -> ties
    dec, idx = cb.quantize(v)
    out["nn_x"] = np16(v)
    out["nn_idx"] = np16(idx).astype(np.uint16)
    dec2, (i1, i2) = cb.quantize_rvq(v[:512])
    out["rvq_i1"] = np16(i1).astype(np.uint16)
    out["rvq_i2"] = np16(i2).astype(np.uint16)
    out["rvq_dec"] = np16(dec2)
    out["packed_table"] = np16(cb.codebook_packed).astype(np.int32)
    np.savez_compressed(os.path.join(OUT, "e8_layer.npz"), **out)


def rht_and_fht():
    out = {}
    torch.manual_seed(5)
    x = torch.randn(3, 256)
    out["fht_x"] = np16(x)
    out["fht_y"] = np16(_pytorch_fht(x.clone()))
    xb = torch.randn(2, 960)
    out["bd_x"] = np16(xb)
    out["bd_blocks"] = np.array(_block_decompose(960))
    out["bd_y"] = np16(block_diagonal_fht(xb.clone(), _block_decompose(960)))
    r = RHT(96, 160, seed=42)
    out["rht_su"] = np16(r.su)
    out["rht_sv"] = np16(r.sv)
    W = torch.randn(96, 160)
    out["rht_W"] = np16(W)
    out["rht_Wt"] = np16(r.transform_weights(W))
    xi = torch.randn(2, 160)
    out["rht_x"] = np16(xi)
    out["rht_xhat"] = np16(r.transform_input(xi))
    np.savez_compressed(os.path.join(OUT, "rht_fht.npz"), **out)


if __name__ == "__main__":
    with torch.no_grad():
        rht_and_fht()
        trellis_storage()
        trellis_viterbi()
        trellis_layer()
        e8_layer()
    for f in sorted(os.listdir(OUT)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(OUT, f)))

"""The grouped call at many tokens: layers that read the same activations (fused q/k/v, gate/up of the
reference's merged linears, glq_vllm/linear_method.py:664-710) through ONE launch of the many-token kernel."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, rel, say, t

TOL = 1e-2

pytestmark = pytest.mark.gpu


def _layers(ms, n, K, seed, shared_sv):
    from glq_amd import hadamard as H
    out = []
    sv0 = None
    for i, m in enumerate(ms):
        packed = O.random_packed(m, n, K, seed + i)
        su, sv = O.rht_signs(m, n, seed + 10 * i)
        if shared_sv:
            sv0 = sv if sv0 is None else sv0
            sv = sv0
        out.append(dict(m=m, packed=packed, su=su.astype(np.float16), sv=sv.astype(np.float16), wscale=0.02 + 0.005 * i))
    bn = O.block_decompose(n)
    return out, bn, H.pack_block_meta(bn).to(DEV)


@pytest.mark.parametrize("ms,n,B,K,shared_sv", [
    ((2048, 512, 512), 2048, 512, 4, False),       # q/k/v of the 3B shape: 16 + 4 + 4 row tiles in one launch
    ((1088, 1088), 2368, 100, 2, True),            # gate/up with one sign vector; several input blocks, one small
    ((1088, 320, 2336), 1088, 333, 3, False),      # three heights, rows of several output blocks
    ((14336,), 512, 700, 4, False),                # a single layer through the grouped entry
])
def test_grouped_many_tokens(ms, n, B, K, shared_sv):
    from glq_amd import ext
    say("grouped many tokens", ms, n, B, K, shared_sv)
    layers, bn, bn_meta = _layers(ms, n, K, 3, shared_sv)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(5)) * 0.7).to(torch.bfloat16)
    xd = x.to(DEV)
    dev = [dict(l, sv_d=t(l["sv"]), su_d=t(l["su"]), p_d=t(l["packed"])) for l in layers]
    if shared_sv:
        for l in dev[1:]:
            l["sv_d"] = dev[0]["sv_d"]                          # the same tensor: one transform of x
    shards = [(l["sv_d"], l["su_d"], l["p_d"], l["wscale"], l["m"], l["m"]) for l in dev]
    y = ext.glq_fused_linear_trellis_3inst_group(xd, shards, torch.tensor(bn), bn_meta, n, n, out_dtype=torch.bfloat16)
    assert y.shape == (B, sum(ms))
    parts = ext.glq_fused_linear_trellis_3inst_group(xd, shards, torch.tensor(bn), bn_meta, n, n,
                                                     out_dtype=torch.bfloat16, separate=True)
    assert [tuple(p.shape) for p in parts] == [(B, m) for m in ms] and all(p.is_contiguous() for p in parts)
    assert torch.equal(torch.cat(parts, 1), y)                  # the two output arrangements hold the same bits
    assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_group(xd, shards, torch.tensor(bn), bn_meta, n, n,
                                                                   out_dtype=torch.bfloat16))
    from glq_amd import hadamard as H
    rows = np.unique(np.concatenate([np.arange(0, B, 41), [B - 1, min(B - 1, 64), min(B - 1, 127)]]))
    off = 0
    for l, d in zip(layers, dev):
        m = l["m"]
        bm = O.block_decompose(m)
        art = {"trellis_packed": l["packed"], "SU": l["su"], "SV": l["sv"], "Wscale": np.float32(l["wscale"]),
               "blocks_m": bm, "blocks_n": bn}
        ref = O.trellis_linear_forward(x[rows].float().numpy(), art, n, m)
        got = y[torch.from_numpy(rows).to(DEV), off:off + m]
        assert rel(got, ref) < TOL, (m, rel(got, ref))
        # the layer on its own: another K split at most, so rounding apart
        one = ext.glq_fused_linear_trellis_3inst_cuda(xd, d["sv_d"], d["su_d"], d["p_d"], torch.tensor(bn), torch.tensor(bm),
                                                      bn_meta, H.pack_block_meta(bm).to(DEV), l["wscale"], n, m, n, m,
                                                      out_dtype=torch.bfloat16)
        assert rel(y[:, off:off + m], one.float().cpu().numpy()) < 4e-3
        off += m


def test_grouped_many_tokens_refusals():
    from glq_amd import ext
    say("grouped many tokens refusals")
    layers, bn, bn_meta = _layers((256,) * 5, 256, 2, 1, False)
    shards = [(t(l["sv"]), t(l["su"]), t(l["packed"]), l["wscale"], l["m"], l["m"]) for l in layers]
    x = torch.zeros(100, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="layers"):
        ext.glq_fused_linear_trellis_3inst_group(x, shards, torch.tensor(bn), bn_meta, 256, 256, out_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):                            # 32 tokens are served, five layers are not
        ext.glq_fused_linear_trellis_3inst_group(x[:32], shards, torch.tensor(bn), bn_meta, 256, 256,
                                                 out_dtype=torch.bfloat16)
    y32 = ext.glq_fused_linear_trellis_3inst_group(x[:32], shards[:2], torch.tensor(bn), bn_meta, 256, 256,
                                                   out_dtype=torch.bfloat16)
    assert y32.shape == (32, 512) and float(y32.abs().max()) == 0.0   # zero activations
    with pytest.raises(RuntimeError, match="separate"):
        ext.glq_fused_linear_trellis_3inst_group(x[:2], shards[:2], torch.tensor(bn), bn_meta, 256, 256,
                                                 out_dtype=torch.bfloat16, separate=True)

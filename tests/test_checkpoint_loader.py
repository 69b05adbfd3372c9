"""Checkpoint loader: a directory in the reference's on-disk format (safetensors + config.json
[+ e8_codebook.pt]) written from the reference's own layer artifacts."""
import json
import os

import numpy as np
import pytest
import torch

from glq_amd import checkpoint as C


def _write(tmp_path, tensors, qcfg):
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(tmp_path, "model.safetensors"))
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump({"model_type": "x", "quantization_config": qcfg}, f)


def _trellis_dir(tmp_path, golden):
    g = golden("trellis_layer")
    tensors = {}
    for tag, name in (("k2", "model.layers.0.self_attn.q_proj"), ("k4", "model.layers.0.mlp.up_proj"),
                      ("k4k2", "model.layers.1.mlp.down_proj")):
        for leaf in ("trellis_packed", "trellis_packed2", "SU", "SV", "Wscale", "inv_resid_scale2"):
            if f"{tag}_{leaf}" in g.files:
                tensors[f"{name}.{leaf}"] = torch.from_numpy(np.asarray(g[f"{tag}_{leaf}"]))
    tensors["model.norm.weight"] = torch.ones(8)
    _write(tmp_path, tensors, {"quant_method": "glq", "codebook": "trellis", "variant": "3inst",
                               "trellis_layout": "kernel", "block_diagonal": True, "codesz": 16, "bpw": 4})
    return g


def test_trellis_checkpoint_loads(tmp_path, golden):
    g = _trellis_dir(str(tmp_path), golden)
    lins = C.load_quantized_linears(str(tmp_path), device="cpu")
    assert sorted(lins) == ["model.layers.0.mlp.up_proj", "model.layers.0.self_attn.q_proj",
                            "model.layers.1.mlp.down_proj"]
    up = lins["model.layers.0.mlp.up_proj"]
    assert (up.out_features, up.in_features) == (96, 192) and up.blocks_m == [64, 32] and up.blocks_n == [128, 64]
    assert torch.equal(up.trellis_packed, torch.from_numpy(g["k4_trellis_packed"]))
    assert up.trellis_packed2.numel() == 0
    down = lins["model.layers.1.mlp.down_proj"]
    assert down.trellis_packed2.shape == (32, 32) and float(down.inv_resid_scale2) == float(g["k4k2_inv_resid_scale2"])


def test_shell_checkpoint_loads_block_diagonal_and_legacy(tmp_path, golden):
    g = golden("e8_layer")
    tensors = {}
    for tag, name in (("bd4", "a.b"), ("p2", "legacy.proj")):
        for leaf in ("Qidxs", "Qidxs2", "SU", "SV", "Wscale", "inv_resid_scale"):
            if f"{tag}_{leaf}" in g.files:
                tensors[f"{name}.{leaf}"] = torch.from_numpy(np.asarray(g[f"{tag}_{leaf}"]))
    _write(str(tmp_path), tensors, {"quant_method": "glq", "codebook": "e8_shell", "block_diagonal": True,
                                    "codesz": 8, "bpw": 4})
    lins = C.load_quantized_linears(str(tmp_path), device="cpu", shapes={"legacy.proj": (48, 100)})
    a = lins["a.b"]
    assert (a.out_features, a.in_features, a.block_diagonal) == (96, 160, True)
    assert torch.equal(a.Qidxs2, torch.from_numpy(g["bd4_Qidxs2"]))
    leg = lins["legacy.proj"]                      # padded to 64 x 128: recognised from the buffer shapes
    assert (leg.out_features, leg.in_features, leg.block_diagonal) == (48, 100, False)
    assert leg.blocks_m == [64] and leg.blocks_n == [128]
    assert float(leg.inv_resid_scale) == 0.0       # 2 bpw: residual keys absent
    # the bundled table is the reference's table
    from oracle import glq_oracle as O
    assert np.array_equal(C.load_shell_table(None).float().numpy(), O.e8_table())
    assert a.codebook is not None and a.codebook.shape == (65536, 8)


def test_loader_refusals(tmp_path, golden):
    _trellis_dir(str(tmp_path), golden)
    cfgp = os.path.join(str(tmp_path), "config.json")
    cfg = json.load(open(cfgp))
    for patch, exc, match in (({"trellis_layout": None}, ValueError, "NATURAL"),
                              ({"variant": "hyb"}, NotImplementedError, "3inst"),
                              ({"codebook": "e8p"}, NotImplementedError, "e8p"),
                              ({"quant_method": "gptq"}, ValueError, "glq")):
        q = dict(cfg["quantization_config"])
        q.update(patch)
        json.dump({"quantization_config": q}, open(cfgp, "w"))
        with pytest.raises(exc, match=match):
            C.load_quantized_linears(str(tmp_path), device="cpu")


@pytest.mark.gpu
def test_loaded_layers_forward_like_the_reference(tmp_path, golden):
    """Loaded modules reproduce the reference's forward outputs stored with the artifacts."""
    from tests.gpu_util import DEV, rel
    g = _trellis_dir(str(tmp_path), golden)
    lins = C.load_quantized_linears(str(tmp_path), device=DEV)
    for tag, name in (("k2", "model.layers.0.self_attn.q_proj"), ("k4", "model.layers.0.mlp.up_proj"),
                      ("k4k2", "model.layers.1.mlp.down_proj")):
        x = torch.from_numpy(g[f"{tag}_x"]).half().to(DEV)
        y = lins[name](x)
        assert rel(y, g[f"{tag}_y"]) < 1e-2, (tag, rel(y, g[f"{tag}_y"]))


def test_quantized_embedding_group_becomes_an_embedding_module(tmp_path, golden):
    """A checkpoint with a quantized embedding beside its linears (Qidxs (vocab, n/8), per-row
    Wscale, one-element SU) loads as E8RHTEmbedding instead of failing as a one-row linear; and
    the 3-bpw secondary table is the first 256 rows of the full table, which is why one table
    serves both stages."""
    from glq_amd.quantized_linear import E8RHTEmbedding
    from oracle import glq_oracle as O
    g = golden("e8_layer")
    rng = np.random.default_rng(0)
    vocab, dim = 50, 64
    tensors = {f"a.b.{leaf}": torch.from_numpy(np.asarray(g[f"bd4_{leaf}"]))
               for leaf in ("Qidxs", "Qidxs2", "SU", "SV", "Wscale", "inv_resid_scale")}
    tensors.update({
        "model.embed_tokens.Qidxs": torch.from_numpy(rng.integers(-32768, 32768, (vocab, dim // 8)).astype(np.int16)),
        "model.embed_tokens.SV": torch.ones(dim, dtype=torch.float16),
        "model.embed_tokens.SU": torch.ones(1, dtype=torch.float16),
        "model.embed_tokens.Wscale": torch.rand(vocab) + 0.5})
    _write(str(tmp_path), tensors, {"quant_method": "glq", "codebook": "e8_shell", "block_diagonal": True,
                                    "codesz": 8, "bpw": 4})
    mods = C.load_quantized_linears(str(tmp_path), device="cpu")
    emb = mods["model.embed_tokens"]
    assert isinstance(emb, E8RHTEmbedding) and (emb.num_embeddings, emb.embedding_dim, emb.n_pad) == (vocab, dim, dim)
    assert torch.equal(emb.Qidxs, tensors["model.embed_tokens.Qidxs"]) and emb.codebook is not None
    assert float(emb.inv_resid_scale.abs().sum()) == 0.0           # single stage: residual keys absent
    assert mods["a.b"].out_features == 96
    table = O.e8_table()
    norms = (table[:256] ** 2).sum(-1)
    assert np.all(norms[1:] >= norms[:-1]) and norms[255] <= 4.0    # the low-norm prefix, in table order
    # the embedding's scale factor is the host model's, not the checkpoint's: it is passed in
    assert emb.embed_scale == 1.0
    for arg, want in (({"model.embed_tokens": 8.0}, 8.0), (4.0, 4.0), ({"other": 3.0}, 1.0)):
        scaled = C.load_quantized_linears(str(tmp_path), device="cpu", embed_scales=arg)["model.embed_tokens"]
        assert scaled.embed_scale == want


def test_prepare_needs_the_gpu(tmp_path, golden):
    """The load-time step runs kernels: on CPU buffers it refuses instead of falling back."""
    _trellis_dir(str(tmp_path), golden)
    lins = C.load_quantized_linears(str(tmp_path), device="cpu")      # prepare is skipped for a CPU load
    with pytest.raises(RuntimeError, match="GPU"):
        next(iter(lins.values())).prepare()

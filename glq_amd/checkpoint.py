"""Loader for GLQ-quantized checkpoints as the reference writes them
(glq/quantize_model.py:2127-2236: safetensors shards + config.json `quantization_config` +
e8_codebook.pt; read side glq/hf_integration.py:403-421, 511-546).

Only what the quantized-linear forward needs: finds every quantized layer in the safetensors
files by its buffer names, builds an `E8RHTLinear` per layer and attaches the shared table.
The rest of the model (norms, embeddings, attention code) belongs to the host framework.
Files are read with safetensors / json / `torch.load(weights_only=True)` only.
"""
from __future__ import annotations

import glob
import json
import os

import numpy as np
import torch

from .quantized_linear import E8RHTEmbedding, E8RHTLinear

LAYER_BUFFERS = ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4", "trellis_packed", "trellis_packed2", "tlut",
                 "SU", "SV", "Wscale", "inv_resid_scale", "inv_resid_scale2", "inv_resid_scale3", "bias")


def read_quantization_config(model_dir: str) -> dict:
    """config.json -> quantization_config, with the reference's guards
    (glq/hf_integration.py:511-531)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f).get("quantization_config")
    if not cfg or cfg.get("quant_method") != "glq":
        raise ValueError("config.json has no glq quantization_config")
    cb = cfg.get("codebook", "e8_shell")
    if cb not in ("e8_shell", "trellis"):
        raise NotImplementedError(f"codebook {cb!r}: only the E8 shell and trellis codebooks are served")
    if cb == "trellis":
        if cfg.get("variant", "hyb") != "3inst":
            raise NotImplementedError("trellis variant %r: only 3inst is served" % cfg.get("variant", "hyb"))
        if cfg.get("trellis_layout") != "kernel":
            raise ValueError('This 3inst trellis checkpoint is stored in the pre-kernel NATURAL layout '
                             '(config.json lacks trellis_layout: "kernel") and cannot be decoded.')
    return cfg


def load_shell_table(model_dir: str | None = None) -> torch.Tensor:
    """(65536, 8) fp16 E8 table: the checkpoint's e8_codebook.pt, else the bundled copy."""
    if model_dir:
        path = os.path.join(model_dir, "e8_codebook.pt")
        if os.path.exists(path):
            data = torch.load(path, map_location="cpu", weights_only=True)
            return data["codebook"].to(torch.float16).contiguous()
    nib = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "data", "e8_shell_nibbles.npy"))
    # bundled words: code of coordinate i in nibble i, value = code / 2 - 3 (glq/codebook.py:102-115)
    codes = np.stack([(nib.astype(np.uint32) >> (4 * i)) & 15 for i in range(8)], -1)
    return torch.from_numpy(codes.astype(np.float32) * 0.5 - 3.0).to(torch.float16)


def _layer_groups(model_dir):
    """{layer prefix: {buffer name: (file, key)}} over all safetensors files."""
    from safetensors import safe_open
    groups = {}
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors files in {model_dir}")
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for key in f.keys():
                prefix, _, leaf = key.rpartition(".")
                if leaf in LAYER_BUFFERS:
                    groups.setdefault(prefix, {})[leaf] = (path, key)
    return {p: g for p, g in groups.items() if "Qidxs" in g or "trellis_packed" in g}


def load_quantized_linears(model_dir: str, device="cuda:0", shapes: dict | None = None, prepare: bool = True,
                           embed_scales: dict | float | None = None) -> dict:
    """{layer name: E8RHTLinear on `device`} for every quantized linear of the checkpoint; a
    quantized embedding (per-row `Wscale`, one-element `SU`) becomes an `E8RHTEmbedding`.

    Block-diagonal checkpoints store unpadded dims, so (out, in) = (len(SU), len(SV)); legacy
    power-of-two padded shell checkpoints need the true shapes in `shapes[name] = (out, in)`
    (the host model's layer shapes), otherwise the padded dims are used as they are.

    `prepare` runs every layer's load-time step (`E8RHTLinear.prepare()`: host copies of the
    scalars, packed tables, folded index streams) so that the first forward call, captured or
    not, finds everything in place.  `embed_scales` gives the factor a scaled embedding multiplies
    its rows by (sqrt(hidden) in Gemma-style models, glq/quantized_linear.py:1364-1370): one value
    for every embedding or `{layer name: value}`.  The factor is a property of the host model, not
    of the checkpoint -- it is not stored in the state dict -- so leaving it out loads such an
    embedding with outputs too small by that factor."""
    from safetensors import safe_open
    cfg = read_quantization_config(model_dir)
    trellis = cfg.get("codebook") == "trellis"
    table = None if trellis else load_shell_table(model_dir).to(device)
    out = {}
    handles = {}
    try:
        for name, group in sorted(_layer_groups(model_dir).items()):
            sd = {}
            for leaf, (path, key) in group.items():
                if path not in handles:
                    handles[path] = safe_open(path, framework="pt", device="cpu")
                sd[leaf] = handles[path].get_tensor(key)
            if "Qidxs" in sd and sd["Wscale"].dim() == 1 and sd["SU"].numel() == 1:
                # a quantized embedding (per-row scales, unit SU, glq/quantized_linear.py:1343-1452)
                vocab, n_pad = sd["Qidxs"].shape[0], sd["SV"].numel()
                dim = (shapes or {}).get(name, (vocab, n_pad))[1]
                if isinstance(embed_scales, dict):
                    scale = float(embed_scales.get(name, 1.0))
                else:
                    scale = 1.0 if embed_scales is None else float(embed_scales)
                emb = E8RHTEmbedding(vocab, dim, embed_scale=scale)
                if emb.n_pad != n_pad:
                    raise RuntimeError(f"{name}: embedding of width {dim} pads to {emb.n_pad}, the checkpoint "
                                       f"stores {n_pad} columns; pass its true width in shapes[name]")
                missing, unexpected = emb.load_state_dict(sd, strict=False)
                if unexpected:
                    raise RuntimeError(f"{name}: unexpected buffers {unexpected}")
                emb = emb.to(device)
                emb.set_codebook(table, table)
                out[name] = emb
                continue
            m_pad, n_pad = sd["SU"].numel(), sd["SV"].numel()
            o, i = (shapes or {}).get(name, (m_pad, n_pad))
            # legacy power-of-two padding is recognised by the module from the buffer shapes
            bd = trellis or bool(cfg.get("block_diagonal", True))
            lin = E8RHTLinear(i, o, bias="bias" in sd, block_diagonal=bd,
                              codebook_type="trellis" if trellis else "e8_shell")
            missing, unexpected = lin.load_state_dict(sd, strict=False)
            if unexpected:
                raise RuntimeError(f"{name}: unexpected buffers {unexpected}")
            lin = lin.to(device)
            if not trellis:
                # one table serves both stages, also at 3 bpw: the 256-entry secondary table of that
                # recipe is the first 256 rows of the full one (glq/codebook.py:348-368), and its
                # indices never exceed 255
                lin.set_codebook(table, table)
            if prepare and torch.device(device).type == "cuda":
                lin.prepare()
            out[name] = lin
    finally:
        handles.clear()
    return out

"""Merged q/k/v of a 2048-wide 4 bpw model through `MergedTrellisLinear.apply`, N tokens, 40 eager calls: the
program behind profiles/merged_linear_qkv_2048_4bpw.txt (GLQ_MERGED_GROUPED=0 in front of it gives the
reference's per-shard op sequence).  Not a test: pytest does not collect it."""
import sys

import torch

sys.path.insert(0, __file__.rsplit("/tests/", 1)[0])
from glq_amd import custom_ops, linear_method as LM   # noqa: E402


def main(tokens):
    custom_ops.register()
    dev, n = "cuda:0", 2048
    g = torch.Generator().manual_seed(0)
    layer = LM.MergedTrellisLinear(n, [2048, 512, 512], bpw=4)
    layer.trellis_packed = LM.GLQShards(torch.randint(-32768, 32768, ((r // 16) * (n // 16), 64), dtype=torch.int16,
                                                      generator=g) for r in (2048, 512, 512))
    layer.Wscale = LM.GLQShards(torch.tensor(0.02) for _ in range(3))
    layer.process_weights_after_loading(dev)
    x = torch.randn(tokens, n, generator=g).to(torch.bfloat16).to(dev)
    for _ in range(40):
        y = layer.apply(x)
    torch.cuda.synchronize()
    print(tuple(y.shape), float(y.float().abs().mean()))


if __name__ == "__main__":
    main(int(sys.argv[1]) if len(sys.argv) > 1 else 8)

"""The decoder `bench.py` times for configs[4] -- 36 layers of the SmolLM3-3B shape, 512-token prompt,
greedy decode -- checked through the properties that need no oracle: graph replay equals eager
decode token for token, two runs give the same tokens and logits bit for bit, and a prompt's last
logits equal those of a one-token step after the prompt without its last token (needs an MI355X;
the oracle covers two layers of this shape in tests/test_gpu_decoder_reference.py)."""
import pytest
import torch

from tests.gpu_util import DEV, rel, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dec():
    from glq_amd.decoder import DecoderConfig, TrellisDecoder
    say("decoder 36 layers: build")
    d = TrellisDecoder(DecoderConfig(), device=DEV, seed=0, max_len=1024)
    yield d
    del d
    torch.cuda.empty_cache()


def _prompt(n=512):
    return torch.randint(0, 128256, (n,), generator=torch.Generator().manual_seed(0)).to(DEV)


def test_full_depth_graph_replay_equals_eager_and_repeats(dec):
    say("decoder 36 layers: graph vs eager, 40 tokens after a 512-token prompt")
    ids = _prompt()
    eager, _, _ = dec.generate(ids, 40, use_graph=False)
    logits_eager = dec._step().clone()                        # the 41st step, eager
    graph, _, _ = dec.generate(ids, 40, use_graph=True)
    dec.graph.replay()
    logits_graph = dec._logits.clone()
    again, _, _ = dec.generate(ids, 40, use_graph=True)
    dec.graph.replay()
    assert torch.equal(eager, graph), (eager != graph).nonzero().flatten().tolist()
    assert torch.equal(graph, again)
    assert torch.equal(logits_eager, logits_graph) and torch.equal(logits_graph, dec._logits)
    assert int(dec.pos.item()) == 512 + 41
    # not a degenerate sequence: random weights still move the arg-max around
    assert graph.unique().numel() > 4


def test_full_depth_step_matches_prefill_of_longer_prompt(dec):
    """513 prompt tokens at once (tile kernels, library attention) against 512 at once plus one
    decode step (fused one-token kernels, cache read back): two routes through 36 layers and 252
    quantized linears.  The bf16 residual stream is rounded differently on the two routes (about
    four roundings of 2^-8 relative size per layer, adding up like a random walk: sqrt(144) * 3.9e-3 =
    4.7e-2 expected at 36 layers); measured 4.6e-2, gated at 8e-2 -- unrelated logits differ by 1.4."""
    say("decoder 36 layers: prefill(513) vs prefill(512) + step")
    ids = _prompt(513)
    full = dec.prefill(ids).clone()
    dec.prefill(ids[:512])
    dec.tok.copy_(ids[512:513])
    step = dec._step()
    err = rel(step, full)
    say("  relative difference of the logits", err)
    assert err < 8e-2, err
    assert int(dec.pos.item()) == 513
    # the routes agree on the next token wherever the margin between the two best logits exceeds
    # twice the largest logit difference
    top2 = full[0].topk(2).values
    if float(top2[0] - top2[1]) > 2 * float((step - full).abs().max()):
        assert int(step.argmax()) == int(full.argmax())
    # the gate means something: the logits of another position are nowhere near
    other = dec.prefill(ids[:300])
    assert rel(other, full) > 0.5

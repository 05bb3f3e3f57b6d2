"""Every forward path is capturable into a hipGraph (no allocation, no host synchronisation, the live-token
count read from device memory; crates/xabe-cuda/src/kernels/moe.rs:34-41, docs/TOOLCHAIN.md:107-142): a
captured pass, replayed several times with eager work and synchronisations between the replays, gives the
eager pass's bits every time."""
import numpy as np
import pytest

from util import activations, make_layer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _replays(torch, stream, capture, outputs, scramble, eager_bits, what, rows=None):
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        capture()                      # warm-up on the capture stream: everything one-time happens here
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            capture()
        for rep in range(4):
            scramble()                 # eager work between replays: the outputs are overwritten
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            for o, want in zip(outputs, eager_bits):
                assert torch.equal(o.view(torch.int32)[:rows], want[:rows]), f"{what}: replay {rep} differs from the eager pass"


@pytest.mark.parametrize("max_tokens,tokens", [(3, 3), (12, 9), (32, 32), (48, 41), (128, 100)])
def test_moe_block_forward_replays(oracle, X, max_tokens, tokens):
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    layer = make_layer(oracle, g, seed=8800 + max_tokens, router_q8=(max_tokens != 12),
                       down_quant=X.ExpertQuant.Q8_0 if max_tokens == 12 else None)
    blk = X.MoeBlock(g)
    x = activations(8801, max_tokens, 2048, tokens)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(layer.dev, x, tokens, ffn, lout)
    torch.cuda.synchronize()
    want = [ffn.view(torch.int32).clone(), lout.view(torch.int32).clone()]
    stream = torch.cuda.Stream()

    def scramble():
        ffn.fill_(float("nan"))
        lout.fill_(float("nan"))

    _replays(torch, stream, lambda: blk.forward(layer.dev, x, tokens, ffn, lout), [ffn, lout], scramble, want,
             f"block {max_tokens}/{tokens}", rows=tokens)   # rows past the live tokens are never written


def test_dense_block_and_lm_head_replay(oracle, X):
    import torch

    H, I = 5120, 17408
    q = X.ExpertQuant.Q6K
    w = X.DenseFfnLayerWeights(1.0 + X.synth_normal_f32(44, H, 0.1), X.QuantTensor(X.synth_quant(q, 41, H * I, 0.02), q),
                               X.QuantTensor(X.synth_quant(q, 42, H * I, 0.02), q), X.QuantTensor(X.synth_quant(q, 43, H * I, 0.02), q))
    blk = X.DenseFfnBlock(H, I, 2)
    x = X.synth_normal_f32(51, 2 * H, 1.0).view(2, H)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(w, x, 2, ffn, lout)
    torch.cuda.synchronize()
    want = [ffn.view(torch.int32).clone(), lout.view(torch.int32).clone()]
    stream = torch.cuda.Stream()
    _replays(torch, stream, lambda: blk.forward(w, x, 2, ffn, lout), [ffn, lout],
             lambda: (ffn.zero_(), lout.zero_()), want, "dense block")

    # eight tokens: gate/up takes four tokens per pass with the activation rows in LDS (a launch that asks for
    # more than the static LDS limit; the limit is raised when the block is created, not on the launch path)
    blk8 = X.DenseFfnBlock(H, I, 8)
    x8 = X.synth_normal_f32(52, 8 * H, 1.0).view(8, H)
    ffn8, lout8 = torch.zeros_like(x8), torch.zeros_like(x8)
    blk8.forward(w, x8, 7, ffn8, lout8)
    torch.cuda.synchronize()
    want8 = [ffn8.view(torch.int32).clone(), lout8.view(torch.int32).clone()]
    _replays(torch, stream, lambda: blk8.forward(w, x8, 7, ffn8, lout8), [ffn8, lout8],
             lambda: (ffn8.fill_(float("nan")), lout8.fill_(float("nan"))), want8, "dense block, 7 of 8 tokens", rows=7)

    g = X.LmHeadGeometry(2048, 8192, 3)
    k = X.LmHeadKernels(g)
    head = X.HeadTensor.q8_0(X.synth_quant(X.ExpertQuant.Q8_0, 61, g.elements(), 0.02))
    hs = X.synth_normal_f32(62, 3 * 2048, 1.0).view(3, 2048)
    logits = torch.zeros(3, g.vocab, device="cuda")
    pv, pi = torch.zeros(512, device="cuda"), torch.zeros(512, dtype=torch.int32, device="cuda")
    out = torch.zeros(1, dtype=torch.int32, device="cuda")

    def head_pass():
        k.forward(head, hs, 3, logits)
        k.argmax(logits[2], g.vocab, pv, pi, out)

    head_pass()
    torch.cuda.synchronize()
    want = [logits.view(torch.int32).clone(), out.clone()]
    _replays(torch, stream, head_pass, [logits, out], lambda: (logits.fill_(-1.0), out.fill_(-5)), want, "LM head + argmax")


def test_token_count_change_inside_a_capture_is_refused(oracle, X):
    """set_valid_tokens is a host-to-device copy: recorded into a graph it would publish, on every replay, whatever
    its source held then.  The count is published before the capture (kernels/moe.rs:5473-5491); a forward whose
    count differs from the published one while the stream is capturing is refused and records nothing, and the
    same forward outside the capture still works."""
    import torch

    g = X.MoeGeometry.qwen3_6(32, 4)
    layer = make_layer(oracle, g, seed=8900)
    blk = X.MoeBlock(g)
    x = activations(8901, 4, 2048, 4)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        blk.forward(layer.dev, x, 4, ffn, lout)       # publishes 4
        stream.synchronize()
        want = lout.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            with pytest.raises(X.moe.InvalidArgument, match="publish the count before the capture begins"):
                blk.forward(layer.dev, x, 2, ffn, lout)
            blk.forward(layer.dev, x, 4, ffn, lout)   # unchanged count: nothing to copy, captured normally
        lout.fill_(float("nan"))
        graph.replay()
        stream.synchronize()
        assert torch.equal(lout.view(torch.int32), want.view(torch.int32))
        # outside the capture the refused width is served, and the cache was not poisoned by the refusal
        lout.zero_()
        blk.forward(layer.dev, x, 2, ffn, lout)
        stream.synchronize()
        assert torch.equal(lout[:2].view(torch.int32), want[:2].view(torch.int32)) and not bool(lout[2:].any())

"""xabe_moe_block_forward_noalloc (no counterpart in the reference: for callers that cannot allocate device
memory) against xabe_moe_block_forward, through the C ABI: same bits, on two calls in a row, the second with a
smaller input; and the size limit is an error, not a fault."""
import pytest

from util import activations, make_layer, run_block

pytestmark = pytest.mark.gpu


def _both(X, oracle, max_tokens, tokens, seed, bias=False, geometry=None, **layer_kw):
    import torch

    g = geometry or X.MoeGeometry.qwen3_6(32, max_tokens)
    layer = make_layer(oracle, g, seed=seed, **layer_kw)
    x = activations(seed + 1, max_tokens, g.hidden, tokens)
    lb = X.synth_normal_f32(seed + 2, g.num_experts, 1.0) if bias else None
    want_ffn, want_l = run_block(X.MoeBlock(g), layer, x, tokens, logit_bias=lb)
    # poisoned outputs: rows past the live tokens must stay untouched, live rows must be overwritten
    ffn = torch.full_like(x, float("nan"))
    lout = torch.full_like(x, float("nan"))
    X.moe_block_forward_noalloc(g, layer.dev, x, tokens, ffn, lout, logit_bias=lb)
    torch.cuda.synchronize()
    assert want_l[:tokens].abs().max() > 0
    assert torch.equal(ffn[:tokens].view(torch.int32), want_ffn[:tokens].view(torch.int32)), (max_tokens, tokens)
    assert torch.equal(lout[:tokens].view(torch.int32), want_l[:tokens].view(torch.int32)), (max_tokens, tokens)
    assert bool(torch.isnan(ffn[tokens:]).all()) and bool(torch.isnan(lout[tokens:]).all())


def test_noalloc_block_equals_the_allocating_block_on_consecutive_calls(oracle):
    import llmxabe_amd as X

    _both(X, oracle, 32, 32, 9500)             # the largest pass the scratch array serves
    _both(X, oracle, 3, 3, 9510, bias=True)    # then a smaller one over the same array (stale contents around it)
    _both(X, oracle, 8, 5, 9520)               # fewer live tokens than the pass holds
    _both(X, oracle, 32, 1, 9530)


def test_noalloc_block_on_the_small_shape_with_512_experts_and_other_formats(oracle):
    """The other shape the three launches serve (hidden 512 / intermediate 256), 512 experts, an f32 router and
    Q8_0 stacks: the same offsets into the array, different strides inside them."""
    import llmxabe_amd as X

    small = lambda t: X.MoeGeometry(512, 8, 512, 256, 32, t)
    _both(X, oracle, 6, 6, 9560, geometry=small(6), expert_quant=X.ExpertQuant.Q8_0, router_q8=False)
    _both(X, oracle, 32, 20, 9570, geometry=small(32), bias=True)
    _both(X, oracle, 3, 3, 9580, down_quant=X.ExpertQuant.Q8_0, router_q8=False)   # the shipped layers' pairing


def test_noalloc_block_allocates_no_device_memory(oracle):
    """What the entry point is for: after a first call on the device, further calls leave the device's free memory
    where it was (hipMemGetInfo through torch; torch's own caching allocator is not involved in the calls)."""
    import torch
    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(32, 8)
    layer = make_layer(oracle, g, seed=9590)
    x = activations(9591, 8, 2048)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    X.moe_block_forward_noalloc(g, layer.dev, x, 8, ffn, lout)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for tokens in (8, 3, 8, 1, 5):
        X.moe_block_forward_noalloc(g, layer.dev, x, tokens, ffn, lout)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_reserved() == reserved0


_FIRST_CALL_UNDER_CAPTURE = r"""
import sys
sys.path.insert(0, {root!r}); sys.path.insert(0, {root!r} + "/tests")
import torch
import llmxabe_amd as X, oracle
from util import activations, make_layer
g = X.MoeGeometry.qwen3_6(32, 2)
layer = make_layer(oracle, g, seed=9600)
x = activations(9601, 2, 2048)
ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
stream = torch.cuda.Stream()
refused = False
with torch.cuda.stream(stream):
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        try:
            X.moe_block_forward_noalloc(g, layer.dev, x, 2, ffn, lout)
        except X.moe.InvalidArgument as e:
            refused = "capturing" in str(e)
    stream.synchronize()
    X.moe_block_forward_noalloc(g, layer.dev, x, 2, ffn, lout)      # outside the capture: served
    stream.synchronize()
assert refused and bool(lout.abs().max() > 0)
print("REFUSED-THEN-SERVED")
"""


def test_noalloc_first_call_on_a_device_is_refused_under_capture():
    """The first call on a device resolves the array's address, which must not happen while the stream captures: a
    fresh process whose first call arrives under capture gets an error and records nothing; the next call is served."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE.format(root=root)], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0 and "REFUSED-THEN-SERVED" in out.stdout, out.stdout[-2000:] + out.stderr[-2000:]


def test_noalloc_block_inside_a_graph(oracle):
    import torch
    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(32, 4)
    layer = make_layer(oracle, g, seed=9540)
    x = activations(9541, 4, 2048, 3)
    want_ffn, want_l = run_block(X.MoeBlock(g), layer, x, 3)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        X.moe_block_forward_noalloc(g, layer.dev, x, 3, ffn, lout)      # first call on the device: outside the capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            X.moe_block_forward_noalloc(g, layer.dev, x, 3, ffn, lout)
        for rep in range(3):
            lout.fill_(float("nan"))
            X.moe_block_forward_noalloc(g, layer.dev, x, 1, ffn, torch.zeros_like(x))   # eager work in between: count 1
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            assert torch.equal(lout[:3].view(torch.int32), want_l[:3].view(torch.int32)), rep


def test_noalloc_block_rejects_what_its_array_cannot_hold(oracle):
    import torch
    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(32, 4)
    layer = make_layer(oracle, g, seed=9550)
    big = X.MoeGeometry.qwen3_6(32, 33)
    x = torch.zeros(33, 2048, device="cuda")
    with pytest.raises(X.moe.UnsupportedGeometry, match="serves at most 32 tokens"):
        X.moe_block_forward_noalloc(big, layer.dev, x, 33, torch.zeros_like(x), torch.zeros_like(x))
    x4 = torch.zeros(4, 2048, device="cuda")
    with pytest.raises(X.moe.TooManyTokens):
        X.moe_block_forward_noalloc(g, layer.dev, x4, 5, torch.zeros_like(x4), torch.zeros_like(x4))
    with pytest.raises(X.moe.BufferLength):
        X.moe_block_forward_noalloc(g, layer.dev, x4[:3], 3, torch.zeros_like(x4), torch.zeros_like(x4))

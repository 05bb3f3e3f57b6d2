"""The post-mixer seam between consecutive layers (the reference's seam-fusion row, docs/BENCHMARKS.md:1376 and
:1761: "the next layer's RMSNorm in the MoE combine kernel's tail ... the mixer skips its norm launch").

A two-layer chain through the fused seam (layer 0's last launch writes layer 1's normalised rows; layer 1 starts from
them and launches no RMSNorm) must be the unfused chain bit for bit, at every width regime, and the chain's output
must match the CPU oracle run layer by layer."""
import numpy as np
import pytest

from util import activations, make_layer, rel_to_peak

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _bits(t):
    import torch

    return t.contiguous().view(torch.int32)


def _chain(X, layers, x, tokens, max_tokens, fused, one_handle=False, decode_fused=True, lean=False):
    """Two blocks in a row.  fused: through the seam; one_handle: the same block handle serves both layers (its own
    normed buffer is the seam's target); lean: no ffn_out, no routed read-back on the first layer."""
    import torch

    g = layers[0].geometry
    blk0 = X.MoeBlock(g)
    blk1 = blk0 if one_handle else X.MoeBlock(g)
    for b in {blk0, blk1}:
        b.set_fused_decode(decode_fused)
    ffn0, l0, ffn1, l1 = (torch.zeros_like(x) for _ in range(4))
    if fused:
        blk0.forward_seam(layers[0].dev, x, tokens, None if lean else ffn0, l0, next_norm_weight=layers[1].dev.post_norm,
                          next_block=None if one_handle else blk1, skip_readback=lean)
        blk1.forward_seam(layers[1].dev, l0, tokens, ffn1, l1, input_normed=True)
    else:
        blk0.forward(layers[0].dev, x, tokens, ffn0, l0)
        blk1.forward(layers[1].dev, l0, tokens, ffn1, l1)
    torch.cuda.synchronize()
    return dict(ffn0=ffn0, l0=l0, ffn1=ffn1, l1=l1, normed1=blk1.normed().view(max_tokens, -1),
                logits1=blk1.router_logits().view(max_tokens, -1), ids1=blk1.buffers().topk_ids().view(max_tokens, -1),
                gate1=blk1.shared_gate(), routed1=blk1.routed().view(max_tokens, -1))


def _two_layers(X, oracle, max_tokens, small=False, **kw):
    g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens) if small else X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    return [make_layer(oracle, g, seed=8100 + 50 * i, **kw) for i in range(2)]


# (max_tokens, live tokens, three-launch decode on): every regime the block has
WIDTHS = [(1, 1, True), (3, 3, True), (8, 5, True), (32, 32, True), (3, 3, False), (12, 9, False), (48, 40, True), (200, 170, True),
          (512, 512, True)]


@pytest.mark.parametrize("max_tokens,tokens,decode_fused", WIDTHS)
def test_two_layer_chain_through_the_seam_is_the_unfused_chain(oracle, X, max_tokens, tokens, decode_fused):
    layers = _two_layers(X, oracle, max_tokens)
    x = activations(8200 + max_tokens, max_tokens, 2048, tokens)
    plain = _chain(X, layers, x, tokens, max_tokens, fused=False, decode_fused=decode_fused)
    assert float(plain["l1"][:tokens].abs().max()) > 0
    for one_handle in (False, True):
        seam = _chain(X, layers, x, tokens, max_tokens, fused=True, one_handle=one_handle, decode_fused=decode_fused)
        for name in ("ffn0", "l0", "ffn1", "l1", "normed1", "logits1", "ids1", "routed1"):
            assert bool((_bits(seam[name][:tokens]) == _bits(plain[name][:tokens])).all()), (name, one_handle)
        assert bool((_bits(seam["gate1"][:tokens]) == _bits(plain["gate1"][:tokens])).all())
        assert not bool(seam["l1"][tokens:].any()) and not bool(seam["l0"][tokens:].any())   # rows past the live count untouched
    lean = _chain(X, layers, x, tokens, max_tokens, fused=True, decode_fused=decode_fused, lean=True)
    assert bool((_bits(lean["l1"][:tokens]) == _bits(plain["l1"][:tokens])).all())
    assert not bool(lean["ffn0"].any())                                                       # no ffn_out was asked for


@pytest.mark.parametrize("max_tokens,tokens", [(3, 3), (32, 20), (96, 96)])
def test_chain_through_the_seam_matches_the_oracle_layer_by_layer(oracle, X, max_tokens, tokens):
    """The oracle's two blocks in a row (each routed from the device's own logits, as the reference's block test
    does) against the fused chain: ids exact, l_out within the regime's tolerance."""
    layers = _two_layers(X, oracle, max_tokens)
    x = activations(8300 + max_tokens, max_tokens, 2048, tokens)
    seam = _chain(X, layers, x, tokens, max_tokens, fused=True)
    tol = 2e-5 if max_tokens < 64 else 1e-3
    xs = x.cpu().numpy()[:tokens]
    # layer 0 on the host, from the chain's input
    g = layers[0].geometry
    blk = X.MoeBlock(g)
    import torch
    f, l = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(layers[0].dev, x, tokens, f, l)
    torch.cuda.synchronize()
    ref0 = oracle.moe_block_forward(layers[0].host, xs, logits_override=blk.router_logits().cpu().numpy().reshape(max_tokens, -1)[:tokens],
                                    threads=8)
    assert rel_to_peak(seam["l0"].cpu().numpy()[:tokens], ref0.l_out) <= tol
    # layer 1 on the host, from the device's l_out of layer 0 (teacher-forced, so the check does not compound)
    l0 = seam["l0"].cpu().numpy()[:tokens]
    ref1 = oracle.moe_block_forward(layers[1].host, l0, logits_override=seam["logits1"].cpu().numpy()[:tokens], threads=8)
    assert np.array_equal(seam["ids1"].cpu().numpy()[:tokens], ref1.topk_ids.astype(np.int32))
    assert rel_to_peak(seam["normed1"].cpu().numpy()[:tokens], ref1.normed) <= 2e-6      # the tail's RMSNorm against rms_norm
    assert rel_to_peak(seam["l1"].cpu().numpy()[:tokens], ref1.l_out) <= tol


def test_seam_on_the_small_shape_and_other_formats(oracle, X):
    """hidden 512 / intermediate 256 (rows shorter than the canonical fold's 2048-element chunk) and Q8_0 stacks."""
    for max_tokens, tokens in ((4, 3), (32, 32), (96, 80)):
        layers = _two_layers(X, oracle, max_tokens, small=True, expert_quant=X.ExpertQuant.Q8_0, router_q8=False)
        x = activations(8400 + max_tokens, max_tokens, 512, tokens)
        plain = _chain(X, layers, x, tokens, max_tokens, fused=False)
        seam = _chain(X, layers, x, tokens, max_tokens, fused=True)
        for name in ("l0", "l1", "normed1", "ids1"):
            assert bool((_bits(seam[name][:tokens]) == _bits(plain[name][:tokens])).all()), (name, max_tokens)


def test_seam_chain_repeats_and_replays_in_a_graph(oracle, X):
    """The decode tail's arrival counters return to zero after every pass: the same chain again, with a different
    live count in between, and as a replayed graph, gives the same bits."""
    import torch

    layers = _two_layers(X, oracle, 8)
    g = layers[0].geometry
    x = activations(8500, 8, 2048)
    want = _chain(X, layers, x, 8, 8, fused=False)["l1"]
    blk = X.MoeBlock(g)
    l0, l1, f = (torch.zeros_like(x) for _ in range(3))
    stream = torch.cuda.Stream()

    def chain(tokens):
        blk.forward_seam(layers[0].dev, x, tokens, f, l0, next_norm_weight=layers[1].dev.post_norm)
        blk.forward_seam(layers[1].dev, l0, tokens, f, l1, input_normed=True)

    with torch.cuda.stream(stream):
        for tokens in (8, 3, 8):
            l1.zero_()
            chain(tokens)
            stream.synchronize()
            assert bool((_bits(l1[:tokens]) == _bits(want[:tokens])).all()), tokens
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            chain(8)
        for rep in range(3):
            l1.zero_()
            graph.replay()
            stream.synchronize()
            assert bool((_bits(l1) == _bits(want)).all()), rep
            chain(8)                                   # eager work between the replays
            stream.synchronize()

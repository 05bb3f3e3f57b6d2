"""The decode-width block (max_tokens <= 32) regrouped into three launches against the same block with one
launch per step (flat per-pair kernels up to 4 tokens, the dispatch-table regime above): every observable
tensor bit for bit, over repeated calls, with fewer live tokens than
the buffer holds, with and without a logit bias, and for each format pairing.  The per-step launches are
the ones the oracle comparisons of test_gpu_decode.py cover; test_block_matches_oracle runs the regrouped
block against the oracle directly."""
import numpy as np
import pytest

from util import activations, make_layer, run_block

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _observe(blk, g, ffn, lout, tokens):
    t, k = tokens, g.experts_per_token
    b = blk.buffers()
    return dict(
        ffn=ffn[:t].cpu().numpy(), l_out=lout[:t].cpu().numpy(),
        normed=blk.normed().view(g.max_tokens, g.hidden)[:t].cpu().numpy(),
        logits=blk.router_logits().view(g.max_tokens, g.num_experts)[:t].cpu().numpy(),
        routed=blk.routed().view(g.max_tokens, g.hidden)[:t].cpu().numpy(),
        shexp=blk.shared_ungated().view(g.max_tokens, g.hidden)[:t].cpu().numpy(),
        gate=blk.shared_gate().view(-1)[:t].cpu().numpy(),
        ids=b.topk_ids().view(g.max_tokens, k)[:t].cpu().numpy(),
        weights=b.topk_weights().view(g.max_tokens, k)[:t].cpu().numpy())


def _same_bits(a, b, what):
    for key in a:
        x, y = a[key], b[key]
        if x.dtype == np.float32:
            x, y = x.view(np.uint32), y.view(np.uint32)
        assert np.array_equal(x, y), f"{what}: {key} differs"


def _compare(X, oracle, g, tokens_seq, seed, router_q8=True, bias=False, expert_quant=None, shared_quant=None,
             down_quant=None, shared_down_quant=None):
    import torch

    layer = make_layer(oracle, g, seed=seed, router_q8=router_q8, expert_quant=expert_quant, shared_quant=shared_quant,
                       down_quant=down_quant, shared_down_quant=shared_down_quant)
    one, many = X.MoeBlock(g), X.MoeBlock(g)
    many.set_fused_decode(False)
    lb = X.synth_normal_f32(seed + 77, g.num_experts, 1.0) if bias else None
    for i, tokens in enumerate(tokens_seq):
        x = activations(seed + 10 + i, g.max_tokens, g.hidden, tokens)
        f1, l1 = run_block(one, layer, x, tokens, logit_bias=lb)
        f2, l2 = run_block(many, layer, x, tokens, logit_bias=lb)
        _same_bits(_observe(one, g, f1, l1, tokens), _observe(many, g, f2, l2, tokens), f"call {i} tokens {tokens}")


@pytest.mark.parametrize("max_tokens,tokens_seq", [(1, (1, 1)), (2, (2, 1, 2)), (3, (3, 1, 2, 3)), (4, (4, 3, 0, 4, 1)),
                                                   (5, (5, 2, 5)), (8, (8, 1, 7)), (16, (16, 9, 0, 16)),
                                                   (27, (27, 19)), (32, (32, 1, 32))])
@pytest.mark.parametrize("router_q8", [True, False])
def test_small_geometry(oracle, X, max_tokens, tokens_seq, router_q8):
    g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens)
    _compare(X, oracle, g, tokens_seq, seed=4100 + max_tokens, router_q8=router_q8, bias=router_q8)


@pytest.mark.parametrize("eq,sq", [("Q6K", "Q6K"), ("Q8_0", "Q8_0"), ("Q8_0", "Q6K")])
def test_small_geometry_format_pairings(oracle, X, eq, sq):
    g = X.MoeGeometry(16, 4, 512, 256, 32, 3)
    _compare(X, oracle, g, (3, 2), seed=4200, expert_quant=getattr(X.ExpertQuant, eq), shared_quant=getattr(X.ExpertQuant, sq))


@pytest.mark.parametrize("eq,dq,sq,sdq", [("Q6K", "Q8_0", "Q8_0", "Q8_0"), ("Q8_0", "Q6K", "Q6K", "Q8_0"),
                                         ("Q6K", "Q8_0", "Q8_0", "Q6K")])
def test_small_geometry_mixed_formats(oracle, X, eq, dq, sq, sdq):
    # down projections in another format than gate/up, as in the shipped layers (gate/up Q6_K, down Q8_0)
    q = lambda n: getattr(X.ExpertQuant, n)
    g = X.MoeGeometry(16, 4, 512, 256, 32, 3)
    _compare(X, oracle, g, (3, 1), seed=4250, expert_quant=q(eq), shared_quant=q(sq), down_quant=q(dq), shared_down_quant=q(sdq))


def test_model_geometry_shipped_layout(oracle, X):
    # gate/up Q6_K, down Q8_0, shared expert Q8_0, f32 router
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(3), 3)
    _compare(X, oracle, g, (3, 2), seed=4350, router_q8=False, down_quant=X.ExpertQuant.Q8_0)
    # and the three launches really serve it: the single-launch hook refuses layouts they do not cover
    layer = make_layer(oracle, g, seed=4350, router_q8=False, down_quant=X.ExpertQuant.Q8_0)
    blk = X.MoeBlock(g)
    x = activations(4360, 3, 2048, 3)
    f, l = run_block(blk, layer, x, 3)
    blk.forward_stage(layer.dev, x, f, l, 2)


@pytest.mark.parametrize("max_tokens,tokens_seq", [(1, (1, 1)), (3, (3, 3, 2)), (4, (4, 1, 4)), (7, (7, 5)), (16, (16, 11)),
                                                   (24, (24, 17)), (32, (32, 29))])
def test_model_geometry(oracle, X, max_tokens, tokens_seq):
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    _compare(X, oracle, g, tokens_seq, seed=4300 + max_tokens, bias=(max_tokens == 3))


def test_model_geometry_f32_router(oracle, X):
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(3), 3)
    _compare(X, oracle, g, (3, 2), seed=4400, router_q8=False)


def test_candidate_expert_replaced_after_verification(oracle, X):
    """Launch B starts streaming the expert ranked k-th by LOGIT and re-streams when the probabilities rank
    another one there.  A zero router with a crafted bias gives logits = bias exactly: two experts one ulp
    apart whose probabilities tie, the larger logit at the higher index, inside the top 8 and across ranks
    8 / 9, so the pairs k = 1, 2 and 7 of every token change expert after the softmax."""
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(3), 3)
    layer = make_layer(oracle, g, seed=4600, router_q8=False)
    layer.dev.router.zero_()
    bias = np.random.default_rng(5).uniform(-8.0, -1.0, 256).astype(np.float32)
    bias[50] = 5.0
    bias[10], bias[200] = 0.001, np.nextafter(np.float32(0.001), np.float32(1))
    bias[120:124] = (-0.1, -0.2, -0.3, -0.4)
    bias[30], bias[220] = -0.5, np.nextafter(np.float32(-0.5), np.float32(0))
    lb = torch.from_numpy(bias).cuda()
    one, many = X.MoeBlock(g), X.MoeBlock(g)
    many.set_fused_decode(False)
    x = activations(4610, 3, 2048)
    f1, l1 = run_block(one, layer, x, 3, logit_bias=lb)
    f2, l2 = run_block(many, layer, x, 3, logit_bias=lb)
    a, b = _observe(one, g, f1, l1, 3), _observe(many, g, f2, l2, 3)
    ref_ids, _ = oracle.route_batch(np.tile(bias, (3, 1)), 8)
    assert list(ref_ids[0]) == [50, 10, 200, 120, 121, 122, 123, 30]
    assert np.array_equal(a["logits"], np.tile(bias, (3, 1)))
    assert np.array_equal(a["ids"], ref_ids.astype(np.int32))
    _same_bits(a, b, "near-tie routing")


def test_many_replays_keep_the_bits(oracle, X):
    # 200 back-to-back passes on one stream, no host work between
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(3), 3)
    layer = make_layer(oracle, g, seed=4500)
    blk = X.MoeBlock(g)
    x = activations(4511, 3, 2048)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(layer.dev, x, 3, ffn, lout)
    torch.cuda.synchronize()
    first = lout.clone()
    for _ in range(200):
        blk.forward(layer.dev, x, 3, ffn, lout)
    torch.cuda.synchronize()
    assert torch.equal(first.view(torch.int32), lout.view(torch.int32))

"""`FfnBlock` (crates/xabe-engine/src/block/ffn.rs:27-228): the two-variant dispatch over the MoE block and
the dense sibling.  Each variant must give the bits of the block it wraps, and a block handed the other
kind's weights must answer FfnKindMismatch before anything is launched."""
import numpy as np
import pytest

from util import activations, make_layer, run_block

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _dense_weights(X, H, I, seed):
    q = X.ExpertQuant.Q6K
    pn = 1.0 + X.synth_normal_f32(seed, H, 0.1)
    t = lambda s: X.QuantTensor(X.synth_quant(q, seed + s, H * I, 0.02), q)
    return X.DenseFfnLayerWeights(pn, t(1), t(2), t(3))


@pytest.mark.parametrize("max_tokens,tokens", [(3, 3), (40, 33), (96, 96)])
def test_moe_variant_equals_moe_block(oracle, X, max_tokens, tokens):
    import torch

    cfg = X.FfnConfig.qwen3_6_35b_a3b()
    g = X.FfnBlock.geometry_for(cfg, X.moe_block_size(max_tokens), max_tokens)
    assert (g.num_experts, g.experts_per_token, g.hidden, g.intermediate) == (256, 8, 2048, 512)
    layer = make_layer(oracle, g, seed=9100 + max_tokens)
    x = activations(9101, max_tokens, 2048, tokens)
    want_ffn, want_l = run_block(X.MoeBlock(g), layer, x, tokens)
    blk = X.FfnBlock(cfg, g)
    assert blk.kind() == X.FfnKind.MOE and blk.tensor_cores_enabled()
    assert blk.geometry() == g
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.publish_tokens(tokens)
    blk.forward(X.FfnLayerWeights(layer.dev), x, tokens, ffn, lout)
    torch.cuda.synchronize()
    assert torch.equal(ffn.view(torch.int32), want_ffn.view(torch.int32))
    assert torch.equal(lout.view(torch.int32), want_l.view(torch.int32))
    moe = blk.as_moe()
    assert moe is not None
    ids = moe.buffers().topk_ids().cpu().numpy().reshape(max_tokens, 8)[:tokens]
    ref_ids, _ = oracle.route_batch(moe.router_logits().cpu().numpy().reshape(max_tokens, 256)[:tokens], 8)
    assert np.array_equal(ids, ref_ids.astype(np.int32))
    assert torch.equal(blk.normed().view(torch.int32), moe.normed().view(torch.int32))


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (8, 5)])
def test_dense_variant_equals_dense_block(X, max_tokens, tokens):
    import torch

    H, I = 1024, 4352                       # rows longer than one 2048-element step on the down side
    cfg = X.FfnConfig(X.FfnKind.DENSE, H, dense_intermediate=I)
    g = X.FfnBlock.geometry_for(cfg, X.moe_block_size(max_tokens), max_tokens)
    assert (g.num_experts, g.experts_per_token, g.hidden, g.intermediate) == (1, 1, H, I)
    w = _dense_weights(X, H, I, 9200)
    x = activations(9201, max_tokens, H, tokens)
    ref = X.DenseFfnBlock(H, I, max_tokens)
    want_ffn, want_l = torch.zeros_like(x), torch.zeros_like(x)
    ref.forward(w, x, tokens, want_ffn, want_l)
    blk = X.FfnBlock(cfg, g)
    assert blk.kind() == X.FfnKind.DENSE and blk.as_moe() is None
    blk.set_exact_decode_regime(True)       # a no-op on the dense block (ffn.rs:146-153)
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(X.FfnLayerWeights(w), x, tokens, ffn, lout)
    torch.cuda.synchronize()
    assert want_ffn[:tokens].abs().max() > 0
    assert torch.equal(ffn.view(torch.int32), want_ffn.view(torch.int32))
    assert torch.equal(lout.view(torch.int32), want_l.view(torch.int32))
    assert torch.equal(blk.normed().view(torch.int32), ref.normed().view(torch.int32))


def test_kind_mismatch_is_an_error_and_launches_nothing(oracle, X):
    import torch

    g = X.MoeGeometry.qwen3_6(32, 2)
    layer = make_layer(oracle, g, seed=9300)
    dense_w = _dense_weights(X, 1024, 4352, 9301)
    x = activations(9302, 2, 2048, 2)
    ffn = torch.full_like(x, 7.0)
    lout = torch.full_like(x, 7.0)
    moe_blk = X.FfnBlock(X.FfnConfig.qwen3_6_35b_a3b(), g)
    with pytest.raises(X.moe.FfnKindMismatch, match="a `moe` feed-forward block was handed `dense` weights"):
        moe_blk.forward(X.FfnLayerWeights(dense_w), x, 2, ffn, lout)
    cfg = X.FfnConfig(X.FfnKind.DENSE, 1024, dense_intermediate=4352)
    dense_blk = X.FfnBlock(cfg, X.FfnBlock.geometry_for(cfg, 32, 2))
    xd = activations(9303, 2, 1024, 2)
    with pytest.raises(X.moe.FfnKindMismatch, match="a `dense` feed-forward block was handed `moe` weights"):
        dense_blk.forward(X.FfnLayerWeights(layer.dev), xd, 2, torch.zeros_like(xd), torch.zeros_like(xd))
    torch.cuda.synchronize()
    assert bool((ffn == 7.0).all()) and bool((lout == 7.0).all())

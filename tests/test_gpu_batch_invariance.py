"""The batch-invariance contract: a token's output is bit-identical whether it is decoded alone or in a
batch (crates/xabe-engine/tests/batch_decode.rs:11-41, tests/moe_differential.rs:1096-1220).  Needs no
oracle: run the token alone (max_tokens = 1) and inside wider passes, compare bits."""
import numpy as np
import pytest

from util import activations, make_layer, run_block

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def setup(oracle):
    import llmxabe_amd as X

    g32 = X.MoeGeometry.qwen3_6(32, 32)
    layer = make_layer(oracle, g32, seed=900)
    return X, layer


def _block_rows(X, layer, x_rows, max_tokens, exact=False):
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    blk = X.MoeBlock(g)
    if exact:
        blk.set_exact_decode_regime(True)
    t = x_rows.shape[0]
    x = torch.zeros(max_tokens, 2048, device="cuda")
    x[:t] = x_rows
    ffn, lout = run_block(blk, layer, x, t)
    return (lout[:t].cpu().numpy(), blk.router_logits().view(max_tokens, 256)[:t].cpu().numpy(),
            blk.buffers().topk_ids().view(max_tokens, 8)[:t].cpu().numpy())


def test_batched_rows_equal_single_stream_bits(setup):
    X, layer = setup
    xs = activations(21, 32, 2048)
    batch32, logits32, ids32 = _block_rows(X, layer, xs, 32)
    for width in (3, 4, 8):                      # flat regime, flat boundary, dispatch-table regime
        rows, logits, ids = _block_rows(X, layer, xs[:width], width)
        assert np.array_equal(rows.view(np.uint32), batch32[:width].view(np.uint32)), width
        assert np.array_equal(logits.view(np.uint32), logits32[:width].view(np.uint32))
        assert np.array_equal(ids, ids32[:width])
    for t in (0, 1, 7, 19, 31):                  # each token alone, through the one-token geometry
        row, logits, ids = _block_rows(X, layer, xs[t:t + 1], 1)
        assert np.array_equal(row[0].view(np.uint32), batch32[t].view(np.uint32)), t
        assert np.array_equal(ids[0], ids32[t])


def test_identical_tokens_in_one_batch_give_identical_rows(setup):
    # batch_decode.rs:333: identical prompts in one batch => bit-identical rows (also the all-collide case)
    X, layer = setup
    xs = activations(22, 32, 2048, coherent=True)
    rows, _, ids = _block_rows(X, layer, xs, 32)
    assert np.all(rows.view(np.uint32) == rows[0].view(np.uint32))
    assert np.all(ids == ids[0])


def test_position_in_batch_does_not_matter(setup):
    X, layer = setup
    xs = activations(23, 32, 2048)
    a, _, _ = _block_rows(X, layer, xs, 32)
    perm = np.random.default_rng(0).permutation(32)
    import torch

    b, _, _ = _block_rows(X, layer, xs[torch.from_numpy(perm).cuda()], 32)
    assert np.array_equal(b.view(np.uint32), a[perm].view(np.uint32))


def test_exact_decode_regime_at_prefill_width_equals_decode(setup):
    # kernels/moe.rs:5436-5452, tests/moe_differential.rs:1401-: a verify window's rows equal plain decode
    X, layer = setup
    xs = activations(24, 12, 2048)
    wide, _, _ = _block_rows(X, layer, xs, 80, exact=True)
    for t in (0, 5, 11):
        row, _, _ = _block_rows(X, layer, xs[t:t + 1], 1)
        assert np.array_equal(row[0].view(np.uint32), wide[t].view(np.uint32)), t

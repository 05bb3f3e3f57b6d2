"""Dense-sibling SwiGLU block (BASELINE configs[4]: hidden 5120, intermediate 17408, Q6_K) against the CPU
oracle: rms_norm -> expert_mlp -> residual add (crates/xabe-engine/src/block/dense_ffn.rs:11-28, tests/
dense_ffn_differential.rs:110-140).  Rows are independent here (no routing), so at prefill width the oracle
is evaluated on a sample of rows."""
import numpy as np
import pytest

from util import rel_to_peak

pytestmark = pytest.mark.gpu

DECODE_REL, MFMA_REL = 2e-5, 1e-3


@pytest.fixture(scope="module")
def dense(oracle):
    import torch
    import llmxabe_amd as X

    H, I = 5120, 17408
    q = X.ExpertQuant.Q6K
    g = X.synth_quant(q, 41, H * I, 0.02)
    u = X.synth_quant(q, 42, H * I, 0.02)
    d = X.synth_quant(q, 43, H * I, 0.02)
    pn = 1.0 + X.synth_normal_f32(44, H, 0.1)
    w = X.DenseFfnLayerWeights(pn, X.QuantTensor(g, q), X.QuantTensor(u, q), X.QuantTensor(d, q))
    torch.cuda.synchronize()
    host = dict(pn=pn.cpu().numpy(), g=g.cpu().numpy(), u=u.cpu().numpy(), d=d.cpu().numpy())
    return X, w, host, H, I


def _run(X, w, H, I, max_tokens, tokens, seed, disable_mfma=False):
    import torch

    blk = X.DenseFfnBlock(H, I, max_tokens)
    if disable_mfma:
        blk.disable_tensor_cores()
    x = X.synth_normal_f32(seed, max_tokens * H, 1.0).view(max_tokens, H)
    x[tokens:] = 0
    ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
    blk.forward(w, x, tokens, ffn, lout)
    torch.cuda.synchronize()
    return x.cpu().numpy(), ffn.cpu().numpy(), lout.cpu().numpy(), blk.normed().cpu().numpy().reshape(max_tokens, H)


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (8, 8), (16, 5)])
def test_dense_decode_matches_oracle(oracle, dense, max_tokens, tokens):
    # tests/dense_ffn_differential.rs:64-85: 5 live tokens in a 16-token buffer
    X, w, host, H, I = dense
    x, ffn, lout, normed = _run(X, w, H, I, max_tokens, tokens, seed=51)
    n_ref, f_ref, l_ref = oracle.dense_block_forward(H, I, 1e-6, host["pn"], host["g"], host["u"], host["d"], x[:tokens],
                                                     threads=16)
    assert rel_to_peak(normed[:tokens], n_ref) <= 2e-6
    r = oracle.compare(ffn[:tokens], f_ref)
    assert rel_to_peak(ffn[:tokens], f_ref) <= DECODE_REL and r.cosine_similarity >= 1 - 1e-6, str(r)
    assert rel_to_peak(lout[:tokens], l_ref) <= DECODE_REL
    assert np.array_equal(lout[:tokens], ffn[:tokens] + x[:tokens])
    assert np.all(ffn[tokens:] == 0) and np.all(lout[tokens:] == 0)


def test_dense_decode_is_batch_invariant(dense):
    X, w, host, H, I = dense
    x8, _, l8, _ = _run(X, w, H, I, 8, 8, seed=52)
    import torch

    for t in (0, 3, 7):
        blk = X.DenseFfnBlock(H, I, 1)
        xt = torch.from_numpy(x8[t:t + 1]).cuda()
        ffn, lout = torch.zeros_like(xt), torch.zeros_like(xt)
        blk.forward(w, xt, 1, ffn, lout)
        torch.cuda.synchronize()
        assert np.array_equal(lout.cpu().numpy()[0].view(np.uint32), l8[t].view(np.uint32)), t


def test_dense_prefill_2048_matches_oracle_on_sampled_rows(oracle, dense):
    X, w, host, H, I = dense
    T = 2048
    x, ffn, lout, normed = _run(X, w, H, I, T, T, seed=53)
    rows = [0, 1, 127, 128, 1000, 2047]
    _, f_ref, l_ref = oracle.dense_block_forward(H, I, 1e-6, host["pn"], host["g"], host["u"], host["d"], x[rows], threads=16)
    r = oracle.compare(ffn[rows], f_ref)
    assert rel_to_peak(ffn[rows], f_ref) <= MFMA_REL and r.cosine_similarity >= 1 - 1e-6, str(r)
    assert rel_to_peak(lout[rows], l_ref) <= MFMA_REL
    # fp32 regime at the same width (tensor cores off) on the tight gate, two rows
    x2, ffn2, _, _ = _run(X, w, H, I, 64, 2, seed=53, disable_mfma=True)
    _, f2, _ = oracle.dense_block_forward(H, I, 1e-6, host["pn"], host["g"], host["u"], host["d"], x2[:2], threads=16)
    assert rel_to_peak(ffn2[:2], f2) <= DECODE_REL


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (8, 8), (16, 13)])
def test_long_row_kernel_equals_the_plain_one(dense, max_tokens, tokens):
    # rows longer than one 2048-element step take the step-outer kernel (weights read once per eight tokens);
    # force_community keeps the row-outer streaming kernel: same operation order per (row, token), same bits
    import torch

    X, w, host, H, I = dense
    g = X.MoeGeometry(1, 1, H, I, X.moe_block_size(max_tokens), max_tokens)
    x = X.synth_normal_f32(77, max_tokens * H, 1.0).view(max_tokens, H)
    outs = []
    for plain in (False, True):
        k = X.MoeKernels(g)
        k.force_community(plain)
        b = k.shared_only_buffers(False)
        k.set_valid_tokens(b, tokens)
        out = torch.zeros(max_tokens, H, device="cuda")
        k.shared_expert(b, w.gate, w.up, w.down, x, out)
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy().copy())
    assert outs[0][:tokens].any() and not outs[0][tokens:].any()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


CHAIN_LAYERS = 64


@pytest.fixture(scope="module")
def dense_chain():
    """configs[4]'s chain: 64 independently seeded layers (14 GB of Q6_K), each block's l_out the next block's input."""
    import torch
    import llmxabe_amd as X

    H, I = 5120, 17408
    q = X.ExpertQuant.Q6K
    layers = []
    for l in range(CHAIN_LAYERS):
        s = 70_000 + 10 * l
        t = lambda r: X.QuantTensor(X.synth_quant(q, s + r, H * I, 0.02), q)
        layers.append(X.DenseFfnLayerWeights(1.0 + X.synth_normal_f32(s, H, 0.1), t(1), t(2), t(3)))
    torch.cuda.synchronize()
    return X, layers, H, I


def _run_chain(X, layers, H, I, x_rows, max_tokens, keep=()):
    import torch

    blk = X.DenseFfnBlock(H, I, max_tokens)
    t = x_rows.shape[0]
    cur = torch.zeros(max_tokens, H, device="cuda")
    cur[:t] = x_rows
    ffn = torch.zeros_like(cur)
    kept = {}
    for l, w in enumerate(layers):
        nxt = torch.zeros_like(cur)
        blk.forward(w, cur, t, ffn, nxt)
        if l in keep:
            kept[l] = (cur[:t].cpu().numpy(), nxt[:t].cpu().numpy())
        cur = nxt
    torch.cuda.synchronize()
    return cur[:t].cpu().numpy(), kept


def test_dense_chain_is_batch_invariant_end_to_end(oracle, dense_chain):
    """Decode at batch 8 and batch 1 through all 64 layers: each token alone equals its row in the batch bit
    for bit at the END of the chain (so at every layer), and sampled layers equal the oracle on the device's
    own layer input."""
    X, layers, H, I = dense_chain
    xs = X.synth_normal_f32(54, 8 * H, 1.0).view(8, H)
    keep = (0, CHAIN_LAYERS // 2, CHAIN_LAYERS - 1)
    batch, kept = _run_chain(X, layers, H, I, xs, 8, keep=keep)
    assert np.all(np.isfinite(batch)) and np.abs(batch).max() > 0
    for t in range(8):
        alone, _ = _run_chain(X, layers, H, I, xs[t:t + 1], 1)
        assert np.array_equal(alone[0].view(np.uint32), batch[t].view(np.uint32)), f"token {t} differs alone vs in the batch"
    c = lambda t: t.cpu().numpy()
    for l in keep:
        w = layers[l]
        x_in, l_dev = kept[l]
        _, _, l_ref = oracle.dense_block_forward(H, I, 1e-6, c(w.post_norm), c(w.gate.bytes), c(w.up.bytes),
                                                 c(w.down.bytes), x_in[:2], threads=16)
        assert rel_to_peak(l_dev[:2], l_ref) <= DECODE_REL, l

"""BASELINE configs[3]: a stack of MoE blocks with independent seeded weights, l_out of one block feeding
the next.  Decode at batch 32 is checked batch-invariant (each token alone through the whole stack equals its
row in the batch, bit for bit) and each layer is checked against the oracle on the device's own input."""
import os

import numpy as np
import pytest

from util import activations, make_layer, rel_to_peak

pytestmark = pytest.mark.gpu

LAYERS = int(os.environ.get("XABE_STACK_LAYERS", "40"))


@pytest.fixture(scope="module")
def stack(oracle):
    import bench
    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(32, 32)
    layers = [bench.make_layer_device_only(X, g, seed=20_000 + 100 * l) for l in range(LAYERS)]
    return X, layers


def _run_stack(X, layers, x_rows, max_tokens, keep_inputs=False):
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    blk = X.MoeBlock(g)
    t = x_rows.shape[0]
    cur = torch.zeros(max_tokens, 2048, device="cuda")
    cur[:t] = x_rows
    ffn = torch.zeros_like(cur)
    inputs, logits = [], []
    for w in layers:
        nxt = torch.zeros_like(cur)
        blk.forward(w, cur, t, ffn, nxt)
        if keep_inputs:
            inputs.append(cur[:t].cpu().numpy())
            logits.append(blk.router_logits().view(max_tokens, 256)[:t].cpu().numpy())
        cur = nxt
    torch.cuda.synchronize()
    return cur[:t].cpu().numpy(), inputs, logits


def test_decode_b32_through_the_stack_is_batch_invariant(stack):
    X, layers = stack
    xs = activations(61, 32, 2048)
    batch, _, _ = _run_stack(X, layers, xs, 32)
    assert np.all(np.isfinite(batch))
    for t in range(32):
        alone, _, _ = _run_stack(X, layers, xs[t:t + 1], 1)
        assert np.array_equal(alone[0].view(np.uint32), batch[t].view(np.uint32)), f"token {t} differs alone vs in the batch"


def test_each_layer_matches_the_oracle_on_the_devices_input(oracle, stack):
    """Teacher-forced: layer l's oracle runs on the device's own layer input and router logits, so the check
    is per block and does not compound."""
    import torch

    X, layers = stack
    xs = activations(62, 3, 2048)
    out, inputs, logits = _run_stack(X, layers, xs, 3, keep_inputs=True)
    g = X.MoeGeometry.qwen3_6(32, 3)
    blk = X.MoeBlock(g)
    for l in list(range(0, LAYERS, max(1, LAYERS // 5)))[:5]:
        w = layers[l]
        c = lambda t: t.cpu().numpy()
        host = oracle.MoeWeights(
            num_experts=256, top_k=8, hidden=2048, intermediate=512, eps=1e-6, post_norm=c(w.post_norm), router_f32=None,
            router_q8=c(w.router), gate_exps=c(w.gate_exps.bytes), up_exps=c(w.up_exps.bytes),
            down_exps=c(w.down_exps.bytes), shared_gate_inp=c(w.shared_gate_inp), shared_gate=c(w.shared_gate.bytes),
            shared_up=c(w.shared_up.bytes), shared_down=c(w.shared_down.bytes))
        ref = oracle.moe_block_forward(host, inputs[l], logits_override=logits[l], threads=8)
        x = torch.from_numpy(inputs[l]).cuda()
        ffn, lout = torch.zeros_like(x), torch.zeros_like(x)
        blk.forward(w, x, 3, ffn, lout)
        torch.cuda.synchronize()
        assert np.array_equal(blk.buffers().topk_ids().cpu().numpy().reshape(3, 8), ref.topk_ids.astype(np.int32)), l
        assert rel_to_peak(lout.cpu().numpy(), ref.l_out) <= 2e-5, l


def test_prefill_8192_chunk_through_the_whole_stack(oracle, stack):
    """The 8192-token prefill chunk (B = 64) through every layer of the stack, each block's l_out the next
    block's input: finite everywhere; every layer's dispatch tables hold each live (token, k) exactly once; on
    sampled layers ALL 8192 rows are routed exactly as the CPU reference routes the device's own logits; and a
    sample of rows of those layers is checked against the oracle block at the matrix-core tolerance."""
    import torch

    X, layers = stack
    T = 8192
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    assert g.block_size == 64
    blk = X.MoeBlock(g)
    cur = activations(63, T, 2048)
    ffn = torch.zeros_like(cur)
    sampled = sorted({0, 2, LAYERS // 2, LAYERS - 1})
    rows = [0, 63, 64, 4097, 8191]
    kept = {}
    all_pairs = np.arange(T * 8)
    for l, w in enumerate(layers):
        nxt = torch.zeros_like(cur)
        blk.forward(w, cur, T, ffn, nxt)
        b = blk.buffers()
        sorted_ids = b.sorted_token_ids().cpu().numpy()
        n = int(b.num_tokens_post_pad().cpu().numpy()[0])
        assert n % 64 == 0 and n <= sorted_ids.size, l
        live = sorted_ids[:n][sorted_ids[:n] != T * 8]
        assert live.size == T * 8 and np.array_equal(np.sort(live), all_pairs), f"layer {l}: dispatch tables"
        assert np.all(sorted_ids[n:] == T * 8), f"layer {l}: sentinel fill"
        if l in sampled:
            kept[l] = dict(x=cur[rows].cpu().numpy(), out=nxt[rows].cpu().numpy(),
                           logits=blk.router_logits().view(T, 256).cpu().numpy(),
                           ids=b.topk_ids().view(T, 8).cpu().numpy())
        assert bool(torch.isfinite(nxt).all()), f"layer {l}: non-finite l_out"
        cur = nxt
    torch.cuda.synchronize()
    c = lambda t: t.cpu().numpy()
    for l, k in kept.items():
        ref_ids, _ = oracle.route_batch(k["logits"], 8)
        assert np.array_equal(k["ids"], ref_ids.astype(np.int32)), f"layer {l}: routing differs from route_batch(device logits)"
        w = layers[l]
        host = oracle.MoeWeights(
            num_experts=256, top_k=8, hidden=2048, intermediate=512, eps=1e-6, post_norm=c(w.post_norm), router_f32=None,
            router_q8=c(w.router), gate_exps=c(w.gate_exps.bytes), up_exps=c(w.up_exps.bytes),
            down_exps=c(w.down_exps.bytes), shared_gate_inp=c(w.shared_gate_inp), shared_gate=c(w.shared_gate.bytes),
            shared_up=c(w.shared_up.bytes), shared_down=c(w.shared_down.bytes))
        ref = oracle.moe_block_forward(host, k["x"], logits_override=k["logits"][rows], threads=8)
        assert np.array_equal(k["ids"][rows], ref.topk_ids.astype(np.int32)), l
        assert rel_to_peak(k["out"], ref.l_out) <= 1e-3, l

"""GPU parity of the matrix-core (MFMA, fp16 operands, fp32 accumulate) regime against the CPU oracle.

Tolerance.  Operands are rounded to fp16 (11-bit significand), so this regime is gated the way the
reference gates its own reduced-precision (int8 tensor-core) path: max |gpu - oracle| relative to the
peak of the reference tensor, and cosine similarity (crates/xabe-engine/tests/moe_differential.rs:140-145:
max_abs <= 1e-4 on outputs of max 1e-2, cos >= 0.9999).  fp16 operands are about 30x finer than int8
activations, and the gates here are correspondingly tighter: MFMA_REL of peak, MFMA_COS."""
import numpy as np
import pytest

from util import activations, make_layer, rel_to_peak, run_block

pytestmark = pytest.mark.gpu

MFMA_REL = 1e-3       # max |gpu - oracle| / max |oracle|   (north_star: max-rel <= 1e-3)
MFMA_COS = 1 - 1e-6


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _route_dispatch(X, g, tokens, logits_np):
    import torch

    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    buf = np.zeros((g.max_tokens, g.num_experts), np.float32)
    buf[:tokens] = logits_np
    k.route_and_dispatch(b, torch.from_numpy(buf).cuda())
    return k, b


def _naive(oracle, host, xs, ids, w, threads=8):
    """naive_forward restricted to the experts in use (dequantised on demand)."""
    E, H, I = host.num_experts, host.hidden, host.intermediate
    bb = oracle.BLOCK_BYTES[host.gate_quant] * (I * H // oracle.BLOCK_ELEMENTS[host.gate_quant])
    out = np.zeros((xs.shape[0], H), np.float32)
    contrib = {}
    for e in np.unique(ids):
        mats = [oracle.dequantize_row(host.gate_quant, m[e * bb:(e + 1) * bb])
                for m in (host.gate_exps, host.up_exps, host.down_exps)]
        for t, kk in zip(*np.nonzero(ids == e)):
            contrib[(t, kk)] = oracle.expert_mlp(*mats, xs[t], H, I)
    for t in range(xs.shape[0]):
        acc = np.zeros(H, np.float32)
        for kk in range(ids.shape[1]):
            acc = (acc + w[t, kk] * contrib[(t, kk)]).astype(np.float32)
        out[t] = acc
    return out


@pytest.mark.parametrize("fmt", ["q6k", "q8_0"])
@pytest.mark.parametrize("max_tokens,tokens,mode", [(64, 64, "uniform"), (96, 70, "uniform"), (256, 200, "one_expert"),
                                                    (300, 300, "coherent")])
def test_grouped_forward_small_geometry(oracle, X, fmt, max_tokens, tokens, mode):
    import torch

    q = X.ExpertQuant.Q6K if fmt == "q6k" else X.ExpertQuant.Q8_0
    g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens)
    layer = make_layer(oracle, g, seed=310, expert_quant=q)
    x = activations(31, max_tokens, 512, tokens, coherent=(mode == "coherent"))
    rng = np.random.default_rng(tokens)
    logits = rng.uniform(-3, 3, (tokens, 8)).astype(np.float32)
    if mode == "one_expert":            # every token collides in one expert's run
        logits[:, 6] = 9.0
        logits[:, 1] = 8.0
    k, b = _route_dispatch(X, g, tokens, logits)
    assert k.tensor_cores_enabled()
    out = torch.zeros(max_tokens, 512, device="cuda")
    k.grouped_forward(b, layer.dev.gate_exps, layer.dev.up_exps, layer.dev.down_exps, x, out)
    torch.cuda.synchronize()
    ids = b.topk_ids().cpu().numpy().reshape(max_tokens, 2)[:tokens]
    w = b.topk_weights().cpu().numpy().reshape(max_tokens, 2)[:tokens]
    assert np.array_equal(ids, oracle.route_batch(logits, 2)[0].astype(np.int32))
    ref = _naive(oracle, layer.host, x.cpu().numpy()[:tokens], ids, w)
    got = out.cpu().numpy()
    r = oracle.compare(got[:tokens], ref)
    assert rel_to_peak(got[:tokens], ref) <= MFMA_REL and r.cosine_similarity >= MFMA_COS, str(r)
    assert np.all(got[tokens:] == 0)
    # the fp32 regime on the same inputs (tensor cores off) stays on the tight gate
    k2, b2 = _route_dispatch(X, g, tokens, logits)
    k2.disable_tensor_cores()
    out2 = torch.zeros(max_tokens, 512, device="cuda")
    k2.grouped_forward(b2, layer.dev.gate_exps, layer.dev.up_exps, layer.dev.down_exps, x, out2)
    torch.cuda.synchronize()
    assert rel_to_peak(out2.cpu().numpy()[:tokens], ref) <= 2e-5


# (layer seed, activations seed, c of the Zipf bias): "benched" is bench.py's `tokens_512_zipf` leg on its first
# layer (layer seed 10000, activations seed 99, b_e = -1.1 ln rank_e), input for input; "steep" a harsher skew
PREFILL_512_CASES = {"uniform": (710, 32, None), "benched": (10000, 99, 1.0), "steep": (710, 32, 2.0)}


@pytest.mark.parametrize("case", sorted(PREFILL_512_CASES))
def test_block_prefill_512_matches_oracle(oracle, X, case):
    """BASELINE configs[2]: a 512-token chunk; the skewed cases put a seeded Zipf(1.1) bias on the router logits
    (`llmxabe_amd.zipf_logit_bias`, the definition bench.py times), so a few experts receive 50+ tokens and many
    receive none."""
    import torch

    tokens = 512
    layer_seed, x_seed, c = PREFILL_512_CASES[case]
    skew = c is not None
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(tokens), tokens)
    layer = make_layer(oracle, g, seed=layer_seed)
    x = activations(x_seed, tokens, 2048)
    bias_np = X.zipf_logit_bias(256, c=c) if skew else None
    bias = torch.from_numpy(bias_np).cuda() if skew else None
    blk = X.MoeBlock(g)
    ffn_out, l_out = run_block(blk, layer, x, tokens, logit_bias=bias)
    dev_logits = blk.router_logits().cpu().numpy().reshape(tokens, 256)
    xs = x.cpu().numpy()
    ref = oracle.moe_block_forward(layer.host, xs, logits_override=dev_logits, threads=16)
    ids = blk.buffers().topk_ids().cpu().numpy().reshape(tokens, 8)
    assert np.array_equal(ids, ref.topk_ids.astype(np.int32))          # routing bit-exact on the device's logits
    own = oracle.moe_block_forward(layer.host, xs[:8], logit_bias=bias_np, threads=8)
    assert rel_to_peak(dev_logits[:8], own.logits) <= 2e-5              # fp32 router, reassociation only
    counts = np.bincount(ids.ravel(), minlength=256)
    if skew:
        assert counts.max() >= 50 and (counts <= 2).sum() >= 64, (counts.max(), (counts <= 2).sum())
    take = lambda t: t.cpu().numpy().reshape(tokens, 2048)
    for name, got, want in (("routed", take(blk.routed()), ref.routed), ("shexp", take(blk.shared_ungated()), ref.shexp),
                            ("ffn_out", take(ffn_out), ref.ffn_out)):
        r = oracle.compare(got, want)
        assert rel_to_peak(got, want) <= MFMA_REL and r.cosine_similarity >= MFMA_COS, (name, str(r))
    assert rel_to_peak(take(l_out), ref.l_out) <= MFMA_REL
    assert np.array_equal(take(l_out), take(ffn_out) + xs)


def test_shared_expert_mma_matches_expert_mlp(oracle, X):
    import torch

    for H, I, T in ((512, 256, 130), (2048, 512, 64)):
        g = X.MoeGeometry(8, 2, H, I, 32, T)
        layer = make_layer(oracle, g, seed=311)
        x = activations(33, T, H, T - 3)
        k = X.MoeKernels(g)
        b = k.buffers()
        k.set_valid_tokens(b, T - 3)
        out = torch.zeros(T, H, device="cuda")
        d = layer.dev
        k.shared_expert_mma(b, d.shared_gate, d.shared_up, d.shared_down, x, out)
        torch.cuda.synchronize()
        h = layer.host
        sg, su, sd = (oracle.dequantize_row(oracle.Q8_0, m) for m in (h.shared_gate, h.shared_up, h.shared_down))
        got, xs = out.cpu().numpy(), x.cpu().numpy()
        ref = np.stack([oracle.expert_mlp(sg, su, sd, xs[t], H, I) for t in range(T - 3)])
        r = oracle.compare(got[:T - 3], ref)
        assert rel_to_peak(got[:T - 3], ref) <= MFMA_REL and r.cosine_similarity >= MFMA_COS, str(r)
        assert np.all(got[T - 3:] == 0)
    k.disable_tensor_cores()
    with pytest.raises(X.moe.UnsupportedGeometry, match="matrix cores are disabled"):
        k.shared_expert_mma(b, d.shared_gate, d.shared_up, d.shared_down, x, out)


def test_prefill_rows_do_not_depend_on_batch_mates(oracle, X):
    """Within the matrix-core regime a token's row is the same bits whatever else is in the pass."""
    import torch

    g = X.MoeGeometry.qwen3_6(32, 128)
    layer = make_layer(oracle, g, seed=712)
    blk = X.MoeBlock(g)
    xa = activations(34, 128, 2048)
    _, la = run_block(blk, layer, xa, 128)
    xb = activations(35, 128, 2048)
    xb[5], xb[77] = xa[77], xa[5]       # same two tokens, other slots, other batch mates
    _, lb = run_block(blk, layer, xb, 100)
    la, lb = la.cpu().numpy(), lb.cpu().numpy()
    assert np.array_equal(la[77].view(np.uint32), lb[5].view(np.uint32))
    assert np.array_equal(la[5].view(np.uint32), lb[77].view(np.uint32))


def test_tall_tiles_give_the_rows_of_the_short_tiles(oracle, X):
    """From ~192 selections per expert up the routed gate/up launch runs 384-row token tiles (eight wavefronts, live
    32-row blocks only); every output element still sees the same operands in the same order, so with the same
    selections a token's routed row in an 8192-token pass is the bits it has in a 128-token pass, where the 64-row
    tiles run."""
    import torch

    g_wide = X.MoeGeometry.qwen3_6(X.moe_block_size(8192), 8192)
    g_small = X.MoeGeometry.qwen3_6(32, 128)
    layer = make_layer(oracle, g_wide, seed=733)
    d = layer.dev
    rng = np.random.default_rng(9)
    logits_s = rng.uniform(-3, 3, (128, 256)).astype(np.float32)
    logits_w = rng.uniform(-3, 3, (8192, 256)).astype(np.float32)
    xs = activations(36, 128, 2048)
    xw = activations(37, 8192, 2048)
    picks = [(0, 17), (5000, 5), (8191, 77), (4095, 127)]       # (row of the wide pass, row of the small pass)
    for rw, r in picks:
        xw[rw] = xs[r]
        logits_w[rw] = logits_s[r]

    def routed(g, tokens, logits, x):
        k, b = _route_dispatch(X, g, tokens, logits)
        assert k.tensor_cores_enabled()
        out = torch.zeros(g.max_tokens, 2048, device="cuda")
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        torch.cuda.synchronize()
        return out.cpu().numpy(), b.topk_ids().cpu().numpy()[:tokens * 8]

    small, _ = routed(g_small, 128, logits_s, xs)
    wide, ids = routed(g_wide, 8192, logits_w, xw)
    # the wide pass did fill tall tiles: every expert took more than 128 rows and at most one tile's worth
    counts = np.bincount(ids.ravel(), minlength=256)
    assert counts.min() > 128 and counts.max() <= 384, (counts.min(), counts.max())
    for rw, r in picks:
        assert np.array_equal(wide[rw].view(np.uint32), small[r].view(np.uint32)), (rw, r)
    # fewer live tokens in the same geometry: the experts' runs end inside the tall tiles' second blocks
    wide2, ids2 = routed(g_wide, 6200, logits_w[:6200], xw)
    assert np.bincount(ids2.ravel(), minlength=256).max() <= 256
    for rw, r in picks[:2]:
        assert np.array_equal(wide2[rw].view(np.uint32), small[r].view(np.uint32)), (rw, r)
    assert np.all(wide2[6200:] == 0)
    # and against the oracle, a few rows
    k, b = _route_dispatch(X, g_wide, 8192, logits_w)
    tw = b.topk_weights().cpu().numpy().reshape(8192, 8)
    rows = [0, 5000, 8191]
    ref = _naive(oracle, layer.host, xw.cpu().numpy()[rows], ids.reshape(8192, 8)[rows], tw[rows])
    assert rel_to_peak(wide[rows], ref) <= MFMA_REL


def test_wide_block_passes_back_to_back_keep_their_own_shared_rows(oracle, X):
    """At matrix-core widths the shared expert runs on a stream of the block's own, forked from the caller's after the
    RMSNorm and joined before the combine.  Passes issued back to back on one block, alternating two inputs, must each
    give the bits of the same pass run alone: a pass's shared rows are not read before they are written, nor
    overwritten by the next pass before its combine has read them.  Eagerly on a caller's stream, and as a captured
    graph replayed with eager passes between the replays."""
    import torch

    tokens = 512
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(tokens), tokens)
    layer = make_layer(oracle, g, seed=710)
    xa, xb = activations(41, tokens, 2048), activations(42, tokens, 2048)
    blk = X.MoeBlock(g)
    alone = {}
    for name, x in (("a", xa), ("b", xb)):
        ffn, lout = run_block(blk, layer, x, tokens)
        torch.cuda.synchronize()
        alone[name] = (ffn.view(torch.int32).clone(), blk.shared_ungated().view(torch.int32).clone())
    assert not torch.equal(alone["a"][0], alone["b"][0])
    stream = torch.cuda.Stream()
    outs = [(torch.zeros_like(xa), torch.zeros_like(xa)) for _ in range(8)]
    with torch.cuda.stream(stream):
        for i, (ffn, lout) in enumerate(outs):
            blk.forward(layer.dev, xa if i % 2 == 0 else xb, tokens, ffn, lout)
        stream.synchronize()
        for i, (ffn, _) in enumerate(outs):
            assert torch.equal(ffn.view(torch.int32), alone["ab"[i % 2]][0]), f"pass {i} of 8 back to back"
        # captured: two passes in one graph (a then b), replayed with an eager pass of the other input in between
        (fa, la), (fb, lb) = outs[0], outs[1]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            blk.forward(layer.dev, xa, tokens, fa, la)
            blk.forward(layer.dev, xb, tokens, fb, lb)
        for rep in range(3):
            fa.fill_(float("nan")); fb.fill_(float("nan"))
            blk.forward(layer.dev, xb if rep % 2 == 0 else xa, tokens, outs[2][0], outs[2][1])
            graph.replay()
            stream.synchronize()
            assert torch.equal(fa.view(torch.int32), alone["a"][0]), f"replay {rep}, first pass"
            assert torch.equal(fb.view(torch.int32), alone["b"][0]), f"replay {rep}, second pass"
            assert torch.equal(blk.shared_ungated().view(torch.int32), alone["b"][1]), f"replay {rep}, shared rows"


def test_block_routes_512_experts_from_the_planes(oracle, X):
    """The same with 512 experts (eight logits per lane of the routing wavefront, the widest it holds) on the small
    test shape: logits, selections and weights of the block are the bits of the step-by-step calls, and the
    selections are the CPU reference's on those logits."""
    import torch

    tokens = 256
    g = X.MoeGeometry(512, 4, 512, 256, 32, tokens)
    layer = make_layer(oracle, g, seed=719)
    x = activations(46, tokens, 512)
    bias = torch.from_numpy(X.zipf_logit_bias(512, seed=11)).cuda()
    blk = X.MoeBlock(g)
    run_block(blk, layer, x, tokens, logit_bias=bias)
    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    logits = torch.zeros(tokens, 512, device="cuda")
    k.router_logits(b, layer.dev.router, layer.dev.router_quant, blk.normed(), logits)
    k.add_logit_bias(b, bias, logits)
    k.route(b, logits)
    torch.cuda.synchronize()
    assert torch.equal(blk.router_logits().view(torch.int32).reshape(tokens, 512), logits.view(torch.int32))
    assert torch.equal(blk.buffers().topk_ids(), b.topk_ids())
    assert torch.equal(blk.buffers().topk_weights().view(torch.int32), b.topk_weights().view(torch.int32))
    ids = blk.buffers().topk_ids().cpu().numpy().reshape(tokens, 4)
    assert np.array_equal(ids, oracle.route_batch(logits.cpu().numpy(), 4)[0].astype(np.int32))


@pytest.mark.parametrize("tokens,biased", [(512, True), (512, False), (2048, True)])
def test_block_routes_from_the_planes_as_the_step_by_step_calls_do(oracle, X, tokens, biased):
    """Where the router GEMM splits its contraction, the block adds the partial planes (and the logit bias) in the
    routing launch instead of a launch of their own.  Same additions in the same order: the logits, the selections
    and the weights the block leaves are the bits of router_logits + add_logit_bias + route called one by one."""
    import torch

    g = X.MoeGeometry.qwen3_6(X.moe_block_size(tokens), tokens)
    layer = make_layer(oracle, g, seed=712)
    x = activations(45, tokens, 2048)
    bias = torch.from_numpy(X.zipf_logit_bias(256, seed=7, c=1.5)).cuda() if biased else None
    blk = X.MoeBlock(g)
    run_block(blk, layer, x, tokens, logit_bias=bias)
    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    logits = torch.zeros(tokens, 256, device="cuda")
    k.router_logits(b, layer.dev.router, layer.dev.router_quant, blk.normed(), logits)
    if biased:
        k.add_logit_bias(b, bias, logits)
    k.route(b, logits)
    torch.cuda.synchronize()
    assert torch.equal(blk.router_logits().view(torch.int32).reshape(tokens, 256), logits.view(torch.int32))
    assert torch.equal(blk.buffers().topk_ids(), b.topk_ids())
    assert torch.equal(blk.buffers().topk_weights().view(torch.int32), b.topk_weights().view(torch.int32))


def test_forward_captured_alone_makes_its_own_tile_lists(oracle, X):
    """The dispatch build leaves the grouped GEMM's token-tile lists, cut for the tile heights of the count then
    published; a forward trusts them only when both were launched eagerly or recorded into the same capture.  A
    forward captured on its own carries its own list build: replayed after a wider pass was published and dispatched
    outside the graph (lists cut for taller tiles), it still gives the bits of the eager forward of that pass."""
    import torch

    T = 8192
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    layer = make_layer(oracle, g, seed=733)
    d = layer.dev
    rng = np.random.default_rng(12)
    logits = torch.from_numpy(rng.uniform(-3, 3, (T, 256)).astype(np.float32)).cuda()
    x = activations(37, T, 2048)
    k = X.MoeKernels(g)
    b = k.buffers()
    out = torch.zeros(T, 2048, device="cuda")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        k.set_valid_tokens(b, 512)
        k.route_and_dispatch(b, logits)
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)       # warm-up of the 64-row form
        stream.synchronize()
        small = out[:512].view(torch.int32).clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)   # the forward alone, 64-row tiles
        out.zero_()
        graph.replay()
        stream.synchronize()
        assert torch.equal(out[:512].view(torch.int32), small)
        # a full pass, published and dispatched eagerly: the lists the dispatch leaves are cut for 128 / 384 rows
        k.set_valid_tokens(b, T)
        k.route_and_dispatch(b, logits)
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        stream.synchronize()
        wide = out.view(torch.int32).clone()
        assert torch.equal(wide[:512], small)            # a token's routed row does not depend on the pass's width
        out.zero_()
        k.route_and_dispatch(b, logits)                  # (lists for the tall tiles again)
        graph.replay()                                   # 64-row kernels over the full pass, from their own lists
        stream.synchronize()
        assert torch.equal(out.view(torch.int32), wide)


def test_eager_forward_after_a_replayed_dispatch_graph_makes_its_own_tile_lists(oracle, X):
    """The other direction: a graph that holds a dispatch build rewrites the device's tile lists on every replay without
    the host knowing.  Capture the dispatch of a full pass (lists cut for 128 / 384 rows), then publish 512 tokens and
    dispatch eagerly (the host now believes the lists are cut for 64 rows), replay the graph, and run the forward
    eagerly: it must not run the 64-row kernels over the graph's tall entries."""
    import torch

    T = 8192
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    layer = make_layer(oracle, g, seed=734)
    d = layer.dev
    rng = np.random.default_rng(13)
    logits = torch.from_numpy(rng.uniform(-3, 3, (T, 256)).astype(np.float32)).cuda()
    x = activations(38, T, 2048)
    k = X.MoeKernels(g)
    b = k.buffers()
    out = torch.zeros(T, 2048, device="cuda")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        # reference rows of the full pass, all eager
        k.set_valid_tokens(b, T)
        k.route_and_dispatch(b, logits)
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        stream.synchronize()
        wide = out.view(torch.int32).clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            k.route_and_dispatch(b, logits)              # the dispatch alone: tall lists on every replay
        graph.replay()
        # a 512-token pass dispatched eagerly: 64-row lists, and the host's bookkeeping says so
        k.set_valid_tokens(b, 512)
        k.route_and_dispatch(b, logits)
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        stream.synchronize()
        assert torch.equal(out[:512].view(torch.int32), wide[:512])
        # the graph rewrites tables and lists for whatever count is published (512 here) at the heights it was captured for
        out.zero_()
        graph.replay()
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        stream.synchronize()
        assert torch.equal(out[:512].view(torch.int32), wide[:512])
        assert not out[512:].any()
        # and the full pass through the same sequence
        k.set_valid_tokens(b, T)
        out.zero_()
        graph.replay()
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        stream.synchronize()
        assert torch.equal(out.view(torch.int32), wide)


@pytest.mark.parametrize("router_q8", [True, False])
def test_router_gemm_tile_widths_give_the_same_bits(oracle, X, router_q8):
    """While its 128-expert tiles are fewer than the compute units (512 tokens) the router GEMM runs 64-expert tiles;
    a logit is the same products added in the same order either way, so a row of a 512-token pass is the bits it
    has in a 2048-token pass (128-expert tiles, the contraction in the same eight parts)."""
    import torch

    g_small = X.MoeGeometry.qwen3_6(X.moe_block_size(512), 512)
    g_wide = X.MoeGeometry.qwen3_6(X.moe_block_size(2048), 2048)
    layer = make_layer(oracle, g_small, seed=716, router_q8=router_q8)
    normed_w = activations(34, 2048, 2048)
    normed_s = normed_w[:512].clone()
    out = []
    for g, normed in ((g_small, normed_s), (g_wide, normed_w)):
        k = X.MoeKernels(g)
        b = k.buffers()
        k.set_valid_tokens(b, g.max_tokens)
        logits = torch.zeros(g.max_tokens, 256, device="cuda")
        k.router_logits(b, layer.dev.router, layer.dev.router_quant, normed, logits)
        torch.cuda.synchronize()
        out.append(logits)
    assert torch.equal(out[0].view(torch.int32), out[1][:512].view(torch.int32))


@pytest.mark.parametrize("router_q8", [True, False])
def test_router_logits_matrix_core_path(oracle, X, router_q8):
    # from 2048 tokens up the router runs on the fp32 matrix instruction: fp32 operands, so the logits agree
    # with the CPU reference to fp32 reassociation (the decode-width kernel's bound), for live rows only
    import torch

    T, live = 2048, 1990
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    layer = make_layer(oracle, g, seed=715, router_q8=router_q8)
    normed = activations(33, T, 2048, live)
    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, live)
    logits = torch.full((T, 256), 7.0, device="cuda")
    d = layer.dev
    k.router_logits(b, d.router, d.router_quant, normed, logits)
    torch.cuda.synchronize()
    got = logits.cpu().numpy()
    assert np.all(got[live:] == 7.0)                                    # rows past the live tokens are not written
    host = layer.host
    w = (oracle.dequantize_row(oracle.Q8_0, host.router_q8) if router_q8 else host.router_f32).reshape(256, 2048)
    rows = np.r_[0:40, 1000:1040, live - 40:live]
    want = normed.cpu().numpy()[rows].astype(np.float64) @ w.astype(np.float64).T
    assert rel_to_peak(got[rows], want) <= 2e-5


@pytest.mark.parametrize("tokens,quant", [(8192, "q6k"), (5000, "q6k"), (3072, "q6k"), (1024, "q6k"), (8192, "q8_0"), (640, "q8_0")])
def test_specialised_wavefronts_give_the_bits_of_the_plain_kernel(oracle, X, tokens, quant):
    """k_mfma_pc (half of a workgroup's wavefronts multiply, half dequantise; 64-element steps; 128-row x 256-weight-row
    tiles; selected with set_mfma_form(2)) against k_mfma_expert on the same pass: every output element sees the same
    fp16 operands in the same order of matrix instructions, so `partial` and the reduced rows are the same bits.
    Several widths, a ragged live count, both formats."""
    import torch

    q = X.ExpertQuant.Q6K if quant == "q6k" else X.ExpertQuant.Q8_0
    T = max(tokens, 64)
    g = X.MoeGeometry.qwen3_6(X.moe_block_size(T), T)
    layer = make_layer(oracle, g, seed=736, expert_quant=q)
    d = layer.dev
    rng = np.random.default_rng(tokens)
    logits = torch.from_numpy(rng.uniform(-3, 3, (T, 256)).astype(np.float32)).cuda()
    x = activations(39, T, 2048)
    live = tokens - 3
    outs = []
    for form in (1, 2):
        k = X.MoeKernels(g)
        k.set_mfma_form(form)
        b = k.buffers()
        k.set_valid_tokens(b, live)
        k.route_and_dispatch(b, logits)
        out = torch.zeros(T, 2048, device="cuda")
        k.grouped_forward(b, d.gate_exps, d.up_exps, d.down_exps, x, out)
        torch.cuda.synchronize()
        outs.append((out, b.partial().clone()))
        del k, b
    assert float(outs[0][0][:live].abs().max()) > 0
    assert torch.equal(outs[0][0].view(torch.int32), outs[1][0].view(torch.int32))
    n = live * 8 * 2048
    assert torch.equal(outs[0][1][:n].view(torch.int32), outs[1][1][:n].view(torch.int32))

"""GPU parity of the decode regime (fp32 accumulate) against the CPU oracle, through the C ABI.

Tolerances.  The decode kernels sum each row in a lane-tiled order with fused multiply-adds, the oracle
sequentially with separately rounded products: the difference is fp32 reassociation only.  The reference
gates its fp32 path at max_abs 5e-7 on outputs of max 1e-2 (5e-5 of peak) and cos >= 1-1e-6
(crates/xabe-engine/tests/moe_differential.rs:147-152); the same form is used here: DECODE_REL of peak."""
import numpy as np
import pytest

from util import activations, make_layer, rel_to_peak, run_block

pytestmark = pytest.mark.gpu

DECODE_REL = 2e-5     # max |gpu - oracle| / max |oracle|
DECODE_COS = 1 - 1e-6


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def _dequant_stacks(oracle, host):
    E = host.num_experts
    f = lambda q, b: oracle.dequantize_row(q, b).reshape(E, -1)
    return f(host.gate_quant, host.gate_exps), f(host.up_quant, host.up_exps), f(host.down_quant, host.down_exps)


def _grouped(X, oracle, g, layer, x, tokens, logits_np, exact=False, flat_only=False):
    """route + dispatch + grouped_forward on the device; naive_forward over dequantised weights on the host."""
    import torch

    k = X.MoeKernels(g)
    if exact:
        k.set_exact_decode_regime(True)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    buf = np.zeros((g.max_tokens, g.num_experts), np.float32)
    buf[:tokens] = logits_np
    k.route_and_dispatch(b, torch.from_numpy(buf).cuda())
    out = torch.zeros(g.max_tokens, g.hidden, device="cuda")
    k.grouped_forward(b, layer.dev.gate_exps, layer.dev.up_exps, layer.dev.down_exps, x, out)
    torch.cuda.synchronize()
    ids = b.topk_ids().cpu().numpy().reshape(g.max_tokens, -1)[:tokens]
    w = b.topk_weights().cpu().numpy().reshape(g.max_tokens, -1)[:tokens]
    return out.cpu().numpy(), ids, w, b


# the reference's synthetic geometry and widths (tests/moe_quant_formats_differential.rs:64-68, :187)
@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (2, 2), (4, 3), (8, 6), (33, 20)])
@pytest.mark.parametrize("fmt", ["q6k", "q8_0"])
def test_grouped_forward_small_geometry(oracle, X, max_tokens, tokens, fmt):
    q = X.ExpertQuant.Q6K if fmt == "q6k" else X.ExpertQuant.Q8_0
    g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens)
    layer = make_layer(oracle, g, seed=300, expert_quant=q)
    x = activations(11, max_tokens, 512, tokens)
    rng = np.random.default_rng(tokens)
    logits = rng.uniform(-3, 3, (tokens, 8)).astype(np.float32)
    out, ids, w, _ = _grouped(X, oracle, g, layer, x, tokens, logits)
    ref_ids, ref_w = oracle.route_batch(logits, 2)
    assert np.array_equal(ids, ref_ids.astype(np.int32))
    gate, up, down = _dequant_stacks(oracle, layer.host)
    ref = oracle.naive_forward(x.cpu().numpy()[:tokens], ref_ids, ref_w, gate, up, down, 512, 256)
    r = oracle.compare(out[:tokens], ref)
    assert rel_to_peak(out[:tokens], ref) <= DECODE_REL and r.cosine_similarity >= DECODE_COS, str(r)
    assert np.all(out[tokens:] == 0)  # rows past `tokens` are never written (moe_differential.rs:828-838)


def _naive_model_ref(oracle, host, xs, ref_ids, ref_w, tokens):
    """naive_forward over the selected experts only (dequantised on demand), model geometry, Q6_K."""
    ref = np.zeros((tokens, 2048), np.float32)
    mat = 512 * 2048 // 256 * 210
    cache = {}
    for t in range(tokens):
        acc = np.zeros(2048, np.float32)
        for kk in range(8):
            e = int(ref_ids[t, kk])
            if e not in cache:
                cache[e] = [oracle.dequantize_row(oracle.Q6K, m[e * mat:(e + 1) * mat])
                            for m in (host.gate_exps, host.up_exps, host.down_exps)]
            c = oracle.expert_mlp(*cache[e], xs[t], 2048, 512)
            acc = (acc + ref_w[t, kk] * c).astype(np.float32)
        ref[t] = acc
    return ref


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (3, 3), (4, 2), (32, 32), (37, 37)])
def test_grouped_forward_model_geometry(oracle, X, max_tokens, tokens):
    g = X.MoeGeometry.qwen3_6(32, max_tokens)
    layer = make_layer(oracle, g, seed=500)
    x = activations(12, max_tokens, 2048, tokens)
    r = oracle.Xorshift64Star(0xA11 + tokens)
    logits = np.stack([r.vec_f32(256, -8.0, 8.0) for _ in range(tokens)])
    out, ids, w, _ = _grouped(X, oracle, g, layer, x, tokens, logits)
    ref_ids, ref_w = oracle.route_batch(logits, 8)
    assert np.array_equal(ids, ref_ids.astype(np.int32))
    ref = _naive_model_ref(oracle, layer.host, x.cpu().numpy(), ref_ids, ref_w, tokens)
    rr = oracle.compare(out[:tokens], ref)
    assert rel_to_peak(out[:tokens], ref) <= DECODE_REL and rr.cosine_similarity >= DECODE_COS, str(rr)


@pytest.mark.parametrize("max_tokens,tokens", [(8, 8), (12, 12), (12, 7)])
def test_exact_decode_regime_matches_naive_forward(oracle, X, max_tokens, tokens):
    """The exact-decode regime (kernels/moe.rs:5436-5452) pins the flat per-pair kernels at widths that would
    otherwise take the dispatch tables; the speculative verify windows of 2-12 rows are its callers
    (tests/moe_differential.rs:1392-1402).  Checked directly against the CPU reference at the fp32 gate."""
    g = X.MoeGeometry.qwen3_6(32, max_tokens)
    layer = make_layer(oracle, g, seed=510)
    x = activations(14, max_tokens, 2048, tokens)
    r = oracle.Xorshift64Star(0xE8AC7 + tokens)
    logits = np.stack([r.vec_f32(256, -8.0, 8.0) for _ in range(tokens)])
    out, ids, w, b = _grouped(X, oracle, g, layer, x, tokens, logits, exact=True)
    ref_ids, ref_w = oracle.route_batch(logits, 8)
    assert np.array_equal(ids, ref_ids.astype(np.int32))
    assert np.abs(w - ref_w).max() <= 1e-6
    ref = _naive_model_ref(oracle, layer.host, x.cpu().numpy(), ref_ids, ref_w, tokens)
    rr = oracle.compare(out[:tokens], ref)
    assert rel_to_peak(out[:tokens], ref) <= DECODE_REL and rr.cosine_similarity >= DECODE_COS, str(rr)
    assert np.all(out[tokens:] == 0)
    # the regime really is the flat one: no dispatch table was built for this pass
    assert int(b.num_tokens_post_pad().cpu().numpy()[0]) == 0
    # and the same pass without the pin (dispatch-table kernels) gives the same bits
    out2, ids2, _, _ = _grouped(X, oracle, g, layer, x, tokens, logits, exact=False)
    assert np.array_equal(ids2, ids) and np.array_equal(out2.view(np.uint32), out.view(np.uint32))


def test_all_tokens_to_one_expert_collides_in_one_dispatch_run(oracle, X):
    """Adversarial routing: every token picks the same experts, so one dispatch run holds all of them."""
    g = X.MoeGeometry(8, 2, 512, 256, 32, 40)
    layer = make_layer(oracle, g, seed=301)
    x = activations(13, 40, 512, 40)
    logits = np.zeros((40, 8), np.float32)
    logits[:, 5] = 4.0
    logits[:, 2] = 3.0
    out, ids, w, _ = _grouped(X, oracle, g, layer, x, 40, logits)
    assert np.all(ids == np.array([5, 2]))
    gate, up, down = _dequant_stacks(oracle, layer.host)
    ref = oracle.naive_forward(x.cpu().numpy(), ids.astype(np.uint32), w, gate, up, down, 512, 256)
    assert rel_to_peak(out, ref) <= DECODE_REL


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (3, 3), (16, 5), (40, 40)])
@pytest.mark.parametrize("geom", ["small", "model"])
def test_shared_expert_matches_expert_mlp(oracle, X, max_tokens, tokens, geom):
    # moe_differential.rs:854-986 (SHARED_GATE 5e-6 on that tensor's scale)
    import torch

    H, I = (512, 256) if geom == "small" else (2048, 512)
    g = X.MoeGeometry(8, 2, H, I, 32, max_tokens)
    layer = make_layer(oracle, g, seed=302)
    x = activations(14, max_tokens, H, tokens)
    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    out = torch.zeros(max_tokens, H, device="cuda")
    k.shared_expert(b, layer.dev.shared_gate, layer.dev.shared_up, layer.dev.shared_down, x, out)
    torch.cuda.synchronize()
    h = layer.host
    sg, su, sd = (oracle.dequantize_row(oracle.Q8_0, m) for m in (h.shared_gate, h.shared_up, h.shared_down))
    got = out.cpu().numpy()
    xs = x.cpu().numpy()
    for t in range(tokens):
        ref = oracle.expert_mlp(sg, su, sd, xs[t], H, I)
        assert rel_to_peak(got[t], ref) <= DECODE_REL, t
    assert np.all(got[tokens:] == 0)


def test_weight_stack_checks(oracle, X):
    # check_stack (kernels/moe.rs:6729-6746)
    import torch

    g = X.MoeGeometry(8, 2, 512, 256, 32, 4)
    layer = make_layer(oracle, g, seed=303)
    k = X.MoeKernels(g)
    b = k.buffers()
    x = activations(1, 4, 512)
    d = layer.dev
    ragged = X.QuantTensor(d.gate_exps.bytes[:-1].clone(), X.ExpertQuant.Q6K)
    with pytest.raises(X.moe.RaggedWeights, match="is not a whole number of 210 B blocks"):
        k.grouped_forward_partial(b, ragged, d.up_exps, d.down_exps, x)
    short = X.QuantTensor(d.gate_exps.bytes[:-210].clone(), X.ExpertQuant.Q6K)
    with pytest.raises(X.moe.WrongElementCount, match="expected 1048576 elements"):
        k.grouped_forward_partial(b, short, d.up_exps, d.down_exps, x)
    with pytest.raises(X.moe.UnsupportedExpertType):
        k.grouped_forward_partial(b, X.QuantTensor(torch.zeros(144 * 4096, dtype=torch.uint8, device="cuda"),
                                                   X.ExpertQuant.Q4K), d.up_exps, d.down_exps, x)
    with pytest.raises(X.moe.BufferLength):
        k.grouped_forward_partial(b, d.gate_exps, d.up_exps, d.down_exps, x[:3])
    so = k.shared_only_buffers(False)
    with pytest.raises(X.moe.SharedOnlyBuffers, match="grouped_forward_partial"):
        k.grouped_forward_partial(so, d.gate_exps, d.up_exps, d.down_exps, x)


@pytest.mark.parametrize("max_tokens,tokens,router_q8,down_q8", [
    (1, 1, True, False), (3, 3, True, False), (3, 3, False, False), (4, 2, True, False), (32, 32, True, False),
    (48, 37, False, False),
    # the shipped layers' layout: gate/up Q6_K, down Q8_0, f32 router
    (3, 3, False, True), (12, 9, False, True), (32, 32, False, True)])
def test_block_matches_oracle(oracle, X, max_tokens, tokens, router_q8, down_q8):
    """Whole block.  Routing contract: the ids are what route_token returns for the device's own logits
    (the reference's method, crates/xabe-engine/tests/moe_block.rs:1012-1016); logits vs the sequential
    gemv at reassociation tolerance; block outputs at DECODE_REL of peak."""
    g = X.MoeGeometry.qwen3_6(32, max_tokens)
    layer = make_layer(oracle, g, seed=700, router_q8=router_q8, down_quant=X.ExpertQuant.Q8_0 if down_q8 else None)
    x = activations(15, max_tokens, 2048, tokens)
    blk = X.MoeBlock(g)
    ffn_out, l_out = run_block(blk, layer, x, tokens)
    xs = x.cpu().numpy()[:tokens]
    dev_logits = blk.router_logits().cpu().numpy().reshape(max_tokens, 256)[:tokens]
    ref = oracle.moe_block_forward(layer.host, xs, logits_override=dev_logits, threads=8)
    own = oracle.moe_block_forward(layer.host, xs, threads=8)
    # logits against the oracle's own router GEMV
    assert rel_to_peak(dev_logits, own.logits) <= DECODE_REL
    b = blk.buffers()
    ids = b.topk_ids().cpu().numpy().reshape(max_tokens, 8)[:tokens]
    assert np.array_equal(ids, ref.topk_ids.astype(np.int32))
    assert np.abs(b.topk_weights().cpu().numpy().reshape(max_tokens, 8)[:tokens] - ref.topk_weights).max() <= 2e-7
    take = lambda t, n=2048: t.cpu().numpy().reshape(max_tokens, n)[:tokens]
    assert rel_to_peak(take(blk.normed()), ref.normed) <= 2e-6
    for name, got, want in (("routed", take(blk.routed()), ref.routed), ("shexp", take(blk.shared_ungated()), ref.shexp),
                            ("ffn_out", take(ffn_out), ref.ffn_out), ("l_out", take(l_out), ref.l_out)):
        r = oracle.compare(got, want)
        assert rel_to_peak(got, want) <= DECODE_REL and r.cosine_similarity >= DECODE_COS, (name, str(r))
    assert np.abs(blk.shared_gate().cpu().numpy()[:tokens] - ref.gate).max() <= 1e-6
    # algebraic self-checks of the composition (block/moe.rs:27-51, :1042-1050)
    assert np.array_equal(take(l_out), take(ffn_out) + xs)                       # residual is the un-normed input
    assert np.all(take(l_out)[tokens:] == 0) if tokens < max_tokens else True
    assert np.all(l_out.cpu().numpy()[tokens:] == 0) and np.all(ffn_out.cpu().numpy()[tokens:] == 0)
    # when the device and the oracle route identically the block agrees with the oracle end to end
    if np.array_equal(own.topk_ids, ref.topk_ids):
        assert rel_to_peak(take(l_out), own.l_out) <= DECODE_REL


def test_block_error_paths(oracle, X):
    import torch

    g = X.MoeGeometry(8, 2, 512, 256, 32, 4)
    layer = make_layer(oracle, g, seed=304)
    blk = X.MoeBlock(g)
    x = activations(1, 4, 512)
    with pytest.raises(X.moe.TooManyTokens):
        blk.forward(layer.dev, x, 5, torch.zeros_like(x), torch.zeros_like(x))
    with pytest.raises(X.moe.BufferLength, match="residual"):
        blk.forward(layer.dev, x[:3], 3, torch.zeros_like(x), torch.zeros_like(x))
    with pytest.raises(X.moe.BufferLength, match="l_out"):
        blk.forward(layer.dev, x, 3, torch.zeros_like(x), torch.zeros_like(x)[:2])


@pytest.mark.parametrize("max_tokens,tokens", [(1, 1), (2, 2), (3, 3), (4, 4), (4, 1)])
def test_fused_shared_is_bit_identical_to_separate_launches(oracle, X, max_tokens, tokens):
    # crates/xabe-engine/tests/moe_fused_shared_differential.rs:1-20: widths 1..4, full and one live token
    import torch

    g = X.MoeGeometry.qwen3_6(32, max_tokens)
    layer = make_layer(oracle, g, seed=720)
    d = layer.dev
    x = activations(41, max_tokens, 2048, tokens)
    rng = np.random.default_rng(max_tokens * 10 + tokens)
    logits = torch.from_numpy(rng.uniform(-8, 8, (max_tokens, 256)).astype(np.float32)).cuda()
    outs = []
    for fused in (True, False):
        k = X.MoeKernels(g)
        b = k.buffers()
        k.set_valid_tokens(b, tokens)
        k.route_and_dispatch(b, logits)
        sh = torch.zeros(max_tokens, 2048, device="cuda")
        if fused:
            assert k.grouped_forward_partial_with_shared(b, d.gate_exps, d.up_exps, d.down_exps, d.shared_gate,
                                                         d.shared_up, d.shared_down, x, sh)
        else:
            k.grouped_forward_partial(b, d.gate_exps, d.up_exps, d.down_exps, x)
            k.shared_expert(b, d.shared_gate, d.shared_up, d.shared_down, x, sh)
        torch.cuda.synchronize()
        outs.append((b.partial().cpu().numpy()[: tokens * 8 * 2048].copy(), sh.cpu().numpy().copy(),
                     b.shared_inter().cpu().numpy()[: tokens * 512].copy()))
    for a, c in zip(outs[0], outs[1]):
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    # not covered above the decode width: nothing is launched, the caller takes the separate paths
    g8 = X.MoeGeometry.qwen3_6(32, 8)
    k8 = X.MoeKernels(g8)
    b8 = k8.buffers()
    x8 = activations(42, 8, 2048)
    sh8 = torch.zeros(8, 2048, device="cuda")
    assert not k8.grouped_forward_partial_with_shared(b8, d.gate_exps, d.up_exps, d.down_exps, d.shared_gate, d.shared_up,
                                                      d.shared_down, x8, sh8)
    assert torch.all(sh8 == 0)


@pytest.mark.parametrize("geom,max_tokens,tokens", [("model", 8, 8), ("model", 32, 29), ("model", 40, 37), ("small", 40, 40), ("small", 5, 5)])
def test_weights_resident_dispatch_kernel_equals_the_plain_one(oracle, X, geom, max_tokens, tokens):
    # the dispatch-table regime (up to 63 tokens) keeps a tile's weights in registers across the block's token
    # chunks; force_community selects the plain per-chunk kernel: same bits, both stages
    import torch

    if geom == "model":
        g = X.MoeGeometry.qwen3_6(X.moe_block_size(max_tokens), max_tokens)
    else:
        g = X.MoeGeometry(8, 2, 512, 256, 32, max_tokens)  # few experts: long runs, several chunks per block
    layer = make_layer(oracle, g, seed=733)
    x = activations(44, max_tokens, g.hidden, tokens)
    r = oracle.Xorshift64Star(0xB22 + tokens)
    logits = np.stack([r.vec_f32(g.num_experts, -8.0, 8.0) for _ in range(tokens)])
    outs = []
    for plain in (False, True):
        k = X.MoeKernels(g)
        k.force_community(plain)
        b = k.buffers()
        k.set_valid_tokens(b, tokens)
        lg = torch.zeros(max_tokens, g.num_experts, device="cuda")
        lg[:tokens] = torch.from_numpy(logits).cuda()
        k.route_and_dispatch(b, lg)
        d = layer.dev
        k.grouped_forward_partial(b, d.gate_exps, d.up_exps, d.down_exps, x)
        torch.cuda.synchronize()
        outs.append(b.partial().cpu().numpy().copy())
    assert outs[0].any()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))

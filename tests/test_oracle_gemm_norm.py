"""Oracle pins: norm.rs, gemv.rs, moe/gemm.rs, compare.rs, and the block composition."""
import numpy as np
import pytest


def test_rms_norm_hand_values(oracle):
    # norm.rs:152-194
    out = oracle.rms_norm([3.0, 4.0], [1.0, 1.0], 0.0)
    assert np.allclose(out, np.array([3.0, 4.0]) / np.sqrt(12.5), atol=1e-6)
    assert np.allclose(oracle.rms_norm([1.0, 1.0], [2.0, 0.5], 0.0), [2.0, 0.5], atol=1e-6)
    z = oracle.rms_norm([0.0, 0.0, 0.0], [1.0, 1.0, 1.0], 1e-6)
    assert np.all(z == 0.0)
    x = oracle.Xorshift64Star(11).vec_f32(128, -3.0, 3.0)
    out = oracle.rms_norm(x, np.ones(128, np.float32), 1e-6)
    assert abs(np.sqrt((out.astype(np.float64) ** 2).mean()) - 1.0) < 1e-3
    ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-6)
    assert np.abs(out - ref).max() < 1e-6


def test_rms_norm_operation_order(oracle):
    """y = (x * inv_rms) * w with inv_rms = 1/sqrt(sum/n + eps), each step rounded to f32."""
    x = oracle.Xorshift64Star(5).vec_f32(2048, -2.0, 2.0)
    w = oracle.Xorshift64Star(6).vec_f32(2048, 0.5, 1.5)
    s = np.float32(0.0)
    for v in x:
        s = np.float32(s + np.float32(v * v))
    inv = np.float32(1.0) / np.sqrt(np.float32(s / np.float32(2048) + np.float32(1e-6)), dtype=np.float32)
    ref = (x * inv).astype(np.float32) * w
    assert np.array_equal(oracle.rms_norm(x, w, 1e-6), ref)


def test_silu_sigmoid(oracle):
    # norm.rs:197-246
    assert oracle.silu(0.0) == 0.0 and abs(oracle.silu(10.0) - 10.0) < 1e-3 and abs(oracle.silu(-10.0)) < 1e-3
    assert oracle.sigmoid(0.0) == 0.5
    assert abs(oracle.sigmoid(20.0) - 1.0) < 1e-6 and abs(oracle.sigmoid(-20.0)) < 1e-6
    for x in (-8.0, -1.5, 0.25, 3.0, 11.0):
        assert abs(1.0 - oracle.sigmoid(x) - oracle.sigmoid(-x)) < 1e-6
    for x in (-3.0, -0.5, 0.7, 4.25):
        e = np.exp(np.float32(-x), dtype=np.float32)
        assert abs(oracle.sigmoid(x) - float(np.float32(1.0) / (np.float32(1.0) + e))) <= 6e-8
        assert abs(oracle.silu(x) - x / (1.0 + np.exp(-x))) < 1e-6
    # silu is x/(1+exp(-x)), not x*sigmoid(x): they differ in the last bit somewhere
    xs = oracle.Xorshift64Star(21).vec_f32(4096, -6.0, 6.0)
    a = np.array([oracle.silu(float(v)) for v in xs], np.float32)
    b = np.array([np.float32(v) * np.float32(oracle.sigmoid(float(v))) for v in xs], np.float32)
    assert np.any(a != b) and np.abs(a - b).max() < 1e-6


def test_swiglu_gates_residual(oracle):
    # norm.rs:204-226, 292-351
    assert np.all(oracle.swiglu([0.0, 0.0], [5.0, -5.0]) == 0.0)
    g = oracle.Xorshift64Star(21).vec_f32(64, -2.0, 2.0)
    u = oracle.Xorshift64Star(22).vec_f32(64, -2.0, 2.0)
    ref = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))) * u
    assert np.abs(oracle.swiglu(g, u) - ref).max() < 1e-6
    assert np.array_equal(oracle.sigmoid_gate([4.0, -6.0], [0.0, 0.0]), np.array([2.0, -3.0], np.float32))
    o = oracle.sigmoid_gate([1.0, 1.0], [30.0, -30.0])
    assert abs(o[0] - 1.0) < 1e-6 and abs(o[1]) < 1e-6
    assert abs(oracle.sigmoid_gate([2.0], [3.0])[0] - oracle.swiglu([3.0], [2.0])[0]) > 1.0
    assert np.array_equal(oracle.residual_add([1.0, -2.0, 3.5], [0.5, 2.0, -3.5]), np.array([1.5, 0, 0], np.float32))


def test_gemv_reference_vectors(oracle):
    # gemv.rs:119-127
    assert oracle.gemv([1, 2, 3, 4, 5, 6], 2, 3, [1.0, 10.0, 100.0]).tolist() == [321.0, 654.0]
    # gemv.rs:185-200: sequential f32 accumulator, not f64
    x = np.ones(8, np.float32)
    x[0] = 16777216.0
    assert oracle.gemv(np.ones(8, np.float32), 1, 8, x)[0] == 16777216.0
    # gemv.rs:175-181
    assert oracle.argmax([1.0, 3.0, 2.0]) == 1 and oracle.argmax([3.0, 3.0, 3.0]) == 0
    assert oracle.argmax([-5.0]) == 0 and oracle.argmax([-3.0, -1.0, -2.0]) == 1
    # order: ascending index, multiply and add rounded separately
    w = oracle.Xorshift64Star(0x6E110002).vec_f32(96, -2.0, 2.0)
    v = oracle.Xorshift64Star(77).vec_f32(96, -2.0, 2.0)
    s = np.float32(0.0)
    for a, b in zip(w, v):
        s = np.float32(s + np.float32(a * b))
    assert oracle.gemv(w, 1, 96, v)[0] == s


def _random_experts(oracle, rng, n, hidden, inter):
    g = np.stack([rng.vec_f32(inter * hidden, -0.3, 0.3) for _ in range(0)] or [np.zeros(0, np.float32)])
    gate, up, down = [], [], []
    for _ in range(n):
        gate.append(rng.vec_f32(inter * hidden, -0.3, 0.3))
        up.append(rng.vec_f32(inter * hidden, -0.3, 0.3))
        down.append(rng.vec_f32(hidden * inter, -0.3, 0.3))
    return np.stack(gate), np.stack(up), np.stack(down)


def test_grouped_matches_naive(oracle):
    # gemm.rs:154-196 (same seed, shapes and draw order)
    rng = oracle.Xorshift64Star(2025)
    T, E, K, H, I, B = 23, 16, 4, 12, 20, 8
    gate, up, down = _random_experts(oracle, rng, E, H, I)
    hs = np.stack([rng.vec_f32(H, -1.0, 1.0) for _ in range(T)])
    logits = np.stack([rng.vec_f32(E, -3.0, 3.0) for _ in range(T)])
    ids, w = oracle.route_batch(logits, K)
    d = oracle.moe_align_block_size(ids, B, E)
    grouped = oracle.grouped_forward(hs, d, B, w.ravel(), K, gate, up, down, H, I)
    naive = oracle.naive_forward(hs, ids, w, gate, up, down, H, I)
    r = oracle.compare(grouped, naive)
    assert r.max_abs_error < 1e-3 and r.cosine_similarity > 1 - 1e-5, str(r)
    # float64 textbook bound
    ref = np.zeros((T, H))
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            G = gate[e].reshape(I, H).astype(np.float64) @ hs[t]
            U = up[e].reshape(I, H).astype(np.float64) @ hs[t]
            A = G / (1 + np.exp(-G)) * U
            ref[t] += w[t, k] * (down[e].reshape(H, I).astype(np.float64) @ A)
    assert np.abs(naive - ref).max() < 1e-4 * max(1.0, np.abs(ref).max())


def test_single_expert_reduces_to_expert_mlp_and_zero_weight(oracle):
    # gemm.rs:198-241
    rng = oracle.Xorshift64Star(2026)
    H, I, T, E = 6, 10, 5, 3
    gate, up, down = _random_experts(oracle, rng, E, H, I)
    hs = np.stack([rng.vec_f32(H, -1.0, 1.0) for _ in range(T)])
    ids = np.zeros((T, 1), np.uint32)
    w = np.ones((T, 1), np.float32)
    d = oracle.moe_align_block_size(ids, 4, E)
    grouped = oracle.grouped_forward(hs, d, 4, w.ravel(), 1, gate, up, down, H, I)
    naive = oracle.naive_forward(hs, ids, w, gate, up, down, H, I)
    for t in range(T):
        direct = oracle.expert_mlp(gate[0], up[0], down[0], hs[t], H, I)
        assert oracle.compare(grouped[t], direct).max_abs_error < 1e-4
        assert oracle.compare(naive[t], direct).max_abs_error < 1e-4
    # gemm.rs:243-266
    H, I = 4, 6
    one = np.ones(H * I, np.float32)
    full = oracle.expert_mlp(one, one, one, np.ones(H, np.float32), H, I)
    assert np.any(full != 0)
    out = oracle.naive_forward(np.ones((1, H), np.float32), np.zeros((1, 1), np.uint32), np.zeros((1, 1), np.float32),
                               one[None], one[None], one[None], H, I)
    assert np.all(out == 0.0)


def test_compare_harness(oracle):
    # compare.rs:285-397 style
    a = np.array([1.0, 2.0, 3.0], np.float32)
    r = oracle.compare(a, a)
    assert r.max_abs_error == 0 and r.cosine_similarity == 1.0 and r.non_finite_count == 0
    r = oracle.compare(a * 0.5, a)
    assert abs(r.cosine_similarity - 1.0) < 1e-6 and r.max_abs_error == 1.5 and r.max_abs_error_index == 2
    r = oracle.compare(np.array([np.nan, 1.0], np.float32), np.array([0.0, 1.0], np.float32))
    assert r.non_finite_count == 1
    r = oracle.compare(np.zeros(3, np.float32), np.zeros(3, np.float32))
    assert r.cosine_similarity == 1.0
    r = oracle.compare(np.array([1e-9], np.float32), np.array([0.0], np.float32))
    assert abs(r.max_rel_error - 1e-3) < 1e-6       # REL_EPS = 1e-6 guards the ratio
    with pytest.raises(ValueError):
        oracle.compare(np.zeros(0, np.float32), np.zeros(0, np.float32))


def _tiny_weights(oracle, E=8, K=2, H=512, I=256, seed=100, router_q8=True):
    n = E * I * H
    W = oracle.MoeWeights(
        num_experts=E, top_k=K, hidden=H, intermediate=I, eps=1e-6,
        post_norm=np.ones(H, np.float32) + oracle.synth_normal_f32(seed + 1, H, 0.1),
        router_f32=None if router_q8 else oracle.synth_normal_f32(seed + 2, E * H, 0.02),
        router_q8=oracle.synth_quant(oracle.Q8_0, seed + 2, E * H, 0.02) if router_q8 else None,
        gate_exps=oracle.synth_quant(oracle.Q6K, seed + 3, n, 0.02),
        up_exps=oracle.synth_quant(oracle.Q6K, seed + 4, n, 0.02),
        down_exps=oracle.synth_quant(oracle.Q6K, seed + 5, n, 0.02),
        shared_gate_inp=oracle.synth_normal_f32(seed + 6, H, 0.02),
        shared_gate=oracle.synth_quant(oracle.Q8_0, seed + 7, I * H, 0.02),
        shared_up=oracle.synth_quant(oracle.Q8_0, seed + 8, I * H, 0.02),
        shared_down=oracle.synth_quant(oracle.Q8_0, seed + 9, I * H, 0.02))
    return W


def test_block_composition_algebra(oracle):
    """xabe-engine block/moe.rs:12-51: the gate is one scalar per token and multiplies the shared
    expert only; the residual is the un-normalised input; weights renormalise over the selected set."""
    W = _tiny_weights(oracle)
    x = oracle.synth_normal_f32(1, 5 * 512, 1.0).reshape(5, 512)
    r = oracle.moe_block_forward(W, x)
    assert np.array_equal(r.l_out, r.ffn_out + x)                       # residual taken before the norm
    assert np.array_equal(r.ffn_out, r.routed + r.shexp * r.gate[:, None])
    assert np.allclose(r.topk_weights.sum(1), 1.0, atol=1e-6)
    # parts against the stand-alone oracle functions
    for t in range(5):
        n = oracle.rms_norm(x[t], W.post_norm, 1e-6)
        assert np.array_equal(n, r.normed[t])
        router = oracle.dequantize_row(oracle.Q8_0, W.router_q8)
        lg = oracle.gemv(router, 8, 512, n)
        assert np.array_equal(lg, r.logits[t])
        ids, w = oracle.route_token(lg, 2)
        assert np.array_equal(ids, r.topk_ids[t]) and np.array_equal(w, r.topk_weights[t])
        g = oracle.sigmoid(float(oracle.gemv(W.shared_gate_inp, 1, 512, n)[0]))
        assert np.float32(g) == r.gate[t]
    # routed == naive_forward over the dequantised stacks
    gate = oracle.dequantize_row(oracle.Q6K, W.gate_exps).reshape(8, -1)
    up = oracle.dequantize_row(oracle.Q6K, W.up_exps).reshape(8, -1)
    down = oracle.dequantize_row(oracle.Q6K, W.down_exps).reshape(8, -1)
    naive = oracle.naive_forward(r.normed, r.topk_ids, r.topk_weights, gate, up, down, 512, 256)
    assert np.array_equal(naive, r.routed)
    sh = oracle.expert_mlp(oracle.dequantize_row(oracle.Q8_0, W.shared_gate), oracle.dequantize_row(oracle.Q8_0, W.shared_up),
                           oracle.dequantize_row(oracle.Q8_0, W.shared_down), r.normed[2], 512, 256)
    assert np.array_equal(sh, r.shexp[2])
    # threads > 1 is the same arithmetic
    r2 = oracle.moe_block_forward(W, x, threads=4)
    assert np.array_equal(r2.l_out, r.l_out)
    # override + bias plumbing
    r3 = oracle.moe_block_forward(W, x, logits_override=r.logits)
    assert np.array_equal(r3.l_out, r.l_out)
    bias = np.zeros(8, np.float32)
    bias[5] = 100.0
    r4 = oracle.moe_block_forward(W, x, logit_bias=bias)
    assert np.all(r4.topk_ids[:, 0] == 5)


def test_block_float64_bound(oracle):
    W = _tiny_weights(oracle, router_q8=False)
    x = oracle.synth_normal_f32(2, 3 * 512, 1.0).reshape(3, 512)
    r = oracle.moe_block_forward(W, x)
    gate = oracle.dequantize_row(oracle.Q6K, W.gate_exps).reshape(8, 256, 512).astype(np.float64)
    up = oracle.dequantize_row(oracle.Q6K, W.up_exps).reshape(8, 256, 512).astype(np.float64)
    down = oracle.dequantize_row(oracle.Q6K, W.down_exps).reshape(8, 512, 256).astype(np.float64)
    sg = oracle.dequantize_row(oracle.Q8_0, W.shared_gate).reshape(256, 512).astype(np.float64)
    su = oracle.dequantize_row(oracle.Q8_0, W.shared_up).reshape(256, 512).astype(np.float64)
    sd = oracle.dequantize_row(oracle.Q8_0, W.shared_down).reshape(512, 256).astype(np.float64)
    mlp = lambda g, u, d, v: d @ ((g @ v) / (1 + np.exp(-(g @ v))) * (u @ v))
    for t in range(3):
        xt = x[t].astype(np.float64)
        n = xt / np.sqrt((xt ** 2).mean() + 1e-6) * W.post_norm
        lg = W.router_f32.reshape(8, 512).astype(np.float64) @ n
        p = np.exp(lg - lg.max())
        p /= p.sum()
        top = sorted(range(8), key=lambda i: (-p[i], i))[:2]
        assert top == r.topk_ids[t].tolist()
        wk = p[top] / p[top].sum()
        routed = sum(wk[k] * mlp(gate[e], up[e], down[e], n) for k, e in enumerate(top))
        g = 1 / (1 + np.exp(-(W.shared_gate_inp.astype(np.float64) @ n)))
        ref = routed + mlp(sg, su, sd, n) * g + xt
        assert np.abs(r.l_out[t] - ref).max() < 1e-5


def test_dense_block(oracle):
    H, I = 512, 768
    g = oracle.synth_quant(oracle.Q6K, 21, H * I, 0.02)
    u = oracle.synth_quant(oracle.Q6K, 22, H * I, 0.02)
    d = oracle.synth_quant(oracle.Q6K, 23, H * I, 0.02)
    pn = np.ones(H, np.float32)
    x = oracle.synth_normal_f32(3, 2 * H, 1.0).reshape(2, H)
    normed, ffn, lout = oracle.dense_block_forward(H, I, 1e-6, pn, g, u, d, x)
    assert np.array_equal(lout, ffn + x)
    for t in range(2):
        n = oracle.rms_norm(x[t], pn, 1e-6)
        assert np.array_equal(n, normed[t])
        ref = oracle.expert_mlp(oracle.dequantize_row(oracle.Q6K, g), oracle.dequantize_row(oracle.Q6K, u),
                                oracle.dequantize_row(oracle.Q6K, d), n, H, I)
        assert np.array_equal(ref, ffn[t])
    _, ffn4, _ = oracle.dense_block_forward(H, I, 1e-6, pn, g, u, d, x, threads=4)
    assert np.array_equal(ffn4, ffn)

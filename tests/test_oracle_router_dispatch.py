"""Oracle pins: route_token (K/moe/router.rs:32-81), moe_align_block_size (K/moe/dispatch.rs:60-131),
MoeGeometry capacities (xabe-cuda kernels/moe.rs:4556-4598)."""
import numpy as np
import pytest


def test_router_reference_vectors(oracle):
    # router.rs:88-108
    logits = [0.1, 3.0, -1.0, 2.5, 0.0, 1.0, -2.0, 4.0]
    ids, w = oracle.route_token(logits, 3)
    assert list(ids) == [7, 1, 3]
    assert abs(float(w.sum()) - 1.0) < 1e-5
    # router.rs:111-132 ties -> lower index, stable across calls
    ids, _ = oracle.route_token([1.0, 1.0, 1.0, 1.0], 2)
    assert list(ids) == [0, 1]
    first = oracle.route_token([0.5] * 6, 3)
    for _ in range(10):
        again = oracle.route_token([0.5] * 6, 3)
        assert np.array_equal(first[0], again[0]) and np.array_equal(first[1], again[1])
    assert list(first[0]) == [0, 1, 2]
    # router.rs:135-141
    ids, w = oracle.route_token([5.0, 1.0, 3.0], 3)
    assert list(ids) == [0, 2, 1] and w[0] > w[1] > w[2]
    # router.rs:144-150
    ids, _ = oracle.route_token([1.0, 2.0, 3.0], 3)
    assert sorted(ids) == [0, 1, 2]
    # router.rs:175-181
    ids, _ = oracle.route_batch(np.array([[3.0, 1.0, 2.0], [1.0, 3.0, 2.0]], np.float32), 2)
    assert ids.tolist() == [[0, 2], [1, 2]]
    # router.rs:184-187
    with pytest.raises(ValueError):
        oracle.route_token([1.0, 2.0], 3)
    # all-tie at the model's shape -> experts 0..7 (xabe-engine tests/moe_differential.rs:394-432)
    ids, w = oracle.route_token(np.zeros(256, np.float32), 8)
    assert list(ids) == list(range(8)) and np.allclose(w, 0.125)


def test_router_matches_brute_force_and_float64_softmax(oracle):
    # router.rs:153-172 shape; brute force: full stable sort on (-p, idx)
    logits = oracle.Xorshift64Star(256).vec_f32(256, -10.0, 10.0)
    ids, w = oracle.route_token(logits, 8)
    assert len(set(ids.tolist())) == 8 and abs(float(w.sum()) - 1.0) < 1e-4
    order = sorted(range(256), key=lambda i: (-float(logits[i]), i))[:8]
    assert ids.tolist() == order
    p = np.exp(logits.astype(np.float64) - logits.max())
    p /= p.sum()
    ref = p[order] / p[order].sum()
    assert np.abs(w - ref).max() < 1e-6
    rng = np.random.default_rng(3)
    for _ in range(50):
        lg = rng.uniform(-8, 8, 256).astype(np.float32)
        ids, _ = oracle.route_token(lg, 8)
        assert ids.tolist() == sorted(range(256), key=lambda i: (-float(lg[i]), i))[:8]


def test_align_vllm_docstring_example(oracle):
    # dispatch.rs:138-169
    topk = [[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]]
    d = oracle.moe_align_block_size(topk, 4, 5)
    S = 12
    assert d.sorted_token_ids.tolist() == [3, 6, 9, S, 0, 4, 10, S, 1, 7, 11, S, 2, 5, 8, S]
    assert d.expert_ids.tolist() == [1, 2, 3, 4]
    assert d.num_tokens_post_pad == 16


def test_align_invariants(oracle):
    # dispatch.rs:172-206: every flat id exactly once at the model's shape
    r = oracle.Xorshift64Star(42)
    topk = np.array([[r.next_u32_below(256) for _ in range(8)] for _ in range(37)], np.uint32)
    d = oracle.moe_align_block_size(topk, 32, 256)
    sent = 37 * 8
    real = d.sorted_token_ids[d.sorted_token_ids != sent]
    assert sorted(real.tolist()) == list(range(sent))
    # dispatch.rs:209-244: each block owned by exactly one expert and holds its tokens
    r = oracle.Xorshift64Star(43)
    topk = np.array([[r.next_u32_below(16) for _ in range(4)] for _ in range(20)], np.uint32)
    d = oracle.moe_align_block_size(topk, 8, 16)
    flat = topk.ravel()
    for b, e in enumerate(d.expert_ids):
        for s in d.sorted_token_ids[b * 8:(b + 1) * 8]:
            if s != 80:
                assert e != -1 and flat[s] == e
    # dispatch.rs:247-256 padding after real tokens
    d = oracle.moe_align_block_size([[0], [0], [1]], 4, 2)
    assert d.sorted_token_ids[2] == 3 and d.sorted_token_ids[3] == 3 and d.sorted_token_ids[5] == 3
    # dispatch.rs:259-266 zero-token experts take no blocks
    d = oracle.moe_align_block_size([[0], [2]], 4, 4)
    assert d.num_tokens_post_pad == 8 and d.expert_ids.tolist() == [0, 2]
    # dispatch.rs:269-279 aligned counts need no padding
    d = oracle.moe_align_block_size([[0], [0], [0], [0]], 4, 1)
    assert d.num_tokens_post_pad == 4 and np.all(d.sorted_token_ids != 4)
    # dispatch.rs:282-291
    with pytest.raises(ValueError):
        oracle.moe_align_block_size([[0]], 0, 1)
    with pytest.raises(ValueError):
        oracle.moe_align_block_size([[5]], 4, 4)


def test_align_brute_force(oracle):
    rng = np.random.default_rng(0)
    for _ in range(30):
        T, K, E, B = rng.integers(1, 9), rng.integers(1, 4), rng.integers(2, 7), rng.integers(1, 5)
        topk = rng.integers(0, E, (T, K)).astype(np.uint32)
        d = oracle.moe_align_block_size(topk, int(B), int(E))
        exp_sorted, exp_ids = [], []
        for e in range(E):
            mine = [i for i, v in enumerate(topk.ravel()) if v == e]
            if not mine:
                continue
            pad = (-len(mine)) % B
            exp_sorted += mine + [T * K] * pad
            exp_ids += [e] * ((len(mine) + pad) // B)
        assert d.sorted_token_ids.tolist() == exp_sorted and d.expert_ids.tolist() == exp_ids


def test_geometry_capacities(oracle):
    # xabe-cuda kernels/moe.rs:6981-6989: qwen3_6(16, 64)
    assert oracle.lib().xo_max_flat_pairs(64, 8) == 512
    assert oracle.sorted_capacity(256, 8, 16, 64) == 4352
    assert oracle.expert_block_capacity(256, 8, 16, 64) == 272
    # moe.rs:6921-6923: qwen3_6(16, 32768)
    assert oracle.sorted_capacity(256, 8, 16, 32768) == 265984
    assert oracle.expert_block_capacity(256, 8, 16, 32768) == 16624
    # moe.rs:6995-7022: brute force on a 4-expert geometry: the bound holds for every routing
    E, K, B, T = 4, 2, 3, 3
    cap = oracle.sorted_capacity(E, K, B, T)
    import itertools
    worst = 0
    pairs = [c for c in itertools.permutations(range(E), K)]
    for combo in itertools.product(pairs, repeat=T):
        d = oracle.moe_align_block_size(np.array(combo, np.uint32), B, E)
        worst = max(worst, d.num_tokens_post_pad)
    assert worst <= cap and cap % B == 0

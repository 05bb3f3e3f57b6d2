"""GPU parity: stand-alone dequant (bit-identical), the synthetic generator (bit-identical), RMSNorm,
routing (ids exact) and the dispatch tables (exact), each against the CPU oracle through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def X():
    import torch
    import llmxabe_amd as X

    assert torch.cuda.is_available()
    return X


def test_dequant_is_bit_identical(oracle, X):
    # crates/xabe-engine/tests/dequant_differential.rs:77-97: 8192 superblocks per tensor, to_bits equality
    import torch

    rng = np.random.default_rng(0)
    raw = rng.integers(0, 256, 210 * 8192, dtype=np.uint8)
    raw.reshape(-1, 210)[:, 208:210] = (rng.standard_normal(8192) * 0.01).astype(np.float16).view(np.uint8).reshape(-1, 2)
    got = X.dequantize(X.ExpertQuant.Q6K, torch.from_numpy(raw).cuda()).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.dequantize_row(oracle.Q6K, raw).view(np.uint32))
    raw8 = rng.integers(0, 256, 34 * 8192 * 8, dtype=np.uint8)
    raw8.reshape(-1, 34)[:, 0:2] = (rng.standard_normal(8192 * 8) * 0.01).astype(np.float16).view(np.uint8).reshape(-1, 2)
    got = X.dequantize(X.ExpertQuant.Q8_0, torch.from_numpy(raw8).cuda()).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.dequantize_row(oracle.Q8_0, raw8).view(np.uint32))
    with pytest.raises(X.moe.RaggedWeights):
        X.dequantize(X.ExpertQuant.Q6K, torch.zeros(211, dtype=torch.uint8, device="cuda"))


def test_synth_generator_matches_oracle_bit_for_bit(oracle, X):
    n = 256 * 4096
    for sigma in (0.02, 1.0):
        a = X.synth_normal_f32(77, n, sigma).cpu().numpy()
        assert np.array_equal(a.view(np.uint32), oracle.synth_normal_f32(77, n, sigma).view(np.uint32))
    q6 = X.synth_quant(X.ExpertQuant.Q6K, 78, n, 0.02).cpu().numpy()
    assert np.array_equal(q6, oracle.synth_quant(oracle.Q6K, 78, n, 0.02))
    q8 = X.synth_quant(X.ExpertQuant.Q8_0, 79, n, 0.02).cpu().numpy()
    assert np.array_equal(q8, oracle.synth_quant(oracle.Q8_0, 79, n, 0.02))
    assert np.array_equal(X.synth_normal_f32(5, 300, 1.0).cpu().numpy(), oracle.synth_normal_f32(5, 300, 1.0))


def test_rms_norm_rows(oracle, X):
    import torch

    rows, width = 7, 2048
    x = X.synth_normal_f32(3, rows * width, 1.0).view(rows, width)
    x[5] = 0  # a zero row normalises to zero, not NaN
    w = 1.0 + X.synth_normal_f32(4, width, 0.1)
    out = torch.empty_like(x)
    X.LayerOpsKernels.rms_norm(x, w, out, rows, width, 1e-6)
    got = out.cpu().numpy()
    xn, wn = x.cpu().numpy(), w.cpu().numpy()
    for r in range(rows):
        ref = oracle.rms_norm(xn[r], wn, 1e-6)
        # fp32 reassociation of the sum of squares only: 2e-6 relative
        assert np.abs(got[r] - ref).max() <= 2e-6 * max(1.0, np.abs(ref).max()), r
    assert np.all(got[5] == 0)
    with pytest.raises(X.moe.BufferLength):
        X.LayerOpsKernels.rms_norm(x, w[:-1], out, rows, width, 1e-6)


@pytest.mark.parametrize("rows,width", [(130, 2048), (64, 512), (67, 1000)])
def test_rms_norm_short_rows_are_the_long_form_s_bits(oracle, X, rows, width):
    """From 64 rows of at most 2048 elements one wavefront normalises a row, fetched and stored as consecutive
    16-byte pieces through LDS; below that one workgroup does.  Both fold the row in the same order."""
    import torch

    x = X.synth_normal_f32(13, rows * width, 1.0).view(rows, width)
    x[3] = 0
    w = 1.0 + X.synth_normal_f32(14, width, 0.1)
    out = torch.empty_like(x)
    X.LayerOpsKernels.rms_norm(x, w, out, rows, width, 1e-6)
    few = torch.empty(9, width, device="cuda")
    X.LayerOpsKernels.rms_norm(x[:9].contiguous(), w, few, 9, width, 1e-6)
    got, ref9 = out.cpu().numpy(), few.cpu().numpy()
    assert np.array_equal(got[:9].view(np.uint32), ref9.view(np.uint32))
    xn, wn = x.cpu().numpy(), w.cpu().numpy()
    for r in (0, 3, rows - 1):
        ref = oracle.rms_norm(xn[r], wn, 1e-6)
        assert np.abs(got[r] - ref).max() <= 2e-6 * max(1.0, np.abs(ref).max()), r


def _route(X, logits_np, max_tokens, tokens, E=256, K=8, block=32):
    import torch

    g = X.MoeGeometry(E, K, 2048, 512, block, max_tokens)
    k = X.MoeKernels(g)
    b = k.buffers()
    k.set_valid_tokens(b, tokens)
    buf = np.zeros((max_tokens, E), np.float32)
    buf[:tokens] = logits_np
    k.route(b, torch.from_numpy(buf).cuda())
    torch.cuda.synchronize()
    return k, b, g


def test_route_ids_are_exact(oracle, X):
    # crates/xabe-engine/tests/moe_differential.rs:314-392: uniform(-8,8), 37 tokens in a 64-token buffer
    r = oracle.Xorshift64Star(0x5EED)
    logits = np.stack([r.vec_f32(256, -8.0, 8.0) for _ in range(37)])
    k, b, g = _route(X, logits, 64, 37)
    ids = b.topk_ids().cpu().numpy().reshape(64, 8)
    w = b.topk_weights().cpu().numpy().reshape(64, 8)
    ref_ids, ref_w = oracle.route_batch(logits, 8)
    assert np.array_equal(ids[:37], ref_ids.astype(np.int32))
    # weights: same arithmetic as the oracle (sequential sums, one division): equal or 1 ulp (exp rounding)
    assert np.abs(w[:37] - ref_w).max() <= 1.2e-7
    assert np.abs(w[:37].sum(1) - 1.0).max() < 1e-6
    assert np.all(ids[37:] == 0) and np.all(w[37:] == 0)  # rows past `tokens` are never written


def test_route_all_tie_selects_lowest_indices(oracle, X):
    # moe_differential.rs:394-432
    for _ in range(3):
        k, b, g = _route(X, np.zeros((5, 256), np.float32), 8, 5)
        ids = b.topk_ids().cpu().numpy().reshape(8, 8)
        assert np.array_equal(ids[:5], np.tile(np.arange(8, dtype=np.int32), (5, 1)))
        assert np.allclose(b.topk_weights().cpu().numpy().reshape(8, 8)[:5], 0.125)


def _near_tie_logits(rows=6, seed=21):
    """Logits whose order disagrees with (probability desc, index asc): pairs one ulp apart, the larger at the
    HIGHER index, far enough below the row maximum that l - max rounds both to the same value.  One pair sits
    inside the top 8, one straddles ranks 8 and 9 (the reference keeps the lower index of each)."""
    rng = np.random.default_rng(seed)
    logits = rng.uniform(-8.0, -1.0, (rows, 256)).astype(np.float32)
    for r in range(rows):
        logits[r, 50 + r] = 5.0
        logits[r, 10], logits[r, 200] = 0.001, np.nextafter(np.float32(0.001), np.float32(1))
        logits[r, 120:124] = (-0.1, -0.2, -0.3, -0.4)
        logits[r, 30], logits[r, 220] = -0.5, np.nextafter(np.float32(-0.5), np.float32(0))
    return logits


def test_route_near_ties_fall_back_to_the_probability_order(oracle, X):
    logits = _near_tie_logits()
    ref_ids, ref_w = oracle.route_batch(logits, 8)
    # the construction does what it says: ranking by logit alone would pick 200 before 10, and 220 not 30
    assert list(ref_ids[0][:3]) == [50, 10, 200] and ref_ids[0][7] == 30 and 220 not in ref_ids[0]
    k, b, g = _route(X, logits, 8, 6)
    ids = b.topk_ids().cpu().numpy().reshape(8, 8)
    w = b.topk_weights().cpu().numpy().reshape(8, 8)
    assert np.array_equal(ids[:6], ref_ids.astype(np.int32))
    assert np.abs(w[:6] - ref_w).max() <= 1.2e-7


def test_route_many_tokens_and_extreme_logits(oracle, X):
    rng = np.random.default_rng(9)
    logits = (rng.standard_normal((512, 256)) * 3).astype(np.float32)
    logits[7, 100] = 200.0          # one dominant expert: the rest underflow to p = 0 and tie by index
    logits[8, :] = -1e30
    k, b, g = _route(X, logits, 512, 512)
    ids = b.topk_ids().cpu().numpy().reshape(512, 8)
    ref_ids, ref_w = oracle.route_batch(logits, 8)
    assert np.array_equal(ids, ref_ids.astype(np.int32))
    w = b.topk_weights().cpu().numpy().reshape(512, 8)
    assert np.abs(w - ref_w).max() <= 2e-7


def test_route_small_expert_counts(oracle, X):
    rng = np.random.default_rng(10)
    for E, K in ((8, 2), (64, 4), (128, 8), (512, 8)):
        logits = rng.uniform(-4, 4, (9, E)).astype(np.float32)
        k, b, g = _route(X, logits, 16, 9, E=E, K=K)
        ids = b.topk_ids().cpu().numpy().reshape(16, K)
        assert np.array_equal(ids[:9], oracle.route_batch(logits, K)[0].astype(np.int32)), (E, K)


@pytest.mark.parametrize("tokens,max_tokens,block", [(37, 64, 32), (5, 8, 32), (200, 256, 32), (1500, 1536, 64),
                                                     (8192, 8192, 64), (700, 8192, 64), (1025, 2048, 64),
                                                     # the one-launch form at and just under its 8192 selections
                                                     (1024, 1024, 32), (1001, 1024, 32), (513, 1024, 64),
                                                     # more chunks than the offsets kernel keeps in registers
                                                     (12000, 16384, 64)])
def test_dispatch_tables_are_exact(oracle, X, tokens, max_tokens, block):
    # moe_differential.rs:438-543: exact incl. padding, sentinel and -1 fill over the whole capacity
    r = oracle.Xorshift64Star(0xD15 + tokens)
    logits = np.stack([r.vec_f32(256, -8.0, 8.0) for _ in range(tokens)])
    k, b, g = _route(X, logits, max_tokens, tokens, block=block)
    k.build_dispatch(b)
    import torch

    torch.cuda.synchronize()
    ids = b.topk_ids().cpu().numpy().reshape(max_tokens, 8)[:tokens]
    d = oracle.moe_align_block_size(ids.astype(np.uint32), block, 256)
    sorted_ids = b.sorted_token_ids().cpu().numpy()
    expert_ids = b.expert_ids().cpu().numpy()
    assert sorted_ids.size == g.sorted_capacity() and expert_ids.size == g.expert_block_capacity()
    n = d.num_tokens_post_pad
    assert int(b.num_tokens_post_pad().cpu().numpy()[0]) == n
    assert np.array_equal(sorted_ids[:n], d.sorted_token_ids.astype(np.int32))
    assert np.all(sorted_ids[n:] == tokens * 8)                     # sentinel = valid * top_k
    assert np.array_equal(expert_ids[: n // block], d.expert_ids)
    assert np.all(expert_ids[n // block:] == -1)
    live = b.bucket_live().cpu().numpy()
    exp_live = (d.sorted_token_ids.reshape(-1, block) != tokens * 8).sum(1)
    assert np.array_equal(live[: n // block], exp_live) and np.all(live[n // block:] == 0)


def test_dispatch_collisions_all_tokens_one_expert(oracle, X):
    logits = np.zeros((40, 256), np.float32)
    logits[:, 200:208] = 5.0
    k, b, g = _route(X, logits, 64, 40)
    k.build_dispatch(b)
    ids = b.topk_ids().cpu().numpy().reshape(64, 8)[:40]
    d = oracle.moe_align_block_size(ids.astype(np.uint32), 32, 256)
    n = d.num_tokens_post_pad
    assert np.array_equal(b.sorted_token_ids().cpu().numpy()[:n], d.sorted_token_ids.astype(np.int32))
    assert np.array_equal(b.expert_ids().cpu().numpy()[: n // 32], d.expert_ids)


def test_dispatch_collisions_at_prefill_width(oracle, X):
    # the counting-sort form of the tables (8192 selections and up): every token to the same eight experts,
    # so each expert's run spans every chunk and every wavefront of the placement
    logits = np.zeros((3000, 256), np.float32)
    logits[:, 100:108] = 5.0
    k, b, g = _route(X, logits, 4096, 3000, block=64)
    k.build_dispatch(b)
    ids = b.topk_ids().cpu().numpy().reshape(4096, 8)[:3000]
    d = oracle.moe_align_block_size(ids.astype(np.uint32), 64, 256)
    n = d.num_tokens_post_pad
    assert int(b.num_tokens_post_pad().cpu().numpy()[0]) == n
    assert np.array_equal(b.sorted_token_ids().cpu().numpy()[:n], d.sorted_token_ids.astype(np.int32))
    assert np.array_equal(b.expert_ids().cpu().numpy()[: n // 64], d.expert_ids)


def test_geometry_and_error_paths(X):
    # kernels/moe.rs:5043-5111: same rules, same reasons
    G = X.MoeGeometry
    bad = [(G(256, 8, 2048, 512, 0, 4), "block_size must be non-zero"),
           (G(256, 0, 2048, 512, 32, 4), "experts_per_token must be non-zero"),
           (G(4, 8, 2048, 512, 32, 4), "experts_per_token must not exceed num_experts"),
           (G(256, 8, 2048, 512, 32, 0), "max_tokens must be non-zero"),
           (G(256, 8, 2000, 512, 32, 4), "hidden must be a multiple of the 128-element tile"),
           (G(256, 8, 2048, 500, 32, 4), "intermediate must be a multiple of the 128-element tile"),
           (G(256, 8, 2048, 512, 128, 4), "block_size exceeds the slots the tensor-core tile stages"),
           (G(256, 8, 2048, 512, 32, 70000), "max_tokens exceeds the 65535 grid limit")]
    for g, reason in bad:
        with pytest.raises(X.moe.UnsupportedGeometry, match=reason):
            X.MoeKernels(g)
    k = X.MoeKernels(G.qwen3_6(32, 4))
    b = k.buffers()
    with pytest.raises(X.moe.TooManyTokens, match="5 tokens exceeds the 4"):
        k.set_valid_tokens(b, 5)
    so = k.shared_only_buffers(False)
    assert so.scope() == X.BufferScope.SharedOnly and so.topk_ids().numel() == 0 and so.partial().numel() == 0
    import torch

    with pytest.raises(X.moe.SharedOnlyBuffers, match="route"):
        k.route(so, torch.zeros(4 * 256, device="cuda"))
    with pytest.raises(X.moe.BufferLength):
        k.route(b, torch.zeros(3 * 256, device="cuda"))


def test_quantize_rows_q8_is_the_reference_s_bytes(oracle, X):
    """MmaKernels::quantize_rows (crates/xabe-cuda/src/kernels/mma.rs:769-811): int8 codes and fp32 scales equal the
    CPU restatement's bit for bit, on random rows, on blocks of zeros (scale 1.0, codes 0), on values that land
    exactly between two codes (rintf: ties to even) and on a block whose largest value is negative; lengths are
    checked as at-least, a ragged contraction is refused."""
    import torch

    rng = np.random.default_rng(77)
    rows, k = 37, 2048
    x = rng.normal(0, 1.5, (rows, k)).astype(np.float32)
    x[3, 64:96] = 0.0                                   # a block of zeros
    x[5, :32] = np.arange(32, dtype=np.float32) * 0.5   # amax 15.5: v * (127 / 15.5) hits .5 ties for some v
    x[5, 31] = 127.0 * 0.25                             # amax 31.75 -> inv = 4: 0.5 * j * 4 = 2 j exactly; and ties:
    x[5, 1] = 0.125                                     # 0.125 * 4 = 0.5 -> rounds to 0 (even)
    x[5, 2] = 0.375                                     # 1.5 -> 2
    x[5, 3] = 0.625                                     # 2.5 -> 2
    x[7, 32:64] = -np.abs(x[7, 32:64]) - 1.0            # every value negative
    want_q, want_s = oracle.quantize_rows_q8(x)
    xd = torch.from_numpy(x).cuda()
    q = torch.zeros(rows, k, dtype=torch.int8, device="cuda")
    sc = torch.zeros(rows, k // 32, dtype=torch.float32, device="cuda")
    X.MmaKernels.quantize_rows(xd, q, sc, rows, k)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), want_q.reshape(rows, k))
    assert np.array_equal(sc.cpu().numpy().view(np.uint32), want_s.reshape(rows, k // 32).view(np.uint32))
    got = q.cpu().numpy()
    assert np.all(got[3, 64:96] == 0) and float(sc[3, 2]) == 1.0
    assert list(got[5, 1:4]) == [0, 2, 2] and got[5, 31] == 127
    assert got[7, 32:64].min() == -127
    # the live rows of a larger buffer: only the first rows are written
    q.fill_(5)
    X.MmaKernels.quantize_rows(xd, q, sc, 2, k)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy()[:2], want_q.reshape(rows, k)[:2]) and bool((q[2:] == 5).all())
    with pytest.raises(X.MoeError, match="not a multiple of 32"):
        X.MmaKernels.quantize_rows(xd, q, sc, rows, 2040)
    with pytest.raises(X.MoeError, match="quantize scales holds"):
        X.MmaKernels.quantize_rows(xd, q, sc[:4], rows, k)

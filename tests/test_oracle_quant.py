"""Oracle pins for Q6_K / Q8_0 (K/quant.rs): the reference's own vectors plus an
independent vectorised numpy re-derivation from the ggml block structs."""
import numpy as np
import pytest


def np_dequant_q6k(raw):
    """Vectorised re-derivation from `block_q6_K {ql[128]; qh[64]; int8 scales[16]; half d}`.
    Element n of a superblock: half = n // 128, lane = (n % 128) // 32, l = n % 32."""
    blk = raw.reshape(-1, 210)
    ql, qh = blk[:, :128], blk[:, 128:192]
    sc = blk[:, 192:208].view(np.int8)
    d = blk[:, 208:210].copy().view(np.float16).astype(np.float32)  # [nb,1]
    n = np.arange(256)
    half, lane, l = n // 128, (n % 128) // 32, n % 32
    qlb = ql[:, half * 64 + (lane % 2) * 32 + l]
    low4 = np.where(lane >= 2, qlb >> 4, qlb & 0xF)
    hi2 = (qh[:, half * 32 + l] >> (2 * lane)) & 3
    q = (low4 | (hi2 << 4)).astype(np.int32) - 32
    s = sc[:, half * 8 + lane * 2 + l // 16].astype(np.float32)
    return ((d * s) * q.astype(np.float32)).astype(np.float32).reshape(-1)


def np_dequant_q8_0(raw):
    blk = raw.reshape(-1, 34)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32)
    return (blk[:, 2:].view(np.int8).astype(np.float32) * d).reshape(-1)


def test_block_sizes(oracle):
    # quant.rs:1063-1072
    assert oracle.BLOCK_BYTES[oracle.Q8_0] == 34 and oracle.BLOCK_BYTES[oracle.Q6K] == 210
    assert int(oracle.lib().xo_block_bytes(oracle.Q6K)) == 210 and int(oracle.lib().xo_block_bytes(oracle.Q8_0)) == 34


def test_q6k_hand_built_superblock(oracle):
    # quant.rs:689-711: ql[0]=1, qh[0]=2, every scale 1, d=2.0 => y[0] = 2.0; every other code is raw 0 => -32*2
    blk = np.zeros(210, np.uint8)
    blk[0], blk[128] = 1, 2
    blk[192:208] = 1
    blk[208:210] = np.array([2.0], np.float16).view(np.uint8)
    y = oracle.dequantize_row(oracle.Q6K, blk)
    assert y[0] == 2.0
    assert np.all(y[1:] == -64.0)


def test_q8_0_all_ff_is_minus_one(oracle):
    # quant.rs:1339-1347: int8 read as signed
    blk = np.full(34, 0xFF, np.uint8)
    blk[0:2] = np.array([1.0], np.float16).view(np.uint8)
    assert np.all(oracle.dequantize_row(oracle.Q8_0, blk) == -1.0)


def test_q6k_negative_scales_and_every_code_position(oracle):
    # one-hot walk: set a single code to +31 with a negative scale and check where it lands
    for n in (0, 31, 32, 63, 64, 95, 96, 127, 128, 200, 255):
        blk = np.zeros(210, np.uint8)
        blk[128:192] = 0xAA        # every hi2 = 2 -> raw 32 -> code 0
        blk[192:208] = np.array([-3], np.int8).view(np.uint8)
        blk[208:210] = np.array([0.5], np.float16).view(np.uint8)
        half, lane, l = n // 128, (n % 128) // 32, n % 32
        raw = 63
        qli = half * 64 + (lane % 2) * 32 + l
        blk[qli] = int(blk[qli]) | ((raw & 0xF) << (4 if lane >= 2 else 0))
        qhi = 128 + half * 32 + l
        blk[qhi] = (int(blk[qhi]) & (0xFF ^ (3 << (2 * lane)))) | ((raw >> 4) << (2 * lane))
        y = oracle.dequantize_row(oracle.Q6K, blk)
        exp = np.zeros(256, np.float32)
        exp[n] = 0.5 * -3 * 31
        assert np.array_equal(y, exp), n


def test_dequant_matches_independent_numpy_on_random_bytes(oracle):
    rng = np.random.default_rng(1)
    raw = rng.integers(0, 256, 210 * 500, dtype=np.uint8)
    raw.reshape(-1, 210)[:, 208:210] = rng.standard_normal(500).astype(np.float16).view(np.uint8).reshape(-1, 2)
    assert np.array_equal(oracle.dequantize_row(oracle.Q6K, raw).view(np.uint32), np_dequant_q6k(raw).view(np.uint32))
    raw8 = rng.integers(0, 256, 34 * 2000, dtype=np.uint8)
    raw8.reshape(-1, 34)[:, 0:2] = rng.standard_normal(2000).astype(np.float16).view(np.uint8).reshape(-1, 2)
    assert np.array_equal(oracle.dequantize_row(oracle.Q8_0, raw8).view(np.uint32), np_dequant_q8_0(raw8).view(np.uint32))


def test_ragged_rows_are_rejected(oracle):
    # quant.rs:1361-1364
    with pytest.raises(ValueError):
        oracle.dequantize_row(oracle.Q6K, np.zeros(211, np.uint8))
    with pytest.raises(ValueError):
        oracle.dequantize_row(oracle.Q8_0, np.zeros(33, np.uint8))


def test_q8_0_round_trip_within_half_a_step(oracle):
    # quant.rs:576-597
    x = oracle.Xorshift64Star(1).vec_f32(32, -4.0, 4.0)
    y = oracle.dequantize_row(oracle.Q8_0, oracle.quantize_row(oracle.Q8_0, x))
    step = np.abs(x).max() / 127.0
    assert oracle.compare(y, x).max_abs_error <= step / 2 + 1e-5


def test_q8_0_zero_and_saturation(oracle):
    # quant.rs:600-615
    z = oracle.quantize_row(oracle.Q8_0, np.zeros(32, np.float32))
    assert np.all(oracle.dequantize_row(oracle.Q8_0, z) == 0.0)
    x = np.zeros(32, np.float32)
    x[0], x[1] = 10.0, -10.0
    b = oracle.quantize_row(oracle.Q8_0, x)
    assert b[2:].view(np.int8)[0] == 127 and b[2:].view(np.int8)[1] == -127


def test_q8_0_bytes_layout(oracle):
    # quant.rs:1297-1317: d (le f16) then 32 int8
    x = (np.arange(32, dtype=np.float32) - 16.0) * 0.25
    b = oracle.quantize_row(oracle.Q8_0, x)
    d = np.float32(4.0) / np.float32(127.0)
    assert b[:2].view(np.float16)[0] == np.float16(d)
    inv = np.float32(1.0) / d
    q = np.sign(x * inv) * np.floor(np.abs(x * inv) + np.float32(0.5))   # round half away from zero
    assert np.array_equal(b[2:].view(np.int8), q.astype(np.int8))


def test_q6k_round_trip_bounds(oracle):
    # quant.rs:618-640 (seed 2, uniform(-4,4)); quant.rs:643-648; quant.rs:673-687 (seed 3, +-100)
    x = oracle.Xorshift64Star(2).vec_f32(256, -4.0, 4.0)
    y = oracle.dequantize_row(oracle.Q6K, oracle.quantize_row(oracle.Q6K, x))
    r = oracle.compare(y, x)
    assert r.max_abs_error < 0.35 and r.cosine_similarity > 0.999, str(r)
    z = oracle.quantize_row(oracle.Q6K, np.zeros(256, np.float32))
    assert np.all(oracle.dequantize_row(oracle.Q6K, z) == 0.0)
    x = oracle.Xorshift64Star(3).vec_f32(256, -100.0, 100.0)
    y = oracle.dequantize_row(oracle.Q6K, oracle.quantize_row(oracle.Q6K, x))
    assert np.all(np.isfinite(y)) and oracle.compare(y, x).cosine_similarity > 0.99


def test_q6k_quantizer_formula_independently(oracle):
    """The reference's amax quantizer (quant.rs:495-567) restated with numpy per group."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(256 * 20) * 0.02).astype(np.float32)
    got = oracle.quantize_row(oracle.Q6K, x).reshape(-1, 210)
    rnd = lambda v: np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
    for b, xb in enumerate(x.reshape(-1, 256)):
        amax = np.abs(xb).max()
        d = np.float32(amax / np.float32(32.0 * 127.0))
        assert got[b, 208:210].view(np.float16)[0] == np.float16(d)
        codes = np.zeros(256, np.int32)
        scales = np.zeros(16, np.int8)
        for half in range(2):
            for lane in range(4):
                for is_ in range(2):
                    pos = half * 128 + lane * 32 + is_ * 16 + np.arange(16)
                    ga = np.abs(xb[pos]).max()
                    sc = np.clip(rnd(np.float32(ga / np.float32(d * np.float32(32.0)))), 0, 127)
                    scales[half * 8 + lane * 2 + is_] = sc
                    den = np.float32(d * np.float32(sc))
                    codes[pos] = np.clip(rnd((xb[pos] / den).astype(np.float32)), -32, 31) if den != 0 else 0
        assert np.array_equal(got[b, 192:208].view(np.int8), scales)
        # decode the codes back out of the packed bytes with the independent dequantiser
        one = got[b].copy()
        one[192:208] = 1
        one[208:210] = np.array([1.0], np.float16).view(np.uint8)
        assert np.array_equal(np_dequant_q6k(one).astype(np.int32), codes)


def test_quantizers_round_exact_halves_away_from_zero(oracle):
    """`f32::round` is half-away-from-zero (quant.rs:75-88, :495-567); C's rintf / numpy's round go to even.
    Inputs built so that the quotient is exactly k + 0.5 in fp32, where the two rules differ; the expected
    codes are written out by hand."""
    # Q8_0: amax 127 -> d = 1, 1/d = 1, so v * inv_d == v
    x = np.zeros(32, np.float32)
    x[:12] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5, 126.5, -126.5, 4.5]
    b = oracle.quantize_row(oracle.Q8_0, x)
    assert b[:2].view(np.float16)[0] == np.float16(1.0)
    assert b[2:14].view(np.int8).tolist() == [127, 1, 2, 3, -1, -2, -3, 4, -4, 127, -127, 5]
    assert np.rint(x[1:9]).tolist() == [0, 2, 2, -0, -2, -2, 4, -4]          # what half-to-even would have stored
    # Q6_K: amax 4064 -> d = 4064 / (32 * 127) = 1.  Group 0 (positions 0..15): amax 4064 -> sc = 127, and
    # x = 127 * (k + 0.5) gives the quotient k + 0.5 exactly.  Group 1 (positions 16..31): amax 336 = 32 * 10.5,
    # so the SCALE itself sits on a half: 11 away from zero, 10 to even; its codes then divide by 11.
    x = np.zeros(256, np.float32)
    x[0] = 4064.0
    x[1:7] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], np.float32) * np.float32(127.0)
    x[16] = 336.0
    x[17:21] = np.array([0.5, 1.5, -0.5, -2.5], np.float32) * np.float32(11.0)
    blk = oracle.quantize_row(oracle.Q6K, x)
    assert blk[208:210].view(np.float16)[0] == np.float16(1.0)
    scales = blk[192:208].view(np.int8)
    assert scales[0] == 127 and scales[1] == 11 and not scales[2:].any()
    one = blk.copy()
    one[192:208] = 1                                                          # read the raw codes back out
    codes = np_dequant_q6k(one).astype(np.int32)
    assert codes[:7].tolist() == [31, 1, 2, 3, -1, -2, -3]                    # 4064/127 = 32 clamps to 31
    assert codes[16:21].tolist() == [31, 1, 2, -1, -3]                        # 336/11 = 30.55 -> 31
    assert not codes[7:16].any() and not codes[21:].any()


def test_q6k_bytes_round_trip(oracle):
    # quant.rs:1319-1337
    x = ((np.arange(256) % 61).astype(np.float32) - 30.0) * np.float32(0.1)
    b = oracle.quantize_row(oracle.Q6K, x)
    assert b.size == 210
    assert np.array_equal(oracle.dequantize_row(oracle.Q6K, b), np_dequant_q6k(b))


def test_synth_generator_is_deterministic_and_normal(oracle):
    a = oracle.synth_normal_f32(11, 256 * 400, 1.0)
    b = oracle.synth_normal_f32(11, 256 * 400, 1.0)
    assert np.array_equal(a, b)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02
    assert abs(np.mean(a ** 4) - 3.0) < 0.2                  # near-normal kurtosis (Irwin-Hall 12: 2.9)
    # chunk independence: element i depends only on (seed, i // 256)
    assert np.array_equal(oracle.synth_normal_f32(11, 256 * 3, 1.0), a[: 256 * 3])
    w = oracle.synth_quant(oracle.Q6K, 7, 256 * 8, 0.02)
    assert np.array_equal(w, oracle.quantize_row(oracle.Q6K, oracle.synth_normal_f32(7, 256 * 8, 0.02)))
    w8 = oracle.synth_quant(oracle.Q8_0, 7, 256 * 8, 0.02)
    assert np.array_equal(w8, oracle.quantize_row(oracle.Q8_0, oracle.synth_normal_f32(7, 256 * 8, 0.02)))


def test_quantize_rows_q8_invariants(oracle):
    # xabe-cuda kernels/mma.rs:118-157
    x = oracle.Xorshift64Star(9).vec_f32(4 * 64, -3.0, 3.0).reshape(4, 64)
    x[1, :32] = 0.0
    q, s = oracle.quantize_rows_q8(x)
    assert s[1, 0] == 1.0 and np.all(q[1, :32] == 0)
    assert np.abs(q).max() == 127
    back = q.astype(np.float32).reshape(4, 2, 32) * s[:, :, None]
    assert np.abs(back.reshape(4, 64) - x).max() <= s.max() / 2 + 1e-6


def test_quantize_rows_q8_closed_forms(oracle):
    """xabe-cuda kernels/mma.rs:118-157 on blocks whose answer is known without the code: with amax = 31.75 the
    factor 127 / amax is exactly 4, so v = j / 8 gives 4 v = j / 2 and rintf's ties go to the even code; a block whose
    only non-zero is negative puts -127 there; the scale is amax / 127 in fp32; a numpy restatement agrees on random
    rows (a dropped clamp, truncation instead of rintf, or amax without the absolute value each fail one of these)."""
    x = np.zeros((2, 64), np.float32)
    x[0, :32] = np.arange(32, dtype=np.float32) / 8.0
    x[0, 31] = 31.75
    x[1, 40] = -2.5
    q, s = oracle.quantize_rows_q8(x)
    assert s[0, 0] == np.float32(31.75) / np.float32(127.0)
    assert list(q[0, :8]) == [0, 0, 1, 2, 2, 2, 3, 4]            # 0, .5, 1, 1.5, 2, 2.5, 3, 3.5 -> ties to even
    assert q[0, 31] == 127
    assert s[0, 1] == 1.0 and not q[0, 32:].any()
    assert q[1, 40] == -127 and s[1, 1] == np.float32(2.5) / np.float32(127.0) and np.count_nonzero(q[1]) == 1
    r = oracle.Xorshift64Star(21).vec_f32(8 * 256, -4.0, 4.0).reshape(8, 256)
    q, s = oracle.quantize_rows_q8(r)
    blocks = r.reshape(8, 8, 32)
    amax = np.abs(blocks).max(axis=2)
    inv = (np.float32(127.0) / amax).astype(np.float32)
    want = np.clip(np.rint((blocks * inv[:, :, None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(q.reshape(8, 8, 32), want)
    assert np.array_equal(s, (amax / np.float32(127.0)).astype(np.float32))

"""Oracle pins: xorshift64* (K/rng.rs:20-55) and binary16 conversion (K/f16.rs:17-100)."""
import numpy as np

MASK = (1 << 64) - 1


def py_xorshift(seed):
    """Independent big-int statement of the published xorshift64* transition."""
    x = seed if seed != 0 else 0x9E3779B97F4A7C15
    while True:
        x ^= x >> 12
        x ^= (x << 25) & MASK
        x ^= x >> 27
        yield (x * 0x2545F4914F6CDD1D) & MASK, x


def test_stream_matches_closed_form(oracle):
    for seed in (1, 2, 42, 0xDEADBEEF, MASK):
        r = oracle.Xorshift64Star(seed)
        g = py_xorshift(seed)
        for _ in range(200):
            assert r.next_u64() == next(g)[0]


def test_first_output_of_seed_one_by_hand(oracle):
    # state 1: x^=x>>12 -> 1; x^=x<<25 -> 0x2000001; x^=x>>27 -> 0x2000001.
    assert oracle.Xorshift64Star(1).next_u64() == (0x2000001 * 0x2545F4914F6CDD1D) & MASK


def test_zero_seed_is_remapped(oracle):
    # rng.rs:21-24, test rng.rs:79-83
    a, b = oracle.Xorshift64Star(0), oracle.Xorshift64Star(0x9E3779B97F4A7C15)
    v = a.next_u64()
    assert v != 0 and v == b.next_u64()


def test_f32_is_top_24_bits_over_2_24(oracle):
    r, g = oracle.Xorshift64Star(7), py_xorshift(7)
    for _ in range(2000):
        x = r.next_f32()
        assert 0.0 <= x < 1.0
        assert x == (next(g)[0] >> 40) / float(1 << 24)


def test_range_and_below(oracle):
    r, g = oracle.Xorshift64Star(99), py_xorshift(99)
    for _ in range(1000):
        assert r.next_u32_below(7) == next(g)[0] % 7
    r, g = oracle.Xorshift64Star(5), py_xorshift(5)
    v = r.vec_f32(64, -4.0, 4.0)
    exp = np.array([np.float32(-4.0) + np.float32((next(g)[0] >> 40) / float(1 << 24)) * np.float32(8.0)
                    for _ in range(64)], dtype=np.float32)
    assert np.array_equal(v, exp)


def test_f16_every_pattern_widens_like_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.from_f16_bits(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))


def test_f16_rounding_is_nearest_even_like_numpy(oracle):
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 4,
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),   # subnormal range
        (rng.standard_normal(2000) * 3e4).astype(np.float32),    # near overflow
        np.array([0.0, -0.0, 1.0, 65504.0, 65520.0, 65519.996, 1e30, -1e30, 1e-10, -1e-10, 2.0**-24, 2.0**-25,
                  1.0 + 2.0**-11, 1.0 + 2.0**-10 + 2.0**-11, 6.1035156e-5], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        ref = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.to_f16_bits(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, ref)


def test_f16_reference_cases(oracle):
    # f16.rs:107-175
    rt = lambda x: oracle.from_f16_bits(oracle.to_f16_bits(x))
    for x in (0.0, 1.0, -1.0, 0.5, 2.0, 1024.0, -1024.0, 65504.0, -65504.0, 0.25, 6.1035156e-5):
        assert rt(x) == np.float32(x)
    assert rt(1.0 + 2.0**-11) == 1.0
    assert rt(1.0 + 2.0**-10 + 2.0**-11) == 1.0 + 2.0**-9
    assert rt(1e30) == float("inf") and rt(-1e30) == float("-inf")
    assert oracle.to_f16_bits(1e-10) == 0 and oracle.to_f16_bits(-1e-10) == 0x8000
    assert rt(2.0**-24) == 2.0**-24 and rt(2.0**-20) == 2.0**-20
    assert oracle.to_f16_bits(float("nan")) & 0x7C00 == 0x7C00 and oracle.to_f16_bits(float("nan")) & 0x3FF

"""LM head, host side (no GPU): geometry arithmetic against the values the reference quotes for the real head
(crates/xabe-cuda/src/kernels/lm_head.rs:1-11, :1318-1392, tests :2060-2200), the validation of
`LmHeadKernels::new`, and the scalar argmax the device reduction is gated against."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def X():
    import llmxabe_amd as X
    return X


def test_geometry_of_the_real_head(X):
    g = X.LmHeadGeometry.qwen3_6(64)
    assert (g.hidden, g.vocab, g.max_tokens) == (2048, 248320, 64)
    assert g.row_bytes() == 2176                      # 64 Q8_0 blocks of 34 bytes
    assert g.weight_bytes() == 540_344_320            # "540 MB read per decoded token"
    assert g.elements() == 508_559_360
    F = X.HeadFormat
    assert g.row_bytes_for(F.Bf16) == 4096 and g.row_bytes_for(F.F16) == 4096 and g.row_bytes_for(F.Q6K) == 8 * 210
    assert g.weight_bytes_for(F.Bf16) == 248320 * 4096
    # a pass over the weights serves MAX_BATCH_TILE tokens
    assert X.MAX_BATCH_TILE == 4 and X.ARGMAX_BLOCKS == 512
    assert [g.weight_passes(t) for t in (1, 3, 4, 5, 8, 37)] == [1, 1, 1, 2, 2, 10]
    assert g.weight_bytes_read(37) == 10 * g.weight_bytes()


def test_head_format_from_ggml(X):
    F = X.HeadFormat
    assert [F.from_ggml(t) for t in (8, 30, 14, 1, 2, 12, 13)] == [F.Q8_0, F.Bf16, F.Q6K, F.F16, F.Q4_0, F.Q4K, F.Q5K]
    assert F.from_ggml(0) is None and F.from_ggml(99) is None


def test_new_rejects_unserviceable_geometries(X):
    # lm_head.rs:1530-1556
    for g, why in ((X.LmHeadGeometry(0, 10, 1), "hidden and vocab must be non-zero"),
                   (X.LmHeadGeometry(2048, 0, 1), "hidden and vocab must be non-zero"),
                   (X.LmHeadGeometry(2000, 10, 1), "multiple of 512"),
                   (X.LmHeadGeometry(2048 + 256, 10, 1), "multiple of 512"),
                   (X.LmHeadGeometry(2048, 10, 0), "max_tokens must be non-zero")):
        with pytest.raises(X.moe.UnsupportedGeometry, match=why):
            X.LmHeadKernels(g)


def test_oracle_argmax_is_first_strict_maximum(oracle):
    # crates/xabe-kernels/src/gemv.rs:103-112 and its tests: first maximum wins; NaN never wins, and a NaN at
    # index 0 is never displaced
    assert oracle.argmax([1.0, 3.0, 2.0, 3.0]) == 1
    assert oracle.argmax([0.5] * 7) == 0
    assert oracle.argmax([np.nan, np.nan]) == 0
    assert oracle.argmax([1.0, np.nan, 2.0]) == 2
    assert oracle.argmax([np.nan, 5.0, 9.0]) == 0
    assert oracle.argmax([-np.inf, -np.inf]) == 0
    assert oracle.argmax([-1.0, np.inf, np.inf]) == 1

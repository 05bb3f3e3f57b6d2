"""The C-ABI library loads and exports every symbol include/xabe_hip.h declares (no GPU needed), and the
host-only entry points behave as the reference's do."""
import ctypes as C
import re

import pytest


def _header_functions():
    from llmxabe_amd import _ffi

    src = "".join(open(p).read() for p in _ffi.HEADER_PATHS)
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(xabe_[a-z0-9_]+)\s*\(", src)))


def test_every_declared_symbol_is_exported_and_bound():
    from llmxabe_amd import _ffi

    names = _header_functions()
    assert len(names) > 60
    lib = _ffi.lib()                       # binds argtypes for every symbol; raises if one is missing
    raw = C.CDLL(_ffi.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} is declared in the header but not exported"
    assert set(names) == set(_ffi.EXPORTED_SYMBOLS), set(names) ^ set(_ffi.EXPORTED_SYMBOLS)
    assert b"gfx950" in lib.xabe_version()


def test_geometry_capacities_match_the_reference_values():
    # crates/xabe-cuda/src/kernels/moe.rs:6981-6989, :6921-6923
    import llmxabe_amd as X

    g = X.MoeGeometry.qwen3_6(16, 64)
    assert (g.num_experts, g.experts_per_token, g.hidden, g.intermediate) == (256, 8, 2048, 512)
    assert g.max_flat_pairs() == 512 and g.sorted_capacity() == 4352 and g.expert_block_capacity() == 272
    g = X.MoeGeometry.qwen3_6(16, 32768)
    assert g.sorted_capacity() == 265984 and g.expert_block_capacity() == 16624
    assert g.stack_elements() == 256 * 512 * 2048
    # crates/xabe-engine/src/forward.rs:163-165
    assert X.moe_block_size(1) == 32 and X.moe_block_size(1152) == 32 and X.moe_block_size(1153) == 64


def test_capacities_agree_with_the_oracle(oracle):
    import llmxabe_amd as X

    for E, K, B, T in ((256, 8, 32, 3), (256, 8, 32, 512), (256, 8, 64, 8192), (8, 2, 32, 6), (4, 2, 3, 3)):
        g = X.MoeGeometry(E, K, 2048, 512, B, T)
        assert g.sorted_capacity() == oracle.sorted_capacity(E, K, B, T)
        assert g.expert_block_capacity() == oracle.expert_block_capacity(E, K, B, T)


def test_expert_quant_tables():
    # crates/xabe-cuda/src/kernels/moe.rs:353-400; the device stride equals the file stride here
    import llmxabe_amd as X

    Q = X.ExpertQuant
    assert [q.block_elements() for q in Q] == [256, 32, 32, 256, 256]
    assert [q.file_block_bytes() for q in Q] == [210, 34, 18, 144, 176]
    assert [q.block_bytes() for q in Q] == [210, 34, 18, 144, 176]
    assert [q.is_community() for q in Q] == [False, False, True, True, True]
    assert X.BLOCK_Q6_K_DEVICE_BYTES == 210
    data = bytes(range(210)) * 3
    assert X.to_device_layout(Q.Q6K, data) == data          # identity: 210-byte streaming, no re-stride
    assert X.to_device_layout(Q.Q8_0, data[:68]) == data[:68]


def test_errors_without_a_device_are_reported_not_crashed():
    """MoeKernels::new validates the geometry before touching the device."""
    import llmxabe_amd as X

    with pytest.raises(X.moe.UnsupportedGeometry, match="block_size must be non-zero"):
        X.MoeKernels(X.MoeGeometry(256, 8, 2048, 512, 0, 4))
    with pytest.raises(X.moe.UnsupportedGeometry, match="dispatch-block capacity exceeds the 65535 grid.y limit"):
        X.MoeKernels(X.MoeGeometry(512, 512, 2048, 512, 1, 65535))


def test_ffn_block_geometry_for_each_architecture():
    # crates/xabe-engine/src/block/ffn.rs:243-256: each architecture gets a geometry and they are not the same one
    import llmxabe_amd as X

    moe = X.FfnBlock.geometry_for(X.FfnConfig.qwen3_6_35b_a3b(), 32, 128)
    dense = X.FfnBlock.geometry_for(X.FfnConfig.qwen3_8_27b(), 32, 128)
    assert (moe.hidden, moe.intermediate, moe.num_experts) == (2048, 512, 256)
    assert (dense.hidden, dense.intermediate, dense.num_experts) == (5120, 17408, 1)
    assert (moe.experts_per_token, dense.experts_per_token) == (8, 1)
    assert (moe.block_size, moe.max_tokens, dense.block_size, dense.max_tokens) == (32, 128, 32, 128)
    with pytest.raises(X.moe.InvalidArgument, match="unknown feed-forward kind"):
        X.FfnBlock.geometry_for(X.FfnConfig(7, 2048), 32, 128)

"""ctypes loader for libxabe_hip.so (the C ABI declared in include/xabe_hip.h).

There is no fallback: if the library is missing or a symbol does not resolve the import
fails, and every wrapper raises on a non-zero status."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libxabe_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "xabe_hip.h")
GGUF_HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "xabe_gguf.h")
LM_HEAD_HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "xabe_lm_head.h")
HEADER_PATHS = (HEADER_PATH, GGUF_HEADER_PATH, LM_HEAD_HEADER_PATH)

sz = C.c_size_t
vp = C.c_void_p


class Geometry(C.Structure):
    _fields_ = [("num_experts", sz), ("experts_per_token", sz), ("hidden", sz), ("intermediate", sz),
                ("block_size", sz), ("max_tokens", sz)]


class QuantTensorC(C.Structure):
    _fields_ = [("bytes", vp), ("len", sz), ("quant", C.c_int)]


class MoeLayerWeightsC(C.Structure):
    _fields_ = [("post_norm", vp), ("router", vp), ("router_quant", C.c_int),
                ("gate_exps", QuantTensorC), ("up_exps", QuantTensorC), ("down_exps", QuantTensorC),
                ("shared_gate_inp", vp),
                ("shared_gate", QuantTensorC), ("shared_up", QuantTensorC), ("shared_down", QuantTensorC)]


class SeamC(C.Structure):
    _fields_ = [("input_normed", C.c_int), ("skip_readback", C.c_int), ("next_norm_weight", vp), ("next_eps", C.c_float),
                ("next_normed", vp), ("next_normed_len", sz), ("next_normed_h", vp), ("next_normed_h_len", sz)]


class DenseLayerWeightsC(C.Structure):
    _fields_ = [("post_norm", vp), ("gate", QuantTensorC), ("up", QuantTensorC), ("down", QuantTensorC)]


class FfnConfigC(C.Structure):
    _fields_ = [("kind", C.c_int), ("hidden", sz), ("num_experts", sz), ("experts_per_token", sz),
                ("expert_intermediate", sz), ("dense_intermediate", sz)]


class FfnLayerWeightsC(C.Structure):
    _fields_ = [("kind", C.c_int), ("moe", MoeLayerWeightsC), ("dense", DenseLayerWeightsC)]


class LmHeadGeometryC(C.Structure):
    _fields_ = [("hidden", sz), ("vocab", sz), ("max_tokens", sz)]


class TensorInfoC(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 4), ("ggml_type", C.c_int),
                ("offset", C.c_uint64), ("n_elements", C.c_uint64), ("n_bytes", C.c_uint64)]


u64 = C.c_uint64
cp = C.c_char_p

_SIGNATURES = {
    "xabe_last_error": (C.c_char_p, []),
    "xabe_status_name": (C.c_char_p, [C.c_int]),
    "xabe_version": (C.c_char_p, []),
    "xabe_moe_geometry_qwen3_6": (Geometry, [sz, sz]),
    "xabe_moe_geometry_max_flat_pairs": (sz, [C.POINTER(Geometry)]),
    "xabe_moe_geometry_sorted_capacity": (sz, [C.POINTER(Geometry)]),
    "xabe_moe_geometry_expert_block_capacity": (sz, [C.POINTER(Geometry)]),
    "xabe_moe_geometry_stack_elements": (sz, [C.POINTER(Geometry)]),
    "xabe_moe_block_size_for": (sz, [sz]),
    "xabe_expert_quant_block_elements": (sz, [C.c_int]),
    "xabe_expert_quant_file_block_bytes": (sz, [C.c_int]),
    "xabe_expert_quant_block_bytes": (sz, [C.c_int]),
    "xabe_expert_quant_is_community": (C.c_int, [C.c_int]),
    "xabe_to_device_layout": (C.c_int, [C.c_int, vp, sz, vp, C.POINTER(sz)]),
    "xabe_moe_kernels_new": (C.c_int, [C.POINTER(Geometry), C.POINTER(vp)]),
    "xabe_moe_kernels_free": (None, [vp]),
    "xabe_moe_kernels_geometry": (C.c_int, [vp, C.POINTER(Geometry)]),
    "xabe_moe_kernels_disable_tensor_cores": (C.c_int, [vp]),
    "xabe_moe_kernels_tensor_cores_enabled": (C.c_int, [vp]),
    "xabe_moe_kernels_force_community": (C.c_int, [vp, C.c_int]),
    "xabe_moe_kernels_set_exact_decode_regime": (C.c_int, [vp, C.c_int]),
    "xabe_moe_kernels_set_mfma_form": (C.c_int, [vp, C.c_int]),
    "xabe_moe_buffers_new": (C.c_int, [vp, vp, C.POINTER(vp)]),
    "xabe_moe_shared_only_buffers_new": (C.c_int, [vp, vp, C.c_int, C.POINTER(vp)]),
    "xabe_moe_buffers_free": (None, [vp]),
    "xabe_moe_buffers_scope": (C.c_int, [vp]),
    "xabe_moe_buffers_topk_ids": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_topk_weights": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_sorted_token_ids": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_expert_ids": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_bucket_live": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_num_tokens_post_pad": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_valid_tokens": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_partial": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_shared_inter": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_buffers_bytes": (sz, [vp]),
    "xabe_moe_set_valid_tokens": (C.c_int, [vp, vp, vp, sz]),
    "xabe_moe_route": (C.c_int, [vp, vp, vp, vp, sz]),
    "xabe_moe_build_dispatch": (C.c_int, [vp, vp, vp]),
    "xabe_moe_route_and_dispatch": (C.c_int, [vp, vp, vp, vp, sz]),
    "xabe_moe_grouped_forward_partial": (C.c_int, [vp, vp, vp, QuantTensorC, QuantTensorC, QuantTensorC, vp, sz]),
    "xabe_moe_grouped_forward_stage": (C.c_int, [vp, vp, vp, QuantTensorC, QuantTensorC, QuantTensorC, vp, sz, C.c_int]),
    "xabe_moe_grouped_forward_partial_with_shared": (C.c_int, [vp, vp, vp] + [QuantTensorC] * 6 + [vp, sz, vp, sz, C.POINTER(C.c_int)]),
    "xabe_moe_grouped_forward": (C.c_int, [vp, vp, vp, QuantTensorC, QuantTensorC, QuantTensorC, vp, sz, vp, sz]),
    "xabe_moe_shared_expert": (C.c_int, [vp, vp, vp, QuantTensorC, QuantTensorC, QuantTensorC, vp, sz, vp, sz]),
    "xabe_moe_shared_expert_mma": (C.c_int, [vp, vp, vp, QuantTensorC, QuantTensorC, QuantTensorC, vp, sz, vp, sz]),
    "xabe_rms_norm": (C.c_int, [vp, vp, sz, vp, sz, vp, sz, sz, sz, C.c_float]),
    "xabe_moe_router_logits": (C.c_int, [vp, vp, vp, vp, sz, C.c_int, vp, sz, vp, sz]),
    "xabe_moe_gate_and_combine": (C.c_int, [vp] * 11),
    "xabe_dense_ffn_add_residual": (C.c_int, [vp] * 6),
    "xabe_moe_add_logit_bias": (C.c_int, [vp] * 5),
    "xabe_dequantize": (C.c_int, [vp, C.c_int, vp, sz, vp, sz]),
    "xabe_mma_quantize_rows": (C.c_int, [vp, vp, sz, vp, sz, vp, sz, sz, sz]),
    "xabe_moe_block_new": (C.c_int, [C.POINTER(Geometry), C.c_float, vp, C.POINTER(vp)]),
    "xabe_moe_block_free": (None, [vp]),
    "xabe_moe_block_publish_tokens": (C.c_int, [vp, vp, sz]),
    "xabe_moe_block_forward": (C.c_int, [vp, vp, C.POINTER(MoeLayerWeightsC), vp, sz, sz, vp, vp, sz, vp, sz]),
    "xabe_moe_block_forward_seam": (C.c_int, [vp, vp, C.POINTER(MoeLayerWeightsC), vp, sz, sz, vp, vp, sz, vp, sz, C.POINTER(SeamC)]),
    "xabe_moe_block_normed_mut": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_normed_h_mut": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_gate_and_combine_seam": (C.c_int, [vp] * 12 + [C.c_float, vp, vp]),
    "xabe_moe_block_forward_noalloc": (C.c_int, [C.POINTER(Geometry), C.c_float, vp, C.POINTER(MoeLayerWeightsC), vp, sz, sz, vp, vp, sz,
                                                 vp, sz]),
    "xabe_moe_block_disable_tensor_cores": (C.c_int, [vp]),
    "xabe_moe_block_set_exact_decode_regime": (C.c_int, [vp, C.c_int]),
    "xabe_moe_block_set_fused_decode": (C.c_int, [vp, C.c_int]),
    "xabe_moe_block_set_mfma_form": (C.c_int, [vp, C.c_int]),
    "xabe_moe_block_forward_stage": (C.c_int, [vp, vp, vp, vp, sz, vp, vp, sz, vp, sz, C.c_int]),
    "xabe_moe_block_tensor_cores_enabled": (C.c_int, [vp]),
    "xabe_moe_block_normed": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_router_logits": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_routed": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_shared_ungated": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_shared_gate": (vp, [vp, C.POINTER(sz)]),
    "xabe_moe_block_buffers": (vp, [vp]),
    "xabe_moe_block_kernels": (vp, [vp]),
    "xabe_dense_ffn_block_new": (C.c_int, [sz, sz, sz, C.c_float, vp, C.POINTER(vp)]),
    "xabe_dense_ffn_block_free": (None, [vp]),
    "xabe_dense_ffn_block_forward": (C.c_int, [vp, vp, C.POINTER(DenseLayerWeightsC), vp, sz, sz, vp, sz, vp, sz]),
    "xabe_dense_ffn_block_disable_tensor_cores": (C.c_int, [vp]),
    "xabe_dense_ffn_block_normed": (vp, [vp, C.POINTER(sz)]),
    "xabe_dense_ffn_block_tensor_cores_enabled": (C.c_int, [vp]),
    "xabe_dense_ffn_block_publish_tokens": (C.c_int, [vp, vp, sz]),
    "xabe_ffn_block_geometry_for": (C.c_int, [C.POINTER(FfnConfigC), sz, sz, C.POINTER(Geometry)]),
    "xabe_ffn_block_new": (C.c_int, [C.POINTER(FfnConfigC), C.POINTER(Geometry), C.c_float, vp, C.POINTER(vp)]),
    "xabe_ffn_block_free": (None, [vp]),
    "xabe_ffn_block_kind": (C.c_int, [vp]),
    "xabe_ffn_block_disable_tensor_cores": (C.c_int, [vp]),
    "xabe_ffn_block_tensor_cores_enabled": (C.c_int, [vp]),
    "xabe_ffn_block_set_exact_decode_regime": (C.c_int, [vp, C.c_int]),
    "xabe_ffn_block_geometry": (C.c_int, [vp, C.POINTER(Geometry)]),
    "xabe_ffn_block_normed": (vp, [vp, C.POINTER(sz)]),
    "xabe_ffn_block_as_moe": (vp, [vp]),
    "xabe_ffn_block_publish_tokens": (C.c_int, [vp, vp, sz]),
    "xabe_ffn_block_forward": (C.c_int, [vp, vp, C.POINTER(FfnLayerWeightsC), vp, sz, sz, vp, sz, vp, sz]),
    "xabe_synth_normal_f32": (C.c_int, [vp, C.c_uint64, sz, C.c_float, vp]),
    "xabe_calibrate_hbm_read": (C.c_int, [vp, vp, sz, vp]),
    "xabe_calibrate_mfma_f16": (C.c_int, [vp, vp, sz, C.c_int, C.POINTER(C.c_double)]),
    "xabe_synth_quant": (C.c_int, [vp, C.c_int, C.c_uint64, sz, C.c_float, vp, sz]),
    # include/xabe_gguf.h
    "xabe_ggml_type_block_size": (u64, [C.c_int]),
    "xabe_ggml_type_size": (u64, [C.c_int]),
    "xabe_ggml_type_name": (cp, [C.c_int]),
    "xabe_ggml_type_bytes_for_elements": (C.c_int, [C.c_int, u64, C.POINTER(u64)]),
    "xabe_gguf_open": (C.c_int, [cp, C.POINTER(vp)]),
    "xabe_gguf_from_bytes": (C.c_int, [vp, sz, C.POINTER(vp)]),
    "xabe_gguf_close": (None, [vp]),
    "xabe_gguf_version": (C.c_uint32, [vp]),
    "xabe_gguf_alignment": (C.c_uint32, [vp]),
    "xabe_gguf_n_kv": (sz, [vp]),
    "xabe_gguf_n_tensors": (sz, [vp]),
    "xabe_gguf_data_offset": (u64, [vp]),
    "xabe_gguf_tensor_at": (C.c_int, [vp, sz, C.POINTER(TensorInfoC)]),
    "xabe_gguf_tensor": (C.c_int, [vp, cp, C.POINTER(TensorInfoC)]),
    "xabe_gguf_tensor_bytes": (vp, [vp, cp, C.POINTER(sz)]),
    "xabe_gguf_key_at": (cp, [vp, sz]),
    "xabe_gguf_value_type_of": (C.c_int, [vp, cp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(u64)]),
    "xabe_gguf_get_u32": (C.c_int, [vp, cp, C.POINTER(C.c_uint32)]),
    "xabe_gguf_get_u64": (C.c_int, [vp, cp, C.POINTER(u64)]),
    "xabe_gguf_get_f32": (C.c_int, [vp, cp, C.POINTER(C.c_float)]),
    "xabe_gguf_get_str": (vp, [vp, cp, C.POINTER(sz)]),
    "xabe_gguf_get_array": (vp, [vp, cp, C.c_int, C.POINTER(u64)]),
    "xabe_gguf_get_string_array_item": (vp, [vp, cp, u64, C.POINTER(sz)]),
    "xabe_moe_layer_upload": (C.c_int, [vp, vp, C.c_uint32, C.POINTER(Geometry), C.POINTER(vp)]),
    "xabe_moe_layer_free": (None, [vp]),
    "xabe_moe_layer_weights_of": (C.POINTER(MoeLayerWeightsC), [vp]),
    "xabe_moe_layer_index": (C.c_uint32, [vp]),
    "xabe_moe_layer_expert_quants": (C.c_int, [vp, C.POINTER(C.c_int * 3)]),
    "xabe_moe_layer_shared_quants": (C.c_int, [vp, C.POINTER(C.c_int * 3)]),
    "xabe_moe_layer_router_types": (C.c_int, [vp, C.POINTER(C.c_int * 2)]),
    "xabe_moe_layer_bytes": (sz, [vp]),
    "xabe_dense_ffn_layer_upload": (C.c_int, [vp, vp, C.c_uint32, sz, sz, C.POINTER(vp)]),
    "xabe_dense_ffn_layer_free": (None, [vp]),
    "xabe_dense_ffn_layer_weights_of": (C.POINTER(DenseLayerWeightsC), [vp]),
    "xabe_dense_ffn_layer_quants": (C.c_int, [vp, C.POINTER(C.c_int * 3)]),
    "xabe_dense_ffn_layer_bytes": (sz, [vp]),
    # include/xabe_lm_head.h
    "xabe_head_format_from_ggml": (C.c_int, [C.c_int]),
    "xabe_lm_head_geometry_qwen3_6": (LmHeadGeometryC, [sz]),
    "xabe_lm_head_row_bytes_for": (sz, [C.POINTER(LmHeadGeometryC), C.c_int]),
    "xabe_lm_head_weight_bytes_for": (sz, [C.POINTER(LmHeadGeometryC), C.c_int]),
    "xabe_lm_head_elements": (sz, [C.POINTER(LmHeadGeometryC)]),
    "xabe_lm_head_weight_passes": (sz, [C.POINTER(LmHeadGeometryC), sz]),
    "xabe_lm_head_weight_bytes_read": (sz, [C.POINTER(LmHeadGeometryC), C.c_int, sz]),
    "xabe_lm_head_new": (C.c_int, [C.POINTER(LmHeadGeometryC), C.POINTER(vp)]),
    "xabe_lm_head_free": (None, [vp]),
    "xabe_lm_head_geometry_of": (C.c_int, [vp, C.POINTER(LmHeadGeometryC)]),
    "xabe_lm_head_forward": (C.c_int, [vp, vp, C.c_int, vp, sz, vp, sz, sz, vp, sz]),
    "xabe_lm_head_argmax": (C.c_int, [vp, vp, vp, sz, sz, vp, sz, vp, sz, vp, sz]),
    "xabe_lm_head_argmax_prob": (C.c_int, [vp, vp, vp, sz, sz, vp, sz]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def lib() -> C.CDLL:
    """The loaded library.  Raises ImportError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C llmxabe_amd/csrc` (or __graft_entry__.build()). "
                "There is no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib

"""The launch API, named as in the reference (`xabe_cuda::kernels::moe`, crates/xabe-cuda/src/kernels/moe.rs):
MoeGeometry, ExpertQuant, QuantTensor, BufferScope, MoeKernels, MoeBuffers, MoeError, to_device_layout.

Device memory is a torch tensor on the GPU (torch is plumbing here: allocator and streams).  Every
method forwards to one C-ABI entry point of libxabe_hip and raises a `MoeError` subclass on failure."""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass

import torch

from . import _ffi
from ._ffi import Geometry, QuantTensorC


# ---------------------------------------------------------------- errors (moe.rs:4602-4637, block/moe.rs:494-547)
class MoeError(RuntimeError):
    status = -1


class Compile(MoeError): status = 1
class Driver(MoeError): status = 2
class Mma(MoeError): status = 3
class UnsupportedGeometry(MoeError): status = 4
class RaggedWeights(MoeError): status = 5
class WrongElementCount(MoeError): status = 6
class TooManyTokens(MoeError): status = 7
class SharedOnlyBuffers(MoeError): status = 8
class BufferLength(MoeError): status = 9
class InvalidArgument(MoeError): status = 10
class UnsupportedExpertType(MoeError): status = 11
class FfnKindMismatch(MoeError): status = 12

_ERRORS = {c.status: c for c in (Compile, Driver, Mma, UnsupportedGeometry, RaggedWeights, WrongElementCount,
                                 TooManyTokens, SharedOnlyBuffers, BufferLength, InvalidArgument,
                                 UnsupportedExpertType, FfnKindMismatch)}


def check(status: int) -> None:
    if status != 0:
        msg = _ffi.lib().xabe_last_error().decode()
        raise _ERRORS.get(status, MoeError)(msg)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ---------------------------------------------------------------- geometry (moe.rs:4523-4598)
@dataclass(frozen=True)
class MoeGeometry:
    num_experts: int
    experts_per_token: int
    hidden: int
    intermediate: int
    block_size: int
    max_tokens: int

    @staticmethod
    def qwen3_6(block_size: int, max_tokens: int) -> "MoeGeometry":
        g = _ffi.lib().xabe_moe_geometry_qwen3_6(block_size, max_tokens)
        return MoeGeometry(g.num_experts, g.experts_per_token, g.hidden, g.intermediate, g.block_size, g.max_tokens)

    def _c(self) -> Geometry:
        return Geometry(self.num_experts, self.experts_per_token, self.hidden, self.intermediate, self.block_size,
                        self.max_tokens)

    def max_flat_pairs(self) -> int:
        return _ffi.lib().xabe_moe_geometry_max_flat_pairs(C.byref(self._c()))

    def sorted_capacity(self) -> int:
        return _ffi.lib().xabe_moe_geometry_sorted_capacity(C.byref(self._c()))

    def expert_block_capacity(self) -> int:
        return _ffi.lib().xabe_moe_geometry_expert_block_capacity(C.byref(self._c()))

    def stack_elements(self) -> int:
        return _ffi.lib().xabe_moe_geometry_stack_elements(C.byref(self._c()))


def moe_block_size(tokens: int) -> int:
    """crates/xabe-engine/src/forward.rs:163-165"""
    return _ffi.lib().xabe_moe_block_size_for(tokens)


# ---------------------------------------------------------------- formats (moe.rs:298-464)
class ExpertQuant(enum.IntEnum):
    Q6K = 0
    Q8_0 = 1
    Q4_0 = 2
    Q4K = 3
    Q5K = 4

    def block_elements(self) -> int:
        return _ffi.lib().xabe_expert_quant_block_elements(int(self))

    def file_block_bytes(self) -> int:
        return _ffi.lib().xabe_expert_quant_file_block_bytes(int(self))

    def block_bytes(self) -> int:
        return _ffi.lib().xabe_expert_quant_block_bytes(int(self))

    def is_community(self) -> bool:
        return bool(_ffi.lib().xabe_expert_quant_is_community(int(self)))


BLOCK_Q6_K_DEVICE_BYTES = 210  # the device holds the file layout; the reference re-strides to 224 (moe.rs:93-97)


def to_device_layout(quant: ExpertQuant, data: bytes) -> bytes:
    """moe.rs:410-444: the identity here."""
    out_len = C.c_size_t(0)
    buf = (C.c_uint8 * len(data)).from_buffer_copy(data)
    out = (C.c_uint8 * len(data))()
    check(_ffi.lib().xabe_to_device_layout(int(quant), buf, len(data), out, C.byref(out_len)))
    return bytes(out[: out_len.value])


@dataclass
class QuantTensor:
    """moe.rs:448-464.  `bytes` is a uint8 CUDA tensor."""
    bytes: torch.Tensor
    quant: ExpertQuant

    def _c(self) -> QuantTensorC:
        assert self.bytes.dtype == torch.uint8 and self.bytes.is_cuda and self.bytes.is_contiguous()
        return QuantTensorC(self.bytes.data_ptr(), self.bytes.numel(), int(self.quant))


class BufferScope(enum.IntEnum):
    Routed = 0
    SharedOnly = 1


# ---------------------------------------------------------------- buffers (moe.rs:4713-4864)
class MoeBuffers:
    def __init__(self, handle: int, owner: bool = True):
        self._h = handle
        self._owner = owner

    def __del__(self):
        if getattr(self, "_h", None) and self._owner:
            try:
                _ffi.lib().xabe_moe_buffers_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def scope(self) -> BufferScope:
        return BufferScope(_ffi.lib().xabe_moe_buffers_scope(self._h))

    def _view(self, name: str, dtype) -> torch.Tensor:
        n = C.c_size_t(0)
        p = getattr(_ffi.lib(), "xabe_moe_buffers_" + name)(self._h, C.byref(n))
        return _wrap(p, n.value, dtype)

    def topk_ids(self): return self._view("topk_ids", torch.int32)
    def topk_weights(self): return self._view("topk_weights", torch.float32)
    def sorted_token_ids(self): return self._view("sorted_token_ids", torch.int32)
    def expert_ids(self): return self._view("expert_ids", torch.int32)
    def bucket_live(self): return self._view("bucket_live", torch.int32)
    def num_tokens_post_pad(self): return self._view("num_tokens_post_pad", torch.int32)
    def valid_tokens(self): return self._view("valid_tokens", torch.int32)
    def partial(self): return self._view("partial", torch.float32)
    def shared_inter(self): return self._view("shared_inter", torch.float32)

    def bytes(self) -> int:
        return _ffi.lib().xabe_moe_buffers_bytes(self._h)


class _Foreign:
    """Exposes library-owned device memory through __cuda_array_interface__ so torch can view it."""

    def __init__(self, ptr: int, n: int, typestr: str):
        self.__cuda_array_interface__ = {"shape": (n,), "typestr": typestr, "data": (ptr, False), "version": 3,
                                         "strides": None}


def _wrap(ptr, n: int, dtype) -> torch.Tensor:
    """A copy of `n` elements of library-owned device memory as a torch tensor."""
    if not ptr or n == 0:
        return torch.empty(0, dtype=dtype, device="cuda")
    typestr = {torch.int32: "<i4", torch.float32: "<f4", torch.uint8: "|u1"}[dtype]
    return torch.as_tensor(_Foreign(int(ptr), n, typestr), device="cuda").clone()


# ---------------------------------------------------------------- kernels (moe.rs:5033-6714)
class MoeKernels:
    def __init__(self, geometry: MoeGeometry):
        """MoeKernels::new (moe.rs:5038-5330)"""
        h = C.c_void_p()
        check(_ffi.lib().xabe_moe_kernels_new(C.byref(geometry._c()), C.byref(h)))
        self._h = h.value
        self._geometry = geometry

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_moe_kernels_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def geometry(self) -> MoeGeometry:
        return self._geometry

    def buffers(self) -> MoeBuffers:
        h = C.c_void_p()
        check(_ffi.lib().xabe_moe_buffers_new(self._h, _stream(), C.byref(h)))
        return MoeBuffers(h.value)

    def shared_only_buffers(self, mma: bool) -> MoeBuffers:
        h = C.c_void_p()
        check(_ffi.lib().xabe_moe_shared_only_buffers_new(self._h, _stream(), int(mma), C.byref(h)))
        return MoeBuffers(h.value)

    def disable_tensor_cores(self): check(_ffi.lib().xabe_moe_kernels_disable_tensor_cores(self._h))
    def tensor_cores_enabled(self) -> bool: return bool(_ffi.lib().xabe_moe_kernels_tensor_cores_enabled(self._h))
    def force_community(self, on: bool): check(_ffi.lib().xabe_moe_kernels_force_community(self._h, int(on)))
    def set_mfma_form(self, form: int):
        """0: by width; 1: k_mfma_expert; 2: k_mfma_pc wherever the shape allows (a comparison switch; see the header)."""
        check(_ffi.lib().xabe_moe_kernels_set_mfma_form(self._h, form))

    def set_exact_decode_regime(self, on: bool): check(_ffi.lib().xabe_moe_kernels_set_exact_decode_regime(self._h, int(on)))

    def set_valid_tokens(self, buffers: MoeBuffers, tokens: int):
        check(_ffi.lib().xabe_moe_set_valid_tokens(self._h, _stream(), buffers._h, tokens))

    def route(self, buffers: MoeBuffers, logits: torch.Tensor):
        check(_ffi.lib().xabe_moe_route(self._h, _stream(), buffers._h, _ptr(logits), logits.numel()))

    def build_dispatch(self, buffers: MoeBuffers):
        check(_ffi.lib().xabe_moe_build_dispatch(self._h, _stream(), buffers._h))

    def route_and_dispatch(self, buffers: MoeBuffers, logits: torch.Tensor):
        check(_ffi.lib().xabe_moe_route_and_dispatch(self._h, _stream(), buffers._h, _ptr(logits), logits.numel()))

    def grouped_forward_partial(self, buffers, gate: QuantTensor, up: QuantTensor, down: QuantTensor, hidden_states):
        check(_ffi.lib().xabe_moe_grouped_forward_partial(self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(),
                                                          _ptr(hidden_states), hidden_states.numel()))

    def grouped_forward_stage(self, buffers, gate, up, down, hidden_states, stage: int):
        check(_ffi.lib().xabe_moe_grouped_forward_stage(self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(),
                                                        _ptr(hidden_states), hidden_states.numel(), stage))

    def grouped_forward_partial_with_shared(self, buffers, gate, up, down, shared_gate, shared_up, shared_down,
                                            hidden_states, out) -> bool:
        fused = C.c_int(0)
        check(_ffi.lib().xabe_moe_grouped_forward_partial_with_shared(
            self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(), shared_gate._c(), shared_up._c(),
            shared_down._c(), _ptr(hidden_states), hidden_states.numel(), _ptr(out), out.numel(), C.byref(fused)))
        return bool(fused.value)

    def grouped_forward(self, buffers, gate, up, down, hidden_states, out):
        check(_ffi.lib().xabe_moe_grouped_forward(self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(),
                                                  _ptr(hidden_states), hidden_states.numel(), _ptr(out), out.numel()))

    def shared_expert(self, buffers, gate, up, down, hidden_states, out):
        check(_ffi.lib().xabe_moe_shared_expert(self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(),
                                                _ptr(hidden_states), hidden_states.numel(), _ptr(out), out.numel()))

    def shared_expert_mma(self, buffers, gate, up, down, hidden_states, out):
        check(_ffi.lib().xabe_moe_shared_expert_mma(self._h, _stream(), buffers._h, gate._c(), up._c(), down._c(),
                                                    _ptr(hidden_states), hidden_states.numel(), _ptr(out), out.numel()))

    # glue kernels the engine used to compile for itself (block/moe.rs:301-483)
    def router_logits(self, buffers, router: torch.Tensor, router_quant, normed, logits):
        q = -1 if router_quant is None else int(router_quant)
        check(_ffi.lib().xabe_moe_router_logits(self._h, _stream(), buffers._h, _ptr(router), router.numel(), q,
                                                _ptr(normed), normed.numel(), _ptr(logits), logits.numel()))

    def add_logit_bias(self, buffers, bias, logits):
        check(_ffi.lib().xabe_moe_add_logit_bias(self._h, _stream(), buffers._h, _ptr(bias), _ptr(logits)))

    def gate_and_combine(self, buffers, shared_gate_inp, normed, shexp, residual, gate, routed, ffn_out, l_out):
        check(_ffi.lib().xabe_moe_gate_and_combine(self._h, _stream(), buffers._h, _ptr(shared_gate_inp), _ptr(normed),
                                                   _ptr(shexp), _ptr(residual), _ptr(gate), _ptr(routed), _ptr(ffn_out),
                                                   _ptr(l_out)))

    def gate_and_combine_seam(self, buffers, shared_gate_inp, normed, shexp, residual, gate, routed, ffn_out, l_out,
                              next_norm_weight=None, next_eps: float = 1e-6, next_normed=None, next_normed_h=None):
        """`gate_and_combine` with the next layer's RMSNorm applied to l_out in the same launch (see the header);
        `routed` and `ffn_out` may be None."""
        check(_ffi.lib().xabe_moe_gate_and_combine_seam(self._h, _stream(), buffers._h, _ptr(shared_gate_inp), _ptr(normed),
                                                        _ptr(shexp), _ptr(residual), _ptr(gate), _ptr(routed), _ptr(ffn_out),
                                                        _ptr(l_out), _ptr(next_norm_weight), next_eps, _ptr(next_normed),
                                                        _ptr(next_normed_h)))

    def dense_ffn_add_residual(self, buffers, ffn_out, residual, l_out):
        check(_ffi.lib().xabe_dense_ffn_add_residual(self._h, _stream(), buffers._h, _ptr(ffn_out), _ptr(residual),
                                                     _ptr(l_out)))


class LayerOpsKernels:
    """crates/xabe-cuda/src/kernels/layer_ops.rs:777-805 (rms_norm only)."""

    @staticmethod
    def rms_norm(x, weight, out, rows: int, width: int, eps: float):
        check(_ffi.lib().xabe_rms_norm(_stream(), _ptr(x), x.numel(), _ptr(weight), weight.numel(), _ptr(out),
                                       out.numel(), rows, width, eps))


class MmaKernels:
    """crates/xabe-cuda/src/kernels/mma.rs:729-811 (quantize_rows only: the matrix-core path here multiplies fp16
    operands and has no use for the int8 form)."""

    @staticmethod
    def quantize_rows(x: torch.Tensor, q: torch.Tensor, scales: torch.Tensor, rows: int, k: int):
        check(_ffi.lib().xabe_mma_quantize_rows(_stream(), _ptr(x), x.numel(), _ptr(q), q.numel(), _ptr(scales),
                                                scales.numel(), rows, k))


def dequantize(quant: ExpertQuant, data: torch.Tensor) -> torch.Tensor:
    """crates/xabe-cuda/src/kernels/dequant.rs: bit-identical to the CPU reference."""
    n = data.numel() // max(1, ExpertQuant(quant).block_bytes()) * ExpertQuant(quant).block_elements()
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    check(_ffi.lib().xabe_dequantize(_stream(), int(quant), _ptr(data), data.numel(), _ptr(out), n))
    return out


def synth_normal_f32(seed: int, n: int, sigma: float) -> torch.Tensor:
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    check(_ffi.lib().xabe_synth_normal_f32(_stream(), seed & 0xFFFFFFFFFFFFFFFF, n, sigma, _ptr(out)))
    return out


ZIPF_BIAS_SEED = 5   # the skewed-routing workload's permutation of the experts


def zipf_logit_bias(num_experts: int, seed: int = ZIPF_BIAS_SEED, s: float = 1.1, c: float = 1.0):
    """The skewed-routing workload's per-expert logit bias, b_e = -c * s * ln(rank_e) with rank a seeded permutation
    of 1..num_experts (selection odds proportional to rank^(-c*s)); a host float32 array.  The reference has no bias
    input: a harness adds it to the logits between the router GEMV and `route`.  One definition for the benchmark and
    the parity tests, so that what is timed is what is checked."""
    import numpy as np

    rank = np.random.default_rng(seed).permutation(num_experts) + 1
    return (-c * s * np.log(rank)).astype(np.float32)


def calibrate_hbm_read(buffer: torch.Tensor, sink: torch.Tensor) -> None:
    """One launch that reads every 16-byte piece of `buffer` once, coalesced; the caller times it."""
    check(_ffi.lib().xabe_calibrate_hbm_read(_stream(), _ptr(buffer), buffer.numel() * buffer.element_size(), _ptr(sink)))


def calibrate_mfma_f16(out: torch.Tensor, iters: int) -> float:
    """One launch of a register-resident fp16 matrix-instruction loop on every SIMD; returns its flop count."""
    flops = C.c_double(0.0)
    check(_ffi.lib().xabe_calibrate_mfma_f16(_stream(), _ptr(out), out.numel(), iters, C.byref(flops)))
    return flops.value


def synth_quant(quant: ExpertQuant, seed: int, n_elements: int, sigma: float) -> torch.Tensor:
    q = ExpertQuant(quant)
    nbytes = n_elements // q.block_elements() * q.block_bytes()
    out = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    check(_ffi.lib().xabe_synth_quant(_stream(), int(q), seed & 0xFFFFFFFFFFFFFFFF, n_elements, sigma, _ptr(out), nbytes))
    return out

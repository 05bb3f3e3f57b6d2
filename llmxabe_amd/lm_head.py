"""Mirror of `xabe_cuda::kernels::lm_head::{LmHeadKernels, LmHeadGeometry, HeadFormat, HeadTensor}`
(crates/xabe-cuda/src/kernels/lm_head.rs:1206-2058).  The kernels live in csrc/lm_head.hip."""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass

import torch

from . import _ffi
from ._ffi import LmHeadGeometryC
from .moe import _ptr, _stream, check

MAX_BATCH_TILE = 4     # tokens one pass over the weights serves (the reference's tile is 8, lm_head.rs:125)
ARGMAX_BLOCKS = 512    # lm_head.rs:169


class HeadFormat(enum.IntEnum):
    """lm_head.rs:1206-1227."""
    Q8_0 = 0
    Bf16 = 1
    Q6K = 2
    F16 = 3
    Q4_0 = 4
    Q4K = 5
    Q5K = 6

    @staticmethod
    def from_ggml(ggml_type: int):
        f = _ffi.lib().xabe_head_format_from_ggml(int(ggml_type))
        return None if f < 0 else HeadFormat(f)


@dataclass(frozen=True)
class HeadTensor:
    """A weight tensor as the file holds it, with its storage format (lm_head.rs:1261-1301)."""
    bytes: torch.Tensor
    format: HeadFormat

    @staticmethod
    def q8_0(b): return HeadTensor(b, HeadFormat.Q8_0)
    @staticmethod
    def bf16(b): return HeadTensor(b, HeadFormat.Bf16)
    @staticmethod
    def q6_k(b): return HeadTensor(b, HeadFormat.Q6K)
    @staticmethod
    def f16(b): return HeadTensor(b, HeadFormat.F16)


@dataclass(frozen=True)
class LmHeadGeometry:
    hidden: int
    vocab: int
    max_tokens: int

    @staticmethod
    def qwen3_6(max_tokens: int) -> "LmHeadGeometry":
        g = _ffi.lib().xabe_lm_head_geometry_qwen3_6(max_tokens)
        return LmHeadGeometry(g.hidden, g.vocab, g.max_tokens)

    def _c(self) -> LmHeadGeometryC:
        return LmHeadGeometryC(self.hidden, self.vocab, self.max_tokens)

    def row_bytes_for(self, fmt) -> int: return _ffi.lib().xabe_lm_head_row_bytes_for(C.byref(self._c()), int(fmt))
    def row_bytes(self) -> int: return self.row_bytes_for(HeadFormat.Q8_0)
    def weight_bytes_for(self, fmt) -> int: return _ffi.lib().xabe_lm_head_weight_bytes_for(C.byref(self._c()), int(fmt))
    def weight_bytes(self) -> int: return self.weight_bytes_for(HeadFormat.Q8_0)
    def elements(self) -> int: return _ffi.lib().xabe_lm_head_elements(C.byref(self._c()))
    def weight_passes(self, tokens: int) -> int: return _ffi.lib().xabe_lm_head_weight_passes(C.byref(self._c()), tokens)

    def weight_bytes_read(self, tokens: int, fmt=HeadFormat.Q8_0) -> int:
        return _ffi.lib().xabe_lm_head_weight_bytes_read(C.byref(self._c()), int(fmt), tokens)


class LmHeadKernels:
    def __init__(self, geometry: LmHeadGeometry):
        h = C.c_void_p()
        check(_ffi.lib().xabe_lm_head_new(C.byref(geometry._c()), C.byref(h)))
        self._h = h.value
        self._geometry = geometry

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_lm_head_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def geometry(self) -> LmHeadGeometry: return self._geometry

    def forward(self, weight: HeadTensor, hidden_states, tokens: int, logits):
        """logits[t][v] = sum_h weight[v][h] * hidden_states[t][h]; rows past `tokens` are left alone."""
        check(_ffi.lib().xabe_lm_head_forward(self._h, _stream(), int(weight.format), _ptr(weight.bytes), weight.bytes.numel()
                                              * weight.bytes.element_size(), _ptr(hidden_states), hidden_states.numel(), tokens,
                                              _ptr(logits), logits.numel()))

    def argmax(self, values, n: int, partial_values, partial_indices, out):
        check(_ffi.lib().xabe_lm_head_argmax(self._h, _stream(), _ptr(values), values.numel(), n, _ptr(partial_values),
                                             partial_values.numel(), _ptr(partial_indices), partial_indices.numel(), _ptr(out),
                                             out.numel()))

    def argmax_prob(self, values, n: int, out):
        check(_ffi.lib().xabe_lm_head_argmax_prob(self._h, _stream(), _ptr(values), values.numel(), n, _ptr(out), out.numel()))

"""Block-level mirrors of `MoeBlock` / `MoeLayerWeights` (crates/xabe-engine/src/block/moe.rs:634-1330)
`DenseFfnBlock` (crates/xabe-engine/src/block/dense_ffn.rs) and `FfnBlock` (crates/xabe-engine/src/block/ffn.rs).
The sequencing itself lives in the
library (csrc/block.hip); these classes hold the handles and the device tensors."""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass
from typing import Optional

import torch

from . import _ffi
from ._ffi import DenseLayerWeightsC, FfnConfigC, FfnLayerWeightsC, Geometry, MoeLayerWeightsC, SeamC
from .moe import ExpertQuant, MoeBuffers, MoeGeometry, QuantTensor, _ptr, _stream, _wrap, check

DEFAULT_RMS_EPS = 1e-6  # block/moe.rs:179


@dataclass
class MoeLayerWeights:
    """Device tensors of one layer (block/moe.rs:634-658).  `router` is f32 [E][H] when
    `router_quant` is None, else Q8_0 bytes."""
    post_norm: torch.Tensor
    router: torch.Tensor
    router_quant: Optional[ExpertQuant]
    gate_exps: QuantTensor
    up_exps: QuantTensor
    down_exps: QuantTensor
    shared_gate_inp: torch.Tensor
    shared_gate: QuantTensor
    shared_up: QuantTensor
    shared_down: QuantTensor

    def _c(self) -> MoeLayerWeightsC:
        return MoeLayerWeightsC(_ptr(self.post_norm), _ptr(self.router),
                                -1 if self.router_quant is None else int(self.router_quant),
                                self.gate_exps._c(), self.up_exps._c(), self.down_exps._c(),
                                _ptr(self.shared_gate_inp), self.shared_gate._c(), self.shared_up._c(),
                                self.shared_down._c())


class MoeBlock:
    def __init__(self, geometry: MoeGeometry, eps: float = DEFAULT_RMS_EPS):
        h = C.c_void_p()
        check(_ffi.lib().xabe_moe_block_new(C.byref(geometry._c()), eps, _stream(), C.byref(h)))
        self._h = h.value
        self._geometry = geometry
        self._eps = eps

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_moe_block_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def geometry(self) -> MoeGeometry: return self._geometry
    def eps(self) -> float: return self._eps
    def disable_tensor_cores(self): check(_ffi.lib().xabe_moe_block_disable_tensor_cores(self._h))
    def set_exact_decode_regime(self, on: bool): check(_ffi.lib().xabe_moe_block_set_exact_decode_regime(self._h, int(on)))
    def tensor_cores_enabled(self) -> bool: return bool(_ffi.lib().xabe_moe_block_tensor_cores_enabled(self._h))
    def set_fused_decode(self, on: bool): check(_ffi.lib().xabe_moe_block_set_fused_decode(self._h, int(on)))
    def set_mfma_form(self, form: int): check(_ffi.lib().xabe_moe_block_set_mfma_form(self._h, form))

    def publish_tokens(self, tokens: int):
        check(_ffi.lib().xabe_moe_block_publish_tokens(self._h, _stream(), tokens))

    def forward(self, w: MoeLayerWeights, residual, tokens: int, ffn_out, l_out, logit_bias=None):
        cw = w._c()
        check(_ffi.lib().xabe_moe_block_forward(self._h, _stream(), C.byref(cw), _ptr(residual), residual.numel(), tokens,
                                                _ptr(logit_bias), _ptr(ffn_out), ffn_out.numel(), _ptr(l_out),
                                                l_out.numel()))

    def forward_seam(self, w: MoeLayerWeights, residual, tokens: int, ffn_out, l_out, logit_bias=None, input_normed=False,
                     next_norm_weight=None, next_block: "MoeBlock | None" = None, next_eps: float | None = None,
                     skip_readback=False):
        """`forward` across the post-mixer seam (see the header): with `next_norm_weight`, the launch that finishes
        l_out also leaves rms_norm(l_out, next_norm_weight) in `next_block`'s normalised-rows buffers (this block's
        own when `next_block` is None: one handle serving every layer); with `input_normed`, this block starts from
        the rows a previous call left there.  `ffn_out` may be None."""
        cw = w._c()
        seam = SeamC(int(input_normed), int(skip_readback), 0, 0.0, 0, 0, 0, 0)
        if next_norm_weight is not None:
            dst = next_block if next_block is not None else self
            n, nh = C.c_size_t(0), C.c_size_t(0)
            seam.next_norm_weight = _ptr(next_norm_weight)
            seam.next_eps = dst._eps if next_eps is None else next_eps
            seam.next_normed = _ffi.lib().xabe_moe_block_normed_mut(dst._h, C.byref(n))
            seam.next_normed_len = n.value
            seam.next_normed_h = _ffi.lib().xabe_moe_block_normed_h_mut(dst._h, C.byref(nh))
            seam.next_normed_h_len = nh.value
        check(_ffi.lib().xabe_moe_block_forward_seam(self._h, _stream(), C.byref(cw), _ptr(residual), residual.numel(), tokens,
                                                     _ptr(logit_bias), _ptr(ffn_out), 0 if ffn_out is None else ffn_out.numel(),
                                                     _ptr(l_out), l_out.numel(), C.byref(seam)))

    def forward_stage(self, w: MoeLayerWeights, residual, ffn_out, l_out, stage: int, logit_bias=None):
        """One of the three decode launches alone (measurement hook; see the header)."""
        cw = w._c()
        check(_ffi.lib().xabe_moe_block_forward_stage(self._h, _stream(), C.byref(cw), _ptr(residual), residual.numel(),
                                                      _ptr(logit_bias), _ptr(ffn_out), ffn_out.numel(), _ptr(l_out),
                                                      l_out.numel(), stage))

    def _view(self, name: str) -> torch.Tensor:
        n = C.c_size_t(0)
        p = getattr(_ffi.lib(), "xabe_moe_block_" + name)(self._h, C.byref(n))
        return _wrap(p, n.value, torch.float32)

    def normed(self): return self._view("normed")
    def router_logits(self): return self._view("router_logits")
    def routed(self): return self._view("routed")
    def shared_ungated(self): return self._view("shared_ungated")
    def shared_gate(self): return self._view("shared_gate")

    def buffers(self) -> MoeBuffers:
        return MoeBuffers(_ffi.lib().xabe_moe_block_buffers(self._h), owner=False)


def moe_block_forward_noalloc(geometry: MoeGeometry, w: MoeLayerWeights, residual, tokens: int, ffn_out, l_out,
                              logit_bias=None, eps: float = DEFAULT_RMS_EPS):
    """`MoeBlock.forward` at decode widths without a block: the working set lives in a device array the library
    holds statically, so the call allocates nothing (no counterpart in the reference; see the header)."""
    cw = w._c()
    check(_ffi.lib().xabe_moe_block_forward_noalloc(C.byref(geometry._c()), eps, _stream(), C.byref(cw), _ptr(residual),
                                                    residual.numel(), tokens, _ptr(logit_bias), _ptr(ffn_out),
                                                    ffn_out.numel(), _ptr(l_out), l_out.numel()))


@dataclass
class DenseFfnLayerWeights:
    post_norm: torch.Tensor
    gate: QuantTensor
    up: QuantTensor
    down: QuantTensor

    def _c(self) -> DenseLayerWeightsC:
        return DenseLayerWeightsC(_ptr(self.post_norm), self.gate._c(), self.up._c(), self.down._c())


class DenseFfnBlock:
    def __init__(self, hidden: int, intermediate: int, max_tokens: int, eps: float = DEFAULT_RMS_EPS):
        h = C.c_void_p()
        check(_ffi.lib().xabe_dense_ffn_block_new(hidden, intermediate, max_tokens, eps, _stream(), C.byref(h)))
        self._h = h.value
        self.hidden, self.intermediate, self.max_tokens = hidden, intermediate, max_tokens

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_dense_ffn_block_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def disable_tensor_cores(self): check(_ffi.lib().xabe_dense_ffn_block_disable_tensor_cores(self._h))

    def forward(self, w: DenseFfnLayerWeights, residual, tokens: int, ffn_out, l_out):
        cw = w._c()
        check(_ffi.lib().xabe_dense_ffn_block_forward(self._h, _stream(), C.byref(cw), _ptr(residual), residual.numel(),
                                                      tokens, _ptr(ffn_out), ffn_out.numel(), _ptr(l_out), l_out.numel()))

    def normed(self) -> torch.Tensor:
        n = C.c_size_t(0)
        p = _ffi.lib().xabe_dense_ffn_block_normed(self._h, C.byref(n))
        return _wrap(p, n.value, torch.float32)

    def publish_tokens(self, tokens: int):
        check(_ffi.lib().xabe_dense_ffn_block_publish_tokens(self._h, _stream(), tokens))

    def tensor_cores_enabled(self) -> bool:
        return bool(_ffi.lib().xabe_dense_ffn_block_tensor_cores_enabled(self._h))


class FfnKind(enum.IntEnum):
    MOE = 0
    DENSE = 1


@dataclass
class FfnConfig:
    """The fields of `ModelConfig` the feed-forward geometry is made from
    (crates/xabe-model/src/config.rs:126-187)."""
    kind: FfnKind
    hidden: int
    num_experts: int = 0
    experts_per_token: int = 0
    expert_intermediate: int = 0
    dense_intermediate: int = 0

    @staticmethod
    def qwen3_6_35b_a3b() -> "FfnConfig":
        return FfnConfig(FfnKind.MOE, 2048, 256, 8, 512, 0)

    @staticmethod
    def qwen3_8_27b() -> "FfnConfig":
        return FfnConfig(FfnKind.DENSE, 5120, 0, 0, 0, 17408)

    def _c(self) -> FfnConfigC:
        return FfnConfigC(int(self.kind), self.hidden, self.num_experts, self.experts_per_token,
                          self.expert_intermediate, self.dense_intermediate)


class FfnLayerWeights:
    """`FfnLayerWeights` (crates/xabe-engine/src/block/ffn.rs:43-48): one layer's weights, either kind."""

    def __init__(self, w):
        if isinstance(w, MoeLayerWeights):
            self.kind = FfnKind.MOE
        elif isinstance(w, DenseFfnLayerWeights):
            self.kind = FfnKind.DENSE
        else:
            raise TypeError("FfnLayerWeights wraps MoeLayerWeights or DenseFfnLayerWeights")
        self.inner = w

    def _c(self) -> FfnLayerWeightsC:
        c = FfnLayerWeightsC()
        c.kind = int(self.kind)
        if self.kind == FfnKind.MOE:
            c.moe = self.inner._c()
        else:
            c.dense = self.inner._c()
        return c


class FfnBlock:
    """`FfnBlock` (crates/xabe-engine/src/block/ffn.rs:27-228): the feed-forward block of one pass shape,
    MoE or dense, chosen once from the configuration."""

    @staticmethod
    def geometry_for(config: FfnConfig, block_size: int, max_tokens: int) -> MoeGeometry:
        g = Geometry()
        check(_ffi.lib().xabe_ffn_block_geometry_for(C.byref(config._c()), block_size, max_tokens, C.byref(g)))
        return MoeGeometry(g.num_experts, g.experts_per_token, g.hidden, g.intermediate, g.block_size, g.max_tokens)

    def __init__(self, config: FfnConfig, geometry: MoeGeometry, eps: float = DEFAULT_RMS_EPS):
        h = C.c_void_p()
        check(_ffi.lib().xabe_ffn_block_new(C.byref(config._c()), C.byref(geometry._c()), eps, _stream(), C.byref(h)))
        self._h = h.value

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_ffn_block_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def kind(self) -> FfnKind: return FfnKind(_ffi.lib().xabe_ffn_block_kind(self._h))
    def disable_tensor_cores(self): check(_ffi.lib().xabe_ffn_block_disable_tensor_cores(self._h))
    def tensor_cores_enabled(self) -> bool: return bool(_ffi.lib().xabe_ffn_block_tensor_cores_enabled(self._h))
    def set_exact_decode_regime(self, on: bool): check(_ffi.lib().xabe_ffn_block_set_exact_decode_regime(self._h, int(on)))

    def geometry(self) -> MoeGeometry:
        g = Geometry()
        check(_ffi.lib().xabe_ffn_block_geometry(self._h, C.byref(g)))
        return MoeGeometry(g.num_experts, g.experts_per_token, g.hidden, g.intermediate, g.block_size, g.max_tokens)

    def normed(self) -> torch.Tensor:
        n = C.c_size_t(0)
        p = _ffi.lib().xabe_ffn_block_normed(self._h, C.byref(n))
        return _wrap(p, n.value, torch.float32)

    def as_moe(self) -> Optional[MoeBlock]:
        """A borrowed view of the routed block, None on the dense path."""
        p = _ffi.lib().xabe_ffn_block_as_moe(self._h)
        return _BorrowedMoeBlock(p, self) if p else None

    def publish_tokens(self, tokens: int):
        check(_ffi.lib().xabe_ffn_block_publish_tokens(self._h, _stream(), tokens))

    def forward(self, w: FfnLayerWeights, residual, tokens: int, ffn_out, l_out):
        cw = w._c()
        check(_ffi.lib().xabe_ffn_block_forward(self._h, _stream(), C.byref(cw), _ptr(residual), residual.numel(), tokens,
                                                _ptr(ffn_out), ffn_out.numel(), _ptr(l_out), l_out.numel()))


class _BorrowedMoeBlock(MoeBlock):
    """A `MoeBlock` view over a handle another object owns (FfnBlock.as_moe)."""

    def __init__(self, handle, owner):  # noqa: D401 - no allocation here
        self._h = handle
        self._owner = owner
        self._geometry = owner.geometry()
        self._eps = None

    def __del__(self):
        self._h = None

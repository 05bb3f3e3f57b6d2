//! What `block/moe.rs` has to change.  The reference's block compiles two glue kernels for itself through NVRTC
//! (router logits, gate-and-combine: crates/xabe-engine/src/block/moe.rs:200-486); CUDA source strings do not cross
//! to HIP, so both are library calls here, and `MoeBlock::forward` (block/moe.rs:1091-1329) calls them in place of
//! its `launch_builder` blocks.  Better: it calls [`MoeBlockHandle::forward`], which runs the same eight steps as
//! three launches at decode widths (62 -> 31 us per three-token block) and forks the shared expert onto a side
//! stream at prefill widths, with the same values in `normed()`, `router_logits()`, `routed()`, `shared_ungated()`,
//! `shared_gate()` and `buffers()` afterwards.
use std::ffi::c_int;
use std::marker::PhantomData;
use std::sync::Arc;

use crate::driver::{HipSlice, HipStream, HipView};
use crate::ffi;
use crate::moe::{check, ExpertQuant, MoeBuffers, MoeError, MoeGeometry, MoeKernels, QuantTensor};

/// The router matrix as the layer holds it: f32 in the shipped file, Q8_0 in the synthetic benchmark layers.
pub enum Router<'a> {
    F32(&'a HipSlice<f32>),
    Q8_0(&'a HipSlice<u8>),
}

impl MoeKernels {
    /// `moe_block_router_logits*` (block/moe.rs:301-382, launch :1150-1184): logits[t][e] = W[e] . normed[t].
    pub fn router_logits(
        &self,
        stream: &Arc<HipStream>,
        buffers: &MoeBuffers,
        router: &Router<'_>,
        normed: &HipSlice<f32>,
        logits: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        let (ptr, len, quant) = match router {
            Router::F32(w) => (w.as_ptr().cast(), w.len(), -1),
            Router::Q8_0(w) => (w.as_ptr().cast(), w.len(), ExpertQuant::Q8_0 as c_int),
        };
        check(unsafe {
            ffi::xabe_moe_router_logits(self.raw, stream.raw(), buffers.raw, ptr, len, quant, normed.as_ptr(), normed.len(),
                                        logits.as_mut_ptr(), logits.len())
        })
    }
    /// `moe_block_gate_and_combine` (block/moe.rs:424-483, launch :1297-1326).
    #[allow(clippy::too_many_arguments)]
    pub fn gate_and_combine(
        &self,
        stream: &Arc<HipStream>,
        buffers: &MoeBuffers,
        shared_gate_inp: &HipSlice<f32>,
        normed: &HipSlice<f32>,
        shexp: &HipSlice<f32>,
        residual: &HipSlice<f32>,
        gate: &mut HipSlice<f32>,
        routed: &mut HipSlice<f32>,
        ffn_out: &mut HipSlice<f32>,
        l_out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_moe_gate_and_combine(self.raw, stream.raw(), buffers.raw, shared_gate_inp.as_ptr(), normed.as_ptr(),
                                           shexp.as_ptr(), residual.as_ptr(), gate.as_mut_ptr(), routed.as_mut_ptr(),
                                           ffn_out.as_mut_ptr(), l_out.as_mut_ptr())
        })
    }
}

/// Device tensors of one layer, borrowed for a call (block/moe.rs:634-658 `MoeLayerWeights`).
pub struct MoeLayerWeights<'a> {
    pub post_norm: &'a HipSlice<f32>,
    pub router: Router<'a>,
    pub gate_exps: QuantTensor<'a>,
    pub up_exps: QuantTensor<'a>,
    pub down_exps: QuantTensor<'a>,
    pub shared_gate_inp: &'a HipSlice<f32>,
    pub shared_gate: QuantTensor<'a>,
    pub shared_up: QuantTensor<'a>,
    pub shared_down: QuantTensor<'a>,
}
impl MoeLayerWeights<'_> {
    fn raw(&self) -> ffi::xabe_moe_layer_weights {
        let (router, router_quant) = match &self.router {
            Router::F32(w) => (w.as_ptr().cast(), -1),
            Router::Q8_0(w) => (w.as_ptr().cast(), ExpertQuant::Q8_0 as c_int),
        };
        ffi::xabe_moe_layer_weights {
            post_norm: self.post_norm.as_ptr(),
            router,
            router_quant,
            gate_exps: self.gate_exps.raw(),
            up_exps: self.up_exps.raw(),
            down_exps: self.down_exps.raw(),
            shared_gate_inp: self.shared_gate_inp.as_ptr(),
            shared_gate: self.shared_gate.raw(),
            shared_up: self.shared_up.raw(),
            shared_down: self.shared_down.raw(),
        }
    }
}

/// The seam to the next layer (reference: docs/BENCHMARKS.md:1376, :1761): the launch that finishes `l_out` also
/// writes the next layer's normalised rows, and a block can start from rows a previous call left in its buffers.
#[derive(Default)]
pub struct Seam<'a> {
    pub input_normed: bool,
    pub skip_readback: bool,
    /// the next layer's post-mixer norm weight and the block whose normalised-rows buffers receive the result
    pub next: Option<(&'a HipSlice<f32>, f32, &'a MoeBlockHandle)>,
}

/// `MoeBlock` (block/moe.rs:895-1330) as one library object: kernels, buffers and the block's scratch.
pub struct MoeBlockHandle {
    raw: *mut ffi::xabe_moe_block,
    geometry: MoeGeometry,
}
unsafe impl Send for MoeBlockHandle {}
macro_rules! readback {
    ($name:ident, $f:ident) => {
        pub fn $name(&self) -> HipView<'_, f32> {
            let mut len = 0usize;
            let ptr = unsafe { ffi::$f(self.raw, &mut len) };
            HipView { ptr, len, _owner: PhantomData }
        }
    };
}
impl MoeBlockHandle {
    pub fn new(stream: &Arc<HipStream>, geometry: MoeGeometry, eps: f32) -> Result<Self, MoeError> {
        let g = ffi::xabe_moe_geometry {
            num_experts: geometry.num_experts,
            experts_per_token: geometry.experts_per_token,
            hidden: geometry.hidden,
            intermediate: geometry.intermediate,
            block_size: geometry.block_size,
            max_tokens: geometry.max_tokens,
        };
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_moe_block_new(&g, eps, stream.raw(), &mut raw) })?;
        Ok(Self { raw, geometry })
    }
    pub fn geometry(&self) -> MoeGeometry {
        self.geometry
    }
    pub(crate) fn raw_mut(&mut self) -> *mut ffi::xabe_moe_block {
        self.raw
    }
    /// block/moe.rs:1081-1089: outside graph capture.
    pub fn publish_tokens(&mut self, stream: &Arc<HipStream>, tokens: usize) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_block_publish_tokens(self.raw, stream.raw(), tokens) })
    }
    /// block/moe.rs:1091-1329
    pub fn forward(
        &mut self,
        stream: &Arc<HipStream>,
        w: &MoeLayerWeights<'_>,
        residual: &HipSlice<f32>,
        tokens: usize,
        ffn_out: &mut HipSlice<f32>,
        l_out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        let cw = w.raw();
        check(unsafe {
            ffi::xabe_moe_block_forward(self.raw, stream.raw(), &cw, residual.as_ptr(), residual.len(), tokens, std::ptr::null(),
                                        ffn_out.as_mut_ptr(), ffn_out.len(), l_out.as_mut_ptr(), l_out.len())
        })
    }
    /// `forward` across the seam; `ffn_out` may be `None`.
    #[allow(clippy::too_many_arguments)]
    pub fn forward_seam(
        &mut self,
        stream: &Arc<HipStream>,
        w: &MoeLayerWeights<'_>,
        residual: &HipSlice<f32>,
        tokens: usize,
        ffn_out: Option<&mut HipSlice<f32>>,
        l_out: &mut HipSlice<f32>,
        seam: &Seam<'_>,
    ) -> Result<(), MoeError> {
        let cw = w.raw();
        let mut cs = ffi::xabe_moe_seam {
            input_normed: seam.input_normed as c_int,
            skip_readback: seam.skip_readback as c_int,
            next_norm_weight: std::ptr::null(),
            next_eps: 0.0,
            next_normed: std::ptr::null_mut(),
            next_normed_len: 0,
            next_normed_h: std::ptr::null_mut(),
            next_normed_h_len: 0,
        };
        if let Some((weight, eps, next)) = seam.next {
            cs.next_norm_weight = weight.as_ptr();
            cs.next_eps = eps;
            cs.next_normed = unsafe { ffi::xabe_moe_block_normed_mut(next.raw, &mut cs.next_normed_len) };
            cs.next_normed_h = unsafe { ffi::xabe_moe_block_normed_h_mut(next.raw, &mut cs.next_normed_h_len) };
        }
        let (fp, fl) = match ffn_out {
            Some(f) => (f.as_mut_ptr(), f.len()),
            None => (std::ptr::null_mut(), 0),
        };
        check(unsafe {
            ffi::xabe_moe_block_forward_seam(self.raw, stream.raw(), &cw, residual.as_ptr(), residual.len(), tokens,
                                             std::ptr::null(), fp, fl, l_out.as_mut_ptr(), l_out.len(), &cs)
        })
    }
    pub fn disable_tensor_cores(&mut self) {
        unsafe { ffi::xabe_moe_block_disable_tensor_cores(self.raw) };
    }
    pub fn set_exact_decode_regime(&mut self, on: bool) {
        unsafe { ffi::xabe_moe_block_set_exact_decode_regime(self.raw, on as c_int) };
    }
    pub fn tensor_cores_enabled(&self) -> bool {
        unsafe { ffi::xabe_moe_block_tensor_cores_enabled(self.raw) != 0 }
    }
    readback!(normed, xabe_moe_block_normed);
    readback!(router_logits, xabe_moe_block_router_logits);
    readback!(routed, xabe_moe_block_routed);
    readback!(shared_ungated, xabe_moe_block_shared_ungated);
    readback!(shared_gate, xabe_moe_block_shared_gate);
}
impl Drop for MoeBlockHandle {
    fn drop(&mut self) {
        unsafe { ffi::xabe_moe_block_free(self.raw) }
    }
}

/// `MoeBlockHandle::forward` at decode widths for callers that cannot allocate device memory (no counterpart in the
/// reference): no handle, the block's working set sits in a device array the library holds statically on each GPU.
/// Limit: `max_tokens` <= 32, hidden <= 2048, intermediate <= 512, <= 512 experts, top-k <= 8; calls that overlap on
/// one GPU race; the first call on a device must not be under stream capture.
#[allow(clippy::too_many_arguments)]
pub fn block_forward_noalloc(
    stream: &Arc<HipStream>,
    geometry: &MoeGeometry,
    eps: f32,
    w: &MoeLayerWeights<'_>,
    residual: &HipSlice<f32>,
    tokens: usize,
    ffn_out: &mut HipSlice<f32>,
    l_out: &mut HipSlice<f32>,
) -> Result<(), MoeError> {
    let g = ffi::xabe_moe_geometry {
        num_experts: geometry.num_experts,
        experts_per_token: geometry.experts_per_token,
        hidden: geometry.hidden,
        intermediate: geometry.intermediate,
        block_size: geometry.block_size,
        max_tokens: geometry.max_tokens,
    };
    let cw = w.raw();
    check(unsafe {
        ffi::xabe_moe_block_forward_noalloc(&g, eps, stream.raw(), &cw, residual.as_ptr(), residual.len(), tokens, std::ptr::null(),
                                            ffn_out.as_mut_ptr(), ffn_out.len(), l_out.as_mut_ptr(), l_out.len())
    })
}

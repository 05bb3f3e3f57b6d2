//! The dense-sibling SwiGLU block (crates/xabe-engine/src/block/dense_ffn.rs:1047-1178): RMSNorm, gate/up + SwiGLU,
//! down, residual add, on the same kernels as the MoE block's shared expert.
//!
//! UNCOMPILED SOURCE (no Rust toolchain in the image this repository is built in).
use std::marker::PhantomData;
use std::sync::Arc;

use crate::driver::{HipSlice, HipStream, HipView};
use crate::ffi;
use crate::moe::{check, MoeError, QuantTensor};

/// dense_ffn.rs:640-700 `DenseFfnLayerWeights`: device tensors of one layer, borrowed for a call.
pub struct DenseFfnLayerWeights<'a> {
    pub post_norm: &'a HipSlice<f32>,
    pub gate: QuantTensor<'a>,
    pub up: QuantTensor<'a>,
    pub down: QuantTensor<'a>,
}
impl DenseFfnLayerWeights<'_> {
    pub(crate) fn raw(&self) -> ffi::xabe_dense_ffn_layer_weights {
        ffi::xabe_dense_ffn_layer_weights {
            post_norm: self.post_norm.as_ptr(),
            gate: self.gate.raw(),
            up: self.up.raw(),
            down: self.down.raw(),
        }
    }
}

/// `DenseFfnBlock` (dense_ffn.rs:836-1178) as one library object.
pub struct DenseFfnBlock {
    raw: *mut ffi::xabe_dense_ffn_block,
    hidden: usize,
    max_tokens: usize,
}
unsafe impl Send for DenseFfnBlock {}
impl DenseFfnBlock {
    pub fn new(stream: &Arc<HipStream>, hidden: usize, intermediate: usize, max_tokens: usize, eps: f32) -> Result<Self, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_dense_ffn_block_new(hidden, intermediate, max_tokens, eps, stream.raw(), &mut raw) })?;
        Ok(Self { raw, hidden, max_tokens })
    }
    /// Outside graph capture, as `MoeBlock::publish_tokens`.
    pub fn publish_tokens(&mut self, stream: &Arc<HipStream>, tokens: usize) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_dense_ffn_block_publish_tokens(self.raw, stream.raw(), tokens) })
    }
    /// dense_ffn.rs:1047-1178
    pub fn forward(
        &mut self,
        stream: &Arc<HipStream>,
        w: &DenseFfnLayerWeights<'_>,
        residual: &HipSlice<f32>,
        tokens: usize,
        ffn_out: &mut HipSlice<f32>,
        l_out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        let cw = w.raw();
        check(unsafe {
            ffi::xabe_dense_ffn_block_forward(self.raw, stream.raw(), &cw, residual.as_ptr(), residual.len(), tokens,
                                              ffn_out.as_mut_ptr(), ffn_out.len(), l_out.as_mut_ptr(), l_out.len())
        })
    }
    pub(crate) fn raw_mut(&mut self) -> *mut ffi::xabe_dense_ffn_block {
        self.raw
    }
    pub fn disable_tensor_cores(&mut self) {
        unsafe { ffi::xabe_dense_ffn_block_disable_tensor_cores(self.raw) };
    }
    pub fn tensor_cores_enabled(&self) -> bool {
        unsafe { ffi::xabe_dense_ffn_block_tensor_cores_enabled(self.raw) != 0 }
    }
    /// The normalised rows of the last pass, `[max_tokens][hidden]`.
    pub fn normed(&self) -> HipView<'_, f32> {
        let mut len = 0usize;
        let ptr = unsafe { ffi::xabe_dense_ffn_block_normed(self.raw, &mut len) };
        debug_assert_eq!(len, self.max_tokens * self.hidden);
        HipView { ptr, len, _owner: PhantomData }
    }
}
impl Drop for DenseFfnBlock {
    fn drop(&mut self) {
        unsafe { ffi::xabe_dense_ffn_block_free(self.raw) }
    }
}

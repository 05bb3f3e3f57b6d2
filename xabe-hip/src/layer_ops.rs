//! `LayerOpsKernels::rms_norm` (crates/xabe-cuda/src/kernels/layer_ops.rs:777-805): every row of the buffer,
//! `x * (1 / sqrt(mean(x^2) + eps)) * w`.  The other members of the reference's `LayerOpsKernels` belong to the
//! mixers and are not part of this crate.
use std::sync::Arc;

use crate::driver::{HipSlice, HipStream};
use crate::ffi;
use crate::moe::{check, MoeError};

pub struct LayerOpsKernels;
impl LayerOpsKernels {
    pub fn new() -> Self {
        Self
    }
    #[allow(clippy::too_many_arguments)]
    pub fn rms_norm(
        &self,
        stream: &Arc<HipStream>,
        x: &HipSlice<f32>,
        weight: &HipSlice<f32>,
        out: &mut HipSlice<f32>,
        rows: usize,
        width: usize,
        eps: f32,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_rms_norm(stream.raw(), x.as_ptr(), x.len(), weight.as_ptr(), weight.len(), out.as_mut_ptr(), out.len(),
                               rows, width, eps)
        })
    }
}
impl Default for LayerOpsKernels {
    fn default() -> Self {
        Self::new()
    }
}

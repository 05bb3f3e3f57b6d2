//! `LmHeadKernels` (crates/xabe-cuda/src/kernels/lm_head.rs:1500-2044): logits[t][v] = W[v] . hidden[t] over a
//! quantized or 16-bit head, and the device half of greedy sampling.
//!
//! UNCOMPILED SOURCE (no Rust toolchain in the image this repository is built in).
use std::ffi::c_int;
use std::sync::Arc;

use crate::driver::{HipSlice, HipStream};
use crate::ffi;
use crate::moe::{check, MoeError};

/// lm_head.rs:169
pub const ARGMAX_BLOCKS: usize = ffi::XABE_LM_HEAD_ARGMAX_BLOCKS;
/// Tokens one pass over the weights serves (the reference's tile is 8; byte accounting goes through
/// [`LmHeadGeometry::weight_passes`]).
pub const MAX_BATCH_TILE: usize = ffi::XABE_LM_HEAD_MAX_BATCH_TILE;

/// lm_head.rs `HeadFormat`; the community formats are recognised and refused (`UnsupportedExpertType`).
#[repr(i32)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum HeadFormat {
    Q8_0 = 0,
    Bf16 = 1,
    Q6K = 2,
    F16 = 3,
    Q4_0 = 4,
    Q4K = 5,
    Q5K = 6,
}

/// The head matrix as the file holds it: `[vocab][hidden]` rows, bytes on the device.
pub struct HeadTensor<'a> {
    pub bytes: &'a HipSlice<u8>,
    pub format: HeadFormat,
}

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct LmHeadGeometry {
    pub hidden: usize,
    pub vocab: usize,
    pub max_tokens: usize,
}
impl LmHeadGeometry {
    fn raw(&self) -> ffi::xabe_lm_head_geometry {
        ffi::xabe_lm_head_geometry { hidden: self.hidden, vocab: self.vocab, max_tokens: self.max_tokens }
    }
    pub fn qwen3_6(max_tokens: usize) -> Self {
        let g = unsafe { ffi::xabe_lm_head_geometry_qwen3_6(max_tokens) };
        Self { hidden: g.hidden, vocab: g.vocab, max_tokens: g.max_tokens }
    }
    pub fn row_bytes_for(&self, format: HeadFormat) -> usize {
        unsafe { ffi::xabe_lm_head_row_bytes_for(&self.raw(), format as c_int) }
    }
    pub fn weight_bytes_for(&self, format: HeadFormat) -> usize {
        unsafe { ffi::xabe_lm_head_weight_bytes_for(&self.raw(), format as c_int) }
    }
    pub fn elements(&self) -> usize {
        unsafe { ffi::xabe_lm_head_elements(&self.raw()) }
    }
    pub fn weight_passes(&self, tokens: usize) -> usize {
        unsafe { ffi::xabe_lm_head_weight_passes(&self.raw(), tokens) }
    }
    pub fn weight_bytes_read(&self, format: HeadFormat, tokens: usize) -> usize {
        unsafe { ffi::xabe_lm_head_weight_bytes_read(&self.raw(), format as c_int, tokens) }
    }
}

pub struct LmHeadKernels {
    raw: *mut ffi::xabe_lm_head,
    geometry: LmHeadGeometry,
}
unsafe impl Send for LmHeadKernels {}
impl LmHeadKernels {
    /// lm_head.rs:1640-1678
    pub fn new(geometry: LmHeadGeometry) -> Result<Self, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_lm_head_new(&geometry.raw(), &mut raw) })?;
        Ok(Self { raw, geometry })
    }
    pub fn geometry(&self) -> LmHeadGeometry {
        self.geometry
    }
    /// lm_head.rs:1694-1935: `logits` is `[max_tokens][vocab]`, rows past `tokens` are left alone.
    pub fn forward(
        &self,
        stream: &Arc<HipStream>,
        weight: &HeadTensor<'_>,
        hidden_states: &HipSlice<f32>,
        tokens: usize,
        logits: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_lm_head_forward(self.raw, stream.raw(), weight.format as c_int, weight.bytes.as_ptr().cast(),
                                      weight.bytes.len(), hidden_states.as_ptr(), hidden_states.len(), tokens,
                                      logits.as_mut_ptr(), logits.len())
        })
    }
    /// lm_head.rs:1937-2003: index of the largest of the first `n` values (lowest index among equals, NaN ignored).
    pub fn argmax(
        &self,
        stream: &Arc<HipStream>,
        values: &HipSlice<f32>,
        n: usize,
        partial_values: &mut HipSlice<f32>,
        partial_indices: &mut HipSlice<i32>,
        out: &mut HipSlice<i32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_lm_head_argmax(self.raw, stream.raw(), values.as_ptr(), values.len(), n, partial_values.as_mut_ptr(),
                                     partial_values.len(), partial_indices.as_mut_ptr(), partial_indices.len(),
                                     out.as_mut_ptr(), out.len())
        })
    }
    /// lm_head.rs:2005-2044: 1 / sum(exp(x - max)) over the first `n` values, the winner's probability.
    pub fn argmax_prob(&self, stream: &Arc<HipStream>, values: &HipSlice<f32>, n: usize, out: &mut HipSlice<f32>) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_lm_head_argmax_prob(self.raw, stream.raw(), values.as_ptr(), values.len(), n, out.as_mut_ptr(), out.len())
        })
    }
}
impl Drop for LmHeadKernels {
    fn drop(&mut self) {
        unsafe { ffi::xabe_lm_head_free(self.raw) }
    }
}

//! Weight ingest over the C ABI: the GGUF container and the upload of one layer's tensors in the formats the file
//! holds (`MoeLayerWeights::upload`, block/moe.rs:660-756; `DenseFfnLayerWeights::upload`, dense_ffn.rs:700-780).
//! A Rust engine can keep `xabe-gguf` (plain Rust, no CUDA) and use only the two upload functions.
//!
//! UNCOMPILED SOURCE (no Rust toolchain in the image this repository is built in).
use std::ffi::{c_int, CString};
use std::marker::PhantomData;
use std::sync::Arc;

use crate::block::MoeBlockHandle;
use crate::dense::DenseFfnBlock;
use crate::driver::{HipSlice, HipStream};
use crate::ffi;
use crate::moe::{check, MoeError, MoeGeometry};

/// A memory-mapped GGUF v3 file (crates/xabe-gguf/src/lib.rs `GgufFile`).
pub struct GgufFile {
    raw: *mut ffi::xabe_gguf_file,
}
unsafe impl Send for GgufFile {}
impl GgufFile {
    pub fn open(path: &str) -> Result<Self, MoeError> {
        let c = CString::new(path).map_err(|e| MoeError::InvalidArgument(e.to_string()))?;
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_gguf_open(c.as_ptr(), &mut raw) })?;
        Ok(Self { raw })
    }
    pub fn version(&self) -> u32 {
        unsafe { ffi::xabe_gguf_version(self.raw) }
    }
    pub fn n_tensors(&self) -> usize {
        unsafe { ffi::xabe_gguf_n_tensors(self.raw) }
    }
    pub fn get_u32(&self, key: &str) -> Result<u32, MoeError> {
        let c = CString::new(key).map_err(|e| MoeError::InvalidArgument(e.to_string()))?;
        let mut v = 0u32;
        check(unsafe { ffi::xabe_gguf_get_u32(self.raw, c.as_ptr(), &mut v) })?;
        Ok(v)
    }
    pub fn get_f32(&self, key: &str) -> Result<f32, MoeError> {
        let c = CString::new(key).map_err(|e| MoeError::InvalidArgument(e.to_string()))?;
        let mut v = 0f32;
        check(unsafe { ffi::xabe_gguf_get_f32(self.raw, c.as_ptr(), &mut v) })?;
        Ok(v)
    }
}
impl Drop for GgufFile {
    fn drop(&mut self) {
        unsafe { ffi::xabe_gguf_close(self.raw) }
    }
}

fn raw_geometry(g: &MoeGeometry) -> ffi::xabe_moe_geometry {
    ffi::xabe_moe_geometry {
        num_experts: g.num_experts,
        experts_per_token: g.experts_per_token,
        hidden: g.hidden,
        intermediate: g.intermediate,
        block_size: g.block_size,
        max_tokens: g.max_tokens,
    }
}

/// One MoE layer's tensors on the device, owned by the library (block/moe.rs:660-756).  `_upload` allocates and
/// synchronises the stream: model load, not the forward path.
pub struct UploadedMoeLayer {
    raw: *mut ffi::xabe_moe_layer,
}
unsafe impl Send for UploadedMoeLayer {}
impl UploadedMoeLayer {
    pub fn upload(stream: &Arc<HipStream>, file: &GgufFile, layer: u32, geometry: &MoeGeometry) -> Result<Self, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_moe_layer_upload(stream.raw(), file.raw, layer, &raw_geometry(geometry), &mut raw) })?;
        Ok(Self { raw })
    }
    /// gate / up / down formats of the expert stacks (`XABE_QUANT_*`).
    pub fn expert_quants(&self) -> Result<[i32; 3], MoeError> {
        let mut q: [c_int; 3] = [0; 3];
        check(unsafe { ffi::xabe_moe_layer_expert_quants(self.raw, q.as_mut_ptr()) })?;
        Ok(q)
    }
    pub fn bytes(&self) -> usize {
        unsafe { ffi::xabe_moe_layer_bytes(self.raw) }
    }
    /// One block pass over this layer's tensors (what `MoeBlock::forward` does with its `MoeLayerWeights`).
    #[allow(clippy::too_many_arguments)]
    pub fn forward(
        &self,
        block: &mut MoeBlockHandle,
        stream: &Arc<HipStream>,
        residual: &HipSlice<f32>,
        tokens: usize,
        ffn_out: &mut HipSlice<f32>,
        l_out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        let w = unsafe { ffi::xabe_moe_layer_weights_of(self.raw) };
        check(unsafe {
            ffi::xabe_moe_block_forward(block.raw_mut(), stream.raw(), w, residual.as_ptr(), residual.len(), tokens,
                                        std::ptr::null(), ffn_out.as_mut_ptr(), ffn_out.len(), l_out.as_mut_ptr(), l_out.len())
        })
    }
}
impl Drop for UploadedMoeLayer {
    fn drop(&mut self) {
        unsafe { ffi::xabe_moe_layer_free(self.raw) }
    }
}

/// One dense layer's tensors on the device (dense_ffn.rs:700-780).
pub struct UploadedDenseFfnLayer {
    raw: *mut ffi::xabe_dense_ffn_layer,
    _not_sync: PhantomData<*mut ()>,
}
unsafe impl Send for UploadedDenseFfnLayer {}
impl UploadedDenseFfnLayer {
    pub fn upload(stream: &Arc<HipStream>, file: &GgufFile, layer: u32, hidden: usize, intermediate: usize) -> Result<Self, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_dense_ffn_layer_upload(stream.raw(), file.raw, layer, hidden, intermediate, &mut raw) })?;
        Ok(Self { raw, _not_sync: PhantomData })
    }
    pub fn bytes(&self) -> usize {
        unsafe { ffi::xabe_dense_ffn_layer_bytes(self.raw) }
    }
    pub fn forward(
        &self,
        block: &mut DenseFfnBlock,
        stream: &Arc<HipStream>,
        residual: &HipSlice<f32>,
        tokens: usize,
        ffn_out: &mut HipSlice<f32>,
        l_out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        let w = unsafe { ffi::xabe_dense_ffn_layer_weights_of(self.raw) };
        check(unsafe {
            ffi::xabe_dense_ffn_block_forward(block.raw_mut(), stream.raw(), w, residual.as_ptr(), residual.len(), tokens,
                                              ffn_out.as_mut_ptr(), ffn_out.len(), l_out.as_mut_ptr(), l_out.len())
        })
    }
}
impl Drop for UploadedDenseFfnLayer {
    fn drop(&mut self) {
        unsafe { ffi::xabe_dense_ffn_layer_free(self.raw) }
    }
}

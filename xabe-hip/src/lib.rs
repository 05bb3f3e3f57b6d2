//! `xabe-hip`: the quantized MoE feed-forward block of llmxabe on one MI355X, behind the names
//! `xabe_cuda::kernels::moe` exports (crates/xabe-cuda/src/kernels/moe.rs) so that `xabe-engine`'s block code
//! compiles against it with its `use` lines changed and little else.
//!
//! UNCOMPILED SOURCE: the image this repository is built in has no Rust toolchain.  `ffi` is generated from the C
//! headers; everything else in this crate is a thin, arithmetic-free wrapper over it.
//!
//! Layout
//! * [`ffi`]     raw `extern "C"` declarations (generated: `python xabe-hip/gen_ffi.py`)
//! * [`driver`]  `HipContext` / `HipStream` / `HipSlice<T>`: cudarc-shaped owners of device memory and streams
//! * [`moe`]     `MoeGeometry`, `ExpertQuant`, `QuantTensor`, `MoeKernels`, `MoeBuffers`, `BufferScope`, `MoeError`,
//!               `to_device_layout`, `BLOCK_Q6_K_DEVICE_BYTES`
//! * [`layer_ops`] `LayerOpsKernels::rms_norm`
//! * [`block`]   what `block/moe.rs` compiled for itself through NVRTC (router logits, gate-and-combine) as library
//!               calls, and the whole-block entry points (`MoeBlockHandle`: three launches at decode widths, the
//!               seam to the next layer's RMSNorm; `block_forward_noalloc`)
//! * [`dense`]   `DenseFfnBlock`, `DenseFfnLayerWeights`
//! * [`lm_head`] `LmHeadKernels`, `LmHeadGeometry`, `HeadTensor`, `HeadFormat`
//! * [`weights`] `GgufFile` and the upload of a layer's tensors (`UploadedMoeLayer`, `UploadedDenseFfnLayer`)
pub mod block;
pub mod dense;
pub mod driver;
pub mod ffi;
pub mod layer_ops;
pub mod lm_head;
pub mod moe;
pub mod weights;

pub use driver::{DriverError, HipContext, HipSlice, HipStream};
pub use moe::{
    to_device_layout, BufferScope, ExpertQuant, MoeBuffers, MoeError, MoeGeometry, MoeKernels, QuantTensor,
    BLOCK_Q6_K_DEVICE_BYTES,
};

//! The launch API under the reference's names (crates/xabe-cuda/src/kernels/moe.rs: `MoeGeometry` :4523-4598,
//! `ExpertQuant` :298-401, `QuantTensor` :448-464, `MoeError` :4602-4637, `BufferScope` :4699-4705, `MoeBuffers`
//! :4713-4864, `MoeKernels` :4969-6714), each method one call into libxabe_hip.
//!
//! Differences a caller sees, all deliberate: `to_device_layout` is the identity (the kernels stream the file's
//! 210-byte Q6_K stride, so `BLOCK_Q6_K_DEVICE_BYTES` is 210, not 224); `shared_expert_mma` takes the quantized
//! stacks directly (there is no `SharedExpertInt8::repack`); the community formats and mixed gate/up formats are
//! rejected with `MoeError::UnsupportedExpertType`.
use std::borrow::Cow;
use std::ffi::{c_int, CStr};
use std::marker::PhantomData;
use std::sync::Arc;

use crate::driver::{DriverError, HipContext, HipSlice, HipStream, HipView};
use crate::ffi;

pub const BLOCK_Q6_K_DEVICE_BYTES: usize = 210;

/// Same fields, same order (moe.rs:4523-4540); `#[repr(C)]` because it crosses the boundary by value.
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct MoeGeometry {
    pub num_experts: usize,
    pub experts_per_token: usize,
    pub hidden: usize,
    pub intermediate: usize,
    pub block_size: usize,
    pub max_tokens: usize,
}
impl MoeGeometry {
    fn raw(&self) -> ffi::xabe_moe_geometry {
        ffi::xabe_moe_geometry {
            num_experts: self.num_experts,
            experts_per_token: self.experts_per_token,
            hidden: self.hidden,
            intermediate: self.intermediate,
            block_size: self.block_size,
            max_tokens: self.max_tokens,
        }
    }
    /// moe.rs:4542-4554
    pub fn qwen3_6(block_size: usize, max_tokens: usize) -> Self {
        let g = unsafe { ffi::xabe_moe_geometry_qwen3_6(block_size, max_tokens) };
        Self {
            num_experts: g.num_experts,
            experts_per_token: g.experts_per_token,
            hidden: g.hidden,
            intermediate: g.intermediate,
            block_size: g.block_size,
            max_tokens: g.max_tokens,
        }
    }
    pub fn max_flat_pairs(&self) -> usize {
        unsafe { ffi::xabe_moe_geometry_max_flat_pairs(&self.raw()) }
    }
    pub fn sorted_capacity(&self) -> usize {
        unsafe { ffi::xabe_moe_geometry_sorted_capacity(&self.raw()) }
    }
    pub fn expert_block_capacity(&self) -> usize {
        unsafe { ffi::xabe_moe_geometry_expert_block_capacity(&self.raw()) }
    }
    pub fn stack_elements(&self) -> usize {
        unsafe { ffi::xabe_moe_geometry_stack_elements(&self.raw()) }
    }
}

/// moe.rs:298-315; the discriminants are the C ABI's codes.
#[repr(i32)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum ExpertQuant {
    Q6K = 0,
    Q8_0 = 1,
    Q4_0 = 2,
    Q4K = 3,
    Q5K = 4,
}
impl ExpertQuant {
    pub fn block_elements(self) -> usize {
        unsafe { ffi::xabe_expert_quant_block_elements(self as c_int) }
    }
    pub fn file_block_bytes(self) -> usize {
        unsafe { ffi::xabe_expert_quant_file_block_bytes(self as c_int) }
    }
    pub fn block_bytes(self) -> usize {
        unsafe { ffi::xabe_expert_quant_block_bytes(self as c_int) }
    }
    pub fn is_community(self) -> bool {
        unsafe { ffi::xabe_expert_quant_is_community(self as c_int) != 0 }
    }
}

/// moe.rs:410-444.  The identity here: callers only ever pass its result to an upload.
pub fn to_device_layout(_quant: ExpertQuant, bytes: &[u8]) -> Cow<'_, [u8]> {
    Cow::Borrowed(bytes)
}

/// moe.rs:448-453
#[derive(Clone, Copy)]
pub struct QuantTensor<'a> {
    pub bytes: &'a HipSlice<u8>,
    pub quant: ExpertQuant,
}
impl QuantTensor<'_> {
    pub(crate) fn raw(&self) -> ffi::xabe_quant_tensor {
        ffi::xabe_quant_tensor { bytes: self.bytes.as_ptr().cast(), len: self.bytes.len(), quant: self.quant as c_int }
    }
}

/// `MoeError` (moe.rs:4602-4637) and the `MoeBlockError` variants that reach this boundary (block/moe.rs:494-547).
/// The library formats the message with the reference's wording; the structured fields of the reference's variants
/// are inside that text.
#[derive(Debug, Clone)]
pub enum MoeError {
    Compile(String),
    Driver(String),
    Mma(String),
    UnsupportedGeometry(String),
    RaggedWeights(String),
    WrongElementCount(String),
    TooManyTokens(String),
    SharedOnlyBuffers(String),
    BufferLength(String),
    InvalidArgument(String),
    UnsupportedExpertType(String),
    FfnKindMismatch(String),
    Other { status: i32, message: String },
}
impl std::fmt::Display for MoeError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        use MoeError::*;
        match self {
            Compile(m) | Driver(m) | Mma(m) | UnsupportedGeometry(m) | RaggedWeights(m) | WrongElementCount(m)
            | TooManyTokens(m) | SharedOnlyBuffers(m) | BufferLength(m) | InvalidArgument(m) | UnsupportedExpertType(m)
            | FfnKindMismatch(m) => f.write_str(m),
            Other { status, message } => write!(f, "status {status}: {message}"),
        }
    }
}
impl std::error::Error for MoeError {}
impl From<DriverError> for MoeError {
    fn from(e: DriverError) -> Self {
        MoeError::Driver(e.to_string())
    }
}

pub(crate) fn check(status: c_int) -> Result<(), MoeError> {
    if status == ffi::XABE_OK {
        return Ok(());
    }
    let message = unsafe { CStr::from_ptr(ffi::xabe_last_error()) }.to_string_lossy().into_owned();
    Err(match status {
        ffi::XABE_ERR_COMPILE => MoeError::Compile(message),
        ffi::XABE_ERR_DRIVER => MoeError::Driver(message),
        ffi::XABE_ERR_MMA => MoeError::Mma(message),
        ffi::XABE_ERR_UNSUPPORTED_GEOMETRY => MoeError::UnsupportedGeometry(message),
        ffi::XABE_ERR_RAGGED_WEIGHTS => MoeError::RaggedWeights(message),
        ffi::XABE_ERR_WRONG_ELEMENT_COUNT => MoeError::WrongElementCount(message),
        ffi::XABE_ERR_TOO_MANY_TOKENS => MoeError::TooManyTokens(message),
        ffi::XABE_ERR_SHARED_ONLY_BUFFERS => MoeError::SharedOnlyBuffers(message),
        ffi::XABE_ERR_BUFFER_LENGTH => MoeError::BufferLength(message),
        ffi::XABE_ERR_INVALID_ARGUMENT => MoeError::InvalidArgument(message),
        ffi::XABE_ERR_UNSUPPORTED_QUANT => MoeError::UnsupportedExpertType(message),
        ffi::XABE_ERR_FFN_KIND_MISMATCH => MoeError::FfnKindMismatch(message),
        status => MoeError::Other { status, message },
    })
}

/// moe.rs:4699-4705
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum BufferScope {
    Routed,
    SharedOnly,
}

/// moe.rs:4713-4766: every scratch buffer of the path, allocated once by [`MoeKernels::buffers`], sized from the
/// geometry only.  The library owns the memory; the accessors hand out views.
pub struct MoeBuffers {
    pub(crate) raw: *mut ffi::xabe_moe_buffers,
}
unsafe impl Send for MoeBuffers {}
macro_rules! view {
    ($name:ident, $t:ty, $f:ident) => {
        pub fn $name(&self) -> HipView<'_, $t> {
            let mut len = 0usize;
            let ptr = unsafe { ffi::$f(self.raw, &mut len) };
            HipView { ptr: ptr as *const $t, len, _owner: PhantomData }
        }
    };
}
impl MoeBuffers {
    pub fn scope(&self) -> BufferScope {
        if unsafe { ffi::xabe_moe_buffers_scope(self.raw) } == ffi::XABE_SCOPE_SHARED_ONLY {
            BufferScope::SharedOnly
        } else {
            BufferScope::Routed
        }
    }
    view!(topk_ids, i32, xabe_moe_buffers_topk_ids);
    view!(topk_weights, f32, xabe_moe_buffers_topk_weights);
    view!(sorted_token_ids, i32, xabe_moe_buffers_sorted_token_ids);
    view!(expert_ids, i32, xabe_moe_buffers_expert_ids);
    view!(bucket_live, i32, xabe_moe_buffers_bucket_live);
    view!(num_tokens_post_pad, i32, xabe_moe_buffers_num_tokens_post_pad);
    view!(valid_tokens, i32, xabe_moe_buffers_valid_tokens);
    view!(partial, f32, xabe_moe_buffers_partial);
    view!(shared_inter, f32, xabe_moe_buffers_shared_inter);
    pub fn bytes(&self) -> usize {
        unsafe { ffi::xabe_moe_buffers_bytes(self.raw) }
    }
}
impl Drop for MoeBuffers {
    fn drop(&mut self) {
        unsafe { ffi::xabe_moe_buffers_free(self.raw) }
    }
}

/// moe.rs:4969-5031.  `new` loads the code object up front (gfx950 only: `MoeError::Compile` elsewhere); every
/// launch method is asynchronous on the stream it is given, sized from the geometry, and capturable.
pub struct MoeKernels {
    pub(crate) raw: *mut ffi::xabe_moe_kernels,
    geometry: MoeGeometry,
}
unsafe impl Send for MoeKernels {}
impl MoeKernels {
    pub fn new(ctx: &Arc<HipContext>, geometry: MoeGeometry) -> Result<Self, MoeError> {
        ctx.bind_to_thread()?;
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_moe_kernels_new(&geometry.raw(), &mut raw) })?;
        Ok(Self { raw, geometry })
    }
    pub fn geometry(&self) -> MoeGeometry {
        self.geometry
    }
    pub fn buffers(&self, stream: &Arc<HipStream>) -> Result<MoeBuffers, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_moe_buffers_new(self.raw, stream.raw(), &mut raw) })?;
        Ok(MoeBuffers { raw })
    }
    pub fn shared_only_buffers(&self, stream: &Arc<HipStream>, mma: bool) -> Result<MoeBuffers, MoeError> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::xabe_moe_shared_only_buffers_new(self.raw, stream.raw(), mma as c_int, &mut raw) })?;
        Ok(MoeBuffers { raw })
    }
    pub fn disable_tensor_cores(&mut self) {
        unsafe { ffi::xabe_moe_kernels_disable_tensor_cores(self.raw) };
    }
    pub fn tensor_cores_enabled(&self) -> bool {
        unsafe { ffi::xabe_moe_kernels_tensor_cores_enabled(self.raw) != 0 }
    }
    pub fn force_community(&mut self, on: bool) {
        unsafe { ffi::xabe_moe_kernels_force_community(self.raw, on as c_int) };
    }
    pub fn set_exact_decode_regime(&mut self, on: bool) {
        unsafe { ffi::xabe_moe_kernels_set_exact_decode_regime(self.raw, on as c_int) };
    }
    /// No counterpart in the reference: which grouped-GEMM kernel the routed launches of a wide pass take (see the
    /// header; same bits).
    pub fn set_mfma_form(&mut self, form: i32) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_kernels_set_mfma_form(self.raw, form) })
    }
    /// moe.rs:5473-5491.  Call it before a capture begins: a change of the count inside one is refused.
    pub fn set_valid_tokens(&self, stream: &Arc<HipStream>, buffers: &mut MoeBuffers, tokens: usize) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_set_valid_tokens(self.raw, stream.raw(), buffers.raw, tokens) })
    }
    pub fn route(&self, stream: &Arc<HipStream>, buffers: &mut MoeBuffers, logits: &HipSlice<f32>) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_route(self.raw, stream.raw(), buffers.raw, logits.as_ptr(), logits.len()) })
    }
    pub fn build_dispatch(&self, stream: &Arc<HipStream>, buffers: &mut MoeBuffers) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_build_dispatch(self.raw, stream.raw(), buffers.raw) })
    }
    pub fn route_and_dispatch(&self, stream: &Arc<HipStream>, buffers: &mut MoeBuffers, logits: &HipSlice<f32>) -> Result<(), MoeError> {
        check(unsafe { ffi::xabe_moe_route_and_dispatch(self.raw, stream.raw(), buffers.raw, logits.as_ptr(), logits.len()) })
    }
    pub fn grouped_forward_partial(
        &self,
        stream: &Arc<HipStream>,
        buffers: &mut MoeBuffers,
        gate: QuantTensor<'_>,
        up: QuantTensor<'_>,
        down: QuantTensor<'_>,
        hidden_states: &HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_moe_grouped_forward_partial(self.raw, stream.raw(), buffers.raw, gate.raw(), up.raw(), down.raw(),
                                                  hidden_states.as_ptr(), hidden_states.len())
        })
    }
    /// moe.rs:6190-6335: `Ok(false)` having launched nothing when the fused grid does not cover the pass.
    #[allow(clippy::too_many_arguments)]
    pub fn grouped_forward_partial_with_shared(
        &self,
        stream: &Arc<HipStream>,
        buffers: &mut MoeBuffers,
        gate: QuantTensor<'_>,
        up: QuantTensor<'_>,
        down: QuantTensor<'_>,
        shared_gate: QuantTensor<'_>,
        shared_up: QuantTensor<'_>,
        shared_down: QuantTensor<'_>,
        hidden_states: &HipSlice<f32>,
        out: &mut HipSlice<f32>,
    ) -> Result<bool, MoeError> {
        let mut fused: c_int = 0;
        check(unsafe {
            ffi::xabe_moe_grouped_forward_partial_with_shared(
                self.raw, stream.raw(), buffers.raw, gate.raw(), up.raw(), down.raw(), shared_gate.raw(), shared_up.raw(),
                shared_down.raw(), hidden_states.as_ptr(), hidden_states.len(), out.as_mut_ptr(), out.len(), &mut fused)
        })?;
        Ok(fused != 0)
    }
    #[allow(clippy::too_many_arguments)]
    pub fn grouped_forward(
        &self,
        stream: &Arc<HipStream>,
        buffers: &mut MoeBuffers,
        gate: QuantTensor<'_>,
        up: QuantTensor<'_>,
        down: QuantTensor<'_>,
        hidden_states: &HipSlice<f32>,
        out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_moe_grouped_forward(self.raw, stream.raw(), buffers.raw, gate.raw(), up.raw(), down.raw(),
                                          hidden_states.as_ptr(), hidden_states.len(), out.as_mut_ptr(), out.len())
        })
    }
    #[allow(clippy::too_many_arguments)]
    pub fn shared_expert(
        &self,
        stream: &Arc<HipStream>,
        buffers: &mut MoeBuffers,
        gate: QuantTensor<'_>,
        up: QuantTensor<'_>,
        down: QuantTensor<'_>,
        hidden_states: &HipSlice<f32>,
        out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_moe_shared_expert(self.raw, stream.raw(), buffers.raw, gate.raw(), up.raw(), down.raw(),
                                        hidden_states.as_ptr(), hidden_states.len(), out.as_mut_ptr(), out.len())
        })
    }
    /// moe.rs:6389-6476, over the quantized stacks themselves (fp16 operands on the matrix cores; no int8 repack).
    #[allow(clippy::too_many_arguments)]
    pub fn shared_expert_mma(
        &self,
        stream: &Arc<HipStream>,
        buffers: &mut MoeBuffers,
        gate: QuantTensor<'_>,
        up: QuantTensor<'_>,
        down: QuantTensor<'_>,
        hidden_states: &HipSlice<f32>,
        out: &mut HipSlice<f32>,
    ) -> Result<(), MoeError> {
        check(unsafe {
            ffi::xabe_moe_shared_expert_mma(self.raw, stream.raw(), buffers.raw, gate.raw(), up.raw(), down.raw(),
                                            hidden_states.as_ptr(), hidden_states.len(), out.as_mut_ptr(), out.len())
        })
    }
}
impl Drop for MoeKernels {
    fn drop(&mut self) {
        unsafe { ffi::xabe_moe_kernels_free(self.raw) }
    }
}

//! The context handle and the device allocation type.

use std::any::Any;
use std::ffi::CStr;
use std::fmt;
use std::os::raw::{c_char, c_void};
use std::sync::Arc;

use ojas_core::{BackendId, DType, DeviceBuffer, OjasError};

use crate::ffi;

/// One `omx_ctx`: a device, its stream, the byte budget the library enforces and the deferred
/// fault word. Closed when the last buffer and backend that share it are gone.
pub struct Ctx {
    raw: *mut ffi::OmxCtx,
}

// The library serialises entry points on the context's own stream; the handle itself is a plain
// pointer that any thread may pass in.
unsafe impl Send for Ctx {}
unsafe impl Sync for Ctx {}

impl Ctx {
    /// Opens device `device` with a budget of `budget_bytes` (0 = unlimited).
    pub fn open(device: i32, budget_bytes: u64) -> Result<Arc<Self>, OjasError> {
        let mut raw = std::ptr::null_mut();
        let rc = unsafe { ffi::omx_open(device, budget_bytes, &mut raw) };
        if rc != ffi::OMX_OK || raw.is_null() {
            return Err(OjasError::DeviceLost {
                backend: BackendId::Hip,
                detail: format!("omx_open(device {device}) returned {rc}: no gfx950 device, or libojas_mi355x.so was built for another one"),
            });
        }
        Ok(Arc::new(Self { raw }))
    }

    pub fn raw(&self) -> *mut ffi::OmxCtx {
        self.raw
    }

    /// The text the library kept for the last failed call on this context.
    pub fn last_error(&self) -> String {
        let mut buf = vec![0 as c_char; 512];
        unsafe { ffi::omx_last_error(self.raw, buf.as_mut_ptr(), buf.len()) };
        unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }

    /// A status code of the C ABI as the `OjasError` variant of the same name.
    pub fn check(&self, op: &'static str, rc: i32) -> Result<(), OjasError> {
        let detail = || self.last_error();
        Err(match rc {
            ffi::OMX_OK => return Ok(()),
            ffi::OMX_SHAPE => OjasError::Shape { op, detail: detail() },
            ffi::OMX_DTYPE => OjasError::Dtype { op, expected: DType::F32, got: DType::Bf16 },
            ffi::OMX_OUT_OF_RANGE => OjasError::OutOfRange { op, detail: detail() },
            ffi::OMX_NON_FINITE => OjasError::NonFinite { op: fault_op(&detail()).unwrap_or(op) },
            ffi::OMX_UNSUPPORTED_HEAD_DIM => OjasError::UnsupportedHeadDim { head_dim: number_after(&detail(), "head_dim"), limit: 256 },
            ffi::OMX_CAPACITY_EXCEEDED => {
                let text = detail();
                OjasError::CapacityExceeded {
                    requested: u64::from(number_after(&text, "requested")),
                    cap: u64::from(number_after(&text, "cap")),
                    live: u64::from(number_after(&text, "live")),
                }
            }
            ffi::OMX_POISONED => OjasError::Poisoned,
            ffi::OMX_DEVICE_LOST => OjasError::DeviceLost { backend: BackendId::Hip, detail: detail() },
            ffi::OMX_WAIT_TIMEOUT => OjasError::WaitTimeout { backend: BackendId::Hip, waited_ms: 0, detail: detail() },
            ffi::OMX_UNSUPPORTED => OjasError::Unsupported { op, detail: detail() },
            ffi::OMX_PLACEMENT => OjasError::Placement { op, expected: Some(BackendId::Hip), found: None },
            _ => OjasError::Backend { id: BackendId::Hip, detail: detail() },
        })
    }
}

impl Drop for Ctx {
    fn drop(&mut self) {
        unsafe { ffi::omx_close(self.raw) };
    }
}

impl fmt::Debug for Ctx {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "Ctx({:p})", self.raw)
    }
}

/// The names the library's fault word can carry, as the `&'static str` an `OjasError` needs.
const FAULT_OPS: &[&str] = &[
    "linear_forward", "linear_backward", "gemm", "causal_sdpa_forward", "causal_sdpa_backward", "rms_norm_forward",
    "rms_norm_backward", "cross_entropy_mean_forward", "cross_entropy_mean_backward", "linear_cross_entropy_mean",
    "embedding_forward", "embedding_backward", "adamw_step", "muon_ns5_step", "clip_grad_norm", "residual_add_forward",
    "accumulate_grad", "scale_grad", "gelu_erf_forward", "gelu_erf_backward", "gelu_tanh_forward", "gelu_tanh_backward",
    "silu_forward", "silu_backward", "mul_forward", "mul_backward", "rope_half_split_forward", "rope_half_split_backward",
    "per_head_sigmoid_gate_forward", "per_head_sigmoid_gate_backward", "value_residual_blend_forward",
    "value_residual_blend_backward", "cached_attention_forward", "kv_cache_write", "cast_bf16", "to_bf16", "to_f32",
];

fn fault_op(detail: &str) -> Option<&'static str> {
    FAULT_OPS.iter().copied().filter(|op| detail.contains(op)).max_by_key(|op| op.len())
}

/// The unsigned number that follows `key` in `text` ("requested 4096, cap 1024, live 0").
fn number_after(text: &str, key: &str) -> u32 {
    text.split(key)
        .nth(1)
        .map(|rest| rest.trim_start_matches(|c: char| !c.is_ascii_digit()))
        .and_then(|rest| rest.split(|c: char| !c.is_ascii_digit()).next())
        .and_then(|digits| digits.parse().ok())
        .unwrap_or(0)
}

/// Device memory from `omx_alloc`; freed (stream-ordered) when the last tensor view drops.
pub struct HipDeviceBuffer {
    ctx: Arc<Ctx>,
    ptr: *mut c_void,
    len: usize,
}

unsafe impl Send for HipDeviceBuffer {}
unsafe impl Sync for HipDeviceBuffer {}

impl HipDeviceBuffer {
    /// `len` bytes on `ctx`'s device. The caller has reserved them from its `Budget` already.
    pub fn alloc(ctx: &Arc<Ctx>, op: &'static str, len: usize) -> Result<Self, OjasError> {
        let mut ptr = std::ptr::null_mut();
        ctx.check(op, unsafe { ffi::omx_alloc(ctx.raw(), len.max(1) as u64, &mut ptr) })?;
        Ok(Self { ctx: Arc::clone(ctx), ptr, len })
    }

    pub fn ptr(&self) -> *mut c_void {
        self.ptr
    }

    pub fn ctx(&self) -> &Arc<Ctx> {
        &self.ctx
    }
}

impl Drop for HipDeviceBuffer {
    fn drop(&mut self) {
        // Work already submitted that reads the block keeps it: the library parks a freed block
        // until the stream has passed the point of the free.
        unsafe { ffi::omx_free(self.ctx.raw(), self.ptr) };
    }
}

impl fmt::Debug for HipDeviceBuffer {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "HipDeviceBuffer({:p}, {} bytes)", self.ptr, self.len)
    }
}

impl DeviceBuffer for HipDeviceBuffer {
    fn backend(&self) -> BackendId {
        BackendId::Hip
    }

    fn byte_len(&self) -> usize {
        self.len
    }

    /// A read after the stream has drained. `omx_download` is also where this library reports a
    /// pending non-finite fault (once): a read that meets one returns `NonFinite` naming the op.
    fn read_bytes(&self, offset: usize, len: usize) -> Result<Vec<u8>, OjasError> {
        let mut out = vec![0u8; len];
        self.ctx.check("DeviceBuffer::read_bytes", unsafe {
            ffi::omx_download(self.ctx.raw(), out.as_mut_ptr().cast(), self.ptr, offset as u64, len as u64)
        })?;
        Ok(out)
    }

    fn as_any(&self) -> &dyn Any {
        self
    }
}

//! `Mi355xBackend`: the four backend traits over the C ABI.
//!
//! Every method has the same shape: the shared validator (`ojas_core::shapes`, before anything is
//! reserved or touched, docs/shape-contract.md), placement of every operand, outputs reserved from
//! the budget and allocated, one `omx_*` call. Tensors are f32 (u32 for ids) unless the caller
//! opted into bf16 operand storage through `cast_bf16` / `to_bf16`; outputs are f32, as the
//! reference's are.

use std::os::raw::c_void;
use std::sync::Arc;

use ojas_core::{
    accumulate_grad_dims, adamw_step_dims, argmax_rows_dims, cached_attention_dims, causal_sdpa_backward_dims,
    causal_sdpa_forward_dims, clip_grad_norm_dims, cross_entropy_mean_backward_dims, cross_entropy_mean_forward_dims,
    embedding_backward_dims, embedding_forward_dims, gelu_erf_backward_dims, gelu_erf_forward_dims,
    gelu_tanh_backward_dims, gelu_tanh_forward_dims, kv_cache_write_dims, linear_backward_dims, linear_ce_dims,
    linear_forward_dims, mul_backward_dims, mul_forward_dims, muon_ns5_step_dims, per_head_sigmoid_gate_backward_dims,
    per_head_sigmoid_gate_forward_dims, permute_dims, residual_add_backward_dims, residual_add_forward_dims,
    rms_norm_backward_dims, rms_norm_forward_dims, rms_qk_norm_backward_dims, rms_qk_norm_forward_dims,
    rope_half_split_backward_dims, rope_half_split_forward_dims, scale_grad_dims, silu_backward_dims, silu_forward_dims,
    topk_rows_dims, value_residual_blend_backward_dims, value_residual_blend_forward_dims, AdamWConfig, Backend,
    BackendCore, BackendFloat, BackendId, BackendInt, BackendModule, Budget, CeChunk, CeGrads, DType, LinearCe,
    MuonNs5Config, Ns5Precision, Numerics, OjasError, OptimizerKind, PerHeadGateGrad, Reservation, RopeLayout, Tensor,
    ValueResidualGrad,
};

use crate::buffer::{Ctx, HipDeviceBuffer};
use crate::ffi;

/// The MI355X backend: one device context and the budget its tensors are charged to.
#[derive(Debug)]
pub struct Mi355xBackend {
    ctx: Arc<Ctx>,
    budget: Budget,
}

/// A reserved and allocated output on its way to becoming a `Tensor`.
struct Output {
    buffer: Arc<HipDeviceBuffer>,
    reservation: Reservation,
    shape: Vec<usize>,
    dtype: DType,
}

impl Output {
    fn ptr(&self) -> *mut c_void {
        self.buffer.ptr()
    }

    fn into_tensor(self) -> Result<Tensor, OjasError> {
        Tensor::from_device_reserved(self.buffer, &self.shape, self.dtype, self.reservation)
    }
}

fn code(dtype: DType) -> i32 {
    match dtype {
        DType::F32 => ffi::OMX_F32,
        DType::Bf16 => ffi::OMX_BF16,
        _ => ffi::OMX_U32,
    }
}

fn window_arg(window: Option<usize>) -> u64 {
    window.map_or(0, |w| w as u64)
}

impl Mi355xBackend {
    /// Device `device` with `budget` as the cap on live tensor bytes.
    pub fn new(device: i32, budget: Budget) -> Result<Self, OjasError> {
        // The library's own cap stays open: the `Budget` is the one authority, charged before every
        // allocation, so a refusal carries the workspace's numbers.
        Ok(Self { ctx: Ctx::open(device, 0)?, budget })
    }

    pub fn ctx(&self) -> &Arc<Ctx> {
        &self.ctx
    }

    fn raw(&self) -> *mut ffi::OmxCtx {
        self.ctx.raw()
    }

    fn check(&self, op: &'static str, rc: i32) -> Result<(), OjasError> {
        self.ctx.check(op, rc)
    }

    /// The device address of a contiguous operand that lives on this context.
    fn operand(&self, op: &'static str, t: &Tensor) -> Result<*const c_void, OjasError> {
        let buffer = t.device_buffer().ok_or(OjasError::Placement { op, expected: Some(BackendId::Hip), found: t.device() })?;
        let ours = buffer
            .as_any()
            .downcast_ref::<HipDeviceBuffer>()
            .filter(|b| Arc::ptr_eq(b.ctx(), &self.ctx))
            .ok_or(OjasError::Placement { op, expected: Some(BackendId::Hip), found: t.device() })?;
        if !t.is_contiguous()? {
            return Err(OjasError::Shape { op, detail: "operand is not contiguous".to_string() });
        }
        Ok(unsafe { ours.ptr().cast::<u8>().add(t.byte_offset()) }.cast())
    }

    /// The same for a tensor an op updates in place: shared storage is refused before any write.
    fn operand_mut(&self, op: &'static str, t: &mut Tensor) -> Result<*mut c_void, OjasError> {
        let ptr = self.operand(op, t)?;
        t.device_buffer_mut()?;
        Ok(ptr.cast_mut())
    }

    fn output(&self, op: &'static str, shape: &[usize], dtype: DType) -> Result<Output, OjasError> {
        let bytes = shape.iter().product::<usize>() * dtype.size();
        let reservation = self.budget.try_reserve(bytes as u64)?;
        let buffer = Arc::new(HipDeviceBuffer::alloc(&self.ctx, op, bytes)?);
        Ok(Output { buffer, reservation, shape: shape.to_vec(), dtype })
    }

    /// One elementwise op of the form out = f(x) or out = f(x, gy): same shape out, f32.
    fn unary(
        &self,
        op: &'static str,
        x: &Tensor,
        gy: Option<&Tensor>,
        call: impl FnOnce(*const c_void, *const c_void, *mut c_void, i32, u64) -> i32,
    ) -> Result<Tensor, OjasError> {
        let n = x.num_elements()? as u64;
        let xp = self.operand(op, x)?;
        let gp = match gy {
            Some(g) => self.operand(op, g)?,
            None => std::ptr::null(),
        };
        let out = self.output(op, x.shape(), DType::F32)?;
        self.check(op, call(xp, gp, out.ptr(), code(x.dtype()), n))?;
        out.into_tensor()
    }
}

impl BackendCore for Mi355xBackend {
    fn id(&self) -> BackendId {
        BackendId::Hip
    }

    fn budget(&self) -> &Budget {
        &self.budget
    }

    fn numerics(&self) -> Numerics {
        Numerics::Fast
    }

    fn bf16_operands(&self) -> bool {
        true
    }

    fn upload(&self, tensor: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "Backend::upload";
        match tensor.device() {
            Some(BackendId::Hip) => return self.operand(OP, tensor).map(|_| tensor.clone()),
            Some(found) => return Err(OjasError::Placement { op: OP, expected: Some(BackendId::Hip), found: Some(found) }),
            None => {}
        }
        let bytes = tensor.to_ne_bytes()?;
        let out = self.output(OP, tensor.shape(), tensor.dtype())?;
        self.check(OP, unsafe { ffi::omx_upload(self.raw(), out.ptr(), 0, bytes.as_ptr().cast(), bytes.len() as u64) })?;
        out.into_tensor()
    }

    fn download(&self, tensor: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "Backend::download";
        self.operand(OP, tensor)?;
        // to_host reads through HipDeviceBuffer::read_bytes: the stream drains, a pending fault is
        // reported, the bytes are copied.
        tensor.to_host(&self.budget)
    }

    fn optimizer_scratch_bytes(&self, kind: OptimizerKind, rows: usize, cols: usize) -> Result<Option<u64>, OjasError> {
        Ok(Some(match kind {
            OptimizerKind::AdamW => 256,
            OptimizerKind::MuonNs5 => unsafe { ffi::omx_muon_scratch_bytes(rows as u64, cols as u64) },
        }))
    }

    fn sync(&self) -> Result<(), OjasError> {
        self.check("sync", unsafe { ffi::omx_sync(self.raw()) })
    }

    fn cast_bf16(&self, tensor: &Tensor) -> Result<Tensor, OjasError> {
        self.unary("cast_bf16", tensor, None, |x, _, y, _, n| unsafe { ffi::omx_cast_bf16(self.raw(), x, y, n) })
    }

    fn to_bf16(&self, tensor: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "to_bf16";
        if tensor.dtype() != DType::F32 {
            return Err(OjasError::Dtype { op: OP, expected: DType::F32, got: tensor.dtype() });
        }
        let x = self.operand(OP, tensor)?;
        let out = self.output(OP, tensor.shape(), DType::Bf16)?;
        self.check(OP, unsafe { ffi::omx_to_bf16(self.raw(), x, out.ptr(), tensor.num_elements()? as u64) })?;
        out.into_tensor()
    }

    fn to_f32(&self, tensor: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "to_f32";
        if tensor.dtype() != DType::Bf16 {
            return Err(OjasError::Dtype { op: OP, expected: DType::Bf16, got: tensor.dtype() });
        }
        let x = self.operand(OP, tensor)?;
        let out = self.output(OP, tensor.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_to_f32(self.raw(), x, out.ptr(), tensor.num_elements()? as u64) })?;
        out.into_tensor()
    }
}

impl BackendFloat for Mi355xBackend {
    /// `[0, 2, 1, 3]` on a rank-4 tensor (the attention layout swap) is the one permutation the
    /// model issues; the others keep the trait's refusal.
    fn permute(&self, input: &Tensor, dims: &[usize]) -> Result<Tensor, OjasError> {
        const OP: &str = "permute";
        let out_shape = permute_dims(input, dims)?;
        if dims != [0, 2, 1, 3] {
            return Err(OjasError::Unsupported { op: OP, detail: format!("axes {dims:?}: only [0, 2, 1, 3] runs on the device") });
        }
        let x = self.operand(OP, input)?;
        let s = input.shape();
        let out = self.output(OP, &out_shape, DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_permute_0213(self.raw(), x, out.ptr(), code(input.dtype()), s[0] as u64, s[1] as u64, s[2] as u64, s[3] as u64)
        })?;
        out.into_tensor()
    }

    fn silu_forward(&self, input: &Tensor) -> Result<Tensor, OjasError> {
        silu_forward_dims(input)?;
        self.unary("silu_forward", input, None, |x, _, y, d, n| unsafe { ffi::omx_silu_forward(self.raw(), x, y, d, n) })
    }

    fn silu_backward(&self, input: &Tensor, grad_output: &Tensor) -> Result<Tensor, OjasError> {
        silu_backward_dims(input, grad_output)?;
        self.unary("silu_backward", input, Some(grad_output), |x, g, y, d, n| unsafe { ffi::omx_silu_backward(self.raw(), x, g, y, d, n) })
    }

    fn mul_forward(&self, a: &Tensor, b: &Tensor) -> Result<Tensor, OjasError> {
        mul_forward_dims(a, b)?;
        self.unary("mul_forward", a, Some(b), |x, y, out, d, n| unsafe { ffi::omx_mul_forward(self.raw(), x, y, out, d, n) })
    }

    fn mul_backward(&self, a: &Tensor, b: &Tensor, grad_output: &Tensor) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "mul_backward";
        let n = mul_backward_dims(a, b, grad_output)? as u64;
        let (ap, bp, gp) = (self.operand(OP, a)?, self.operand(OP, b)?, self.operand(OP, grad_output)?);
        let (ga, gb) = (self.output(OP, a.shape(), DType::F32)?, self.output(OP, b.shape(), DType::F32)?);
        self.check(OP, unsafe { ffi::omx_mul_backward(self.raw(), ap, bp, gp, ga.ptr(), gb.ptr(), code(a.dtype()), n) })?;
        Ok((ga.into_tensor()?, gb.into_tensor()?))
    }

    fn residual_add_forward(&self, x: &Tensor, y: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "residual_add_forward";
        let n = residual_add_forward_dims(x, y)? as u64;
        let (xp, yp) = (self.operand(OP, x)?, self.operand(OP, y)?);
        let out = self.output(OP, x.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_residual_add(self.raw(), xp, code(x.dtype()), yp, code(y.dtype()), out.ptr(), ffi::OMX_F32, n) })?;
        out.into_tensor()
    }

    /// Both gradients of x + y are the output's gradient: two views of it, no kernel.
    fn residual_add_backward(&self, x: &Tensor, y: &Tensor, grad_output: &Tensor) -> Result<(Tensor, Tensor), OjasError> {
        residual_add_backward_dims(x, y, grad_output)?;
        self.operand("residual_add_backward", grad_output)?;
        Ok((grad_output.clone(), grad_output.clone()))
    }

    fn gelu_erf_forward(&self, input: &Tensor) -> Result<Tensor, OjasError> {
        gelu_erf_forward_dims(input)?;
        self.unary("gelu_erf_forward", input, None, |x, _, y, d, n| unsafe { ffi::omx_gelu_forward(self.raw(), x, y, d, n, 0) })
    }

    fn gelu_erf_backward(&self, input: &Tensor, grad_output: &Tensor) -> Result<Tensor, OjasError> {
        gelu_erf_backward_dims(input, grad_output)?;
        self.unary("gelu_erf_backward", input, Some(grad_output), |x, g, y, d, n| unsafe { ffi::omx_gelu_backward(self.raw(), x, g, y, d, n, 0) })
    }

    fn gelu_tanh_forward(&self, input: &Tensor) -> Result<Tensor, OjasError> {
        gelu_tanh_forward_dims(input)?;
        self.unary("gelu_tanh_forward", input, None, |x, _, y, d, n| unsafe { ffi::omx_gelu_forward(self.raw(), x, y, d, n, 1) })
    }

    fn gelu_tanh_backward(&self, input: &Tensor, grad_output: &Tensor) -> Result<Tensor, OjasError> {
        gelu_tanh_backward_dims(input, grad_output)?;
        self.unary("gelu_tanh_backward", input, Some(grad_output), |x, g, y, d, n| unsafe { ffi::omx_gelu_backward(self.raw(), x, g, y, d, n, 1) })
    }

    /// The global norm comes back to the host (a sync point, where a pending fault is reported);
    /// the scaling, when the norm is above `max_norm`, happens in place on the device.
    fn clip_grad_norm(&self, grads: &mut [Tensor], max_norm: f32) -> Result<f32, OjasError> {
        const OP: &str = "clip_grad_norm";
        clip_grad_norm_dims(grads)?;
        let mut ptrs = Vec::with_capacity(grads.len());
        let mut lens = Vec::with_capacity(grads.len());
        for g in grads.iter_mut() {
            lens.push(g.num_elements()? as u64);
            ptrs.push(self.operand_mut(OP, g)?);
        }
        let mut norm = 0.0f32;
        self.check(OP, unsafe { ffi::omx_clip_grad_norm(self.raw(), ptrs.as_ptr(), lens.as_ptr(), ptrs.len() as u64, max_norm, &mut norm) })?;
        Ok(norm)
    }

    fn accumulate_grad(&self, acc: &mut Tensor, grad: &Tensor) -> Result<(), OjasError> {
        const OP: &str = "accumulate_grad";
        let n = accumulate_grad_dims(acc, grad)? as u64;
        let g = self.operand(OP, grad)?;
        let a = self.operand_mut(OP, acc)?;
        self.check(OP, unsafe { ffi::omx_accumulate_grad(self.raw(), a, g, n) })
    }

    fn scale_grad(&self, grad: &mut Tensor, scale: f32) -> Result<(), OjasError> {
        const OP: &str = "scale_grad";
        let n = scale_grad_dims(grad)? as u64;
        let g = self.operand_mut(OP, grad)?;
        self.check(OP, unsafe { ffi::omx_scale_grad(self.raw(), g, scale, n) })
    }
}

impl BackendInt for Mi355xBackend {
    fn argmax_rows(&self, x: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "argmax_rows";
        let (rows, cols) = argmax_rows_dims(x)?;
        let xp = self.operand(OP, x)?;
        let out = self.output(OP, &[rows], DType::U32)?;
        self.check(OP, unsafe { ffi::omx_argmax_rows(self.raw(), xp, rows as u64, cols as u64, out.ptr()) })?;
        out.into_tensor()
    }

    fn topk_rows(&self, x: &Tensor, k: usize) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "topk_rows";
        let (rows, cols) = topk_rows_dims(x, k)?;
        let xp = self.operand(OP, x)?;
        let (values, indices) = (self.output(OP, &[rows, k], DType::F32)?, self.output(OP, &[rows, k], DType::U32)?);
        self.check(OP, unsafe { ffi::omx_topk_rows(self.raw(), xp, rows as u64, cols as u64, k as u64, values.ptr(), indices.ptr()) })?;
        Ok((values.into_tensor()?, indices.into_tensor()?))
    }
}

impl BackendModule for Mi355xBackend {
    fn embedding_forward(&self, table: &Tensor, token_ids: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "embedding_forward";
        let d = embedding_forward_dims(table, token_ids)?;
        let (t, ids) = (self.operand(OP, table)?, self.operand(OP, token_ids)?);
        let out = self.output(OP, &d.out_shape, DType::F32)?;
        // An id outside the table raises the device fault word; the next sync reports OutOfRange.
        self.check(OP, unsafe { ffi::omx_embedding_forward(self.raw(), t, code(table.dtype()), ids, out.ptr(), ffi::OMX_F32, d.tokens as u64, d.vocab as u64, d.dim as u64) })?;
        out.into_tensor()
    }

    fn embedding_backward(&self, table: &Tensor, token_ids: &Tensor, grad_output: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "embedding_backward";
        let d = embedding_backward_dims(table, token_ids, grad_output)?;
        let (ids, g) = (self.operand(OP, token_ids)?, self.operand(OP, grad_output)?);
        let out = self.output(OP, table.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_embedding_backward(self.raw(), ids, g, code(grad_output.dtype()), out.ptr(), d.tokens as u64, d.vocab as u64, d.dim as u64) })?;
        out.into_tensor()
    }

    fn linear_forward(&self, input: &Tensor, weight: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "linear_forward";
        let d = linear_forward_dims(input, weight)?;
        let (x, w) = (self.operand(OP, input)?, self.operand(OP, weight)?);
        let out = self.output(OP, &d.out_shape, DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_linear_forward(self.raw(), x, code(input.dtype()), w, code(weight.dtype()), out.ptr(), ffi::OMX_F32, d.rows as u64, d.in_features as u64, d.out_features as u64)
        })?;
        out.into_tensor()
    }

    fn linear_backward(&self, input: &Tensor, weight: &Tensor, grad_output: &Tensor) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "linear_backward";
        let d = linear_backward_dims(input, weight, grad_output)?;
        let (x, w, g) = (self.operand(OP, input)?, self.operand(OP, weight)?, self.operand(OP, grad_output)?);
        let (gx, gw) = (self.output(OP, input.shape(), DType::F32)?, self.output(OP, weight.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_linear_backward(self.raw(), x, w, g, code(input.dtype()), gx.ptr(), ffi::OMX_F32, gw.ptr(), ffi::OMX_F32, d.rows as u64, d.in_features as u64, d.out_features as u64)
        })?;
        Ok((gx.into_tensor()?, gw.into_tensor()?))
    }

    /// The input half alone (a frozen weight): the entry point skips the product it is not asked for.
    fn linear_backward_input(&self, input: &Tensor, weight: &Tensor, grad_output: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "linear_backward_input";
        let d = linear_backward_dims(input, weight, grad_output)?;
        let (w, g) = (self.operand(OP, weight)?, self.operand(OP, grad_output)?);
        let gx = self.output(OP, input.shape(), DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_linear_backward(self.raw(), std::ptr::null(), w, g, code(weight.dtype()), gx.ptr(), ffi::OMX_F32, std::ptr::null_mut(), ffi::OMX_F32, d.rows as u64, d.in_features as u64, d.out_features as u64)
        })?;
        gx.into_tensor()
    }

    fn rms_norm_forward(&self, input: &Tensor, weight: &Tensor, eps: f32) -> Result<Tensor, OjasError> {
        const OP: &str = "rms_norm_forward";
        let d = rms_norm_forward_dims(input, weight, eps)?;
        let (x, w) = (self.operand(OP, input)?, self.operand(OP, weight)?);
        let out = self.output(OP, input.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_rms_norm_forward(self.raw(), x, code(input.dtype()), w, out.ptr(), ffi::OMX_F32, d.rows as u64, d.dim as u64, eps) })?;
        out.into_tensor()
    }

    fn rms_norm_backward(&self, input: &Tensor, weight: &Tensor, grad_output: &Tensor, eps: f32) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "rms_norm_backward";
        let d = rms_norm_backward_dims(input, weight, grad_output, eps)?;
        let (x, w, g) = (self.operand(OP, input)?, self.operand(OP, weight)?, self.operand(OP, grad_output)?);
        let (gx, gw) = (self.output(OP, input.shape(), DType::F32)?, self.output(OP, weight.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_rms_norm_backward(self.raw(), x, code(input.dtype()), w, g, code(grad_output.dtype()), gx.ptr(), ffi::OMX_F32, gw.ptr(), d.rows as u64, d.dim as u64, eps)
        })?;
        Ok((gx.into_tensor()?, gw.into_tensor()?))
    }

    fn rope_half_split_forward(&self, x: &Tensor, cos: &Tensor, sin: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "rope_half_split_forward";
        let d = rope_half_split_forward_dims(x, cos, sin)?;
        let (time, heads) = match d.layout {
            RopeLayout::Same => (0, 0),
            RopeLayout::TimeDim { time, heads } => (time as u64, heads as u64),
        };
        let (xp, c, s) = (self.operand(OP, x)?, self.operand(OP, cos)?, self.operand(OP, sin)?);
        let out = self.output(OP, x.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_rope_half_split_forward(self.raw(), xp, c, s, out.ptr(), code(x.dtype()), d.rows as u64, d.dim as u64, time, heads) })?;
        out.into_tensor()
    }

    fn rope_half_split_backward(&self, grad_output: &Tensor, cos: &Tensor, sin: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "rope_half_split_backward";
        let d = rope_half_split_backward_dims(grad_output, cos, sin)?;
        let (time, heads) = match d.layout {
            RopeLayout::Same => (0, 0),
            RopeLayout::TimeDim { time, heads } => (time as u64, heads as u64),
        };
        let (g, c, s) = (self.operand(OP, grad_output)?, self.operand(OP, cos)?, self.operand(OP, sin)?);
        let out = self.output(OP, grad_output.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_rope_half_split_backward(self.raw(), g, c, s, out.ptr(), code(grad_output.dtype()), d.rows as u64, d.dim as u64, time, heads) })?;
        out.into_tensor()
    }

    fn rms_qk_norm_forward(&self, q: &Tensor, k: &Tensor, q_weight: &Tensor, k_weight: &Tensor, eps: f32) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "rms_norm_forward"; // the name every backend reports for this pair (docs/shape-contract.md, decision 3)
        let (dq, dk) = rms_qk_norm_forward_dims(q, k, q_weight, k_weight, eps)?;
        let (qp, kp, qw, kw) = (self.operand(OP, q)?, self.operand(OP, k)?, self.operand(OP, q_weight)?, self.operand(OP, k_weight)?);
        let (qo, ko) = (self.output(OP, q.shape(), DType::F32)?, self.output(OP, k.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_rms_qk_norm_forward(self.raw(), qp, kp, code(q.dtype()), qw, kw, qo.ptr(), ko.ptr(), ffi::OMX_F32, dq.rows as u64, dk.rows as u64, dq.dim as u64, eps)
        })?;
        Ok((qo.into_tensor()?, ko.into_tensor()?))
    }

    fn rms_qk_norm_backward(
        &self,
        q: &Tensor,
        k: &Tensor,
        q_weight: &Tensor,
        k_weight: &Tensor,
        grad_q: &Tensor,
        grad_k: &Tensor,
        eps: f32,
    ) -> Result<(Tensor, Tensor, Tensor, Tensor), OjasError> {
        const OP: &str = "rms_norm_backward";
        let (dq, dk) = rms_qk_norm_backward_dims(q, k, q_weight, k_weight, grad_q, grad_k, eps)?;
        let (qp, kp, qw, kw) = (self.operand(OP, q)?, self.operand(OP, k)?, self.operand(OP, q_weight)?, self.operand(OP, k_weight)?);
        let (gqp, gkp) = (self.operand(OP, grad_q)?, self.operand(OP, grad_k)?);
        let (gq, gk) = (self.output(OP, q.shape(), DType::F32)?, self.output(OP, k.shape(), DType::F32)?);
        let (gqw, gkw) = (self.output(OP, q_weight.shape(), DType::F32)?, self.output(OP, k_weight.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_rms_qk_norm_backward(self.raw(), qp, kp, code(q.dtype()), qw, kw, gqp, gkp, code(grad_q.dtype()), gq.ptr(), gk.ptr(), ffi::OMX_F32, gqw.ptr(), gkw.ptr(), dq.rows as u64, dk.rows as u64, dq.dim as u64, eps)
        })?;
        Ok((gq.into_tensor()?, gk.into_tensor()?, gqw.into_tensor()?, gkw.into_tensor()?))
    }

    fn causal_sdpa_forward(&self, q: &Tensor, k: &Tensor, v: &Tensor, window: Option<usize>) -> Result<(Tensor, Tensor), OjasError> {
        const OP: &str = "causal_sdpa_forward";
        let d = causal_sdpa_forward_dims(q, k, v, window)?;
        let (qp, kp, vp) = (self.operand(OP, q)?, self.operand(OP, k)?, self.operand(OP, v)?);
        let (out, lse) = (self.output(OP, q.shape(), DType::F32)?, self.output(OP, &[d.batch, d.heads, d.seq], DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_causal_sdpa_forward(self.raw(), qp, kp, vp, code(q.dtype()), out.ptr(), ffi::OMX_F32, lse.ptr(), d.batch as u64, d.heads as u64, d.kv_heads as u64, d.seq as u64, d.head_dim as u64, window_arg(window))
        })?;
        Ok((out.into_tensor()?, lse.into_tensor()?))
    }

    fn causal_sdpa_backward(
        &self,
        q: &Tensor,
        k: &Tensor,
        v: &Tensor,
        output: &Tensor,
        lse: &Tensor,
        grad_output: &Tensor,
        window: Option<usize>,
    ) -> Result<(Tensor, Tensor, Tensor), OjasError> {
        const OP: &str = "causal_sdpa_backward";
        let d = causal_sdpa_backward_dims(q, k, v, output, lse, grad_output, window)?;
        let (qp, kp, vp) = (self.operand(OP, q)?, self.operand(OP, k)?, self.operand(OP, v)?);
        let (op, lp, gp) = (self.operand(OP, output)?, self.operand(OP, lse)?, self.operand(OP, grad_output)?);
        let (gq, gk, gv) = (self.output(OP, q.shape(), DType::F32)?, self.output(OP, k.shape(), DType::F32)?, self.output(OP, v.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_causal_sdpa_backward(self.raw(), qp, kp, vp, op, lp, gp, code(q.dtype()), code(output.dtype()), code(grad_output.dtype()), gq.ptr(), gk.ptr(), gv.ptr(), ffi::OMX_F32, d.batch as u64, d.heads as u64, d.kv_heads as u64, d.seq as u64, d.head_dim as u64, window_arg(window))
        })?;
        Ok((gq.into_tensor()?, gk.into_tensor()?, gv.into_tensor()?))
    }

    /// Autocast routes a bf16-tagged saved output here (ojas-core/src/autocast.rs:1200-1233): the
    /// library reruns the forward in its own workspace and keeps the output unrounded.
    fn causal_sdpa_backward_recompute(&self, q: &Tensor, k: &Tensor, v: &Tensor, grad_output: &Tensor, window: Option<usize>) -> Result<(Tensor, Tensor, Tensor), OjasError> {
        const OP: &str = "causal_sdpa_backward";
        let d = causal_sdpa_forward_dims(q, k, v, window)?;
        if grad_output.shape() != q.shape() {
            return Err(OjasError::Shape { op: OP, detail: format!("grad_output {:?} must match q {:?}", grad_output.shape(), q.shape()) });
        }
        let (qp, kp, vp, gp) = (self.operand(OP, q)?, self.operand(OP, k)?, self.operand(OP, v)?, self.operand(OP, grad_output)?);
        let (gq, gk, gv) = (self.output(OP, q.shape(), DType::F32)?, self.output(OP, k.shape(), DType::F32)?, self.output(OP, v.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_causal_sdpa_backward_recompute(self.raw(), qp, kp, vp, gp, code(q.dtype()), code(grad_output.dtype()), gq.ptr(), gk.ptr(), gv.ptr(), ffi::OMX_F32, d.batch as u64, d.heads as u64, d.kv_heads as u64, d.seq as u64, d.head_dim as u64, window_arg(window))
        })?;
        Ok((gq.into_tensor()?, gk.into_tensor()?, gv.into_tensor()?))
    }

    fn per_head_sigmoid_gate_forward(&self, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor) -> Result<Tensor, OjasError> {
        self.gate_forward("per_head_sigmoid_gate_forward", input, weight, bias, attn_out, false).map(|(y, _)| y)
    }

    fn per_head_sigmoid_gate_forward_saving(&self, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor) -> Result<(Tensor, Option<Tensor>), OjasError> {
        self.gate_forward("per_head_sigmoid_gate_forward", input, weight, bias, attn_out, true)
    }

    fn per_head_sigmoid_gate_backward(&self, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor, grad_output: &Tensor) -> Result<PerHeadGateGrad, OjasError> {
        self.gate_backward(input, weight, bias, attn_out, grad_output, None)
    }

    fn per_head_sigmoid_gate_backward_saved(&self, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor, grad_output: &Tensor, scales: &Tensor) -> Result<PerHeadGateGrad, OjasError> {
        self.gate_backward(input, weight, bias, attn_out, grad_output, Some(scales))
    }

    fn value_residual_blend_forward(&self, value: &Tensor, value0: &Tensor, lambda: &Tensor) -> Result<Tensor, OjasError> {
        const OP: &str = "value_residual_blend_forward";
        let n = value_residual_blend_forward_dims(value, value0, lambda)? as u64;
        let (v, v0, l) = (self.operand(OP, value)?, self.operand(OP, value0)?, self.operand(OP, lambda)?);
        let out = self.output(OP, value.shape(), DType::F32)?;
        self.check(OP, unsafe { ffi::omx_value_residual_blend_forward(self.raw(), v, v0, l, out.ptr(), code(value.dtype()), n) })?;
        out.into_tensor()
    }

    fn value_residual_blend_backward(&self, value: &Tensor, value0: &Tensor, lambda: &Tensor, grad_output: &Tensor) -> Result<ValueResidualGrad, OjasError> {
        const OP: &str = "value_residual_blend_backward";
        let n = value_residual_blend_backward_dims(value, value0, lambda, grad_output)? as u64;
        let (v, v0, l, g) = (self.operand(OP, value)?, self.operand(OP, value0)?, self.operand(OP, lambda)?, self.operand(OP, grad_output)?);
        let (gv, gv0, gl) = (self.output(OP, value.shape(), DType::F32)?, self.output(OP, value0.shape(), DType::F32)?, self.output(OP, lambda.shape(), DType::F32)?);
        self.check(OP, unsafe { ffi::omx_value_residual_blend_backward(self.raw(), v, v0, l, g, gv.ptr(), gv0.ptr(), code(value.dtype()), gl.ptr(), n) })?;
        Ok(ValueResidualGrad { value: gv.into_tensor()?, value0: gv0.into_tensor()?, lambda: gl.into_tensor()? })
    }

    fn cross_entropy_mean_forward(&self, logits: &Tensor, targets: &Tensor, ignore_index: Option<u32>) -> Result<Tensor, OjasError> {
        const OP: &str = "cross_entropy_mean_forward";
        let d = cross_entropy_mean_forward_dims(logits, targets)?;
        let (l, t) = (self.operand(OP, logits)?, self.operand(OP, targets)?);
        let out = self.output(OP, &[1], DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_cross_entropy_mean_forward(self.raw(), l, code(logits.dtype()), t, d.rows as u64, d.vocab as u64, i32::from(ignore_index.is_some()), ignore_index.unwrap_or(0), out.ptr())
        })?;
        out.into_tensor()
    }

    fn cross_entropy_mean_backward(&self, logits: &Tensor, targets: &Tensor, ignore_index: Option<u32>) -> Result<Tensor, OjasError> {
        const OP: &str = "cross_entropy_mean_backward";
        let d = cross_entropy_mean_backward_dims(logits, targets)?;
        let (l, t) = (self.operand(OP, logits)?, self.operand(OP, targets)?);
        let out = self.output(OP, logits.shape(), DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_cross_entropy_mean_backward(self.raw(), l, code(logits.dtype()), t, d.rows as u64, d.vocab as u64, i32::from(ignore_index.is_some()), ignore_index.unwrap_or(0), out.ptr(), ffi::OMX_F32)
        })?;
        out.into_tensor()
    }

    fn adamw_step(&self, param: &mut Tensor, grad: &Tensor, moment1: &mut Tensor, moment2: &mut Tensor, step: u64, config: AdamWConfig) -> Result<(), OjasError> {
        const OP: &str = "adamw_step";
        let n = adamw_step_dims(param, grad, moment1, moment2)? as u64;
        let g = self.operand(OP, grad)?;
        let (p, m1, m2) = (self.operand_mut(OP, param)?, self.operand_mut(OP, moment1)?, self.operand_mut(OP, moment2)?);
        let c = ffi::OmxAdamwConfig { lr: config.lr, beta1: config.beta1, beta2: config.beta2, eps: config.eps, weight_decay: config.weight_decay };
        // The library checks the scalars (check_adamw's rules) and the inputs before it writes anything.
        self.check(OP, unsafe { ffi::omx_adamw_step(self.raw(), p, g, m1, m2, n, step, &c, std::ptr::null_mut()) })
    }

    fn muon_ns5_step(&self, param: &mut Tensor, grad: &Tensor, momentum: &mut Tensor, config: MuonNs5Config) -> Result<(), OjasError> {
        const OP: &str = "muon_ns5_step";
        let d = muon_ns5_step_dims(param, grad, momentum)?;
        let g = self.operand(OP, grad)?;
        let (p, m) = (self.operand_mut(OP, param)?, self.operand_mut(OP, momentum)?);
        let c = ffi::OmxMuonConfig {
            lr: config.lr,
            momentum: config.momentum,
            weight_decay: config.weight_decay,
            nesterov: i32::from(config.nesterov),
            ns5_bf16: i32::from(config.ns5 != Ns5Precision::F32),
        };
        self.check(OP, unsafe { ffi::omx_muon_ns5_step(self.raw(), p, g, m, d.rows as u64, d.cols as u64, &c, std::ptr::null_mut()) })
    }

    fn linear_cross_entropy_mean(&self, input: &Tensor, weight: &Tensor, targets: &Tensor, ignore_index: Option<u32>, chunk: CeChunk, grads: CeGrads) -> Result<LinearCe, OjasError> {
        const OP: &str = "linear_cross_entropy_mean";
        let d = linear_ce_dims(input, weight, targets, chunk)?;
        let (x, w, t) = (self.operand(OP, input)?, self.operand(OP, weight)?, self.operand(OP, targets)?);
        let loss = self.output(OP, &[1], DType::F32)?;
        let gx = if grads.input { Some(self.output(OP, input.shape(), DType::F32)?) } else { None };
        let gw = if grads.weight { Some(self.output(OP, weight.shape(), DType::F32)?) } else { None };
        self.check(OP, unsafe {
            ffi::omx_linear_cross_entropy_mean(
                self.raw(), x, w, code(input.dtype()), t, d.rows as u64, d.model_dim as u64, d.vocab as u64, i32::from(ignore_index.is_some()),
                ignore_index.unwrap_or(0), chunk.rows as u64, chunk.cols as u64, loss.ptr(), gx.as_ref().map_or(std::ptr::null_mut(), Output::ptr), ffi::OMX_F32,
                gw.as_ref().map_or(std::ptr::null_mut(), Output::ptr),
            )
        })?;
        Ok(LinearCe { loss: loss.into_tensor()?, grad_input: gx.map(Output::into_tensor).transpose()?, grad_weight: gw.map(Output::into_tensor).transpose()? })
    }

    fn cached_attention_forward(&self, q: &Tensor, k_cache: &Tensor, v_cache: &Tensor, kv_len: usize, window: Option<usize>) -> Result<Tensor, OjasError> {
        const OP: &str = "cached_attention_forward";
        let d = cached_attention_dims(q, k_cache, v_cache, kv_len, window)?;
        let (qp, kp, vp) = (self.operand(OP, q)?, self.operand(OP, k_cache)?, self.operand(OP, v_cache)?);
        let out = self.output(OP, q.shape(), DType::F32)?;
        self.check(OP, unsafe {
            ffi::omx_cached_attention_forward(self.raw(), qp, kp, vp, code(k_cache.dtype()), out.ptr(), d.batch as u64, d.new as u64, d.heads as u64, d.kv_heads as u64, d.head_dim as u64, d.capacity as u64, kv_len as u64, window_arg(window))
        })?;
        out.into_tensor()
    }

    fn kv_cache_write(&self, cache: &mut Tensor, src: &Tensor, at: usize) -> Result<(), OjasError> {
        const OP: &str = "kv_cache_write";
        let d = kv_cache_write_dims(cache, src, at)?;
        let s = self.operand(OP, src)?;
        let dtype = code(cache.dtype());
        let c = self.operand_mut(OP, cache)?;
        self.check(OP, unsafe { ffi::omx_kv_cache_write(self.raw(), c, dtype, s, d.batch as u64, d.capacity as u64, d.kv_heads as u64, d.head_dim as u64, d.new as u64, at as u64) })
    }
}

impl Mi355xBackend {
    fn gate_forward(&self, op: &'static str, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor, saving: bool) -> Result<(Tensor, Option<Tensor>), OjasError> {
        let d = per_head_sigmoid_gate_forward_dims(input, weight, bias, attn_out)?;
        let (x, w, b, a) = (self.operand(op, input)?, self.operand(op, weight)?, self.operand(op, bias)?, self.operand(op, attn_out)?);
        let y = self.output(op, attn_out.shape(), DType::F32)?;
        let gates = if saving { Some(self.output(op, &[d.rows, d.heads], DType::F32)?) } else { None };
        self.check(op, unsafe {
            ffi::omx_per_head_sigmoid_gate_forward(self.raw(), x, w, code(input.dtype()), b, a, code(attn_out.dtype()), y.ptr(), ffi::OMX_F32, gates.as_ref().map_or(std::ptr::null_mut(), Output::ptr), d.rows as u64, d.d_model as u64, d.heads as u64, d.head_dim as u64)
        })?;
        Ok((y.into_tensor()?, gates.map(Output::into_tensor).transpose()?))
    }

    fn gate_backward(&self, input: &Tensor, weight: &Tensor, bias: &Tensor, attn_out: &Tensor, grad_output: &Tensor, scales: Option<&Tensor>) -> Result<PerHeadGateGrad, OjasError> {
        const OP: &str = "per_head_sigmoid_gate_backward";
        let d = per_head_sigmoid_gate_backward_dims(input, weight, bias, attn_out, grad_output)?;
        let (x, w, b, a, g) = (self.operand(OP, input)?, self.operand(OP, weight)?, self.operand(OP, bias)?, self.operand(OP, attn_out)?, self.operand(OP, grad_output)?);
        let saved = match scales {
            Some(s) => self.operand(OP, s)?,
            None => std::ptr::null(),
        };
        let (gi, gw, gb, ga) = (self.output(OP, input.shape(), DType::F32)?, self.output(OP, weight.shape(), DType::F32)?, self.output(OP, bias.shape(), DType::F32)?, self.output(OP, attn_out.shape(), DType::F32)?);
        self.check(OP, unsafe {
            ffi::omx_per_head_sigmoid_gate_backward(self.raw(), x, w, code(input.dtype()), b, a, code(attn_out.dtype()), g, code(grad_output.dtype()), saved, gi.ptr(), ffi::OMX_F32, gw.ptr(), gb.ptr(), ga.ptr(), ffi::OMX_F32, d.rows as u64, d.d_model as u64, d.heads as u64, d.head_dim as u64)
        })?;
        Ok(PerHeadGateGrad { input: gi.into_tensor()?, weight: gw.into_tensor()?, bias: gb.into_tensor()?, attn_out: ga.into_tensor()? })
    }
}

impl Backend for Mi355xBackend {}

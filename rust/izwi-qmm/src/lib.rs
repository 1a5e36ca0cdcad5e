//! Safe wrappers over the C ABI of `libizwi_qmm.so` for izwi-core.
//!
//! What izwi-core gets: [`HipQMatMul`], a drop-in for the `QMatMul` inside
//! `Qwen3Projection::Quantized` (qwen3/core.rs:671-674; constructed at core.rs:710-715 and, packed,
//! core.rs:846-889; applied at core.rs:791-831), and [`HipDecodeLayer`], one decoder layer of
//! `Qwen3Layer::forward` (core.rs:1863-1881) for one token on device-resident buffers, which is the
//! call sequence the measured decode figures come from.
//!
//! Errors map onto the kinds of `izwi_core::Error` (crates/izwi-core/src/error.rs:6-53):
//! `IZWI_QMM_ERR_INVALID` -> `InvalidInput`, `IZWI_QMM_ERR_UNSUPPORTED` / `IZWI_QMM_ERR_NO_DEVICE` ->
//! `ModelLoadError`, `IZWI_QMM_ERR_HIP` -> `InferenceError`; the message is the library's own
//! (`izwi_qmm_last_error`, thread-local).
use std::ffi::CStr;
use std::os::raw::{c_int, c_void};

use izwi_qmm_sys as sys;

/// The error kinds of `izwi_core::Error` this path can produce; `From<Error> for izwi_core::Error`
/// is one `match` in izwi-core.
#[derive(Debug, Clone, PartialEq, Eq)]
pub enum Error {
    InvalidInput(String),
    ModelLoadError(String),
    InferenceError(String),
}

impl std::fmt::Display for Error {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        match self {
            Error::InvalidInput(m) => write!(f, "Invalid input: {m}"),
            Error::ModelLoadError(m) => write!(f, "Model loading failed: {m}"),
            Error::InferenceError(m) => write!(f, "Inference error: {m}"),
        }
    }
}
impl std::error::Error for Error {}
pub type Result<T> = std::result::Result<T, Error>;

fn check(rc: c_int) -> Result<()> {
    if rc == sys::IZWI_QMM_OK {
        return Ok(());
    }
    // SAFETY: the library returns a NUL-terminated string that lives until the thread's next failing call.
    let msg = unsafe { CStr::from_ptr(sys::izwi_qmm_last_error()) }.to_string_lossy().into_owned();
    Err(match rc {
        sys::IZWI_QMM_ERR_INVALID => Error::InvalidInput(msg),
        sys::IZWI_QMM_ERR_UNSUPPORTED | sys::IZWI_QMM_ERR_NO_DEVICE => Error::ModelLoadError(msg),
        _ => Error::InferenceError(msg),
    })
}

/// `candle_core::quantized::GgmlDType`, the block formats the library multiplies.
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum GgmlDType {
    Q8_0,
    Q4K,
    Q6K,
}
impl GgmlDType {
    pub fn id(self) -> c_int {
        match self {
            GgmlDType::Q8_0 => sys::IZWI_QMM_Q8_0,
            GgmlDType::Q4K => sys::IZWI_QMM_Q4_K,
            GgmlDType::Q6K => sys::IZWI_QMM_Q6_K,
        }
    }
}

/// Activation / output element type of the fused call (`izwi_qmm_out_dtype`).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum ElemType {
    F32,
    BF16,
}
impl ElemType {
    fn id(self) -> c_int {
        match self {
            ElemType::F32 => sys::IZWI_QMM_OUT_F32,
            ElemType::BF16 => sys::IZWI_QMM_OUT_BF16,
        }
    }
}

/// A HIP stream handle (`hipStream_t`); null is the default stream.
#[derive(Debug, Clone, Copy)]
pub struct Stream(pub *mut c_void);
impl Stream {
    pub const DEFAULT: Stream = Stream(std::ptr::null_mut());
}

/// `quantized_storage_bytes` (core.rs:891-909).
pub fn quantized_storage_bytes(rows: usize, cols: usize, dtype: GgmlDType) -> Result<u64> {
    let mut out = 0u64;
    check(unsafe { sys::izwi_qmm_storage_bytes(dtype.id(), rows as i64, cols as i64, &mut out) })?;
    Ok(out)
}

/// The quantized weight of one projection on the device: `QTensor` + `QMatMul`.
pub struct HipQMatMul {
    w: *mut sys::IzwiQmmWeight,
    n: usize,
    k: usize,
}
// Handles are immutable after creation and the library's calls are thread-safe on shared handles.
unsafe impl Send for HipQMatMul {}
unsafe impl Sync for HipQMatMul {}
impl Drop for HipQMatMul {
    fn drop(&mut self) {
        unsafe { sys::izwi_qmm_weight_destroy(self.w) }
    }
}

impl HipQMatMul {
    /// `QMatMul::from_arc(qtensor)` (core.rs:710-715): `blocks` are the tensor's GGUF block bytes
    /// (`QTensor::data()`), `n` output and `k` input features.
    pub fn from_blocks(dtype: GgmlDType, n: usize, k: usize, blocks: &[u8]) -> Result<Self> {
        let mut w = std::ptr::null_mut();
        check(unsafe {
            sys::izwi_qmm_weight_create(dtype.id(), n as i64, k as i64, blocks.as_ptr().cast(), blocks.len() as u64,
                                        sys::IZWI_QMM_HOST, &mut w)
        })?;
        Ok(Self { w, n, k })
    }

    /// `packed_qmatmul_from_qtensors` (core.rs:846-889): the parts' rows one after the other.
    pub fn packed(dtype: GgmlDType, k: usize, parts: &[(&[u8], usize)]) -> Result<Self> {
        let rows: Vec<i64> = parts.iter().map(|(_, r)| *r as i64).collect();
        let ptrs: Vec<*const c_void> = parts.iter().map(|(b, _)| b.as_ptr().cast()).collect();
        let lens: Vec<u64> = parts.iter().map(|(b, _)| b.len() as u64).collect();
        let mut w = std::ptr::null_mut();
        check(unsafe {
            sys::izwi_qmm_weight_create_packed(dtype.id(), parts.len() as i32, rows.as_ptr(), k as i64, ptrs.as_ptr(),
                                               lens.as_ptr(), sys::IZWI_QMM_HOST, &mut w)
        })?;
        Ok(Self { w, n: rows.iter().sum::<i64>() as usize, k })
    }

    pub fn out_features(&self) -> usize {
        self.n
    }
    pub fn in_features(&self) -> usize {
        self.k
    }
    pub fn raw(&self) -> *const sys::IzwiQmmWeight {
        self.w
    }

    /// Marks the LM head, so that the `lm_head_*` profile counters separate out (core.rs:1696-1702).
    pub fn set_lm_head(&mut self, is_lm_head: bool) -> Result<()> {
        check(unsafe { sys::izwi_qmm_weight_set_lm_head(self.w, is_lm_head as c_int) })
    }

    /// `QTensor::dequantize`, bit-identical to candle-core's `to_float`, into host memory.
    pub fn dequantize(&self) -> Result<Vec<f32>> {
        let mut out = vec![0f32; self.n * self.k];
        check(unsafe { sys::izwi_qmm_dequantize_f32(self.w, out.as_mut_ptr(), sys::IZWI_QMM_HOST, std::ptr::null_mut()) })?;
        Ok(out)
    }

    /// `QMatMul::forward` on host memory (core.rs:812): `x` is `[m, k]` row-major f32, the result
    /// `[m, n]`.  Staged and synchronous: the literal drop-in for a Candle CPU tensor.
    pub fn forward_host(&self, x: &[f32], m: usize) -> Result<Vec<f32>> {
        if x.len() != m * self.k {
            return Err(Error::InvalidInput(format!("expected {} activations, got {}", m * self.k, x.len())));
        }
        let mut y = vec![0f32; m * self.n];
        check(unsafe {
            sys::izwi_qmm_forward_f32(self.w, x.as_ptr(), m as i64, y.as_mut_ptr(), sys::IZWI_QMM_HOST, std::ptr::null_mut())
        })?;
        Ok(y)
    }

    /// The same on device buffers, asynchronous on `stream`.
    ///
    /// # Safety
    /// `x` must point to `m * k` and `y` to `m * n` f32 values in device memory of the weight's GPU,
    /// valid until the work queued on `stream` has run.
    pub unsafe fn forward_device(&self, x: *const f32, m: usize, y: *mut f32, stream: Stream) -> Result<()> {
        check(sys::izwi_qmm_forward_f32(self.w, x, m as i64, y, sys::IZWI_QMM_DEVICE, stream.0))
    }

    /// The whole `Quantized` arm of `Qwen3Projection::forward` (core.rs:795-829) plus the layer's
    /// residual add (core.rs:1875, 1879): `y = x W^T (+ residual)`, x and y in their own types.
    ///
    /// # Safety
    /// Device pointers of the stated element types and sizes; `residual` may be null or alias `y`.
    pub unsafe fn forward_fused_device(&self, x: *const c_void, x_type: ElemType, m: usize, residual: *const c_void,
                                       y: *mut c_void, y_type: ElemType, stream: Stream) -> Result<()> {
        check(sys::izwi_qmm_forward_fused(self.w, x, x_type.id(), m as i64, residual, y, y_type.id(),
                                          sys::IZWI_QMM_DEVICE, stream.0))
    }

    /// bf16 activations in, f32 or bf16 out (prefill sizes: the bf16 matrix-core kernel).
    ///
    /// # Safety
    /// Device pointers: `x` to `m * k` bf16 values, `y` to `m * n` values of `y_type`.
    pub unsafe fn forward_bf16_device(&self, x: *const u16, m: usize, y: *mut c_void, y_type: ElemType,
                                      stream: Stream) -> Result<()> {
        check(sys::izwi_qmm_forward_bf16(self.w, x, m as i64, y, y_type.id(), sys::IZWI_QMM_DEVICE, stream.0))
    }
}

/// The `Separate` arms of `Qwen3QkvProjection::forward` / `Qwen3GateUpProjection::forward`
/// (core.rs:1119-1127, 1274-1282) as one call: up to four weights of equal k on the same x.
///
/// # Safety
/// Device pointers; `ys[i]` holds `m * weights[i].out_features()` f32 values.
pub unsafe fn forward_group_device(weights: &[&HipQMatMul], x: *const f32, m: usize, ys: &[*mut f32],
                                   stream: Stream) -> Result<()> {
    if weights.len() != ys.len() {
        return Err(Error::InvalidInput("one output per weight".into()));
    }
    let ws: Vec<*const sys::IzwiQmmWeight> = weights.iter().map(|w| w.raw()).collect();
    check(sys::izwi_qmm_forward_group_f32(ws.as_ptr(), ws.len() as i32, x, m as i64, ys.as_ptr(), sys::IZWI_QMM_DEVICE,
                                          stream.0))
}

/// `Qwen3Mlp::forward` (core.rs:1786-1798): `down(silu(gate x) * up x)` as one call.
///
/// # Safety
/// Device pointers: `x` `[m, hidden]`, `y` `[m, hidden]` f32.
pub unsafe fn mlp_forward_device(gate: &HipQMatMul, up: &HipQMatMul, down: &HipQMatMul, x: *const f32, m: usize,
                                 y: *mut f32, stream: Stream) -> Result<()> {
    check(sys::izwi_qmm_mlp_forward_f32(gate.raw(), up.raw(), down.raw(), x, m as i64, y, sys::IZWI_QMM_DEVICE, stream.0))
}

/// `Qwen3RuntimeProfileSnapshot` (core.rs:571-582) from the library's counters.
pub fn profile_snapshot() -> Result<sys::IzwiQmmProfileSnapshot> {
    let mut s = sys::IzwiQmmProfileSnapshot::default();
    check(unsafe { sys::izwi_qmm_profile_snapshot_get(&mut s) })?;
    Ok(s)
}

/// Reserves the stream's scratch buffer ahead of a HIP graph capture (no call allocates afterwards).
pub fn scratch_reserve(bytes: u64, stream: Stream) -> Result<()> {
    check(unsafe { sys::izwi_qmm_scratch_reserve(bytes, stream.0) })
}

/// Shape constants of a decoder layer's attention.
#[derive(Debug, Clone, Copy)]
pub struct AttentionCfg {
    pub heads: i64,
    pub kv_heads: i64,
    pub head_dim: i64,
    pub eps: f32,
    pub scale: f32,
}

/// One decoder layer for one token on device-resident state (`Qwen3Layer::forward`, core.rs:1863-1881).
/// Norm weights are device f32 vectors; the caches are `[kv_heads, capacity, head_dim]` f32.
pub struct HipDecodeLayer {
    pub q: HipQMatMul,
    pub k: HipQMatMul,
    pub v: HipQMatMul,
    pub o: HipQMatMul,
    pub gate: HipQMatMul,
    pub up: HipQMatMul,
    pub down: HipQMatMul,
    pub input_norm: *const f32,
    pub post_norm: *const f32,
    pub qk_norm: *const f32, // [2 * head_dim]: q weight, then k weight
    pub k_cache: *mut f32,
    pub v_cache: *mut f32,
    pub kv_capacity: i64,
}

/// Per-token device buffers the model allocates once.
pub struct HipDecodeScratch {
    pub q: *mut f32,
    pub k: *mut f32,
    pub v: *mut f32,
    pub attn: *mut f32,
    pub h: *mut f32,
}

impl HipDecodeLayer {
    /// `x`: device f32 `[hidden]`, updated in place (both residual adds happen inside the o / down
    /// calls).  Six launches, all asynchronous on `stream`; nothing allocates, so the whole token can
    /// be captured into a HIP graph after one eager token (or `scratch_reserve`).
    ///
    /// # Safety
    /// Every pointer is device memory of the sizes the field comments state, on the weights' GPU.
    pub unsafe fn forward_token(&self, x: *mut f32, cos_sin: *const f32, pos: i64, cfg: &AttentionCfg,
                                s: &HipDecodeScratch, stream: Stream) -> Result<()> {
        let ws = [self.q.raw(), self.k.raw(), self.v.raw()];
        let ys = [s.q, s.k, s.v];
        // input_layernorm + q | k | v: one launch
        check(sys::izwi_qmm_forward_group_normed_f32(ws.as_ptr(), 3, x, 1, self.input_norm, cfg.eps, ys.as_ptr(),
                                                     sys::IZWI_QMM_DEVICE, stream.0))?;
        // q / k head norm + rotary + cache append + attention over pos + 1 positions
        check(sys::izwi_decode_attention_step_f32(s.q, s.k, s.v, self.qk_norm, cos_sin, cfg.heads, cfg.kv_heads,
                                                  cfg.head_dim, cfg.eps, self.k_cache, self.v_cache, self.kv_capacity,
                                                  pos, cfg.scale, s.attn, stream.0))?;
        // o_proj + residual, in place in x
        check(sys::izwi_qmm_forward_fused(self.o.raw(), s.attn.cast(), sys::IZWI_QMM_OUT_F32, 1, x.cast(), x.cast(),
                                          sys::IZWI_QMM_OUT_F32, sys::IZWI_QMM_DEVICE, stream.0))?;
        // post_attention_layernorm + gate | up + silu(gate) * up: one launch
        check(sys::izwi_qmm_forward_gate_up_silu_normed_f32(self.gate.raw(), self.up.raw(), x, 1, self.post_norm,
                                                            cfg.eps, s.h, sys::IZWI_QMM_DEVICE, stream.0))?;
        // down_proj + residual, in place in x
        check(sys::izwi_qmm_forward_fused(self.down.raw(), s.h.cast(), sys::IZWI_QMM_OUT_F32, 1, x.cast(), x.cast(),
                                          sys::IZWI_QMM_OUT_F32, sys::IZWI_QMM_DEVICE, stream.0))
    }
}

/// Final norm + LM head + greedy argmax behind the last layer (core.rs:1690-1702, chat.rs:574-597).
///
/// # Safety
/// Device pointers: `x` `[hidden]`, `logits` `[vocab]` f32, `token` one u32.
pub unsafe fn logits_and_argmax(lm_head: &HipQMatMul, x: *const f32, final_norm: *const f32, eps: f32, logits: *mut f32,
                                token: *mut u32, stream: Stream) -> Result<()> {
    check(sys::izwi_qmm_forward_normed_f32(lm_head.raw(), x, 1, final_norm, eps, logits, sys::IZWI_QMM_DEVICE, stream.0))?;
    check(sys::izwi_argmax_f32(logits, 1, lm_head.out_features() as i64, token, sys::IZWI_QMM_DEVICE, stream.0))
}

/// The MLP half of a layer for a batch of 3..=64 decode tokens on activation records (the producers
/// write the quantized activations, no quantizer launch of its own): four launches.
///
/// # Safety
/// Device pointers; `rec_h` / `rec_i` hold `izwi_qmm_records_bytes(dtype, m, hidden / intermediate)` bytes.
#[allow(clippy::too_many_arguments)]
pub unsafe fn mlp_on_records(dtype: GgmlDType, gate: &HipQMatMul, up: &HipQMatMul, down: &HipQMatMul, x: *const f32,
                             post_norm: *const f32, eps: f32, m: usize, rec_h: *mut c_void, rec_i: *mut c_void,
                             g: *mut f32, u: *mut f32, y: *mut f32, stream: Stream) -> Result<()> {
    let hidden = gate.in_features() as i64;
    let inter = gate.out_features() as i64;
    check(sys::izwi_rms_norm_quantize_records_f32(dtype.id(), x, post_norm, m as i64, hidden, eps, rec_h, stream.0))?;
    let gu = [gate.raw(), up.raw()];
    let gu_out = [g, u];
    check(sys::izwi_qmm_forward_group_records_f32(gu.as_ptr(), 2, rec_h, m as i64, gu_out.as_ptr(), stream.0))?;
    check(sys::izwi_qmm_silu_mul_quantize_records_f32(dtype.id(), g, u, m as i64, inter, rec_i, stream.0))?;
    let d = [down.raw()];
    let d_out = [y];
    check(sys::izwi_qmm_forward_group_records_f32(d.as_ptr(), 1, rec_i, m as i64, d_out.as_ptr(), stream.0))
}

/// `impl Module for HipQMatMul`: what `Qwen3Projection::forward` calls (core.rs:812).  Host tensors in,
/// host tensor out (Candle 0.10.2 has no HIP device); a model that keeps its activations on the GPU
/// calls `forward_device` / `forward_fused_device` with its own buffers instead.
#[cfg(feature = "candle")]
impl candle_core::Module for HipQMatMul {
    fn forward(&self, x: &candle_core::Tensor) -> candle_core::Result<candle_core::Tensor> {
        let dims = x.dims().to_vec();
        let m: usize = dims[..dims.len() - 1].iter().product();
        let xs = x.to_dtype(candle_core::DType::F32)?.contiguous()?.flatten_all()?.to_vec1::<f32>()?;
        let y = self.forward_host(&xs, m).map_err(candle_core::Error::wrap)?;
        let mut out_dims = dims;
        *out_dims.last_mut().unwrap() = self.n;
        candle_core::Tensor::from_vec(y, out_dims, x.device())
    }
}

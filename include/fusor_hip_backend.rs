//! Safe wrappers over `fusor_hip_sys.rs`: the types a `Hip` arm of the reference's enums holds.
//!
//! `fusor-ml/fusor` dispatches on `Device::{Cpu,Gpu}` (src/device.rs:7-13), `QMatrix::{Cpu*,Gpu}`
//! (src/quantized.rs:80-99) and `Tensor::{Cpu,Gpu}` (src/lib.rs:91-94).  A maintainer adds
//! `Device::Hip(HipDevice)`, `QMatrix::Hip(HipQMatrix)` and `Tensor::Hip(HipTensor<R>)` and forwards each
//! method to the one of the same name below; `HipLlama` is the whole-decoder fast path for
//! `models/kalosm-llama` (`Model::from_gguf` + `forward` + the greedy loop).
//!
//! Written without a Rust toolchain at hand (none in the build image): it has not been compiled.  It uses
//! `std` only and expects `fusor_hip_sys.rs` as the sibling module `fusor_hip_sys` of the same crate.  The C side serialises nothing: every call on one device goes through `HipDevice::lock()`.
#![allow(dead_code)]

use std::ffi::{c_void, CString};
use std::path::Path;
use std::ptr;
use std::sync::{Arc, Mutex, MutexGuard};

use crate::fusor_hip_sys as sys;

/// `fusor::Error::Gpu`-like error of this backend: the C status and its message.
#[derive(Debug, Clone)]
pub struct HipError {
    pub status: sys::FhStatus,
    pub message: String,
}

impl std::fmt::Display for HipError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "fusor-hip error {}: {}", self.status, self.message)
    }
}
impl std::error::Error for HipError {}

pub type Result<T> = std::result::Result<T, HipError>;

fn check(status: sys::FhStatus) -> Result<()> {
    if status == sys::FH_OK {
        Ok(())
    } else {
        Err(HipError { status, message: sys::last_error() })
    }
}

// ------------------------------------------------------------------------------------------ device
struct DeviceInner {
    raw: *mut sys::FhDevice,
    calls: Mutex<()>,
}
// The handle may move between threads; calls are serialised by `calls`.
unsafe impl Send for DeviceInner {}
unsafe impl Sync for DeviceInner {}
impl Drop for DeviceInner {
    fn drop(&mut self) {
        unsafe { sys::fh_device_destroy(self.raw) };
    }
}

/// `Device::Hip` (cheap to clone, like the reference's `Arc`-backed devices).
#[derive(Clone)]
pub struct HipDevice(Arc<DeviceInner>);

impl HipDevice {
    /// `Device::gpu()` (fusor/src/device.rs:29-39): `FH_ERR_NO_DEVICE` when there is no gfx950 device.
    pub fn new(ordinal: i32) -> Result<Self> {
        let mut raw = ptr::null_mut();
        check(unsafe { sys::fh_device_create(ordinal, &mut raw) })?;
        Ok(HipDevice(Arc::new(DeviceInner { raw, calls: Mutex::new(()) })))
    }
    fn raw(&self) -> *mut sys::FhDevice {
        self.0.raw
    }
    fn lock(&self) -> MutexGuard<'_, ()> {
        self.0.calls.lock().unwrap_or_else(|e| e.into_inner())
    }
    /// Blocks until everything enqueued so far has run (`materialize()` / `poll_wait()` in the reference).
    pub fn sync(&self) -> Result<()> {
        let _g = self.lock();
        check(unsafe { sys::fh_device_sync(self.raw()) })
    }
}

// ------------------------------------------------------------------------------------------ buffers and tensors
struct Buffer {
    dev: HipDevice,
    ptr: *mut c_void,
    bytes: usize,
}
unsafe impl Send for Buffer {}
unsafe impl Sync for Buffer {}
impl Buffer {
    fn new(dev: &HipDevice, bytes: usize) -> Result<Self> {
        let mut p = ptr::null_mut();
        let _g = dev.lock();
        check(unsafe { sys::fh_malloc(dev.raw(), bytes, &mut p) })?;
        Ok(Buffer { dev: dev.clone(), ptr: p, bytes })
    }
}
impl Drop for Buffer {
    fn drop(&mut self) {
        let _g = self.dev.lock();
        unsafe { sys::fh_free(self.dev.raw(), self.ptr) };
    }
}

/// `Tensor::Hip`: a contiguous row-major f32 tensor of rank `R` on the device.
#[derive(Clone)]
pub struct HipTensor<const R: usize> {
    buf: Arc<Buffer>,
    shape: [usize; R],
}

impl<const R: usize> HipTensor<R> {
    pub fn shape(&self) -> &[usize; R] {
        &self.shape
    }
    pub fn device(&self) -> &HipDevice {
        &self.buf.dev
    }
    fn len(&self) -> usize {
        self.shape.iter().product()
    }
    fn ptr(&self) -> *const f32 {
        self.buf.ptr as *const f32
    }
    fn ptr_mut(&self) -> *mut f32 {
        self.buf.ptr as *mut f32
    }
    /// `Tensor::uninit`
    pub fn uninit(dev: &HipDevice, shape: [usize; R]) -> Result<Self> {
        let n: usize = shape.iter().product();
        Ok(HipTensor { buf: Arc::new(Buffer::new(dev, n * 4)?), shape })
    }
    /// `Tensor::from_slice` (fusor/src/lib.rs:356-368)
    pub fn from_slice(dev: &HipDevice, shape: [usize; R], data: &[f32]) -> Result<Self> {
        assert_eq!(data.len(), shape.iter().product::<usize>(), "shape does not match the data");
        let t = Self::uninit(dev, shape)?;
        let _g = dev.lock();
        check(unsafe { sys::fh_upload(dev.raw(), t.buf.ptr, data.as_ptr().cast(), data.len() * 4) })?;
        Ok(t)
    }
    /// `as_slice().await`: blocks until the stream reaches the copy.
    pub fn to_vec(&self) -> Result<Vec<f32>> {
        let mut out = vec![0f32; self.len()];
        let dev = self.device();
        let _g = dev.lock();
        check(unsafe { sys::fh_download(dev.raw(), out.as_mut_ptr().cast(), self.buf.ptr, out.len() * 4) })?;
        Ok(out)
    }
    fn rows_cols(&self) -> (usize, usize) {
        let cols = self.shape[R - 1];
        (self.len() / cols.max(1), cols)
    }
    /// `Tensor::q_mat_mul` (fusor/src/lib.rs:1132-1223): the last dimension is contracted with the weight's
    /// in_features; a mismatch panics as the reference does (cpu/src/quantized.rs:270-274).
    pub fn q_mat_mul(&self, w: &HipQMatrix) -> Result<Self> {
        let (m, k) = self.rows_cols();
        assert_eq!(k, w.shape[1], "Matrix dimension mismatch: lhs columns != weight in_features");
        let mut shape = self.shape;
        shape[R - 1] = w.shape[0];
        let y = Self::uninit(self.device(), shape)?;
        let _g = self.device().lock();
        check(unsafe { sys::fh_qmatmul(w.raw, self.ptr(), m as i32, y.ptr_mut()) })?;
        Ok(y)
    }
    /// `silu(x . Wg^T) * (x . Wu^T)` with `gate_up = QMatrix::concat_rows(&[gate, up])`
    /// (models/kalosm-llama/src/raw/attention_layer.rs:186-196), one launch.
    pub fn q_mat_mul_swiglu(&self, gate_up: &HipQMatrix) -> Result<Self> {
        let (m, k) = self.rows_cols();
        assert_eq!(k, gate_up.shape[1]);
        let mut shape = self.shape;
        shape[R - 1] = gate_up.shape[0] / 2;
        let y = Self::uninit(self.device(), shape)?;
        let _g = self.device().lock();
        check(unsafe { sys::fh_qmatmul_swiglu(gate_up.raw, self.ptr(), m as i32, y.ptr_mut()) })?;
        Ok(y)
    }
    /// `rms_norm_fused` / `rms_norm_residual_fused` (fusor/src/composite/normalization.rs:287-401)
    pub fn rms_norm_fused(&self, residual: Option<&Self>, weight: &HipTensor<1>, bias: Option<&HipTensor<1>>, eps: f32) -> Result<Self> {
        let (rows, cols) = self.rows_cols();
        let y = Self::uninit(self.device(), self.shape)?;
        let _g = self.device().lock();
        check(unsafe {
            sys::fh_rms_norm(
                self.device().raw(),
                self.ptr(),
                residual.map_or(ptr::null(), |r| r.ptr()),
                weight.ptr(),
                bias.map_or(ptr::null(), |b| b.ptr()),
                eps,
                rows as i32,
                cols as i32,
                y.ptr_mut(),
            )
        })?;
        Ok(y)
    }
    /// `(a + b) + c` (raw/mod.rs:1036)
    pub fn add3(&self, b: &Self, c: Option<&Self>) -> Result<Self> {
        let y = Self::uninit(self.device(), self.shape)?;
        let _g = self.device().lock();
        check(unsafe {
            sys::fh_add3(self.device().raw(), self.ptr(), b.ptr(), c.map_or(ptr::null(), |t| t.ptr()), y.ptr_mut(), self.len() as i64)
        })?;
        Ok(y)
    }
}

impl HipTensor<1> {
    /// `top_k_pairs(k)` (fusor/src/lib.rs:416-447), k <= 256
    pub fn top_k_pairs(&self, k: usize) -> Result<Vec<(u32, f32)>> {
        if k == 0 {
            return Ok(Vec::new());
        }
        let dev = self.device();
        let ids = Buffer::new(dev, k * 4)?;
        let vals = Buffer::new(dev, k * 4)?;
        let found = Buffer::new(dev, 4)?;
        let (mut hi, mut hv, mut hf) = (vec![0u32; k], vec![0f32; k], [0u32; 1]);
        let _g = dev.lock();
        unsafe {
            check(sys::fh_top_k(dev.raw(), self.ptr(), self.len() as i64, k as i32, ids.ptr.cast(), vals.ptr.cast(), found.ptr.cast()))?;
            check(sys::fh_download(dev.raw(), hi.as_mut_ptr().cast(), ids.ptr, k * 4))?;
            check(sys::fh_download(dev.raw(), hv.as_mut_ptr().cast(), vals.ptr, k * 4))?;
            check(sys::fh_download(dev.raw(), hf.as_mut_ptr().cast(), found.ptr, 4))?;
        }
        let n = hf[0] as usize;
        Ok(hi.into_iter().zip(hv).take(n).collect())
    }

    /// `sample_standard_token` / `sample_mirostat2_token` (fusor-ml/core/src/sampling/pipeline.rs): `params.kind`
    /// selects the sampler, `mu` is the Mirostat state (a one-element tensor, updated in place).
    /// `None` when no logit is finite.
    pub fn sample_token(&self, params: &sys::FhSamplerParams, previous_tokens: &[u32], mu: Option<&HipTensor<1>>) -> Result<Option<u32>> {
        let dev = self.device();
        let result = Buffer::new(dev, 8)?;
        let mut host = [0u32; 2];
        let _g = dev.lock();
        unsafe {
            check(sys::fh_sample_token(
                dev.raw(), self.ptr(), self.len() as i64, params,
                if previous_tokens.is_empty() { std::ptr::null() } else { previous_tokens.as_ptr() },
                previous_tokens.len() as u32, std::ptr::null(),
                mu.map_or(std::ptr::null_mut(), |t| t.ptr() as *mut f32), result.ptr.cast(), std::ptr::null_mut(), std::ptr::null_mut(),
            ))?;
            check(sys::fh_download(dev.raw(), host.as_mut_ptr().cast(), result.ptr, 8))?;
        }
        Ok((host[0] == 1).then_some(host[1]))
    }
}

impl HipTensor<4> {
    /// `flash_attention(&k, &v, scale, mask)` (fusor/src/composite/flash_attention.rs:58-109) for contiguous
    /// `[b, h, s, d]` operands; `mask_kind` is one of `sys::FH_MASK_*`, `mask` the additive mask when it needs one.
    pub fn flash_attention(&self, k: &Self, v: &Self, scale: f32, mask_kind: i32, mask: Option<&HipTensor<2>>) -> Result<Self> {
        let [b, hq, sq, d] = self.shape;
        let [_, hkv, skv, _] = k.shape;
        assert_eq!(hq % hkv, 0, "Number of Q heads must be divisible by number of K/V heads");
        let out = Self::uninit(self.device(), self.shape)?;
        let _g = self.device().lock();
        check(unsafe {
            sys::fh_flash_attention(
                self.device().raw(),
                sys::FH_F32,
                self.ptr().cast(),
                (hq * sq * d) as i64,
                (sq * d) as i64,
                d as i64,
                k.ptr().cast(),
                v.ptr().cast(),
                (hkv * skv * d) as i64,
                (skv * d) as i64,
                d as i64,
                b as i32,
                hq as i32,
                hkv as i32,
                sq as i32,
                skv as i32,
                d as i32,
                scale,
                mask_kind,
                mask.map_or(ptr::null(), |m| m.ptr()),
                out.ptr_mut().cast(),
            )
        })?;
        Ok(out)
    }
}

// ------------------------------------------------------------------------------------------ weights
/// `QMatrix::Hip`
pub struct HipQMatrix {
    dev: HipDevice,
    raw: *mut sys::FhQMatrix,
    shape: [usize; 2],
    ggml_type: u32,
}
unsafe impl Send for HipQMatrix {}
unsafe impl Sync for HipQMatrix {}
impl Drop for HipQMatrix {
    fn drop(&mut self) {
        let _g = self.dev.lock();
        unsafe { sys::fh_qmatrix_free(self.raw) };
    }
}

impl HipQMatrix {
    pub fn shape(&self) -> &[usize; 2] {
        &self.shape
    }
    pub fn ggml_type(&self) -> u32 {
        self.ggml_type
    }
    /// `QMatrix::from_raw_bytes` (fusor/src/quantized.rs:183-225); `FH_ERR_UNSUPPORTED` maps to
    /// `GgufReadError::UnsupportedDType`.
    pub fn from_raw_bytes(dev: &HipDevice, shape: [usize; 2], bytes: &[u8], ggml_type: u32) -> Result<Self> {
        let mut raw = ptr::null_mut();
        let _g = dev.lock();
        check(unsafe {
            sys::fh_qmatrix_from_gguf_bytes(dev.raw(), ggml_type, shape[0] as i64, shape[1] as i64, bytes.as_ptr().cast(), bytes.len(), &mut raw)
        })?;
        Ok(HipQMatrix { dev: dev.clone(), raw, shape, ggml_type })
    }
    /// `QMatrix::concat_rows` (fusor/src/quantized.rs:102-112): `None` where the reference returns `None`.
    pub fn concat_rows(parts: &[&Self]) -> Result<Option<Self>> {
        let first = match parts.first() {
            Some(f) => *f,
            None => return Ok(None),
        };
        let raws: Vec<*const sys::FhQMatrix> = parts.iter().map(|p| p.raw as *const sys::FhQMatrix).collect();
        let mut raw = ptr::null_mut();
        let _g = first.dev.lock();
        let st = unsafe { sys::fh_qmatrix_concat_rows(first.dev.raw(), raws.as_ptr(), raws.len() as i32, &mut raw) };
        if st == sys::FH_ERR_UNSUPPORTED {
            return Ok(None);
        }
        check(st)?;
        let rows: usize = parts.iter().map(|p| p.shape[0]).sum();
        Ok(Some(HipQMatrix { dev: first.dev.clone(), raw, shape: [rows, first.shape[1]], ggml_type: first.ggml_type }))
    }
    /// `QMatrix::dequantize` (fusor/src/quantized.rs:233-279): bit-exact `GgufBlock::dequantize` values.
    pub fn dequantize(&self) -> Result<HipTensor<2>> {
        let out = HipTensor::<2>::uninit(&self.dev, self.shape)?;
        let _g = self.dev.lock();
        check(unsafe { sys::fh_qmatrix_dequantize(self.raw, out.ptr_mut()) })?;
        Ok(out)
    }
}

// ------------------------------------------------------------------------------------------ model files and the decoder
/// `GgufMetadata` + `VarBuilder` over one mapped file.
pub struct HipGguf {
    raw: *mut sys::FhGguf,
}
unsafe impl Send for HipGguf {}
impl Drop for HipGguf {
    fn drop(&mut self) {
        unsafe { sys::fh_gguf_close(self.raw) };
    }
}
impl HipGguf {
    pub fn open(path: &Path) -> Result<Self> {
        let c = CString::new(path.to_string_lossy().as_bytes()).expect("path with a NUL byte");
        let mut raw = ptr::null_mut();
        check(unsafe { sys::fh_gguf_open(c.as_ptr(), &mut raw) })?;
        Ok(HipGguf { raw })
    }
    /// `GgufMetadata::get_value(key)` for integer values (`to_u32()` and friends); `None` when the key is absent.
    pub fn get_int(&self, key: &str) -> Result<Option<i64>> {
        let c = CString::new(key).expect("key with a NUL byte");
        let mut v = 0i64;
        let st = unsafe { sys::fh_gguf_meta_int(self.raw, c.as_ptr(), &mut v) };
        if st == sys::FH_ERR_NOT_FOUND {
            return Ok(None);
        }
        check(st)?;
        Ok(Some(v))
    }
    /// `VarBuilder::get(key, device)` (fusor/src/varbuilder.rs:79-127)
    pub fn get(&self, key: &str, dev: &HipDevice) -> Result<HipQMatrix> {
        let c = CString::new(key).expect("key with a NUL byte");
        let mut raw = ptr::null_mut();
        let _g = dev.lock();
        check(unsafe { sys::fh_qmatrix_from_gguf_tensor(dev.raw(), self.raw, c.as_ptr(), &mut raw) })?;
        let (mut ty, mut n, mut k, mut bytes) = (0u32, 0i64, 0i64, 0u64);
        check(unsafe { sys::fh_qmatrix_info(raw, &mut ty, &mut n, &mut k, &mut bytes) })?;
        Ok(HipQMatrix { dev: dev.clone(), raw, shape: [n as usize, k as usize], ggml_type: ty })
    }
}

/// The Llama-architecture decoder of `models/kalosm-llama/src/raw/mod.rs` driven inside the library: prompt in one
/// pass, then decode steps replayed from a captured graph with the sampled token kept on the device.
pub struct HipLlama {
    dev: HipDevice,
    raw: *mut sys::FhLlama,
    pub config: sys::FhLlamaConfig,
}
unsafe impl Send for HipLlama {}
impl Drop for HipLlama {
    fn drop(&mut self) {
        let _g = self.dev.lock();
        unsafe { sys::fh_llama_destroy(self.raw) };
    }
}
impl HipLlama {
    /// `Model::from_gguf` (raw/mod.rs:284-648) for architecture `llama`; `max_context` caps the KV cache,
    /// `rope_scaling` is the reference's argument of that name (raw/mod.rs:271).
    pub fn from_gguf(dev: &HipDevice, file: &HipGguf, max_context: Option<usize>, rope_scaling: Option<sys::FhRopeScaling>) -> Result<Self> {
        let mut config = sys::FhLlamaConfig::default();
        check(unsafe { sys::fh_llama_config_from_gguf(file.raw, &mut config) })?;
        if let Some(c) = max_context {
            config.ctx = config.ctx.min(c as i32);
        }
        let mut raw = ptr::null_mut();
        {
            let _g = dev.lock();
            check(unsafe { sys::fh_llama_create(dev.raw(), &config, &mut raw) })?;
        }
        // the guard lives in an inner scope: an early return drops it before `model`, whose Drop takes the lock
        let model = HipLlama { dev: dev.clone(), raw, config };
        {
            let _g = dev.lock();
            check(unsafe { sys::fh_llama_load_gguf(model.raw, file.raw) })?;
            if let Some(scaling) = rope_scaling.as_ref() {
                check(unsafe { sys::fh_llama_set_rope_scaling(model.raw, scaling) })?;
            }
            check(unsafe { sys::fh_llama_finalize(model.raw) })?;
        }
        Ok(model)
    }
    /// `Model::forward` (raw/mod.rs:851-865): logits of the last of `tokens` at the current position.
    pub fn forward(&mut self, tokens: &[u32]) -> Result<Vec<f32>> {
        let mut logits = vec![0f32; self.config.vocab as usize];
        let _g = self.dev.lock();
        check(unsafe { sys::fh_llama_forward(self.raw, tokens.as_ptr(), tokens.len() as i32, logits.as_mut_ptr(), ptr::null_mut()) })?;
        Ok(logits)
    }
    /// The lines the last `forward` traced (`KALOSM_TRACE_LAYER_NAN`, `KALOSM_TRACE_FORWARD_TIMING`,
    /// `FUSOR_TRACE_GPU_KERNELS` in the environment, or the `trace_*` options of the device); the reference hands
    /// the same lines to `tracing::warn!` / `tracing::info!` (raw/mod.rs:46-52, :946-950, :1041-1043).
    pub fn trace_text(&self) -> Result<String> {
        let mut len = 0usize;
        check(unsafe { sys::fh_llama_trace_text(self.raw, ptr::null_mut(), 0, &mut len) })?;
        let mut buf = vec![0u8; len + 1];
        check(unsafe { sys::fh_llama_trace_text(self.raw, buf.as_mut_ptr().cast(), len + 1, ptr::null_mut()) })?;
        buf.truncate(len);
        Ok(String::from_utf8_lossy(&buf).into_owned())
    }
    /// Greedy decoding of `steps` tokens after `first_token`, entirely on the device.
    pub fn decode_greedy(&mut self, first_token: u32, steps: usize) -> Result<Vec<u32>> {
        let mut out = vec![0u32; steps];
        let _g = self.dev.lock();
        check(unsafe { sys::fh_llama_decode_greedy(self.raw, first_token, steps as i32, out.as_mut_ptr(), ptr::null_mut()) })?;
        Ok(out)
    }
    /// Sampled decoding with the token resident on the device (models/kalosm-llama/src/model/inference.rs:38-173):
    /// `randoms` holds one uniform number per step (the host RNG of the reference's sampler draws them),
    /// `previous` the token history before `first_token`, `repetition_range` the window of the penalty (at most 64);
    /// `mu` is the Mirostat state, updated in place (unused by the standard sampler).  A step without a finite
    /// logit yields `u32::MAX`.
    pub fn decode_sampled(
        &mut self,
        first_token: u32,
        params: &sys::FhSamplerParams,
        randoms: &[f32],
        previous: &[u32],
        repetition_range: u32,
        mu: &mut f32,
    ) -> Result<Vec<u32>> {
        let mut out = vec![0u32; randoms.len()];
        let _g = self.dev.lock();
        check(unsafe {
            sys::fh_llama_decode_sampled(
                self.raw, first_token, randoms.len() as i32, params, randoms.as_ptr(),
                if previous.is_empty() { ptr::null() } else { previous.as_ptr() }, previous.len() as u32,
                repetition_range, mu, out.as_mut_ptr(), ptr::null_mut(),
            )
        })?;
        Ok(out)
    }
    /// `KvCache::reset` for every layer.
    pub fn reset(&mut self) -> Result<()> {
        let _g = self.dev.lock();
        check(unsafe { sys::fh_llama_reset(self.raw) })
    }
}

//! The `Hip` arms of the reference's enum facade, method by method.
//!
//! `fusor-ml/fusor` dispatches every tensor operation with a `match` on `Tensor::{Cpu,Gpu}`
//! (src/lib.rs:91-94), `QMatrix::{Cpu*,Gpu}` (src/quantized.rs:80-99) and `Device::{Cpu,Gpu}`
//! (src/device.rs:7-13).  The HIP backend is a third variant of each enum; this file holds, for every
//! method `models/kalosm-llama` calls through the facade, the arm a maintainer adds, next to the place it
//! goes (reference file:line).  The wrapper types (`HipDevice`, `HipTensor<R>`, `HipQMatrix`, ...) are those
//! of `fusor_hip_backend.rs`; the few methods that file does not have yet are defined at the end of this one.
//!
//! Written without a Rust toolchain at hand (none in the build image): not compiled.  The arms are written
//! against the reference tree as checked out beside this repository; generic bounds are abbreviated where
//! they do not change with the new variant.
#![allow(dead_code)]

use crate::fusor_hip_backend::{HipDevice, HipError, HipQMatrix, HipTensor};
use crate::fusor_hip_sys as sys;

// =====================================================================================================
// fusor/src/device.rs
// =====================================================================================================
//
//  pub enum Device {                                         // :7-13
//      Cpu,
//      Gpu(crate::gpu::Device),
// +    Hip(HipDevice),
//  }
//
//  impl Device {
// +    /// A gfx950 device through libfusor_hip.so; `Err` when there is none (FH_ERR_NO_DEVICE).
// +    pub fn hip(ordinal: i32) -> Result<Self, Error> {
// +        HipDevice::new(ordinal).map(Device::Hip).map_err(|e| Error::msg(e.to_string()))
// +    }
//
//      pub async fn auto() -> Self {                         // :60-78: HIP first, then wgpu, then CPU
// +        if let Ok(hip) = Self::hip(0) {
// +            return hip;
// +        }
//          match Self::gpu().await { Ok(gpu) => gpu, Err(_) => Device::Cpu }
//      }
//  }

// =====================================================================================================
// fusor/src/quantized.rs
// =====================================================================================================
//
//  pub enum QMatrix { CpuQ4_0(..), .., CpuF32(..), Gpu(fusor_core::QMatrix),      // :80-99
// +    Hip(HipQMatrix),
//  }
//
//  pub fn from_raw_bytes(device: &Device, shape, bytes: &[u8], ty: GgmlType) -> Result<Self, Error>   // :183-225
// +        Device::Hip(dev) => {
// +            let [n, k] = <[usize; 2]>::try_from(shape.as_ref()).map_err(|_| Error::msg("2-D weights only"))?;
// +            HipQMatrix::from_raw_bytes(dev, [n, k], bytes, ty as u32)       // GgmlType's discriminants are GGUF's
// +                .map(QMatrix::Hip)
// +                .map_err(|e| match e.status {
// +                    sys::FH_ERR_UNSUPPORTED => Error::from(GgufReadError::UnsupportedDType(ty as u32)),
// +                    _ => Error::msg(e.to_string()),
// +                })
// +        }
//
//  pub fn shape(&self) -> &[usize]                  // + QMatrix::Hip(q) => q.shape(),
//  pub fn ggml_type(&self) -> GgmlType              // + QMatrix::Hip(q) => GgmlType::try_from(q.ggml_type()).unwrap(),
//  pub fn is_cpu(&self) -> bool                     // + QMatrix::Hip(_) => false,
//
//  pub fn concat_rows(matrices: &[&Self]) -> Option<Self>                           // :102-112
// +        if let Some(QMatrix::Hip(_)) = matrices.first() {
// +            let parts: Option<Vec<&HipQMatrix>> =
// +                matrices.iter().map(|m| if let QMatrix::Hip(q) = m { Some(q) } else { None }).collect();
// +            return HipQMatrix::concat_rows(&parts?).ok().flatten().map(QMatrix::Hip);   // None on mixed types
// +        }
//
//  pub fn dequantize<const R: usize>(&self) -> Tensor<R, f32>                       // :233-279
// +        QMatrix::Hip(q) => {
// +            let dense = q.dequantize().expect("fusor-hip dequantize");             // [n, k] f32
// +            Tensor::Hip(dense.reshape(std::array::from_fn(|i| self.shape()[i])))
// +        }

// =====================================================================================================
// fusor/src/lib.rs
// =====================================================================================================
//
//  pub enum Tensor<const R: usize, D, B = ConcreteTensor<D, R>> {                   // :91-94
//      Cpu(..), Gpu(gpu::Tensor<R, D>),
// +    Hip(HipTensor<R>),                     // f32 only; f16 tensors stay on the existing variants
//  }
//
//  Tensor::from_slice / new / zeros (:356-368)      // + Device::Hip(dev) => Tensor::Hip(HipTensor::from_slice(dev, shape, data)?)
//  Tensor::as_slice().await (:356-368)              // + Tensor::Hip(t) => TensorSlice::from_vec(t.shape(), t.to_vec()?)
//  Tensor::shape / device                           // + Tensor::Hip(t) => *t.shape()  /  Device::Hip(t.device().clone())
//  reshape / squeeze / unsqueeze on contiguous data // + Tensor::Hip(t) => Tensor::Hip(t.reshape(new_shape))
//  transpose(1, 2) of [b, s, h, d] (attention_layer.rs:371-374) stays a VIEW: the Hip arm records the strides and
//  hands them to fh_rope_pair / fh_flash_attention_ex, which take (batch, head, position) strides; no copy.
//
//  pub fn matmul(&self, rhs: &Tensor<R, D, B2>) -> Tensor<R, D>                     // :1094-1103
// +        if let (Tensor::Hip(a), Tensor::Hip(b)) = (self, rhs) {
// +            return Tensor::Hip(a.matmul(b).expect("fusor-hip matmul"));
// +        }
//
//  pub fn q_mat_mul(&self, weights: &QMatrix) -> Tensor<R, f32>                     // :1132-1223
//      // rank 1 needs no [1, K] detour on this backend (fh_qmatmul takes m = 1), so `gpu_native` gains:
// +        let gpu_native = gpu_native || matches!((self, weights), (Tensor::Hip(_), QMatrix::Hip(_)));
//      match (self, weights) {
// +        // every block type AND dense F16 / F32 rows: the library routes them itself
// +        (Tensor::Hip(lhs), QMatrix::Hip(rhs)) => Tensor::Hip(lhs.q_mat_mul(rhs).expect("fusor-hip q_mat_mul")),
//          ..
//          _ => panic!("Cannot mix CPU and GPU tensors in q_mat_mul"),
//      }
//
//  pub async fn top_k_pairs(&self, k: usize) -> Result<Vec<(u32, f32)>, Error>      // :416-447
// +        Tensor::Hip(t) => t.top_k_pairs(k).map_err(|e| Error::msg(e.to_string())),   // same order and tie rule
//
//  impl Add / Mul for Tensor (:638-641), `silu()` (composite/activations.rs:47-65):
// +        (Tensor::Hip(a), Tensor::Hip(b)) => Tensor::Hip(a.add3(b, None)?)          // a + b
// +        silu(gate) * up, the only use of silu in the decoder (attention_layer.rs:186-196):
// +        (Tensor::Hip(g), Tensor::Hip(u)) => Tensor::Hip(g.silu_mul(u)?)

// =====================================================================================================
// fusor/src/composite/normalization.rs
// =====================================================================================================
//
//  pub fn rms_norm_fused(&self, weight, bias, eps) -> Tensor<R, D>                  // :287-326
// +        if let (Tensor::Hip(x), Tensor::Hip(w)) = (self, weight) {
// +            let b = bias.map(|b| if let Tensor::Hip(b) = b { b } else { panic!("bias on another device") });
// +            return Tensor::Hip(x.rms_norm_fused(None, w, b, eps).expect("fusor-hip rms_norm"));
// +        }
//
//  pub fn rms_norm_residual_fused(&self, residual, weight, bias, eps) -> Tensor<R, D>   // :356-401
// +        if let (Tensor::Hip(x), Tensor::Hip(r), Tensor::Hip(w)) = (self, residual, weight) {
// +            let b = bias.map(|b| if let Tensor::Hip(b) = b { b } else { panic!("bias on another device") });
// +            return Tensor::Hip(x.rms_norm_fused(Some(r), w, b, eps).expect("fusor-hip rms_norm"));
// +        }

// =====================================================================================================
// fusor/src/composite/rope.rs
// =====================================================================================================
//
//  pub fn forward(&self, q, k, start_pos) -> (Tensor<4, f32>, Tensor<4, f32>)       // :284-305
// +        if let (Tensor::Hip(q), Tensor::Hip(k), Tensor::Hip(cos), Tensor::Hip(sin)) = (q, k, &self.cos, &self.sin) {
// +            let (q, k) = rope_pair(q, k, cos, sin, start_pos, false).expect("fusor-hip rope");
// +            return (Tensor::Hip(q), Tensor::Hip(k));
// +        }
//  pub fn forward_interleaved(&self, q, k, start_pos)                                // :309-329
// +        ... the same with `true`: pairs (2i, 2i + 1), the layout of the llama architecture (raw/mod.rs:488-490)
//
//  RopeCache::new (:248-275): the tables are built on the device by `rope_tables` below, bit-equal to the CPU
//  construction (f32 powf / outer product / sin, cos).

// =====================================================================================================
// fusor/src/composite/flash_attention.rs
// =====================================================================================================
//
//  pub fn flash_attention(&self, k, v, scale, mask: Option<(&Tensor<2, D>, MaskKind)>) -> Tensor<4, D>   // :58-109
// +        if let (Tensor::Hip(q), Tensor::Hip(k), Tensor::Hip(v)) = (self, k, v) {
// +            let (kind, m) = match mask {
// +                None => (sys::FH_MASK_NONE, None),
// +                Some((_, MaskKind::Causal)) => (sys::FH_MASK_CAUSAL, None),          // generated in the kernel
// +                Some((m, MaskKind::QKMask)) => (sys::FH_MASK_ADDITIVE, Some(m)),
// +                Some((m, MaskKind::BatchKeyMask)) => (sys::FH_MASK_BATCH_KEY, Some(m)),
// +            };
// +            let m = m.map(|m| if let Tensor::Hip(m) = m { m } else { panic!("Mask must be on the same device") });
// +            return Tensor::Hip(q.flash_attention(k, v, scale, kind, m).expect("fusor-hip flash_attention"));
// +        }

// =====================================================================================================
// fusor/src/cache/kv_cache.rs and tensor_cache.rs
// =====================================================================================================
//
//  TensorCache<D> gains a device-resident variant: one `HipKvCache` (below) holds K and V of every layer.
//  pub fn append(&mut self, device, k, v) -> (keys, values)                          // kv_cache.rs:49-63
// +        if let (Device::Hip(_), Tensor::Hip(k), Tensor::Hip(v)) = (device, k, v) {
// +            let cache = self.hip.get_or_insert_with(|| HipKvCache::new(k.device(), 1, k.shape()[1], k.shape()[3], self.max_len));
// +            let (keys, values) = cache.append(0, k, v).expect("fusor-hip kv append");   // views of [0 .. len]
// +            return (Tensor::Hip(keys), Tensor::Hip(values));
// +        }
//  pub fn reset(&mut self)                                                           // :40-44
// +        if let Some(c) = &mut self.hip { c.reset().expect("fusor-hip kv reset"); }

// =====================================================================================================
// fusor/src/layers/embedding.rs
// =====================================================================================================
//
//  pub fn forward(&self, indices: &Tensor<N, u32, B>) -> Tensor<M, T>                // :43-89
// +                (Tensor::Cpu(ids), QMatrix::Hip(table)) => {                       // token ids arrive from the host
// +                    let flat: Vec<u32> = ids.as_ref().flatten_all().as_slice().to_vec();
// +                    let rows = embed_rows(table, &flat).expect("fusor-hip embedding");   // [count, embedding_dim]
// +                    Tensor::Hip(rows.reshape(final_dims))
// +                }

// =====================================================================================================
// Wrapper methods the arms above use and fusor_hip_backend.rs does not define yet
// =====================================================================================================
fn check(status: sys::FhStatus) -> Result<(), HipError> {
    if status == sys::FH_OK {
        Ok(())
    } else {
        Err(HipError { status, message: sys::last_error() })
    }
}

impl<const R: usize> HipTensor<R> {
    /// `Tensor::matmul` (fusor/src/lib.rs:1094-1103): the last two dimensions are the matrices, the others the batch.
    pub fn matmul(&self, rhs: &Self) -> Result<Self, HipError> {
        assert!(R >= 2, "Matrix multiplication requires at least 2 dimensions");
        let (m, k, n) = (self.shape()[R - 2], self.shape()[R - 1], rhs.shape()[R - 1]);
        assert_eq!(k, rhs.shape()[R - 2], "matmul: inner dimensions differ");
        assert_eq!(self.shape()[..R - 2], rhs.shape()[..R - 2], "matmul: batch dimensions differ");
        let batch: usize = self.shape()[..R - 2].iter().product();
        let mut shape = *self.shape();
        shape[R - 1] = n;
        let out = Self::uninit(self.device(), shape)?;
        let _g = self.device().lock_calls();
        check(unsafe {
            sys::fh_matmul(self.device().raw_handle(), sys::FH_F32, self.raw_ptr().cast(), (m * k) as i64, k as i64, 1,
                           rhs.raw_ptr().cast(), (k * n) as i64, n as i64, 1, batch as i32, m as i32, k as i32, n as i32,
                           out.raw_ptr_mut().cast())
        })?;
        Ok(out)
    }

    /// `silu(self) * up` (composite/activations.rs:47-65, attention_layer.rs:195)
    pub fn silu_mul(&self, up: &Self) -> Result<Self, HipError> {
        assert_eq!(self.shape(), up.shape());
        let out = Self::uninit(self.device(), *self.shape())?;
        let count: usize = self.shape().iter().product();
        let _g = self.device().lock_calls();
        check(unsafe { sys::fh_swiglu(self.device().raw_handle(), self.raw_ptr(), up.raw_ptr(), out.raw_ptr_mut(), count as i64) })?;
        Ok(out)
    }
}

/// `RopeCache::new` (composite/rope.rs:248-275): cos and sin tables `[context_length, head_dim / 2]`.
pub fn rope_tables(dev: &HipDevice, head_dim: usize, context_length: usize, theta: f32) -> Result<(HipTensor<2>, HipTensor<2>), HipError> {
    let cos = HipTensor::<2>::uninit(dev, [context_length, head_dim / 2])?;
    let sin = HipTensor::<2>::uninit(dev, [context_length, head_dim / 2])?;
    let _g = dev.lock_calls();
    check(unsafe { sys::fh_rope_tables(dev.raw_handle(), head_dim as i32, context_length as i32, theta, cos.raw_ptr_mut(), sin.raw_ptr_mut()) })?;
    Ok((cos, sin))
}

/// `RopeCache::forward{,_interleaved}` (composite/rope.rs:284-329) for contiguous `[b, h, s, d]` tensors.
pub fn rope_pair(q: &HipTensor<4>, k: &HipTensor<4>, cos: &HipTensor<2>, sin: &HipTensor<2>, start_pos: usize,
                 interleaved: bool) -> Result<(HipTensor<4>, HipTensor<4>), HipError> {
    let [b, hq, s, d] = *q.shape();
    let hk = k.shape()[1];
    let (qo, ko) = (HipTensor::<4>::uninit(q.device(), *q.shape())?, HipTensor::<4>::uninit(k.device(), *k.shape())?);
    let _g = q.device().lock_calls();
    check(unsafe {
        sys::fh_rope_pair(q.device().raw_handle(), q.raw_ptr(), (hq * s * d) as i64, (s * d) as i64, d as i64, k.raw_ptr(),
                          (hk * s * d) as i64, (s * d) as i64, d as i64, b as i32, hq as i32, hk as i32, s as i32, d as i32,
                          cos.raw_ptr(), sin.raw_ptr(), cos.shape()[0] as i32, start_pos as i32, interleaved as i32,
                          qo.raw_ptr_mut(), ko.raw_ptr_mut())
    })?;
    Ok((qo, ko))
}

/// `Embedding::forward` on a quantized table (layers/embedding.rs:43-89): rows `ids` of the table, dequantised.
pub fn embed_rows(table: &HipQMatrix, ids: &[u32]) -> Result<HipTensor<2>, HipError> {
    let out = HipTensor::<2>::uninit(table.device(), [ids.len(), table.shape()[1]])?;
    let _g = table.device().lock_calls();
    check(unsafe { sys::fh_embed_rows(table.raw_handle(), std::ptr::null(), ids.as_ptr(), ids.len() as i32, out.raw_ptr_mut()) })?;
    Ok(out)
}

/// `KvCache` (cache/kv_cache.rs:24-63) for all layers of a model: f32 like the reference's (raw/cache.rs:18).
pub struct HipKvCache {
    dev: HipDevice,
    raw: *mut sys::FhKvCache,
    kv_heads: usize,
    head_dim: usize,
}
unsafe impl Send for HipKvCache {}
impl Drop for HipKvCache {
    fn drop(&mut self) {
        let _g = self.dev.lock_calls();
        unsafe { sys::fh_kvcache_destroy(self.raw) };
    }
}
impl HipKvCache {
    pub fn new(dev: &HipDevice, layers: usize, kv_heads: usize, head_dim: usize, max_len: usize) -> Self {
        let mut raw = std::ptr::null_mut();
        let _g = dev.lock_calls();
        let st = unsafe { sys::fh_kvcache_create(dev.raw_handle(), layers as i32, kv_heads as i32, head_dim as i32, max_len as i32, sys::FH_F32, &mut raw) };
        assert_eq!(st, sys::FH_OK, "{}", sys::last_error());
        HipKvCache { dev: dev.clone(), raw, kv_heads, head_dim }
    }
    /// Appends `[1, kv_heads, s, head_dim]` keys and values of `layer`; returns views of positions `0 .. len`.
    pub fn append(&mut self, layer: usize, k: &HipTensor<4>, v: &HipTensor<4>) -> Result<(HipTensor<4>, HipTensor<4>), HipError> {
        let s = k.shape()[2];
        let _g = self.dev.lock_calls();
        check(unsafe { sys::fh_kvcache_append(self.raw, layer as i32, k.raw_ptr(), v.raw_ptr(), (s * self.head_dim) as i64, self.head_dim as i64, s as i32) })?;
        let (mut len, mut cap) = (0i32, 0i32);
        let (mut kp, mut vp) = (std::ptr::null(), std::ptr::null());
        check(unsafe { sys::fh_kvcache_view(self.raw, layer as i32, &mut len, &mut cap, &mut kp, &mut vp) })?;
        // views into the cache: head stride `capacity * head_dim`, handed to fh_flash_attention_ex as kv_sh
        Ok((HipTensor::view(&self.dev, kp, [1, self.kv_heads, len as usize, self.head_dim], [0, cap as usize * self.head_dim, self.head_dim, 1]),
            HipTensor::view(&self.dev, vp, [1, self.kv_heads, len as usize, self.head_dim], [0, cap as usize * self.head_dim, self.head_dim, 1])))
    }
    pub fn reset(&mut self) -> Result<(), HipError> {
        let _g = self.dev.lock_calls();
        check(unsafe { sys::fh_kvcache_reset(self.raw) })
    }
}

// Accessors the functions above expect on the wrapper types (one-line additions to fusor_hip_backend.rs):
//   HipDevice::raw_handle(&self) -> *mut sys::FhDevice        the private `raw()` made crate-visible
//   HipDevice::lock_calls(&self) -> MutexGuard<'_, ()>        the private `lock()` made crate-visible
//   HipTensor::raw_ptr / raw_ptr_mut                           the private `ptr()` / `ptr_mut()` made crate-visible
//   HipTensor::reshape(self, shape) -> HipTensor<R2>           same buffer, new shape (element counts equal)
//   HipTensor::view(dev, ptr, shape, strides) -> HipTensor<4>  a borrowed, strided view (no ownership of the buffer)
//   HipQMatrix::raw_handle(&self) -> *const sys::FhQMatrix, HipQMatrix::device(&self) -> &HipDevice

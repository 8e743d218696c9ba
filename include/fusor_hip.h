/*
 * fusor_hip.h -- C ABI of libfusor_hip.so, an AMD Instinct MI355X (gfx950) backend for
 * the quantized-inference hot path of Fusor (floneum/kalosm).
 *
 * The reference has no C ABI: its backend seam is the Rust enum facade of the
 * `fusor` crate (`Tensor::{Cpu,Gpu}`, `QMatrix::{Cpu*,Gpu}`, `Device::{Cpu,Gpu}`).
 * Each entry point below names the reference method it stands in for
 * (paths relative to the reference tree).  A Rust `Hip` arm of those enums binds
 * these symbols one to one.
 *
 * Conventions
 *   - Every function returns fh_status (0 = ok, negative = error); the message of
 *     the last error on the calling thread is fh_last_error().  Nothing aborts or
 *     throws across the boundary.  The reference panics on programmer errors
 *     (shape mismatch: fusor-ml/cpu/src/quantized.rs:270-274); here they are
 *     FH_ERR_INVALID.
 *   - All device pointers (`*_dev`) come from fh_malloc on the same fh_device.
 *     Work is enqueued on the device's single HIP stream and is asynchronous;
 *     fh_device_sync and the blocking copies are the only synchronisation points
 *     (the reference executes at `materialize()/as_slice()`,
 *     fusor-ml/core/src/tensor/mod.rs:197-274).
 *   - Calls on one fh_device must be serialised by the caller; handles may move
 *     between threads.
 *   - Tensors are row-major contiguous f32 unless a stride argument says otherwise.
 */
#ifndef FUSOR_HIP_H
#define FUSOR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef int32_t fh_status;
enum {
    FH_OK = 0,
    FH_ERR_INVALID = -1,     /* bad argument / shape mismatch */
    FH_ERR_HIP = -2,         /* a HIP runtime call failed */
    FH_ERR_UNSUPPORTED = -3, /* GgufReadError::UnsupportedDType (fusor-ml/core/src/quantized/mod.rs:485) */
    FH_ERR_OOM = -4,
    FH_ERR_NO_DEVICE = -5,   /* Device::gpu() failed (fusor-ml/fusor/src/device.rs:29-39) */
    FH_ERR_IO = -6,          /* GgufReadError::Io (fusor-ml/gguf/src/lib.rs:224-225): unreadable or truncated file */
    FH_ERR_NOT_FOUND = -7    /* Error::VarBuilder "Key ... not found" (fusor-ml/fusor/src/varbuilder.rs:81-83) */
};

/* GgmlType ids, fusor-ml/gguf/src/lib.rs:35-50.  Q4_0, Q8_0, Q4_K and Q6_K weights are re-laid-out for the
 * matrix-core kernels; Q5_0, Q5_K and dense F32 (0) / F16 (1) weights keep the file's layout and run through
 * the per-element kernels (every fh_qmatrix_* call, fh_embed_rows, fh_qmatmul, fh_qmatmul_add2 / _swiglu). */
enum { FH_Q4_0 = 2, FH_Q5_0 = 6, FH_Q8_0 = 8, FH_Q4_K = 12, FH_Q5_K = 13, FH_Q6_K = 14 };

/* MaskKind, fusor-ml/fusor/src/composite/flash_attention.rs:12-24 */
enum { FH_MASK_NONE = 0, FH_MASK_CAUSAL = 1, FH_MASK_ADDITIVE = 2 /* QKMask [sq, skv] */,
       FH_MASK_BATCH_KEY = 3 /* BatchKeyMask [b, skv], added for every head and query of a batch entry */ };

/* element types of attention operands */
enum { FH_F32 = 0, FH_F16 = 1 };

typedef struct fh_device fh_device;
typedef struct fh_qmatrix fh_qmatrix;
typedef struct fh_kvcache fh_kvcache;
typedef struct fh_llama fh_llama;
typedef struct fh_graph fh_graph;
typedef struct fh_gguf fh_gguf;

const char *fh_last_error(void);
/* Version string of the library, and the gfx target it was built for. */
const char *fh_version(void);

/* ------------------------------------------------------------------ device
 * Device::gpu() / Device::auto(), fusor-ml/fusor/src/device.rs:29-39, :60-78. */
fh_status fh_device_count(int32_t *count);
fh_status fh_device_create(int32_t ordinal, fh_device **out);
fh_status fh_device_destroy(fh_device *dev);
fh_status fh_device_sync(fh_device *dev);
/* Name, compute-unit count and memory of the device (for reports). */
fh_status fh_device_info(fh_device *dev, char *name, size_t name_cap, int32_t *compute_units,
                         uint64_t *total_mem_bytes);

/* Tensor::from_slice / new / zeros / as_slice, fusor-ml/fusor/src/lib.rs:356-368. */
fh_status fh_malloc(fh_device *dev, size_t bytes, void **out_dev);
fh_status fh_free(fh_device *dev, void *ptr_dev);
fh_status fh_memset(fh_device *dev, void *ptr_dev, int32_t byte, size_t bytes);
fh_status fh_upload(fh_device *dev, void *dst_dev, const void *src_host, size_t bytes);   /* blocking */
fh_status fh_download(fh_device *dev, void *dst_host, const void *src_dev, size_t bytes); /* blocking */
fh_status fh_copy(fh_device *dev, void *dst_dev, const void *src_dev, size_t bytes);      /* async */

/* Event timing on the device's stream (the reference's FUSOR_TRACE_GPU_KERNELS timestamp
 * queries, fusor-ml/core/src/compute_graph/resolve/run.rs:483-497). */
fh_status fh_timer_start(fh_device *dev);
fh_status fh_timer_stop(fh_device *dev, float *elapsed_ms); /* blocks until the stream reaches it */

/* debug_check_nan_f32, models/kalosm-llama/src/raw/mod.rs:9-58: what that probe logs about an f32 tensor - the
 * counts of NaN, +inf and -inf, the largest finite magnitude and the indices of the first NaNs (up to four, in
 * ascending order).  Blocking. */
typedef struct {
    uint64_t nan, pos_inf, neg_inf;
    float max_abs;
    uint32_t first_nan_count;
    uint64_t first_nan[4];
} fh_finite_stats;
fh_status fh_check_finite(fh_device *dev, const float *x_dev, int64_t count, fh_finite_stats *out_host);

/* Record-and-replay of a sequence of operator calls (the reference records a lazy graph and submits one
 * command buffer per resolve, fusor-ml/core/src/compute_graph/resolve/run.rs).  Between begin and end the
 * operator calls on `dev` are captured into a hipGraph instead of running; fh_graph_launch replays them.
 * Every buffer the captured calls touch must stay alive and unchanged in address; run the same calls once
 * eagerly first so that the library's internal scratch buffers are already sized (a capture that would
 * have to allocate fails with FH_ERR_INVALID).  Blocking calls (upload, download, sync, free) are not
 * allowed while capturing. */
fh_status fh_graph_begin(fh_device *dev);
fh_status fh_graph_end(fh_device *dev, fh_graph **out);
fh_status fh_graph_launch(fh_graph *g);
fh_status fh_graph_free(fh_graph *g);

/* ----------------------------------------------------------------- weights
 * QMatrix::from_raw_bytes(&Device, shape, &[u8], GgmlType), fusor-ml/fusor/src/quantized.rs:183-225.
 * `bytes` is the raw GGUF block stream of an [n, k] weight (blocks contiguous along k);
 * it is re-laid-out on the device, the host buffer is not referenced after return. */
fh_status fh_qmatrix_from_gguf_bytes(fh_device *dev, uint32_t ggml_type, int64_t n, int64_t k,
                                     const void *bytes, size_t len, fh_qmatrix **out);
/* QMatrix::concat_rows, fusor-ml/fusor/src/quantized.rs:102-112.  Where the reference returns None (parts of
 * different type or k, fusor-ml/core/src/quantized/mod.rs:329-337) the status is FH_ERR_UNSUPPORTED. */
fh_status fh_qmatrix_concat_rows(fh_device *dev, const fh_qmatrix *const *parts, int32_t count,
                                 fh_qmatrix **out);
fh_status fh_qmatrix_free(fh_qmatrix *q);
/* QMatrix::shape / ggml_type, fusor-ml/fusor/src/quantized.rs:114-180. */
fh_status fh_qmatrix_info(const fh_qmatrix *q, uint32_t *ggml_type, int64_t *n, int64_t *k,
                          uint64_t *device_bytes);
/* QMatrix::dequantize::<R>() -> Tensor<R,f32>, fusor-ml/fusor/src/quantized.rs:233-279.
 * out_dev is [n, k] f32; values are bit-identical to GgufBlock::dequantize
 * (fusor-ml/gguf/src/lib.rs:828-846, :1284-1288, :1526-1556, :2034-2085). */
fh_status fh_qmatrix_dequantize(const fh_qmatrix *q, float *out_dev);
/* Embedding::forward, fusor-ml/fusor/src/layers/embedding.rs:43-89: out[t,:] = dequantize(W)[ids[t],:].
 * ids_dev is u32 [count] on the device; ids >= n give FH_ERR_INVALID only when checked on the host
 * (pass ids_host != NULL to have them validated before launch). */
fh_status fh_embed_rows(const fh_qmatrix *q, const uint32_t *ids_dev, const uint32_t *ids_host,
                        int32_t count, float *out_dev);

/* ------------------------------------------------------------------ matmul
 * Tensor<R,f32>::q_mat_mul(&QMatrix), fusor-ml/fusor/src/lib.rs:1132-1223 ->
 * fusor-ml/cpu/src/quantized.rs:246-365: y[m, n] = sum_k x[m, k] * dequantize(W)[n, k].
 * x_dev [m, k] f32, y_dev [m, n] f32.  Any m >= 1; m <= 16 takes the bandwidth-tuned
 * decode kernels, larger m the MFMA tile kernel. */
fh_status fh_qmatmul(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev);
/* Epilogue forms the reference folds into the same dispatch:
 *   fh_qmatmul_add2:  y = (x.W^T + a) + b       raw/attention_layer.rs:168-173
 *   fh_qmatmul_swiglu: W = concat_rows(gate, up); y[m, i] = silu(g[m,i]) * u[m,i], y is [m, n/2]
 *                                               raw/attention_layer.rs:186-196 */
fh_status fh_qmatmul_add2(const fh_qmatrix *q, const float *x_dev, int32_t m, const float *a_dev,
                          const float *b_dev, float *y_dev);
fh_status fh_qmatmul_swiglu(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev);
/* Prefill activations given as bf16 (raw u16 bit patterns): same product, x_dev is [m, k] bf16. */
fh_status fh_qmatmul_bf16(const fh_qmatrix *q, const uint16_t *x_bf16_dev, int32_t m, float *y_dev);
/* The Q8_0 x Q8 variant: activations quantised per 32 along k exactly as BlockQ8_0::quantize
 * (fusor-ml/gguf/src/lib.rs:1150-1230, round half to even as on an AVX2 host) and each block
 * combined as GgufBlock::vec_dot (fusor-ml/gguf/src/lib.rs:1315-1358): integer dot, then
 * (sum as f32) * (d_w * d_a), summed over blocks in k order.  Q8_0 and Q4_0 weights only.
 * isums_dev (optional, int32 [m, n, k/32]) receives the exact integer block sums. */
fh_status fh_qmatmul_q8(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev,
                        int32_t *isums_dev);
/* BlockQ8_0::quantize over a flat f32 array (count % 32 == 0): out_dev is count/32 blocks of 34 bytes. */
fh_status fh_q8_0_quantize(fh_device *dev, const float *x_dev, int64_t count, void *out_dev);

/* Kernel selection override for measurement (the reference's FUSOR_* tile overrides,
 * fusor-ml/tile-ir-kernels/src/dispatch.rs:15-20).  key/value pairs documented in the README of
 * the csrc directory; unknown keys give FH_ERR_INVALID.
 * "deterministic" = 1: the decoder's device-side decode steps never add k-split partial sums with float atomics
 * (the output projection and the Q6_K down projection otherwise do, which makes the last bits of a step vary
 * from run to run): every run then gives the same bits, as the reference's CPU path does on one machine, at
 * about a tenth of the decode rate.  Every other entry point is deterministic as it is. */
fh_status fh_set_option(fh_device *dev, const char *key, int64_t value);

/* -------------------------------------------------------------------- norm
 * rms_norm_fused / rms_norm_residual_fused, fusor-ml/fusor/src/composite/normalization.rs:287-401:
 * y = ((x [+ residual]) / sqrt(mean((x [+ residual])^2) + eps)) * w [+ bias].  residual_dev and
 * bias_dev may be NULL.  x, residual, y are [rows, cols]; w, bias are [cols]. */
fh_status fh_rms_norm(fh_device *dev, const float *x_dev, const float *residual_dev,
                      const float *w_dev, const float *bias_dev, float eps, int32_t rows,
                      int32_t cols, float *y_dev);

/* -------------------------------------------------------------------- rope
 * RopeCache::new, fusor-ml/fusor/src/composite/rope.rs:241-275 and
 * models/kalosm-llama/src/raw/rope.rs:63-85: cos/sin tables [ctx, head_dim/2] built on the
 * host in f32 (powf, mul, cosf/sinf) and uploaded. */
fh_status fh_rope_tables(fh_device *dev, int32_t head_dim, int32_t ctx, float theta, float *cos_dev,
                         float *sin_dev);
/* create_inverse_frequency with a `rope_freqs.weight` tensor, models/kalosm-llama/src/raw/rope.rs:41-48:
 * inverse frequency i is multiplied by freq_weight_host[i] (head_dim/2 host floats; NULL: no weights). */
fh_status fh_rope_tables_weighted(fh_device *dev, int32_t head_dim, int32_t ctx, float theta,
                                  const float *freq_weight_host, float *cos_dev, float *sin_dev);
/* RopeScalingConfig, models/kalosm-llama/src/raw/mod.rs:163-169, applied as create_inverse_frequency does
 * (raw/rope.rs:20-38) before the weights; scaling and freq_weight_host may each be NULL. */
typedef struct {
    float factor, high_freq_factor, low_freq_factor;
    int32_t original_max_position_embeddings;
} fh_rope_scaling;
fh_status fh_rope_tables_scaled(fh_device *dev, int32_t head_dim, int32_t ctx, float theta,
                                const fh_rope_scaling *scaling, const float *freq_weight_host,
                                float *cos_dev, float *sin_dev);
/* RopeCache::forward{,_interleaved}(&q, &k, start_pos), rope.rs:284-329.  q is [b, hq, s, d] and
 * k is [b, hk, s, d] as VIEWS: element (b, h, t, c) of q lives at q_dev[b*q_sb + h*q_sh + t*q_st + c]
 * (strides in elements), likewise k.  Outputs are contiguous [b, h, s, d].  One launch rotates both. */
fh_status fh_rope_pair(fh_device *dev, const float *q_dev, int64_t q_sb, int64_t q_sh, int64_t q_st,
                       const float *k_dev, int64_t k_sb, int64_t k_sh, int64_t k_st, int32_t b,
                       int32_t hq, int32_t hk, int32_t s, int32_t d, const float *cos_dev,
                       const float *sin_dev, int32_t table_rows, int32_t start_pos,
                       int32_t interleaved, float *q_out_dev, float *k_out_dev);

/* ---------------------------------------------------------------- KV cache
 * KvCache::new / append / reset, fusor-ml/fusor/src/cache/kv_cache.rs:24-63 and
 * tensor_cache.rs:70-114, :304-312.  One object holds all layers.  Storage is
 * [layer][kv_head][capacity][head_dim] per K and V, f32 (the reference's cache type,
 * models/kalosm-llama/src/raw/cache.rs:18) or f16.  Capacity grows to the next power of two
 * (minimum 256, capped at max_len) preserving contents; exceeding max_len is FH_ERR_INVALID unless
 * the cache was switched to a sliding window (fh_kvcache_set_sliding). */
fh_status fh_kvcache_create(fh_device *dev, int32_t layers, int32_t kv_heads, int32_t head_dim,
                            int32_t max_len, int32_t dtype, fh_kvcache **out);
fh_status fh_kvcache_destroy(fh_kvcache *c);
/* Sliding-window caches (KvCache with a window, fusor-ml/fusor/src/cache/tensor_cache.rs:175-202):
 * once an append would exceed max_len the cache keeps the last max_len positions of [cached | new].
 * Applies to fh_kvcache_append; the decoder driver's captured steps do not evict. */
fh_status fh_kvcache_set_sliding(fh_kvcache *c, int32_t on);
fh_status fh_kvcache_reset(fh_kvcache *c);
/* Append s positions to `layer`.  k and v are [kv_heads, s, head_dim] f32 views with head stride
 * `sh` and position stride `st` (elements).  The cache length advances when the LAST layer is
 * appended (all layers receive the same s per step). */
fh_status fh_kvcache_append(fh_kvcache *c, int32_t layer, const float *k_dev, const float *v_dev,
                            int64_t sh, int64_t st, int32_t s);
/* Current length, capacity, and the device pointers of one layer's K and V planes
 * ([kv_heads, capacity, head_dim]). */
fh_status fh_kvcache_view(const fh_kvcache *c, int32_t layer, int32_t *len, int32_t *capacity,
                          const void **k_dev, const void **v_dev);

/* ------------------------------------------------------------------ dense matmul
 * Tensor::matmul, fusor-ml/fusor/src/lib.rs:1094-1103 (CPU form fusor-ml/cpu/src/matmul.rs:226-352; f16:
 * :159-179): C[b] = A[b] . B[b] with A [batch, m, k], B [batch, k, n], C contiguous [batch, m, n]; dtype FH_F32 or
 * FH_F16 for all three.  A and B are views: element (b, i, j) of A is a_dev[b * a_sb + i * a_sr + j * a_sc] (element
 * strides), likewise B, so transposed or sliced operands need no copy by the caller (the reference copies
 * non-contiguous operands to scratch first, matmul.rs:299-328).  f32 operands are multiplied as exact two-term f16
 * splits of values normalised per row of A and per column of B on the matrix cores with f32 accumulation (the
 * reference's gemm kernel order is not pinned: results agree to f32 rounding); f16 results are rounded once from the
 * f32 sum like the reference's f16 instantiation.  Dense F16 / F32 weight matrices of fh_qmatmul run through the
 * same tiles from 17 activation rows on. */
fh_status fh_matmul(fh_device *dev, int32_t dtype, const void *a_dev, int64_t a_sb, int64_t a_sr, int64_t a_sc,
                    const void *b_dev, int64_t b_sb, int64_t b_sr, int64_t b_sc, int32_t batch, int32_t m,
                    int32_t k, int32_t n, void *c_dev);

/* --------------------------------------------------------------- attention
 * Tensor<4>::flash_attention(&k, &v, scale, Option<(&mask, MaskKind)>),
 * fusor-ml/fusor/src/composite/flash_attention.rs:58-109 (GQA: kv head = h / (hq / hkv)).
 * q [b, hq, sq, d] view with strides (elements) q_sb, q_sh, q_st; k, v [b, hkv, skv, d] views
 * with strides kv_sb, kv_sh, kv_st; out contiguous [b, hq, sq, d].  dtype is FH_F32 or FH_F16 for
 * q/k/v/out alike (kv may be f16 with f32 q via fh_flash_attention_ex).  mask_dev is
 * [sq, skv] f32 for FH_MASK_ADDITIVE, ignored otherwise.  FH_MASK_CAUSAL lets query i see keys
 * j <= i + (skv - sq) (attention_mask.rs:46-66 with the offset padding of mask_cache.rs:73-88).
 * d <= 256; d of 64 or 128 takes the tuned kernels. */
fh_status fh_flash_attention(fh_device *dev, int32_t dtype, const void *q_dev, int64_t q_sb,
                             int64_t q_sh, int64_t q_st, const void *k_dev, const void *v_dev,
                             int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int32_t b, int32_t hq,
                             int32_t hkv, int32_t sq, int32_t skv, int32_t d, float scale,
                             int32_t mask_kind, const float *mask_dev, void *out_dev);
/* As above with separate element types: q/out of q_dtype, k/v of kv_dtype. */
fh_status fh_flash_attention_ex(fh_device *dev, int32_t q_dtype, int32_t kv_dtype, const void *q_dev,
                                int64_t q_sb, int64_t q_sh, int64_t q_st, const void *k_dev,
                                const void *v_dev, int64_t kv_sb, int64_t kv_sh, int64_t kv_st,
                                int32_t b, int32_t hq, int32_t hkv, int32_t sq, int32_t skv,
                                int32_t d, float scale, int32_t mask_kind, const float *mask_dev,
                                void *out_dev);

/* One query position per head against skv cached keys (b = 1, sq = 1, head_dim 128, no mask), for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference.  fh_flash_attention keeps the partial results of its key parts in a buffer the
 * library grows with hipMalloc; this variant keeps them in a file-scope device array of 540 672 bytes (64 query
 * heads x 16 key parts x 132 floats) that every GPU the library runs on holds until the process ends, and calls
 * no hipMalloc, hipFree or other allocating routine.  q and out are [hq, 128] contiguous, of q_dtype; k and v are
 * [hkv, skv, 128] views of kv_dtype with head stride kv_sh and position stride kv_st (elements, multiples of 8).
 * For f32 caches, and for f16 caches of fewer than 4096 keys, it runs the same kernels with the same cut of the key
 * range as fh_flash_attention and returns the same bits; for f16 caches from 4096 keys on fh_flash_attention takes
 * its matrix-core kernel while this entry point keeps the vector-ALU one with its 16 parts, and the two agree within
 * the attention tolerance (1e-2 absolute or 1e-3 relative).  hq x parts beyond the
 * array (more than 64 heads at 16 parts) is FH_ERR_INVALID with a message; shapes outside the list above are
 * FH_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two
 * device handles, two threads) race; calls on one handle's stream are ordered and safe.  Nothing needs clearing
 * between calls: every slot the merge reads is written by the same call first. */
fh_status fh_flash_attention_decode_static(fh_device *dev, int32_t q_dtype, int32_t kv_dtype,
                                           const void *q_dev, const void *k_dev, const void *v_dev,
                                           int64_t kv_sh, int64_t kv_st, int32_t hq, int32_t hkv, int32_t d,
                                           float scale, int32_t skv, void *out_dev);

/* -------------------------------------------------------------------- glue
 * silu(g) * u, fusor-ml/fusor/src/composite/activations.rs:47-65 + raw/attention_layer.rs:195 */
fh_status fh_swiglu(fh_device *dev, const float *gate_dev, const float *up_dev, float *y_dev,
                    int64_t count);
/* (a + b) + c, models/kalosm-llama/src/raw/mod.rs:1036; c_dev may be NULL for a + b. */
fh_status fh_add3(fh_device *dev, const float *a_dev, const float *b_dev, const float *c_dev,
                  float *y_dev, int64_t count);
/* [s, h, d] -> [h, s, d] (reshape + transpose(1,2) + to_concrete) and back; f32. */
fh_status fh_transpose_shd(fh_device *dev, const float *x_dev, int32_t s, int32_t h, int32_t d,
                           float *y_dev);
fh_status fh_cast_f32_f16(fh_device *dev, const float *x_dev, void *y_f16_dev, int64_t count);
fh_status fh_cast_f16_f32(fh_device *dev, const void *x_f16_dev, float *y_dev, int64_t count);
fh_status fh_cast_f32_bf16(fh_device *dev, const float *x_dev, void *y_bf16_dev, int64_t count);
/* Tensor::top_k_pairs(1), fusor-ml/fusor/src/lib.rs:416-447: largest finite value, ties to the
 * larger index, non-finite skipped; *id_dev = 0xFFFFFFFF when nothing is finite. */
fh_status fh_argmax(fh_device *dev, const float *x_dev, int64_t count, uint32_t *id_dev);
/* Tensor::top_k_pairs(k), fusor-ml/fusor/src/lib.rs:416-447, 1 <= k <= 256: ids_dev[k] / values_dev[k] in
 * descending order of the value, ties to the larger index, non-finite values skipped; *found_dev
 * (optional) = number of pairs found, the rest is filled with id 0xFFFFFFFF / NaN. */
fh_status fh_top_k(fh_device *dev, const float *x_dev, int64_t count, int32_t k, uint32_t *ids_dev,
                   float *values_dev, uint32_t *found_dev);

/* Token sampling on the device, fusor-ml/core/src/sampling: logit processors (row_kernels.rs:150-205:
 * repetition penalty over the previous tokens, then temperature), exact top-k in descending order (ties to
 * the larger id), then one of two samplers over the sorted candidates: the standard one (row_kernels.rs:799-919:
 * min_p against exp(value - max), top_p of the filtered weight, weighted pick) or Mirostat 2 (:672-797: cutoff
 * where the surprise -log2(p) exceeds mu, weighted pick, mu -= eta * (surprise - tau)).  `random` is the caller's
 * uniform number in [0, 1) (GpuStandardSamplerParams / GpuMirostat2SamplerParams, sampling/mod.rs:96-114).
 * The reference's retry status (0) never occurs: the top-k here is exact. */
#define FH_SAMPLER_STANDARD 0u
#define FH_SAMPLER_MIROSTAT2 1u
#define FH_SAMPLE_STATUS_SAMPLED 1u /* GPU_SAMPLE_STATUS_SAMPLED, sampling/mod.rs:25 */
#define FH_SAMPLE_STATUS_INVALID 2u /* no finite logit, sampling/mod.rs:26 */
#define FH_SAMPLER_PREVIOUS_TOKENS 64 /* GPU_SAMPLER_PREVIOUS_TOKENS, sampling/mod.rs:22 */
typedef struct fh_sampler_params {
    uint32_t kind;  /* FH_SAMPLER_* */
    uint32_t top_k; /* 1 .. 256 */
    float temperature;        /* 0 leaves the logits as they are */
    float repetition_penalty; /* applied when above 1 */
    float top_p, min_p;       /* standard sampler */
    float tau, eta;           /* Mirostat 2 */
    float random;
} fh_sampler_params;
/* sample_token_pending, sampling/pipeline.rs: result_dev[0] = status, result_dev[1] = token id.  previous_host:
 * the caller's token history, of which the last 64 are used (63 when previous_tail_dev, one id left in device
 * memory by an earlier call, is appended: processors.rs:20-81).  mu_dev: the Mirostat state (one float, device),
 * updated in place; may be NULL for the standard sampler.  ids_dev / values_dev (optional, top_k entries each)
 * receive the processed candidates in sorted order (a processed -0.0 reads 0.0), id 0xFFFFFFFF / NaN where
 * fewer were finite. */
fh_status fh_sample_token(fh_device *dev, const float *logits_dev, int64_t count, const fh_sampler_params *params,
                          const uint32_t *previous_host, uint32_t n_previous, const uint32_t *previous_tail_dev,
                          float *mu_dev, uint32_t *result_dev, uint32_t *ids_dev, float *values_dev);

/* -------------------------------------------------------------- GGUF files
 * GgufMetadata::read, fusor-ml/gguf/src/lib.rs:559-613: versions 1 .. 3, metadata key/values, tensor
 * directory (dimensions reversed to row-major order, :583), payload start rounded up to
 * `general.alignment` (default 32, :597-606).  Host code only: no device is needed.  Error mapping of
 * GgufReadError (:222-241): Io -> FH_ERR_IO, MagicBytesMismatch / InvalidBool / InvalidValueType /
 * InvalidTensorSize -> FH_ERR_INVALID, UnsupportedVersion / UnsupportedDType -> FH_ERR_UNSUPPORTED.
 * fh_gguf_open maps the file read-only; fh_gguf_open_memory parses a caller-owned buffer that must outlive
 * the handle.  Strings are handed out as (pointer, length) into the file image: not NUL-terminated, trailing
 * NUL bytes already dropped (:330-332), bytes not re-encoded (the reference replaces invalid UTF-8). */
fh_status fh_gguf_open(const char *path, fh_gguf **out);
fh_status fh_gguf_open_memory(const void *bytes, size_t len, fh_gguf **out);
fh_status fh_gguf_close(fh_gguf *g);
fh_status fh_gguf_info(const fh_gguf *g, uint32_t *version, uint64_t *tensor_count, uint64_t *metadata_count,
                       uint64_t *alignment, uint64_t *tensor_data_offset);
/* GgufMetadataValueType ids, fusor-ml/gguf/src/lib.rs:349-379 */
enum {
    FH_GGUF_U8 = 0, FH_GGUF_I8 = 1, FH_GGUF_U16 = 2, FH_GGUF_I16 = 3, FH_GGUF_U32 = 4, FH_GGUF_I32 = 5,
    FH_GGUF_F32 = 6, FH_GGUF_BOOL = 7, FH_GGUF_STRING = 8, FH_GGUF_ARRAY = 9, FH_GGUF_U64 = 10,
    FH_GGUF_I64 = 11, FH_GGUF_F64 = 12
};
/* Metadata entries in file order (a repeated key keeps its last value, as the reference's map insert). */
fh_status fh_gguf_meta_key(const fh_gguf *g, uint64_t index, const char **key, uint32_t *value_type);
/* GgufMetadata::get_value, :301-311: a key starting with '.' matches the shortest stored key ending with
 * it (`.attention.head_count` finds `llama.attention.head_count`).  All getters below look keys up this
 * way and return FH_ERR_NOT_FOUND for a missing key, FH_ERR_INVALID for a value of another kind. */
fh_status fh_gguf_meta_find(const fh_gguf *g, const char *key, const char **full_key, uint32_t *value_type);
/* to_u8 .. to_i64 (:544-551): any integer type, converted like Rust's `as`. */
fh_status fh_gguf_meta_int(const fh_gguf *g, const char *key, int64_t *out);
/* to_f32 / to_f64 (:552-553): F32 or F64 only. */
fh_status fh_gguf_meta_float(const fh_gguf *g, const char *key, double *out);
fh_status fh_gguf_meta_bool(const fh_gguf *g, const char *key, int32_t *out);
fh_status fh_gguf_meta_string(const fh_gguf *g, const char *key, const char **bytes, uint64_t *len);
/* to_array (:556): element type and count; `packed` (optional) points at the little-endian elements of
 * an array of fixed-size values and is NULL for arrays of strings or arrays. */
fh_status fh_gguf_meta_array(const fh_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count,
                             const void **packed);
fh_status fh_gguf_meta_array_int(const fh_gguf *g, const char *key, uint64_t index, int64_t *out);
fh_status fh_gguf_meta_array_float(const fh_gguf *g, const char *key, uint64_t index, double *out);
fh_status fh_gguf_meta_array_string(const fh_gguf *g, const char *key, uint64_t index, const char **bytes,
                                    uint64_t *len);
/* GgufTensorMetadata (:254-259): shape in row-major order (outermost first), offset relative to the
 * payload start. */
#define FH_GGUF_MAX_RANK 8
typedef struct {
    const char *name; /* owned by the handle */
    uint32_t ggml_type;
    int32_t rank;
    int64_t shape[FH_GGUF_MAX_RANK];
    uint64_t offset;
} fh_gguf_tensor;
fh_status fh_gguf_tensor_info(const fh_gguf *g, uint64_t index, fh_gguf_tensor *out);
fh_status fh_gguf_tensor_find(const fh_gguf *g, const char *name, uint64_t *index);
/* GgufTensorMetadata::read_tensor_bytes (:262-286): the raw block stream inside the file image. */
fh_status fh_gguf_tensor_data(const fh_gguf *g, uint64_t index, const void **bytes, size_t *len);
/* VarBuilder::get, fusor-ml/fusor/src/varbuilder.rs:79-127: the named tensor as a device weight. */
fh_status fh_qmatrix_from_gguf_tensor(fh_device *dev, const fh_gguf *g, const char *name, fh_qmatrix **out);

/* ----------------------------------------------------------------- decoder
 * Model::forward for the Llama architecture, models/kalosm-llama/src/raw/mod.rs:851-865,
 * :925-1049 (Separate attention variant + Llama feed-forward, interleaved RoPE), with the
 * greedy decode loop of model/inference.rs:11-396 reduced to argmax. */
typedef struct {
    int32_t n_layers, d_model, n_heads, n_kv_heads, head_dim, ffn, vocab, ctx;
    float eps, theta;
    int32_t kv_dtype;       /* FH_F32 (reference) or FH_F16 */
    int32_t fuse_qkv;       /* concat_rows(q, k, v) as raw/mod.rs:511 */
    int32_t fuse_gate_up;   /* concat_rows(gate, up) as raw/attention_layer.rs:96-107 */
    int32_t use_graph;      /* capture one decode step in a hipGraph and replay it */
} fh_llama_config;

fh_status fh_llama_create(fh_device *dev, const fh_llama_config *cfg, fh_llama **out);
fh_status fh_llama_destroy(fh_llama *m);
/* Load one GGUF tensor by its GGUF name (`token_embd.weight`, `blk.N.attn_q.weight`, ...,
 * models/kalosm-llama/src/raw/mod.rs:473-604).  ggml_type 0 (F32) for norm vectors and for
 * `rope_freqs.weight` (head_dim / 2 factors the inverse frequencies are multiplied by,
 * raw/rope.rs:44-48). */
fh_status fh_llama_load_tensor(fh_llama *m, const char *name, uint32_t ggml_type, int64_t n,
                               int64_t k, const void *bytes, size_t len);
/* Fuse/concatenate what the config asks for and allocate the step buffers; call once after loading. */
/* The `rope_scaling` argument of Model::from_gguf (models/kalosm-llama/src/raw/mod.rs:264-285, kept in the
 * LlamaConfig, :120): long-context scaling of the RoPE inverse frequencies (raw/rope.rs:20-38), applied when
 * fh_llama_finalize builds the tables, before the rope_freqs.weight factors.  NULL: none.  Call before finalize. */
fh_status fh_llama_set_rope_scaling(fh_llama *m, const fh_rope_scaling *scaling);
fh_status fh_llama_finalize(fh_llama *m);
fh_status fh_llama_reset(fh_llama *m);
/* Run `count` new tokens at the current position; logits_host (optional, [vocab]) and
 * hidden_host (optional, [d_model], the final-norm hidden state) are of the LAST token.  When the new tokens do not
 * fit the context, the cache is cleared and the last context_length - 32 (at least 8) of all tokens, cached and
 * new, are run again from position 0, as Model::forward does (raw/mod.rs:769-801).  The device-side decode loops
 * below stop at the context length with FH_ERR_INVALID instead. */
fh_status fh_llama_forward(fh_llama *m, const uint32_t *tokens_host, int32_t count,
                           float *logits_host, float *hidden_host);
/* Trace of the last fh_llama_forward, as text lines.  Off by default; fh_set_option keys (or the reference's
 * environment variables, looked up when the device is created, which also send the lines to stderr):
 *   "trace_nan" = 1 (KALOSM_TRACE_LAYER_NAN, models/kalosm-llama/src/raw/mod.rs:955-1041): the embedding and, for
 *     every layer, the normed input, the attention output and the layer output are probed with fh_check_finite; a
 *     tensor with a NaN or an infinity gives one "trace_nan layer=.. label=.. .." line (debug_check_nan_f32, :9-58).
 *   "trace_timing" = 1 (KALOSM_TRACE_FORWARD_TIMING, raw/mod.rs:943-1043): "[timing] text layer loop: .. ms";
 *     = 2 (FUSOR_TRACE_GPU_KERNELS, fusor-ml/core/src/compute_graph/resolve/run.rs:141, :483-497): also one
 *     "[timing] layer L <stage>: .. us" line per stage of every layer, from events on the stream.
 *   "trace_stderr" = 1: the lines go to stderr as well.
 * The device-side decode loops (captured steps) are never traced.  buf receives at most capacity - 1 bytes and a
 * terminating NUL; *length (optional) the full length. */
fh_status fh_llama_trace_text(const fh_llama *m, char *buf, size_t capacity, size_t *length);
/* Greedy decode: feeds `first_token`, then each argmax, for `steps` steps entirely on the device
 * (the sampled id stays resident, as the reference's run-ahead path, model/inference.rs:38-173);
 * out_tokens_host receives the `steps` sampled ids.  elapsed_ms (optional) is the device time. */
fh_status fh_llama_decode_greedy(fh_llama *m, uint32_t first_token, int32_t steps,
                                 uint32_t *out_tokens_host, float *elapsed_ms);
/* Bytes of weights read per decoded token (for roofline reports). */
/* Sampled decode with the token resident on the device (models/kalosm-llama/src/model/inference.rs:38-173): every
 * step samples from the logits as fh_sample_token does and feeds the id to the next step without a host round
 * trip.  randoms_host[steps]: one uniform number per step.  previous_host: the history before first_token (the
 * last repetition_range <= 64 ids count, first_token and the sampled ids are appended as they come).  *mu: the
 * Mirostat state, in and out (ignored by the standard sampler, may be NULL then).  A step without a finite
 * logit stores 0xFFFFFFFF and continues with id 0. */
fh_status fh_llama_decode_sampled(fh_llama *m, uint32_t first_token, int32_t steps, const fh_sampler_params *params,
                                  const float *randoms_host, const uint32_t *previous_host, uint32_t n_previous,
                                  uint32_t repetition_range, float *mu, uint32_t *out_tokens_host, float *elapsed_ms);
fh_status fh_llama_weight_bytes(const fh_llama *m, uint64_t *bytes);
/* Model parameters from GGUF metadata, models/kalosm-llama/src/raw/mod.rs:377-416 (architecture
 * `llama` only; kv_dtype f32, fusions and graph replay switched on: adjust before fh_llama_create,
 * e.g. a smaller ctx than the file's context_length). */
fh_status fh_llama_config_from_gguf(const fh_gguf *g, fh_llama_config *cfg);
/* Load every decoder tensor of the file (raw/mod.rs:418-604: token_embd, output_norm, output,
 * rope_freqs, blk.N.*); f16 vectors are widened to f32.  Call fh_llama_finalize afterwards. */
fh_status fh_llama_load_gguf(fh_llama *m, const fh_gguf *g);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* FUSOR_HIP_H */

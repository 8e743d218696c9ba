// Row and pointwise kernels of the decoder: rms_norm (+residual), RoPE pair, SwiGLU, residual adds,
// head transposes, casts, greedy argmax, KV-cache append.
#include "fh_internal.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

typedef _Float16 fh_half;

__device__ __forceinline__ float block_sum(float v, float *sh) { // blockDim multiple of 64, <= 1024
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += sh[i];
    return t;
}

// ------------------------------------------------------------------------------ rms_norm
// fusor-ml/fusor/src/composite/normalization.rs:404-460 (x^2, sum/len, +eps, sqrt, x/rms, *w, +b),
// residual form :394-397.  One workgroup per row.
__global__ __launch_bounds__(1024) void k_rms_norm(const float *__restrict__ x, const float *__restrict__ res,
                                                    const float *__restrict__ w, const float *__restrict__ bias,
                                                    float eps, int cols, float *__restrict__ y) {
    __shared__ float sh[16];
    const int64_t off = (int64_t)blockIdx.x * cols;
    float acc = 0.f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        float t = x[off + c];
        if (res) t = t + res[off + c];
        acc = fmaf(t, t, acc);
    }
    float total = block_sum(acc, sh);
    float mean = total / (float)cols;
    float rms = sqrtf(mean + eps);
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        float t = x[off + c];
        if (res) t = t + res[off + c];
        float o = (t / rms) * w[c];
        if (bias) o = o + bias[c];
        y[off + c] = o;
    }
}

// Same arithmetic for rows of at most 4096 columns (a multiple of 4): 256 threads keep the row in registers
// (up to four float4 each), so x and the residual are read once.
__global__ __launch_bounds__(256) void k_rms_norm_reg(const float *__restrict__ x, const float *__restrict__ res,
                                                       const float *__restrict__ w, const float *__restrict__ bias,
                                                       float eps, int cols, float *__restrict__ y) {
    __shared__ float sh[16];
    const int64_t off = (int64_t)blockIdx.x * cols;
    const int n4 = cols >> 2;
    float4 v[4];
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c4 = threadIdx.x + i * 256;
        v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c4 < n4) {
            v[i] = *(const float4 *)(x + off + 4 * c4);
            if (res) {
                const float4 r = *(const float4 *)(res + off + 4 * c4);
                v[i].x = v[i].x + r.x; v[i].y = v[i].y + r.y; v[i].z = v[i].z + r.z; v[i].w = v[i].w + r.w;
            }
            acc = fmaf(v[i].x, v[i].x, acc);
            acc = fmaf(v[i].y, v[i].y, acc);
            acc = fmaf(v[i].z, v[i].z, acc);
            acc = fmaf(v[i].w, v[i].w, acc);
        }
    }
    const float total = block_sum(acc, sh);
    const float rms = sqrtf(total / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c4 = threadIdx.x + i * 256;
        if (c4 < n4) {
            const float4 ww = *(const float4 *)(w + 4 * c4);
            float4 o = make_float4((v[i].x / rms) * ww.x, (v[i].y / rms) * ww.y, (v[i].z / rms) * ww.z, (v[i].w / rms) * ww.w);
            if (bias) {
                const float4 bb = *(const float4 *)(bias + 4 * c4);
                o.x = o.x + bb.x; o.y = o.y + bb.y; o.z = o.z + bb.z; o.w = o.w + bb.w;
            }
            *(float4 *)(y + off + 4 * c4) = o;
        }
    }
}

extern "C" fh_status fh_rms_norm(fh_device *dev, const float *x_dev, const float *residual_dev, const float *w_dev,
                                 const float *bias_dev, float eps, int32_t rows, int32_t cols, float *y_dev) {
    FH_REQUIRE(dev && x_dev && w_dev && y_dev, "NULL argument");
    FH_REQUIRE(rows > 0 && cols > 0, "empty input [%d, %d]", rows, cols);
    const bool aligned = (((uintptr_t)x_dev | (uintptr_t)y_dev | (uintptr_t)w_dev | (uintptr_t)residual_dev |
                           (uintptr_t)bias_dev) & 15) == 0;
    if (cols % 4 == 0 && cols <= 4096 && cols >= 256 && aligned) {
        k_rms_norm_reg<<<dim3((unsigned)rows), dim3(256), 0, dev->stream>>>(x_dev, residual_dev, w_dev, bias_dev, eps,
                                                                           cols, y_dev);
    } else {
        int threads = cols >= 4096 ? 1024 : (cols >= 1024 ? 256 : 64);
        k_rms_norm<<<dim3((unsigned)rows), dim3(threads), 0, dev->stream>>>(x_dev, residual_dev, w_dev, bias_dev, eps,
                                                                           cols, y_dev);
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ rope
// Tables: fusor-ml/fusor/src/composite/rope.rs:241-246 + models/kalosm-llama/src/raw/rope.rs:63-85.
// Built on the host in f32 with the C library (the reference builds them with Rust's f32
// powf/sin/cos, i.e. the platform libm).
// create_inverse_frequency, models/kalosm-llama/src/raw/rope.rs:9-50: base frequencies, then the optional
// long-context scaling (frequencies whose wavelength exceeds original_max / low_freq_factor are divided by `factor`;
// the smooth branch is taken only where the wavelength EQUALS original_max / high_freq_factor, as the reference
// writes it at :32), then the optional per-frequency weights of the file.
extern "C" fh_status fh_rope_tables_scaled(fh_device *dev, int32_t head_dim, int32_t ctx, float theta,
                                           const fh_rope_scaling *scaling, const float *freq_weight_host, float *cos_dev,
                                           float *sin_dev) {
    FH_REQUIRE(dev && cos_dev && sin_dev, "NULL argument");
    FH_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && ctx > 0, "bad head_dim %d / ctx %d", head_dim, ctx);
    int half = head_dim / 2;
    std::vector<float> inv(half), c((size_t)ctx * half), s((size_t)ctx * half);
    for (int i = 0; i < head_dim; i += 2) inv[i / 2] = 1.0f / powf(theta, (float)i / (float)head_dim);
    if (scaling) {
        const float orig = (float)scaling->original_max_position_embeddings;
        const float low_wavelen = orig / scaling->low_freq_factor, high_wavelen = orig / scaling->high_freq_factor;
        const float two_pi = 2.0f * 3.14159265358979323846f;
        for (int i = 0; i < half; i++) {
            const float wavelen = two_pi / inv[i];
            if (wavelen > low_wavelen) inv[i] = inv[i] / scaling->factor;
            else if (wavelen == high_wavelen) {
                const float smooth = (orig / wavelen - scaling->low_freq_factor) /
                                     (scaling->high_freq_factor - scaling->low_freq_factor);
                inv[i] = (1.0f - smooth) * inv[i] / scaling->factor + smooth * inv[i];
            }
        }
    }
    if (freq_weight_host)
        for (int i = 0; i < half; i++) inv[i] = inv[i] * freq_weight_host[i];
    for (int p = 0; p < ctx; p++)
        for (int i = 0; i < half; i++) {
            float a = (float)p * inv[i];
            c[(size_t)p * half + i] = cosf(a);
            s[(size_t)p * half + i] = sinf(a);
        }
    FH_TRY(fh_upload(dev, cos_dev, c.data(), c.size() * 4));
    FH_TRY(fh_upload(dev, sin_dev, s.data(), s.size() * 4));
    return FH_OK;
}

extern "C" fh_status fh_rope_tables_weighted(fh_device *dev, int32_t head_dim, int32_t ctx, float theta,
                                             const float *freq_weight_host, float *cos_dev, float *sin_dev) {
    return fh_rope_tables_scaled(dev, head_dim, ctx, theta, nullptr, freq_weight_host, cos_dev, sin_dev);
}

extern "C" fh_status fh_rope_tables(fh_device *dev, int32_t head_dim, int32_t ctx, float theta, float *cos_dev,
                                    float *sin_dev) {
    return fh_rope_tables_weighted(dev, head_dim, ctx, theta, nullptr, cos_dev, sin_dev);
}

// rope.rs:77-108 (interleaved) and :46-68 (half split).  Each product is rounded on its own.
// One thread per rotated pair; q and k share the launch (the reference's fused pair kernel,
// fusor-ml/core/src/composite/rope_fused.rs:31-75).  pos_dev, when not NULL, overrides start_pos.
__global__ __launch_bounds__(256) void k_rope_pair(const float *__restrict__ q, int64_t q_sb, int64_t q_sh, int64_t q_st,
                                                    const float *__restrict__ k, int64_t k_sb, int64_t k_sh, int64_t k_st,
                                                    int b, int hq, int hk, int s, int d, const float *__restrict__ cs,
                                                    const float *__restrict__ sn, int table_rows, int start_pos,
                                                    const int *__restrict__ pos_dev, int interleaved,
                                                    float *__restrict__ qo, float *__restrict__ ko) {
    const int half = d >> 1;
    const int64_t nq = (int64_t)b * hq * s * half, nk = (int64_t)b * hk * s * half;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nq + nk) return;
    const bool isk = idx >= nq;
    if (isk) idx -= nq;
    const int h = isk ? hk : hq;
    int i = (int)(idx % half);
    int64_t r = idx / half;
    int t = (int)(r % s);
    r /= s;
    int hh = (int)(r % h), bb = (int)(r / h);
    const float *src = isk ? k + bb * k_sb + hh * k_sh + t * k_st : q + bb * q_sb + hh * q_sh + t * q_st;
    float *dst = (isk ? ko : qo) + (((int64_t)bb * h + hh) * s + t) * d;
    int pos = (pos_dev ? *pos_dev : start_pos) + t;
    if (pos >= table_rows) pos = table_rows - 1; // host validates; never read outside the table
    const float c = cs[(int64_t)pos * half + i], sv = sn[(int64_t)pos * half + i];
    if (interleaved) {
        float x0 = src[2 * i], x1 = src[2 * i + 1];
        float ac = x0 * c, bs = x1 * sv, as = x0 * sv, bc = x1 * c;
        dst[2 * i] = ac - bs;
        dst[2 * i + 1] = as + bc;
    } else {
        float x0 = src[i], x1 = src[i + half];
        float a0 = x0 * c, r0 = (-x1) * sv, a1 = x1 * c, r1 = x0 * sv;
        dst[i] = a0 + r0;
        dst[i + half] = a1 + r1;
    }
}

extern "C" fh_status fh_rope_pair(fh_device *dev, const float *q_dev, int64_t q_sb, int64_t q_sh, int64_t q_st,
                                  const float *k_dev, int64_t k_sb, int64_t k_sh, int64_t k_st, int32_t b, int32_t hq,
                                  int32_t hk, int32_t s, int32_t d, const float *cos_dev, const float *sin_dev,
                                  int32_t table_rows, int32_t start_pos, int32_t interleaved, float *q_out_dev,
                                  float *k_out_dev) {
    FH_REQUIRE(dev && q_dev && k_dev && cos_dev && sin_dev && q_out_dev && k_out_dev, "NULL argument");
    FH_REQUIRE(b > 0 && hq > 0 && hk > 0 && s > 0 && d > 0 && d % 2 == 0, "bad shape");
    FH_REQUIRE(start_pos >= 0 && start_pos + s <= table_rows, "positions [%d, %d) exceed the %d table rows", start_pos,
               start_pos + s, table_rows);
    int64_t total = ((int64_t)b * hq * s + (int64_t)b * hk * s) * (d / 2);
    k_rope_pair<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream>>>(
        q_dev, q_sb, q_sh, q_st, k_dev, k_sb, k_sh, k_st, b, hq, hk, s, d, cos_dev, sin_dev, table_rows, start_pos,
        nullptr, interleaved, q_out_dev, k_out_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_rope_pair_devpos(fh_device *dev, const float *q, const float *k, int hq, int hk, int d, const float *cos_t,
                              const float *sin_t, int table_rows, const int *pos_dev, float *q_out, float *k_out) {
    int64_t total = (int64_t)(hq + hk) * (d / 2);
    k_rope_pair<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream>>>(
        q, 0, d, 0, k, 0, d, 0, 1, hq, hk, 1, d, cos_t, sin_t, table_rows, 0, pos_dev, 1, q_out, k_out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ pointwise
// silu(x) = x / (exp(-x) + 1), fusor-ml/fusor/src/composite/activations.rs:47-65
__global__ void k_swiglu(const float *__restrict__ g, const float *__restrict__ u, float *__restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float x = g[i];
        y[i] = (x / (expf(-x) + 1.0f)) * u[i];
    }
}
// gu is [rows, 2f]: gate | up per row; y is [rows, f]
__global__ void k_swiglu_rows(const float *__restrict__ gu, int rows, int f, float *__restrict__ y) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)rows * f) return;
    int64_t r = i / f, c = i % f;
    float x = gu[r * 2 * f + c];
    y[i] = (x / (expf(-x) + 1.0f)) * gu[r * 2 * f + f + c];
}
__global__ void k_add3(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ c,
                       float *__restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float t = a[i] + b[i];
        y[i] = c ? t + c[i] : t;
    }
}
__global__ void k_transpose_shd(const float *__restrict__ x, int s, int h, int d, float *__restrict__ y) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t n = (int64_t)s * h * d;
    if (i >= n) return;
    int c = (int)(i % d);
    int64_t r = i / d;
    int hh = (int)(r % h), t = (int)(r / h); // input index (t, hh, c)
    y[((int64_t)hh * s + t) * d + c] = x[i];
}
__global__ void k_f32_f16(const float *__restrict__ x, fh_half *__restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = (fh_half)x[i];
}
__global__ void k_f16_f32(const fh_half *__restrict__ x, float *__restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = (float)x[i];
}
__global__ void k_f32_bf16(const float *__restrict__ x, uint16_t *__restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        uint32_t u = __float_as_uint(x[i]);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) y[i] = (uint16_t)((u >> 16) | 0x40); // quiet NaN
        else y[i] = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);            // round to nearest even
    }
}

#define FH_GRID1D(n) dim3((unsigned)(((n) + 255) / 256)), dim3(256), 0, dev->stream
#define FH_CHECK_COUNT(n) FH_REQUIRE((n) > 0 && ((n) + 255) / 256 < (1ll << 31), "count %lld out of range", (long long)(n))

extern "C" fh_status fh_swiglu(fh_device *dev, const float *gate_dev, const float *up_dev, float *y_dev, int64_t count) {
    FH_REQUIRE(dev && gate_dev && up_dev && y_dev, "NULL argument");
    FH_CHECK_COUNT(count);
    k_swiglu<<<FH_GRID1D(count)>>>(gate_dev, up_dev, y_dev, count);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
fh_status fh_swiglu_rows(fh_device *dev, const float *gu, int rows, int f, float *y) {
    int64_t count = (int64_t)rows * f;
    k_swiglu_rows<<<FH_GRID1D(count)>>>(gu, rows, f, y);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
extern "C" fh_status fh_add3(fh_device *dev, const float *a_dev, const float *b_dev, const float *c_dev, float *y_dev,
                             int64_t count) {
    FH_REQUIRE(dev && a_dev && b_dev && y_dev, "NULL argument");
    FH_CHECK_COUNT(count);
    k_add3<<<FH_GRID1D(count)>>>(a_dev, b_dev, c_dev, y_dev, count);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
extern "C" fh_status fh_transpose_shd(fh_device *dev, const float *x_dev, int32_t s, int32_t h, int32_t d, float *y_dev) {
    FH_REQUIRE(dev && x_dev && y_dev, "NULL argument");
    int64_t count = (int64_t)s * h * d;
    FH_CHECK_COUNT(count);
    k_transpose_shd<<<FH_GRID1D(count)>>>(x_dev, s, h, d, y_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
extern "C" fh_status fh_cast_f32_f16(fh_device *dev, const float *x_dev, void *y_f16_dev, int64_t count) {
    FH_REQUIRE(dev && x_dev && y_f16_dev, "NULL argument");
    FH_CHECK_COUNT(count);
    k_f32_f16<<<FH_GRID1D(count)>>>(x_dev, (fh_half *)y_f16_dev, count);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
extern "C" fh_status fh_cast_f16_f32(fh_device *dev, const void *x_f16_dev, float *y_dev, int64_t count) {
    FH_REQUIRE(dev && x_f16_dev && y_dev, "NULL argument");
    FH_CHECK_COUNT(count);
    k_f16_f32<<<FH_GRID1D(count)>>>((const fh_half *)x_f16_dev, y_dev, count);
    FH_HIP(hipGetLastError());
    return FH_OK;
}
extern "C" fh_status fh_cast_f32_bf16(fh_device *dev, const float *x_dev, void *y_bf16_dev, int64_t count) {
    FH_REQUIRE(dev && x_dev && y_bf16_dev, "NULL argument");
    FH_CHECK_COUNT(count);
    k_f32_bf16<<<FH_GRID1D(count)>>>(x_dev, (uint16_t *)y_bf16_dev, count);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ argmax
// fusor-ml/fusor/src/lib.rs:416-447 with k = 1: largest finite value, ties to the larger index.
// Single workgroup; the logits row (vocab x 4 B) is small next to the lm-head weights.
__device__ __forceinline__ void amax_merge(float &v, uint32_t &id, float ov, uint32_t oid) {
    if (oid == 0xFFFFFFFFu) return;
    if (id == 0xFFFFFFFFu || ov > v || (ov == v && oid > id)) {
        v = ov;
        id = oid;
    }
}
// Stage 1 (pv != NULL): workgroup b scans its slice of x and writes its best (value, id) to pv/pi[b].
// Stage 2 (pv == NULL in the launch of one workgroup): x is the partial values, xi their ids.
// The last stage can also finish a decode step (tail.ids != NULL): the id becomes the next step's input (0 when
// no logit was finite), is appended to the step's output list, and the KV cache's device-side length goes up by one.
__global__ __launch_bounds__(1024) void k_argmax(const float *__restrict__ x, const uint32_t *__restrict__ xi, int64_t n,
                                                  uint32_t *__restrict__ out, float *__restrict__ pv,
                                                  uint32_t *__restrict__ pi, FhStepTail tail) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    float v = 0.f;
    uint32_t id = 0xFFFFFFFFu;
    const int64_t per = (n + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * per, hi = lo + per < n ? lo + per : n;
    for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        float t = x[i];
        uint32_t tid_ = xi ? xi[i] : (uint32_t)i;
        if (isfinite(t) && tid_ != 0xFFFFFFFFu) amax_merge(v, id, t, tid_);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(v, o, 64);
        uint32_t oid = (uint32_t)__shfl_xor((int)id, o, 64);
        amax_merge(v, id, ov, oid);
    }
    int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        sv[w] = v;
        si[w] = id;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < (int)(blockDim.x >> 6); i++) amax_merge(v, id, sv[i], si[i]);
        if (pv) {
            pv[blockIdx.x] = v;
            pi[blockIdx.x] = id;
        } else {
            *out = id;
            if (tail.ids) {
                tail.ids[0] = id == 0xFFFFFFFFu ? 0u : id;
                tail.out_tokens[*tail.step] = id;
                *tail.step = *tail.step + 1;
                *tail.kv_len = *tail.kv_len + 1;
            }
        }
    }
}
extern "C" fh_status fh_argmax(fh_device *dev, const float *x_dev, int64_t count, uint32_t *id_dev) {
    return fh_argmax_step(dev, x_dev, count, id_dev, FhStepTail{});
}
fh_status fh_argmax_step(fh_device *dev, const float *x_dev, int64_t count, uint32_t *id_dev, FhStepTail tail) {
    FH_REQUIRE(dev && x_dev && id_dev, "NULL argument");
    FH_REQUIRE(count > 0 && count < 0xFFFFFFFFll, "count %lld out of range", (long long)count);
    if (count <= 8192) {
        k_argmax<<<dim3(1), dim3(1024), 0, dev->stream>>>(x_dev, nullptr, count, id_dev, nullptr, nullptr, tail);
    } else {
        const int parts = 128;
        float *pv = (float *)dev->small_buf;
        uint32_t *pi = (uint32_t *)(pv + parts);
        k_argmax<<<dim3(parts), dim3(256), 0, dev->stream>>>(x_dev, nullptr, count, nullptr, pv, pi, FhStepTail{});
        k_argmax<<<dim3(1), dim3(128), 0, dev->stream>>>(pv, pi, parts, id_dev, nullptr, nullptr, tail);
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ top-k
// Tensor::top_k_pairs(k), fusor-ml/fusor/src/lib.rs:416-447: the k largest FINITE logits in descending order, ties
// to the larger token id.  (value, id) becomes one 64-bit key whose unsigned order is that order (-0.0 ranks with
// +0.0, as the reference's float compare does); every workgroup sorts 1024 keys (bitonic, descending, two keys per
// thread) and keeps its first k; passes repeat over the survivors until one workgroup is left.
__device__ __forceinline__ uint64_t topk_key(float v, uint32_t id) {
    uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return 0; // infinities and NaNs are skipped
    if (b == 0x80000000u) b = 0;
    const uint32_t o = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((uint64_t)o << 32) | id;
}

__device__ __forceinline__ float topk_value(uint64_t key) {
    const uint32_t o = (uint32_t)(key >> 32);
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o);
}

// Logit processors of the sampling front end (fusor-ml/core/src/sampling/row_kernels.rs:150-205; the host form is
// process_logit, models/kalosm-llama/src/sampler.rs:275-307): a finite logit whose id is among the previous tokens is
// multiplied (<= 0) or divided (> 0) by a repetition penalty above 1, then every logit is divided by a non-zero
// temperature; what is not finite before or after is skipped.  `prev` holds up to 64 ids in device memory (membership
// only, so the order of the slots does not matter), its length is *prev_len when that pointer is given.
struct TopkProc {
    int on;
    float temperature, penalty;
    const uint32_t *prev;
    const uint32_t *prev_len;
    uint32_t n_prev;
};

// Sampler that ends the last pass (row_kernels.rs:484-660 helpers, :672-797 Mirostat 2, :799-919 standard):
// weights exp(value - max) of the sorted candidates, a cutoff, then the first candidate whose running weight reaches
// random * (sum of the weights before the cutoff).  result = [status, token]: 1 sampled, 2 no finite logit.
struct TopkSample {
    int on;
    uint32_t kind;
    float top_p, min_p, tau, eta, random;
    const float *randoms; // device; entry *step (entry 0 without `step`) replaces `random`
    const int *step;
    float *mu;            // Mirostat state, device
    uint32_t *result;
};

__device__ void topk_sample(const uint64_t *s, float *w, int k, const TopkSample &a) {
    // called by thread 0 after w[i] = exp(value_i - value_0) (0 for a missing candidate) is in LDS
    const float eps = 1.0e-20f;
    if (!s[0]) {
        a.result[0] = 2u;
        a.result[1] = 0u;
        return;
    }
    const float random = a.randoms ? a.randoms[a.step ? *a.step : 0] : a.random;
    int cutoff = k;
    float cutoff_sum = 0.f, mu = 0.f;
    if (a.kind == 1u) {
        float total = 0.f;
        for (int i = 0; i < k; i++) total += w[i];
        total = fmaxf(total, eps);
        mu = *a.mu;
        for (int i = 0; i < k; i++) {
            const float p = fmaxf(w[i] / total, eps);
            if (-log2f(p) > mu) {
                cutoff = i > 1 ? i : 1;
                break;
            }
        }
        for (int i = 0; i < cutoff; i++) cutoff_sum += w[i];
    } else {
        float filtered = 0.f;
        for (int i = 0; i < k; i++)
            if (w[i] >= a.min_p) filtered += w[i];
        const float target = __fmul_rn(fmaxf(filtered, eps), a.top_p);
        for (int i = 0; i < k; i++) {
            if (w[i] >= a.min_p) {
                cutoff_sum += w[i];
                if (cutoff_sum >= target) {
                    cutoff = i + 1;
                    break;
                }
            } else {
                cutoff = i;
                break;
            }
        }
        if (cutoff == 0) {
            cutoff = 1;
            cutoff_sum = w[0];
        }
    }
    cutoff_sum = fmaxf(cutoff_sum, eps);
    const float threshold = __fmul_rn(random, cutoff_sum);
    uint32_t token = (uint32_t)s[0];
    float prob = w[0] / cutoff_sum, cum = 0.f;
    for (int i = 0; i < cutoff; i++) {
        cum += w[i];
        if (cum >= threshold) {
            token = s[i] ? (uint32_t)s[i] : 0xFFFFFFFFu;
            prob = w[i] / cutoff_sum;
            break;
        }
    }
    if (a.kind == 1u) {
        const float surprise = -log2f(fmaxf(prob, eps));
        *a.mu = __fsub_rn(mu, __fmul_rn(a.eta, __fsub_rn(surprise, a.tau)));
    }
    a.result[0] = 1u;
    a.result[1] = token;
}

template <bool FIRST>
__global__ __launch_bounds__(512) void k_topk_pass(const float *__restrict__ x, const uint64_t *__restrict__ keys_in,
                                                   int64_t n_in, int k, int last, uint64_t *__restrict__ keys_out,
                                                   uint32_t *__restrict__ ids_out, float *__restrict__ vals_out,
                                                   uint32_t *__restrict__ found_out, TopkProc proc, TopkSample samp) {
    __shared__ uint64_t s[2048];
    __shared__ uint32_t s_prev[64];
    __shared__ float s_w[256];
    const int tid = threadIdx.x;
    const int64_t base = (int64_t)blockIdx.x * 1024;
    uint32_t n_prev = 0;
    if (FIRST && proc.on && proc.penalty > 1.0f) {
        n_prev = proc.prev_len ? *proc.prev_len : proc.n_prev;
        n_prev = n_prev < 64u ? n_prev : 64u;
        if (tid < 64) s_prev[tid] = (uint32_t)tid < n_prev ? proc.prev[tid] : 0u;
        __syncthreads();
    }
    // Thread t holds the keys at positions 2t and 2t + 1 of the bitonic network (which input lands where does not
    // matter): partners at distance 1 are in its own registers, up to distance 64 in its wavefront (lane exchange),
    // beyond that in another wavefront (through LDS, two buffers in turn so that one barrier per stage is enough).
    uint64_t kk[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int64_t idx = base + tid + 512 * h;
        uint64_t key = 0ull;
        if (idx < n_in) {
            if (FIRST) {
                float v = x[idx];
                if (proc.on && (__float_as_uint(v) & 0x7F800000u) != 0x7F800000u) {
                    bool repeated = false;
                    for (uint32_t j = 0; j < n_prev; j++) repeated |= s_prev[j] == (uint32_t)idx;
                    if (repeated) v = v <= 0.0f ? __fmul_rn(v, proc.penalty) : __fdiv_rn(v, proc.penalty);
                    if (proc.temperature != 0.0f) v = __fdiv_rn(v, proc.temperature);
                }
                key = topk_key(v, (uint32_t)idx);
            } else {
                key = keys_in[idx];
            }
        }
        kk[h] = key;
    }
    int flip = 0;
#pragma unroll
    for (int size = 2; size <= 1024; size <<= 1) {
        const bool down = ((2 * tid) & size) == 0; // this run is sorted descending
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (stride == 1) {
                if ((kk[0] < kk[1]) == down) {
                    const uint64_t t = kk[0];
                    kk[0] = kk[1];
                    kk[1] = t;
                }
                continue;
            }
            const int m = stride >> 1; // distance in threads
            uint64_t o[2];
            if (stride <= 64) {
                o[0] = __shfl_xor(kk[0], m);
                o[1] = __shfl_xor(kk[1], m);
            } else {
                uint64_t *buf = s + 1024 * flip;
                flip ^= 1;
                buf[2 * tid] = kk[0];
                buf[2 * tid + 1] = kk[1];
                __syncthreads();
                o[0] = buf[2 * (tid ^ m)];
                o[1] = buf[2 * (tid ^ m) + 1];
            }
            const bool keep_max = ((tid & m) == 0) == down;
#pragma unroll
            for (int h = 0; h < 2; h++) kk[h] = keep_max ? (kk[h] > o[h] ? kk[h] : o[h]) : (kk[h] < o[h] ? kk[h] : o[h]);
        }
    }
    __syncthreads();
    s[2 * tid] = kk[0];
    s[2 * tid + 1] = kk[1];
    __syncthreads();
    if (!last) {
        for (int i = tid; i < k; i += 512) keys_out[(int64_t)blockIdx.x * k + i] = s[i];
        return;
    }
    if (ids_out)
        for (int i = tid; i < k; i += 512) {
            const uint64_t key = s[i];
            ids_out[i] = key ? (uint32_t)key : 0xFFFFFFFFu;
            // the processed value is the one the key carries; the plain top-k returns the stored logit (-0.0 kept)
            vals_out[i] = key ? (proc.on ? topk_value(key) : x[(uint32_t)key]) : __uint_as_float(0x7FC00000u);
        }
    if (tid == 0 && found_out) {
        int c = 0;
        while (c < k && s[c]) c++;
        *found_out = (uint32_t)c;
    }
    if (samp.on) {
        if (tid < k) s_w[tid] = s[tid] ? expf(topk_value(s[tid]) - topk_value(s[0])) : 0.f;
        __syncthreads();
        if (tid == 0) topk_sample(s, s_w, k, samp);
    }
}

static fh_status topk_run(fh_device *dev, const float *x_dev, int64_t count, int32_t k, uint32_t *ids_dev,
                          float *values_dev, uint32_t *found_dev, const TopkProc &proc, const TopkSample &samp) {
    int64_t n = count, blocks = (n + 1023) / 1024;
    uint64_t *buf[2] = {nullptr, nullptr};
    if (blocks > 1) {
        const size_t half = ((size_t)blocks * k * 8 + 255) & ~(size_t)255;
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, 2 * half));
        buf[0] = (uint64_t *)dev->ksplit_buf;
        buf[1] = (uint64_t *)((uint8_t *)dev->ksplit_buf + half);
    }
    const uint64_t *in = nullptr;
    bool first = true;
    int turn = 0;
    for (;;) {
        const int last = blocks == 1;
        if (first)
            k_topk_pass<true><<<dim3((unsigned)blocks), dim3(512), 0, dev->stream>>>(
                x_dev, nullptr, n, k, last, buf[turn], ids_dev, values_dev, found_dev, proc, samp);
        else
            k_topk_pass<false><<<dim3((unsigned)blocks), dim3(512), 0, dev->stream>>>(
                x_dev, in, n, k, last, buf[turn], ids_dev, values_dev, found_dev, proc, samp);
        FH_HIP(hipGetLastError());
        if (last) break;
        in = buf[turn];
        turn ^= 1;
        n = blocks * k;
        blocks = (n + 1023) / 1024;
        first = false;
    }
    return FH_OK;
}

extern "C" fh_status fh_top_k(fh_device *dev, const float *x_dev, int64_t count, int32_t k, uint32_t *ids_dev,
                              float *values_dev, uint32_t *found_dev) {
    FH_REQUIRE(dev && x_dev && ids_dev && values_dev, "NULL argument");
    FH_REQUIRE(count > 0 && count < 0xFFFFFFFFll, "count %lld out of range", (long long)count);
    FH_REQUIRE(k >= 1 && k <= 256, "k = %d out of range (1 .. 256)", k);
    TopkProc proc = {};
    TopkSample samp = {};
    return topk_run(dev, x_dev, count, k, ids_dev, values_dev, found_dev, proc, samp);
}

// Device-side form used by the decoder's sampled decode loop: previous tokens, their count, the random numbers and
// the step index all live in device memory, so the same launches can be replayed as a graph.
fh_status fh_sample_token_dev(fh_device *dev, const float *logits_dev, int64_t count, const fh_sampler_params *p,
                              const uint32_t *prev_dev, const uint32_t *prev_len_dev, uint32_t n_prev,
                              const float *randoms_dev, const int *step_dev, float *mu_dev, uint32_t *result_dev,
                              uint32_t *ids_dev, float *values_dev) {
    FH_REQUIRE(p->kind == FH_SAMPLER_STANDARD || p->kind == FH_SAMPLER_MIROSTAT2, "sampler kind %u unknown", p->kind);
    FH_REQUIRE(p->top_k >= 1 && p->top_k <= 256, "top_k = %u out of range (1 .. 256)", p->top_k);
    FH_REQUIRE(p->kind != FH_SAMPLER_MIROSTAT2 || mu_dev, "Mirostat 2 needs its state");
    FH_REQUIRE((ids_dev == nullptr) == (values_dev == nullptr), "ids and values go together");
    TopkProc proc = {1, p->temperature, p->repetition_penalty, prev_dev, prev_len_dev, n_prev};
    TopkSample samp = {1, p->kind, p->top_p, p->min_p, p->tau, p->eta, p->random, randoms_dev, step_dev, mu_dev, result_dev};
    return topk_run(dev, logits_dev, count, (int32_t)p->top_k, ids_dev, values_dev, nullptr, proc, samp);
}

extern "C" fh_status fh_sample_token(fh_device *dev, const float *logits_dev, int64_t count, const fh_sampler_params *params,
                                     const uint32_t *previous_host, uint32_t n_previous, const uint32_t *previous_tail_dev,
                                     float *mu_dev, uint32_t *result_dev, uint32_t *ids_dev, float *values_dev) {
    FH_REQUIRE(dev && logits_dev && params && result_dev, "NULL argument");
    FH_REQUIRE(count > 0 && count < 0xFFFFFFFFll, "count %lld out of range", (long long)count);
    FH_REQUIRE(n_previous == 0 || previous_host, "previous tokens missing");
    // fixed_previous_tokens_data{,_with_gpu_tail}, fusor-ml/core/src/sampling/processors.rs:20-81: the last 64 ids,
    // or the last 63 followed by the id another kernel left in device memory.
    const uint32_t room = previous_tail_dev ? 63u : 64u;
    const uint32_t keep = n_previous < room ? n_previous : room;
    uint32_t *prev = (uint32_t *)((uint8_t *)dev->small_buf + 60 * 1024); // the last 4 KB of the 64 KB buffer: no other user
    if (keep) FH_TRY(fh_upload(dev, prev, previous_host + (n_previous - keep), (size_t)keep * 4));
    if (previous_tail_dev)
        FH_HIP(hipMemcpyAsync(prev + keep, previous_tail_dev, 4, hipMemcpyDeviceToDevice, dev->stream));
    return fh_sample_token_dev(dev, logits_dev, count, params, prev, nullptr, keep + (previous_tail_dev ? 1u : 0u), nullptr,
                               nullptr, mu_dev, result_dev, ids_dev, values_dev);
}

// ------------------------------------------------------------------------------ KV cache
// fusor-ml/fusor/src/cache/tensor_cache.rs:70-114 (in-place slice write into a grown backing buffer),
// :304-312 (power-of-two growth, minimum 256, capped at max_len).
static int kv_alloc_len(int required, int max_len) {
    int min_alloc = 256 < max_len ? 256 : max_len;
    int p = 1;
    while (p < required) p <<= 1;
    if (p < min_alloc) p = min_alloc;
    if (p > max_len) p = max_len;
    return p;
}

extern "C" fh_status fh_kvcache_create(fh_device *dev, int32_t layers, int32_t kv_heads, int32_t head_dim,
                                       int32_t max_len, int32_t dtype, fh_kvcache **out) {
    FH_REQUIRE(dev && out, "NULL argument");
    FH_REQUIRE(layers > 0 && kv_heads > 0 && head_dim > 0 && max_len > 0, "bad cache shape");
    FH_REQUIRE(dtype == FH_F32 || dtype == FH_F16, "cache dtype must be FH_F32 or FH_F16");
    fh_kvcache *c = new fh_kvcache();
    c->dev = dev;
    c->layers = layers;
    c->kv_heads = kv_heads;
    c->head_dim = head_dim;
    c->max_len = max_len;
    c->dtype = dtype;
    hipError_t e = hipMalloc((void **)&c->len_dev, 256);
    if (e != hipSuccess) {
        delete c;
        FH_FAIL(FH_ERR_OOM, "hipMalloc failed: %s", hipGetErrorString(e));
    }
    int zero = 0;
    (void)hipMemcpy(c->len_dev, &zero, 4, hipMemcpyHostToDevice);
    *out = c;
    return FH_OK;
}

extern "C" fh_status fh_kvcache_destroy(fh_kvcache *c) {
    if (!c) return FH_OK;
    (void)hipStreamSynchronize(c->dev->stream);
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    if (c->len_dev) (void)hipFree(c->len_dev);
    delete c;
    return FH_OK;
}

__global__ void k_set_int(int *p, int v) { *p = v; }

extern "C" fh_status fh_kvcache_reset(fh_kvcache *c) {
    FH_REQUIRE(c, "NULL argument");
    c->len = 0; // the reference drops its buffers (tensor_cache.rs:60-65); capacity is kept here
    k_set_int<<<1, 1, 0, c->dev->stream>>>(c->len_dev, 0);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// copy [layers][heads][old_cap][d] -> [layers][heads][new_cap][d] for the first `len` positions
__global__ void k_kv_regrow(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t rows, int len,
                            int old_cap, int new_cap, int words_per_pos) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t per_row = (int64_t)len * words_per_pos;
    if (i >= rows * per_row) return;
    int64_t r = i / per_row, o = i % per_row;
    dst[r * new_cap * words_per_pos + o] = src[r * old_cap * words_per_pos + o];
}

fh_status fh_kvcache_reserve(fh_kvcache *c, int required) {
    FH_REQUIRE(required <= c->max_len, "KV cache overflow: %d positions needed, max_len %d", required, c->max_len);
    if (required <= c->capacity) return FH_OK;
    int cap = kv_alloc_len(required, c->max_len);
    size_t es = fh_dtype_size(c->dtype);
    size_t bytes = (size_t)c->layers * c->kv_heads * cap * c->head_dim * es;
    void *nk = nullptr, *nv = nullptr;
    FH_HIP(hipMalloc(&nk, bytes));
    hipError_t e = hipMalloc(&nv, bytes);
    if (e != hipSuccess) {
        (void)hipFree(nk);
        FH_FAIL(FH_ERR_OOM, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    hipStream_t s = c->dev->stream;
    // New cache memory starts as NaN bit patterns (f32 and f16 alike): a kernel that lets a row past the live length
    // reach its result then fails in every run, not only when the allocation happens to hold such bytes.
    FH_HIP(hipMemsetAsync(nk, 0xFF, bytes, s));
    FH_HIP(hipMemsetAsync(nv, 0xFF, bytes, s));
    if (c->len > 0 && c->k) {
        int wpp = (int)(c->head_dim * es / 4);
        int64_t rows = (int64_t)c->layers * c->kv_heads, total = rows * c->len * wpp;
        dim3 grid((unsigned)((total + 255) / 256));
        k_kv_regrow<<<grid, 256, 0, s>>>((const uint32_t *)c->k, (uint32_t *)nk, rows, c->len, c->capacity, cap, wpp);
        k_kv_regrow<<<grid, 256, 0, s>>>((const uint32_t *)c->v, (uint32_t *)nv, rows, c->len, c->capacity, cap, wpp);
    }
    FH_HIP(hipStreamSynchronize(s));
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    c->k = nk;
    c->v = nv;
    c->capacity = cap;
    return FH_OK;
}

// k_src / v_src: [heads, s, d] f32 views, each with its own head and position stride (elements).
// The write position comes from pos_dev when given (graph replay), else from p0.
template <typename TO>
__global__ void k_kv_append(const float *__restrict__ ks, int64_t k_sh, int64_t k_st, const float *__restrict__ vs,
                            int64_t v_sh, int64_t v_st, int heads, int s, int d, TO *__restrict__ kc,
                            TO *__restrict__ vc, int cap, int p0, const int *__restrict__ pos_dev) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t n = (int64_t)heads * s * d;
    if (i >= n) return;
    int c = (int)(i % d);
    int64_t r = i / d;
    int t = (int)(r % s), h = (int)(r / s);
    int pos = (pos_dev ? *pos_dev : p0) + t;
    if (pos >= cap) return; // the host guarantees capacity; never write outside the plane
    int64_t dofs = ((int64_t)h * cap + pos) * d + c;
    kc[dofs] = (TO)ks[h * k_sh + t * k_st + c];
    vc[dofs] = (TO)vs[h * v_sh + t * v_st + c];
}

static fh_status kv_append_launch(fh_kvcache *c, int layer, const float *k, int64_t k_sh, int64_t k_st, const float *v,
                                  int64_t v_sh, int64_t v_st, int s, int p0, const int *pos_dev) {
    size_t plane = (size_t)c->kv_heads * c->capacity * c->head_dim;
    int64_t n = (int64_t)c->kv_heads * s * c->head_dim;
    dim3 grid((unsigned)((n + 255) / 256));
    hipStream_t stream = c->dev->stream;
    if (c->dtype == FH_F32)
        k_kv_append<float><<<grid, 256, 0, stream>>>(k, k_sh, k_st, v, v_sh, v_st, c->kv_heads, s, c->head_dim,
                                                     (float *)c->k + layer * plane, (float *)c->v + layer * plane,
                                                     c->capacity, p0, pos_dev);
    else
        k_kv_append<fh_half><<<grid, 256, 0, stream>>>(k, k_sh, k_st, v, v_sh, v_st, c->kv_heads, s, c->head_dim,
                                                       (fh_half *)c->k + layer * plane, (fh_half *)c->v + layer * plane,
                                                       c->capacity, p0, pos_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// Append with separate K / V strides at an explicit position; capacity must already be reserved.
fh_status fh_kvcache_append_kv(fh_kvcache *c, int layer, const float *k, int64_t k_sh, int64_t k_st, const float *v,
                               int64_t v_sh, int64_t v_st, int s, int pos) {
    FH_REQUIRE(pos + s <= c->capacity, "KV append [%d, %d) beyond the reserved capacity %d", pos, pos + s, c->capacity);
    return kv_append_launch(c, layer, k, k_sh, k_st, v, v_sh, v_st, s, pos, nullptr);
}

fh_status fh_kvcache_set_len_dev(fh_kvcache *c, int len) {
    k_set_int<<<1, 1, 0, c->dev->stream>>>(c->len_dev, len);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_kvcache_set_sliding(fh_kvcache *c, int32_t on) {
    FH_REQUIRE(c, "NULL argument");
    c->sliding = on != 0;
    return FH_OK;
}

extern "C" fh_status fh_kvcache_append(fh_kvcache *c, int32_t layer, const float *k_dev, const float *v_dev, int64_t sh,
                                       int64_t st, int32_t s) {
    FH_REQUIRE(c && k_dev && v_dev, "NULL argument");
    FH_REQUIRE(layer >= 0 && layer < c->layers && s > 0, "bad layer %d / s %d", layer, s);
    if (c->sliding && c->len + s > c->max_len) {
        // TensorCache::append_gpu_evict, fusor-ml/fusor/src/cache/tensor_cache.rs:175-202: the cache becomes the
        // last max_len positions of [cached | new]
        const int max = c->max_len, evict = c->len + s - max;
        const int keep = c->len > evict ? c->len - evict : 0; // cached rows that survive, moved to the front
        const int skip = s > max ? s - max : 0;               // new rows that fall out at once
        FH_TRY(fh_kvcache_reserve(c, max));
        if (keep > 0) {
            const size_t es = fh_dtype_size(c->dtype), row = (size_t)c->head_dim * es;
            const size_t pitch = (size_t)c->capacity * row, width = (size_t)keep * row;
            const size_t plane = (size_t)c->kv_heads * pitch;
            FH_TRY(fh_dev_scratch(c->dev, &c->dev->act_buf, &c->dev->act_cap, (size_t)c->kv_heads * width));
            for (void *base : {c->k, c->v}) { // through a scratch copy: the ranges overlap
                uint8_t *lp = (uint8_t *)base + (size_t)layer * plane;
                FH_HIP(hipMemcpy2DAsync(c->dev->act_buf, width, lp + (size_t)evict * row, pitch, width, c->kv_heads,
                                        hipMemcpyDeviceToDevice, c->dev->stream));
                FH_HIP(hipMemcpy2DAsync(lp, pitch, c->dev->act_buf, width, width, c->kv_heads, hipMemcpyDeviceToDevice,
                                        c->dev->stream));
            }
        }
        FH_TRY(kv_append_launch(c, layer, k_dev + (int64_t)skip * st, sh, st, v_dev + (int64_t)skip * st, sh, st, s - skip,
                                keep, nullptr));
        if (layer == c->layers - 1) {
            c->len = max;
            k_set_int<<<1, 1, 0, c->dev->stream>>>(c->len_dev, c->len);
            FH_HIP(hipGetLastError());
        }
        return FH_OK;
    }
    FH_TRY(fh_kvcache_reserve(c, c->len + s));
    FH_TRY(kv_append_launch(c, layer, k_dev, sh, st, v_dev, sh, st, s, c->len, nullptr));
    if (layer == c->layers - 1) {
        c->len += s;
        k_set_int<<<1, 1, 0, c->dev->stream>>>(c->len_dev, c->len);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

// Graph-replayed decode step: position read from len_dev; the host mirrors the length afterwards.
fh_status fh_kvcache_append_devpos(fh_kvcache *c, int layer, const float *k, const float *v, int64_t sh) {
    return kv_append_launch(c, layer, k, sh, 0, v, sh, 0, 1, 0, c->len_dev);
}

// One-token decode step: interleaved RoPE of q and k at position *pos_dev, the rotated k and the raw v written
// straight into the cache row (RopeCache::forward_interleaved + KvCache::append in one launch).
// q, k, v are [heads, d] with head stride d.
template <typename TO>
__global__ __launch_bounds__(256) void k_rope_kv_decode(const float *__restrict__ q, const float *__restrict__ k,
                                                         const float *__restrict__ v, int hq, int hk, int d,
                                                         const float *__restrict__ cs, const float *__restrict__ sn,
                                                         int table_rows, const int *__restrict__ pos_dev,
                                                         float *__restrict__ qo, TO *__restrict__ kc,
                                                         TO *__restrict__ vc, int cap) {
    const int half = d >> 1;
    const int npair = (hq + hk) * half, nv = hk * d;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= npair + nv) return;
    int pos = *pos_dev;
    if (pos >= cap) return; // the host reserves capacity before the step
    if (idx < npair) {
        const int i = idx % half, h = idx / half;
        const int tp = pos < table_rows ? pos : table_rows - 1;
        const float c = cs[(int64_t)tp * half + i], s = sn[(int64_t)tp * half + i];
        const bool isk = h >= hq;
        const float *src = isk ? k + (h - hq) * d : q + h * d;
        const float x0 = src[2 * i], x1 = src[2 * i + 1];
        const float ac = x0 * c, bs = x1 * s, as = x0 * s, bc = x1 * c;
        const float y0 = ac - bs, y1 = as + bc;
        if (isk) {
            TO *dst = kc + ((int64_t)(h - hq) * cap + pos) * d;
            dst[2 * i] = (TO)y0;
            dst[2 * i + 1] = (TO)y1;
        } else {
            qo[h * d + 2 * i] = y0;
            qo[h * d + 2 * i + 1] = y1;
        }
    } else {
        const int e = idx - npair, h = e / d, c = e % d;
        vc[((int64_t)h * cap + pos) * d + c] = (TO)v[h * d + c];
    }
}

fh_status fh_rope_kv_decode(fh_kvcache *c, int layer, const float *q, const float *k, const float *v, int hq,
                            const float *cos_t, const float *sin_t, int table_rows, float *q_out) {
    const int hk = c->kv_heads, d = c->head_dim;
    const size_t plane = (size_t)hk * c->capacity * d;
    const int total = (hq + hk) * (d / 2) + hk * d;
    dim3 grid((unsigned)((total + 255) / 256));
    hipStream_t s = c->dev->stream;
    if (c->dtype == FH_F32)
        k_rope_kv_decode<float><<<grid, 256, 0, s>>>(q, k, v, hq, hk, d, cos_t, sin_t, table_rows, c->len_dev, q_out,
                                                     (float *)c->k + layer * plane, (float *)c->v + layer * plane,
                                                     c->capacity);
    else
        k_rope_kv_decode<fh_half><<<grid, 256, 0, s>>>(q, k, v, hq, hk, d, cos_t, sin_t, table_rows, c->len_dev, q_out,
                                                       (fh_half *)c->k + layer * plane, (fh_half *)c->v + layer * plane,
                                                       c->capacity);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_kvcache_view(const fh_kvcache *c, int32_t layer, int32_t *len, int32_t *capacity,
                                     const void **k_dev, const void **v_dev) {
    FH_REQUIRE(c, "NULL argument");
    FH_REQUIRE(layer >= 0 && layer < c->layers, "bad layer %d", layer);
    size_t plane = (size_t)c->kv_heads * c->capacity * c->head_dim * fh_dtype_size(c->dtype);
    if (len) *len = c->len;
    if (capacity) *capacity = c->capacity;
    if (k_dev) *k_dev = c->k ? (const uint8_t *)c->k + layer * plane : nullptr;
    if (v_dev) *v_dev = c->v ? (const uint8_t *)c->v + layer * plane : nullptr;
    return FH_OK;
}

// ------------------------------------------------------------------------------ non-finite probe
// debug_check_nan_f32, models/kalosm-llama/src/raw/mod.rs:9-58: counts of NaN / +inf / -inf, the largest finite
// magnitude and the indices of the first four NaNs of an f32 tensor.  Workgroup g scans the g-th contiguous segment
// (threads strided inside it, so a thread meets its indices in ascending order and its first four are its smallest);
// the four smallest of a workgroup come out of four rounds of a 64-bit LDS minimum; the host merges the workgroups.
struct FiniteRec {
    uint32_t nan, pos_inf, neg_inf, max_bits;
    uint64_t first[4];
};
__global__ __launch_bounds__(1024) void k_check_finite(const float *x, int64_t n, int64_t seg, FiniteRec *out) {
    __shared__ uint32_t s_cnt[4];
    __shared__ unsigned long long s_min;
    const int64_t lo = (int64_t)blockIdx.x * seg, hi = min(n, lo + seg);
    if (threadIdx.x < 4) s_cnt[threadIdx.x] = 0;
    uint32_t c_nan = 0, c_pi = 0, c_ni = 0, mx = 0;
    uint64_t mine[4] = {~0ull, ~0ull, ~0ull, ~0ull};
    for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const uint32_t b = __float_as_uint(x[i]), a = b & 0x7FFFFFFFu;
        if (a > 0x7F800000u) {
            if (c_nan < 4) mine[c_nan] = (uint64_t)i;
            c_nan++;
        } else if (a == 0x7F800000u) {
            if (b >> 31) c_ni++;
            else c_pi++;
        } else if (a > mx) {
            mx = a; // the bit patterns of non-negative floats order like the floats
        }
    }
    __syncthreads();
    if (c_nan) atomicAdd(&s_cnt[0], c_nan);
    if (c_pi) atomicAdd(&s_cnt[1], c_pi);
    if (c_ni) atomicAdd(&s_cnt[2], c_ni);
    if (mx) atomicMax(&s_cnt[3], mx);
    uint64_t last = 0;
    bool have_last = false;
    for (int r = 0; r < 4; r++) {
        if (threadIdx.x == 0) s_min = ~0ull;
        __syncthreads();
        uint64_t cand = ~0ull;
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (mine[j] != ~0ull && (!have_last || mine[j] > last) && mine[j] < cand) cand = mine[j];
        if (cand != ~0ull) atomicMin(&s_min, (unsigned long long)cand);
        __syncthreads();
        last = s_min;
        have_last = true;
        if (threadIdx.x == 0) out[blockIdx.x].first[r] = last;
        __syncthreads();
        if (last == ~0ull) {
            if (threadIdx.x == 0)
                for (int q = r + 1; q < 4; q++) out[blockIdx.x].first[q] = ~0ull;
            break;
        }
    }
    if (threadIdx.x == 0) {
        out[blockIdx.x].nan = s_cnt[0];
        out[blockIdx.x].pos_inf = s_cnt[1];
        out[blockIdx.x].neg_inf = s_cnt[2];
        out[blockIdx.x].max_bits = s_cnt[3];
    }
}

extern "C" fh_status fh_check_finite(fh_device *dev, const float *x_dev, int64_t count, fh_finite_stats *out_host) {
    FH_REQUIRE(dev && x_dev && out_host, "NULL argument");
    FH_REQUIRE(count > 0, "count %lld out of range", (long long)count);
    const int groups = (int)std::min<int64_t>(256, (count + 1023) / 1024);
    const int64_t seg = (count + groups - 1) / groups;
    FH_REQUIRE(seg < (1ll << 32), "count %lld too large", (long long)count);
    FiniteRec *rec = (FiniteRec *)dev->small_buf; // 256 records of 48 bytes
    k_check_finite<<<dim3(groups), dim3(1024), 0, dev->stream>>>(x_dev, count, seg, rec);
    FH_HIP(hipGetLastError());
    std::vector<FiniteRec> h(groups);
    FH_TRY(fh_download(dev, h.data(), rec, sizeof(FiniteRec) * groups));
    fh_finite_stats s = {};
    uint32_t mx = 0;
    for (const FiniteRec &r : h) { // segments ascend with the workgroup index, so do the indices
        s.nan += r.nan;
        s.pos_inf += r.pos_inf;
        s.neg_inf += r.neg_inf;
        mx = std::max(mx, r.max_bits);
        for (int j = 0; j < 4 && r.first[j] != ~0ull && s.first_nan_count < 4; j++) s.first_nan[s.first_nan_count++] = r.first[j];
    }
    memcpy(&s.max_abs, &mx, 4);
    *out_host = s;
    return FH_OK;
}

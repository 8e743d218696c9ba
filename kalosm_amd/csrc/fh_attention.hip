// softmax(q.k^T * scale [+ mask]) . v with grouped-query heads.
// Reference: fusor-ml/fusor/src/composite/flash_attention.rs:58-236 (semantics),
// fusor-ml/core/src/row_program.rs:1210-1382 (the fused GPU kernel this replaces).
//
//   k_attn_decode + k_attn_combine   one query position: split-KV, both K and V read once, all q heads
//                                    of a KV head share the read (bandwidth kernel)
//   k_attn_rows                      any shape: one workgroup per (batch, head, query row), streaming
//                                    KV in 256-key tiles with an online softmax (fallback / cross-check)
#include "fh_internal.h"

#include <type_traits>

typedef _Float16 fh_half;

template <typename T>
__device__ __forceinline__ void load8(const T *p, float *o);
template <>
__device__ __forceinline__ void load8<float>(const float *p, float *o) {
    float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<fh_half>(const fh_half *p, float *o) {
    uint4 r = *(const uint4 *)p;
    fh_half h[8];
    __builtin_memcpy(h, &r, 16);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = (float)h[i];
}
template <typename T>
__device__ __forceinline__ float ld1(const T *p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void st1(T *p, float v) { *p = (T)v; }

// ------------------------------------------------------------------------------ decode (sq == 1)
// grid (splits, hkv, b); 256 threads.  LP = lanes per key row = D / 8.  The workgroup owns keys
// [c0, c1) of one KV head and the G query heads that share it.
// partial layout: [b][hq][split][D + 2]: o (unnormalised), m, l
template <typename TQ, typename TKV, int D, int G>
__global__ __launch_bounds__(256) void k_attn_decode(const TQ *__restrict__ q, int64_t q_sb, int64_t q_sh,
                                                      const TKV *__restrict__ k, const TKV *__restrict__ v,
                                                      int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int hq, int hkv,
                                                      int skv, const int *__restrict__ len_dev, float scale,
                                                      const float *__restrict__ mask, int chunk,
                                                      float *__restrict__ part, int splits) {
    constexpr int LP = D / 8;        // lanes per row
    constexpr int RPW = 64 / LP;     // rows per wavefront per iteration
    extern __shared__ float sm[];
    float *s_sc = sm;                 // [G][chunk]
    float *s_red = sm + G * chunk;    // [4 waves][G][D]  (also scratch for max/sum: needs >= 8*G)
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, grp = lane / LP, c = lane % LP;
    const int split = blockIdx.x, kh = blockIdx.y, bi = blockIdx.z;
    if (len_dev) skv = *len_dev + 1;
    const int c0 = split * chunk, c1 = min(skv, c0 + chunk);
    const int nk = c1 - c0; // may be <= 0 for trailing splits of a device-side length
    const TKV *kb = k + bi * kv_sb + kh * kv_sh, *vb = v + bi * kv_sb + kh * kv_sh;
    float qr[G][8];
#pragma unroll
    for (int h = 0; h < G; h++) {
        const TQ *qp = q + bi * q_sb + (int64_t)(kh * G + h) * q_sh + 8 * c;
#pragma unroll
        for (int i = 0; i < 8; i++) qr[h][i] = ld1(qp + i);
    }
    // pass 1: scores
    for (int t0 = wave * RPW; t0 < nk; t0 += 4 * RPW) {
        const int t = t0 + grp;
        float kv8[8];
        if (t < nk) load8<TKV>(kb + (int64_t)(c0 + t) * kv_st + 8 * c, kv8);
        else {
#pragma unroll
            for (int i = 0; i < 8; i++) kv8[i] = 0.f;
        }
#pragma unroll
        for (int h = 0; h < G; h++) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) a = fmaf(qr[h][i], kv8[i], a);
#pragma unroll
            for (int o = LP / 2; o > 0; o >>= 1) a += __shfl_xor(a, o, 64);
            if (c == 0 && t < nk) {
                float sc = a * scale;
                if (mask) sc = sc + mask[c0 + t];
                s_sc[h * chunk + t] = sc;
            }
        }
    }
    __syncthreads();
    // softmax statistics per head: wave w handles heads w, w+4
    float mh[G], lh[G];
    for (int h = wave; h < G; h += 4) {
        float mx = -INFINITY;
        for (int t = lane; t < nk; t += 64) mx = fmaxf(mx, s_sc[h * chunk + t]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        float sum = 0.f;
        for (int t = lane; t < nk; t += 64) {
            float sv = s_sc[h * chunk + t];
            float p = (mx == -INFINITY) ? 0.f : __expf(sv - mx);
            s_sc[h * chunk + t] = p;
            sum += p;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        if (lane == 0) {
            s_red[2 * h] = mx;
            s_red[2 * h + 1] = sum;
        }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < G; h++) {
        mh[h] = s_red[2 * h];
        lh[h] = s_red[2 * h + 1];
    }
    __syncthreads();
    // pass 2: o[h][8c..8c+8) += p[h][t] * v[t][8c..8c+8)
    float o[G][8];
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) o[h][i] = 0.f;
    for (int t0 = wave * RPW; t0 < nk; t0 += 4 * RPW) {
        const int t = t0 + grp;
        if (t < nk) {
            float v8[8];
            load8<TKV>(vb + (int64_t)(c0 + t) * kv_st + 8 * c, v8);
#pragma unroll
            for (int h = 0; h < G; h++) {
                const float p = s_sc[h * chunk + t];
#pragma unroll
                for (int i = 0; i < 8; i++) o[h][i] = fmaf(p, v8[i], o[h][i]);
            }
        }
    }
    // reduce over the RPW row groups of the wavefront, then over the 4 wavefronts
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float a = o[h][i];
#pragma unroll
            for (int of = LP; of < 64; of <<= 1) a += __shfl_xor(a, of, 64);
            o[h][i] = a;
        }
    if (grp == 0) {
#pragma unroll
        for (int h = 0; h < G; h++)
#pragma unroll
            for (int i = 0; i < 8; i++) s_red[(wave * G + h) * D + 8 * c + i] = o[h][i];
    }
    __syncthreads();
    for (int idx = tid; idx < G * D; idx += 256) {
        const int h = idx / D, dd = idx % D;
        float a = s_red[(0 * G + h) * D + dd] + s_red[(1 * G + h) * D + dd] + s_red[(2 * G + h) * D + dd] +
                  s_red[(3 * G + h) * D + dd];
        float *pp = part + (((int64_t)bi * hq + kh * G + h) * splits + split) * (D + 2);
        pp[dd] = a;
        if (dd == 0) {
            pp[D] = mh[h];
            pp[D + 1] = lh[h];
        }
    }
}

template <typename TO, int D>
__global__ __launch_bounds__(D) void k_attn_combine(const float *__restrict__ part, int splits, TO *__restrict__ out) {
    const int64_t bh = blockIdx.x;
    const float *pp = part + bh * splits * (D + 2);
    float mx = -INFINITY;
    for (int s = 0; s < splits; s++) mx = fmaxf(mx, pp[s * (D + 2) + D]);
    float num = 0.f, den = 0.f;
    for (int s = 0; s < splits; s++) {
        const float m = pp[s * (D + 2) + D];
        const float w = (m == -INFINITY) ? 0.f : __expf(m - mx);
        num = fmaf(pp[s * (D + 2) + threadIdx.x], w, num);
        den = fmaf(pp[s * (D + 2) + D + 1], w, den);
    }
    st1(out + bh * D + threadIdx.x, num / den);
}

// ------------------------------------------------------------------------------ generic rows
// grid (sq, hq, b); 256 threads.  Online softmax over 256-key tiles.
template <typename TQ, typename TKV>
__global__ __launch_bounds__(256) void k_attn_rows(const TQ *__restrict__ q, int64_t q_sb, int64_t q_sh, int64_t q_st,
                                                    const TKV *__restrict__ k, const TKV *__restrict__ v,
                                                    int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int hq, int hkv,
                                                    int sq, int skv, int d, float scale, int mask_kind,
                                                    const float *__restrict__ mask, TQ *__restrict__ out) {
    extern __shared__ float sm[];
    float *s_q = sm;            // [d]
    float *s_p = sm + d;        // [256]
    float *s_o = s_p + 256;     // [256]  partial outputs of the upper half of the workgroup
    __shared__ float s_w[8];
    const int tid = threadIdx.x;
    const int i = blockIdx.x, h = blockIdx.y, bi = blockIdx.z;
    const int kh = h / (hq / hkv);
    const TQ *qp = q + bi * q_sb + h * q_sh + (int64_t)i * q_st;
    const TKV *kb = k + bi * kv_sb + kh * kv_sh, *vb = v + bi * kv_sb + kh * kv_sh;
    for (int c = tid; c < d; c += 256) s_q[c] = ld1(qp + c);
    __syncthreads();
    int limit = skv; // keys [0, limit) are visible
    if (mask_kind == FH_MASK_CAUSAL) limit = min(skv, i + (skv - sq) + 1);
    float m_run = -INFINITY, l_run = 0.f;
    // each thread owns output column tid % d for half tid / d of every key tile (d <= 128)
    const int halves = 256 / d, oc = tid % d, oh = tid / d;
    float acc = 0.f;
    for (int t0 = 0; t0 < limit; t0 += 256) {
        const int t = t0 + tid;
        float sc = -INFINITY;
        if (t < limit) {
            const TKV *kr = kb + (int64_t)t * kv_st;
            float a = 0.f;
            for (int c = 0; c < d; c++) a = fmaf(s_q[c], ld1(kr + c), a);
            sc = a * scale;
            if (mask_kind == FH_MASK_ADDITIVE) sc = sc + mask[(int64_t)i * skv + t];
            if (mask_kind == FH_MASK_BATCH_KEY) sc = sc + mask[(int64_t)bi * skv + t];
        }
        float mx = sc;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        if ((tid & 63) == 0) s_w[tid >> 6] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(s_w[0], s_w[1]), fmaxf(s_w[2], s_w[3]));
        const float m_new = fmaxf(m_run, mx);
        const float p = (sc == -INFINITY) ? 0.f : __expf(sc - m_new);
        float ps = p;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ps += __shfl_xor(ps, o, 64);
        s_p[tid] = p;
        if ((tid & 63) == 0) s_w[4 + (tid >> 6)] = ps;
        __syncthreads();
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
        l_run = l_run * alpha + ((s_w[4] + s_w[5]) + (s_w[6] + s_w[7]));
        m_run = m_new;
        acc *= alpha;
        const int tn = min(256, limit - t0);
        if (oh < halves) {
            for (int tt = oh; tt < tn; tt += halves) acc = fmaf(s_p[tt], ld1(vb + (int64_t)(t0 + tt) * kv_st + oc), acc);
        }
        __syncthreads();
    }
    s_o[tid] = acc;
    __syncthreads();
    if (tid < d) {
        float a = 0.f;
        for (int hh = 0; hh < halves; hh++) a += s_o[hh * d + tid];
        st1(out + (((int64_t)bi * hq + h) * sq + i) * d + tid, a / l_run);
    }
}

// ------------------------------------------------------------------------------ host side
static int pick_chunk(fh_device *dev, int skv, int hkv, int b) {
    if (dev->opt_attn_splits > 0) {
        int ch = (int)((skv + dev->opt_attn_splits - 1) / dev->opt_attn_splits);
        ch = (ch + 15) / 16 * 16;
        return ch < 16 ? 16 : (ch > 1024 ? 1024 : ch);
    }
    // aim at >= 2 workgroups per CU, between 32 and 256 keys each
    int64_t want = (int64_t)dev->compute_units * 2;
    int64_t splits = (want + (int64_t)hkv * b - 1) / ((int64_t)hkv * b);
    int ch = (int)((skv + splits - 1) / splits);
    ch = (ch + 15) / 16 * 16;
    if (ch < 32) ch = 32;
    if (ch > 256) ch = 256;
    return ch;
}

template <typename TQ, typename TKV, int D, int G>
static fh_status decode_launch(fh_device *dev, const void *q, int64_t q_sb, int64_t q_sh, const void *k, const void *v,
                               int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int skv,
                               const int *len_dev, float scale, const float *mask, void *out) {
    // with a device-side length the grid is sized for the capacity, so keep the chunks small
    int chunk = len_dev ? 32 : pick_chunk(dev, skv, hkv, b);
    int splits = (skv + chunk - 1) / chunk;
    size_t part_bytes = (size_t)b * hq * splits * (D + 2) * 4;
    FH_TRY(fh_dev_scratch(dev, (void **)&dev->part_buf, &dev->part_cap, part_bytes));
    size_t red = (size_t)4 * G * D;
    if (red < (size_t)8 * G) red = 8 * G;
    size_t lds = ((size_t)G * chunk + red) * 4;
    k_attn_decode<TQ, TKV, D, G><<<dim3(splits, hkv, b), dim3(256), lds, dev->stream>>>(
        (const TQ *)q, q_sb, q_sh, (const TKV *)k, (const TKV *)v, kv_sb, kv_sh, kv_st, hq, hkv, skv, len_dev, scale,
        mask, chunk, dev->part_buf, splits);
    FH_HIP(hipGetLastError());
    k_attn_combine<TQ, D><<<dim3((unsigned)(b * hq)), dim3(D), 0, dev->stream>>>(dev->part_buf, splits, (TQ *)out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <typename TQ, typename TKV, int D>
static fh_status decode_dispatch_g(fh_device *dev, int G, const void *q, int64_t q_sb, int64_t q_sh, const void *k,
                                   const void *v, int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv,
                                   int skv, const int *len_dev, float scale, const float *mask, void *out) {
    // any group size up to 8 (Llama-3.2-3B has 24 query heads on 8 KV heads: groups of 3)
#define FH_DECODE_G(G_)                                                                                                  \
    case G_:                                                                                                            \
        return decode_launch<TQ, TKV, D, G_>(dev, q, q_sb, q_sh, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, skv, len_dev, scale, \
                                             mask, out)
    switch (G) {
        FH_DECODE_G(1); FH_DECODE_G(2); FH_DECODE_G(3); FH_DECODE_G(4);
        FH_DECODE_G(5); FH_DECODE_G(6); FH_DECODE_G(7); FH_DECODE_G(8);
    }
#undef FH_DECODE_G
    return FH_ERR_UNSUPPORTED;
}

template <typename TQ, typename TKV>
static fh_status attn_typed(fh_device *dev, const void *q, int64_t q_sb, int64_t q_sh, int64_t q_st, const void *k,
                            const void *v, int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int sq,
                            int skv, int d, float scale, int mask_kind, const float *mask, void *out) {
    const int G = hq / hkv;
    const bool aligned = (kv_st % 8 == 0) && (kv_sh % 8 == 0) && (kv_sb % 8 == 0);
    // one batch entry, head_dim 128, contiguous query heads, no additive mask: the decode-step kernel (an f16
    // query is widened into the device's small buffer first)
    const bool masked = mask_kind == FH_MASK_ADDITIVE || mask_kind == FH_MASK_BATCH_KEY;
    if (sq == 1 && b == 1 && d == 128 && aligned && q_sh == d && !masked && hq <= 64 &&
        dev->opt_attn_kernel != 1) {
        constexpr bool QH = !std::is_same<TQ, float>::value;
        const int kvt = std::is_same<TKV, float>::value ? FH_F32 : FH_F16;
        fh_status st = fh_attention_decode_hostlen(dev, kvt, q, QH, k, v, kv_sh, kv_st, hq, hkv, d, scale, skv, out, QH);
        if (st == FH_ERR_UNSUPPORTED && QH) { // the two-pass kernel reads an f32 query: widen it first
            FH_TRY(fh_cast_f16_f32(dev, q, (float *)dev->small_buf, (int64_t)hq * d));
            st = fh_attention_decode_hostlen(dev, kvt, dev->small_buf, false, k, v, kv_sh, kv_st, hq, hkv, d, scale, skv, out,
                                             QH);
        }
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    if (sq == 1 && aligned && (d == 128 || d == 64) && G <= 8 &&
        mask_kind != FH_MASK_BATCH_KEY) {
        const float *mrow = mask_kind == FH_MASK_ADDITIVE ? mask : nullptr;
        fh_status st = d == 128 ? decode_dispatch_g<TQ, TKV, 128>(dev, G, q, q_sb, q_sh, k, v, kv_sb, kv_sh, kv_st, b, hq,
                                                                 hkv, skv, nullptr, scale, mrow, out)
                                : decode_dispatch_g<TQ, TKV, 64>(dev, G, q, q_sb, q_sh, k, v, kv_sb, kv_sh, kv_st, b, hq,
                                                                hkv, skv, nullptr, scale, mrow, out);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    FH_REQUIRE(d <= 256, "head_dim %d is not supported (at most 256)", d);
    size_t lds = ((size_t)d + 512) * 4;
    k_attn_rows<TQ, TKV><<<dim3(sq, hq, b), dim3(256), lds, dev->stream>>>(
        (const TQ *)q, q_sb, q_sh, q_st, (const TKV *)k, (const TKV *)v, kv_sb, kv_sh, kv_st, hq, hkv, sq, skv, d, scale,
        mask_kind, mask, (TQ *)out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_flash_attention_ex(fh_device *dev, int32_t q_dtype, int32_t kv_dtype, const void *q_dev,
                                           int64_t q_sb, int64_t q_sh, int64_t q_st, const void *k_dev,
                                           const void *v_dev, int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int32_t b,
                                           int32_t hq, int32_t hkv, int32_t sq, int32_t skv, int32_t d, float scale,
                                           int32_t mask_kind, const float *mask_dev, void *out_dev) {
    FH_REQUIRE(dev && q_dev && k_dev && v_dev && out_dev, "NULL argument");
    FH_REQUIRE(b > 0 && hq > 0 && hkv > 0 && sq > 0 && skv > 0 && d > 0, "empty attention operand");
    FH_REQUIRE(hq % hkv == 0, "number of Q heads (%d) must be divisible by number of K/V heads (%d)", hq, hkv);
    FH_REQUIRE(mask_kind >= FH_MASK_NONE && mask_kind <= FH_MASK_BATCH_KEY, "bad mask kind %d", mask_kind);
    FH_REQUIRE((mask_kind != FH_MASK_ADDITIVE && mask_kind != FH_MASK_BATCH_KEY) || mask_dev, "additive mask is NULL");
    FH_REQUIRE(sq <= 65535 && hq <= 65535 && b <= 65535, "grid dimension too large");
    const bool qh = q_dtype == FH_F16, kh = kv_dtype == FH_F16;
    FH_REQUIRE((qh || q_dtype == FH_F32) && (kh || kv_dtype == FH_F32), "dtype must be FH_F32 or FH_F16");
    // many query rows of head_dim 64 / 128 without an additive mask: the matrix-core kernel (all-f32 inputs go
    // through its split-operand form, which keeps f32 accuracy; attn_kernel = 2 asks for plain f16 rounding)
    if (sq >= 32 && dev->opt_attn_kernel != 1 && mask_kind != FH_MASK_BATCH_KEY) {
        fh_status st = fh_attention_prefill_mfma(dev, q_dtype, kv_dtype, q_dev, q_sb, q_sh, q_st, k_dev, v_dev, kv_sb, kv_sh,
                                                 kv_st, b, hq, hkv, sq, skv, d, scale, mask_kind, out_dev);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
#define FH_ATTN_ARGS dev, q_dev, q_sb, q_sh, q_st, k_dev, v_dev, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, d, scale, mask_kind, mask_dev, out_dev
    if (!qh && !kh) return attn_typed<float, float>(FH_ATTN_ARGS);
    if (!qh && kh) return attn_typed<float, fh_half>(FH_ATTN_ARGS);
    if (qh && kh) return attn_typed<fh_half, fh_half>(FH_ATTN_ARGS);
    FH_FAIL(FH_ERR_UNSUPPORTED, "f16 queries with an f32 KV are not supported");
#undef FH_ATTN_ARGS
}

extern "C" fh_status fh_flash_attention(fh_device *dev, int32_t dtype, const void *q_dev, int64_t q_sb, int64_t q_sh,
                                        int64_t q_st, const void *k_dev, const void *v_dev, int64_t kv_sb,
                                        int64_t kv_sh, int64_t kv_st, int32_t b, int32_t hq, int32_t hkv, int32_t sq,
                                        int32_t skv, int32_t d, float scale, int32_t mask_kind, const float *mask_dev,
                                        void *out_dev) {
    return fh_flash_attention_ex(dev, dtype, dtype, q_dev, q_sb, q_sh, q_st, k_dev, v_dev, kv_sb, kv_sh, kv_st, b, hq,
                                 hkv, sq, skv, d, scale, mask_kind, mask_dev, out_dev);
}

// Decode step with the KV length on the device (for graph replay): keys [0, *len_dev] are visible.
// The grid is sized for max_len; splits past the live length write m = -inf, l = 0 and are ignored.
fh_status fh_attention_decode_devlen_v1(fh_device *dev, int kv_dtype, const float *q, const void *k, const void *v,
                                     int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale,
                                     const int *len_dev, int max_len, float *out) {
    const int G = hq / hkv;
    FH_REQUIRE(d == 128 || d == 64, "head_dim %d unsupported", d);
    fh_status st;
    if (kv_dtype == FH_F16)
        st = d == 128 ? decode_dispatch_g<float, fh_half, 128>(dev, G, q, 0, d, k, v, 0, kv_sh, kv_st, 1, hq, hkv, max_len, len_dev, scale, nullptr, out)
                      : decode_dispatch_g<float, fh_half, 64>(dev, G, q, 0, d, k, v, 0, kv_sh, kv_st, 1, hq, hkv, max_len, len_dev, scale, nullptr, out);
    else
        st = d == 128 ? decode_dispatch_g<float, float, 128>(dev, G, q, 0, d, k, v, 0, kv_sh, kv_st, 1, hq, hkv, max_len, len_dev, scale, nullptr, out)
                      : decode_dispatch_g<float, float, 64>(dev, G, q, 0, d, k, v, 0, kv_sh, kv_st, 1, hq, hkv, max_len, len_dev, scale, nullptr, out);
    if (st == FH_ERR_UNSUPPORTED) FH_FAIL(st, "GQA group size %d unsupported in the decode kernel", G);
    return st;
}

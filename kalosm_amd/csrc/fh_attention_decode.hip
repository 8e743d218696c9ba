// Attention of ONE query position against a KV cache whose length lives on the device (graph-replayed decode
// steps): softmax(q . K^T * scale) . V with grouped-query heads.
// Reference: fusor-ml/fusor/src/composite/flash_attention.rs:58-236 (semantics, no mask for a single query:
// models/kalosm-llama/src/raw/mod.rs:969-972).
//
// grid (S splits, kv heads).  The keys of one KV head are dealt to the splits in granules of 16 (granule i goes
// to split i mod S), so which rows a workgroup reads does not depend on the device-side length: the first four
// rows of every lane group, K and V, are requested before the length has arrived (rows past the length are
// read from the cache allocation and masked afterwards), and one memory latency covers the usual context.  A
// workgroup serves the G query heads that share its KV head: K and V rows are read once for all of them.  A key
// row is spread over D / 8 lanes (32 bytes of f32 or 16 bytes of f16 each).  Partial results go to [q head][split][D + 4]:
// unnormalised output, running max, running sum; k_attn_combine_dl (or the consumer of the partials) merges them.
#include "fh_internal.h"

typedef _Float16 fh_half;

template <typename T>
__device__ __forceinline__ void ad_load8(const T *p, float *o);
template <>
__device__ __forceinline__ void ad_load8<float>(const float *p, float *o) {
    const float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
template <>
__device__ __forceinline__ void ad_load8<fh_half>(const fh_half *p, float *o) {
    const uint4 r = *(const uint4 *)p;
    fh_half h[8];
    __builtin_memcpy(h, &r, 16);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = (float)h[i];
}

// One lane's eight elements of a cache row as they sit in the prefetch ring: f32 rows converted (nothing to do),
// f16 rows still packed (four registers instead of eight, so the ring can be twice as deep).
template <typename T>
struct AdRow;
template <>
struct AdRow<float> {
    float v[8];
    __device__ __forceinline__ void load(const float *p) { ad_load8<float>(p, v); }
    __device__ __forceinline__ void load_get(const float *p, float *o) const { ad_load8<float>(p, o); }
    __device__ __forceinline__ void get(float *o) const {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = v[i];
    }
};
template <>
struct AdRow<fh_half> {
    uint4 raw;
    __device__ __forceinline__ void load(const fh_half *p) { raw = *(const uint4 *)p; }
    __device__ __forceinline__ void get(float *o) const {
        fh_half h[8];
        __builtin_memcpy(h, &raw, 16);
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = (float)h[i];
    }
};

template <int CTRL>
__device__ __forceinline__ float ad_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
// sum over the 16 lanes of a DPP row (all lanes get it): xor 1, xor 2, then mirrors of 8 and 16 over uniform groups
__device__ __forceinline__ float ad_row16_sum(float a) {
    a += ad_dpp<0xB1>(a);
    a += ad_dpp<0x4E>(a);
    a += ad_dpp<0x141>(a);
    a += ad_dpp<0x140>(a);
    return a;
}
// lanes 0-31: a[l] + a[l + 32]; lanes 32-63: b[l - 32] + b[l]  (one swap and one add fold two registers)
__device__ __forceinline__ float ad_fold32(float a, float b) {
    auto s = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}
// rows of 16 lanes (r0, r1, r2, r3) of a and b -> (a.r0 + a.r1, b.r0 + b.r1, a.r2 + a.r3, b.r2 + b.r3)
__device__ __forceinline__ float ad_fold16(float a, float b) {
    auto s = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}
// sum over the four rows of 16 lanes of a wavefront (lane i of every row gets it)
__device__ __forceinline__ float ad_rows_sum(float a) {
    const uint32_t u = __float_as_uint(a);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);
    const uint32_t w = __float_as_uint(a);
    auto s32 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(s32[0]) + __uint_as_float(s32[1]);
}

template <typename TKV, int D, int G, int NWV>
__global__ __launch_bounds__(64 * NWV) void k_attn_decode_dl(const float *__restrict__ q, const TKV *__restrict__ k,
                                                              const TKV *__restrict__ v, int64_t kv_sh, int64_t kv_st,
                                                              const int *__restrict__ len_dev, int len_host,
                                                              float scale, int chunk_max, int cap, int gtot,
                                                              float *__restrict__ part) {
    // ring depth: rows in flight per lane group (every refill costs a full memory round trip, so long parts
    // want all their iterations in the ring; packed f16 rows make eight slots as cheap as four f32 ones)
    constexpr int LP = D / 8, RPW = 64 / LP, RW = NWV * RPW, U = sizeof(TKV) == 2 ? 8 : 4;
    static_assert(NWV >= G, "one wavefront per query head for the softmax statistics");
    extern __shared__ float sm[];
    float *s_sc = sm;                  // [G][chunk_max]
    float *s_red = sm + G * chunk_max; // [NWV][G][D]
    __shared__ float s_stat[2 * G];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, grp = lane / LP, c = lane % LP;
    // blockIdx.z: which G of the gtot query heads of this KV head (the K and V rows are then read once per group)
    const int split = blockIdx.x, S = gridDim.x, kh = blockIdx.y, h0 = kh * gtot + (int)blockIdx.z * G;
    const TKV *kb = k + kh * kv_sh + 8 * c, *vb = v + kh * kv_sh + 8 * c;
    const int trow = wave * RPW + grp; // local row of this lane group inside an iteration of RW rows
    // local row -> cache row: granule (local / 16) of this split is granule (local / 16) * S + split of the head
    auto cache_row = [&](int lr) { return ((lr >> 4) * S + split) * 16 + (lr & 15); };

    // the first U0 rows of every lane group are requested blind (U0 * RW = 128 local rows = 1024 keys with 8 splits); the
    // other prefetched rows wait for the length, so that a short context does not pay for requests it drops
    constexpr int U0 = 32 / NWV < U ? 32 / NWV : U;
    AdRow<TKV> kpre[U], vpre[U];
#pragma unroll
    for (int u = 0; u < U0; u++) {
        const int t = cache_row(u * RW + trow);
        kpre[u].load(kb + (int64_t)(t < cap ? t : 0) * kv_st);
    }
#pragma unroll
    for (int u = 0; u < U0; u++) {
        const int t = cache_row(u * RW + trow);
        vpre[u].load(vb + (int64_t)(t < cap ? t : 0) * kv_st);
    }
    __builtin_amdgcn_sched_barrier(0); // the requests above do not wait for the length
    // the step's own key is already appended at index len; a caller that knows the length passes it by value
    const int skv = (len_dev ? *len_dev : len_host) + 1;
    // local rows of this split: 16 per whole granule it owns, plus the tail if the last, partial granule is its own
    const int gfull = skv >> 4;
    int nk = gfull > split ? ((gfull - split + S - 1) / S) * 16 : 0;
    if (gfull % S == split) nk += skv & 15;
    if (nk > chunk_max) nk = chunk_max;
#pragma unroll
    for (int u = U0; u < U; u++) {
        const int lr = u * RW + trow;
        if (u * RW < nk) {
            kpre[u].load(kb + (int64_t)cache_row(lr < nk ? lr : 0) * kv_st);
            vpre[u].load(vb + (int64_t)cache_row(lr < nk ? lr : 0) * kv_st);
        }
    }
    // (rows past nk hold whatever the cache allocation held: every use below is guarded by the row index)
    const int niter = (nk + RW - 1) / RW;
    float qr[G][8];
#pragma unroll
    for (int h = 0; h < G; h++) {
        const float4 a = *(const float4 *)(q + (int64_t)(h0 + h) * D + 8 * c);
        const float4 b = *(const float4 *)(q + (int64_t)(h0 + h) * D + 8 * c + 4);
        qr[h][0] = a.x; qr[h][1] = a.y; qr[h][2] = a.z; qr[h][3] = a.w;
        qr[h][4] = b.x; qr[h][5] = b.y; qr[h][6] = b.z; qr[h][7] = b.w;
    }
    // ---- scores
    auto score = [&](const AdRow<TKV> &row, int t) {
        float kv8[8];
        row.get(kv8);
#pragma unroll
        for (int h = 0; h < G; h++) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) a = fmaf(qr[h][i], kv8[i], a);
            a = ad_row16_sum(a);
            if (c == 0 && t < nk) s_sc[h * chunk_max + t] = a * scale;
        }
    };
    // a ring of U rows per lane group: the slot of iteration it is refilled with the row of iteration it + U
    for (int it0 = 0; it0 < niter; it0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int it = it0 + u;
            if (it < niter) {
                score(kpre[u], it * RW + trow);
                if ((it + U) * RW < nk) {
                    const int lr = (it + U) * RW + trow;
                    kpre[u].load(kb + (int64_t)cache_row(lr < nk ? lr : 0) * kv_st);
                }
            }
        }
    }
    __syncthreads();
    // ---- softmax statistics: wavefront h owns query head h
    if (wave < G) {
        const int h = wave;
        float mx = -INFINITY;
        for (int t = lane; t < nk; t += 64) mx = fmaxf(mx, s_sc[h * chunk_max + t]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        float sum = 0.f;
        for (int t = lane; t < nk; t += 64) {
            const float p = __expf(s_sc[h * chunk_max + t] - mx);
            s_sc[h * chunk_max + t] = p;
            sum += p;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        if (lane == 0) {
            s_stat[2 * h] = mx;
            s_stat[2 * h + 1] = sum;
        }
    }
    __syncthreads();
    // ---- o[h][8c .. 8c+8) += p[h][t] * v[t][8c .. 8c+8)
    float o[G][8];
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) o[h][i] = 0.f;
    auto accum = [&](const AdRow<TKV> &row, int t) {
        if (t < nk) {
            float v8[8];
            row.get(v8);
#pragma unroll
            for (int h = 0; h < G; h++) {
                const float p = s_sc[h * chunk_max + t];
#pragma unroll
                for (int i = 0; i < 8; i++) o[h][i] = fmaf(p, v8[i], o[h][i]);
            }
        }
    };
    for (int it0 = 0; it0 < niter; it0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int it = it0 + u;
            if (it < niter) {
                accum(vpre[u], it * RW + trow);
                if ((it + U) * RW < nk) {
                    const int lr = (it + U) * RW + trow;
                    vpre[u].load(vb + (int64_t)cache_row(lr < nk ? lr : 0) * kv_st);
                }
            }
        }
    }
    // ---- add the row groups of the wavefront, then the wavefronts
    if constexpr (G == 4) {
        // four heads x one dim fold into one register: row r of 16 lanes ends with head r's total, so every lane
        // stores eight sums of "its" head (6 operations per 4 values instead of 6 per value)
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            f[i] = ad_fold16(ad_fold32(o[0][i], o[2][i]), ad_fold32(o[1][i], o[3][i]));
        float *dst = s_red + (wave * G + grp) * D + 8 * c;
        *(float4 *)dst = make_float4(f[0], f[1], f[2], f[3]);
        *(float4 *)(dst + 4) = make_float4(f[4], f[5], f[6], f[7]);
    } else if constexpr (G == 2) {
        // row r ends with head r % 2, dims i + 4 (r / 2)
        float f[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            f[i] = ad_fold16(ad_fold32(o[0][i], o[0][i + 4]), ad_fold32(o[1][i], o[1][i + 4]));
        *(float4 *)(s_red + (wave * G + (grp & 1)) * D + 8 * c + 4 * (grp >> 1)) = make_float4(f[0], f[1], f[2], f[3]);
    } else if constexpr (G == 1) {
        // row r ends with dims i + 2 r
        float f[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            f[i] = ad_fold16(ad_fold32(o[0][i], o[0][i + 4]), ad_fold32(o[0][i + 2], o[0][i + 6]));
        *(float2 *)(s_red + wave * D + 8 * c + 2 * grp) = make_float2(f[0], f[1]);
    } else {
#pragma unroll
        for (int h = 0; h < G; h++)
#pragma unroll
            for (int i = 0; i < 8; i++) o[h][i] = ad_rows_sum(o[h][i]);
        if (grp == 0) {
#pragma unroll
            for (int h = 0; h < G; h++) {
                float *dst = s_red + (wave * G + h) * D + 8 * c;
                *(float4 *)dst = make_float4(o[h][0], o[h][1], o[h][2], o[h][3]);
                *(float4 *)(dst + 4) = make_float4(o[h][4], o[h][5], o[h][6], o[h][7]);
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < G * D; idx += 64 * NWV) {
        const int h = idx / D, dd = idx % D;
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; w++) a += s_red[(w * G + h) * D + dd];
        float *pp = part + ((int64_t)(h0 + h) * S + split) * (D + 4);
        pp[dd] = a;
        if (dd == 0) {
            pp[D] = nk > 0 ? s_stat[2 * h] : -INFINITY;
            pp[D + 1] = nk > 0 ? s_stat[2 * h + 1] : 0.f;
        }
    }
}

// max over the four rows of 16 lanes of a wavefront (lane i of every row gets it)
__device__ __forceinline__ float ad_rows_max(float a) {
    const uint32_t u = __float_as_uint(a);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = fmaxf(__uint_as_float(s16[0]), __uint_as_float(s16[1]));
    const uint32_t w = __float_as_uint(a);
    auto s32 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__uint_as_float(s32[0]), __uint_as_float(s32[1]));
}

// ------------------------------------------------------------------------------ one pass over long caches
// The same part of the same grid as k_attn_decode_dl, for parts of many keys: a lane group (16 lanes, 8 dims each)
// takes C rows at a time, K and V row of a key together, and keeps a running maximum, denominator and weighted V sum
// per query head (online softmax); nothing is staged in LDS and no barrier separates scores from P.V, so the
// arithmetic of one wavefront runs under the transfers of the others.  Lane groups and wavefronts are merged at
// the end.  Partials as k_attn_decode_dl writes them: [head][part][D weighted sums | max | denominator | 2 unused].
template <typename TKV, int G, int NWV>
__global__ __launch_bounds__(64 * NWV) void k_attn_decode_1p(const void *__restrict__ qv, int q_f16, const TKV *__restrict__ k,
                                                              const TKV *__restrict__ v, int64_t kv_sh, int64_t kv_st,
                                                              const int *__restrict__ len_dev, int len_host, float scale,
                                                              int cap, int gtot, float *__restrict__ part) {
    constexpr int D = 128, LP = D / 8, RPW = 64 / LP, RW = NWV * RPW;
    constexpr int C = sizeof(TKV) == 2 ? 4 : 2; // rows of a chunk per lane group: 2 KB of K and V per lane group
    __shared__ float s_red[NWV * G * D];
    __shared__ float s_st[NWV * G * 2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, grp = lane / LP, c = lane % LP;
    const int split = blockIdx.x, S = gridDim.x, kh = blockIdx.y, h0 = kh * gtot + (int)blockIdx.z * G;
    const TKV *kb = k + kh * kv_sh + 8 * c, *vb = v + kh * kv_sh + 8 * c;
    const int trow = wave * RPW + grp;
    const int skv = (len_dev ? *len_dev : len_host) + 1;
    const int gfull = skv >> 4;
    int nk = gfull > split ? ((gfull - split + S - 1) / S) * 16 : 0;
    if (gfull % S == split) nk += skv & 15;
    const int niter = (nk + RW - 1) / RW;
    float qr[G][8]; // the query may arrive as f16 (a caller's tensor) or f32 (the decoder's own)
#pragma unroll
    for (int h = 0; h < G; h++) {
        if (q_f16) AdRow<fh_half>{*(const uint4 *)((const fh_half *)qv + (int64_t)(h0 + h) * D + 8 * c)}.get(qr[h]);
        else AdRow<float>().load_get((const float *)qv + (int64_t)(h0 + h) * D + 8 * c, qr[h]);
#pragma unroll
        for (int i = 0; i < 8; i++) qr[h][i] *= scale;
    }
    float m[G], l[G], o[G][8];
#pragma unroll
    for (int h = 0; h < G; h++) {
        m[h] = -INFINITY;
        l[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) o[h][i] = 0.f;
    }
    // a chunk: C rows per lane group.  With few query heads per workgroup there are registers for two chunks: the
    // next one is requested before the current one is multiplied (requests past the end re-read a live row and
    // are ignored).
    constexpr bool DB = G <= 2;
    AdRow<TKV> kr[DB ? 2 : 1][C], vr[DB ? 2 : 1][C];
    auto issue = [&](int b, int it0) {
#pragma unroll
        for (int j = 0; j < C; j++) {
            const int lr = (it0 + j) * RW + trow; // local row -> granule (lr / 16) * S + split of the head's rows
            const int lv = lr < nk ? lr : 0;
            int row = ((lv >> 4) * S + split) * 16 + (lv & 15);
            row = row < cap ? row : 0; // rows past the live ones are read from a valid address and never used
            kr[b][j].load(kb + (int64_t)row * kv_st);
            vr[b][j].load(vb + (int64_t)row * kv_st);
        }
    };
    auto process = [&](int b, int it0) {
        float sc[C][G];
#pragma unroll
        for (int j = 0; j < C; j++) {
            const bool ok = (it0 + j) * RW + trow < nk;
            float k8[8];
            kr[b][j].get(k8);
#pragma unroll
            for (int h = 0; h < G; h++) {
                float a = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) a = fmaf(qr[h][i], k8[i], a);
                a = ad_row16_sum(a);
                sc[j][h] = ok ? a : -INFINITY;
            }
        }
#pragma unroll
        for (int h = 0; h < G; h++) {
            float cm = sc[0][h];
#pragma unroll
            for (int j = 1; j < C; j++) cm = fmaxf(cm, sc[j][h]);
            const float mn = fmaxf(m[h], cm);
            const float ref = mn == -INFINITY ? 0.f : mn; // nothing live yet: every weight below becomes exp(-inf) = 0
            const float alpha = __expf(m[h] - ref);
            l[h] *= alpha;
#pragma unroll
            for (int i = 0; i < 8; i++) o[h][i] *= alpha;
#pragma unroll
            for (int j = 0; j < C; j++) {
                const float p = __expf(sc[j][h] - ref);
                sc[j][h] = p;
                l[h] += p;
            }
            m[h] = mn;
        }
#pragma unroll
        for (int j = 0; j < C; j++) {
            float v8[8];
            vr[b][j].get(v8);
#pragma unroll
            for (int h = 0; h < G; h++)
#pragma unroll
                for (int i = 0; i < 8; i++) o[h][i] = fmaf(sc[j][h], v8[i], o[h][i]);
        }
    };
    if constexpr (DB) {
        issue(0, 0);
        if (niter <= C) { // a short part (the usual decode step): one chunk, nothing to overlap
            // (a part without keys multiplies nothing: its clamped rows lie past the live ones and may hold anything,
            // and a weight of zero does not silence a NaN)
            if (niter > 0) process(0, 0);
        } else {
            // no branches around the requests (a wait after a branch waits for everything in flight): the last trips
            // re-read a live row and ignore it
            for (int it0 = 0; it0 < niter; it0 += 2 * C) {
                issue(1, it0 + C);
                __builtin_amdgcn_sched_barrier(0); // the requests stay ahead of the arithmetic on the other chunk
                process(0, it0);
                __builtin_amdgcn_sched_barrier(0);
                issue(0, it0 + 2 * C);
                __builtin_amdgcn_sched_barrier(0);
                process(1, it0 + C);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    } else {
        for (int it0 = 0; it0 < niter; it0 += C) {
            issue(0, it0);
            process(0, it0);
        }
    }
    // ---- the four lane groups of the wavefront, then the wavefronts
#pragma unroll
    for (int h = 0; h < G; h++) {
        const float ma = ad_rows_max(m[h]);
        const float ref = ma == -INFINITY ? 0.f : ma;
        const float f = __expf(m[h] - ref);
        const float la = ad_rows_sum(l[h] * f);
        float oa[8];
#pragma unroll
        for (int i = 0; i < 8; i++) oa[i] = ad_rows_sum(o[h][i] * f);
        if (grp == 0) {
            float *dst = s_red + (wave * G + h) * D + 8 * c;
            *(float4 *)dst = make_float4(oa[0], oa[1], oa[2], oa[3]);
            *(float4 *)(dst + 4) = make_float4(oa[4], oa[5], oa[6], oa[7]);
            if (c == 0) {
                s_st[(wave * G + h) * 2] = ma;
                s_st[(wave * G + h) * 2 + 1] = la;
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < G * D; idx += 64 * NWV) {
        const int h = idx / D, dd = idx % D;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < NWV; w++) mx = fmaxf(mx, s_st[(w * G + h) * 2]);
        const float ref = mx == -INFINITY ? 0.f : mx;
        float a = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; w++) {
            const float f = __expf(s_st[(w * G + h) * 2] - ref);
            a = fmaf(s_red[(w * G + h) * D + dd], f, a);
            den = fmaf(s_st[(w * G + h) * 2 + 1], f, den);
        }
        float *pp = part + ((int64_t)(h0 + h) * S + split) * (D + 4);
        pp[dd] = a;
        if (dd == 0) {
            pp[D] = mx;
            pp[D + 1] = den;
        }
    }
}

// Merge of the parts of one head: thread t fetches the statistics of part t (all parts at once instead of one
// dependent load per loop trip), the weights go through LDS, and the weighted rows are summed eight loads at a time.
template <int D, typename TO = float>
__global__ __launch_bounds__(D) void k_attn_combine_dl(const float *__restrict__ part, int splits, TO *__restrict__ out) {
    static_assert(D >= 128, "one thread per part: up to 128 parts");
    __shared__ float s_m[D], s_w[D];
    const int64_t h = blockIdx.x;
    const int t = threadIdx.x;
    const float *pp = part + h * splits * (D + 4);
    float m = -INFINITY, l = 0.f;
    if (t < splits) {
        m = pp[t * (D + 4) + D];
        l = pp[t * (D + 4) + D + 1];
    }
    s_m[t] = m;
    __syncthreads();
    float mx = -INFINITY;
    for (int s = 0; s < splits; s++) mx = fmaxf(mx, s_m[s]);
    const float w = (m == -INFINITY) ? 0.f : __expf(m - mx);
    s_w[t] = w;
    s_m[t] = l * w; // reuse: weighted denominators
    __syncthreads();
    float num = 0.f, den = 0.f;
    int s = 0;
    for (; s + 8 <= splits; s += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = pp[(s + u) * (D + 4) + t];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            num = fmaf(v[u], s_w[s + u], num);
            den += s_m[s + u];
        }
    }
    for (; s < splits; s++) {
        num = fmaf(pp[s * (D + 4) + t], s_w[s], num);
        den += s_m[s];
    }
    out[h * D + t] = (TO)(num / den);
}

template <typename TKV, int G, int NWV>
static fh_status ad_launch(fh_device *dev, const float *q, const void *k, const void *v, int64_t kv_sh, int64_t kv_st,
                           int hq, int hkv, float scale, const int *len_dev, int max_len, float *out, int *splits_out,
                           int gtot, int len_host = 0, int splits_req = 0, bool out_f16 = false, bool one_pass = false,
                           bool q_f16 = false, float *part_fixed = nullptr) {
    constexpr int D = 128;
    // splits: 8 measured best from a few hundred to a few thousand keys (MI355X); it is also the most the output
    // projection merges while staging its input.  The option allows 4 .. 16; a caller with a long cache and its
    // own merge asks for more.
    int S = dev->opt_attn_splits > 0 ? (int)dev->opt_attn_splits : 8;
    S = S < 4 ? 4 : (S > 16 ? 16 : S);
    if (splits_req > 0) S = splits_req;
    FH_REQUIRE(!q_f16 || (one_pass && G <= 4), "an f16 query needs the one-pass kernel");
    if (one_pass && G <= 4) {
        // partial results: the device's growable buffer, or a buffer the caller fixed (no allocation then)
        float *part = part_fixed;
        if (!part) {
            FH_TRY(fh_dev_scratch(dev, (void **)&dev->part_buf, &dev->part_cap, (size_t)hq * S * (D + 4) * 4));
            part = dev->part_buf;
        }
        k_attn_decode_1p<TKV, (G <= 4 ? G : 4), NWV><<<dim3((unsigned)S, (unsigned)hkv, (unsigned)(gtot / G)), dim3(64 * NWV), 0,
                                                       dev->stream>>>(q, q_f16 ? 1 : 0, (const TKV *)k, (const TKV *)v, kv_sh,
                                                                      kv_st, len_dev, len_host, scale, max_len, gtot, part);
        FH_HIP(hipGetLastError());
        if (splits_out) *splits_out = S;
        if (out) {
            if (out_f16)
                k_attn_combine_dl<D, fh_half><<<dim3((unsigned)hq), dim3(D), 0, dev->stream>>>(part, S, (fh_half *)out);
            else k_attn_combine_dl<D><<<dim3((unsigned)hq), dim3(D), 0, dev->stream>>>(part, S, out);
            FH_HIP(hipGetLastError());
        }
        return FH_OK;
    }
    FH_REQUIRE(!part_fixed, "a fixed partial buffer needs the one-pass kernel");
    const int chunk_max = (((max_len + 15) / 16 + S - 1) / S) * 16; // most local rows of a split
    const size_t lds = ((size_t)G * chunk_max + (size_t)NWV * G * D) * 4;
    FH_REQUIRE(lds <= 150 * 1024, "KV capacity %d too large for the decode attention kernel", max_len);
    FH_TRY(fh_dev_scratch(dev, (void **)&dev->part_buf, &dev->part_cap, (size_t)hq * S * (D + 4) * 4));
    FH_TRY(fh_kernel_lds(dev, (const void *)k_attn_decode_dl<TKV, D, G, NWV>, 152 * 1024));
    k_attn_decode_dl<TKV, D, G, NWV><<<dim3((unsigned)S, (unsigned)hkv, (unsigned)(gtot / G)), dim3(64 * NWV), lds, dev->stream>>>(
        q, (const TKV *)k, (const TKV *)v, kv_sh, kv_st, len_dev, len_host, scale, chunk_max, max_len, gtot, dev->part_buf);
    FH_HIP(hipGetLastError());
    if (splits_out) *splits_out = S;
    if (out) {
        if (out_f16)
            k_attn_combine_dl<D, fh_half><<<dim3((unsigned)hq), dim3(D), 0, dev->stream>>>(dev->part_buf, S, (fh_half *)out);
        else k_attn_combine_dl<D><<<dim3((unsigned)hq), dim3(D), 0, dev->stream>>>(dev->part_buf, S, out);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

// Merge the partials fh_attention_decode_devlen left in the device's scratch (head_dim 128).
fh_status fh_attention_combine_dl(fh_device *dev, int hq, int splits, float *out) {
    k_attn_combine_dl<128><<<dim3((unsigned)hq), dim3(128), 0, dev->stream>>>(dev->part_buf, splits, out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// out != NULL: the attention output [hq, d].  out == NULL: the partials stay in the device's scratch
// ([hq][*splits_out][d + 4]) for a consumer that merges them itself.
static fh_status ad_any(fh_device *dev, int kv_dtype, const float *q, const void *k, const void *v, int64_t kv_sh,
                        int64_t kv_st, int hq, int hkv, int d, float scale, const int *len_dev, int max_len, float *out,
                        int *splits_out, int len_host, int splits_req, bool out_f16, int heads_req = 0, int waves_req = 0,
                        bool q_f16 = false, float *part_fixed = nullptr);

fh_status fh_attention_decode_devlen(fh_device *dev, int kv_dtype, const float *q, const void *k, const void *v,
                                     int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale,
                                     const int *len_dev, int max_len, float *out, int *splits_out) {
    return ad_any(dev, kv_dtype, q, k, v, kv_sh, kv_st, hq, hkv, d, scale, len_dev, max_len, out, splits_out, 0, 0, false);
}

// Merge of many parts: four thread groups of 128 take every fourth part each (a quarter of the dependent load
// rounds of k_attn_combine_dl), then add up through LDS.
template <typename TO>
__global__ __launch_bounds__(512) void k_attn_combine_wide(const float *__restrict__ part, int splits, TO *__restrict__ out) {
    constexpr int D = 128, PG = 4;
    __shared__ float s_m[128], s_w[128], s_num[PG][D], s_den[PG];
    const int64_t h = blockIdx.x;
    const int t = threadIdx.x & 127, pg = threadIdx.x >> 7;
    const float *pp = part + h * splits * (D + 4);
    float m = -INFINITY, l = 0.f;
    if (pg == 0) {
        if (t < splits) {
            m = pp[t * (D + 4) + D];
            l = pp[t * (D + 4) + D + 1];
        }
        s_m[t] = m;
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int s = 0; s < splits; s++) mx = fmaxf(mx, s_m[s]);
    __syncthreads();
    if (pg == 0) {
        const float w = (m == -INFINITY) ? 0.f : __expf(m - mx);
        s_w[t] = w;
        s_m[t] = l * w; // reuse: weighted denominators
    }
    __syncthreads();
    float num = 0.f, den = 0.f;
    int s = pg;
    for (; s + 7 * PG < splits; s += 8 * PG) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = pp[(s + u * PG) * (D + 4) + t];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            num = fmaf(v[u], s_w[s + u * PG], num);
            den += s_m[s + u * PG];
        }
    }
    for (; s < splits; s += PG) {
        num = fmaf(pp[s * (D + 4) + t], s_w[s], num);
        den += s_m[s];
    }
    s_num[pg][t] = num;
    if (t == 0) s_den[pg] = den;
    __syncthreads();
    if (pg == 0) {
        num = (s_num[0][t] + s_num[1][t]) + (s_num[2][t] + s_num[3][t]);
        den = (s_den[0] + s_den[1]) + (s_den[2] + s_den[3]);
        out[h * D + t] = (TO)(num / den);
    }
}

// Merge `splits` partials per head ([hq][splits][132] floats) into out [hq, 128], f32 or f16.
fh_status fh_attention_combine_parts(fh_device *dev, const float *part, int hq, int splits, void *out, bool out_f16) {
    FH_REQUIRE(splits >= 1 && splits <= 128, "the merge takes 1 .. 128 parts");
    if (splits > 16) {
        if (out_f16) k_attn_combine_wide<fh_half><<<dim3((unsigned)hq), dim3(512), 0, dev->stream>>>(part, splits, (fh_half *)out);
        else k_attn_combine_wide<float><<<dim3((unsigned)hq), dim3(512), 0, dev->stream>>>(part, splits, (float *)out);
    } else if (out_f16) k_attn_combine_dl<128, fh_half><<<dim3((unsigned)hq), dim3(128), 0, dev->stream>>>(part, splits, (fh_half *)out);
    else k_attn_combine_dl<128><<<dim3((unsigned)hq), dim3(128), 0, dev->stream>>>(part, splits, (float *)out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// One f32 query per head against `skv` cached keys known on the host; `out` is f32 or f16 [hq, d].  The key
// range is cut into more parts the longer it is (every part is a workgroup per KV head and query-head group).
fh_status fh_attention_decode_hostlen(fh_device *dev, int kv_dtype, const void *q, bool q_f16, const void *k,
                                      const void *v, int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale,
                                      int skv, void *out, bool out_f16) {
    // long f16 caches: the matrix-core kernel (attn_kernel = 5 forces it from 32 keys up, any other non-zero value keeps the vector-ALU kernels)
    const int mfma_min = dev->opt_attn_kernel == 5 ? 32 : 4096;
    if (kv_dtype == FH_F16 && d == 128 && hq % hkv == 0 && hq / hkv <= 16 && skv >= mfma_min &&
        (dev->opt_attn_kernel == 0 || dev->opt_attn_kernel == 5) && dev->opt_attn_heads == 0 && kv_st % 8 == 0 && kv_sh % 8 == 0) {
        // parts: four wavefronts each, two chunks of 32 keys per wavefront, at most 128 parts for the merge (measured on
        // MI355X, 32 / 8 heads: 19.2 us against 22.0 us of the vector-ALU kernel at 16384 keys, level at 4096)
        const int nct = (skv + 31) / 32;
        int splits = dev->opt_attn_splits > 0 ? (int)dev->opt_attn_splits : nct / 8;
        splits = splits < 1 ? 1 : (splits > 128 ? 128 : splits);
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->part_buf, &dev->part_cap, (size_t)hq * splits * (128 + 4) * 4));
        fh_status st = fh_attention_decode_mfma(dev, q, q_f16, k, v, kv_sh, kv_st, hq, hkv, d, scale, skv, splits, dev->part_buf);
        if (st != FH_ERR_UNSUPPORTED) {
            if (st != FH_OK) return st;
            return fh_attention_combine_parts(dev, dev->part_buf, hq, splits, out, out_f16);
        }
    }
    if (q_f16 && (dev->opt_attn_kernel == 4 || (dev->opt_attn_heads > 4))) return FH_ERR_UNSUPPORTED; // caller widens q
    int splits = skv <= 2048 ? 8 : 16;
    if (dev->opt_attn_splits > 0) splits = dev->opt_attn_splits > 128 ? 128 : (int)dev->opt_attn_splits;
    // long caches are bandwidth bound: all query heads of a KV head in one workgroup, so K and V are read once
    // (measured on MI355X, 32 / 8 heads, f16 cache: 1 head x 8 parts x 16 wavefronts at 1024 keys, 2 x 16 x 8 at
    // 4096 and 16384)
    const int heads = dev->opt_attn_heads > 0 ? (int)dev->opt_attn_heads : (skv <= 2048 ? 1 : 2);
    return ad_any(dev, kv_dtype, (const float *)q, k, v, kv_sh, kv_st, hq, hkv, d, scale, nullptr, skv, (float *)out, nullptr,
                  skv - 1, splits, out_f16, heads, skv > 2048 ? 8 : 0, q_f16);
}

// ------------------------------------------------------------------------------ no allocation at call time
// The partial results of the key parts normally live in a buffer the library grows with hipMalloc.  Callers that
// must not allocate (a stream under graph capture, a serving loop that forbids it) use the entry point below: its
// partials live in this array, which exists once per GPU from the moment the library's code is loaded there until
// the process ends.  Room for 64 query heads x 16 key parts x (128 + 4) floats.
#define FH_STATIC_SCRATCH_BYTES (64 * 16 * (128 + 4) * 4)
static __device__ __align__(256) unsigned char fh_static_scratch[FH_STATIC_SCRATCH_BYTES];

// Called by fh_device_create with the device current: in host code the array's name is only a stand-in, its
// address on THIS device comes from the runtime and is kept in the device handle.
fh_status fh_static_scratch_init(fh_device *dev) {
    void *p = nullptr;
    FH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(fh_static_scratch)));
    FH_REQUIRE(p, "hipGetSymbolAddress returned no address for the static scratch");
    dev->static_scratch = p;
    dev->static_scratch_bytes = FH_STATIC_SCRATCH_BYTES;
    return FH_OK;
}

extern "C" fh_status fh_flash_attention_decode_static(fh_device *dev, int32_t q_dtype, int32_t kv_dtype,
                                                      const void *q_dev, const void *k_dev, const void *v_dev,
                                                      int64_t kv_sh, int64_t kv_st, int32_t hq, int32_t hkv, int32_t d,
                                                      float scale, int32_t skv, void *out_dev) {
    FH_REQUIRE(dev && q_dev && k_dev && v_dev && out_dev, "NULL argument");
    FH_REQUIRE(dev->static_scratch, "the device handle has no static scratch");
    FH_REQUIRE(hq > 0 && hkv > 0 && skv > 0, "empty attention operand");
    FH_REQUIRE(hq % hkv == 0, "number of Q heads (%d) must be divisible by number of K/V heads (%d)", hq, hkv);
    const bool qh = q_dtype == FH_F16, kh = kv_dtype == FH_F16;
    FH_REQUIRE((qh || q_dtype == FH_F32) && (kh || kv_dtype == FH_F32), "dtype must be FH_F32 or FH_F16");
    if (qh && !kh) FH_FAIL(FH_ERR_UNSUPPORTED, "f16 queries with an f32 KV are not supported");
    if (d != 128 || kv_st % 8 || kv_sh % 8)
        FH_FAIL(FH_ERR_UNSUPPORTED, "the allocation-free decode attention needs head_dim 128 and K / V strides that are "
                                    "multiples of 8 elements (got d = %d, strides %lld, %lld)", d, (long long)kv_sh,
                (long long)kv_st);
    // the same cut of the key range as fh_flash_attention makes for one query position
    int splits = skv <= 2048 ? 8 : 16;
    if (dev->opt_attn_splits > 0) splits = dev->opt_attn_splits > 128 ? 128 : (int)dev->opt_attn_splits;
    const size_t need = (size_t)hq * splits * (128 + 4) * 4;
    if (need > dev->static_scratch_bytes)
        FH_FAIL(FH_ERR_INVALID, "%d query heads x %d key parts need %zu bytes of partial results; the static scratch "
                                "holds %zu (at most 64 heads x 16 parts): use fh_flash_attention", hq, splits, need,
                dev->static_scratch_bytes);
    const int heads = dev->opt_attn_heads > 0 ? (int)dev->opt_attn_heads : (skv <= 2048 ? 1 : 2);
    // Every (head, part) slot the merge reads is written by this call's first kernel, parts without keys
    // included, so nothing has to be cleared between calls.
    return ad_any(dev, kv_dtype, (const float *)q_dev, k_dev, v_dev, kv_sh, kv_st, hq, hkv, d, scale, nullptr, skv,
                  (float *)out_dev, nullptr, skv - 1, splits, qh, heads, skv > 2048 ? 8 : 0, qh, (float *)dev->static_scratch);
}

static fh_status ad_any(fh_device *dev, int kv_dtype, const float *q, const void *k, const void *v, int64_t kv_sh,
                        int64_t kv_st, int hq, int hkv, int d, float scale, const int *len_dev, int max_len, float *out,
                        int *splits_out, int len_host, int splits_req, bool out_f16, int heads_req, int waves_req,
                        bool q_f16, float *part_fixed) {
    const int gtot = hq / hkv;
    // any number of query heads per KV head: a workgroup takes 1, 2, 4 or 8 of them, whichever divides the group
    if (d != 128 || gtot < 1 || kv_st % 8 || kv_sh % 8) return FH_ERR_UNSUPPORTED;
    // query heads per workgroup: the arithmetic of a workgroup grows with them, the K and V reads do not; one
    // (the workgroups of a KV head then share the rows through the L2) measured best on MI355X for 4 heads per KV
    // head at contexts of some hundred keys: 256 workgroups instead of 64
    int G = dev->opt_attn_heads > 0 ? (int)dev->opt_attn_heads : 1;
    if (heads_req > 0) G = heads_req > gtot ? gtot : heads_req;
    while (G > 1 && (gtot % G || (G != 2 && G != 4 && G != 8))) G /= 2;
    // 8 wavefronts per workgroup instead of 16
    const bool w8 = (dev->opt_attn_waves == 8 || (dev->opt_attn_waves == 0 && waves_req == 8)) && G <= 8;
    // the one-pass kernel unless attn_kernel = 4 asks for the two-pass one (or 8 heads per workgroup are wanted)
    const bool one_pass = dev->opt_attn_kernel != 4 || part_fixed;
    if (part_fixed && G > 4) G = 4; // the one-pass kernel takes at most four query heads per workgroup
#define AD_ARGS dev, q, k, v, kv_sh, kv_st, hq, hkv, scale, len_dev, max_len, out, splits_out, gtot, len_host, splits_req, out_f16, one_pass, q_f16, part_fixed
#define AD_GO(TKV_)                                                                       \
    switch (G) {                                                                          \
    case 1: return w8 ? ad_launch<TKV_, 1, 8>(AD_ARGS) : ad_launch<TKV_, 1, 16>(AD_ARGS); \
    case 2: return w8 ? ad_launch<TKV_, 2, 8>(AD_ARGS) : ad_launch<TKV_, 2, 16>(AD_ARGS); \
    case 4: return w8 ? ad_launch<TKV_, 4, 8>(AD_ARGS) : ad_launch<TKV_, 4, 16>(AD_ARGS); \
    default: return w8 ? ad_launch<TKV_, 8, 8>(AD_ARGS) : ad_launch<TKV_, 8, 16>(AD_ARGS); \
    }
    if (kv_dtype == FH_F16) {
        AD_GO(fh_half)
    }
    AD_GO(float)
#undef AD_GO
#undef AD_ARGS
}

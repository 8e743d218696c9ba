// Attention of ONE query position against a long f16 KV cache, on the matrix cores: softmax(q . K^T * scale) . V
// for the G <= 16 query heads that share a KV head, head_dim 128.
// Reference: fusor-ml/fusor/src/composite/flash_attention.rs:58-236 (semantics, no mask for a single query:
// models/kalosm-llama/src/raw/mod.rs:969-972).
//
// The vector-ALU kernels of fh_attention_decode.hip spend about 130 lane operations per key and KV head (dot
// products, lane reductions, conversions); at sixteen thousand keys that arithmetic is as long as the transfer of the
// cache.  Here the query heads of a KV head are the 16 columns of v_mfma_f32_16x16x32_f16 (unused columns are zero):
//   scores  S^T (16 keys x 16 heads) = K (16 keys x 128) . Q^T          four products per 16 keys; the K operand
//           is the 16 bytes a lane loaded from the cache (lane (key i, g) holds d = 32 s + 8 g .. +7 of step s)
//   output  O^T (128 x 16 heads)    += V^T (16 d x 32 keys) . P^T       eight products per 32 keys; P^T is the
//           score accumulator, exponentiated, as it sits in the registers; V^T comes from the wavefront's own
//           LDS tile of V rows through the transposing load (ds_read_b64_tr_b16)
// so a wavefront spends about 140 instructions per 32 keys and the kernel is a stream of cache rows.
// grid (S parts, KV heads); chunk c of 32 keys belongs to part c mod S, and the wavefronts of a workgroup take the
// part's chunks in turn, each with its own running maximum, denominator and output; the next chunk of a wavefront
// is in flight (128 registers) while the current one is multiplied.  No barrier until the wavefronts merge at the
// end (LDS operations of one wavefront execute in order, and every wavefront reads only the tile it wrote).
// Partials as the other decode kernels write them: [head][part][128 weighted sums | max | denominator | 2 unused].
#include "fh_internal.h"

typedef _Float16 fh_half;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4))); // 16 bytes of a cache row as they were loaded

__device__ __forceinline__ float am_rows_max(float a) { // over the four 16-lane rows of the wavefront
    const uint32_t u = __float_as_uint(a);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = fmaxf(__uint_as_float(s16[0]), __uint_as_float(s16[1]));
    const uint32_t w = __float_as_uint(a);
    auto s32 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__uint_as_float(s32[0]), __uint_as_float(s32[1]));
}
__device__ __forceinline__ float am_rows_sum(float a) {
    const uint32_t u = __float_as_uint(a);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);
    const uint32_t w = __float_as_uint(a);
    auto s32 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(s32[0]) + __uint_as_float(s32[1]);
}
// keys k .. k+3 and k+16 .. k+19 of the dim this lane stands for (two transposing loads of 4 keys)
__device__ __forceinline__ half8 am_vt8(const fh_half *p, int row_stride) {
    const short4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p);
    const short4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)(p + 16 * row_stride));
    half8 r;
    __builtin_memcpy(&r, &a, 8);
    __builtin_memcpy((char *)&r + 8, &b, 8);
    return r;
}

template <int NWV>
__global__ __launch_bounds__(64 * NWV) void k_attn_decode_mfma(const void *__restrict__ qv, int q_f16, const fh_half *__restrict__ k,
                                                                const fh_half *__restrict__ v, int64_t kv_sh, int64_t kv_st,
                                                                int skv, float scale, int gtot, float *__restrict__ part) {
    constexpr int D = 128, VS = D + 16, CK = 32, DT = D / 16;
    // one V tile per wavefront; the same bytes hold the wavefronts' outputs for the merge at the end
    __shared__ __attribute__((aligned(16))) unsigned char s_raw[NWV * 16 * D * 4 > NWV * CK * VS * 2 ? NWV * 16 * D * 4 : NWV * CK * VS * 2];
    __shared__ float s_st[NWV * 16 * 2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, S = gridDim.x, kh = blockIdx.y, h0 = kh * gtot;
    fh_half *sv = (fh_half *)s_raw + wave * CK * VS;
    const fh_half *kb = k + kh * kv_sh + 8 * g, *vb = v + kh * kv_sh + 8 * g;

    // Q^T operand: lane (head i, g) holds d = 32 s + 8 g .. +7 of step s (zeros for the unused columns)
    half8 qf[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        fh_half t[8];
#pragma unroll
        for (int e = 0; e < 8; e++) t[e] = (fh_half)0.f;
        if (i < gtot) {
            if (q_f16) {
                const uint4 r = *(const uint4 *)((const fh_half *)qv + (int64_t)(h0 + i) * D + 32 * s + 8 * g);
                __builtin_memcpy(t, &r, 16);
            } else {
                const float *qp = (const float *)qv + (int64_t)(h0 + i) * D + 32 * s + 8 * g;
                const float4 a = *(const float4 *)qp, b = *(const float4 *)(qp + 4);
                t[0] = (fh_half)a.x; t[1] = (fh_half)a.y; t[2] = (fh_half)a.z; t[3] = (fh_half)a.w;
                t[4] = (fh_half)b.x; t[5] = (fh_half)b.y; t[6] = (fh_half)b.z; t[7] = (fh_half)b.w;
            }
        }
        __builtin_memcpy(&qf[s], t, 16);
    }
    const float sc2 = scale * 1.4426950408889634f; // scores in the log2 domain
    const int nct = (skv + CK - 1) / CK;            // chunks of the head
    const int nc = nct > split ? (nct - split + S - 1) / S : 0; // chunks of this part
    float m_run = -INFINITY, l_run = 0.f;
    floatx4 acc[DT];
#pragma unroll
    for (int t = 0; t < DT; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    u32x4 kr0[2][4], vr0[2][4], kr1[2][4], vr1[2][4]; // two buffers of [16-key block][step]
    auto issue = [&](u32x4 (&kr)[2][4], u32x4 (&vr)[2][4], int j) { // local chunk j of the part (past the end: the last row again, never used)
        const int row0 = CK * (j * S + split);
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            int row = row0 + 16 * blk + i;
            row = row < skv ? row : skv - 1;
            const fh_half *kp = kb + (int64_t)row * kv_st, *vp = vb + (int64_t)row * kv_st;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                kr[blk][s] = *(const u32x4 *)(kp + 32 * s);
                vr[blk][s] = *(const u32x4 *)(vp + 32 * s);
            }
        }
    };
    auto process = [&](const u32x4 (&kr)[2][4], const u32x4 (&vr)[2][4], int j) {
        const int row0 = CK * (j * S + split);
        // ---- scores of the two 16-key blocks: register r of block blk is key row0 + 16 blk + 4 g + r, column = head
        floatx4 st[2];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            st[blk] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; s++) {
                st[blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, kr[blk][s]), qf[s], st[blk], 0, 0, 0);
            }
        }
        // ---- V rows into the wavefront's LDS tile (a clamped row past the end holds live data and meets a zero weight)
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
            for (int s = 0; s < 4; s++) *(u32x4 *)(sv + (16 * blk + i) * VS + 32 * s + 8 * g) = vr[blk][s];
        // ---- mask the keys past the end (only the last chunk has any), running max over the chunk
        float mx = -INFINITY;
        if (row0 + CK > skv) {
#pragma unroll
            for (int blk = 0; blk < 2; blk++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (row0 + 16 * blk + 4 * g + r >= skv) st[blk][r] = -INFINITY;
        }
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
            for (int r = 0; r < 4; r++) mx = fmaxf(mx, st[blk][r]);
        mx = am_rows_max(mx) * sc2; // a chunk that is processed has at least one live key: finite
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        fh_half pt[8];
        float ps = 0.f;
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float p = __builtin_amdgcn_exp2f(fmaf(st[blk][r], sc2, -m_new));
                ps += p;
                pt[4 * blk + r] = (fh_half)p;
            }
        half8 pb; // k-slot (g, e): block e / 4, key 4 g + e % 4 - the order the two transposing loads deliver
        __builtin_memcpy(&pb, pt, 16);
        l_run = l_run * alpha + ps; // per lane: the four rows of a column are summed once, at the end
        m_run = m_new;
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int t = 0; t < DT; t++) acc[t] *= alpha;
        }
        // ---- O^T tile t (16 d x 16 heads) += V^T . P^T; source lane s of a 16-lane row addresses keys 4 g + s / 4,
        // d 16 t + 4 (s % 4) .. +3 and receives d 16 t + s of keys 4 g .. 4 g + 3 (then of keys 16 + 4 g .. +3)
        const fh_half *vp = sv + (4 * g + (i >> 2)) * VS + 4 * (i & 3);
#pragma unroll
        for (int t = 0; t < DT; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(am_vt8(vp + 16 * t, VS), pb, acc[t], 0, 0, 0);
    };
    // the wavefront's chunks: wave, wave + NWV, ...; two per trip, each requested one chunk ahead
    // (no branches around the requests - a wait after a branch waits for everything in flight: requests past the
    // end re-read the last live row and are dropped)
    issue(kr0, vr0, wave);
    for (int j = wave; j < nc; j += 2 * NWV) {
        issue(kr1, vr1, j + NWV);
        __builtin_amdgcn_sched_barrier(0); // the requests stay ahead of the arithmetic on the other chunk
        process(kr0, vr0, j);
        __builtin_amdgcn_sched_barrier(0);
        issue(kr0, vr0, j + 2 * NWV);
        __builtin_amdgcn_sched_barrier(0);
        if (j + NWV < nc) process(kr1, vr1, j + NWV);
        __builtin_amdgcn_sched_barrier(0);
    }
    // ---- merge the wavefronts: lane (head i, g) holds d = 16 t + 4 g + r of tile t
    l_run = am_rows_sum(l_run);
    __syncthreads(); // every wavefront is done with its V tile
    float *so = (float *)s_raw;
    if (i < gtot) {
#pragma unroll
        for (int t = 0; t < DT; t++)
            *(float4 *)(so + (wave * 16 + i) * D + 16 * t + 4 * g) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
        if (g == 0) {
            s_st[(wave * 16 + i) * 2] = m_run;
            s_st[(wave * 16 + i) * 2 + 1] = l_run;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < gtot * D; idx += 64 * NWV) {
        const int h = idx / D, dd = idx % D;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < NWV; w++) mx = fmaxf(mx, s_st[(w * 16 + h) * 2]);
        const float ref = mx == -INFINITY ? 0.f : mx;
        float a = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; w++) {
            const float f = __builtin_amdgcn_exp2f(s_st[(w * 16 + h) * 2] - ref);
            a = fmaf(so[(w * 16 + h) * D + dd], f, a);
            den = fmaf(s_st[(w * 16 + h) * 2 + 1], f, den);
        }
        float *pp = part + ((int64_t)(h0 + h) * S + split) * (D + 4);
        pp[dd] = a;
        if (dd == 0) {
            pp[D] = mx * 0.6931471805599453f; // the merge works with natural exponents
            pp[D + 1] = den;
        }
    }
}

// Partials of `splits` parts per head into `part` ([hq][splits][132] floats).  FH_ERR_UNSUPPORTED for shapes this
// kernel is not written for (the caller keeps the vector-ALU kernels).
fh_status fh_attention_decode_mfma(fh_device *dev, const void *q, bool q_f16, const void *k, const void *v,
                                   int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale, int skv,
                                   int splits, float *part) {
    const int gtot = hkv > 0 ? hq / hkv : 0;
    if (d != 128 || gtot < 1 || gtot > 16 || hq % hkv || kv_st % 8 || kv_sh % 8 || skv < 1 || splits < 1 || splits > 128 ||
        hkv > 65535)
        return FH_ERR_UNSUPPORTED;
    k_attn_decode_mfma<4><<<dim3((unsigned)splits, (unsigned)hkv), dim3(256), 0, dev->stream>>>(
        q, q_f16 ? 1 : 0, (const fh_half *)k, (const fh_half *)v, kv_sh, kv_st, skv, scale, gtot, part);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

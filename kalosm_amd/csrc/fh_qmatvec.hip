// Decode-side quantized matmul (1 <= m <= 16 activation rows): y[m, n] = sum_k x[m, k] * deq(W)[n, k].
// Reference: fusor-ml/fusor/src/lib.rs:1132-1223 -> fusor-ml/cpu/src/quantized.rs:246-675.
//
// Two kernel families:
//   k_qmv_generic  one wavefront per weight row, per-element decode, f32 FMA.  Any format, any m.
//                  The reference path restated for the GPU; also the cross-check of the fast kernels.
//   k_qmv_*_mfma   HBM-bandwidth kernels.  A wavefront owns a tile of 16 weight rows and a range of
//                  k.  The 4-bit codes are turned into f16 SUBNORMAL integers (code * 2^-24) with
//                  one AND per two codes and fed to v_mfma_f32_16x16x32_f16 as the B operand; the A
//                  operand holds the activations as an exact two-term f16 split (hi + lo) of the
//                  block-normalised f32 values.  Products are exact; scales are applied in f32 on
//                  the 16x16 accumulator whose columns are the lane's own weight row.  The min term
//                  of Q4_K uses the factorisation  y = d*sum_j sc_j*(q.x)_j - dmin*sum_j m_j*(sum x)_j.
#include "fh_blocks.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float fh_silu(float x) { return x / (__expf(-x) + 1.0f); }

// ------------------------------------------------------------------------------ generic
template <int T, int EPI>
__global__ __launch_bounds__(256) void k_qmv_generic(QView q, const float *__restrict__ x, int m,
                                                      float *__restrict__ y, const float *__restrict__ ea,
                                                      const float *__restrict__ eb) {
    const int MB = 4;
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
    int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= nout) return;
    int m0 = blockIdx.y * MB;
    float acc[MB] = {0.f, 0.f, 0.f, 0.f}, acc2[MB] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t k = lane; k < q.k; k += 64) {
        float w = deq_elem<T>(q, row, k);
        float w2 = EPI == FH_EPI_SWIGLU ? deq_elem<T>(q, row + nout, k) : 0.f;
#pragma unroll
        for (int i = 0; i < MB; i++)
            if (m0 + i < m) {
                float xv = x[(int64_t)(m0 + i) * q.k + k];
                acc[i] = fmaf(xv, w, acc[i]);
                if (EPI == FH_EPI_SWIGLU) acc2[i] = fmaf(xv, w2, acc2[i]);
            }
    }
#pragma unroll
    for (int i = 0; i < MB; i++) {
        float v = wave_sum(acc[i]);
        float v2 = EPI == FH_EPI_SWIGLU ? wave_sum(acc2[i]) : 0.f;
        if (lane == 0 && m0 + i < m) {
            int64_t o = (int64_t)(m0 + i) * nout + row;
            if (EPI == FH_EPI_ADD2) v = (v + ea[o]) + eb[o];
            if (EPI == FH_EPI_SWIGLU) v = (v / (expf(-v) + 1.0f)) * v2;
            y[o] = v;
        }
    }
}

template <int T>
static fh_status launch_generic(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                                const float *b) {
    int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    dim3 grid((unsigned)((nout + 3) / 4), (unsigned)((m + 3) / 4)), block(256);
    QView v = fh_view(q);
    hipStream_t s = q->dev->stream;
    if (epi == FH_EPI_NONE) k_qmv_generic<T, FH_EPI_NONE><<<grid, block, 0, s>>>(v, x, m, y, a, b);
    else if (epi == FH_EPI_ADD2) k_qmv_generic<T, FH_EPI_ADD2><<<grid, block, 0, s>>>(v, x, m, y, a, b);
    else k_qmv_generic<T, FH_EPI_SWIGLU><<<grid, block, 0, s>>>(v, x, m, y, a, b);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ activation staging
// x [m, k] f32 -> operand image for the MFMA kernels whose step covers 32 consecutive k:
//   xp   halfs, index (((s*4 + g)*nc + col)*8 + h): step s = k/32, g = (k%32)/8, col = 2*row + part
//        (part 0 = hi, 1 = lo), h = slot of k%8 under the byte order [0,2,1,3,4,6,5,7] that the
//        nibble masks 0x000F000F / (>>8) produce.
//   sx   f32 [m, k/32]: sum of the ORIGINAL x over each 32 (the min / centre terms)
//   fs   f32 [m, ceil(k/256)]: 2^(24 - e) where 2^e is the power of two that normalised the
//        256-group to [2^14, 2^15) before the split (undoes both it and the 2^-24 of the codes)
// One wavefront per (row, 256-group); lane owns 4 consecutive k.
__global__ __launch_bounds__(256) void k_act_prep32(const float *__restrict__ x, int m, int k, int nc,
                                                     _Float16 *__restrict__ xp, float *__restrict__ sx,
                                                     float *__restrict__ fs) {
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int k256 = (k + 255) >> 8;
    int64_t gid = (int64_t)blockIdx.x * 4 + wave;
    if (gid >= (int64_t)m * k256) return;
    int row = (int)(gid / k256), b = (int)(gid % k256);
    int k0 = b * 256 + lane * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (k0 < k) v = *(const float4 *)(x + (int64_t)row * k + k0); // k % 32 == 0, so a lane is all in or all out
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    int e = 0;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex); // amax = f * 2^ex, f in [0.5, 1)  ->  floor(log2) = ex - 1
        e = 14 - (ex - 1);
        e = e > 100 ? 100 : (e < -100 ? -100 : e);
    }
    float sc = ldexpf(1.0f, e);
    float xs[4] = {v.x * sc, v.y * sc, v.z * sc, v.w * sc};
    _Float16 hi[4], lo[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        hi[i] = (_Float16)xs[i];
        lo[i] = (_Float16)(xs[i] - (float)hi[i]);
    }
    if (k0 < k) {
        int s = k0 >> 5, g = (k0 & 31) >> 3, half = (k0 & 7) >> 2; // half: slots 0..3 or 4..7
        int64_t base = (((int64_t)s * 4 + g) * nc + 2 * row) * 8 + half * 4;
        _Float16 oh[4] = {hi[0], hi[2], hi[1], hi[3]};
        _Float16 ol[4] = {lo[0], lo[2], lo[1], lo[3]};
        uint2 ph, pl;
        __builtin_memcpy(&ph, oh, 8);
        __builtin_memcpy(&pl, ol, 8);
        *(uint2 *)(xp + base) = ph;     // column 2*row     (hi)
        *(uint2 *)(xp + base + 8) = pl; // column 2*row + 1 (lo)
    }
    float s4 = (v.x + v.y) + (v.z + v.w);
    s4 += __shfl_xor(s4, 1, 64);
    s4 += __shfl_xor(s4, 2, 64);
    s4 += __shfl_xor(s4, 4, 64);
    if ((lane & 7) == 0 && k0 < k) sx[(int64_t)row * (k >> 5) + (k0 >> 5)] = s4;
    if (lane == 0) fs[(int64_t)row * k256 + b] = ldexpf(1.0f, 24 - e);
}

// ------------------------------------------------------------------------------ Q4_K MFMA
// Workgroup = S wavefronts on one 16-row tile (two tiles with the SwiGLU epilogue); wavefront w
// takes blocks [w*per, (w+1)*per).  Lane l: j = l & 15 is its weight row inside the tile (B operand
// column, and the accumulator column), g = l >> 4 its k-group inside a 32-step.
// NC = staged activation columns = 2 * rows (hi, lo per row), NC in {2, 4}.
template <int NC, int EPI>
__global__ __launch_bounds__(1024) void k_qmv_q4k_mfma(QView q, const uint4 *__restrict__ xp,
                                                        const float *__restrict__ sx, const float *__restrict__ fs,
                                                        float *__restrict__ y, const float *__restrict__ ea,
                                                        const float *__restrict__ eb, int S) {
    constexpr int M = NC / 2;
    extern __shared__ uint4 lds[];
    const int kb = (int)q.kb, k32 = kb * 8;
    uint4 *l_xp = lds;                              // k32 * 4 * NC
    float *l_sx = (float *)(lds + k32 * 4 * NC);    // M * k32
    float *l_fs = l_sx + M * k32;                   // M * kb
    float *l_red = l_fs + M * kb;                   // S * 2 * M * 16
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, g = lane >> 4;
    for (int i = tid; i < k32 * 4 * NC; i += blockDim.x) l_xp[i] = xp[i];
    for (int i = tid; i < M * k32; i += blockDim.x) l_sx[i] = sx[i];
    for (int i = tid; i < M * kb; i += blockDim.x) l_fs[i] = fs[i];
    __syncthreads();

    const int per = (kb + S - 1) / S;
    const int b0 = wave * per, b1 = min(kb, b0 + per);
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t tiles_out = (EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n + 15) / 16; // exact /16 for SwiGLU (host checks)
    const uint32_t LO = 0x000F000Fu, HI = 0x00F000F0u;
    float outv[NT][M];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int64_t tile = (int64_t)blockIdx.x + (int64_t)t * tiles_out;
        const uint8_t *rec = q.data + (tile * q.recs + b0) * 2304;
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
        float mins[M];
#pragma unroll
        for (int i = 0; i < M; i++) mins[i] = 0.f;
        for (int b = b0; b < b1; b++, rec += 2304) {
            const uint4 h = *(const uint4 *)(rec + 16 * j);
            const uint4 qa = *(const uint4 *)(rec + 256 + lane * 16);
            const uint4 qb = *(const uint4 *)(rec + 1280 + lane * 16);
            const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
            const float d16 = d * 0.0625f;
            const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
            const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
            floatx4 accb = {0.f, 0.f, 0.f, 0.f};
            const uint4 *xs = l_xp + ((b * 8) * 4 + g) * NC + j; // + step * 4 * NC
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const uint4 w = p ? qb : qa;
                const uint32_t scw = p ? sc_hi : sc_lo;
#pragma unroll
                for (int u = 0; u < 2; u++) { // u = 0: dwords x,y (chunk 2p)   u = 1: dwords z,w (chunk 2p+1)
                    const uint32_t w0 = u ? w.z : w.x, w1 = u ? w.w : w.y;
                    const uint32_t w0s = w0 >> 8, w1s = w1 >> 8;
#pragma unroll
                    for (int hn = 0; hn < 2; hn++) { // low nibbles (sub-block 4p+2u), high nibbles (4p+2u+1)
                        const uint32_t msk = hn ? HI : LO;
                        uint4 bo = make_uint4(w0 & msk, w0s & msk, w1 & msk, w1s & msk);
                        const int jj = 2 * u + hn; // sub-block within the p half
                        uint4 ao = make_uint4(0, 0, 0, 0);
                        if (j < NC) ao = xs[(4 * p + jj) * 4 * NC];
                        half8 av, bv;
                        __builtin_memcpy(&av, &ao, 16);
                        __builtin_memcpy(&bv, &bo, 16);
                        floatx4 z = {0.f, 0.f, 0.f, 0.f};
                        floatx4 dd = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, z, 0, 0, 0);
                        const float scf = (float)((scw >> (8 * jj)) & 0xFFu) * (hn ? d16 : d);
                        accb[0] = fmaf(dd[0], scf, accb[0]);
                        accb[1] = fmaf(dd[1], scf, accb[1]);
                        if (NC > 2) {
                            accb[2] = fmaf(dd[2], scf, accb[2]);
                            accb[3] = fmaf(dd[3], scf, accb[3]);
                        }
                    }
                }
            }
            // undo the block normalisation (and the 2^-24 of the codes); only g == 0 lanes carry data
#pragma unroll
            for (int r = 0; r < NC; r++) acc[r] = fmaf(accb[r], l_fs[(r >> 1) * kb + b], acc[r]);
            // min term: lane group g covers sub-blocks 2g, 2g+1
            const uint32_t mw = (g & 2) ? mn_hi : mn_lo;
            const int sh = (g & 1) * 16;
            const float ma = (float)((mw >> sh) & 0xFFu) * dmin, mb = (float)((mw >> (sh + 8)) & 0xFFu) * dmin;
#pragma unroll
            for (int i = 0; i < M; i++) {
                const float2 s2 = *(const float2 *)(l_sx + i * k32 + b * 8 + 2 * g);
                mins[i] = fmaf(ma, s2.x, mins[i]);
                mins[i] = fmaf(mb, s2.y, mins[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < M; i++) {
            float mt = mins[i];
            mt += __shfl_xor(mt, 16, 64);
            mt += __shfl_xor(mt, 32, 64);
            outv[t][i] = (acc[2 * i] + acc[2 * i + 1]) - mt; // meaningful in lanes 0..15 (g == 0)
        }
    }
    // cross-wavefront reduction over the k ranges
    if (lane < 16) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int i = 0; i < M; i++) l_red[((wave * NT + t) * M + i) * 16 + lane] = outv[t][i];
    }
    __syncthreads();
    if (tid < 16 * M) {
        const int i = tid >> 4, jr = tid & 15;
        float v[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float s = 0.f;
            for (int w = 0; w < S; w++) s += l_red[((w * NT + t) * M + i) * 16 + jr];
            v[t] = s;
        }
        const int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
        const int64_t row = (int64_t)blockIdx.x * 16 + jr;
        if (row < nout) {
            const int64_t o = (int64_t)i * nout + row;
            float r = v[0];
            if (EPI == FH_EPI_ADD2) r = (r + ea[o]) + eb[o];
            if (EPI == FH_EPI_SWIGLU) r = (r / (__expf(-r) + 1.0f)) * v[NT - 1];
            y[o] = r;
        }
    }
}

static size_t q4k_lds_bytes(int64_t kb, int nc, int S, int nt) {
    int m = nc / 2;
    return (size_t)kb * 8 * 4 * nc * 16 + (size_t)m * kb * 8 * 4 + (size_t)m * kb * 4 + (size_t)S * nt * m * 16 * 4;
}

static fh_status launch_q4k_mfma(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                                 const float *b) {
    fh_device *dev = q->dev;
    const int nc = 2 * m;
    const int64_t k = q->k, kb = q->kb;
    const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int nt = epi == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t tiles = (nout + 15) / 16;
    // staging buffer: xp | sx | fs
    size_t xp_bytes = (size_t)(k / 32) * 4 * nc * 16, sx_bytes = (size_t)m * (k / 32) * 4, fs_bytes = (size_t)m * kb * 4;
    size_t sx_off = (xp_bytes + 255) & ~(size_t)255, fs_off = (sx_off + sx_bytes + 255) & ~(size_t)255;
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, fs_off + fs_bytes + 256));
    uint8_t *ab = (uint8_t *)dev->act_buf;
    {
        int64_t waves = (int64_t)m * kb;
        k_act_prep32<<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, dev->stream>>>(
            x, m, (int)k, nc, (_Float16 *)ab, (float *)(ab + sx_off), (float *)(ab + fs_off));
        FH_HIP(hipGetLastError());
    }
    // wavefronts per tile: enough to put ~12 wavefronts on each CU, at least one block each
    int S = dev->opt_matvec_waves > 0 ? (int)dev->opt_matvec_waves : 0;
    if (!S) {
        int64_t want = ((int64_t)dev->compute_units * 12 + tiles - 1) / tiles;
        S = (int)(want < 1 ? 1 : want);
        if (S > 16) S = 16;
        if (nt == 2 && S > 8) S = 8;
    }
    if (S > kb) S = (int)kb;
    if (S > 16) S = 16;
    size_t lds = q4k_lds_bytes(kb, nc, S, nt);
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED; // caller falls back
    dim3 grid((unsigned)tiles), block(64 * S);
    QView v = fh_view(q);
    const uint4 *xp = (const uint4 *)ab;
    const float *sx = (const float *)(ab + sx_off), *fs = (const float *)(ab + fs_off);
#define FH_Q4K_LAUNCH(NC_, EPI_)                                                                              \
    do {                                                                                                      \
        static bool attr_done = false;                                                                        \
        if (!attr_done) {                                                                                     \
            FH_HIP(hipFuncSetAttribute((const void *)k_qmv_q4k_mfma<NC_, EPI_>,                               \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));              \
            attr_done = true;                                                                                 \
        }                                                                                                     \
        k_qmv_q4k_mfma<NC_, EPI_><<<grid, block, lds, dev->stream>>>(v, xp, sx, fs, y, a, b, S);              \
    } while (0)
    if (nc == 2) {
        if (epi == FH_EPI_NONE) FH_Q4K_LAUNCH(2, FH_EPI_NONE);
        else if (epi == FH_EPI_ADD2) FH_Q4K_LAUNCH(2, FH_EPI_ADD2);
        else FH_Q4K_LAUNCH(2, FH_EPI_SWIGLU);
    } else {
        if (epi == FH_EPI_NONE) FH_Q4K_LAUNCH(4, FH_EPI_NONE);
        else if (epi == FH_EPI_ADD2) FH_Q4K_LAUNCH(4, FH_EPI_ADD2);
        else FH_Q4K_LAUNCH(4, FH_EPI_SWIGLU);
    }
#undef FH_Q4K_LAUNCH
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ dispatch
fh_status fh_launch_qmatvec(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                            const float *b) {
    fh_device *dev = q->dev;
    if (epi == FH_EPI_SWIGLU) FH_REQUIRE(q->n % 32 == 0, "SwiGLU epilogue needs n %% 32 == 0 (n = %lld)", (long long)q->n);
    int kernel = (int)dev->opt_matvec_kernel;
    if (kernel != 1 && q->type == FH_Q4_K && m <= 2) {
        fh_status st = launch_q4k_mfma(q, x, m, y, epi, a, b);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    switch (q->type) {
    case FH_Q4_0: return launch_generic<FH_Q4_0>(q, x, m, y, epi, a, b);
    case FH_Q8_0: return launch_generic<FH_Q8_0>(q, x, m, y, epi, a, b);
    case FH_Q4_K: return launch_generic<FH_Q4_K>(q, x, m, y, epi, a, b);
    case FH_Q6_K: return launch_generic<FH_Q6_K>(q, x, m, y, epi, a, b);
    }
    FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported type %u", q->type);
}

static fh_status qmm_check(const fh_qmatrix *q, const void *x, int m, const void *y) {
    FH_REQUIRE(q && x && y, "NULL argument");
    FH_REQUIRE(m >= 1, "m = %d", m);
    return FH_OK;
}

extern "C" fh_status fh_qmatmul(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev) {
    FH_TRY(qmm_check(q, x_dev, m, y_dev));
    if (m > 16 && q->dev->opt_matmul_kernel != 1) return fh_launch_qmatmul_tile(q, x_dev, 0, m, y_dev);
    return fh_launch_qmatvec(q, x_dev, m, y_dev, FH_EPI_NONE, nullptr, nullptr);
}

extern "C" fh_status fh_qmatmul_add2(const fh_qmatrix *q, const float *x_dev, int32_t m, const float *a_dev,
                                     const float *b_dev, float *y_dev) {
    FH_TRY(qmm_check(q, x_dev, m, y_dev));
    FH_REQUIRE(a_dev && b_dev, "NULL residual");
    return fh_launch_qmatvec(q, x_dev, m, y_dev, FH_EPI_ADD2, a_dev, b_dev);
}

extern "C" fh_status fh_qmatmul_swiglu(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev) {
    FH_TRY(qmm_check(q, x_dev, m, y_dev));
    return fh_launch_qmatvec(q, x_dev, m, y_dev, FH_EPI_SWIGLU, nullptr, nullptr);
}

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

// ------------------------------------------------------------------------------ Q4_K MFMA
// Work split: a workgroup owns T tiles of 16 weight rows (2T with the SwiGLU epilogue: T gate tiles and
// the T matching up tiles); its S wavefronts split k, wavefront w taking blocks [w*per, (w+1)*per) one
// 256-block per round.  Lane l: j = l & 15 is its weight row inside a tile (B operand column and
// accumulator column), g = l >> 4 its k-group inside a 32-wide MFMA step.
//
// Per round a wavefront
//   1. has the T x 2304 B of the NEXT round already in flight (register double buffer),
//   2. stages its 256 activations per row: each 32-group is normalised by a power of two to
//      [2^14, 2^15), split exactly into f16 hi + lo, and written to wavefront-private LDS in operand
//      order (step s = k/32, g = (k%32)/8, slots in the byte order [0,2,1,3,4,6,5,7] that the nibble
//      masks produce); the group sums of the original x and the factors 2^(24-e) go beside them,
//   3. runs 8 MFMA steps per tile (one per sub-block) and applies d * sc_j * 2^(24-e_j) in f32.
// M = activation rows (1 or 2); operand columns are (hi, lo) per row.
struct Q4KRegs {
    uint4 h, qa, qb;
};

template <int M, int T, int EPI>
__global__ __launch_bounds__((T * (EPI == FH_EPI_SWIGLU ? 2 : 1)) >= 2 ? 512 : 1024) void k_qmv_q4k_mfma(QView q, const float *__restrict__ x, float *__restrict__ y,
                                                        const float *__restrict__ ea, const float *__restrict__ eb,
                                                        int S, int per) {
    constexpr int NC = 2 * M;
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1;
    constexpr int TT = T * NT;
    constexpr int WLDS = 32 * NC + 4 * M; // uint4 per wavefront: operand image + (sums, factors)
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, g = lane >> 4;
    uint4 *w_xp = lds + wave * WLDS;
    float *w_sf = (float *)(w_xp + 32 * NC); // [m][0..7] group sums, [m][8..15] factors
    float *l_red = (float *)(lds + S * WLDS); // [S][TT][M][16]
    const int kb = (int)q.kb, K = (int)q.k;
    const int b0 = wave * per;
    const int nb = min(per, kb - b0); // <= 0 for surplus wavefronts
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
    const int64_t tiles_out = (nout + 15) / 16;

    const uint8_t *tb[TT];
    bool tv[TT];
#pragma unroll
    for (int t = 0; t < TT; t++) {
        const int64_t to = (int64_t)blockIdx.x * T + (t % T);
        tv[t] = to < tiles_out;
        const int64_t tile = to + (int64_t)(t / T) * (nout / 16); // up tiles follow the gate tiles (n % 32 == 0)
        tb[t] = q.data + (tile * q.recs + b0) * 2304;
    }
    Q4KRegs cur[TT], nxt[TT];
    float4 xc[M], xn[M];
    auto loadw = [&](Q4KRegs *w, int r) {
#pragma unroll
        for (int t = 0; t < TT; t++) {
            if (tv[t]) {
                const uint8_t *rec = tb[t] + (int64_t)r * 2304;
                w[t].h = *(const uint4 *)(rec + 16 * j);
                w[t].qa = *(const uint4 *)(rec + 256 + lane * 16);
                w[t].qb = *(const uint4 *)(rec + 1280 + lane * 16);
            } else {
                w[t].h = w[t].qa = w[t].qb = make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto loadx = [&](float4 *xv, int r) {
#pragma unroll
        for (int i = 0; i < M; i++) xv[i] = *(const float4 *)(x + (int64_t)i * K + (int64_t)(b0 + r) * 256 + lane * 4);
    };
    float acc[TT][NC], mins[TT][M];
#pragma unroll
    for (int t = 0; t < TT; t++) {
#pragma unroll
        for (int i = 0; i < NC; i++) acc[t][i] = 0.f;
#pragma unroll
        for (int i = 0; i < M; i++) mins[t][i] = 0.f;
    }
    if (nb > 0) {
        loadw(cur, 0);
        loadx(xc, 0);
    }
    const uint32_t LO = 0x000F000Fu, HI = 0x00F000F0u;
    for (int r = 0; r < nb; r++) {
        if (r + 1 < nb) {
            loadw(nxt, r + 1);
            loadx(xn, r + 1);
        }
        // ---- stage the activations of this block (lane owns k = 4*lane .. 4*lane+3)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
        for (int i = 0; i < M; i++) {
            const float4 v = xc[i];
            float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
            amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
            int e = 0;
            if (amax > 0.f && amax < INFINITY) {
                int ex;
                (void)frexpf(amax, &ex); // amax = f * 2^ex, f in [0.5, 1)
                e = 15 - ex;
                e = e > 100 ? 100 : (e < -100 ? -100 : e);
            }
            const float sc = ldexpf(1.0f, e);
            const float xs[4] = {v.x * sc, v.y * sc, v.z * sc, v.w * sc};
            _Float16 hi[4], lo[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                hi[c] = (_Float16)xs[c];
                lo[c] = (_Float16)(xs[c] - (float)hi[c]);
            }
            const _Float16 oh[4] = {hi[0], hi[2], hi[1], hi[3]}, ol[4] = {lo[0], lo[2], lo[1], lo[3]};
            uint2 ph, pl;
            __builtin_memcpy(&ph, oh, 8);
            __builtin_memcpy(&pl, ol, 8);
            const int s = lane >> 3, gg = (lane >> 1) & 3, half = lane & 1;
            uint2 *dst = (uint2 *)(w_xp + (s * 4 + gg) * NC + 2 * i);
            dst[half] = ph;     // column 2i   (hi)
            dst[2 + half] = pl; // column 2i+1 (lo)
            float s4 = (v.x + v.y) + (v.z + v.w);
            s4 += __shfl_xor(s4, 1, 64);
            s4 += __shfl_xor(s4, 2, 64);
            s4 += __shfl_xor(s4, 4, 64);
            if ((lane & 7) == 0) {
                w_sf[i * 16 + s] = s4;
                w_sf[i * 16 + 8 + s] = ldexpf(1.0f, 24 - e);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        // ---- operands shared by the T tiles
        half8 av[8];
#pragma unroll
        for (int st = 0; st < 8; st++) {
            uint4 ao = make_uint4(0, 0, 0, 0);
            if (j < NC) ao = w_xp[(st * 4 + g) * NC + j];
            __builtin_memcpy(&av[st], &ao, 16);
        }
        float fac[M][8], sxa[M], sxb[M];
#pragma unroll
        for (int i = 0; i < M; i++) {
            const float4 f0 = *(const float4 *)(w_sf + i * 16 + 8), f1 = *(const float4 *)(w_sf + i * 16 + 12);
            fac[i][0] = f0.x; fac[i][1] = f0.y; fac[i][2] = f0.z; fac[i][3] = f0.w;
            fac[i][4] = f1.x; fac[i][5] = f1.y; fac[i][6] = f1.z; fac[i][7] = f1.w;
            const float2 s2 = *(const float2 *)(w_sf + i * 16 + 2 * g);
            sxa[i] = s2.x;
            sxb[i] = s2.y;
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint4 h = cur[t].h;
            const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
            const float d16 = d * 0.0625f;
            const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
            const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const uint4 w = p ? cur[t].qb : cur[t].qa;
                const uint32_t scw = p ? sc_hi : sc_lo;
#pragma unroll
                for (int u = 0; u < 2; u++) { // dwords x,y = chunk 2p; dwords z,w = chunk 2p+1
                    const uint32_t w0 = u ? w.z : w.x, w1 = u ? w.w : w.y;
                    const uint32_t w0s = w0 >> 8, w1s = w1 >> 8;
#pragma unroll
                    for (int hn = 0; hn < 2; hn++) { // low nibbles = sub-block 4p+2u, high nibbles = 4p+2u+1 (x16)
                        const uint32_t msk = hn ? HI : LO;
                        const uint4 bo = make_uint4(w0 & msk, w0s & msk, w1 & msk, w1s & msk);
                        half8 bv;
                        __builtin_memcpy(&bv, &bo, 16);
                        const int jj = 2 * u + hn, sb = 4 * p + jj;
                        const floatx4 z = {0.f, 0.f, 0.f, 0.f};
                        const floatx4 dd = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[sb], bv, z, 0, 0, 0);
                        const float scf = (float)((scw >> (8 * jj)) & 0xFFu) * (hn ? d16 : d);
#pragma unroll
                        for (int i = 0; i < M; i++) {
                            const float tm = scf * fac[i][sb];
                            acc[t][2 * i] = fmaf(dd[2 * i], tm, acc[t][2 * i]);
                            acc[t][2 * i + 1] = fmaf(dd[2 * i + 1], tm, acc[t][2 * i + 1]);
                        }
                    }
                }
            }
            // min term: lane group g covers sub-blocks 2g, 2g+1
            const uint32_t mw = (g & 2) ? mn_hi : mn_lo;
            const int sh = (g & 1) * 16;
            const float ma = (float)((mw >> sh) & 0xFFu) * dmin, mb = (float)((mw >> (sh + 8)) & 0xFFu) * dmin;
#pragma unroll
            for (int i = 0; i < M; i++) {
                mins[t][i] = fmaf(ma, sxa[i], mins[t][i]);
                mins[t][i] = fmaf(mb, sxb[i], mins[t][i]);
            }
        }
#pragma unroll
        for (int t = 0; t < TT; t++) cur[t] = nxt[t];
#pragma unroll
        for (int i = 0; i < M; i++) xc[i] = xn[i];
    }
    // ---- reduce over the k ranges of the S wavefronts
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int i = 0; i < M; i++) {
            float mt = mins[t][i];
            mt += __shfl_xor(mt, 16, 64);
            mt += __shfl_xor(mt, 32, 64);
            const float v = (acc[t][2 * i] + acc[t][2 * i + 1]) - mt; // meaningful in lanes 0..15
            if (lane < 16) l_red[((wave * TT + t) * M + i) * 16 + lane] = v;
        }
    __syncthreads();
    if (tid < T * M * 16) {
        const int t = tid / (M * 16), i = (tid / 16) % M, jr = tid & 15;
        float v0 = 0.f, v1 = 0.f;
        for (int w = 0; w < S; w++) {
            v0 += l_red[((w * TT + t) * M + i) * 16 + jr];
            if (NT == 2) v1 += l_red[((w * TT + t + T) * M + i) * 16 + jr];
        }
        const int64_t row = ((int64_t)blockIdx.x * T + t) * 16 + jr;
        if (row < nout) {
            const int64_t o = (int64_t)i * nout + row;
            float r = v0;
            if (EPI == FH_EPI_ADD2) r = (r + ea[o]) + eb[o];
            if (EPI == FH_EPI_SWIGLU) r = (r / (__expf(-r) + 1.0f)) * v1;
            y[o] = r;
        }
    }
}

template <int M, int T>
static fh_status launch_q4k_t(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b,
                              int S, int per, unsigned grid, size_t lds) {
    hipStream_t st = q->dev->stream;
    QView v = fh_view(q);
#define FH_Q4K_LAUNCH(EPI_)                                                                                     \
    do {                                                                                                        \
        FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmv_q4k_mfma<M, T, EPI_>, 160 * 1024));                    \
        k_qmv_q4k_mfma<M, T, EPI_><<<dim3(grid), dim3(64 * S), lds, st>>>(v, x, y, a, b, S, per);                \
    } while (0)
    if (epi == FH_EPI_NONE) FH_Q4K_LAUNCH(FH_EPI_NONE);
    else if (epi == FH_EPI_ADD2) FH_Q4K_LAUNCH(FH_EPI_ADD2);
    else FH_Q4K_LAUNCH(FH_EPI_SWIGLU);
#undef FH_Q4K_LAUNCH
    FH_HIP(hipGetLastError());
    return FH_OK;
}

static fh_status launch_q4k_mfma(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                                 const float *b) {
    fh_device *dev = q->dev;
    const int64_t kb = q->kb;
    const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int nt = epi == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t tiles = (nout + 15) / 16;
    int T = (int)dev->opt_matvec_tiles;
    if (T != 1 && T != 2 && T != 4) T = tiles >= 1024 ? 4 : (tiles >= 512 ? 2 : 1);
    if (nt == 2 && T == 4) T = 2; // at most 4 tile streams per wavefront
    const int smax = T * nt >= 2 ? 8 : 16; // the multi-tile variants keep two register sets of T tiles
    int S = dev->opt_matvec_waves > 0 ? (int)dev->opt_matvec_waves : smax;
    if (S > smax) S = smax;
    if (S > kb) S = (int)kb;
    const int per = (int)((kb + S - 1) / S);
    S = (int)((kb + per - 1) / per);
    const int nc = 2 * m;
    size_t lds = (size_t)S * (32 * nc + 4 * m) * 16 + (size_t)S * T * nt * m * 16 * 4;
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED;
    unsigned grid = (unsigned)((tiles + T - 1) / T);
    if (m == 1) {
        if (T == 1) return launch_q4k_t<1, 1>(q, x, y, epi, a, b, S, per, grid, lds);
        if (T == 2) return launch_q4k_t<1, 2>(q, x, y, epi, a, b, S, per, grid, lds);
        return launch_q4k_t<1, 4>(q, x, y, epi, a, b, S, per, grid, lds);
    }
    if (T == 1) return launch_q4k_t<2, 1>(q, x, y, epi, a, b, S, per, grid, lds);
    if (T == 2) return launch_q4k_t<2, 2>(q, x, y, epi, a, b, S, per, grid, lds);
    return launch_q4k_t<2, 4>(q, x, y, epi, a, b, S, per, grid, lds);
}

// ------------------------------------------------------------------------------ dispatch
fh_status fh_launch_qmatvec(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                            const float *b) {
    fh_device *dev = q->dev;
    if (epi == FH_EPI_SWIGLU) FH_REQUIRE(q->n % 32 == 0, "SwiGLU epilogue needs n %% 32 == 0 (n = %lld)", (long long)q->n);
    int kernel = (int)dev->opt_matvec_kernel;
    if (kernel == 4 && fh_qmatvec_batch_supports(q, m, epi)) return fh_launch_qmatvec_batch(q, x, m, y, epi, a, b);
    if (kernel != 1 && kernel != 3 && (q->type == FH_Q4_K || q->type == FH_Q5_K || ((q->type == FH_Q4_0 || q->type == FH_Q8_0 || q->type == FH_Q5_0) && q->k % 256 == 0)) && m == 1) {
        fh_status st = fh_launch_q4k_m1(q, x, y, epi, a, b);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    // the 5-bit formats have the single-row kernel only: a few rows are a launch each (10 us a row against 110 - 640 us
    // for 2 .. 16 rows through the per-element kernel at 14336 x 4096)
    if (kernel != 1 && kernel != 3 && (q->type == FH_Q5_K || q->type == FH_Q5_0) && q->k % 256 == 0 && m >= 2 && m <= 16) {
        const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
        fh_status st = FH_OK;
        for (int r = 0; r < m && st == FH_OK; r++)
            st = fh_launch_q4k_m1(q, x + (int64_t)r * q->k, y + (int64_t)r * nout, epi, a ? a + (int64_t)r * nout : nullptr,
                                  b ? b + (int64_t)r * nout : nullptr);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    if (kernel == 0 && q->type != FH_Q6_K && !fh_single_row_only(q->type) && m >= 2 && m <= 4 && dev->opt_matvec_rows != 1) {
        fh_status st = fh_launch_q4k_rows(q, x, m, y, epi, a, b);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    if (kernel != 1 && q->type == FH_Q6_K && m == 1) {
        fh_status st = fh_launch_q6k_m1(q, x, y, epi, a, b);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    if (kernel == 0 && fh_qmatvec_batch_supports(q, m, epi)) return fh_launch_qmatvec_batch(q, x, m, y, epi, a, b);
    if (kernel != 1 && q->type == FH_Q4_K && m <= 2) {
        fh_status st = launch_q4k_mfma(q, x, m, y, epi, a, b);
        if (st != FH_ERR_UNSUPPORTED) return st;
    }
    switch (q->type) {
    case FH_Q4_0: return launch_generic<FH_Q4_0>(q, x, m, y, epi, a, b);
    case FH_Q8_0: return launch_generic<FH_Q8_0>(q, x, m, y, epi, a, b);
    case FH_Q4_K: return launch_generic<FH_Q4_K>(q, x, m, y, epi, a, b);
    case FH_Q6_K: return launch_generic<FH_Q6_K>(q, x, m, y, epi, a, b);
    case FH_Q5_0: return launch_generic<FH_Q5_0>(q, x, m, y, epi, a, b);
    case FH_Q5_K: return launch_generic<FH_Q5_K>(q, x, m, y, epi, a, b);
    case FH_W_F32: return launch_generic<FH_W_F32>(q, x, m, y, epi, a, b);
    case FH_W_F16: return launch_generic<FH_W_F16>(q, x, m, y, epi, a, b);
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
    const int64_t mk = q->dev->opt_matmul_kernel;
    // dense f16 / f32 weight rows (core/src/quantized/matmul/kernel.rs:132-193 routes them to the dense matmul) take
    // the matrix-core tiles as well once there are rows to fill them
    const bool dense = (q->type == FH_W_F16 || q->type == FH_W_F32) && q->k % 32 == 0;
    // (the 5-bit formats have no batch kernel for 2 .. 16 rows: rows are a launch each up to 12, tiles above)
    const int tile_from = (q->type == FH_Q5_K || q->type == FH_Q5_0) && q->k % 256 == 0 ? 12 : 16;
    if (((m > tile_from && mk != 1) || mk >= 2) && (!fh_is_plain(q->type) || dense)) return fh_launch_qmatmul_tile(q, x_dev, 0, m, y_dev);
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

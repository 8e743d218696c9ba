// Q6_K decode matvec for ONE activation row: y[n] = sum_k x[k] * deq(W)[n, k] with
//   deq = (d * sc_G) * (code - 32),  G = 16-element group        (fusor-ml/gguf/src/lib.rs:2034-2085)
// evaluated as   y = sum_blocks d * sum_G sc_G * [ (code . x)_G - 32 * (sum x)_G ].
//
// Same construction as the Q4_K kernel: the 6-bit codes are f16 SUBNORMAL integers (code * 2^-24) in the B
// operand of v_mfma_f32_16x16x32_f16, assembled from a low-nibble word and a high-bits word with one
// shift+AND (+OR) per code pair; the A operand row (2*G' + part) carries the hi / lo half of the exact f16
// split of the normalised activations of group G' = G mod 8 and zeros elsewhere, so the four steps of a half
// block chained through the accumulator leave D[2G' + part][row] = (code . x_part)_G for eight groups at once
// (two accumulator tiles per 256-block).  Lane (row j, group g) then owns groups 2g, 2g+1 of both halves of
// its own row and applies d * sc_G * 2^(24 - e_G).
#include "fh_blocks.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct Q6KRegs {
    uint4 l0, l1, h;
    uint32_t sc;
    uint16_t d;
};

#define DPP_XOR1 0xB1 // quad_perm [1,0,3,2]
#define DPP_XOR2 0x4E // quad_perm [2,3,0,1]
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}

#define Q6K_IMG 65 // uint4 per block image: 8 steps x 4 lane groups x (hi, lo) + one all-zero slot
#define Q6K_SF 32  // floats per block: 16 group sums, 16 factors

template <int TS, int PER, int EPI>
__global__ __launch_bounds__(1024) void k_qmv_q6k_m1(QView q, const float *__restrict__ x, float *__restrict__ y,
                                                      const float *__restrict__ ea, const float *__restrict__ eb,
                                                      int SW, const float *__restrict__ xup) {
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1;
    constexpr int TW = TS / NT;
    constexpr int XB = (PER + TS - 1) / TS;
    extern __shared__ uint4 lds[];
    // gridDim.y > 1: k is split over workgroups (blocks [boff, boff + kb) here) that add into y with atomics
    const int kb = SW * PER, boff = (int)blockIdx.y * kb; // the host launches with SW * PER * gridDim.y == q.kb
    uint4 *img = lds;
    float *sf = (float *)(lds + kb * Q6K_IMG);
    float *l_red = sf + kb * Q6K_SF; // [TS][SW][16]
    const int tid = threadIdx.x, lane = tid & 63, j = lane & 15, g = lane >> 4;
    // the wavefront index as a scalar: everything derived from it (tile, record address) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = TS * SW;
    const int stream = wave % TS, slice = wave / TS;
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
    const int64_t tiles_out = (nout + 15) / 16;
    const int64_t to = (int64_t)blockIdx.x * TW + (stream % TW);
    const bool tvalid = to < tiles_out;
    const int64_t tile = to + (int64_t)(stream / TW) * (nout / 16);
    const int b0 = slice * PER;

    // a tile past the end re-reads the last one (never stored)
    const int64_t tl = tvalid ? tile : tile - (to - (tiles_out - 1));
    const uint8_t *rec = q.data + (tl * q.recs + boff + b0) * 3360;

    // ---- 0. activations first (short, needed first)
    // With xup the input is silu(x) * xup (the SwiGLU of a gate | up projection, raw/attention_layer.rs:195),
    // evaluated while staging.
    float4 xv[XB], uv[XB];
#pragma unroll
    for (int i = 0; i < XB; i++) {
        // one tile stream: a wavefront stages exactly the blocks it multiplies (no other wavefront needs them)
        const int b = TS == 1 ? b0 + i : wave + i * nwaves;
        const int64_t at = (int64_t)(boff + (b < kb ? b : 0)) * 256 + lane * 4;
        xv[i] = *(const float4 *)(x + at);
        if (xup) uv[i] = *(const float4 *)(xup + at);
    }
    // The activation requests stay ahead of the weight requests: loads return in order, so the staging can wait
    // for them alone while the weights are still in flight.
    __builtin_amdgcn_sched_barrier(0);
    // ---- 1. all weight bytes of this wavefront
    Q6KRegs w[PER];
    {
#pragma unroll
        for (int r = 0; r < PER; r++) {
            const uint8_t *p = rec + r * 3360;
            w[r].l0 = *(const uint4 *)(p + lane * 16);
            w[r].l1 = *(const uint4 *)(p + 1024 + lane * 16);
            w[r].h = *(const uint4 *)(p + 2048 + lane * 16);
            w[r].sc = *(const uint32_t *)(p + 3072 + lane * 4);
            w[r].d = *(const uint16_t *)(p + 3328 + 2 * j);
        }
    }
    // ---- 2. stage x: lane owns k = 256*b + 4*lane .. +3, i.e. a quarter of group G = lane / 4
#pragma unroll
    for (int i = 0; i < XB; i++) {
        // no branch (the compiler would sink the activation loads into it, behind the weight loads): a wavefront
        // without a block of its own stages block 0 once more, writing the values wavefront 0 writes
        const int b = TS == 1 ? b0 + i : (wave + i * nwaves < kb ? wave + i * nwaves : 0);
        float4 v = xv[i];
        if (xup)
            v = make_float4((v.x / (__expf(-v.x) + 1.0f)) * uv[i].x, (v.y / (__expf(-v.y) + 1.0f)) * uv[i].y,
                            (v.z / (__expf(-v.z) + 1.0f)) * uv[i].z, (v.w / (__expf(-v.w) + 1.0f)) * uv[i].w);
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, dpp_f32<DPP_XOR1>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_XOR2>(amax));
        int e = 141 - (int)((__float_as_uint(amax) >> 23) & 0xFFu); // 14 - floor(log2 amax); specials clamp
        e = e > 100 ? 100 : (e < -100 ? -100 : e);
        const float sc = __uint_as_float((uint32_t)(e + 127) << 23);
        const float xs[4] = {v.x * sc, v.y * sc, v.z * sc, v.w * sc};
        _Float16 hi[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            hi[c] = (_Float16)xs[c];
            lo[c] = (_Float16)(xs[c] - (float)hi[c]);
        }
        uint2 ph, pl;
        __builtin_memcpy(&ph, hi, 8);
        __builtin_memcpy(&pl, lo, 8);
        const int s = lane >> 3, gg = (lane >> 1) & 3, sub = lane & 1;
        uint2 *dst = (uint2 *)(img + b * Q6K_IMG + (s * 4 + gg) * 2);
        dst[sub] = ph;     // hi: slots 4*sub .. +3
        dst[2 + sub] = pl; // lo
        if (lane == 0) img[b * Q6K_IMG + 64] = make_uint4(0, 0, 0, 0);
        float s4 = (v.x + v.y) + (v.z + v.w);
        s4 += dpp_f32<DPP_XOR1>(s4);
        s4 += dpp_f32<DPP_XOR2>(s4);
        if ((lane & 3) == 0) {
            sf[b * Q6K_SF + (lane >> 2)] = s4;
            sf[b * Q6K_SF + 16 + (lane >> 2)] = __uint_as_float((uint32_t)(24 - e + 127) << 23);
        }
    }
    if (TS > 1) __syncthreads(); // with one tile stream the image a wavefront reads is the one it wrote
    // ---- 3. two chains of four MFMA steps per block
    const int gl = j >> 1, part = j & 1; // this lane's A row is (group gl of a half block, hi | lo)
    const uint4 *pa[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const bool real = ((t & 3) == (gl >> 1)) && ((g >> 1) == (gl & 1));
        pa[t] = img + b0 * Q6K_IMG + (real ? (t * 4 + g) * 2 + part : 64);
    }
    const float *psf = sf + b0 * Q6K_SF + 2 * g;
    const uint32_t LO = 0x000F000Fu, HB = 0x00300030u;
    float acc = 0.f, cen = 0.f;
#pragma unroll
    for (int r = 0; r < PER; r++) {
        floatx4 dd[2];
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
            floatx4 c = {0.f, 0.f, 0.f, 0.f};
            const uint4 lq = hb ? w[r].l1 : w[r].l0;
#pragma unroll
            for (int tt = 0; tt < 4; tt++) {
                const int t = 4 * hb + tt;
                const uint32_t lw = tt == 0 ? lq.x : (tt == 1 ? lq.y : (tt == 2 ? lq.z : lq.w));
                const uint32_t hsel = (t >> 1) == 0 ? w[r].h.x : ((t >> 1) == 1 ? w[r].h.y : ((t >> 1) == 2 ? w[r].h.z : w[r].h.w));
                uint4 bo;
                if ((t & 1) == 0) {
                    bo.x = (lw & LO) | (hsel & HB);
                    bo.y = ((lw >> 4) & LO) | ((hsel >> 2) & HB);
                    bo.z = ((lw >> 8) & LO) | ((hsel >> 4) & HB);
                    bo.w = ((lw >> 12) & LO) | ((hsel >> 6) & HB);
                } else {
                    bo.x = (lw & LO) | ((hsel << 4) & HB);
                    bo.y = ((lw >> 4) & LO) | ((hsel << 2) & HB);
                    bo.z = ((lw >> 8) & LO) | ((hsel >> 8) & HB);
                    bo.w = ((lw >> 12) & LO) | ((hsel >> 10) & HB);
                }
                const uint4 ao = pa[t][r * Q6K_IMG];
                half8 av, bv;
                __builtin_memcpy(&av, &ao, 16);
                __builtin_memcpy(&bv, &bo, 16);
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, c, 0, 0, 0);
            }
            dd[hb] = c;
        }
        const float d = fh_h2f(w[r].d);
        const int scw = (int)w[r].sc;
        const float s0 = (float)((scw << 24) >> 24), s1 = (float)((scw << 16) >> 24), s2 = (float)((scw << 8) >> 24),
                    s3 = (float)(scw >> 24);
        const float2 sx0 = *(const float2 *)(psf + r * Q6K_SF), sx1 = *(const float2 *)(psf + r * Q6K_SF + 8);
        const float2 f0 = *(const float2 *)(psf + r * Q6K_SF + 16), f1 = *(const float2 *)(psf + r * Q6K_SF + 24);
        acc = fmaf(dd[0][0] + dd[0][1], (s0 * d) * f0.x, acc);
        acc = fmaf(dd[0][2] + dd[0][3], (s1 * d) * f0.y, acc);
        acc = fmaf(dd[1][0] + dd[1][1], (s2 * d) * f1.x, acc);
        acc = fmaf(dd[1][2] + dd[1][3], (s3 * d) * f1.y, acc);
        float cs = s0 * sx0.x;
        cs = fmaf(s1, sx0.y, cs);
        cs = fmaf(s2, sx1.x, cs);
        cs = fmaf(s3, sx1.y, cs);
        cen = fmaf(d, cs, cen);
    }
    float v = fmaf(-32.0f, cen, acc);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    if (lane < 16) l_red[(stream * SW + slice) * 16 + lane] = v;
    __syncthreads();
    if (tid < TW * 16) {
        const int t = tid >> 4, jr = tid & 15;
        float v0 = 0.f, v1 = 0.f;
        for (int s = 0; s < SW; s++) {
            v0 += l_red[(t * SW + s) * 16 + jr];
            if (NT == 2) v1 += l_red[((t + TW) * SW + s) * 16 + jr];
        }
        const int64_t row = ((int64_t)blockIdx.x * TW + t) * 16 + jr;
        if (row < nout) {
            float rr = v0;
            if (EPI == FH_EPI_ADD2) rr = (rr + ea[row]) + eb[row];
            if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * v1;
            if (EPI == FH_EPI_ACC) unsafeAtomicAdd(y + row, (blockIdx.y == 0 && ea) ? rr + ea[row] : rr);
            else y[row] = rr;
        }
    }
}

template <int TS, int PER, int EPI>
static fh_status q6k_m1_launch(const fh_qmatrix *q, const float *x, float *y, const float *a, const float *b, int SW,
                               unsigned grid, size_t lds, unsigned ksplit = 1, const float *xup = nullptr) {
    static bool attr_done = false;
    if (!attr_done) {
        FH_HIP(hipFuncSetAttribute((const void *)k_qmv_q6k_m1<TS, PER, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024));
        attr_done = true;
    }
    k_qmv_q6k_m1<TS, PER, EPI><<<dim3(grid, ksplit), dim3(64 * TS * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, xup);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <int TS, int EPI>
static fh_status q6k_m1_per(int per, const fh_qmatrix *q, const float *x, float *y, const float *a, const float *b,
                            int SW, unsigned grid, size_t lds) {
    if (per == 1) return q6k_m1_launch<TS, 1, EPI>(q, x, y, a, b, SW, grid, lds);
    if (per == 2) return q6k_m1_launch<TS, 2, EPI>(q, x, y, a, b, SW, grid, lds);
    return q6k_m1_launch<TS, 4, EPI>(q, x, y, a, b, SW, grid, lds);
}

// Returns FH_ERR_UNSUPPORTED when the shape does not fit this kernel (the caller falls back).
fh_status fh_launch_q6k_m1(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b) {
    fh_device *dev = q->dev;
    const int kb = (int)q->kb;
    const int nt = epi == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int64_t tiles = (nout + 15) / 16;
    int per = (int)dev->opt_matvec_per;
    // measured on MI355X: vocabulary-sized matrices want 4 blocks per wavefront, layer-sized ones 2
    if (per != 1 && per != 2 && per != 4) per = tiles >= 4096 ? 4 : (tiles >= 512 ? 2 : (kb > 16 ? 2 : 1));
    while (per > 1 && kb % per) per /= 2; // the kernel wants SW * PER == kb
    int SW = kb / per;
    while (SW > 16 && per < 4 && kb % (per * 2) == 0) {
        per *= 2;
        SW = kb / per;
    }
    if (SW > 16) return FH_ERR_UNSUPPORTED;
    int TW = (int)dev->opt_matvec_tiles;
    if (TW != 1 && TW != 2 && TW != 4) TW = (tiles >= 512 && tiles < 4096) ? 2 : 1;
    while (TW > 1 && TW * nt * SW > 16) TW /= 2;
    const int TS = TW * nt;
    if (TS * SW > 16 || (TS != 1 && TS != 2 && TS != 4)) return FH_ERR_UNSUPPORTED;
    size_t lds = (size_t)kb * Q6K_IMG * 16 + (size_t)kb * Q6K_SF * 4 + (size_t)TS * SW * 64;
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED;
    unsigned grid = (unsigned)((tiles + TW - 1) / TW);
#define Q6K_M1_GO(TS_, EPI_) return q6k_m1_per<TS_, EPI_>(per, q, x, y, a, b, SW, grid, lds)
    if (epi == FH_EPI_SWIGLU) {
        if (TS == 2) Q6K_M1_GO(2, FH_EPI_SWIGLU);
        Q6K_M1_GO(4, FH_EPI_SWIGLU);
    }
    if (epi == FH_EPI_ADD2) {
        if (TS == 1) Q6K_M1_GO(1, FH_EPI_ADD2);
        if (TS == 2) Q6K_M1_GO(2, FH_EPI_ADD2);
        Q6K_M1_GO(4, FH_EPI_ADD2);
    }
    if (TS == 1) Q6K_M1_GO(1, FH_EPI_NONE);
    if (TS == 2) Q6K_M1_GO(2, FH_EPI_NONE);
    Q6K_M1_GO(4, FH_EPI_NONE);
#undef Q6K_M1_GO
}

// y += W . x + add with k split over `ksplit` workgroups per row tile (atomic adds, so the summation order - and the
// last bits of the result - vary from run to run).  For matrices with few row tiles and a long k (the down projection
// of a decode step accumulating into the residual stream) the smaller workgroups overlap their load and compute phases.
// With xup the input is silu(x) * xup.
fh_status fh_launch_q6k_m1_acc(const fh_qmatrix *q, const float *x, const float *xup, float *y_inout, const float *add) {
    fh_device *dev = q->dev;
    const int kb = (int)q->kb;
    int ks = (int)dev->opt_matvec_splitk;
    if (ks <= 0) ks = kb % 4 == 0 ? kb / 4 : 0; // four blocks per workgroup measured best (MI355X, k = 14336)
    if (ks < 2 || kb % ks) return FH_ERR_UNSUPPORTED;
    const int kbl = kb / ks;
    int per = (int)dev->opt_matvec_per;
    if (per != 1 && per != 2 && per != 4) per = 1;
    while (per > 1 && kbl % per) per /= 2;
    const int SW = kbl / per;
    if (SW > 16) return FH_ERR_UNSUPPORTED;
    const int64_t tiles = (q->n + 15) / 16;
    size_t lds = (size_t)kbl * Q6K_IMG * 16 + (size_t)kbl * Q6K_SF * 4 + (size_t)SW * 64;
    if (per == 1) return q6k_m1_launch<1, 1, FH_EPI_ACC>(q, x, y_inout, add, nullptr, SW, (unsigned)tiles, lds, (unsigned)ks, xup);
    if (per == 2) return q6k_m1_launch<1, 2, FH_EPI_ACC>(q, x, y_inout, add, nullptr, SW, (unsigned)tiles, lds, (unsigned)ks, xup);
    return q6k_m1_launch<1, 4, FH_EPI_ACC>(q, x, y_inout, add, nullptr, SW, (unsigned)tiles, lds, (unsigned)ks, xup);
}

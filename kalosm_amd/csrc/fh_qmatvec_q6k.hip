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
#include "fh_mv_lanes.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct Q6KRegs {
    uint4 l0, l1, h;
    uint32_t sc;
    uint16_t d;
};

#define Q6K_IMG 65 // uint4 per block image: 8 steps x 4 lane groups x (hi, lo) + one all-zero slot
#define Q6K_SF 32  // floats per block: 16 group sums, 16 factors

// Workgroup = SW wavefronts, one per k-slice of PER blocks; a wavefront multiplies its slice of TPW row tiles (with
// the SwiGLU epilogue: gate tiles and the matching up tiles), stages the activations of its own blocks only (no
// barrier before the products) and requests all its weight bytes before anything else.
template <int TPW, int PER, int EPI>
__global__ __launch_bounds__(1024) void k_qmv_q6k_m1(QView q, const float *__restrict__ x, float *__restrict__ y,
                                                      const float *__restrict__ ea, const float *__restrict__ eb,
                                                      int SW, const float *__restrict__ xup) {
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1;
    constexpr int TOUT = TPW / NT; // output tiles of the workgroup
    extern __shared__ uint4 lds[];
    // gridDim.y > 1: k is split over workgroups (blocks [boff, boff + kb) here) that add into y with atomics
    const int kb = SW * PER, boff = (int)blockIdx.y * kb; // the host launches with SW * PER * gridDim.y == q.kb
    uint4 *img = lds;
    float *sf = (float *)(lds + kb * Q6K_IMG);
    float *l_red = sf + kb * Q6K_SF; // [TPW][SW][16]
    const int tid = threadIdx.x, lane = tid & 63, j = lane & 15, g = lane >> 4;
    // the wavefront index as a scalar: everything derived from it (record addresses) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
    const int64_t tiles_out = (nout + 15) / 16;
    const int b0 = wave * PER;
    const uint8_t *rec[TPW];
#pragma unroll
    for (int tp = 0; tp < TPW; tp++) {
        const int64_t to = (int64_t)blockIdx.x * TOUT + (tp % TOUT);
        const int64_t tile = to + (int64_t)(tp / TOUT) * (nout / 16); // up tiles follow the gate tiles
        // a tile past the end re-reads the last one (never stored)
        const int64_t tl = to < tiles_out ? tile : tile - (to - (tiles_out - 1));
        rec[tp] = q.data + (tl * q.recs + boff + b0) * 3360;
    }

    // ---- 0. activations first (short, needed first)
    // With xup the input is silu(x) * xup (the SwiGLU of a gate | up projection, raw/attention_layer.rs:195),
    // evaluated while staging.
    float4 xv[PER], uv[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int64_t at = (int64_t)(boff + b0 + i) * 256 + lane * 4;
        xv[i] = *(const float4 *)(x + at);
        if (xup) uv[i] = *(const float4 *)(xup + at);
    }
    // The activation requests stay ahead of the weight requests: loads return in order, so the staging can wait
    // for them alone while the weights are still in flight.
    __builtin_amdgcn_sched_barrier(0);
    // ---- 1. all weight bytes of this wavefront
    Q6KRegs w[TPW][PER];
#pragma unroll
    for (int r = 0; r < PER; r++)
#pragma unroll
        for (int tp = 0; tp < TPW; tp++) {
            const uint8_t *p = rec[tp] + r * 3360;
            w[tp][r].l0 = *(const uint4 *)(p + lane * 16);
            w[tp][r].l1 = *(const uint4 *)(p + 1024 + lane * 16);
            w[tp][r].h = *(const uint4 *)(p + 2048 + lane * 16);
            w[tp][r].sc = *(const uint32_t *)(p + 3072 + lane * 4);
            w[tp][r].d = *(const uint16_t *)(p + 3328 + 2 * j);
        }
    // ---- 2. stage x: lane owns k = 256*b + 4*lane .. +3, i.e. a quarter of group G = lane / 4.  A wavefront stages
    // exactly the blocks it multiplies.  (No branch around this: the compiler would sink the activation loads
    // into it, behind the weight loads.)
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int b = b0 + i;
        float4 v = xv[i];
        if (xup)
            v = make_float4((v.x / (__expf(-v.x) + 1.0f)) * uv[i].x, (v.y / (__expf(-v.y) + 1.0f)) * uv[i].y,
                            (v.z / (__expf(-v.z) + 1.0f)) * uv[i].z, (v.w / (__expf(-v.w) + 1.0f)) * uv[i].w);
        const float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        // non-negative floats order like their bit patterns: the cross-lane maximum is an integer one
        uint32_t am = __float_as_uint(amax);
        am = max(am, dpp_u32<DPP_XOR1>(am));
        am = max(am, dpp_u32<DPP_XOR2>(am));
        int e = 141 - (int)((am >> 23) & 0xFFu); // 14 - floor(log2 amax); specials clamp
        e = e > 100 ? 100 : (e < -100 ? -100 : e);
        const float sc = __uint_as_float((uint32_t)(e + 127) << 23);
        const float xq[4] = {v.x, v.y, v.z, v.w};
        _Float16 hi[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; c++) { // x * sc is exact (a power of two), so the fused form rounds like the split one
            hi[c] = (_Float16)(xq[c] * sc);
            lo[c] = (_Float16)__builtin_fmaf(xq[c], sc, -(float)hi[c]);
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
    // ---- 3. two chains of four MFMA steps per block and tile; the TPW tiles share every operand read
    // This lane's A row is (group gl of a half block, hi | lo): it holds data in steps m and m + 4 with m = gl / 2
    // if its lane group covers the k of that group (g / 2 == gl % 2), zeros otherwise.  Those lanes are bits
    // 4m, 4m + 1 of the rows 0, 1 and bits 4m + 2, 4m + 3 of the rows 2, 3.
    const int gl = j >> 1, part = j & 1;
    uint32_t pa[8];
    {
        const uint32_t own = lds_addr(img + b0 * Q6K_IMG + ((gl >> 1) * 4 + g) * 2 + part);
        const uint32_t zero = lds_addr(img + b0 * Q6K_IMG + 64);
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int m = t & 3;
            const uint64_t mask = ((uint64_t)0x00030003u << (4 * m)) | ((uint64_t)0x000C000Cu << (4 * m + 32));
            pa[t] = sel_lanes(mask, own + (t >> 2) * 32 * 16, zero);
        }
    }
    // the operands do not depend on the weights: RING of them are always on their way from the LDS
    constexpr int RING = 4;
    uint4 ring[RING];
#pragma unroll
    for (int t = 0; t < RING; t++) ring[t] = lds_read16(pa[t % 8] + (t / 8) * Q6K_IMG * 16);
    const float *psf = sf + b0 * Q6K_SF + 2 * g;
    const uint32_t LO = 0x000F000Fu, HB = 0x00300030u;
    float acc[TPW], cen[TPW];
#pragma unroll
    for (int tp = 0; tp < TPW; tp++) acc[tp] = cen[tp] = 0.f;
#pragma unroll
    for (int r = 0; r < PER; r++) {
        floatx4 dd[TPW][2];
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
#pragma unroll
            for (int tp = 0; tp < TPW; tp++) dd[tp][hb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < 4; tt++) {
                const int t = 4 * hb + tt, ti = r * 8 + t;
                const uint4 ao = ring[ti % RING];
                half8 av;
                __builtin_memcpy(&av, &ao, 16);
#pragma unroll
                for (int tp = 0; tp < TPW; tp++) {
                    const uint4 lq = hb ? w[tp][r].l1 : w[tp][r].l0;
                    const uint4 hq = w[tp][r].h;
                    const uint32_t lw = tt == 0 ? lq.x : (tt == 1 ? lq.y : (tt == 2 ? lq.z : lq.w));
                    const uint32_t hsel = (t >> 1) == 0 ? hq.x : ((t >> 1) == 1 ? hq.y : ((t >> 1) == 2 ? hq.z : hq.w));
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
                    half8 bv;
                    __builtin_memcpy(&bv, &bo, 16);
                    dd[tp][hb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, dd[tp][hb], 0, 0, 0);
                }
                if (ti + RING < PER * 8)
                    ring[ti % RING] = lds_read16(pa[(ti + RING) % 8] + ((ti + RING) / 8) * Q6K_IMG * 16);
            }
        }
        const float2 sx0 = *(const float2 *)(psf + r * Q6K_SF), sx1 = *(const float2 *)(psf + r * Q6K_SF + 8);
        const float2 f0 = *(const float2 *)(psf + r * Q6K_SF + 16), f1 = *(const float2 *)(psf + r * Q6K_SF + 24);
#pragma unroll
        for (int tp = 0; tp < TPW; tp++) {
            const float d = fh_h2f(w[tp][r].d);
            const int scw = (int)w[tp][r].sc;
            const float s0 = (float)((scw << 24) >> 24), s1 = (float)((scw << 16) >> 24),
                        s2 = (float)((scw << 8) >> 24), s3 = (float)(scw >> 24);
            acc[tp] = fmaf(dd[tp][0][0] + dd[tp][0][1], (s0 * d) * f0.x, acc[tp]);
            acc[tp] = fmaf(dd[tp][0][2] + dd[tp][0][3], (s1 * d) * f0.y, acc[tp]);
            acc[tp] = fmaf(dd[tp][1][0] + dd[tp][1][1], (s2 * d) * f1.x, acc[tp]);
            acc[tp] = fmaf(dd[tp][1][2] + dd[tp][1][3], (s3 * d) * f1.y, acc[tp]);
            float cs = s0 * sx0.x;
            cs = fmaf(s1, sx0.y, cs);
            cs = fmaf(s2, sx1.x, cs);
            cs = fmaf(s3, sx1.y, cs);
            cen[tp] = fmaf(d, cs, cen[tp]);
        }
    }
#pragma unroll
    for (int tp = 0; tp < TPW; tp++) {
        const float v = rows_sum(fmaf(-32.0f, cen[tp], acc[tp]));
        if (lane < 16) l_red[(tp * SW + wave) * 16 + lane] = v;
    }
    __syncthreads();
    if (tid < TOUT * 16) {
        const int t = tid >> 4, jr = tid & 15;
        float v0 = 0.f, v1 = 0.f;
        for (int s = 0; s < SW; s++) {
            v0 += l_red[(t * SW + s) * 16 + jr];
            if (NT == 2) v1 += l_red[((t + TOUT) * SW + s) * 16 + jr];
        }
        const int64_t row = ((int64_t)blockIdx.x * TOUT + t) * 16 + jr;
        if (row < nout) {
            float rr = v0;
            if (EPI == FH_EPI_ADD2) rr = (rr + ea[row]) + eb[row];
            if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * v1;
            if (EPI == FH_EPI_ACC) unsafeAtomicAdd(y + row, (blockIdx.y == 0 && ea) ? rr + ea[row] : rr);
            else y[row] = rr;
        }
    }
}

template <int TPW, int PER, int EPI>
static fh_status q6k_m1_launch(const fh_qmatrix *q, const float *x, float *y, const float *a, const float *b, int SW,
                               unsigned grid, size_t lds, unsigned ksplit = 1, const float *xup = nullptr) {
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmv_q6k_m1<TPW, PER, EPI>, 160 * 1024));
    k_qmv_q6k_m1<TPW, PER, EPI><<<dim3(grid, ksplit), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, xup);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// (tiles per wavefront, blocks per wavefront) with at most four block tiles (56 registers of weights) per wavefront
template <int EPI>
static fh_status q6k_m1_shape(int tpw, int per, const fh_qmatrix *q, const float *x, float *y, const float *a,
                              const float *b, int SW, unsigned grid, size_t lds, unsigned ksplit = 1,
                              const float *xup = nullptr) {
    if constexpr (EPI != FH_EPI_SWIGLU) {
        if (tpw == 1 && per == 1) return q6k_m1_launch<1, 1, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
        if (tpw == 1 && per == 2) return q6k_m1_launch<1, 2, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
        if (tpw == 1 && per == 4) return q6k_m1_launch<1, 4, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
    }
    if (tpw == 2 && per == 1) return q6k_m1_launch<2, 1, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
    if (tpw == 2 && per == 2) return q6k_m1_launch<2, 2, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
    if (tpw == 4 && per == 1) return q6k_m1_launch<4, 1, EPI>(q, x, y, a, b, SW, grid, lds, ksplit, xup);
    return FH_ERR_UNSUPPORTED;
}

// Returns FH_ERR_UNSUPPORTED when the shape does not fit this kernel (the caller falls back).
fh_status fh_launch_q6k_m1(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b) {
    fh_device *dev = q->dev;
    const int kb = (int)q->kb;
    const int nt = epi == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int64_t tiles = (nout + 15) / 16;
    // tiles per wavefront (they share the staged activations and every operand read): two once there are more
    // tiles than compute units; the SwiGLU epilogue needs the gate and the up tile in one wavefront
    int tpw = (int)dev->opt_matvec_tiles;
    if (tpw != 1 && tpw != 2 && tpw != 4) tpw = tiles > dev->compute_units ? 2 : 1;
    if (epi == FH_EPI_SWIGLU && tpw < 2) tpw = 2;
    // blocks per wavefront (all requested up front): vocabulary-sized matrices want two (measured on MI355X)
    int per = (int)dev->opt_matvec_per;
    if (per != 1 && per != 2 && per != 4) per = tiles >= 4096 ? 2 : 1;
    while (per > 1 && (kb % per || tpw * per > 4)) per /= 2;
    while (kb / per > 16 && tpw * per < 4 && kb % (per * 2) == 0) per *= 2; // the kernel wants SW * PER == kb
    while (kb / per > 16 && tpw > nt && kb % (per * 2) == 0) { // long k: fewer tiles, more blocks per wavefront
        tpw /= 2;
        per *= 2;
    }
    const int SW = kb / per;
    if (SW > 16 || kb % per || tpw * per > 4) return FH_ERR_UNSUPPORTED;
    size_t lds = (size_t)kb * Q6K_IMG * 16 + (size_t)kb * Q6K_SF * 4 + (size_t)tpw * SW * 64;
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED;
    const int tout = tpw / nt;
    unsigned grid = (unsigned)((tiles + tout - 1) / tout);
    if (epi == FH_EPI_SWIGLU) return q6k_m1_shape<FH_EPI_SWIGLU>(tpw, per, q, x, y, a, b, SW, grid, lds);
    if (epi == FH_EPI_ADD2) return q6k_m1_shape<FH_EPI_ADD2>(tpw, per, q, x, y, a, b, SW, grid, lds);
    return q6k_m1_shape<FH_EPI_NONE>(tpw, per, q, x, y, a, b, SW, grid, lds);
}

// y += W . x + add with k split over `ksplit` workgroups per row tile group (atomic adds, so the summation order -
// and the last bits of the result - vary from run to run).  For matrices with few row tiles and a long k (the down
// projection of a decode step accumulating into the residual stream) the smaller workgroups overlap their load and
// compute phases.  With xup the input is silu(x) * xup.
fh_status fh_launch_q6k_m1_acc(const fh_qmatrix *q, const float *x, const float *xup, float *y_inout, const float *add) {
    fh_device *dev = q->dev;
    const int kb = (int)q->kb;
    int ks = (int)dev->opt_matvec_splitk;
    if (ks <= 0) ks = kb % 4 == 0 ? kb / 4 : 0; // four blocks per workgroup measured best (MI355X, k = 14336)
    if (ks < 2 || kb % ks) return FH_ERR_UNSUPPORTED;
    const int kbl = kb / ks;
    int tpw = (int)dev->opt_down_tiles;
    if (tpw != 1 && tpw != 2 && tpw != 4) tpw = 1;
    int per = (int)dev->opt_matvec_per;
    if (per != 1 && per != 2 && per != 4) per = 1;
    while (per > 1 && (kbl % per || tpw * per > 4)) per /= 2;
    const int SW = kbl / per;
    if (SW > 16) return FH_ERR_UNSUPPORTED;
    const int64_t tiles = (q->n + 15) / 16;
    size_t lds = (size_t)kbl * Q6K_IMG * 16 + (size_t)kbl * Q6K_SF * 4 + (size_t)tpw * SW * 64;
    const unsigned grid = (unsigned)((tiles + tpw - 1) / tpw);
    return q6k_m1_shape<FH_EPI_ACC>(tpw, per, q, x, y_inout, add, nullptr, SW, grid, lds, (unsigned)ks, xup);
}

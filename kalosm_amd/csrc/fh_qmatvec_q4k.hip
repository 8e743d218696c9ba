// Q4_K decode matvec for ONE activation row (the batch-1 token loop): y[n] = sum_k x[k] * deq(W)[n, k].
// Reference: fusor-ml/cpu/src/quantized.rs:246-675 (semantics); the factorised form
//   y = d * sum_j sc_j * (q . x)_j  -  dmin * sum_j m_j * (sum x)_j      (j = 32-element sub-block)
// is the one the reference's own GPU kernel uses (fusor-ml/tile-ir-kernels/src/kernels/qgemv_q4k_ggml.rs:64-158).
//
// Mapping onto v_mfma_f32_16x16x32_f16.  B operand: 16 weight rows x 32 k of one sub-block; the 4-bit
// codes become f16 SUBNORMAL integers (code * 2^-24, or code * 16 * 2^-24 for the high nibbles) with one
// AND per two codes.  A operand: 16 rows x 32 k where row (2*s + part) holds the hi (part 0) or lo (part 1)
// half of the exact two-term f16 split of the normalised activations of sub-block s and is ZERO for the
// other sub-blocks.  Chaining the 8 steps of a 256-block through the accumulator therefore leaves
// D[2s + part][row] = (q . x_part)_s for all eight sub-blocks at once: lane (row j, group g) holds the four
// values of sub-blocks 2g and 2g+1 of its own row and applies that row's d * sc_s * 2^(24-e_s) itself.
//
// Workgroup = SW wavefronts, one per k-slice of PER blocks; a wavefront multiplies its slice of TPW row tiles
// (with the SwiGLU epilogue: gate tiles and the matching up tiles).  All TPW x PER x 2304 B of a wavefront are
// requested before anything else; meanwhile it stages the activations of its own blocks (nobody else needs
// them, so there is no barrier before the products): each 32-group is normalised by a power of two to
// [2^14, 2^15) (odd groups 16x lower, which folds the x16 of the high nibbles), split into f16 hi + lo and stored
// in operand order, with the group sums of the original x and the factors beside them.
#include "fh_blocks.h"
#include "fh_mv_lanes.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct Q4KRegs {
    uint4 h, qa, qb, qc, qd; // qc, qd: Q8_0 only (four records per 256 activations)
};

// Arguments of the rope + KV-append epilogue (the fused q|k|v projection of a decode step): rows [0, qd) are query
// rows (rotated, written to qo), [qd, qd + kd) key rows (rotated, written to the cache row of the device-side
// position), the rest value rows (copied to the cache).  RopeCache::forward_interleaved + KvCache::append
// (fusor/src/composite/rope.rs:300-329, fusor/src/cache/kv_cache.rs:49-63).
struct FhRopeArgs {
    const float *cs, *sn;
    const int *pos;
    float *qo;
    void *kc, *vc;
    int qd, kd, hd, cap, table_rows, f16;
};
struct Q4kExtra {
    const float *xres = nullptr, *nw = nullptr;
    float eps = 0.f;
    int nsplit = 0;
    FhRopeArgs rk = {};
    int ksplit = 1; // workgroups along k (FH_EPI_ACC only)
};

#define Q4K_IMG 65 // uint4 per block image: 8 steps x 4 groups x (hi, lo) + one all-zero slot

// FMT = FH_Q4_0: the same kernel on eight 32-blocks (two records of the tiled Q4_0 layout, 2304 bytes as well) per
// 256 activations: sub-block s is block s, its scale the block's f16 d, its offset 8 d (gguf/src/lib.rs Q4_0:
// d * (q - 8)); a byte carries elements i (low nibble) and i + 16 (high nibble), so lane group g multiplies the
// elements 4g .. 4g+3 and 16+4g .. 16+4g+3 of its block and the staging writes the activations in that order.
// FMT = FH_Q8_0: eight 32-blocks = four records of 1088 bytes; a code byte q becomes the f16 1152 + q (xor 0x80,
// then v_perm_b32 sets it under the high byte 0x64: 1024 + (q + 128) exactly), so the offset is 1152 d and the
// activation factor carries no 2^24.
// FMT = FH_Q5_K: Q4_K plus one high bit per code (gguf/src/lib.rs:1819-1861).  The tiled record is the Q4_K record
// followed by the lanes' qh bytes: lane (row j, group g) holds the bytes 8 g .. 8 g + 7 of its row's qh, whose bit s is
// the fifth bit of the lane's element in sub-block s: one rotate and one and-or per operand word put it on bit 4 (low
// nibbles) or 8 (high nibbles) of the 16-bit code, still an exact f16 subnormal.
// FMT = FH_Q5_0: Q4_0 plus one high bit per code (gguf/src/lib.rs:1046-1073), d * (code - 16): the Q4_0 record followed
// by one byte per lane and block with the fifth bits of the lane's eight elements.
// MR > 1: MR activation rows (nsplit then carries the number of valid ones; plain input, epilogues none / add2):
// the weights are unpacked once per step and multiplied with the operand of every row; a wavefront stages its
// blocks of all rows, images interleaved [block][row] so that every operand address is the base plus a constant.
// RS > 1 (Q4_K, one row, plain input, epilogues none / add2): a workgroup owns 16 / RS rows of a tile and
// a wavefront multiplies them over RS consecutive blocks at once: MFMA column c is row c % (16 / RS) of block
// c / (16 / RS), A row i carries the (hi | lo) halves of sub-blocks (i >> 1) % (8 / RS) + a * (8 / RS) of block
// i / (16 / RS) in the steps of accumulator a = 0 .. RS - 1.  The accumulator entries whose row and column name the
// same block are the dots; the rest is discarded.  As many MFMAs per weight byte as with whole tiles, RS times the
// workgroups: matrices with fewer row tiles than compute units fill the device in one launch.
template <int FMT, int TPW, int PER, int EPI, int IN, int MR = 1, int RS = 1>
__device__ __forceinline__ void qmv_q4k_m1_body(QView q, const float *__restrict__ x, float *__restrict__ y,
                                                      const float *__restrict__ ea, const float *__restrict__ eb,
                                                      int SW, const float *__restrict__ xres,
                                                      const float *__restrict__ nw, float eps, int nsplit,
                                                      FhRopeArgs rk) {
    static_assert(MR == 1 || (IN == 0 && (EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2)), "rows: plain input, none / add2");
    static_assert(MR == 1 || MR == 2 || MR == 4, "rows per launch");
    static_assert(RS == 1 || (FMT == FH_Q4_K && TPW == 1 && MR == 1 && IN == 0 && (EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2)),
                  "row split: Q4_K, one tile part, one row, plain input, epilogues none / add2");
    static_assert(RS == 1 || RS == 2 || RS == 4, "row split");
    constexpr int NB = PER * RS; // blocks a wavefront stages and multiplies
    // SwiGLU with one tile per wavefront: the "tile" is rows 8h .. 8h+7 of a gate tile (columns 0-7 of the MFMA) and
    // the same rows of the matching up tile (columns 8-15), h = workgroup parity: workgroups half as heavy as with a
    // whole gate and a whole up tile, which divides the Llama FFN evenly over the compute units
    // Q4_K: the sums of the activations per sub-block (they multiply the block minimums) come from one more MFMA per
    // block, whose B operand is the constant code 1 and whose A operand is the whole image (every row at once),
    // instead of from adds and lane exchanges in the staging
    constexpr bool ONES = FMT == FH_Q4_K || FMT == FH_Q5_K;
    constexpr bool Q5 = FMT == FH_Q5_K || FMT == FH_Q5_0;
    constexpr bool Q40 = FMT == FH_Q4_0 || FMT == FH_Q5_0; // eight 32-blocks per 256 activations, a byte = elements i, i + 16
    constexpr bool HP = EPI == FH_EPI_SWIGLU && TPW == 1;
    static_assert(!(HP && Q5) && (!Q5 || (MR == 1 && RS == 1)), "5-bit formats: whole tiles, one row");
    constexpr int NT = (EPI == FH_EPI_SWIGLU && !HP) ? 2 : 1;
    constexpr int TOUT = TPW / NT; // output tiles of the workgroup
    extern __shared__ uint4 lds[];
    // gridDim.y > 1: k is split over workgroups (blocks [boff, boff + kb) here) that add into y with atomics
    const int kb = SW * NB, boff = (int)blockIdx.y * kb; // the host launches with SW * NB * gridDim.y == q.kb
    uint4 *img = lds;
    float *sf = (float *)(lds + kb * MR * Q4K_IMG); // per block and row: [0..7] group sums, [8..15] factors
    float *l_red = sf + kb * MR * 16;               // [MR][TPW][SW][16]
    float *l_ss = l_red + MR * TPW * 16 * 16;       // per wavefront: sum of squares of the blocks it staged
    const int tid = threadIdx.x, lane = tid & 63, j = lane & 15, g = lane >> 4;
    // the wavefront index as a scalar: everything derived from it (record addresses) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q.n / 2 : q.n;
    const int64_t tiles_out = (nout + 15) / 16;
    const int b0 = wave * NB;
    // bytes of a tiled record, and per 256 activations and tile
    constexpr int REC = FMT == FH_Q4_0 ? 1152 : (FMT == FH_Q8_0 ? 1088 : (FMT == FH_Q5_0 ? 1408 : (FMT == FH_Q5_K ? 2816 : 2304)));
    constexpr int CHUNK = FMT == FH_Q8_0 ? 4352 : ((FMT == FH_Q5_0 || FMT == FH_Q5_K) ? 2816 : 2304);
    const uint8_t *ph[TPW], *pq[TPW];
    if constexpr (HP) {
        const int64_t tile = (int64_t)(blockIdx.x >> 1) + (j < 8 ? 0 : nout / 16);
        // per lane: gate or up record
        const uint8_t *rec = q.data + tile * q.recs * REC + (int64_t)(boff + b0) * CHUNK;
        const int rr = 8 * (int)(blockIdx.x & 1) + (j & 7);
        if (FMT == FH_Q4_0) {
            ph[0] = rec + (g >> 1) * 1152 + 1024 + 8 * rr + 4 * (g & 1);
            pq[0] = rec + (16 * g + rr) * 16;
        } else if (FMT == FH_Q8_0) {
            ph[0] = rec + g * 1088 + 1024 + 4 * rr;
            pq[0] = rec + (16 * g + rr) * 16;
        } else {
            ph[0] = rec + 16 * rr;
            pq[0] = rec + 256 + (16 * g + rr) * 16;
        }
    }
    if constexpr (RS > 1) { // column j: row (16 / RS) * part + j % (16 / RS) of the tile, block j / (16 / RS) of the group
        constexpr int RW = 16 / RS;
        const int64_t tile = (int64_t)(blockIdx.x / RS);
        const int rr = RW * (int)(blockIdx.x % RS) + j % RW;
        const uint8_t *rec = q.data + tile * q.recs * REC + (int64_t)(boff + b0 + j / RW) * CHUNK;
        ph[0] = rec + 16 * rr;
        pq[0] = rec + 256 + (16 * g + rr) * 16;
    }
#pragma unroll
    for (int tp = 0; tp < ((HP || RS > 1) ? 0 : TPW); tp++) {
        const int64_t to = (int64_t)blockIdx.x * TOUT + (tp % TOUT);
        const int64_t tile = to + (int64_t)(tp / TOUT) * (nout / 16); // up tiles follow the gate tiles
        // a tile past the end re-reads the last tile (its rows are never stored)
        const int64_t tl = to < tiles_out ? tile : tile - (to - (tiles_out - 1));
        const uint8_t *rec = q.data + tl * q.recs * REC + (int64_t)(boff + b0) * CHUNK;
        if (Q40) { // d of the blocks 2g, 2g+1 of this lane's row; quants of the two records
            ph[tp] = rec + (g >> 1) * REC + 1024 + 8 * j + 4 * (g & 1);
            pq[tp] = rec + lane * 16;
        } else if (FMT == FH_Q8_0) { // record g holds the blocks 2g, 2g+1
            ph[tp] = rec + g * 1088 + 1024 + 4 * j;
            pq[tp] = rec + lane * 16;
        } else {
            ph[tp] = rec + 16 * j;
            pq[tp] = rec + 256 + lane * 16;
        }
    }

    // ---- 0. the activations of this wavefront's blocks are requested first: they are needed first and are short
    // With nw the input is rms_norm(x [+ xres]) * nw (composite/normalization.rs:287-401): the weight nw is
    // folded into the staged values and the common factor 1 / rms is applied to the finished dot product.
    float4 xv[NB * MR], rv[NB], wv[NB], pacc[IN == 2 ? PER : 1][8];
    float2 pm[IN == 2 ? PER : 1][8];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int64_t at = (int64_t)(boff + b0 + i) * 256 + lane * 4;
        if (IN != 2) xv[i] = *(const float4 *)(x + at);
#pragma unroll
        for (int mr = 1; mr < MR; mr++) // rows past the valid ones repeat the last (never stored)
            xv[mr * NB + i] = *(const float4 *)(x + (int64_t)(mr < nsplit ? mr : nsplit - 1) * q.k + at);
        if (IN == 1 && xres) rv[i] = *(const float4 *)(xres + at);
        if (IN == 1) wv[i] = *(const float4 *)(nw + at);
        if (IN == 2) { // x holds attention partials [head][nsplit][128 + 4]: unnormalised output, max, sum
            const float *pp = x + (at >> 7) * nsplit * 132;
#pragma unroll
            for (int s = 0; s < 8; s++)
                if (s < nsplit) {
                    pacc[i][s] = *(const float4 *)(pp + s * 132 + (at & 127));
                    pm[i][s] = *(const float2 *)(pp + s * 132 + 128);
                }
        }
    }
    // The activation requests stay ahead of the weight requests: loads return in order, so the staging below can
    // wait for them alone (vmcnt > 0) while the weights are still in flight.
    __builtin_amdgcn_sched_barrier(0);
    // ---- 1. every weight byte of this wavefront goes in flight (the host guarantees SW * PER == kb, so no
    // block is out of range).
    Q4KRegs w[TPW][PER];
#pragma unroll
    for (int r = 0; r < PER; r++)
#pragma unroll
        for (int tp = 0; tp < TPW; tp++) {
            if constexpr (FMT == FH_Q5_0) { // the Q4_0 records, each followed by the lane's fifth bits (one byte per block)
                w[tp][r].h.x = *(const uint32_t *)(ph[tp] + r * CHUNK);
                w[tp][r].qa = *(const uint4 *)(pq[tp] + r * CHUNK);
                w[tp][r].qb = *(const uint4 *)(pq[tp] + r * CHUNK + REC);
                w[tp][r].qc.x = *(const uint32_t *)(pq[tp] + 1152 - 12 * lane + r * CHUNK);
                w[tp][r].qc.y = *(const uint32_t *)(pq[tp] + 1152 - 12 * lane + r * CHUNK + REC);
            } else if constexpr (FMT == FH_Q5_K) { // the Q4_K record followed by the lane's eight qh bytes
                w[tp][r].h = *(const uint4 *)(ph[tp] + r * CHUNK);
                w[tp][r].qa = *(const uint4 *)(pq[tp] + r * CHUNK);
                w[tp][r].qb = *(const uint4 *)(pq[tp] + r * CHUNK + 1024);
                const uint2 hb = *(const uint2 *)(pq[tp] + 2048 - 8 * lane + r * CHUNK);
                w[tp][r].qc.x = hb.x;
                w[tp][r].qc.y = hb.y;
            } else if (FMT == FH_Q4_0) {
                w[tp][r].h.x = *(const uint32_t *)(ph[tp] + r * 2304);
                w[tp][r].qa = *(const uint4 *)(pq[tp] + r * 2304);
                w[tp][r].qb = *(const uint4 *)(pq[tp] + r * 2304 + 1152);
            } else if (FMT == FH_Q8_0) {
                w[tp][r].h.x = *(const uint32_t *)(ph[tp] + r * 4352);
                w[tp][r].qa = *(const uint4 *)(pq[tp] + r * 4352);
                w[tp][r].qb = *(const uint4 *)(pq[tp] + r * 4352 + 1088);
                w[tp][r].qc = *(const uint4 *)(pq[tp] + r * 4352 + 2176);
                w[tp][r].qd = *(const uint4 *)(pq[tp] + r * 4352 + 3264);
            } else {
                w[tp][r].h = *(const uint4 *)(ph[tp] + r * RS * 2304);
                w[tp][r].qa = *(const uint4 *)(pq[tp] + r * RS * 2304);
                w[tp][r].qb = *(const uint4 *)(pq[tp] + r * RS * 2304 + 1024);
            }
        }
    // ---- 2. stage x (lane owns k = 256*b + 4*lane .. +3).  A wavefront stages exactly the blocks it multiplies:
    // nobody else reads its part of the image, so there is no barrier between this and the products.  (No branch
    // around it either: the compiler would sink the activation loads into it, behind the weight loads.)
    float ss = 0.f;
#pragma unroll
    for (int ii = 0; ii < NB * MR; ii++) {
        const int i = ii % NB;
        const int b = (b0 + i) * MR + ii / NB; // image index: [block][row]
        float4 v = xv[ii];
        if (IN == 2) { // merge the splits: softmax weights exp(m_s - max), then num / den
            float mx = -INFINITY;
#pragma unroll
            for (int s = 0; s < 8; s++)
                if (s < nsplit) mx = fmaxf(mx, pm[i][s].x);
            float den = 0.f;
            v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int s = 0; s < 8; s++)
                if (s < nsplit) {
                    const float w = pm[i][s].x == -INFINITY ? 0.f : __expf(pm[i][s].x - mx);
                    den = fmaf(pm[i][s].y, w, den);
                    v.x = fmaf(pacc[i][s].x, w, v.x); v.y = fmaf(pacc[i][s].y, w, v.y);
                    v.z = fmaf(pacc[i][s].z, w, v.z); v.w = fmaf(pacc[i][s].w, w, v.w);
                }
            v = make_float4(v.x / den, v.y / den, v.z / den, v.w / den);
        }
        if (IN == 1 && xres) v = make_float4(v.x + rv[i].x, v.y + rv[i].y, v.z + rv[i].z, v.w + rv[i].w);
        if (IN == 1) {
            float s2 = v.x * v.x;
            s2 = fmaf(v.y, v.y, s2); s2 = fmaf(v.z, v.z, s2); s2 = fmaf(v.w, v.w, s2);
            ss += s2;
            v = make_float4(v.x * wv[i].x, v.y * wv[i].y, v.z * wv[i].z, v.w * wv[i].w);
        }
        float amax;
        asm("v_max3_f32 %0, |%1|, |%2|, |%3|" : "=v"(amax) : "v"(v.x), "v"(v.y), "v"(v.z));
        asm("v_max_f32_e64 %0, %1, |%2|" : "=v"(amax) : "v"(amax), "v"(v.w));
        // non-negative floats order like their bit patterns: the cross-lane maximum is an integer one
        uint32_t am = __float_as_uint(amax);
        am = max(am, dpp_u32<DPP_XOR1>(am));
        am = max(am, dpp_u32<DPP_XOR2>(am));
        am = max(am, dpp_u32<DPP_HALF_MIRROR>(am)); // quads are uniform now: lane 7-i is in the other quad
        // Q4_K: lanes 2 gg, 2 gg + 1 of a sub-block fill the two halves of operand slot gg; odd sub-blocks are the
        // high nibbles.  Q4_0: lanes gg and gg + 4 do, the second with the high nibbles' elements.
        const int s = lane >> 3, gg = Q40 ? lane & 3 : (lane >> 1) & 3;
        const int half = Q40 ? (lane >> 2) & 1 : lane & 1;
        // e = 14 - floor(log2(amax)) from the exponent field (zero / subnormal / inf / nan just clamp)
        int e = 141 - (int)((am >> 23) & 0xFFu);
        e = e > 100 ? 100 : (e < -100 ? -100 : e);
        const int eo = e - (FMT == FH_Q8_0 ? 0 : 4 * (Q40 ? half : s & 1)); // high nibbles: codes x 16
        const float sc = __uint_as_float((uint32_t)(eo + 127) << 23);
        // hi = f16(x * sc), lo = f16(x * sc - hi) (x * sc is exact, a power of two, so the fused form rounds once),
        // written straight into the halves of the packed words in operand order (elements 0, 2 | 1, 3)
        uint2 ph, pl;
        asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(ph.x) : "v"(v.x), "v"(sc));
        asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(ph.y) : "v"(v.y), "v"(sc));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(ph.x) : "v"(v.z), "v"(sc));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(ph.y) : "v"(v.w), "v"(sc));
        asm("v_fma_mixlo_f16 %0, %1, %2, -%3 op_sel_hi:[0,0,1]" : "=v"(pl.x) : "v"(v.x), "v"(sc), "v"(ph.x));
        asm("v_fma_mixlo_f16 %0, %1, %2, -%3 op_sel_hi:[0,0,1]" : "=v"(pl.y) : "v"(v.y), "v"(sc), "v"(ph.y));
        asm("v_fma_mixhi_f16 %0, %1, %2, -%3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "+v"(pl.x) : "v"(v.z), "v"(sc), "v"(ph.x));
        asm("v_fma_mixhi_f16 %0, %1, %2, -%3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "+v"(pl.y) : "v"(v.w), "v"(sc), "v"(ph.y));
        uint2 *dst = (uint2 *)(img + b * Q4K_IMG + (s * 4 + gg) * 2);
        dst[half] = ph;     // hi
        dst[2 + half] = pl; // lo
        if (lane == 0) img[b * Q4K_IMG + 64] = make_uint4(0, 0, 0, 0);
        const float fct = __uint_as_float((uint32_t)((FMT == FH_Q8_0 ? 0 : 24) - e + 127) << 23);
        if constexpr (ONES) {
            if ((lane & 7) == 0) sf[b * 16 + 8 + s] = fct;
        } else {
            float s4 = (v.x + v.y) + (v.z + v.w);
            s4 += dpp_f32<DPP_XOR1>(s4);
            s4 += dpp_f32<DPP_XOR2>(s4);
            s4 += dpp_f32<DPP_HALF_MIRROR>(s4);
            if ((lane & 7) == 0) {
                sf[b * 16 + s] = s4;
                sf[b * 16 + 8 + s] = fct;
            }
        }
    }
    if (IN == 1) {
        ss += dpp_f32<DPP_XOR1>(ss);
        ss += dpp_f32<DPP_XOR2>(ss);
        ss += dpp_f32<DPP_HALF_MIRROR>(ss);
        ss += dpp_f32<DPP_ROW_MIRROR>(ss); // rows of 16 are uniform now
        ss = rows_sum(ss);
        if (lane == 0) l_ss[wave] = ss;
    }
    // ---- 3. eight chained MFMA steps per block and tile; the TPW tiles share every operand read
    if constexpr (RS > 1) {
        constexpr int SL = 8 / RS, RW = 16 / RS;
        const int blk = j / RW, sloc = (j >> 1) % SL, part = j & 1;
        // A row j: block blk of the group, local sub-block sloc; in step st it carries sub-block st when
        // st % SL == sloc and is zero otherwise
        const uint32_t base = lds_addr(img + (b0 + blk) * Q4K_IMG + g * 2 + part);
        const uint32_t zero = lds_addr(img + b0 * Q4K_IMG + 64);
        uint32_t pa[8];
#pragma unroll
        for (int st = 0; st < 8; st++) {
            const uint64_t m16 = RS == 2 ? (0x0303ull << (2 * (st & 3))) : (0x3333ull << (2 * (st & 1)));
            pa[st] = sel_lanes(m16 * 0x0001000100010001ull, base + st * 8 * 16, zero);
        }
        constexpr int RING = 4;
        uint4 ring[RING];
        auto operand = [&](int t) { return lds_read16(pa[t % 8] + (t / 8) * RS * Q4K_IMG * 16); };
#pragma unroll
        for (int t = 0; t < RING; t++) ring[t] = operand(t);
        const uint32_t LO = 0x000F000Fu, HI = 0x00F000F0u;
        // accumulator entries (rows 4 g .. 4 g + 3, column j) belong together when both name the same block
        const bool valid = g / (4 / RS) == blk;
        const float *psf = sf + (b0 + blk) * 16;
        float acc = 0.f, mins = 0.f;
#pragma unroll
        for (int r = 0; r < PER; r++) {
            floatx4 dd[RS], dsum[RS];
            const uint4 one = make_uint4(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u); // f16 1.0
            half8 ov;
            __builtin_memcpy(&ov, &one, 16);
#pragma unroll
            for (int a = 0; a < RS; a++) {
                dd[a] = floatx4{0.f, 0.f, 0.f, 0.f};
                const uint4 ao = lds_read16(base + ((a * SL + sloc) * 8 + r * RS * Q4K_IMG) * 16);
                half8 av;
                __builtin_memcpy(&av, &ao, 16);
                dsum[a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, ov, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            }
#pragma unroll
            for (int st = 0; st < 8; st++) {
                const int t = r * 8 + st;
                half8 av, bv;
                const uint4 ao = ring[t % RING];
                __builtin_memcpy(&av, &ao, 16);
                const uint4 wq = (st & 4) ? w[0][r].qb : w[0][r].qa;
                const uint32_t w0 = (st & 2) ? wq.z : wq.x, w1 = (st & 2) ? wq.w : wq.y;
                const uint32_t msk = (st & 1) ? HI : LO;
                const uint4 bo = make_uint4(w0 & msk, (w0 >> 8) & msk, w1 & msk, (w1 >> 8) & msk);
                __builtin_memcpy(&bv, &bo, 16);
                dd[st / SL] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, dd[st / SL], 0, 0, 0);
                if (t + RING < PER * 8) ring[t % RING] = operand(t + RING);
            }
            const uint4 h = w[0][r].h;
            const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
            const uint32_t sc_l = h.y & 0x3F3F3F3Fu, sc_h = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
            const uint32_t mn_l = h.z & 0x3F3F3F3Fu, mn_h = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
#pragma unroll
            for (int a = 0; a < RS; a++) {
                // rows 4 g .. 4 g + 3 of accumulator a: sub-blocks s0, s0 + 1 (hi, lo each)
                const int s0 = a * SL + (2 * g) % SL;
                const float2 fc = *(const float2 *)(psf + r * RS * 16 + 8 + s0);
                const float sxa = (dsum[a][0] + dsum[a][1]) * (fc.x * 0x1p-24f);
                const float sxb = (dsum[a][2] + dsum[a][3]) * (fc.y * 0x1p-20f);
                const uint32_t scw = ((s0 & 4) ? sc_h : sc_l) >> ((s0 & 2) * 8);
                const uint32_t mnw = ((s0 & 4) ? mn_h : mn_l) >> ((s0 & 2) * 8);
                const float sca = (float)(scw & 0xFFu), scb = (float)((scw >> 8) & 0xFFu);
                const float mna = (float)(mnw & 0xFFu), mnb = (float)((mnw >> 8) & 0xFFu);
                acc = fmaf(dd[a][0] + dd[a][1], (sca * d) * fc.x, acc);
                acc = fmaf(dd[a][2] + dd[a][3], (scb * d) * fc.y, acc);
                mins = fmaf(mna * dmin, sxa, mins);
                mins = fmaf(mnb * dmin, sxb, mins);
            }
        }
        float v = rows_sum(valid ? acc - mins : 0.f);
        v += __shfl_xor(v, 8, 64); // the blocks of a row sit RW columns apart
        if (RS == 4) v += __shfl_xor(v, 4, 64);
        if (lane < RW) l_red[wave * 16 + lane] = v;
    } else {
        const int mysb = j >> 1, part = j & 1;
        // per-lane operand address of each step: its own sub-block's (hi|lo) in step mysb, the zero slot otherwise.
        // Lanes with (lane >> 1) % 8 == st are bits 2 st, 2 st + 1 of every 16.
        uint32_t pa[8];
        const uint32_t own = lds_addr(img + b0 * MR * Q4K_IMG + (mysb * 4 + g) * 2 + part);
        {
            const uint32_t zero = lds_addr(img + b0 * MR * Q4K_IMG + 64);
    #pragma unroll
            for (int st = 0; st < 8; st++) pa[st] = sel_lanes(0x0003000300030003ull << (2 * st), own, zero);
        }
        // the operands do not depend on the weights: RING of them are always on their way from the LDS
        constexpr int RING = 4;
        uint4 ring[RING];
        // operand number t = (block r, step st, row mr) in the order of use; its image is (r * MR + mr) after the base
        auto operand = [&](int t) {
            const int mr = t % MR, st = (t / MR) % 8, r = t / (8 * MR);
            return lds_read16(pa[st] + (r * MR + mr) * Q4K_IMG * 16);
        };
    #pragma unroll
        for (int t = 0; t < RING; t++) ring[t] = operand(t);
        const float *psf = sf + b0 * MR * 16 + 2 * g;
        const uint32_t LO = 0x000F000Fu, HI = 0x00F000F0u;
        // lane group g applies sub-blocks 2g, 2g+1: bytes (g&1)*2, +1 of the low (g < 2) or high (g >= 2) scale word
        const uint32_t selhi = (g & 2) ? 0xFFFFFFFFu : 0u;
        const int sh = (g & 1) * 16;
        float acc[TPW][MR], mins[TPW][MR];
    #pragma unroll
        for (int tp = 0; tp < TPW; tp++)
    #pragma unroll
            for (int mr = 0; mr < MR; mr++) acc[tp][mr] = mins[tp][mr] = 0.f;
    #pragma unroll
        for (int r = 0; r < PER; r++) {
            floatx4 dd[TPW][MR];
    #pragma unroll
            for (int tp = 0; tp < TPW; tp++)
    #pragma unroll
                for (int mr = 0; mr < MR; mr++) dd[tp][mr] = floatx4{0.f, 0.f, 0.f, 0.f};
            // rows 2s, 2s + 1 of dsum: the sum of the staged hi / lo values of sub-block s (the same in every
            // column, so one product serves all tiles)
            floatx4 dsum[ONES ? MR : 1];
            if constexpr (ONES) {
                const uint4 one = make_uint4(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u); // f16 1.0
                half8 ov;
                __builtin_memcpy(&ov, &one, 16);
    #pragma unroll
                for (int mr = 0; mr < MR; mr++) {
                    const uint4 ao = lds_read16(own + (r * MR + mr) * Q4K_IMG * 16);
                    half8 av;
                    __builtin_memcpy(&av, &ao, 16);
                    dsum[mr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, ov, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                }
            }
    #pragma unroll
            for (int st = 0; st < 8; st++) {
                const int t = (r * 8 + st) * MR;
                half8 av[MR];
    #pragma unroll
                for (int mr = 0; mr < MR; mr++) {
                    const uint4 ao = ring[(t + mr) % RING];
                    __builtin_memcpy(&av[mr], &ao, 16);
                }
    #pragma unroll
                for (int tp = 0; tp < TPW; tp++) {
                    const uint4 wq = FMT == FH_Q8_0 ? ((st >> 1) == 0 ? w[tp][r].qa : ((st >> 1) == 1 ? w[tp][r].qb : ((st >> 1) == 2 ? w[tp][r].qc : w[tp][r].qd)))
                                                     : ((st & 4) ? w[tp][r].qb : w[tp][r].qa);
                    uint4 bo;
                    if (FMT == FH_Q8_0) { // eight code bytes of block st -> f16 1152 + q, pairs in the order of the staging
                        const uint32_t c0 = ((st & 1) ? wq.z : wq.x) ^ 0x80808080u, c1 = ((st & 1) ? wq.w : wq.y) ^ 0x80808080u;
                        const uint32_t k64 = 0x64646464u;
                        bo = make_uint4(__builtin_amdgcn_perm(k64, c0, 0x04020400u), __builtin_amdgcn_perm(k64, c0, 0x04030401u),
                                        __builtin_amdgcn_perm(k64, c1, 0x04020400u), __builtin_amdgcn_perm(k64, c1, 0x04030401u));
                    } else if (Q40) { // one word per block: low nibbles, then high nibbles
                        const uint32_t w0 = (st & 3) == 0 ? wq.x : ((st & 3) == 1 ? wq.y : ((st & 3) == 2 ? wq.z : wq.w));
                        bo = make_uint4(w0 & LO, (w0 >> 8) & LO, w0 & HI, (w0 >> 8) & HI);
                        if constexpr (FMT == FH_Q5_0) {
                            // the block's byte of fifth bits: bits 0-3 for the low-nibble elements of the lane's four
                            // bytes, bits 4-7 for the high-nibble ones; a multiplication copies four bits to the two
                            // halves of a word, the mask keeps the one of each half (on bit 4 / 8 of the 16-bit code)
                            const uint32_t hw = ((st & 4) ? w[tp][r].qc.y : w[tp][r].qc.x) >> (8 * (st & 3));
                            const uint32_t l4 = hw & 0xFu, h4 = (hw >> 4) & 0xFu;
                            bo.x |= (l4 * 0x40010u) & 0x00100010u;
                            bo.y |= (l4 * 0x20008u) & 0x00100010u;
                            bo.z |= (h4 * 0x400100u) & 0x01000100u;
                            bo.w |= (h4 * 0x200080u) & 0x01000100u;
                        }
                    } else {
                        const uint32_t w0 = (st & 2) ? wq.z : wq.x, w1 = (st & 2) ? wq.w : wq.y;
                        const uint32_t msk = (st & 1) ? HI : LO;
                        bo = make_uint4(w0 & msk, (w0 >> 8) & msk, w1 & msk, (w1 >> 8) & msk);
                        if constexpr (FMT == FH_Q5_K) { // bit st of qh byte e is the fifth bit of element e in this step
                            const int pos = (st & 1) ? 8 : 4;
                            const uint32_t m5 = 0x00010001u << pos, hx = w[tp][r].qc.x, hy = w[tp][r].qc.y;
                            const int r0 = (st - pos) & 31, r1 = (8 + st - pos) & 31;
                            bo.x |= __builtin_amdgcn_alignbit(hx, hx, r0) & m5;
                            bo.y |= __builtin_amdgcn_alignbit(hx, hx, r1) & m5;
                            bo.z |= __builtin_amdgcn_alignbit(hy, hy, r0) & m5;
                            bo.w |= __builtin_amdgcn_alignbit(hy, hy, r1) & m5;
                        }
                    }
                    half8 bv;
                    __builtin_memcpy(&bv, &bo, 16);
    #pragma unroll
                    for (int mr = 0; mr < MR; mr++)
                        dd[tp][mr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[mr], bv, dd[tp][mr], 0, 0, 0);
                }
    #pragma unroll
                for (int mr = 0; mr < MR; mr++)
                    if (t + mr + RING < PER * 8 * MR) ring[(t + mr) % RING] = operand(t + mr + RING);
            }
    #pragma unroll
            for (int mr = 0; mr < MR; mr++) {
                const float2 fc = *(const float2 *)(psf + (r * MR + mr) * 16 + 8);
                float2 sx;
                if constexpr (ONES) { // odd sub-blocks are staged 16 times lower (their codes are 16 times higher)
                    sx.x = (dsum[mr][0] + dsum[mr][1]) * (fc.x * 0x1p-24f);
                    sx.y = (dsum[mr][2] + dsum[mr][3]) * (fc.y * 0x1p-20f);
                } else {
                    sx = *(const float2 *)(psf + (r * MR + mr) * 16);
                }
    #pragma unroll
                for (int tp = 0; tp < TPW; tp++) {
                    const uint4 h = w[tp][r].h;
                    if (Q40 || FMT == FH_Q8_0) {
                        const float off = FMT == FH_Q8_0 ? 1152.0f : (FMT == FH_Q5_0 ? 16.0f : 8.0f);
                        const float da = fh_h2f((uint16_t)(h.x & 0xFFFF)), db = fh_h2f((uint16_t)(h.x >> 16));
                        acc[tp][mr] = fmaf(dd[tp][mr][0] + dd[tp][mr][1], da * fc.x, acc[tp][mr]);
                        acc[tp][mr] = fmaf(dd[tp][mr][2] + dd[tp][mr][3], db * fc.y, acc[tp][mr]);
                        mins[tp][mr] = fmaf(off * da, sx.x, mins[tp][mr]);
                        mins[tp][mr] = fmaf(off * db, sx.y, mins[tp][mr]);
                        continue;
                    }
                    const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
                    const uint32_t sc_l = h.y & 0x3F3F3F3Fu, sc_h = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
                    const uint32_t mn_l = h.z & 0x3F3F3F3Fu, mn_h = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
                    const uint32_t scw = ((sc_l & ~selhi) | (sc_h & selhi)) >> sh;
                    const uint32_t mnw = ((mn_l & ~selhi) | (mn_h & selhi)) >> sh;
                    const float sca = (float)(scw & 0xFFu), scb = (float)((scw >> 8) & 0xFFu);
                    const float mna = (float)(mnw & 0xFFu), mnb = (float)((mnw >> 8) & 0xFFu);
                    const float sa = (sca * d) * fc.x, sb = (scb * d) * fc.y;
                    acc[tp][mr] = fmaf(dd[tp][mr][0] + dd[tp][mr][1], sa, acc[tp][mr]);
                    acc[tp][mr] = fmaf(dd[tp][mr][2] + dd[tp][mr][3], sb, acc[tp][mr]);
                    mins[tp][mr] = fmaf(mna * dmin, sx.x, mins[tp][mr]);
                    mins[tp][mr] = fmaf(mnb * dmin, sx.y, mins[tp][mr]);
                }
            }
        }
    #pragma unroll
        for (int mr = 0; mr < MR; mr++)
    #pragma unroll
            for (int tp = 0; tp < TPW; tp++) {
                const float v = rows_sum(acc[tp][mr] - mins[tp][mr]);
                if (lane < 16) l_red[((mr * TPW + tp) * SW + wave) * 16 + lane] = v;
            }
    }
    __syncthreads();
    if (tid < (RS > 1 ? 16 / RS : TOUT * 16 * MR)) {
        const int t = (tid >> 4) % TOUT, mr = (tid >> 4) / TOUT, jr = tid & 15;
        float v0 = 0.f, v1 = 0.f;
        for (int s = 0; s < SW; s++) {
            v0 += l_red[((mr * TPW + t) * SW + s) * 16 + jr];
            if (NT == 2) v1 += l_red[((t + TOUT) * SW + s) * 16 + jr];
        }
        if (IN == 1) {
            float tot = 0.f;
            for (int w2 = 0; w2 < SW; w2++) tot += l_ss[w2];
            const float rms = sqrtf(tot / (float)q.k + eps);
            v0 = v0 / rms;
            v1 = v1 / rms;
        }
        const int64_t row = RS > 1 ? (int64_t)(blockIdx.x / RS) * 16 + (int)(blockIdx.x % RS) * (16 / RS) + jr
                                   : ((int64_t)blockIdx.x * TOUT + t) * 16 + jr;
        if constexpr (HP) {
            const float up = __shfl_xor(v0, 8, 64); // column j + 8 is the up row of gate row j
            if (jr < 8) y[(int64_t)blockIdx.x * 8 + jr] = (v0 / (__expf(-v0) + 1.0f)) * up;
        } else if (EPI == FH_EPI_ROPEKV) {
            const float other = __shfl_xor(v0, 1, 64); // the pair (2i, 2i+1) sits in neighbouring lanes
            const int pos = *rk.pos;
            if (row < nout && pos < rk.cap) {
                const int r = (int)row;
                if (r < rk.qd + rk.kd) {
                    const int rh = r < rk.qd ? r : r - rk.qd, e = rh % rk.hd, i = e >> 1, half = rk.hd >> 1;
                    const int tp = pos < rk.table_rows ? pos : rk.table_rows - 1;
                    const float c = rk.cs[(int64_t)tp * half + i], sn = rk.sn[(int64_t)tp * half + i];
                    const float x0 = (r & 1) ? other : v0, x1 = (r & 1) ? v0 : other;
                    const float ac = x0 * c, bs = x1 * sn, as = x0 * sn, bc = x1 * c;
                    const float yv = (r & 1) ? as + bc : ac - bs;
                    if (r < rk.qd) rk.qo[r] = yv;
                    else {
                        const int64_t at = ((int64_t)(rh / rk.hd) * rk.cap + pos) * rk.hd + e;
                        if (rk.f16) ((_Float16 *)rk.kc)[at] = (_Float16)yv;
                        else ((float *)rk.kc)[at] = yv;
                    }
                } else {
                    const int rh = r - rk.qd - rk.kd;
                    const int64_t at = ((int64_t)(rh / rk.hd) * rk.cap + pos) * rk.hd + rh % rk.hd;
                    if (rk.f16) ((_Float16 *)rk.vc)[at] = (_Float16)v0;
                    else ((float *)rk.vc)[at] = v0;
                }
            }
        } else if (MR > 1) {
            if (row < nout && mr < nsplit) {
                // k split over gridDim.y workgroups: part p writes its own plane of 16 rows, a second launch adds them
                const int64_t at = (int64_t)mr * nout + row + (int64_t)blockIdx.y * 16 * nout;
                y[at] = EPI == FH_EPI_ADD2 ? (v0 + ea[at]) + eb[at] : v0;
            }
        } else if (row < nout) {
            float rr = v0;
            if (EPI == FH_EPI_ADD2) rr = (rr + ea[row]) + eb[row];
            if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * v1;
            if (EPI == FH_EPI_ACC) unsafeAtomicAdd(y + row, (blockIdx.y == 0 && ea) ? rr + ea[row] : rr);
            else y[row] = rr;
        }
    }
}

// The kernel proper.  With at most two block tiles per wavefront the register budget of eight wavefronts per SIMD
// (64 VGPRs) is enforced: the kernel lives on the number of bytes in flight per compute unit.
#define Q4K_M1_PARAMS                                                                                              \
    QView q, const float *__restrict__ x, float *__restrict__ y, const float *__restrict__ ea,                    \
        const float *__restrict__ eb, int SW, const float *__restrict__ xres, const float *__restrict__ nw, float eps, int nsplit, FhRopeArgs rk
template <int TPW, int PER, int EPI, int IN>
__global__ __launch_bounds__(1024) void k_qmv_q4k_m1(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FH_Q4_K, TPW, PER, EPI, IN>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}
template <int TPW, int PER, int EPI, int IN>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_qmv_q4k_m1_w8(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FH_Q4_K, TPW, PER, EPI, IN>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}
// 16 / RS rows of a tile per workgroup, RS blocks at once per wavefront (matrices with few row tiles)
template <int RS, int PER, int EPI, int IN>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_qmv_q4k_m1_rs(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FH_Q4_K, 1, PER, EPI, IN, 1, RS>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}
// 2 .. 4 activation rows (plain input; epilogues none / add2); nsplit = number of valid rows
template <int FMT, int TPW, int PER, int EPI, int MR>
__global__ __launch_bounds__(1024) void k_qmv_q4k_mr(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FMT, TPW, PER, EPI, 0, MR>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}
// Q4_0 / Q8_0 weights (plain input; epilogues none / add2 / SwiGLU)
template <int FMT, int TPW, int PER, int EPI>
__global__ __launch_bounds__(1024) void k_qmv_q40_m1(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FMT, TPW, PER, EPI, 0>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}
template <int FMT, int TPW, int PER, int EPI>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_qmv_q40_m1_w8(Q4K_M1_PARAMS) {
    qmv_q4k_m1_body<FMT, TPW, PER, EPI, 0>(q, x, y, ea, eb, SW, xres, nw, eps, nsplit, rk);
}

template <int TPW, int PER, int EPI>
static fh_status q4k_m1_launch(const fh_qmatrix *q, const float *x, float *y, const float *a, const float *b, int SW,
                               unsigned grid, size_t lds, const Q4kExtra &ex) {
    typedef void (*kern_t)(QView, const float *, float *, const float *, const float *, int, const float *, const float *,
                           float, int, FhRopeArgs);
    kern_t kern;
    const int in = ex.nsplit > 0 ? 2 : (ex.nw ? 1 : 0); // input: plain, rms_norm, attention partials
    if (q->type == FH_Q5_0) { // (17 registers of weights per block tile, as Q8_0)
        if constexpr ((EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2 || EPI == FH_EPI_SWIGLU) && !(EPI == FH_EPI_SWIGLU && TPW == 1)) {
            if (in != 0) return FH_ERR_UNSUPPORTED;
            if constexpr (TPW * PER == 1) kern = k_qmv_q40_m1_w8<FH_Q5_0, TPW, PER, EPI>;
            else kern = k_qmv_q40_m1<FH_Q5_0, TPW, PER, EPI>;
            FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
            kern<<<dim3(grid, 1), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, nullptr, nullptr, 0.f, 0,
                                                                        ex.rk);
            FH_HIP(hipGetLastError());
            return FH_OK;
        } else {
            return FH_ERR_UNSUPPORTED;
        }
    }
    if (q->type == FH_Q5_K) { // (14 registers of weights per block tile: budgeted like Q8_0)
        if constexpr ((EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2 || EPI == FH_EPI_SWIGLU) && !(EPI == FH_EPI_SWIGLU && TPW == 1)) {
            if (in != 0) return FH_ERR_UNSUPPORTED;
            if constexpr (TPW * PER == 1) kern = k_qmv_q40_m1_w8<FH_Q5_K, TPW, PER, EPI>;
            else kern = k_qmv_q40_m1<FH_Q5_K, TPW, PER, EPI>;
            FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
            kern<<<dim3(grid, 1), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, nullptr, nullptr, 0.f, 0,
                                                                        ex.rk);
            FH_HIP(hipGetLastError());
            return FH_OK;
        } else {
            return FH_ERR_UNSUPPORTED;
        }
    }
    if (q->type == FH_Q4_0 || q->type == FH_Q8_0) {
        if constexpr (EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2 || EPI == FH_EPI_SWIGLU) {
            if (in != 0) return FH_ERR_UNSUPPORTED;
            const bool q8 = q->type == FH_Q8_0;
            if constexpr (TPW * PER <= 2) { // Q8_0 holds 17 registers of weights per block tile: one fits the budget
                if constexpr (TPW * PER == 1) kern = q8 ? k_qmv_q40_m1_w8<FH_Q8_0, TPW, PER, EPI> : k_qmv_q40_m1_w8<FH_Q4_0, TPW, PER, EPI>;
                else kern = q8 ? k_qmv_q40_m1<FH_Q8_0, TPW, PER, EPI> : k_qmv_q40_m1_w8<FH_Q4_0, TPW, PER, EPI>;
            } else {
                kern = q8 ? k_qmv_q40_m1<FH_Q8_0, TPW, PER, EPI> : k_qmv_q40_m1<FH_Q4_0, TPW, PER, EPI>;
            }
            FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
            kern<<<dim3(grid, 1), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, nullptr, nullptr, 0.f, 0,
                                                                        ex.rk);
            FH_HIP(hipGetLastError());
            return FH_OK;
        } else {
            return FH_ERR_UNSUPPORTED;
        }
    }
    if constexpr (TPW * PER <= 2) {
        kern = in == 2 ? k_qmv_q4k_m1<TPW, PER, EPI, 2>
                       : (in == 1 ? k_qmv_q4k_m1_w8<TPW, PER, EPI, 1> : k_qmv_q4k_m1_w8<TPW, PER, EPI, 0>);
    } else if constexpr (EPI == FH_EPI_ACC && PER == 1) {
        kern = in == 2 ? k_qmv_q4k_m1<TPW, PER, EPI, 2>
                       : (in == 1 ? k_qmv_q4k_m1<TPW, PER, EPI, 1> : k_qmv_q4k_m1<TPW, PER, EPI, 0>);
    } else {
        if (in == 2) return FH_ERR_UNSUPPORTED; // the merge of the attention partials needs the registers
        kern = in == 1 ? k_qmv_q4k_m1<TPW, PER, EPI, 1> : k_qmv_q4k_m1<TPW, PER, EPI, 0>;
    }
    FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
    kern<<<dim3(grid, (unsigned)ex.ksplit), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, ex.xres,
                                                                                  ex.nw, ex.eps, ex.nsplit, ex.rk);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <int EPI>
static fh_status q4k_m1_launch_rs(int rs, int per, const fh_qmatrix *q, const float *x, float *y, const float *a,
                                  const float *b, int SW, unsigned grid, size_t lds, const Q4kExtra &ex) {
    if constexpr (EPI == FH_EPI_NONE || EPI == FH_EPI_ADD2) {
        typedef void (*kern_t)(QView, const float *, float *, const float *, const float *, int, const float *,
                               const float *, float, int, FhRopeArgs);
        kern_t kern = nullptr;
        if (rs == 2 && per == 1) kern = k_qmv_q4k_m1_rs<2, 1, EPI, 0>;
        else if (rs == 2 && per == 2) kern = k_qmv_q4k_m1_rs<2, 2, EPI, 0>;
        else if (rs == 4 && per == 1) kern = k_qmv_q4k_m1_rs<4, 1, EPI, 0>;
        else return FH_ERR_UNSUPPORTED;
        FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
        kern<<<dim3(grid, 1), dim3(64 * SW), lds, q->dev->stream>>>(fh_view(q), x, y, a, b, SW, ex.xres, ex.nw, ex.eps, 0,
                                                                    ex.rk);
        FH_HIP(hipGetLastError());
        return FH_OK;
    } else {
        return FH_ERR_UNSUPPORTED;
    }
}

// (tiles per wavefront, blocks per wavefront) with at most four block tiles (48 registers of weights) per wavefront
template <int EPI>
static fh_status q4k_m1_shape(int tpw, int per, const fh_qmatrix *q, const float *x, float *y, const float *a,
                              const float *b, int SW, unsigned grid, size_t lds, const Q4kExtra &ex) {
    if (tpw == 1 && per == 1) return q4k_m1_launch<1, 1, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    if (tpw == 1 && per == 2) return q4k_m1_launch<1, 2, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    if (tpw == 1 && per == 4) return q4k_m1_launch<1, 4, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    if (tpw == 2 && per == 1) return q4k_m1_launch<2, 1, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    if (tpw == 4 && per == 1) return q4k_m1_launch<4, 1, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    if constexpr (EPI != FH_EPI_ACC) {
        if (tpw == 2 && per == 2) return q4k_m1_launch<2, 2, EPI>(q, x, y, a, b, SW, grid, lds, ex);
    }
    return FH_ERR_UNSUPPORTED;
}

// Long k (the staged images of all rows of all of k do not fit the LDS, or more than 16 wavefronts): k in `parts`
// workgroups of at most 16 blocks each, one block per wavefront and two row tiles per workgroup, so that two
// workgroups fit a compute unit; every part writes its own plane and a second launch adds the planes in order and
// applies the epilogue.
template <int FMT, int EPI, int MR>
static fh_status q4k_mr_parts(const fh_qmatrix *q, const float *x, int m, float *y, const float *a, const float *b) {
    fh_device *dev = q->dev;
    const int kb = (int)(q->k / 256);
    int parts = 2;
    while (parts <= 16 && (kb % parts != 0 || kb / parts > 16)) parts++;
    if (parts > 16) return FH_ERR_UNSUPPORTED;
    const int SW = kb / parts;
    const size_t lds = (size_t)SW * MR * Q4K_IMG * 16 + (size_t)SW * MR * 64 + (size_t)MR * 2 * 16 * 64 + 64;
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED;
    const int64_t tiles = (q->n + 15) / 16;
    int tpw = (int)dev->opt_matvec_tiles;
    if (tpw != 1 && tpw != 2) tpw = tiles * parts > 2 * (int64_t)dev->compute_units ? 2 : 1;
    FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)parts * 16 * q->n * 4));
    typedef void (*kern_t)(QView, const float *, float *, const float *, const float *, int, const float *, const float *,
                           float, int, FhRopeArgs);
    const kern_t kern = tpw == 2 ? (kern_t)k_qmv_q4k_mr<FMT, 2, 1, FH_EPI_NONE, MR> : (kern_t)k_qmv_q4k_mr<FMT, 1, 1, FH_EPI_NONE, MR>;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
    kern<<<dim3((unsigned)((tiles + tpw - 1) / tpw), (unsigned)parts), dim3(64 * SW), lds, dev->stream>>>(
        fh_view(q), x, (float *)dev->ksplit_buf, nullptr, nullptr, SW, nullptr, nullptr, 0.f, m, FhRopeArgs{});
    FH_HIP(hipGetLastError());
    return fh_launch_kparts_reduce(dev, (const float *)dev->ksplit_buf, parts, m, q->n, y, EPI, a, b);
}

// y[m, n] for m = 2 .. 4 activation rows of a Q4_K matrix (epilogues none / add2): the weights are unpacked once
// for all rows.  Long k goes through q4k_mr_parts.
template <int FMT, int EPI, int MR>
static fh_status q4k_mr_go(const fh_qmatrix *q, const float *x, int m, float *y, const float *a, const float *b) {
    fh_device *dev = q->dev;
    const int kb = (int)(q->k / 256);
    int per = 1;
    while (kb / per > 16 && per < 2 && kb % (per * 2) == 0) per *= 2;
    const int SW = kb / per;
    if (kb % per) return FH_ERR_UNSUPPORTED;
    const size_t lds = (size_t)kb * MR * Q4K_IMG * 16 + (size_t)kb * MR * 64 + (size_t)MR * 2 * 16 * 64 + 64;
    if (SW > 16 || lds > 160 * 1024) return q4k_mr_parts<FMT, EPI, MR>(q, x, m, y, a, b);
    const int64_t tiles = (q->n + 15) / 16;
    // two row tiles per wavefront (one staging for both) once there are more tiles than compute units
    int tpw = (int)dev->opt_matvec_tiles;
    if (tpw != 1 && tpw != 2) tpw = tiles > dev->compute_units ? 2 : 1;
    if (per == 2) tpw = 1;
    const unsigned grid = (unsigned)((tiles + tpw - 1) / tpw);
    typedef void (*kern_t)(QView, const float *, float *, const float *, const float *, int, const float *, const float *,
                           float, int, FhRopeArgs);
    const kern_t kern = per == 2 ? (kern_t)k_qmv_q4k_mr<FMT, 1, 2, EPI, MR>
                                 : (tpw == 2 ? (kern_t)k_qmv_q4k_mr<FMT, 2, 1, EPI, MR> : (kern_t)k_qmv_q4k_mr<FMT, 1, 1, EPI, MR>);
    FH_TRY(fh_kernel_lds(q->dev, (const void *)kern, 160 * 1024));
    kern<<<dim3(grid, 1), dim3(64 * SW), lds, dev->stream>>>(fh_view(q), x, y, a, b, SW, nullptr, nullptr, 0.f, m, FhRopeArgs{});
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <int FMT>
static fh_status q4k_rows_fmt(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a, const float *b) {
    if (epi == FH_EPI_ADD2)
        return m == 2 ? q4k_mr_go<FMT, FH_EPI_ADD2, 2>(q, x, m, y, a, b) : q4k_mr_go<FMT, FH_EPI_ADD2, 4>(q, x, m, y, a, b);
    return m == 2 ? q4k_mr_go<FMT, FH_EPI_NONE, 2>(q, x, m, y, a, b) : q4k_mr_go<FMT, FH_EPI_NONE, 4>(q, x, m, y, a, b);
}

fh_status fh_launch_q4k_rows(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a, const float *b) {
    if (m < 2 || m > 4 || (epi != FH_EPI_NONE && epi != FH_EPI_ADD2)) return FH_ERR_UNSUPPORTED;
    if (q->type != FH_Q4_K && !((q->type == FH_Q4_0 || q->type == FH_Q8_0) && q->k % 256 == 0)) return FH_ERR_UNSUPPORTED;
    // three or four rows of a very tall matrix: the batch kernel (four tiles share one staging) measured better
    if (m > 2 && (q->n + 15) / 16 > 4 * (int64_t)q->dev->compute_units) return FH_ERR_UNSUPPORTED;
    if (q->type == FH_Q4_0) return q4k_rows_fmt<FH_Q4_0>(q, x, m, y, epi, a, b);
    if (q->type == FH_Q8_0) return q4k_rows_fmt<FH_Q8_0>(q, x, m, y, epi, a, b);
    return q4k_rows_fmt<FH_Q4_K>(q, x, m, y, epi, a, b);
}

// Returns FH_ERR_UNSUPPORTED when the shape does not fit this kernel (the caller falls back).
fh_status fh_launch_q4k_m1(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b) {
    return fh_launch_q4k_m1_norm(q, x, nullptr, nullptr, 0.f, y, epi, a, b);
}

static fh_status q4k_m1_any(const fh_qmatrix *q, const float *x, const Q4kExtra &ex, float *y, int epi, const float *a,
                            const float *b);

// The same product with the input merged from the partial results of the decode-step attention
// (x = [head][nsplit][128 + 4]; head_dim 128, nsplit <= 8).
fh_status fh_launch_q4k_m1_attn(const fh_qmatrix *q, const float *part, int nsplit, float *y) {
    if (nsplit < 1 || nsplit > 8 || q->k % 128) return FH_ERR_UNSUPPORTED;
    Q4kExtra ex;
    ex.nsplit = nsplit;
    return q4k_m1_any(q, part, ex, y, FH_EPI_NONE, nullptr, nullptr);
}

// y += W . merged attention partials, k split over `ksplit` workgroups per row tile (atomic adds: the summation
// order, and with it the last bits, vary from run to run).  The output projection of a decode step accumulating
// into the residual stream.
fh_status fh_launch_q4k_m1_attn_acc(const fh_qmatrix *q, const float *part, int nsplit, float *y_inout) {
    if (nsplit < 1 || nsplit > 8 || q->k % 128) return FH_ERR_UNSUPPORTED;
    Q4kExtra ex;
    ex.nsplit = nsplit;
    ex.ksplit = q->dev->opt_matvec_splitk > 0 ? (int)q->dev->opt_matvec_splitk : (q->kb % 4 == 0 ? (int)(q->kb / 4) : 0);
    if (ex.ksplit < 2) return FH_ERR_UNSUPPORTED;
    return q4k_m1_any(q, part, ex, y_inout, FH_EPI_ACC, nullptr, nullptr);
}

// The same product with the input taken as rms_norm(x [+ xres]) * nw when nw is given.
fh_status fh_launch_q4k_m1_norm(const fh_qmatrix *q, const float *x, const float *xres, const float *nw, float eps,
                                float *y, int epi, const float *a, const float *b) {
    Q4kExtra ex;
    ex.xres = xres;
    ex.nw = nw;
    ex.eps = eps;
    return q4k_m1_any(q, x, ex, y, epi, a, b);
}

// The fused q|k|v projection of a decode step: rms_norm(x) * nw as input (nw may be NULL: plain x), rotated
// query rows to q_out, rotated key rows and value rows into the cache row of the device-side position.
fh_status fh_launch_q4k_m1_ropekv(const fh_qmatrix *q, const float *x, const float *nw, float eps, fh_kvcache *c,
                                  int layer, int hq, const float *cos_t, const float *sin_t, int table_rows,
                                  float *q_out) {
    const int hd = c->head_dim, qd = hq * hd, kd = c->kv_heads * hd;
    if (q->n != qd + 2 * kd || hd % 16) return FH_ERR_UNSUPPORTED;
    const size_t plane = (size_t)c->kv_heads * c->capacity * hd * fh_dtype_size(c->dtype);
    Q4kExtra ex;
    ex.nw = nw;
    ex.eps = eps;
    ex.rk = FhRopeArgs{cos_t, sin_t, c->len_dev, q_out, (uint8_t *)c->k + layer * plane, (uint8_t *)c->v + layer * plane,
                       qd, kd, hd, c->capacity, table_rows, c->dtype == FH_F16 ? 1 : 0};
    return q4k_m1_any(q, x, ex, nullptr, FH_EPI_ROPEKV, nullptr, nullptr);
}

static fh_status q4k_m1_any(const fh_qmatrix *q, const float *x, const Q4kExtra &ex, float *y, int epi, const float *a,
                            const float *b) {
    fh_device *dev = q->dev;
    if (q->type != FH_Q4_K && !((q->type == FH_Q4_0 || q->type == FH_Q8_0) && q->k % 256 == 0 && ex.ksplit == 1) &&
        !((q->type == FH_Q5_K || (q->type == FH_Q5_0 && q->k % 256 == 0)) && ex.ksplit == 1 && !ex.nw && ex.nsplit == 0))
        return FH_ERR_UNSUPPORTED;
    const int64_t kb256 = q->k / 256; // 256-element blocks (Q4_0: eight of its 32-blocks, two records)
    if (ex.ksplit < 1 || kb256 % ex.ksplit || (ex.ksplit > 1 && (epi != FH_EPI_ACC || ex.nw))) return FH_ERR_UNSUPPORTED;
    const int kb = (int)kb256 / ex.ksplit; // blocks per workgroup
    const int nt = epi == FH_EPI_SWIGLU ? 2 : 1;
    const int64_t nout = epi == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int64_t tiles = (nout + 15) / 16;
    // Few row tiles (k / v projections): 16 / rs rows per workgroup, rs blocks at once per wavefront, so that the
    // launch has rs times the workgroups
    if (q->type == FH_Q4_K && (epi == FH_EPI_NONE || epi == FH_EPI_ADD2) && ex.nsplit == 0 && ex.ksplit == 1 && !ex.nw) {
        int rs = (int)dev->opt_matvec_rowsplit;
        if (rs != 1 && rs != 2 && rs != 4) rs = tiles * 2 <= dev->compute_units ? 2 : 1; // measured: 4 parts gain nothing over 2
        int per = (int)dev->opt_matvec_per == 2 && rs == 2 ? 2 : 1;
        while (rs > 1 && kb % (rs * per)) rs /= 2;
        while (kb / (rs * per) > 16 && rs == 2 && per == 1 && kb % 4 == 0) per = 2;
        if (rs > 1 && kb / (rs * per) <= 16) {
            const size_t lds = (size_t)kb * Q4K_IMG * 16 + (size_t)kb * 64 + 16 * 64 + 64;
            if (lds <= 160 * 1024) {
                const int SW = kb / (rs * per);
                const unsigned grid = (unsigned)(tiles * rs);
                if (epi == FH_EPI_ADD2) return q4k_m1_launch_rs<FH_EPI_ADD2>(rs, per, q, x, y, a, b, SW, grid, lds, ex);
                return q4k_m1_launch_rs<FH_EPI_NONE>(rs, per, q, x, y, a, b, SW, grid, lds, ex);
            }
        }
    }
    // tiles per wavefront (they share the staged activations and every operand read): two once there are more
    // tiles than compute units; the SwiGLU epilogue needs the gate and the up tile in one wavefront
    int tpw = (int)dev->opt_matvec_tiles;
    if (tpw != 1 && tpw != 2 && tpw != 4) tpw = tiles > dev->compute_units ? 2 : 1;
    // SwiGLU: half a gate tile and half an up tile per wavefront when the rows allow it (workgroups half as heavy)
    const bool half_pairs = epi == FH_EPI_SWIGLU && nout % 16 == 0 && dev->opt_matvec_tiles <= 1 && q->type != FH_Q5_K && q->type != FH_Q5_0;
    if (epi == FH_EPI_SWIGLU) tpw = half_pairs ? 1 : (tpw < 2 ? 2 : tpw);
    if (ex.nsplit > 0) { // merging attention partials: every workgroup merges its slice again, so fewer, fatter ones
        tpw = (int)dev->opt_wo_tiles;
        if (tpw != 1 && tpw != 2 && tpw != 4) tpw = 4;
        if (epi != FH_EPI_ACC) tpw = 1;
    } else if (epi == FH_EPI_ACC) tpw = 1;
    // blocks per wavefront (all requested up front): one wavefront per block as long as 16 wavefronts cover k
    int per = (int)dev->opt_matvec_per;
    if (per != 1 && per != 2 && per != 4) per = half_pairs ? 2 : 1;
    while (per > 1 && (kb % per || tpw * per > (ex.nsplit > 0 ? 2 : 4))) per /= 2;
    while (kb / per > 16 && tpw * per < 4 && kb % (per * 2) == 0) per *= 2; // the kernel wants SW * PER == kb
    while (kb / per > 16 && tpw > nt && kb % (per * 2) == 0) { // long k: fewer tiles, more blocks per wavefront
        tpw /= 2;
        per *= 2;
    }
    const int SW = kb / per;
    if (SW > 16 || kb % per || tpw * per > 4) return FH_ERR_UNSUPPORTED;
    size_t lds = (size_t)kb * Q4K_IMG * 16 + (size_t)kb * 64 + (size_t)tpw * 16 * 64 + 64;
    if (lds > 160 * 1024) return FH_ERR_UNSUPPORTED;
    const int tout = half_pairs ? 1 : tpw / nt;
    unsigned grid = half_pairs ? (unsigned)(2 * tiles) : (unsigned)((tiles + tout - 1) / tout);
    switch (epi) {
    case FH_EPI_SWIGLU: return q4k_m1_shape<FH_EPI_SWIGLU>(tpw, per, q, x, y, a, b, SW, grid, lds, ex);
    case FH_EPI_ADD2: return q4k_m1_shape<FH_EPI_ADD2>(tpw, per, q, x, y, a, b, SW, grid, lds, ex);
    case FH_EPI_ACC: return q4k_m1_shape<FH_EPI_ACC>(tpw, per, q, x, y, a, b, SW, grid, lds, ex);
    case FH_EPI_ROPEKV: return q4k_m1_shape<FH_EPI_ROPEKV>(tpw, per, q, x, y, a, b, SW, grid, lds, ex);
    default: return q4k_m1_shape<FH_EPI_NONE>(tpw, per, q, x, y, a, b, SW, grid, lds, ex);
    }
}

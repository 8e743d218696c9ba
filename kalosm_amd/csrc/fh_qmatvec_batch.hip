// Decode-side quantized matmul for 1..16 activation rows, all four block formats, on the matrix cores.
//   Y[m, n] = sum_k X[m, k] * deq(W)[n, k]          (fusor-ml/cpu/src/quantized.rs:246-675)
//
// One v_mfma_f32_16x16x32_f16 multiplies 16 activation rows (A operand: row m = lane % 16, k = 8 * (lane / 16) .. +8)
// with 16 weight rows (B operand: column n = lane % 16, same k), so a lane ends up with the outputs of ONE weight
// row and FOUR activation rows (m = 4 * (lane / 16) + i): the per-block weight scale is a per-lane scalar.
//
// Exactness: a weight code c (4, 6 or 8 bits) is used as the f16 subnormal c * 2^-24 straight from a mask of the
// packed bytes; each 256-element chunk of an activation row is scaled by a power of two into the f16 range and
// split into f16 hi + lo, so code * activation products are exact and accumulate in f32.  The block scale
// (d * sc, d) multiplies the per-block MFMA result, the block offset (dmin * m, 32 * d * sc, 8 * d, 128 * d)
// multiplies the f32 sum of the block's activations: the same algebra as GgufBlock::dequantize followed by the
// dot product, re-associated.
//
// A workgroup of TW x TS wavefronts owns TW row tiles (16 rows each) and all of k: in round r wavefront (tw, ts)
// multiplies tile tw with the 256-element chunk r * TS + ts.  The TS chunks of a round are staged once in LDS for
// all tiles (double buffered, one barrier per round); every wavefront keeps the weights of its next D chunks in
// flight (the kernel is bound by memory latency, not by arithmetic).  The slices are added through LDS in a fixed
// order and the epilogue is applied at the store.
#include "fh_blocks.h"

#include <algorithm>
#include <type_traits>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define QB_DPP_XOR1 0xB1         // quad_perm [1,0,3,2]
#define QB_DPP_XOR2 0x4E         // quad_perm [2,3,0,1]
#define QB_DPP_HALF_MIRROR 0x141 // lane i <- lane 7-i within each group of 8
template <int CTRL>
__device__ __forceinline__ float qb_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}

// LDS image of one staged chunk (bytes): activation planes [plane][MR rows][ROW], group sums [NG][16], factors [16].
// MFMA rows m >= MR read row m % MR: they produce values that are never stored.
template <int T, int MR>
struct QbLds {
    static constexpr int NG = T == FH_Q6_K ? 16 : 8;     // offset groups per chunk
    static constexpr int ROW = T == FH_Q6_K ? 520 : 264; // halfs per plane row (dword stride = 4 mod 64)
    static constexpr int PLANES = T == FH_Q6_K ? 1 : 2;  // Q6_K interleaves hi | lo per 16-group
    static constexpr int PLANE = MR * ROW;               // halfs
    static constexpr int S_OFF = PLANES * PLANE * 2, F_OFF = S_OFF + NG * 16 * 4, BYTES = F_OFF + 64;
};

// ------------------------------------------------------------------------------ weights of one (tile, chunk)
template <int T>
struct QbW;
template <>
struct QbW<FH_Q4_K> {
    uint4 a, b, h;
    __device__ __forceinline__ void load(const QView &q, int64_t tile, int c, int lane) {
        const uint8_t *rec = q.data + (tile * q.recs + c) * 2304;
        h = *(const uint4 *)(rec + 16 * (lane & 15));
        a = *(const uint4 *)(rec + 256 + lane * 16);
        b = *(const uint4 *)(rec + 1280 + lane * 16);
    }
};
template <>
struct QbW<FH_Q6_K> {
    uint4 l0, l1, hh;
    uint32_t sc[4];
    uint32_t d;
    __device__ __forceinline__ void load(const QView &q, int64_t tile, int c, int lane) {
        const uint8_t *rec = q.data + (tile * q.recs + c) * 3360;
        const int j = lane & 15;
        l0 = *(const uint4 *)(rec + lane * 16);
        l1 = *(const uint4 *)(rec + 1024 + lane * 16);
        hh = *(const uint4 *)(rec + 2048 + lane * 16);
#pragma unroll
        for (int qd = 0; qd < 4; qd++) sc[qd] = *(const uint32_t *)(rec + 3072 + (qd * 16 + j) * 4);
        d = fh_ld16(rec + 3328 + 2 * j);
    }
};
template <>
struct QbW<FH_Q8_0> {
    uint4 w[4];
    uint32_t d[4];
    __device__ __forceinline__ void load(const QView &q, int64_t tile, int c, int lane) {
        const uint8_t *rec = q.data + (tile * q.recs + 4 * c) * 1088;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            w[r] = *(const uint4 *)(rec + r * 1088 + lane * 16);
            d[r] = *(const uint32_t *)(rec + r * 1088 + 1024 + 4 * (lane & 15));
        }
    }
};
template <>
struct QbW<FH_Q4_0> {
    uint4 w[2];
    uint2 d[2];
    __device__ __forceinline__ void load(const QView &q, int64_t tile, int c, int lane) {
        const uint8_t *rec = q.data + (tile * q.recs + 2 * c) * 1152;
#pragma unroll
        for (int r = 0; r < 2; r++) {
            w[r] = *(const uint4 *)(rec + r * 1152 + lane * 16);
            d[r] = *(const uint2 *)(rec + r * 1152 + 1024 + 8 * (lane & 15));
        }
    }
};

__device__ __forceinline__ half8 qb_h8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const uint4 u = make_uint4(a, b, c, d);
    half8 v;
    __builtin_memcpy(&v, &u, 16);
    return v;
}

// ------------------------------------------------------------------------------ one chunk of one tile
// Where the activation operands of a chunk come from: `opnd(off)` is the A operand at half offset `off` of the
// lane's image row, `sum(off)` the four group sums at float offset `off`, `fac()` the four row factors.
template <int T, int MR>
struct QbLdsSrc { // a staged image in LDS
    typedef QbLds<T, MR> L;
    const _Float16 *xa;
    const float *S, *F;
    __device__ __forceinline__ QbLdsSrc(const uint8_t *img, int lane)
        : xa((const _Float16 *)img + ((lane & 15) & (MR - 1)) * L::ROW + 8 * (lane >> 4)),
          S((const float *)(img + L::S_OFF) + 4 * (lane >> 4)), F((const float *)(img + L::F_OFF) + 4 * (lane >> 4)) {}
    __device__ __forceinline__ half8 opnd(int off) const { return *(const half8 *)(xa + off); }
    __device__ __forceinline__ float4 sum(int off) const { return *(const float4 *)(S + off); }
    __device__ __forceinline__ float4 fac() const { return *(const float4 *)F; }
};

// Steps S0 .. S1-1 of the eight a chunk has (a 32-group each; Q6_K: two 16-groups each):
// tot[i] += scale * (codes . x_scaled), off[i] += offset * sum(x), for the rows m = 4g + i of the lane.
template <int T, int MR, int S0, int S1, class Src>
__device__ __forceinline__ void qb_steps(const QbW<T> &W, const Src &src, float *tot, float *off) {
    typedef QbLds<T, MR> L;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint32_t LO = 0x000F000Fu, HI = 0x00F000F0u;
    if constexpr (T == FH_Q4_K) {
        const float d = fh_h2f((uint16_t)(W.h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(W.h.x >> 16));
        const uint32_t sc_l = W.h.y & 0x3F3F3F3Fu, sc_h = (W.h.w & 0x0F0F0F0Fu) | ((W.h.y >> 2) & 0x30303030u);
        const uint32_t mn_l = W.h.z & 0x3F3F3F3Fu, mn_h = ((W.h.w >> 4) & 0x0F0F0F0Fu) | ((W.h.z >> 2) & 0x30303030u);
#pragma unroll
        for (int s = S0; s < S1; s++) {
            const uint4 wq = (s & 4) ? W.b : W.a;
            const uint32_t w0 = (s & 2) ? wq.z : wq.x, w1 = (s & 2) ? wq.w : wq.y;
            const uint32_t msk = (s & 1) ? HI : LO;
            const half8 bv = qb_h8(w0 & msk, (w0 >> 8) & msk, w1 & msk, (w1 >> 8) & msk);
            const half8 ah = src.opnd(32 * s), al = src.opnd(L::PLANE + 32 * s);
            floatx4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bv, zero, 0, 0, 0);
            r = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bv, r, 0, 0, 0);
            const float sc = (float)(((s < 4 ? sc_l : sc_h) >> (8 * (s & 3))) & 0xFFu);
            const float mn = (float)(((s < 4 ? mn_l : mn_h) >> (8 * (s & 3))) & 0xFFu);
            const float sw = (sc * d) * ((s & 1) ? 0.0625f : 1.0f), ow = mn * dmin; // high nibbles carry a factor 16
            const float4 sv = src.sum(16 * s);
            tot[0] = fmaf(sw, r[0], tot[0]); tot[1] = fmaf(sw, r[1], tot[1]);
            tot[2] = fmaf(sw, r[2], tot[2]); tot[3] = fmaf(sw, r[3], tot[3]);
            off[0] = fmaf(ow, sv.x, off[0]); off[1] = fmaf(ow, sv.y, off[1]);
            off[2] = fmaf(ow, sv.z, off[2]); off[3] = fmaf(ow, sv.w, off[3]);
        }
    } else if constexpr (T == FH_Q6_K) {
        const float d = fh_h2f((uint16_t)W.d);
#pragma unroll
        for (int t = S0; t < S1; t++) {
            const uint4 lq = (t & 4) ? W.l1 : W.l0;
            const uint32_t lw = (t & 3) == 0 ? lq.x : (t & 3) == 1 ? lq.y : (t & 3) == 2 ? lq.z : lq.w;
            const uint32_t hw = (t >> 1) == 0 ? W.hh.x : (t >> 1) == 1 ? W.hh.y : (t >> 1) == 2 ? W.hh.z : W.hh.w;
            uint32_t o[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int hs = q6k_hbit(t, p) - 4; // bring the two high bits of the pair to bits 4-5
                const uint32_t hb = hs >= 0 ? (hw >> hs) : (hw << (-hs));
                o[p] = ((lw >> (4 * p)) & LO) | (hb & 0x00300030u);
            }
            // lanes 0-31 hold the codes of group 2t, lanes 32-63 those of group 2t+1.  One operand per group with
            // its codes in both halves: they meet hi in lanes 0-31 and lo in lanes 32-63 of the activation operand
            // (v_permlane32_swap: first result = lanes 0-31 of the source in both halves, second = lanes 32-63).
            uint32_t oa[4], ob[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                auto sw2 = __builtin_amdgcn_permlane32_swap(o[p], o[p], false, false);
                oa[p] = sw2[0];
                ob[p] = sw2[1];
            }
            const half8 ba = qb_h8(oa[0], oa[1], oa[2], oa[3]), bb = qb_h8(ob[0], ob[1], ob[2], ob[3]);
            const half8 a0 = src.opnd(64 * t), a1 = src.opnd(64 * t + 32);
            const floatx4 r0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, ba, zero, 0, 0, 0);
            const floatx4 r1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bb, zero, 0, 0, 0);
            const uint32_t scw = W.sc[t & 3] >> (16 * (t >> 2));
            const float s0 = d * (float)(int)(int8_t)(scw & 0xFFu), s1 = d * (float)(int)(int8_t)((scw >> 8) & 0xFFu);
            const float4 v0 = src.sum(32 * t), v1 = src.sum(32 * t + 16);
            tot[0] = fmaf(s0, r0[0], tot[0]); tot[1] = fmaf(s0, r0[1], tot[1]);
            tot[2] = fmaf(s0, r0[2], tot[2]); tot[3] = fmaf(s0, r0[3], tot[3]);
            tot[0] = fmaf(s1, r1[0], tot[0]); tot[1] = fmaf(s1, r1[1], tot[1]);
            tot[2] = fmaf(s1, r1[2], tot[2]); tot[3] = fmaf(s1, r1[3], tot[3]);
            const float o0 = 32.f * s0, o1 = 32.f * s1;
            off[0] = fmaf(o0, v0.x, off[0]); off[1] = fmaf(o0, v0.y, off[1]);
            off[2] = fmaf(o0, v0.z, off[2]); off[3] = fmaf(o0, v0.w, off[3]);
            off[0] = fmaf(o1, v1.x, off[0]); off[1] = fmaf(o1, v1.y, off[1]);
            off[2] = fmaf(o1, v1.z, off[2]); off[3] = fmaf(o1, v1.w, off[3]);
        }
    } else {
#pragma unroll
        for (int s = S0; s < S1; s++) {
            half8 bv;
            float sw, ow;
            if constexpr (T == FH_Q8_0) {
                const uint4 wq = W.w[s >> 1];
                const uint32_t w0 = ((s & 1) ? wq.z : wq.x) ^ 0x80808080u, w1 = ((s & 1) ? wq.w : wq.y) ^ 0x80808080u;
                bv = qb_h8(__builtin_amdgcn_perm(0, w0, 0x0C010C00u), __builtin_amdgcn_perm(0, w0, 0x0C030C02u),
                           __builtin_amdgcn_perm(0, w1, 0x0C010C00u), __builtin_amdgcn_perm(0, w1, 0x0C030C02u));
                const uint32_t dd = W.d[s >> 1];
                sw = fh_h2f((uint16_t)((s & 1) ? (dd >> 16) : (dd & 0xFFFF)));
                ow = 128.f * sw; // codes are q + 128
            } else {
                const uint4 wq = W.w[s >> 2];
                const uint32_t w0 = (s & 3) == 0 ? wq.x : (s & 3) == 1 ? wq.y : (s & 3) == 2 ? wq.z : wq.w;
                bv = qb_h8(w0 & LO, (w0 >> 8) & LO, (w0 >> 4) & LO, (w0 >> 12) & LO);
                const uint2 dd = W.d[s >> 2];
                const uint32_t dw = (s & 2) ? dd.y : dd.x;
                sw = fh_h2f((uint16_t)((s & 1) ? (dw >> 16) : (dw & 0xFFFF)));
                ow = 8.f * sw;
            }
            const half8 ah = src.opnd(32 * s), al = src.opnd(L::PLANE + 32 * s);
            floatx4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bv, zero, 0, 0, 0);
            r = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bv, r, 0, 0, 0);
            const float4 sv = src.sum(16 * s);
            tot[0] = fmaf(sw, r[0], tot[0]); tot[1] = fmaf(sw, r[1], tot[1]);
            tot[2] = fmaf(sw, r[2], tot[2]); tot[3] = fmaf(sw, r[3], tot[3]);
            off[0] = fmaf(ow, sv.x, off[0]); off[1] = fmaf(ow, sv.y, off[1]);
            off[2] = fmaf(ow, sv.z, off[2]); off[3] = fmaf(ow, sv.w, off[3]);
        }
    }
}

// yacc[i] += factor[m] * sum_blocks scale * (codes . x_scaled) - sum_blocks offset * sum(x), m = 4g + i.
template <int T, int MR>
__device__ __forceinline__ void qb_chunk(const QbW<T> &W, const uint8_t *img, int lane, float *yacc) {
    const QbLdsSrc<T, MR> src(img, lane);
    float tot[4] = {0.f, 0.f, 0.f, 0.f}, off[4] = {0.f, 0.f, 0.f, 0.f};
    qb_steps<T, MR, 0, 8>(W, src, tot, off);
    const float4 fv = src.fac();
    yacc[0] += fv.x * tot[0] - off[0];
    yacc[1] += fv.y * tot[1] - off[1];
    yacc[2] += fv.z * tot[2] - off[2];
    yacc[3] += fv.w * tot[3] - off[3];
}

// ------------------------------------------------------------------------------ staging of one activation row chunk
// The wavefront holds row m of the chunk, lane c elements 4c .. 4c+3.  Positions inside the LDS row follow the
// order in which the format's code masks deliver the weights of a lane (see qb_chunk).
// Image of one chunk for the kernel that reads its operands straight from memory: the sixteen A operands of a
// chunk in the order the multiply asks for them (32-group s: hi 2s, lo 2s+1; Q6_K: 16-group G: hi | lo in operand G),
// each as the 64 lanes' 16 bytes back to back (one fully used 1 KB request per operand), then sums and factors.
template <int T>
struct QdImg {
    static constexpr int NG = T == FH_Q6_K ? 16 : 8;
    static constexpr int S_OFF = 16 * 1024, F_OFF = S_OFF + NG * 16 * 4, BYTES = F_OFF + 64;
    // byte offset of half `pos` (a multiple of 4) of plane `plane` of row m
    __device__ static __forceinline__ int at(int pos, int plane, int m) {
        const int opnd = T == FH_Q6_K ? pos / 32 : 2 * (pos / 32) + plane;
        return (opnd * 64 + ((pos % 32) / 8) * 16 + m) * 16 + (pos % 8) * 2;
    }
};

template <int T, int MR, bool FRAG = false>
__device__ __forceinline__ void qb_stage(uint8_t *img, int m, int lane, float4 v) {
    typedef QbLds<T, MR> L;
    constexpr int S_OFF = FRAG ? QdImg<T>::S_OFF : L::S_OFF, F_OFF = FRAG ? QdImg<T>::F_OFF : L::F_OFF;
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, qb_dpp<QB_DPP_XOR1>(amax));
    amax = fmaxf(amax, qb_dpp<QB_DPP_XOR2>(amax));
    amax = fmaxf(amax, qb_dpp<QB_DPP_HALF_MIRROR>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 8, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
    int e = 141 - (int)((__float_as_uint(amax) >> 23) & 0xFFu); // 14 - floor(log2 amax); zero / inf / nan clamp
    e = e > 100 ? 100 : (e < -100 ? -100 : e);
    const float sc = __uint_as_float((uint32_t)(e + 127) << 23);
    const float xs[4] = {v.x * sc, v.y * sc, v.z * sc, v.w * sc};
    _Float16 hi[4], lo[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        hi[c] = (_Float16)xs[c];
        lo[c] = (_Float16)(xs[c] - (float)hi[c]);
    }
    const bool swap = T == FH_Q4_K || T == FH_Q4_0; // nibble masks deliver bytes 0,2 then 1,3 of a word
    const _Float16 oh[4] = {hi[0], swap ? hi[2] : hi[1], swap ? hi[1] : hi[2], hi[3]};
    const _Float16 ol[4] = {lo[0], swap ? lo[2] : lo[1], swap ? lo[1] : lo[2], lo[3]};
    uint2 ph, pl;
    __builtin_memcpy(&ph, oh, 8);
    __builtin_memcpy(&pl, ol, 8);
    _Float16 *row = (_Float16 *)img + m * L::ROW;
    float s4 = (v.x + v.y) + (v.z + v.w);
    s4 += qb_dpp<QB_DPP_XOR1>(s4);
    s4 += qb_dpp<QB_DPP_XOR2>(s4);
    float *S = (float *)(img + S_OFF);
    if (T == FH_Q6_K) {
        const int G = lane >> 2, e0 = 4 * (lane & 3);
        if constexpr (FRAG) {
            *(uint2 *)(img + QdImg<T>::at(32 * G + e0, 0, m)) = ph;
            *(uint2 *)(img + QdImg<T>::at(32 * G + 16 + e0, 0, m)) = pl;
        } else {
            *(uint2 *)(row + 32 * G + e0) = ph;
            *(uint2 *)(row + 32 * G + 16 + e0) = pl;
        }
        if ((lane & 3) == 0) S[G * 16 + m] = s4;
    } else {
        int pos = 4 * lane;
        if (T == FH_Q4_0) { // low nibbles are elements 0..15 of a block, high nibbles 16..31; a lane group has 4 + 4
            const int c = lane & 7;
            pos = 32 * (lane >> 3) + (c < 4 ? 8 * c : 8 * (c - 4) + 4);
        }
        if constexpr (FRAG) {
            *(uint2 *)(img + QdImg<T>::at(pos, 0, m)) = ph;
            *(uint2 *)(img + QdImg<T>::at(pos, 1, m)) = pl;
        } else {
            *(uint2 *)(row + pos) = ph;
            *(uint2 *)(row + L::PLANE + pos) = pl;
        }
        s4 += qb_dpp<QB_DPP_HALF_MIRROR>(s4);
        if ((lane & 7) == 0) S[(lane >> 3) * 16 + m] = s4;
    }
    if (lane == 0) ((float *)(img + F_OFF))[m] = __uint_as_float((uint32_t)(24 - e + 127) << 23);
}

// ------------------------------------------------------------------------------ kernel
// MR: activation rows held per image (4 or 16, m <= MR); TW x TS = 8 wavefronts; D weight chunks in flight.
// One wavefront per (chunk, row): the LDS image of every chunk, written to global memory [chunk][image bytes].
template <int T, int MR, bool FRAG = false>
__global__ __launch_bounds__(256) void k_qb_prep(const float *__restrict__ x, int M, int64_t K, uint8_t *__restrict__ out) {
    typedef QbLds<T, MR> L;
    constexpr int IMG = FRAG ? QdImg<T>::BYTES : (L::BYTES + 15) & ~15;
    const int lane = threadIdx.x & 63, m = blockIdx.y * 4 + (threadIdx.x >> 6), c = blockIdx.x;
    if (m >= M) return;
    const float4 v = *(const float4 *)(x + (int64_t)m * K + (int64_t)c * 256 + lane * 4);
    qb_stage<T, MR, FRAG>(out + (int64_t)c * IMG, m, lane, v);
}

template <int T, int MR, int TW, int TS, int EPI, bool PRE>
__global__ __launch_bounds__(512) void k_qmv_batch(QView q, const float *__restrict__ x,
                                                   const uint8_t *__restrict__ ximg, int M, float *__restrict__ y,
                                                   const float *__restrict__ ea, const float *__restrict__ eb) {
    typedef QbLds<T, MR> L;
    static_assert(TW * TS == 8, "eight wavefronts");
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1, TWO = TW / NT; // output tiles per workgroup
    constexpr int D = T == FH_Q6_K ? 2 : 4; // chunks of weights in flight per wavefront (register budget)
    constexpr int RPW = TS * MR / 8, NE = 256 * TW;
    constexpr int IMG = (L::BYTES + 15) & ~15, ROUND = TS * IMG;
    constexpr int OUT_BYTES = 8 * 16 * 17 * 4;
    constexpr int LDS_BYTES = 2 * ROUND > OUT_BYTES ? 2 * ROUND : OUT_BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, g = lane >> 4;
    const int tw = wave / TS, ts = wave % TS;
    const int64_t K = q.k;
    const int C = (int)(K >> 8), R = (C + TS - 1) / TS;
    const int64_t nout = NT == 2 ? q.n / 2 : q.n;
    const int64_t tiles_out = (nout + 15) / 16;
    int64_t to = (int64_t)blockIdx.x * TWO + (tw % TWO);
    if (to >= tiles_out) to = tiles_out - 1; // a tile past the end re-reads the last one; its rows are never stored
    const int64_t tile = to + (int64_t)(tw / TWO) * (nout / 16); // up tiles follow the gate tiles

    // Round images come either from f32 activations converted here (PRE = false; staging duty of this wavefront in
    // every round: items i = wave + 8r -> chunk slot i % TS, row i / TS) or as copies of images k_qb_prep wrote
    // (PRE = true: the conversion is done once per call instead of once per workgroup).
    constexpr int CPT = (ROUND / 16 + 511) / 512; // 16-byte pieces per thread and round
    constexpr int NXR = PRE ? CPT : RPW;
    float4 xr[2][NXR];
    auto load_x = [&](float4 *xv, int rr) {
        if constexpr (PRE) {
            const int valid = (C - rr * TS < TS ? C - rr * TS : TS) * (IMG / 16);
            const float4 *src = (const float4 *)ximg + (int64_t)rr * (ROUND / 16);
#pragma unroll
            for (int r = 0; r < CPT; r++) {
                const int i = tid + 512 * r;
                xv[r] = i < valid ? src[i] : make_float4(0, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                const int i = wave + 8 * r, slot = i % TS, m = i / TS, c = rr * TS + slot;
                // rows past M are not staged and chunks past C not multiplied: their loads repeat the last valid ones
                xv[r] = *(const float4 *)(x + (int64_t)(m < M ? m : M - 1) * K + (int64_t)(c < C ? c : C - 1) * 256 + lane * 4);
            }
        }
    };
    auto stage = [&](const float4 *xv, int rr) {
        uint8_t *base = lds + (rr & 1) * ROUND;
        if constexpr (PRE) {
#pragma unroll
            for (int r = 0; r < CPT; r++) {
                const int i = tid + 512 * r;
                if (i < ROUND / 16) ((float4 *)base)[i] = xv[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                const int i = wave + 8 * r, slot = i % TS, m = i / TS;
                if (m < M) qb_stage<T, MR>(base + slot * IMG, m, lane, xv[r]);
            }
        }
    };
    auto chunk_of = [&](int rr) {
        const int c = rr * TS + ts;
        return c < C ? c : C - 1; // a slice without a chunk in the last round re-reads the last one and skips the math
    };
    load_x(xr[0], 0);
    __builtin_amdgcn_sched_barrier(0); // the first activations stay ahead of the weights in the request order
    QbW<T> wr[D];
    // no branches around the first requests (a wait after a branch becomes a wait for everything in flight): a
    // slice with fewer than D rounds repeats its last chunk, a single round repeats its activations
#pragma unroll
    for (int d = 0; d < D; d++) wr[d].load(q, tile, chunk_of(d < R ? d : R - 1), lane);
    load_x(xr[1], R > 1 ? 1 : 0);
    __builtin_amdgcn_sched_barrier(0);
    stage(xr[0], 0);
    float yacc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < R; r0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            const int rr = r0 + d;
            if (rr < R) {
                __syncthreads(); // image rr is complete; the other buffer is no longer read
                if (rr + 2 < R) load_x(xr[d & 1], rr + 2);
                if (rr * TS + ts < C) qb_chunk<T, MR>(wr[d], lds + (rr & 1) * ROUND + ts * IMG, lane, yacc);
                if (rr + D < R) wr[d].load(q, tile, chunk_of(rr + D), lane);
                if (rr + 1 < R) stage(xr[(d + 1) & 1], rr + 1);
            }
        }
    }
    // ---- add the slices through LDS in a fixed order, then epilogue and store: element e = (tile, m, n)
    __syncthreads();
    float *o = (float *)lds; // [ts][tw][16][17]
#pragma unroll
    for (int i = 0; i < 4; i++) o[((ts * TW + tw) * 16 + 4 * g + i) * 17 + j] = yacc[i];
    __syncthreads();
    auto total = [&](int e) {
        const int at = ((e >> 8) * 16 + ((e >> 4) & 15)) * 17 + (e & 15);
        float s = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < TS; k2++) s += o[k2 * TW * 16 * 17 + at];
        return s;
    };
    for (int e = tid; e < NE / NT; e += 512) {
        const int t2 = e >> 8, m = (e >> 4) & 15, jn = e & 15;
        const int64_t n = ((int64_t)blockIdx.x * TWO + t2) * 16 + jn;
        if (m < M && n < nout) {
            float rr = total(e);
            const int64_t at = (int64_t)m * nout + n;
            if (EPI == FH_EPI_ADD2) rr = (rr + ea[at]) + eb[at];
            if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * total(e + NE / 2);
            y[at] = rr;
        }
    }
}

template <int T, int MR, int TW, int TS, int EPI>
static fh_status qb_launch(const fh_qmatrix *q, const float *x, int m, float *y, const float *a, const float *b) {
    constexpr int TWO = EPI == FH_EPI_SWIGLU ? TW / 2 : TW;
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q->n / 2 : q->n;
    const int64_t groups = ((nout + 15) / 16 + TWO - 1) / TWO;
    FH_REQUIRE(groups <= 0x7FFFFFFF, "matrix too large for one launch");
    fh_device *dev = q->dev;
    // Converting the activations costs about as much as multiplying one tile by them: with many workgroups or
    // many rows it is done once, in a launch of its own.
    const int64_t pre_opt = dev->opt_matvec_per; // 0 auto, 1 never, 2 always
    const bool pre = pre_opt == 2 || (pre_opt == 0 && m > 2);
    if (pre) {
        constexpr int IMG = (QbLds<T, MR>::BYTES + 15) & ~15;
        const int chunks = (int)(q->k / 256);
        FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, (size_t)chunks * IMG));
        k_qb_prep<T, MR><<<dim3((unsigned)chunks, (unsigned)((m + 3) / 4)), dim3(256), 0, dev->stream>>>(
            x, m, q->k, (uint8_t *)dev->act_buf);
        k_qmv_batch<T, MR, TW, TS, EPI, true><<<dim3((unsigned)groups), dim3(512), 0, dev->stream>>>(
            fh_view(q), x, (const uint8_t *)dev->act_buf, m, y, a, b);
    } else {
        k_qmv_batch<T, MR, TW, TS, EPI, false><<<dim3((unsigned)groups), dim3(512), 0, dev->stream>>>(
            fh_view(q), x, nullptr, m, y, a, b);
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ images read straight from memory
// A second kernel for the same product: one wavefront per (row tile(s), chunk), no staging.  The wavefront reads
// the activation operands of its chunk from the image k_qb_prep wrote (16 rows; it stays in the L2) half a chunk
// at a time into registers, requests its weights once, and multiplies.  Nothing waits for another wavefront until
// the slices are added, so a chunk costs one memory round trip instead of a staged round with a barrier.  Long k
// is cut into gridDim.y parts whose partial sums a second launch adds in a fixed order.
template <int T>
struct QdRegs {
    typedef QbLds<T, 16> L;
    static constexpr int NS = T == FH_Q6_K ? 8 : 4;
    half8 a[8];
    float4 s[NS];
    template <int H>
    __device__ __forceinline__ void load(const uint8_t *img, int lane) {
        const uint8_t *A = img + lane * 16;
        const float *S = (const float *)(img + QdImg<T>::S_OFF) + 4 * (lane >> 4);
        if constexpr (T == FH_Q6_K) {
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] = *(const half8 *)(A + (8 * H + i) * 1024);
#pragma unroll
            for (int i = 0; i < 8; i++) s[i] = *(const float4 *)(S + 16 * (8 * H + i));
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                a[i] = *(const half8 *)(A + (2 * (4 * H + i)) * 1024);
                a[4 + i] = *(const half8 *)(A + (2 * (4 * H + i) + 1) * 1024);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) s[i] = *(const float4 *)(S + 16 * (4 * H + i));
        }
    }
    // the second half from the wavefront's LDS copy: operands 8 .. 15 as 1 KB each, then the half's 64 group sums
    __device__ __forceinline__ void load_second_half_lds(const uint8_t *limg, int lane) {
        static_assert(T != FH_Q6_K, "layout of the two-plane formats");
        const uint8_t *A = limg + lane * 16;
        const float *S = (const float *)(limg + 8192) + 4 * (lane >> 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            a[i] = *(const half8 *)(A + (2 * i) * 1024);
            a[4 + i] = *(const half8 *)(A + (2 * i + 1) * 1024);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) s[i] = *(const float4 *)(S + 16 * i);
    }
    // the offsets qb_steps asks for, folded to register indices (its loops are unrolled: `off` is a constant)
    __device__ __forceinline__ half8 opnd(int off) const {
        if constexpr (T == FH_Q6_K) return a[(off / 32) & 7];
        else return off >= L::PLANE ? a[4 + (((off - L::PLANE) / 32) & 3)] : a[(off / 32) & 3];
    }
    __device__ __forceinline__ float4 sum(int off) const { return s[(off / 16) & (NS - 1)]; }
};

#define QD_LDS_IMG 8448 // bytes of LDS per wavefront for the second half of a chunk's image: 8 operands + 64 sums

template <int T, int TPW, int EPI>
__global__ __launch_bounds__(1024) void k_qmv_direct(QView q, const uint8_t *__restrict__ ximg, int M, int cps,
                                                     float *__restrict__ y, float *__restrict__ part,
                                                     const float *__restrict__ ea, const float *__restrict__ eb) {
    constexpr int IMG = QdImg<T>::BYTES;
    constexpr int NT = EPI == FH_EPI_SWIGLU ? 2 : 1, TOUT = TPW / NT;
    constexpr bool LDS_HALF = TPW == 4;
    extern __shared__ float qd_o[]; // [wavefront][TPW][16 rows][17]; with LDS_HALF first [wavefront][QD_LDS_IMG bytes]
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int j = lane & 15, g = lane >> 4, SW = blockDim.x >> 6;
    const int C = (int)(q.k >> 8);
    const int64_t nout = NT == 2 ? q.n / 2 : q.n, tiles_out = (nout + 15) / 16;
    const int c = blockIdx.y * cps + wave;
    float yacc[TPW][4];
#pragma unroll
    for (int tp = 0; tp < TPW; tp++)
#pragma unroll
        for (int i = 0; i < 4; i++) yacc[tp][i] = 0.f;
    if (wave < cps && c < C) { // uniform per wavefront
        const uint8_t *img = ximg + (size_t)c * IMG;
        QdRegs<T> a;
        a.template load<0>(img, lane);
        const float4 fv = *(const float4 *)((const float *)(img + QdImg<T>::F_OFF) + 4 * g);
        __builtin_amdgcn_sched_barrier(0); // activations (L2) are requested ahead of the weights (HBM)
        QbW<T> w[TPW];
#pragma unroll
        for (int tp = 0; tp < TPW; tp++) {
            int64_t to = (int64_t)blockIdx.x * TOUT + (tp % TOUT);
            if (to >= tiles_out) to = tiles_out - 1; // a tile past the end re-reads the last one; never stored
            w[tp].load(q, to + (int64_t)(tp / TOUT) * (nout / 16), c, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        // Four tiles per wavefront leave no registers for the second half of the image: it is requested now as well,
        // into the wavefront's 8448 bytes of LDS (LDS-direct loads: lane l's 16 bytes land at base + 16 l, which is
        // the operand layout), so that it is there when the first half has been multiplied.
        uint8_t *limg = (uint8_t *)qd_o + wave * QD_LDS_IMG;
        if constexpr (LDS_HALF) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                __builtin_amdgcn_global_load_lds((const uint32_t *)(img + (8 + i) * 1024 + lane * 16),
                                                 (__attribute__((address_space(3))) uint32_t *)(limg + i * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const uint32_t *)(img + QdImg<T>::S_OFF) + 64 + lane,
                                             (__attribute__((address_space(3))) uint32_t *)(limg + 8192), 4, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // each half of the chunk goes into the tile's output as soon as it is multiplied: the scaled sums and
        // offsets live for one half of one tile only
        auto half = [&](auto H) {
#pragma unroll
            for (int tp = 0; tp < TPW; tp++) {
                float tot[4] = {0.f, 0.f, 0.f, 0.f}, off[4] = {0.f, 0.f, 0.f, 0.f};
                qb_steps<T, 16, 4 * decltype(H)::value, 4 * decltype(H)::value + 4>(w[tp], a, tot, off);
                yacc[tp][0] += fv.x * tot[0] - off[0];
                yacc[tp][1] += fv.y * tot[1] - off[1];
                yacc[tp][2] += fv.z * tot[2] - off[2];
                yacc[tp][3] += fv.w * tot[3] - off[3];
            }
        };
        half(std::integral_constant<int, 0>{});
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (LDS_HALF) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            a.load_second_half_lds(limg, lane);
        } else {
            a.template load<1>(img, lane);
        }
        half(std::integral_constant<int, 1>{});
    }
    if constexpr (LDS_HALF) __syncthreads(); // the sums below reuse the image bytes of every wavefront
#pragma unroll
    for (int tp = 0; tp < TPW; tp++)
#pragma unroll
        for (int i = 0; i < 4; i++) qd_o[((wave * TPW + tp) * 16 + 4 * g + i) * 17 + j] = yacc[tp][i];
    __syncthreads();
    auto total = [&](int tp, int m, int jn) { // slices in wavefront order
        float s = 0.f;
        for (int w2 = 0; w2 < SW; w2++) s += qd_o[((w2 * TPW + tp) * 16 + m) * 17 + jn];
        return s;
    };
    if (part) { // partial sums of this k part, one row of `part` per (part, activation row): [gridDim.y][16][q.n]
        for (int e = tid; e < TPW * 256; e += blockDim.x) {
            const int tp = e >> 8, m = (e >> 4) & 15, jn = e & 15;
            const int64_t to = (int64_t)blockIdx.x * TOUT + (tp % TOUT);
            const int64_t row = (to + (int64_t)(tp / TOUT) * (nout / 16)) * 16 + jn;
            if (m < M && to < tiles_out && row < q.n) part[((int64_t)blockIdx.y * 16 + m) * q.n + row] = total(tp, m, jn);
        }
        return;
    }
    for (int e = tid; e < TOUT * 256; e += blockDim.x) {
        const int t2 = e >> 8, m = (e >> 4) & 15, jn = e & 15;
        const int64_t n = ((int64_t)blockIdx.x * TOUT + t2) * 16 + jn;
        if (m < M && n < nout) {
            float rr = total(t2, m, jn);
            const int64_t at = (int64_t)m * nout + n;
            if (EPI == FH_EPI_ADD2) rr = (rr + ea[at]) + eb[at];
            if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * total(t2 + TOUT, m, jn);
            y[at] = rr;
        }
    }
}

// y = epilogue(sum over the k parts), parts added in order.
template <int EPI>
__global__ __launch_bounds__(256) void k_qd_reduce(const float *__restrict__ part, int parts, int M, int64_t nfull,
                                                   int64_t nout, float *__restrict__ y, const float *__restrict__ ea,
                                                   const float *__restrict__ eb) {
    const int64_t at = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= (int64_t)M * nout) return;
    const int m = (int)(at / nout);
    const int64_t n = at % nout;
    float rr = 0.f, up = 0.f;
    for (int p = 0; p < parts; p++) {
        rr += part[((int64_t)p * 16 + m) * nfull + n];
        if (EPI == FH_EPI_SWIGLU) up += part[((int64_t)p * 16 + m) * nfull + nout + n];
    }
    if (EPI == FH_EPI_ADD2) rr = (rr + ea[at]) + eb[at];
    if (EPI == FH_EPI_SWIGLU) rr = (rr / (__expf(-rr) + 1.0f)) * up;
    y[at] = rr;
}

// The same sum for the k parts of another kernel: planes [parts][16][n], epilogue none / add2.
fh_status fh_launch_kparts_reduce(fh_device *dev, const float *part, int parts, int m, int64_t n, float *y, int epi,
                                  const float *a, const float *b) {
    const int64_t total = (int64_t)m * n;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (epi == FH_EPI_ADD2) k_qd_reduce<FH_EPI_ADD2><<<grid, block, 0, dev->stream>>>(part, parts, m, n, n, y, a, b);
    else if (epi == FH_EPI_NONE) k_qd_reduce<FH_EPI_NONE><<<grid, block, 0, dev->stream>>>(part, parts, m, n, n, y, a, b);
    else FH_FAIL(FH_ERR_UNSUPPORTED, "epilogue %d of a k-part sum", epi);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <int T, int EPI>
static fh_status qd_launch(const fh_qmatrix *q, const float *x, int m, float *y, const float *a, const float *b) {
    fh_device *dev = q->dev;
    constexpr int IMG = QdImg<T>::BYTES;
    const int C = (int)(q->k / 256);
    const int parts = (C + 15) / 16, cps = (C + parts - 1) / parts; // at most 16 wavefronts (chunks) per workgroup
    const int64_t nout = EPI == FH_EPI_SWIGLU ? q->n / 2 : q->n, tiles = (nout + 15) / 16;
    // two tiles per wavefront share the activation operands once the device is covered more than twice
    const int64_t force = dev->opt_matvec_tiles;
    // and four once that still leaves a workgroup for most compute units (every workgroup fetches the image of its
    // chunks), for the formats whose four tiles fit the 128 registers of a 16-wavefront workgroup
    const bool four = EPI != FH_EPI_SWIGLU && (T == FH_Q4_K || T == FH_Q4_0) && (force == 4 || (force == 0 && 2 * tiles * parts >= 7 * (int64_t)dev->compute_units));
    const bool two = !four && (EPI == FH_EPI_SWIGLU || force == 2 || (force == 0 && tiles * parts > 2 * (int64_t)dev->compute_units));
    const int64_t groups = EPI == FH_EPI_SWIGLU ? tiles : (four ? (tiles + 3) / 4 : two ? (tiles + 1) / 2 : tiles);
    FH_REQUIRE(groups <= 0x7FFFFFFF, "matrix too large for one launch");
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, (size_t)C * IMG));
    float *part = nullptr;
    if (parts > 1) {
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)parts * 16 * q->n * 4));
        part = (float *)dev->ksplit_buf;
    }
    k_qb_prep<T, 16, true><<<dim3((unsigned)C, (unsigned)((m + 3) / 4)), dim3(256), 0, dev->stream>>>(
        x, m, q->k, (uint8_t *)dev->act_buf);
    const dim3 grid((unsigned)groups, (unsigned)parts), block(64 * cps);
    const size_t lds = four ? std::max((size_t)cps * 4 * 16 * 17 * 4, (size_t)cps * QD_LDS_IMG) : (size_t)cps * (two ? 2 : 1) * 16 * 17 * 4;
    if (four) {
        if constexpr (EPI != FH_EPI_SWIGLU && (T == FH_Q4_K || T == FH_Q4_0)) {
            if (lds > 64 * 1024) FH_TRY(fh_kernel_lds(dev, (const void *)k_qmv_direct<T, 4, EPI>, lds));
            k_qmv_direct<T, 4, EPI><<<grid, block, lds, dev->stream>>>(fh_view(q), (const uint8_t *)dev->act_buf, m, cps, y,
                                                                      part, a, b);
        }
    } else if (two)
        k_qmv_direct<T, 2, EPI><<<grid, block, lds, dev->stream>>>(fh_view(q), (const uint8_t *)dev->act_buf, m, cps, y,
                                                                  part, a, b);
    else if constexpr (EPI != FH_EPI_SWIGLU)
        k_qmv_direct<T, 1, EPI><<<grid, block, lds, dev->stream>>>(fh_view(q), (const uint8_t *)dev->act_buf, m, cps, y,
                                                                  part, a, b);
    if (part) {
        const int64_t total = (int64_t)m * nout;
        k_qd_reduce<EPI><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream>>>(part, parts, m, q->n, nout, y,
                                                                                              a, b);
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// m <= 4: one tile (SwiGLU: gate + up tile) per workgroup, k over 8 (4) slices.  m <= 16: four tiles, two slices:
// the staged activations (4 bytes per element and row) are then shared by enough weight rows.
template <int T, int EPI>
static fh_status qb_shape(const fh_qmatrix *q, const float *x, int m, float *y, const float *a, const float *b) {
    const int64_t tiles = (q->n + 15) / 16;
    const int64_t force = q->dev->opt_matvec_tiles; // 0 auto, else tiles per workgroup
    if (m <= 4 && q->dev->opt_matvec_direct != 2) {
        if constexpr (EPI == FH_EPI_SWIGLU) return qb_launch<T, 4, 2, 4, EPI>(q, x, m, y, a, b);
        else {
            if (force == 2 || (force == 0 && tiles >= 512)) return qb_launch<T, 4, 2, 4, EPI>(q, x, m, y, a, b);
            return qb_launch<T, 4, 1, 8, EPI>(q, x, m, y, a, b);
        }
    }
    if (q->dev->opt_matvec_direct != 1) return qd_launch<T, EPI>(q, x, m, y, a, b);
    if (force == 2 || (force == 0 && tiles <= 512)) return qb_launch<T, 16, 2, 4, EPI>(q, x, m, y, a, b);
    return qb_launch<T, 16, 4, 2, EPI>(q, x, m, y, a, b);
}

template <int T>
static fh_status qb_epi(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a, const float *b) {
    if (epi == FH_EPI_ADD2) return qb_shape<T, FH_EPI_ADD2>(q, x, m, y, a, b);
    if (epi == FH_EPI_SWIGLU) return qb_shape<T, FH_EPI_SWIGLU>(q, x, m, y, a, b);
    return qb_shape<T, FH_EPI_NONE>(q, x, m, y, a, b);
}

bool fh_qmatvec_batch_supports(const fh_qmatrix *q, int m, int epi) {
    if (m < 1 || m > 16 || q->k % 256 != 0 || fh_single_row_only(q->type)) return false;
    if (epi == FH_EPI_SWIGLU && (q->n % 32) != 0) return false;
    return true;
}

fh_status fh_launch_qmatvec_batch(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                                  const float *b) {
    FH_REQUIRE(fh_qmatvec_batch_supports(q, m, epi), "shape not supported by the batch kernel");
    switch (q->type) {
    case FH_Q4_0: return qb_epi<FH_Q4_0>(q, x, m, y, epi, a, b);
    case FH_Q8_0: return qb_epi<FH_Q8_0>(q, x, m, y, epi, a, b);
    case FH_Q4_K: return qb_epi<FH_Q4_K>(q, x, m, y, epi, a, b);
    case FH_Q6_K: return qb_epi<FH_Q6_K>(q, x, m, y, epi, a, b);
    }
    FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported type %u", q->type);
}

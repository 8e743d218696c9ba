// Quantized matmul for many activation rows (prefill, and decode batches above 2) on the matrix cores:
//   Y[m, n] = sum_k X[m, k] * deq(W)[n, k]          (fusor-ml/cpu/src/quantized.rs:246-675)
//
// Tile kernel: a workgroup owns TN weight rows x TM activation rows and walks k in steps of 32.  Per step the
// 32-wide slab of the weight tile is decoded from the tiled GGUF layout with exactly the arithmetic of
// GgufBlock::dequantize (f32), split into an f16 pair hi + lo (w = hi + lo to 2^-22), and put in LDS; the
// activation slab comes from f16 planes prepared once per call (k_act_split: each row scaled by a power of
// two into the f16 range, hi + lo for f32 input, a single exact term for bf16 input).  The contraction runs on
// v_mfma_f32_32x32x16_f16 as  w_hi*x_hi + w_lo*x_hi (+ w_hi*x_lo)  with f32 accumulation, so the only
// deviation from the f32 reference is the summation order and the 2^-22 residues.
#include "fh_blocks.h"
#include <type_traits>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// lo half of the two-term f16 split of w whose hi half is h.  A non-finite w (inf, NaN) keeps its kind in h alone:
// inf - inf would put a NaN into the lo plane and turn every product of the row into NaN, where the reference's
// f32 arithmetic gives +-inf.
__device__ __forceinline__ _Float16 fh_split_lo(float w, _Float16 h) {
    const float d = w - (float)h;
    return (_Float16)(d == d ? d : 0.f);
}

// adds the two k halves of the tiles of a split last round (see k_qmm_tile2j) into y
__global__ void k_qmm_tail_sum(const float *__restrict__ planes, int tail, int full, int tiles_n, int m, int64_t n,
                               float *__restrict__ y);
// Tiles of the last round of workgroups that are worth splitting along k: more tiles than compute units and a
// remainder of at most half of them (matmul_kernel = 11: never)
static int qmm_tail_tiles(const fh_device *dev, int tiles) {
    const int cus = dev->compute_units;
    const int tail = tiles > cus ? tiles % cus : 0;
    return (tail * 2 > cus || dev->opt_matmul_kernel == 11) ? 0 : tail;
}

#define QMM_LDK 40 // halfs per LDS row: 32 + 8 padding (80 B stride: 16-byte reads of 16 rows hit 16 distinct chunks)
// The pipelined kernels use unpadded rows of 32 halfs (four 16-byte pieces) instead, piece c of row r at position
// c ^ ((r >> 2) & 3): the 16-byte reads of 16 consecutive rows at one c and the writes of four consecutive rows cover the
// 64 banks once.  QMM_AT(row, pos): half offset of position pos (0 .. 31) of row `row` inside a plane.
#define QMM_AT(row, pos) ((row) * 32 + 8 * ((((pos) >> 3)) ^ (((row) >> 2) & 3)) + ((pos) & 7))

// ------------------------------------------------------------------------------ activation planes
// One workgroup per row.  xh / xl are [m, kp] f16 (zero from k to kp), rs[m] = 2^-e undoes the normalisation at the
// store.  IN: 0 f32, 1 bf16, 2 f16 input; element c of row r is at r * srow + c * scol.
template <int IN>
__global__ __launch_bounds__(256) void k_act_split(const void *__restrict__ xin, int64_t srow, int64_t scol, int k, int kp,
                                                    _Float16 *__restrict__ xh, _Float16 *__restrict__ xl,
                                                    float *__restrict__ rs, _Float16 *__restrict__ xs = nullptr) {
    __shared__ float sh[4];
    const int64_t off = (int64_t)blockIdx.x * srow, oo = (int64_t)blockIdx.x * kp;
    auto ld = [&](int c) -> float {
        if (IN == 1) return __uint_as_float((uint32_t)((const uint16_t *)xin)[off + c * scol] << 16);
        if (IN == 2) return (float)((const _Float16 *)xin)[off + c * scol];
        return ((const float *)xin)[off + c * scol];
    };
    float amax = 0.f;
    for (int c = threadIdx.x; c < k; c += 256) amax = fmaxf(amax, fabsf(ld(c)));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    int e = 141 - (int)((__float_as_uint(amax) >> 23) & 0xFFu); // 14 - floor(log2 amax); zero / inf / nan clamp
    e = e > 100 ? 100 : (e < -100 ? -100 : e);
    const float sc = __uint_as_float((uint32_t)(e + 127) << 23);
    // A row with an infinity: its finite values vanish next to it (sc flushes them to zero), the infinity itself is
    // carried as +-32768 and the row's output scale is infinite, so that the product comes out as +-inf with the
    // sign of the reference's f32 sum (NaN where the other operand is zero or NaN) instead of inf * 0 = NaN from the
    // lo plane of the other operand.
    const bool infrow = amax == INFINITY;
    for (int c = threadIdx.x; c < kp; c += 256) {
        float v = c < k ? ld(c) * sc : 0.f;
        if (infrow && fabsf(v) == INFINITY) v = copysignf(32768.f, v);
        const _Float16 h = (_Float16)v;
        xh[oo + c] = h;
        if (IN != 1) xl[oo + c] = fh_split_lo(v, h);
        if (xs) { // (kp is a multiple of 256 then) sums of the 32-groups of the normalised row, / 64, as hi + lo planes
            float t = v;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
            if ((threadIdx.x & 31) == 0) {
                t *= 0.015625f;
                const _Float16 th = (_Float16)t;
                const int64_t at = (int64_t)blockIdx.x * (kp >> 5) + (c >> 5);
                xs[at] = th;
                xs[at + (int64_t)gridDim.x * (kp >> 5)] = (_Float16)(t - (float)th);
            }
        }
    }
    if (threadIdx.x == 0) rs[blockIdx.x] = infrow ? INFINITY : __uint_as_float((uint32_t)(127 - e) << 23);
}

// The same for contiguous rows with k a multiple of 8 and at most 16384: a thread holds its (up to 64) elements of
// the row in registers between the maximum and the conversion, so the row is read once, in 16- or 32-byte loads, and
// written in 16-byte stores.  Values, sums and scale are those of k_act_split.
template <int IN>
__global__ __launch_bounds__(256) void k_act_split_rows(const void *__restrict__ xin, int k, _Float16 *__restrict__ xh,
                                                         _Float16 *__restrict__ xl, float *__restrict__ rs,
                                                         _Float16 *__restrict__ xs) {
    constexpr int NCH = 8; // chunks of 8 elements per thread
    __shared__ float sh[4];
    const int64_t oo = (int64_t)blockIdx.x * k;
    const int nch = (k + 2047) / 2048;
    float v[NCH][8];
    float amax = 0.f;
#pragma unroll
    for (int it = 0; it < NCH; it++) {
        const int c = (it * 256 + (int)threadIdx.x) * 8;
        if (it < nch && c < k) {
            if (IN == 1) {
                const uint4 u = *(const uint4 *)((const uint16_t *)xin + oo + c);
                const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[it][2 * e] = __uint_as_float(w[e] << 16);
                    v[it][2 * e + 1] = __uint_as_float(w[e] & 0xFFFF0000u);
                }
            } else {
                const float4 a = *(const float4 *)((const float *)xin + oo + c), b = *(const float4 *)((const float *)xin + oo + c + 4);
                v[it][0] = a.x, v[it][1] = a.y, v[it][2] = a.z, v[it][3] = a.w;
                v[it][4] = b.x, v[it][5] = b.y, v[it][6] = b.z, v[it][7] = b.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[it][e] = 0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[it][e]));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    int e2 = 141 - (int)((__float_as_uint(amax) >> 23) & 0xFFu); // 14 - floor(log2 amax); zero / inf / nan clamp
    e2 = e2 > 100 ? 100 : (e2 < -100 ? -100 : e2);
    const float sc = __uint_as_float((uint32_t)(e2 + 127) << 23);
    const bool infrow = amax == INFINITY;
#pragma unroll
    for (int it = 0; it < NCH; it++) {
        const int c = (it * 256 + (int)threadIdx.x) * 8;
        const bool live = it < nch && c < k; // (uniform over the four threads of a 32-group: k is a multiple of 8 ... and of 32 with xs)
        _Float16 h[8], l[8];
        float t = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float w = v[it][e] * sc;
            if (infrow && fabsf(w) == INFINITY) w = copysignf(32768.f, w); // as in k_act_split
            h[e] = (_Float16)w;
            l[e] = fh_split_lo(w, h[e]);
            t += w;
        }
        if (live) {
            uint4 u;
            __builtin_memcpy(&u, h, 16);
            *(uint4 *)(xh + oo + c) = u;
            if (IN != 1) {
                __builtin_memcpy(&u, l, 16);
                *(uint4 *)(xl + oo + c) = u;
            }
        }
        if (xs) { // sums of the 32-groups (four neighbouring threads), / 64, as hi + lo planes
            t += __shfl_xor(t, 1, 64);
            t += __shfl_xor(t, 2, 64);
            if (live && (threadIdx.x & 3) == 0) {
                t *= 0.015625f;
                const _Float16 th = (_Float16)t;
                const int64_t at = (int64_t)blockIdx.x * (k >> 5) + (c >> 5);
                xs[at] = th;
                xs[at + (int64_t)gridDim.x * (k >> 5)] = (_Float16)(t - (float)th);
            }
        }
    }
    if (threadIdx.x == 0) rs[blockIdx.x] = infrow ? INFINITY : __uint_as_float((uint32_t)(127 - e2) << 23);
}

// Rows of a dense right-hand side as the tile kernel's "weights": row r (one output column of the product) scaled by
// its own power of two into the f16 range, written as f32 [rows, kp] (zero from k to kp); cs[r] = 2^-e for the store.
template <bool F16>
__global__ __launch_bounds__(256) void k_dense_rows(const void *__restrict__ bin, int64_t srow, int64_t scol, int k, int kp,
                                                     float *__restrict__ out, float *__restrict__ cs) {
    __shared__ float sh[4];
    const int64_t off = (int64_t)blockIdx.x * srow, oo = (int64_t)blockIdx.x * kp;
    auto ld = [&](int c) -> float {
        if (F16) return (float)((const _Float16 *)bin)[off + c * scol];
        return ((const float *)bin)[off + c * scol];
    };
    float amax = 0.f;
    for (int c = threadIdx.x; c < k; c += 256) amax = fmaxf(amax, fabsf(ld(c)));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    int e = 141 - (int)((__float_as_uint(amax) >> 23) & 0xFFu);
    e = e > 100 ? 100 : (e < -100 ? -100 : e);
    const float sc = __uint_as_float((uint32_t)(e + 127) << 23);
    for (int c = threadIdx.x; c < kp; c += 256) out[oo + c] = c < k ? ld(c) * sc : 0.f;
    if (threadIdx.x == 0) cs[blockIdx.x] = __uint_as_float((uint32_t)(127 - e) << 23);
}

// ------------------------------------------------------------------------------ weight slab decode
// Eight dequantised weights of row (tile16*16 + j), lane group g, k-step ks (32 wide).  pos[i] is the position
// of w[i] inside the step.  Arithmetic as in fh_blocks.h (bit-exact f32 decode).
template <int T>
__device__ __forceinline__ void decode8(const QView &q, int64_t tile16, int j, int g, int ks, float *w, int &p0, int &p1) {
    p0 = 8 * g;     // position of w[0..3]
    p1 = 8 * g + 4; // position of w[4..7]
    if (T == FH_W_F32 || T == FH_W_F16) { // dense rows [n][k]: row-major, no blocks
        int64_t row = tile16 * 16 + j;
        if (row >= q.n) row = q.n - 1; // rows past the end repeat the last one and are never stored
        const int64_t at = row * q.k + (int64_t)ks * 32 + 8 * g;
        if (T == FH_W_F32) {
            const float4 a = *(const float4 *)((const float *)q.data + at), b = *(const float4 *)((const float *)q.data + at + 4);
            w[0] = a.x * q.wscale; w[1] = a.y * q.wscale; w[2] = a.z * q.wscale; w[3] = a.w * q.wscale;
            w[4] = b.x * q.wscale; w[5] = b.y * q.wscale; w[6] = b.z * q.wscale; w[7] = b.w * q.wscale;
        } else {
            const uint4 u = *(const uint4 *)((const _Float16 *)q.data + at);
            _Float16 h[8];
            __builtin_memcpy(h, &u, 16);
#pragma unroll
            for (int i = 0; i < 8; i++) w[i] = (float)h[i];
        }
    } else if (T == FH_Q8_0) {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 1)) * 1088;
        const int u = ks & 1;
        const uint2 c = *(const uint2 *)(rec + (g * 16 + j) * 16 + 8 * u);
        const float d = fh_h2f(fh_ld16(rec + 1024 + 4 * j + 2 * u));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)(int)(int8_t)(c.x >> (8 * i)) * d;
            w[4 + i] = (float)(int)(int8_t)(c.y >> (8 * i)) * d;
        }
    } else if (T == FH_Q4_0) {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 2)) * 1152;
        const int u = ks & 3;
        const uint32_t c = *(const uint32_t *)(rec + (g * 16 + j) * 16 + 4 * u);
        const float d = fh_h2f(fh_ld16(rec + 1024 + 8 * j + 2 * u));
        p0 = 4 * g;
        p1 = 16 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)((int)((c >> (8 * i)) & 15u) - 8) * d;
            w[4 + i] = (float)((int)((c >> (8 * i + 4)) & 15u) - 8) * d;
        }
    } else if (T == FH_Q5_0) { // the Q4_0 record plus one byte of fifth bits per lane and block; d * (code - 16)
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 2)) * 1408;
        const int u = ks & 3;
        const uint32_t c = *(const uint32_t *)(rec + (g * 16 + j) * 16 + 4 * u);
        const uint32_t hb = rec[q50_qh_off(j, u, g)];
        const float d = fh_h2f(fh_ld16(rec + 1024 + 8 * j + 2 * u));
        p0 = 4 * g;
        p1 = 16 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)((int)(((c >> (8 * i)) & 15u) | (((hb >> i) & 1u) << 4)) - 16) * d;
            w[4 + i] = (float)((int)(((c >> (8 * i + 4)) & 15u) | (((hb >> (4 + i)) & 1u) << 4)) - 16) * d;
        }
    } else if (T == FH_Q4_K || T == FH_Q5_K) { // Q5_K: the Q4_K record plus the lane's eight qh bytes
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 3)) * (T == FH_Q5_K ? 2816 : 2304);
        const int sb = ks & 7, p = sb >> 2, u = (sb >> 1) & 1, hn = sb & 1;
        const uint2 c = *(const uint2 *)(rec + 256 + p * 1024 + (g * 16 + j) * 16 + 8 * u);
        uint2 hb = make_uint2(0, 0);
        if (T == FH_Q5_K) hb = *(const uint2 *)(rec + 2304 + (g * 16 + j) * 8);
        const uint4 h = *(const uint4 *)(rec + 16 * j);
        const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
        const uint32_t scw = sb < 4 ? (h.y & 0x3F3F3F3Fu) : ((h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u));
        const uint32_t mnw = sb < 4 ? (h.z & 0x3F3F3F3Fu) : (((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u));
        const float scale = (float)((scw >> (8 * (sb & 3))) & 0xFFu) * d;
        const float off = (float)((mnw >> (8 * (sb & 3))) & 0xFFu) * dmin;
        const int sh = 4 * hn;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float a = scale * (float)(((c.x >> (8 * i + sh)) & 15u) + (((hb.x >> (8 * i + sb)) & 1u) << 4));
            const float b = scale * (float)(((c.y >> (8 * i + sh)) & 15u) + (((hb.y >> (8 * i + sb)) & 1u) << 4));
            w[i] = a - off;
            w[4 + i] = b - off;
        }
    } else { // FH_Q6_K
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 3)) * 3360;
        const int t = ks & 7;
        const uint32_t lw = *(const uint32_t *)(rec + q6k_lword_off(j, t, g));
        const uint32_t hw = *(const uint32_t *)(rec + q6k_hword_off(j, t, g));
        const int sc = (int)(int8_t)rec[q6k_sc_off(j, 2 * t + (g >> 1))];
        const float ds = fh_h2f(fh_ld16(rec + q6k_d_off(j))) * (float)sc;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int pp = i >> 1, odd = i & 1;
            const int nib = (int)((lw >> (4 * (pp + 4 * odd))) & 15u);
            const int hb = (int)((hw >> (q6k_hbit(t, pp) + 16 * odd)) & 3u);
            w[i] = ds * (float)(((hb << 4) | nib) - 32);
        }
    }
}

// ------------------------------------------------------------------------------ tile kernel
// Wavefronts are arranged WGN x WGM; each owns FN x FM MFMA tiles of 32 x 32.  NTERM = 1: single activation
// term (bf16 input); 2: hi + lo (f32 input).
template <int T, int NTERM, int WGN, int WGM, int FN, int FM>
__global__ __launch_bounds__(64 * WGN * WGM) void k_qmm_tile(QView q, const _Float16 *__restrict__ xh,
                                                              const _Float16 *__restrict__ xl,
                                                              const float *__restrict__ rs, int m,
                                                              float *__restrict__ y,
                                                              const float *__restrict__ cs = nullptr) {
    constexpr int TN = WGN * FN * 32, TM = WGM * FM * 32, NTH = 64 * WGN * WGM;
    __shared__ __attribute__((aligned(16))) _Float16 s_ah[TN * QMM_LDK], s_al[TN * QMM_LDK], s_bh[TM * QMM_LDK];
    __shared__ __attribute__((aligned(16))) _Float16 s_bl[NTERM == 2 ? TM * QMM_LDK : 8];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wn = wave / WGM, wm = wave % WGM;
    const int64_t n0 = (int64_t)blockIdx.x * TN;
    const int m0 = blockIdx.y * TM;
    const int K = (int)q.k, ksteps = K / 32;
    const int64_t tiles16 = (q.n + 15) / 16;
    floatx16 acc[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    for (int ks = 0; ks < ksteps; ks++) {
        __syncthreads(); // the previous step's operands are consumed
        // ---- weights: TN * 4 (row, group) pairs of 8
#pragma unroll
        for (int i = 0; i < (TN * 4 + NTH - 1) / NTH; i++) {
            const int p = tid + i * NTH;
            if (p < TN * 4) {
                const int t16 = p >> 6, l = p & 63, g = l >> 4, j = l & 15;
                int64_t tile = (n0 >> 4) + t16;
                if (tile >= tiles16) tile = tiles16 - 1; // rows past the end decode a valid tile and are never stored
                float w[8];
                int p0, p1;
                decode8<T>(q, tile, j, g, ks, w, p0, p1);
                _Float16 hi[8], lo[8];
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    hi[c] = (_Float16)w[c];
                    lo[c] = (T == FH_W_F32 || T == FH_W_F16) ? fh_split_lo(w[c], hi[c]) : (_Float16)(w[c] - (float)hi[c]);
                }
                const int row = t16 * 16 + j;
                uint2 a0, a1, b0, b1;
                __builtin_memcpy(&a0, hi, 8);
                __builtin_memcpy(&a1, hi + 4, 8);
                __builtin_memcpy(&b0, lo, 8);
                __builtin_memcpy(&b1, lo + 4, 8);
                *(uint2 *)(s_ah + row * QMM_LDK + p0) = a0;
                *(uint2 *)(s_ah + row * QMM_LDK + p1) = a1;
                *(uint2 *)(s_al + row * QMM_LDK + p0) = b0;
                *(uint2 *)(s_al + row * QMM_LDK + p1) = b1;
            }
        }
        // ---- activations: TM rows x 32 halfs (two 16-byte pieces per row... four 16-byte pieces: 64 B)
#pragma unroll
        for (int i = 0; i < (TM * 4 + NTH - 1) / NTH; i++) {
            const int p = tid + i * NTH;
            if (p < TM * 4) {
                const int row = p >> 2, c = p & 3;
                const int mm = m0 + row;
                uint4 vh = make_uint4(0, 0, 0, 0), vl = make_uint4(0, 0, 0, 0);
                if (mm < m) {
                    vh = *(const uint4 *)(xh + (int64_t)mm * K + ks * 32 + c * 8);
                    if (NTERM == 2) vl = *(const uint4 *)(xl + (int64_t)mm * K + ks * 32 + c * 8);
                }
                *(uint4 *)(s_bh + row * QMM_LDK + c * 8) = vh;
                if (NTERM == 2) *(uint4 *)(s_bl + row * QMM_LDK + c * 8) = vl;
            }
        }
        __syncthreads();
        // ---- contraction
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int ko = kk * 16 + 8 * (lane >> 5), li = lane & 31;
            half8 ah[FN], al[FN], bh[FM], bl[FM];
#pragma unroll
            for (int a = 0; a < FN; a++) {
                const int row = (wn * FN + a) * 32 + li;
                ah[a] = *(const half8 *)(s_ah + row * QMM_LDK + ko);
                al[a] = *(const half8 *)(s_al + row * QMM_LDK + ko);
            }
#pragma unroll
            for (int b = 0; b < FM; b++) {
                const int row = (wm * FM + b) * 32 + li;
                bh[b] = *(const half8 *)(s_bh + row * QMM_LDK + ko);
                if (NTERM == 2) bl[b] = *(const half8 *)(s_bl + row * QMM_LDK + ko);
            }
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int b = 0; b < FM; b++) {
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[a], bh[b], acc[a][b], 0, 0, 0);
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[a], bh[b], acc[a][b], 0, 0, 0);
                    if (NTERM == 2) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[a], bl[b], acc[a][b], 0, 0, 0);
                }
        }
    }
    // ---- store: lane holds column m = lane % 32 and rows n = 8*(r/4) + 4*(lane/32) + r%4 of each 32 x 32 tile
    const bool vec = (q.n & 3) == 0;
#pragma unroll
    for (int b = 0; b < FM; b++) {
        const int mm = m0 + (wm * FM + b) * 32 + (lane & 31);
        if (mm >= m) continue;
        const float s = rs[mm] * q.winv;
#pragma unroll
        for (int a = 0; a < FN; a++) {
            const int64_t nb = n0 + (wn * FN + a) * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const int64_t nn = nb + 8 * r4;
                float4 v = make_float4(acc[a][b][4 * r4] * s, acc[a][b][4 * r4 + 1] * s, acc[a][b][4 * r4 + 2] * s,
                                       acc[a][b][4 * r4 + 3] * s);
                if (cs) { // a dense right-hand side: every output column has its own factor
                    v.x *= cs[nn < q.n ? nn : q.n - 1];
                    v.y *= cs[nn + 1 < q.n ? nn + 1 : q.n - 1];
                    v.z *= cs[nn + 2 < q.n ? nn + 2 : q.n - 1];
                    v.w *= cs[nn + 3 < q.n ? nn + 3 : q.n - 1];
                }
                float *dst = y + (int64_t)mm * q.n + nn;
                if (vec && nn + 3 < q.n) {
                    *(float4 *)dst = v;
                } else {
                    if (nn < q.n) dst[0] = v.x;
                    if (nn + 1 < q.n) dst[1] = v.y;
                    if (nn + 2 < q.n) dst[2] = v.z;
                    if (nn + 3 < q.n) dst[3] = v.w;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------ pipelined 128 x 256 tile kernel
// The same product for many activation rows: 8 wavefronts (2 x 4) of 64 x 64 each, so the decode of a weight slab is
// shared by 256 activation rows.  The raw block bytes and the activation slab of step s+2 are in flight in
// registers, step s+1 is decoded into the second LDS buffer while the MFMAs of step s (issued first) drain: one
// barrier per step.
struct QmmRaw {
    uint32_t a, b; // code words
    uint4 h;       // scale material (format dependent)
    uint32_t e0, e1; // fifth bits (Q5_0: one byte; Q5_K: the lane's eight qh bytes)
};

template <int T>
__device__ __forceinline__ void qmm_load_raw(const QView &q, int64_t tile16, int j, int g, int ks, QmmRaw &r) {
    r.a = r.b = r.e0 = r.e1 = 0;
    r.h = make_uint4(0, 0, 0, 0);
    if (T == FH_Q8_0) {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 1)) * 1088;
        const int u = ks & 1;
        const uint2 c = *(const uint2 *)(rec + (g * 16 + j) * 16 + 8 * u);
        r.a = c.x;
        r.b = c.y;
        r.h.x = fh_ld16(rec + 1024 + 4 * j + 2 * u);
    } else if (T == FH_Q4_0 || T == FH_Q5_0) {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 2)) * (T == FH_Q5_0 ? 1408 : 1152);
        const int u = ks & 3;
        r.a = *(const uint32_t *)(rec + (g * 16 + j) * 16 + 4 * u);
        r.h.x = fh_ld16(rec + 1024 + 8 * j + 2 * u);
        if (T == FH_Q5_0) r.e0 = rec[q50_qh_off(j, u, g)];
    } else if (T == FH_Q4_K || T == FH_Q5_K) {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 3)) * (T == FH_Q5_K ? 2816 : 2304);
        const int sb = ks & 7, p = sb >> 2, u = (sb >> 1) & 1;
        const uint2 c = *(const uint2 *)(rec + 256 + p * 1024 + (g * 16 + j) * 16 + 8 * u);
        r.a = c.x;
        r.b = c.y;
        r.h = *(const uint4 *)(rec + 16 * j);
        if (T == FH_Q5_K) {
            const uint2 hb = *(const uint2 *)(rec + 2304 + (g * 16 + j) * 8);
            r.e0 = hb.x;
            r.e1 = hb.y;
        }
    } else {
        const uint8_t *rec = q.data + (tile16 * q.recs + (ks >> 3)) * 3360;
        const int t = ks & 7;
        r.a = *(const uint32_t *)(rec + q6k_lword_off(j, t, g));
        r.b = *(const uint32_t *)(rec + q6k_hword_off(j, t, g));
        r.h.x = rec[q6k_sc_off(j, 2 * t + (g >> 1))];
        r.h.y = fh_ld16(rec + q6k_d_off(j));
    }
}

// Eight dequantised weights from the raw words (arithmetic of fh_blocks.h), and their positions in the step.
template <int T>
__device__ __forceinline__ void qmm_decode_raw(const QmmRaw &r, int g, int ks, float *w, int &p0, int &p1) {
    p0 = 8 * g;
    p1 = 8 * g + 4;
    if (T == FH_Q8_0) {
        const float d = fh_h2f((uint16_t)r.h.x);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)(int)(int8_t)(r.a >> (8 * i)) * d;
            w[4 + i] = (float)(int)(int8_t)(r.b >> (8 * i)) * d;
        }
    } else if (T == FH_Q4_0) {
        const float d = fh_h2f((uint16_t)r.h.x);
        p0 = 4 * g;
        p1 = 16 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)((int)((r.a >> (8 * i)) & 15u) - 8) * d;
            w[4 + i] = (float)((int)((r.a >> (8 * i + 4)) & 15u) - 8) * d;
        }
    } else if (T == FH_Q5_0) {
        const float d = fh_h2f((uint16_t)r.h.x);
        p0 = 4 * g;
        p1 = 16 + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (float)((int)(((r.a >> (8 * i)) & 15u) | (((r.e0 >> i) & 1u) << 4)) - 16) * d;
            w[4 + i] = (float)((int)(((r.a >> (8 * i + 4)) & 15u) | (((r.e0 >> (4 + i)) & 1u) << 4)) - 16) * d;
        }
    } else if (T == FH_Q4_K || T == FH_Q5_K) {
        const int sb = ks & 7, hn = sb & 1;
        const uint4 h = r.h;
        const float d = fh_h2f((uint16_t)(h.x & 0xFFFF)), dmin = fh_h2f((uint16_t)(h.x >> 16));
        const uint32_t scw = sb < 4 ? (h.y & 0x3F3F3F3Fu) : ((h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u));
        const uint32_t mnw = sb < 4 ? (h.z & 0x3F3F3F3Fu) : (((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u));
        const float scale = (float)((scw >> (8 * (sb & 3))) & 0xFFu) * d;
        const float off = (float)((mnw >> (8 * (sb & 3))) & 0xFFu) * dmin;
        const int sh = 4 * hn;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float a = scale * (float)(((r.a >> (8 * i + sh)) & 15u) + (T == FH_Q5_K ? ((r.e0 >> (8 * i + sb)) & 1u) << 4 : 0u));
            const float b = scale * (float)(((r.b >> (8 * i + sh)) & 15u) + (T == FH_Q5_K ? ((r.e1 >> (8 * i + sb)) & 1u) << 4 : 0u));
            w[i] = a - off;
            w[4 + i] = b - off;
        }
    } else {
        const int t = ks & 7;
        const float ds = fh_h2f((uint16_t)r.h.y) * (float)(int)(int8_t)r.h.x;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int pp = i >> 1, odd = i & 1;
            const int nib = (int)((r.a >> (4 * (pp + 4 * odd))) & 15u);
            const int hb = (int)((r.b >> (q6k_hbit(t, pp) + 16 * odd)) & 3u);
            w[i] = ds * (float)(((hb << 4) | nib) - 32);
        }
    }
}

// WN x (8 / WN) wavefronts of (32 FN) x (32 FM) outputs each: 128 weight rows x 256, 128 or 64 activation rows.
template <int T, int NTERM, int WN, int FN, int FM>
__global__ __launch_bounds__(512) void k_qmm_tile2(QView q, const _Float16 *__restrict__ xh,
                                                   const _Float16 *__restrict__ xl, const float *__restrict__ rs,
                                                   int m, float *__restrict__ y, int tiles_n = 0, int full = 0, int tail = 0,
                                                   float *__restrict__ planes = nullptr) {
    constexpr int WM = 8 / WN, TN = WN * FN * 32, TM = WM * FM * 32;
    static_assert(TN == 128, "512 threads decode 128 weight rows x 4 pieces per step");
    constexpr int NB = (TM * 4 + 511) / 512; // 16-byte activation pieces per thread, plane and step
    constexpr int A_H = TN * 32, B_H = TM * 32;         // halfs per plane
    constexpr int BUF = 2 * A_H + NTERM * B_H;                    // halfs per buffer: A hi, A lo, B hi (, B lo)
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[]; // two buffers
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wn = wave / WM, wm = wave % WM;
    // tiles_n > 0: one-dimensional grid with the tiles of the last round split along k, as in k_qmm_tile2j
    const int lin = (int)blockIdx.x, split = tiles_n > 0 && lin >= full, tile = split ? full + ((lin - full) >> 1) : lin;
    const int64_t n0 = (int64_t)(tiles_n > 0 ? tile % tiles_n : (int)blockIdx.x) * TN;
    const int m0 = (tiles_n > 0 ? tile / tiles_n : (int)blockIdx.y) * TM;
    // gridDim.z > 1: the k steps are split over workgroups, each writing its partial product to its own [m, n] plane
    // of y (the host sums the planes); a split holds an even number of steps, so LDS buffer parity is that of ks
    const int K = (int)q.k, kparts = split ? 2 : (int)gridDim.z, kpart = split ? (lin - full) & 1 : (int)blockIdx.z;
    const int kper = K / 32 / kparts, kbeg = kpart * kper, ksteps = kbeg + kper;
    y += (size_t)blockIdx.z * (size_t)m * (size_t)q.n;
    const int64_t tiles16 = (q.n + 15) / 16;
    // this thread's weight duty: row a_row of the tile, lane group a_g (8 weights per step)
    const int a_row = tid >> 2, a_g = tid & 3, a_j = a_row & 15;
    int64_t a_tile = (n0 >> 4) + (a_row >> 4);
    if (a_tile >= tiles16) a_tile = tiles16 - 1; // rows past the end decode a valid tile and are never stored
    // activation duty: NB 16-byte pieces per plane and step
    // piece i (0, 1): row (tid + 512 i) / 4 of the tile, 16-byte column (tid + 512 i) % 4 = tid % 4
    // (a 64-row tile has 256 pieces: the upper half of the workgroup repeats the lower half's, same values)
    const int b_c = tid & 3, b_row0 = (tid >> 2) % TM, b_row1 = (b_row0 + 128) % TM;
    // rows past the end repeat the last one (never stored)
    const int64_t b_off0 = (int64_t)(m0 + b_row0 < m ? m0 + b_row0 : m - 1) * K + b_c * 8;
    const int64_t b_off1 = (int64_t)(m0 + b_row1 < m ? m0 + b_row1 : m - 1) * K + b_c * 8;
    // two register sets (even / odd steps), named so that no indexing survives into the generated code
    struct Slab {
        QmmRaw raw;
        uint4 h0, h1, l0, l1;
    } s0, s1;
    auto fetch = [&](Slab &sl, int ks) {
        qmm_load_raw<T>(q, a_tile, a_j, a_g, ks, sl.raw);
        sl.h0 = *(const uint4 *)(xh + b_off0 + ks * 32);
        sl.h1 = NB == 2 ? *(const uint4 *)(xh + b_off1 + ks * 32) : sl.h0;
        if (NTERM == 2) {
            sl.l0 = *(const uint4 *)(xl + b_off0 + ks * 32);
            sl.l1 = NB == 2 ? *(const uint4 *)(xl + b_off1 + ks * 32) : sl.l0;
        }
    };
    auto stage = [&](const Slab &sl, int ks) {
        _Float16 *buf = smem + (ks & 1) * BUF;
        float w[8];
        int p0, p1;
        qmm_decode_raw<T>(sl.raw, a_g, ks, w, p0, p1);
        _Float16 hi[8], lo[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            hi[c] = (_Float16)w[c];
            lo[c] = (T == FH_W_F32 || T == FH_W_F16) ? fh_split_lo(w[c], hi[c]) : (_Float16)(w[c] - (float)hi[c]);
        }
        uint2 a0, a1, l0, l1;
        __builtin_memcpy(&a0, hi, 8);
        __builtin_memcpy(&a1, hi + 4, 8);
        __builtin_memcpy(&l0, lo, 8);
        __builtin_memcpy(&l1, lo + 4, 8);
        *(uint2 *)(buf + QMM_AT(a_row, p0)) = a0;
        *(uint2 *)(buf + QMM_AT(a_row, p1)) = a1;
        *(uint2 *)(buf + A_H + QMM_AT(a_row, p0)) = l0;
        *(uint2 *)(buf + A_H + QMM_AT(a_row, p1)) = l1;
        *(uint4 *)(buf + 2 * A_H + QMM_AT(b_row0, b_c * 8)) = sl.h0;
        if (NB == 2) *(uint4 *)(buf + 2 * A_H + QMM_AT(b_row1, b_c * 8)) = sl.h1;
        if (NTERM == 2) {
            *(uint4 *)(buf + 2 * A_H + B_H + QMM_AT(b_row0, b_c * 8)) = sl.l0;
            if (NB == 2) *(uint4 *)(buf + 2 * A_H + B_H + QMM_AT(b_row1, b_c * 8)) = sl.l1;
        }
    };
    floatx16 acc[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    fetch(s0, kbeg);
    if (kper > 1) fetch(s1, kbeg + 1);
    stage(s0, kbeg);
    // one k step; `mine` is the register set that held step ks (free again), `other` holds step ks + 1
    auto kstep = [&](int ks, Slab &mine, const Slab &other) {
            if (ks < ksteps) {
                __syncthreads(); // buffer ks & 1 is complete; the other one is no longer read
                if (ks + 2 < ksteps) fetch(mine, ks + 2);
                const _Float16 *buf = smem + (ks & 1) * BUF;
#pragma unroll
                for (int kk = 0; kk < 2; kk++) {
                    const int ko = kk * 16 + 8 * (lane >> 5), li = lane & 31;
                    half8 ah[FN], al[FN], bhv[FM], blv[FM];
#pragma unroll
                    for (int a = 0; a < FN; a++) {
                        const int row = (wn * FN + a) * 32 + li;
                        ah[a] = *(const half8 *)(buf + QMM_AT(row, ko));
                        al[a] = *(const half8 *)(buf + A_H + QMM_AT(row, ko));
                    }
#pragma unroll
                    for (int b = 0; b < FM; b++) {
                        const int row = (wm * FM + b) * 32 + li;
                        bhv[b] = *(const half8 *)(buf + 2 * A_H + QMM_AT(row, ko));
                        if (NTERM == 2) blv[b] = *(const half8 *)(buf + 2 * A_H + B_H + QMM_AT(row, ko));
                    }
#pragma unroll
                    for (int a = 0; a < FN; a++)
#pragma unroll
                        for (int b = 0; b < FM; b++) {
                            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[a], bhv[b], acc[a][b], 0, 0, 0);
                            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[a], bhv[b], acc[a][b], 0, 0, 0);
                            if (NTERM == 2)
                                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[a], blv[b], acc[a][b], 0, 0, 0);
                        }
                }
                if (ks + 1 < ksteps) stage(other, ks + 1);
            }
    };
    for (int ks0 = kbeg; ks0 < ksteps; ks0 += 2) { // the register sets alternate: no indexing survives into the code
        kstep(ks0, s0, s1);
        kstep(ks0 + 1, s1, s0);
    }
    const bool vec = (q.n & 3) == 0;
#pragma unroll
    for (int b = 0; b < FM; b++) {
        const int mm = m0 + (wm * FM + b) * 32 + (lane & 31);
        if (mm >= m) continue;
        const float s = rs[mm];
#pragma unroll
        for (int a = 0; a < FN; a++) {
            const int64_t nb = n0 + (wn * FN + a) * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const int64_t nn = nb + 8 * r4;
                const float4 v = make_float4(acc[a][b][4 * r4] * s, acc[a][b][4 * r4 + 1] * s, acc[a][b][4 * r4 + 2] * s,
                                             acc[a][b][4 * r4 + 3] * s);
                float *dst = y + (int64_t)mm * q.n + nn;
                if (split) {
                    if (nn < q.n) *(float4 *)(planes + (((int64_t)kpart * tail + (tile - full)) * TM + (mm - m0)) * TN + (nn - n0)) = v;
                } else if (vec && nn + 3 < q.n) {
                    *(float4 *)dst = v;
                } else {
                    if (nn < q.n) dst[0] = v.x;
                    if (nn + 1 < q.n) dst[1] = v.y;
                    if (nn + 2 < q.n) dst[2] = v.z;
                    if (nn + 3 < q.n) dst[3] = v.w;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------ integer codes, scale after the MFMA
// Q8_0 and Q4_0 (one f16 scale per 32 weights = one k step): the weight operand is the integer code itself
// (-128 .. 127, -8 .. 7: exact in f16, ONE term instead of the hi + lo pair of a dequantised weight), the products of
// a step are collected in a zeroed accumulator and the block scale is applied to it in f32:
//   acc += d[n, step] * sum_k x[m, k] * code[n, k]
// which is the reference's sum with d factored out of each block.  The roles of the MFMA operands are swapped against
// k_qmm_tile2 (A = activations, B = weights), so a lane holds ONE weight row of the output tile and d is a per-lane
// scalar: 16 multiply-adds per lane, block and 32 x 32 tile against two MFMAs saved.  Same tile (128 weight rows x 256
// activation rows, 8 wavefronts of 64 x 64), same pipeline (raw bytes and activation slab of step s+2 in registers,
// step s+1 decoded into the second LDS buffer, one barrier per step).
typedef _Float16 qmm_half2 __attribute__((ext_vector_type(2)));

template <int T, int NTERM, int WM>
__global__ __launch_bounds__(128 * WM) void k_qmm_tile2i(QView q, const _Float16 *__restrict__ xh,
                                                    const _Float16 *__restrict__ xl, const float *__restrict__ rs,
                                                    int m, float *__restrict__ y, int tiles_n, int full, int tail,
                                                    float *__restrict__ planes) {
    static_assert(T == FH_Q8_0 || T == FH_Q4_0, "formats with one scale per 32 weights");
    // WM = 4: eight wavefronts, 256 activation rows; WM = 2: four wavefronts, 128 activation rows - two such workgroups
    // share a compute unit and are at different points of their steps (one's MFMAs under the other's scaling and staging)
    constexpr int WN = 2, FN = 2, FM = 2, TN = WN * FN * 32, TM = WM * FM * 32, NT = 128 * WM, NA = 512 / NT;
    constexpr int A_H = TN * 32, B_H = TM * 32;       // halfs per plane
    constexpr int BUF = A_H + NTERM * B_H + 2 * TN;            // halfs per buffer: codes, x hi (, x lo), TN f32 scales
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[]; // two buffers
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31;
    const int wn = wave / WM, wm = wave % WM;
    // tiles_n > 0: one-dimensional grid with the tiles of the last round split along k, as in k_qmm_tile2j
    const int lin = (int)blockIdx.x, split = tiles_n > 0 && lin >= full, tile = split ? full + ((lin - full) >> 1) : lin;
    const int64_t n0 = (int64_t)(tiles_n > 0 ? tile % tiles_n : (int)blockIdx.x) * TN;
    const int m0 = (tiles_n > 0 ? tile / tiles_n : (int)blockIdx.y) * TM;
    const int K = (int)q.k, kpart = split ? (lin - full) & 1 : 0;
    const int kfirst = split && kpart ? K / 64 : 0, ksteps = split && !kpart ? K / 64 : K / 32; // steps [kfirst, ksteps)
    const int64_t tiles16 = (q.n + 15) / 16;
    // weight duty: NA items (row, lane group) of 8 codes per step; activation duty: two 16-byte pieces per plane and step
    const int a_g = tid & 3, a_j = (tid >> 2) & 15;
    int a_row[NA];
    int64_t a_tile[NA];
#pragma unroll
    for (int u = 0; u < NA; u++) {
        a_row[u] = (tid >> 2) + u * (NT / 4);
        a_tile[u] = (n0 >> 4) + (a_row[u] >> 4);
        if (a_tile[u] >= tiles16) a_tile[u] = tiles16 - 1; // rows past the end decode a valid tile and are never stored
    }
    const int b_c = tid & 3, b_row0 = tid >> 2, b_row1 = b_row0 + TM / 2;
    const int64_t b_off0 = (int64_t)(m0 + b_row0 < m ? m0 + b_row0 : m - 1) * K + b_c * 8;
    const int64_t b_off1 = (int64_t)(m0 + b_row1 < m ? m0 + b_row1 : m - 1) * K + b_c * 8;
    struct Slab {
        QmmRaw raw[NA];
        uint4 h0, h1, l0, l1;
    } s0, s1;
    auto fetch = [&](Slab &sl, int ks) {
#pragma unroll
        for (int u = 0; u < NA; u++) qmm_load_raw<T>(q, a_tile[u], a_j, a_g, ks, sl.raw[u]);
        sl.h0 = *(const uint4 *)(xh + b_off0 + ks * 32);
        sl.h1 = *(const uint4 *)(xh + b_off1 + ks * 32);
        if (NTERM == 2) {
            sl.l0 = *(const uint4 *)(xl + b_off0 + ks * 32);
            sl.l1 = *(const uint4 *)(xl + b_off1 + ks * 32);
        }
    };
    // two code bytes (already 0 .. 255 resp. 0 .. 15) under the high byte 0x64 are the halfs 1024 + u; minus the bias
    auto codes2 = [&](uint32_t bytes, uint32_t sel, float bias) -> uint32_t {
        const uint32_t w = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
        qmm_half2 h;
        __builtin_memcpy(&h, &w, 4);
        h = h - qmm_half2{(_Float16)bias, (_Float16)bias};
        uint32_t o;
        __builtin_memcpy(&o, &h, 4);
        return o;
    };
    auto stage = [&](const Slab &sl, int ks) {
        _Float16 *buf = smem + (ks & 1) * BUF;
#pragma unroll
        for (int u = 0; u < NA; u++) {
        if (T == FH_Q8_0) { // bytes 0 .. 3 of a, then of b: positions 8 g .. 8 g + 7 of the step
            const uint32_t ua = sl.raw[u].a ^ 0x80808080u, ub = sl.raw[u].b ^ 0x80808080u;
            uint4 c;
            c.x = codes2(ua, 0x04010400u, 1152.f);
            c.y = codes2(ua, 0x04030402u, 1152.f);
            c.z = codes2(ub, 0x04010400u, 1152.f);
            c.w = codes2(ub, 0x04030402u, 1152.f);
            *(uint4 *)(buf + QMM_AT(a_row[u], 8 * a_g)) = c;
        } else { // low nibbles: positions 4 g .. 4 g + 3, high nibbles: 16 + 4 g .. 16 + 4 g + 3
            const uint32_t lo = sl.raw[u].a & 0x0F0F0F0Fu, hi = (sl.raw[u].a >> 4) & 0x0F0F0F0Fu;
            uint2 c0, c1;
            c0.x = codes2(lo, 0x04010400u, 1032.f);
            c0.y = codes2(lo, 0x04030402u, 1032.f);
            c1.x = codes2(hi, 0x04010400u, 1032.f);
            c1.y = codes2(hi, 0x04030402u, 1032.f);
            *(uint2 *)(buf + QMM_AT(a_row[u], 4 * a_g)) = c0;
            *(uint2 *)(buf + QMM_AT(a_row[u], 16 + 4 * a_g)) = c1;
        }
        ((float *)(buf + A_H + NTERM * B_H))[a_row[u]] = fh_h2f((uint16_t)sl.raw[u].h.x); // the four threads of a row: same value
        }
        *(uint4 *)(buf + A_H + QMM_AT(b_row0, b_c * 8)) = sl.h0;
        *(uint4 *)(buf + A_H + QMM_AT(b_row1, b_c * 8)) = sl.h1;
        if (NTERM == 2) {
            *(uint4 *)(buf + A_H + B_H + QMM_AT(b_row0, b_c * 8)) = sl.l0;
            *(uint4 *)(buf + A_H + B_H + QMM_AT(b_row1, b_c * 8)) = sl.l1;
        }
    };
    floatx16 acc[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    fetch(s0, kfirst);
    if (ksteps > kfirst + 1) fetch(s1, kfirst + 1);
    stage(s0, kfirst);
    auto kstep = [&](int ks, Slab &mine, const Slab &other) {
        if (ks < ksteps) {
            __syncthreads(); // buffer ks & 1 is complete; the other one is no longer read
            fetch(mine, ks + 2 < ksteps ? ks + 2 : ksteps - 1); // (no branch in the step: past the end, a repeat)
            const _Float16 *buf = smem + (ks & 1) * BUF;
            floatx16 part[FN][FM];
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int b = 0; b < FM; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) part[a][b][r] = 0.f;
            // all operands of the step first (12 or 16 reads of 16 bytes), then the products weight tile by weight tile:
            // the scaling of tile a runs under the MFMAs of tile a + 1 (a wavefront hides vector instructions under its
            // own MFMAs), the scaling of the last tile under the decode of the next slab
            half8 wc[2][FN], xhv[2][FM], xlv[2][FM];
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const int ko = kk * 16 + 8 * (lane >> 5);
#pragma unroll
                for (int a = 0; a < FN; a++) wc[kk][a] = *(const half8 *)(buf + QMM_AT(((wn * FN + a) * 32 + li), ko));
#pragma unroll
                for (int b = 0; b < FM; b++) {
                    const int row = (wm * FM + b) * 32 + li;
                    xhv[kk][b] = *(const half8 *)(buf + A_H + QMM_AT(row, ko));
                    if (NTERM == 2) xlv[kk][b] = *(const half8 *)(buf + A_H + B_H + QMM_AT(row, ko));
                }
            }
            const float *sd = (const float *)(buf + A_H + NTERM * B_H);
            float dl[FN];
#pragma unroll
            for (int a = 0; a < FN; a++) dl[a] = sd[(wn * FN + a) * 32 + li]; // the lane's weight rows
#pragma unroll
            for (int a = 0; a < FN; a++) {
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int b = 0; b < FM; b++) {
                        part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xhv[kk][b], wc[kk][a], part[a][b], 0, 0, 0);
                        if (NTERM == 2)
                            part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xlv[kk][b], wc[kk][a], part[a][b], 0, 0, 0);
                    }
            }
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int b = 0; b < FM; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[a][b][r] = fmaf(part[a][b][r], dl[a], acc[a][b][r]);
            stage(other, ks + 1 < ksteps ? ks + 1 : ks); // (no branch: the last step stages a repeat nobody reads)
            {
                constexpr int MPT = 2 * FM * NTERM; // MFMAs per weight tile
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * (FN + NTERM * FM) + FN, 0); // the operand and scale reads
                __builtin_amdgcn_sched_group_barrier(0x008, MPT, 0);                          // tile 0
#pragma unroll
                for (int a = 1; a < FN; a++)
#pragma unroll
                    for (int i = 0; i < MPT; i++) { // tile a, with the 16 FM multiply-adds of tile a - 1 spread under it
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 16 * FM / MPT, 0);
                    }
            }
        }
    };
    for (int ks0 = kfirst; ks0 < ksteps; ks0 += 2) { // the register sets alternate: no indexing survives into the code
        kstep(ks0, s0, s1);
        kstep(ks0 + 1, s1, s0);
    }
    // lane = weight row n (column of the MFMA result), register r = activation row 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int a = 0; a < FN; a++) {
        const int64_t nn = n0 + (wn * FN + a) * 32 + li;
        if (nn >= q.n) continue;
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int ml = (wm * FM + b) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), mm = m0 + ml;
                if (mm >= m) continue;
                const float v = acc[a][b][r] * rs[mm];
                if (split) planes[(((int64_t)kpart * tail + (tile - full)) * TM + ml) * TN + (nn - n0)] = v;
                else y[(int64_t)mm * q.n + nn] = v;
            }
    }
}

// The integer-code kernel with two blocks of 32 weights per step (64 of k): half as many workgroup barriers and
// operand-read latencies per weight, one 16-byte load per weight item and step (the repack keeps the two blocks'
// codes of a lane side by side). One activation plane only (f16 / bf16 activations); k must be a multiple of 64.
// One-dimensional grid: workgroup t < full owns output tile t (n tile t % tiles_n, m tile t / tiles_n) over all of k.
// When the tiles do not fill the last round of workgroups on the device (tiles mod compute units at most half the
// compute units), the host makes those last tiles two workgroups each, one per half of k, which together fill the round
// for half its time: workgroup full + 2 u + h takes half h of tile full + u and writes the whole tile to
// planes[h][u][TM][TN]; k_qmm_tail_sum adds the two halves into y.
template <int T, int WM>
__global__ __launch_bounds__(128 * WM) void k_qmm_tile2j(QView q, const _Float16 *__restrict__ xh,
                                                    const float *__restrict__ rs, int m, float *__restrict__ y,
                                                    int tiles_n, int full, int tail, float *__restrict__ planes) {
    static_assert(T == FH_Q8_0 || T == FH_Q4_0, "formats with one scale per 32 weights");
    // An LDS row is 64 halfs = eight 16-byte pieces; piece c of row r sits at position c ^ sw(r), sw(r) = bit 1 of r
    // (as bit 2) and bits 2 .. 3 of r: the 16-byte reads of 16 consecutive rows at one c, the 64-byte code writes of four
    // consecutive rows and the 128-byte activation writes of two rows all cover the 64 banks once
    constexpr int LDK = 64;
    auto sw = [](int row) { return ((row >> 1) & 1) << 2 | ((row >> 2) & 3); };
    constexpr int WN = 2, FN = 2, FM = 2, TN = WN * FN * 32, TM = WM * FM * 32, NT = 128 * WM, NA = 512 / NT;
    constexpr int A_H = TN * LDK, B_H = TM * LDK; // halfs per plane
    constexpr int BUF = A_H + B_H + 4 * TN;       // halfs per buffer: codes, activations, 2 TN f32 scales
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[]; // two buffers
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, li = lane & 31;
    const int wn = wave / WM, wm = wave % WM;
    const int lin = (int)blockIdx.x, split = lin >= full, tile = split ? full + ((lin - full) >> 1) : lin;
    const int64_t n0 = (int64_t)(tile % tiles_n) * TN;
    const int m0 = (tile / tiles_n) * TM;
    const int K = (int)q.k;
    const int kfirst = split && ((lin - full) & 1) ? K / 128 : 0, ksteps = split && !((lin - full) & 1) ? K / 128 : K / 64;
    const int64_t tiles16 = (q.n + 15) / 16;
    const int a_g = tid & 3, a_j = (tid >> 2) & 15;
    int a_row[NA];
    const uint8_t *a_rec[NA];
#pragma unroll
    for (int u = 0; u < NA; u++) {
        a_row[u] = (tid >> 2) + u * (NT / 4);
        int64_t t = (n0 >> 4) + (a_row[u] >> 4);
        if (t >= tiles16) t = tiles16 - 1; // rows past the end decode a valid tile and are never stored
        a_rec[u] = q.data + t * q.recs * (T == FH_Q8_0 ? 1088 : 1152);
    }
    // Activation duty: four 16-byte pieces per step, the eight threads of a row cover its 128 bytes.  The pieces go from
    // memory straight into the LDS buffer (LDS-direct loads: lane l's 16 bytes land at base + 16 l, eight rows of 128
    // bytes per wavefront and request), no registers and no LDS write instruction; the swizzle is applied on the memory
    // side: the lane at position p of a row fetches piece p ^ sw(row).
    int64_t b_off[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int rl = (tid >> 3) + i * (NT / 8), row = m0 + rl;
        b_off[i] = (int64_t)(row < m ? row : m - 1) * K + ((tid & 7) ^ sw(rl)) * 8;
    }
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    struct Slab {
        uint32_t c0[NA], c1[NA], c2[NA], c3[NA], d[NA];
    } sl;
    auto fetch_x = [&](int ks, int into) { // the pieces of step ks into the buffer of step `into` (nobody reads it any more)
        _Float16 *dst = smem + (into & 1) * BUF + A_H + (8 * wave) * LDK;
#pragma unroll
        for (int i = 0; i < 4; i++)
            __builtin_amdgcn_global_load_lds((const uint32_t *)(xh + b_off[i] + ks * 64),
                                             (__attribute__((address_space(3))) uint32_t *)(dst + i * (NT / 8) * LDK), 16, 0, 0);
    };
    auto fetch = [&](int ks) {
#pragma unroll
        for (int u = 0; u < NA; u++) {
            if (T == FH_Q8_0) { // a record holds 64 of k: this step
                const uint8_t *rec = a_rec[u] + (int64_t)ks * 1088;
                const u32x4 c = *(const u32x4 *)(rec + (a_g * 16 + a_j) * 16);
                sl.c0[u] = c.x, sl.c1[u] = c.y, sl.c2[u] = c.z, sl.c3[u] = c.w;
                sl.d[u] = *(const uint32_t *)(rec + 1024 + 4 * a_j);
            } else { // a record holds 128 of k: two steps
                const uint8_t *rec = a_rec[u] + (int64_t)(ks >> 1) * 1152;
                const uint2 c = *(const uint2 *)(rec + (a_g * 16 + a_j) * 16 + 8 * (ks & 1));
                sl.c0[u] = c.x, sl.c1[u] = c.y;
                sl.d[u] = *(const uint32_t *)(rec + 1024 + 8 * a_j + 4 * (ks & 1));
            }
        }
    };
    // two code bytes (already 0 .. 255 resp. 0 .. 15) under the high byte 0x64 are the halfs 1024 + u; minus the bias
    auto codes2 = [&](uint32_t bytes, uint32_t sel, float bias) -> uint32_t {
        const uint32_t w = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
        qmm_half2 h;
        __builtin_memcpy(&h, &w, 4);
        h = h - qmm_half2{(_Float16)bias, (_Float16)bias};
        uint32_t o;
        __builtin_memcpy(&o, &h, 4);
        return o;
    };
    auto stage = [&](int ks) {
        _Float16 *buf = smem + (ks & 1) * BUF;
        float *sd = (float *)(buf + A_H + B_H);
#pragma unroll
        for (int u = 0; u < NA; u++) {
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                _Float16 *dst = buf + a_row[u] * LDK;
                const int sr = sw(a_row[u]);
                if (T == FH_Q8_0) { // bytes 0 .. 3 of the first word, then of the second: positions 8 g .. 8 g + 7
                    const uint32_t ua = (blk ? sl.c2[u] : sl.c0[u]) ^ 0x80808080u;
                    const uint32_t ub = (blk ? sl.c3[u] : sl.c1[u]) ^ 0x80808080u;
                    uint4 c;
                    c.x = codes2(ua, 0x04010400u, 1152.f);
                    c.y = codes2(ua, 0x04030402u, 1152.f);
                    c.z = codes2(ub, 0x04010400u, 1152.f);
                    c.w = codes2(ub, 0x04030402u, 1152.f);
                    *(uint4 *)(dst + 8 * ((4 * blk + a_g) ^ sr)) = c;
                } else { // low nibbles: positions 4 g .. 4 g + 3, high nibbles: 16 + 4 g .. 16 + 4 g + 3
                    const uint32_t w = blk ? sl.c1[u] : sl.c0[u];
                    const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
                    uint2 c0, c1;
                    c0.x = codes2(lo, 0x04010400u, 1032.f);
                    c0.y = codes2(lo, 0x04030402u, 1032.f);
                    c1.x = codes2(hi, 0x04010400u, 1032.f);
                    c1.y = codes2(hi, 0x04030402u, 1032.f);
                    *(uint2 *)(dst + 8 * ((4 * blk + (a_g >> 1)) ^ sr) + 4 * (a_g & 1)) = c0;
                    *(uint2 *)(dst + 8 * ((4 * blk + 2 + (a_g >> 1)) ^ sr) + 4 * (a_g & 1)) = c1;
                }
                sd[blk * TN + a_row[u]] = fh_h2f((uint16_t)(sl.d[u] >> (16 * blk))); // the four threads of a row: same value
            }
        }
    };
    floatx16 acc[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    auto compute = [&](int ks) {
        const _Float16 *buf = smem + (ks & 1) * BUF;
        const float *sd = (const float *)(buf + A_H + B_H);
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            floatx16 part[FN][FM];
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int b = 0; b < FM; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) part[a][b][r] = 0.f;
            half8 wc[2][FN], xhv[2][FM];
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const int ko = 8 * ((4 * blk + 2 * kk + (lane >> 5)) ^ sw(li)); // (tile bases are multiples of 32 rows)
#pragma unroll
                for (int a = 0; a < FN; a++) wc[kk][a] = *(const half8 *)(buf + ((wn * FN + a) * 32 + li) * LDK + ko);
#pragma unroll
                for (int b = 0; b < FM; b++) xhv[kk][b] = *(const half8 *)(buf + A_H + ((wm * FM + b) * 32 + li) * LDK + ko);
            }
            float dl[FN];
#pragma unroll
            for (int a = 0; a < FN; a++) dl[a] = sd[blk * TN + (wn * FN + a) * 32 + li]; // the lane's weight rows
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int b = 0; b < FM; b++)
                        part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xhv[kk][b], wc[kk][a], part[a][b], 0, 0, 0);
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int b = 0; b < FM; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[a][b][r] = fmaf(part[a][b][r], dl[a], acc[a][b][r]);
        }
        {
            // block 0: reads, weight tile 0, weight tile 1 over the multiply-adds of tile 0; block 1: reads, tile 0 over
            // the multiply-adds of block 0's tile 1, tile 1 over those of its tile 0; the last 32 run under the decode
            constexpr int MPT = 2 * FM;
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * (FN + FM) + FN, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, MPT, 0);
#pragma unroll
            for (int i = 0; i < MPT; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 16 * FM / MPT, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * (FN + FM) + FN, 0);
#pragma unroll
            for (int i = 0; i < 2 * MPT; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 16 * FM / MPT, 0);
            }
        }
    };
    fetch_x(kfirst, kfirst);
    fetch(kfirst);
    stage(kfirst);
    // (A schedule in which the second wavefront of every SIMD runs half a step behind the first - one multiplies while
    // the other decodes and stages, two barriers per step - was measured slower: 422 against 378 us at 2048 x 14336 x 4096.)
    for (int ks = kfirst; ks < ksteps; ks++) { // steps [kfirst, ksteps)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the activation pieces of buffer ks & 1 have landed
        __syncthreads(); // buffer ks & 1 is complete; the other one is no longer read
        fetch_x(ks + 1 < ksteps ? ks + 1 : ks, ks + 1);
        fetch(ks + 1 < ksteps ? ks + 1 : ks); // (no branch in the step: past the end, a repeat)
        compute(ks);
        stage(ks + 1); // (no branch: the last step stages a repeat nobody reads)
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // no LDS-direct load outlives the workgroup's LDS
    // lane = weight row n (column of the MFMA result), register r = activation row 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int a = 0; a < FN; a++) {
        const int64_t nn = n0 + (wn * FN + a) * 32 + li;
        if (nn >= q.n) continue;
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int ml = (wm * FM + b) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), mm = m0 + ml;
                if (mm >= m) continue;
                const float v = acc[a][b][r] * rs[mm]; // (a power of two: the halves may be scaled before they are added)
                if (split) planes[(((int64_t)((lin - full) & 1) * tail + (tile - full)) * TM + ml) * TN + (nn - n0)] = v;
                else y[(int64_t)mm * q.n + nn] = v;
            }
    }
}

// y tile = planes[0][u] + planes[1][u] for the tail tiles u of k_qmm_tile2j (256 x 128 tiles); one workgroup per 16 rows
__global__ void k_qmm_tail_sum(const float *__restrict__ planes, int tail, int full, int tiles_n, int m, int64_t n,
                               float *__restrict__ y) {
    const int u = blockIdx.x >> 4, tile = full + u, row = ((blockIdx.x & 15) << 4) + (threadIdx.x >> 5), c4 = (threadIdx.x & 31) * 4;
    const int mm = (tile / tiles_n) * 256 + row;
    const int64_t nn = (int64_t)(tile % tiles_n) * 128 + c4;
    if (mm >= m || nn >= n) return;
    const float4 a = *(const float4 *)(planes + (((int64_t)u) * 256 + row) * 128 + c4);
    const float4 b = *(const float4 *)(planes + (((int64_t)tail + u) * 256 + row) * 128 + c4);
    float *dst = y + (int64_t)mm * n + nn;
    const float s[4] = {a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w};
    for (int i = 0; i < 4 && nn + i < n; i++) dst[i] = s[i];
}

template <int T, int WM>
static fh_status qmm_launch_tile2j(const fh_qmatrix *q, const _Float16 *xh, const float *rs, int m, float *y) {
    constexpr int TM = WM * 64;
    constexpr size_t lds = 2 * (size_t)(128 * 64 + TM * 64 + 4 * 128) * 2;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmm_tile2j<T, WM>, (int)lds));
    fh_device *dev = q->dev;
    const int tiles_n = (int)((q->n + 127) / 128), tiles = tiles_n * ((m + TM - 1) / TM);
    // the last round of workgroups: split its tiles along k when they fill at most half the device
    const int tail = (q->k % 128 != 0 || WM != 4) ? 0 : qmm_tail_tiles(dev, tiles);
    float *planes = nullptr;
    if (tail) {
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)2 * tail * TM * 128 * 4));
        planes = dev->ksplit_buf;
    }
    k_qmm_tile2j<T, WM><<<dim3((unsigned)(tiles + tail)), 128 * WM, lds, dev->stream>>>(fh_view(q), xh, rs, m, y, tiles_n,
                                                                                     tiles - tail, tail, planes);
    FH_HIP(hipGetLastError());
    if (tail) {
        k_qmm_tail_sum<<<dim3((unsigned)(tail * 16)), 512, 0, dev->stream>>>(planes, tail, tiles - tail, tiles_n, m, q->n, y);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

template <int T, int NTERM, int WM>
static fh_status qmm_launch_tile2i(const fh_qmatrix *q, const _Float16 *xh, const _Float16 *xl, const float *rs, int m,
                                   float *y) {
    constexpr int TM = WM * 64;
    constexpr size_t lds = 2 * (size_t)(128 * 32 + NTERM * TM * 32 + 2 * 128) * 2;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmm_tile2i<T, NTERM, WM>, (int)lds));
    dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + TM - 1) / TM));
    if (WM == 4 && q->k % 128 == 0) { // split the tiles of a short last round along k
        fh_device *dev = q->dev;
        const int tiles = (int)(grid.x * grid.y), tail = qmm_tail_tiles(dev, tiles);
        if (tail) {
            FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)2 * tail * 256 * 128 * 4));
            k_qmm_tile2i<T, NTERM, WM><<<dim3((unsigned)(tiles + tail)), 128 * WM, lds, dev->stream>>>(
                fh_view(q), xh, xl, rs, m, y, (int)grid.x, tiles - tail, tail, dev->ksplit_buf);
            FH_HIP(hipGetLastError());
            k_qmm_tail_sum<<<dim3((unsigned)(tail * 16)), 512, 0, dev->stream>>>(dev->ksplit_buf, tail, tiles - tail, (int)grid.x, m,
                                                                                q->n, y);
            FH_HIP(hipGetLastError());
            return FH_OK;
        }
    }
    k_qmm_tile2i<T, NTERM, WM><<<grid, 128 * WM, lds, q->dev->stream>>>(fh_view(q), xh, xl, rs, m, y, 0, 0, 0, nullptr);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ Q4_K on integer codes
// Q4_K: w = d * sc_s * q - dmin * m_s (sub-block s of 32, 8 per 256-block; q 0 .. 15, sc and m 0 .. 63).  The weight
// operand is the integer sc_s * q (at most 945: exact in f16; a nibble under the byte 0x64 is the f16 1024 + q, and
// one packed f16 fma (1024 + q) * sc - 1024 sc gives two codes), the products of a whole 256-block collect in one zeroed
// accumulator, and the block's d is applied to it once (acc += d * part: 16 multiply-adds per lane, 32 x 32 tile and 256
// of k, where the formats with a scale per 32 pay them per 32).  The offsets are one more MFMA per 256-block: the
// integers m_s against the sums of the activations of each sub-block (prepared with the activation planes, / 64 to stay
// in the f16 range, as hi + lo), scaled by -64 dmin.  One MFMA per counted product (two with f32 activations) instead
// of two (three) in the split form.  Tile and pipeline as k_qmm_tile2i.
// gridDim.z > 1: k split in runs of whole 256-blocks, partial planes at y + z * m * n.
template <int NTERM>
__global__ __launch_bounds__(512) void k_qmm_tile2k(QView q, const _Float16 *__restrict__ xh, const _Float16 *__restrict__ xl,
                                                      const _Float16 *__restrict__ xs, const float *__restrict__ rs, int m,
                                                      float *__restrict__ y, int tiles_n, int full, int tail,
                                                      float *__restrict__ planes) {
    constexpr int WM = 4, WN = 2, FN = 2, FM = 2, TN = WN * FN * 32, TM = WM * FM * 32;
    // LDS rows of 32 halfs = four 16-byte pieces, piece c of row r at position c ^ ((r >> 2) & 3): the 16-byte reads of 16
    // consecutive rows at one c and the 64-byte writes of four consecutive rows cover the 64 banks once (no padding)
    constexpr int LDK = 32;
    auto sw = [](int row) { return (row >> 2) & 3; };
    constexpr int A_H = TN * LDK, B_H = TM * LDK; // halfs per plane
    constexpr int BUF = A_H + NTERM * B_H;                // halfs per buffer: codes, x hi (, x lo)
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[]; // two buffers, then the per-256-block operands
    _Float16 *s_mn = smem + 2 * BUF;            // [TN][8] offsets m_s as f16 integers
    _Float16 *s_xs = s_mn + TN * 8;             // [2][TM][8] activation sums, hi and lo plane
    float *s_d = (float *)(s_xs + 2 * TM * 8);  // [TN][2]: d, -64 dmin
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31;
    const int wn = wave / WM, wm = wave % WM;
    // tiles_n > 0: one-dimensional grid with the tiles of the last round split along k, as in k_qmm_tile2j
    const int lin = (int)blockIdx.x, split = tiles_n > 0 && lin >= full, tile = split ? full + ((lin - full) >> 1) : lin;
    const int64_t n0 = (int64_t)(tiles_n > 0 ? tile % tiles_n : (int)blockIdx.x) * TN;
    const int m0 = (tiles_n > 0 ? tile / tiles_n : (int)blockIdx.y) * TM;
    const int kparts = split ? 2 : (int)gridDim.z, kpart = split ? (lin - full) & 1 : (int)blockIdx.z;
    const int K = (int)q.k, nsb = (K >> 8) / kparts, sb0 = kpart * nsb; // 256-blocks of this workgroup
    const int ksteps = nsb * 8, kbase = sb0 * 8;
    y += (int64_t)blockIdx.z * m * q.n;
    const int64_t tiles16 = (q.n + 15) / 16;
    // weight duty: one item (row, lane group) of 8 codes per step; activation duty: two 16-byte pieces per plane and step;
    // sums: threads 0 .. 255 the hi plane's 16 bytes of one row per 256-block, threads 256 .. 511 the lo plane's
    const int a_g = tid & 3, a_j = (tid >> 2) & 15, a_row = tid >> 2;
    int64_t a_tile = (n0 >> 4) + (a_row >> 4);
    if (a_tile >= tiles16) a_tile = tiles16 - 1; // rows past the end decode a valid tile and are never stored
    const uint8_t *a_rec = q.data + a_tile * q.recs * 2304;
    const int b_c = tid & 3, b_row0 = tid >> 2, b_row1 = b_row0 + TM / 2;
    const int64_t b_off0 = (int64_t)(m0 + b_row0 < m ? m0 + b_row0 : m - 1) * K + b_c * 8;
    const int64_t b_off1 = (int64_t)(m0 + b_row1 < m ? m0 + b_row1 : m - 1) * K + b_c * 8;
    const int x_row = tid & 255, x_pl = tid >> 8;
    const _Float16 *x_src = xs + (int64_t)x_pl * m * (K >> 5) + (int64_t)(m0 + x_row < m ? m0 + x_row : m - 1) * (K >> 5);
    struct Slab {
        uint32_t a, b;
        u32x4 h, h0, h1, l0, l1;
    } s0, s1;
    auto fetch = [&](Slab &sl, int ks) { // ks: step of this workgroup's range
        const int g = kbase + ks, S = g >> 3, sb = g & 7;
        const uint8_t *rec = a_rec + (int64_t)S * 2304;
        const uint2 c = *(const uint2 *)(rec + 256 + (sb >> 2) * 1024 + (a_g * 16 + a_j) * 16 + 8 * ((sb >> 1) & 1));
        sl.a = c.x, sl.b = c.y;
        sl.h = *(const u32x4 *)(rec + 16 * a_j);
        sl.h0 = *(const u32x4 *)(xh + b_off0 + g * 32);
        sl.h1 = *(const u32x4 *)(xh + b_off1 + g * 32);
        if (NTERM == 2) {
            sl.l0 = *(const u32x4 *)(xl + b_off0 + g * 32);
            sl.l1 = *(const u32x4 *)(xl + b_off1 + g * 32);
        }
    };
    // two bytes (0 .. 63 each) under the high byte 0x64: the halfs 1024 + u
    auto up2 = [&](uint32_t bytes, uint32_t sel) -> qmm_half2 {
        const uint32_t w = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
        qmm_half2 h;
        __builtin_memcpy(&h, &w, 4);
        return h;
    };
    auto bits = [&](qmm_half2 h) -> uint32_t {
        uint32_t o;
        __builtin_memcpy(&o, &h, 4);
        return o;
    };
    const qmm_half2 k1024 = {(_Float16)1024.f, (_Float16)1024.f};
    // the slab of step ks (sub-block sb of its 256-block) into buffer ks & 1; with sb == 1 - at the end of the block's
    // first step, when nobody reads the block before any more - the block's offsets, scales and sums (xsv) go along
    auto stage = [&](const Slab &sl, int ks, u32x4 xsv) {
        const int sb = (kbase + ks) & 7;
        _Float16 *buf = smem + (ks & 1) * BUF;
        const uint32_t scw = sb < 4 ? (sl.h.y & 0x3F3F3F3Fu) : ((sl.h.w & 0x0F0F0F0Fu) | ((sl.h.y >> 2) & 0x30303030u));
        const uint32_t scb = (scw >> (8 * (sb & 3))) & 0xFFu;
        const qmm_half2 sc2 = up2(scb | (scb << 16), 0x04020400u) - k1024;
        const qmm_half2 nb = sc2 * qmm_half2{(_Float16)-1024.f, (_Float16)-1024.f}; // exact: at most 63 * 2^10
        const int sh = 4 * (sb & 1);
        const uint32_t wa = (sl.a >> sh) & 0x0F0F0F0Fu, wb = (sl.b >> sh) & 0x0F0F0F0Fu;
        u32x4 c;
        c.x = bits(__builtin_elementwise_fma(up2(wa, 0x04010400u), sc2, nb));
        c.y = bits(__builtin_elementwise_fma(up2(wa, 0x04030402u), sc2, nb));
        c.z = bits(__builtin_elementwise_fma(up2(wb, 0x04010400u), sc2, nb));
        c.w = bits(__builtin_elementwise_fma(up2(wb, 0x04030402u), sc2, nb));
        *(u32x4 *)(buf + a_row * LDK + 8 * (a_g ^ sw(a_row))) = c;
        *(u32x4 *)(buf + A_H + b_row0 * LDK + 8 * (b_c ^ sw(b_row0))) = sl.h0;
        *(u32x4 *)(buf + A_H + b_row1 * LDK + 8 * (b_c ^ sw(b_row1))) = sl.h1;
        if (NTERM == 2) {
            *(u32x4 *)(buf + A_H + B_H + b_row0 * LDK + 8 * (b_c ^ sw(b_row0))) = sl.l0;
            *(u32x4 *)(buf + A_H + B_H + b_row1 * LDK + 8 * (b_c ^ sw(b_row1))) = sl.l1;
        }
        if (sb == 1) {
            const uint32_t m03 = sl.h.z & 0x3F3F3F3Fu, m47 = ((sl.h.w >> 4) & 0x0F0F0F0Fu) | ((sl.h.z >> 2) & 0x30303030u);
            u32x4 mn;
            mn.x = bits(up2(m03, 0x04010400u) - k1024);
            mn.y = bits(up2(m03, 0x04030402u) - k1024);
            mn.z = bits(up2(m47, 0x04010400u) - k1024);
            mn.w = bits(up2(m47, 0x04030402u) - k1024);
            *(u32x4 *)(s_mn + a_row * 8) = mn; // (the four threads of a row: the same values)
            s_d[2 * a_row] = fh_h2f((uint16_t)(sl.h.x & 0xFFFF));
            s_d[2 * a_row + 1] = -64.f * fh_h2f((uint16_t)(sl.h.x >> 16));
            *(u32x4 *)(s_xs + (x_pl * TM + x_row) * 8) = xsv;
        }
    };
    floatx16 acc[FN][FM], part[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f, part[a][b][r] = 0.f;

    auto kstep = [&](int ks, Slab &mine, const Slab &other) {
        __syncthreads(); // buffer ks & 1 is complete; the other one is no longer read
        // the sums of this step's 256-block (staged after the block's first step): requested before the slab, so that
        // waiting for them does not wait for the slab
        const u32x4 xsv = *(const u32x4 *)(x_src + ((kbase + ks) >> 3) * 8);
        __builtin_amdgcn_sched_barrier(0);
        fetch(mine, ks + 2 < ksteps ? ks + 2 : ksteps - 1); // (no branch around the requests: past the end, a repeat)
        const _Float16 *buf = smem + (ks & 1) * BUF;
        half8 wc[2][FN], xhv[2][FM], xlv[2][FM];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int ko = 8 * ((2 * kk + (lane >> 5)) ^ sw(li)); // (tile bases are multiples of 32 rows)
#pragma unroll
            for (int a = 0; a < FN; a++) wc[kk][a] = *(const half8 *)(buf + ((wn * FN + a) * 32 + li) * LDK + ko);
#pragma unroll
            for (int b = 0; b < FM; b++) {
                const int row = (wm * FM + b) * 32 + li;
                xhv[kk][b] = *(const half8 *)(buf + A_H + row * LDK + ko);
                if (NTERM == 2) xlv[kk][b] = *(const half8 *)(buf + A_H + B_H + row * LDK + ko);
            }
        }
#pragma unroll
        for (int a = 0; a < FN; a++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int b = 0; b < FM; b++) {
                    part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xhv[kk][b], wc[kk][a], part[a][b], 0, 0, 0);
                    if (NTERM == 2)
                        part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xlv[kk][b], wc[kk][a], part[a][b], 0, 0, 0);
                }
        if (((kbase + ks) & 7) == 7) { // the 256-block is complete: its scale, then its offsets
            half8 mnv[FN], xsh[FM], xsl[FM];
            const half8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int a = 0; a < FN; a++) mnv[a] = lane < 32 ? *(const half8 *)(s_mn + ((wn * FN + a) * 32 + li) * 8) : zero8;
#pragma unroll
            for (int b = 0; b < FM; b++) {
                const int row = (wm * FM + b) * 32 + li;
                xsh[b] = lane < 32 ? *(const half8 *)(s_xs + row * 8) : zero8;
                xsl[b] = lane < 32 ? *(const half8 *)(s_xs + (TM + row) * 8) : zero8;
            }
#pragma unroll
            for (int a = 0; a < FN; a++) {
                const float d = s_d[2 * ((wn * FN + a) * 32 + li)], nd = s_d[2 * ((wn * FN + a) * 32 + li) + 1];
#pragma unroll
                for (int b = 0; b < FM; b++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[a][b][r] = fmaf(part[a][b][r], d, acc[a][b][r]);
#pragma unroll
                    for (int r = 0; r < 16; r++) part[a][b][r] = 0.f;
                    part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xsh[b], mnv[a], part[a][b], 0, 0, 0);
                    part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xsl[b], mnv[a], part[a][b], 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[a][b][r] = fmaf(part[a][b][r], nd, acc[a][b][r]);
#pragma unroll
                    for (int r = 0; r < 16; r++) part[a][b][r] = 0.f;
                }
            }
        }
        if (ks + 1 < ksteps) stage(other, ks + 1, xsv); // (the last step has nothing to stage)
        // the sums are waited for in every step (they are the oldest request: the slab stays in flight), or the request
        // would still be pending at the next barrier and the wait there would take the slab with it
        asm volatile("" ::"v"(xsv));
    };
    fetch(s0, 0);
    fetch(s1, 1);
    stage(s0, 0, u32x4{0, 0, 0, 0});
    for (int ks0 = 0; ks0 < ksteps; ks0 += 2) { // the register sets alternate: no indexing survives into the code
        kstep(ks0, s0, s1);
        kstep(ks0 + 1, s1, s0);
    }
    // lane = weight row n (column of the MFMA result), register r = activation row 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int a = 0; a < FN; a++) {
        const int64_t nn = n0 + (wn * FN + a) * 32 + li;
        if (nn >= q.n) continue;
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int ml = (wm * FM + b) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), mm = m0 + ml;
                if (mm >= m) continue;
                const float v = acc[a][b][r] * rs[mm];
                if (split) planes[(((int64_t)kpart * tail + (tile - full)) * TM + ml) * TN + (nn - n0)] = v;
                else y[(int64_t)mm * q.n + nn] = v;
            }
    }
}

// ------------------------------------------------------------------------------ Q6_K on integer codes
// Q6_K: w = d * sc_g * (q - 32) (16-element groups g, sc int8, q 0 .. 63).  sc * (q - 32) needs 12 bits, one more than an
// f16 holds, so the weight operand is two exact terms: (sc & ~15) * (q - 32) (a multiple of 16 up to 4096 in size) and
// (sc & 15) * (q - 32) (at most 480), both accumulated into one zeroed accumulator over a whole 256-block, to which the
// block's d is applied once.  As many MFMAs as the split form (two per product), but the decode is integer and packed
// f16 work (the 6-bit codes of two weights come out of the tiled words as one 32-bit pattern under 0x6400 = the f16
// pair 1024 + q) instead of f32 arithmetic and two-term rounding, and there is no rounding at all before the f32
// accumulation.  One activation plane (f16 / bf16 activations); tile, pipeline, k split and the split last round as
// k_qmm_tile2k.
__global__ __launch_bounds__(512) void k_qmm_tile2q(QView q, const _Float16 *__restrict__ xh, const float *__restrict__ rs,
                                                      int m, float *__restrict__ y, int tiles_n, int full, int tail,
                                                      float *__restrict__ planes) {
    // 64 of k (an even and an odd sub-block step of the tiled record) per step and workgroup barrier; LDS rows of 64 halfs
    // with the 16-byte pieces XOR-swizzled as in k_qmm_tile2j
    constexpr int LDK = 64;
    auto sw = [](int row) { return ((row >> 1) & 1) << 2 | ((row >> 2) & 3); };
    constexpr int WM = 4, WN = 2, FN = 2, FM = 2, TN = WN * FN * 32, TM = WM * FM * 32;
    constexpr int A_H = TN * LDK, B_H = TM * LDK; // halfs per plane
    constexpr int BUF = 2 * A_H + B_H;            // halfs per buffer: codes (high part, low part), x
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) _Float16 smem[]; // two buffers, then d per weight row
    float *s_d = (float *)(smem + 2 * BUF);
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, li = lane & 31;
    const int wn = wave / WM, wm = wave % WM;
    const int lin = (int)blockIdx.x, split = tiles_n > 0 && lin >= full, tile = split ? full + ((lin - full) >> 1) : lin;
    const int64_t n0 = (int64_t)(tiles_n > 0 ? tile % tiles_n : (int)blockIdx.x) * TN;
    const int m0 = (tiles_n > 0 ? tile / tiles_n : (int)blockIdx.y) * TM;
    const int kparts = split ? 2 : (int)gridDim.z, kpart = split ? (lin - full) & 1 : (int)blockIdx.z;
    const int K = (int)q.k, nsb = (K >> 8) / kparts, sb0 = kpart * nsb; // 256-blocks of this workgroup
    const int ksteps = nsb * 4, kbase = sb0 * 4;                        // steps of 64
    y += (int64_t)blockIdx.z * m * q.n;
    const int64_t tiles16 = (q.n + 15) / 16;
    const int a_g = tid & 3, a_j = (tid >> 2) & 15, a_row = tid >> 2, a_sw = sw(a_row);
    int64_t a_tile = (n0 >> 4) + (a_row >> 4);
    if (a_tile >= tiles16) a_tile = tiles16 - 1; // rows past the end decode a valid tile and are never stored
    const uint8_t *a_rec = q.data + a_tile * q.recs * 3360;
    // Activation duty: four 16-byte pieces per step, the eight threads of a row cover its 128 bytes.  The pieces go from
    // memory straight into the LDS buffer (LDS-direct loads: lane l's 16 bytes land at base + 16 l, eight rows of 128
    // bytes per wavefront and request), no registers and no LDS write instruction; the swizzle is applied on the memory
    // side: the lane at position p of a row fetches piece p ^ sw(row).
    int64_t b_off[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int rl = (tid >> 3) + i * 64, row = m0 + rl;
        b_off[i] = (int64_t)(row < m ? row : m - 1) * K + ((tid & 7) ^ sw(rl)) * 8;
    }
    // The weight bytes of a step (HBM or the memory-side cache) are requested two steps before they are decoded, into one
    // of two register sets (even / odd steps); the activation pieces (L2) one step before.
    struct WSlab {
        uint32_t a0, a1, b, sc0, sc1, d;
    };
    auto fetch_w = [&](int ks_, WSlab &sl) { // ks: step of this workgroup's range (past the end: a repeat of the last)
        const int ks = ks_ < ksteps ? ks_ : ksteps - 1;
        const int g = kbase + ks, t = 2 * (g & 3); // the even sub-block step; t + 1 shares its word of two-bit parts
        const uint8_t *rec = a_rec + (int64_t)(g >> 2) * 3360;
        const uint2 a = *(const uint2 *)(rec + q6k_lword_off(a_j, t, a_g));
        sl.a0 = a.x, sl.a1 = a.y;
        sl.b = *(const uint32_t *)(rec + q6k_hword_off(a_j, t, a_g));
        sl.sc0 = rec[q6k_sc_off(a_j, 2 * t + (a_g >> 1))];
        sl.sc1 = rec[q6k_sc_off(a_j, 2 * t + 2 + (a_g >> 1))];
        sl.d = fh_ld16(rec + q6k_d_off(a_j));
    };
    auto fetch_x = [&](int ks_) { // into buffer ks & 1, which nobody reads any more
        const int ks = ks_ < ksteps ? ks_ : ksteps - 1;
        const int g = kbase + ks;
        _Float16 *dst = smem + (ks_ & 1) * BUF + 2 * A_H + (8 * wave) * LDK;
#pragma unroll
        for (int i = 0; i < 4; i++)
            __builtin_amdgcn_global_load_lds((const uint32_t *)(xh + b_off[i] + g * 64),
                                             (__attribute__((address_space(3))) uint32_t *)(dst + i * 64 * LDK), 16, 0, 0);
    };
    auto stage = [&](int ks, const WSlab &sl) {
        _Float16 *buf = smem + (ks & 1) * BUF;
        const qmm_half2 k1056 = {(_Float16)1056.f, (_Float16)1056.f};
#pragma unroll
        for (int blk = 0; blk < 2; blk++) { // blk = parity of the sub-block step: the two-bit parts sit elsewhere in odd steps
            const int sc = (int)(int8_t)(blk ? sl.sc1 : sl.sc0);
            const uint32_t aw = blk ? sl.a1 : sl.a0;
            const _Float16 fl = (_Float16)(float)(sc & 15), fh = (_Float16)(float)(sc & ~15); // exact: small integers
            const qmm_half2 sl2 = {fl, fl}, sh2 = {fh, fh};
            u32x4 chi, clo;
#pragma unroll
            for (int p = 0; p < 4; p++) { // weights 2 p and 2 p + 1 of the item: positions 8 g + 2 p, + 1 of the sub-block
                const uint32_t lo4 = (aw >> (4 * p)) & 0x000F000Fu;
                uint32_t hi2;
                if (!blk) hi2 = sl.b >> (2 * p);
                else hi2 = p == 0 ? sl.b << 4 : (p == 1 ? sl.b << 2 : (p == 2 ? sl.b >> 8 : sl.b >> 10));
                const uint32_t v = lo4 | (hi2 & 0x00300030u) | 0x64006400u; // the f16 pair 1024 + q
                qmm_half2 h;
                __builtin_memcpy(&h, &v, 4);
                h = h - k1056; // q - 32
                const qmm_half2 a = h * sh2, b = h * sl2;
                uint32_t ua, ub;
                __builtin_memcpy(&ua, &a, 4);
                __builtin_memcpy(&ub, &b, 4);
                chi[p] = ua, clo[p] = ub;
            }
            *(u32x4 *)(buf + a_row * LDK + 8 * ((4 * blk + a_g) ^ a_sw)) = chi;
            *(u32x4 *)(buf + A_H + a_row * LDK + 8 * ((4 * blk + a_g) ^ a_sw)) = clo;
        }
        // the block's d, staged with its second step: nobody reads the previous block's any more
        if (((kbase + ks) & 3) == 1) s_d[a_row] = fh_h2f((uint16_t)sl.d); // (the four threads of a row: the same value)
    };
    floatx16 acc[FN][FM], part[FN][FM];
#pragma unroll
    for (int a = 0; a < FN; a++)
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f, part[a][b][r] = 0.f;

    WSlab w0, w1;
    fetch_x(0);
    fetch_w(0, w0);
    fetch_w(1, w1);
    stage(0, w0);
    fetch_w(2, w0);
    auto step = [&](int ks, WSlab &wn1) { // wn1: the weights of step ks + 1
        // The activation pieces of buffer ks & 1 were requested a step ago, before the last five weight loads: all but
        // those have to be back.  Then the barrier: buffer ks & 1 is complete; the other one is no longer read.
        asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        __syncthreads();
        fetch_x(ks + 1);
        const _Float16 *buf = smem + (ks & 1) * BUF;
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            half8 wh[2][FN], wl[2][FN], xv[2][FM];
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const int ko = 8 * ((4 * blk + 2 * kk + (lane >> 5)) ^ sw(li)); // (tile bases are multiples of 32 rows)
#pragma unroll
                for (int a = 0; a < FN; a++) {
                    wh[kk][a] = *(const half8 *)(buf + ((wn * FN + a) * 32 + li) * LDK + ko);
                    wl[kk][a] = *(const half8 *)(buf + A_H + ((wn * FN + a) * 32 + li) * LDK + ko);
                }
#pragma unroll
                for (int b = 0; b < FM; b++) xv[kk][b] = *(const half8 *)(buf + 2 * A_H + ((wm * FM + b) * 32 + li) * LDK + ko);
            }
#pragma unroll
            for (int a = 0; a < FN; a++)
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int b = 0; b < FM; b++) {
                        part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xv[kk][b], wh[kk][a], part[a][b], 0, 0, 0);
                        part[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xv[kk][b], wl[kk][a], part[a][b], 0, 0, 0);
                    }
        }
        if (((kbase + ks) & 3) == 3) { // the 256-block is complete: its scale
#pragma unroll
            for (int a = 0; a < FN; a++) {
                const float d = s_d[(wn * FN + a) * 32 + li];
#pragma unroll
                for (int b = 0; b < FM; b++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[a][b][r] = fmaf(part[a][b][r], d, acc[a][b][r]);
#pragma unroll
                    for (int r = 0; r < 16; r++) part[a][b][r] = 0.f;
                }
            }
        }
        if (ks + 1 < ksteps) stage(ks + 1, wn1); // (the last step has nothing to stage)
        fetch_w(ks + 3, wn1);
    };
    for (int ks = 0; ks < ksteps; ks += 2) { // (four steps per 256-block: an even count)
        step(ks, w1);
        step(ks + 1, w0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // no LDS-direct load outlives the workgroup's LDS
    // lane = weight row n (column of the MFMA result), register r = activation row 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int a = 0; a < FN; a++) {
        const int64_t nn = n0 + (wn * FN + a) * 32 + li;
        if (nn >= q.n) continue;
#pragma unroll
        for (int b = 0; b < FM; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int ml = (wm * FM + b) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), mm = m0 + ml;
                if (mm >= m) continue;
                const float v = acc[a][b][r] * rs[mm];
                if (split) planes[(((int64_t)kpart * tail + (tile - full)) * TM + ml) * TN + (nn - n0)] = v;
                else y[(int64_t)mm * q.n + nn] = v;
            }
    }
}

// y = sum of the partial planes of a k-split product, in plane order (deterministic)
__global__ void k_qmm_sum_planes(const float4 *__restrict__ part, int planes, int64_t n4, float4 *__restrict__ y) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    float4 a = part[i];
    for (int p = 1; p < planes; p++) {
        const float4 b = part[(int64_t)p * n4 + i];
        a = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
    }
    y[i] = a;
}

static fh_status qmm_launch_tile2q(const fh_qmatrix *q, const _Float16 *xh, const float *rs, int m, float *y, int ksplit) {
    constexpr size_t lds = 2 * (size_t)(2 * 128 * 64 + 256 * 64) * 2 + 128 * 4;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmm_tile2q, (int)lds));
    fh_device *dev = q->dev;
    dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + 255) / 256), (unsigned)ksplit);
    if (ksplit == 1 && q->k % 512 == 0) { // split the tiles of a short last round along k
        const int tiles = (int)(grid.x * grid.y), tail = qmm_tail_tiles(dev, tiles);
        if (tail) {
            FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)2 * tail * 256 * 128 * 4));
            k_qmm_tile2q<<<dim3((unsigned)(tiles + tail)), 512, lds, dev->stream>>>(fh_view(q), xh, rs, m, y, (int)grid.x, tiles - tail,
                                                                                 tail, dev->ksplit_buf);
            FH_HIP(hipGetLastError());
            k_qmm_tail_sum<<<dim3((unsigned)(tail * 16)), 512, 0, dev->stream>>>(dev->ksplit_buf, tail, tiles - tail, (int)grid.x, m,
                                                                                q->n, y);
            FH_HIP(hipGetLastError());
            return FH_OK;
        }
    }
    float *dst = y;
    if (ksplit > 1) {
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)ksplit * m * q->n * 4));
        dst = dev->ksplit_buf;
    }
    k_qmm_tile2q<<<grid, 512, lds, dev->stream>>>(fh_view(q), xh, rs, m, dst, 0, 0, 0, nullptr);
    FH_HIP(hipGetLastError());
    if (ksplit > 1) {
        const int64_t n4 = (int64_t)m * q->n / 4;
        k_qmm_sum_planes<<<dim3((unsigned)((n4 + 255) / 256)), 256, 0, dev->stream>>>((const float4 *)dst, ksplit, n4, (float4 *)y);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

template <int NTERM>
static fh_status qmm_launch_tile2k(const fh_qmatrix *q, const _Float16 *xh, const _Float16 *xl, const _Float16 *xs,
                                   const float *rs, int m, float *y, int ksplit) {
    constexpr size_t lds = 2 * (size_t)(128 * 32 + NTERM * 256 * 32) * 2 + 128 * 8 * 2 + 2 * 256 * 8 * 2 + 128 * 2 * 4;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmm_tile2k<NTERM>, (int)lds));
    dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + 255) / 256), (unsigned)ksplit);
    if (ksplit == 1 && q->k % 512 == 0) { // split the tiles of a short last round along k
        fh_device *dev = q->dev;
        const int tiles = (int)(grid.x * grid.y), tail = qmm_tail_tiles(dev, tiles);
        if (tail) {
            FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)2 * tail * 256 * 128 * 4));
            k_qmm_tile2k<NTERM><<<dim3((unsigned)(tiles + tail)), 512, lds, dev->stream>>>(
                fh_view(q), xh, xl, xs, rs, m, y, (int)grid.x, tiles - tail, tail, dev->ksplit_buf);
            FH_HIP(hipGetLastError());
            k_qmm_tail_sum<<<dim3((unsigned)(tail * 16)), 512, 0, dev->stream>>>(dev->ksplit_buf, tail, tiles - tail, (int)grid.x, m,
                                                                                q->n, y);
            FH_HIP(hipGetLastError());
            return FH_OK;
        }
    }
    float *dst = y;
    if (ksplit > 1) {
        fh_device *dev = q->dev;
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)ksplit * m * q->n * 4));
        dst = dev->ksplit_buf;
    }
    k_qmm_tile2k<NTERM><<<grid, 512, lds, q->dev->stream>>>(fh_view(q), xh, xl, xs, rs, m, dst, 0, 0, 0, nullptr);
    FH_HIP(hipGetLastError());
    if (ksplit > 1) {
        const int64_t n4 = (int64_t)m * q->n / 4;
        k_qmm_sum_planes<<<dim3((unsigned)((n4 + 255) / 256)), 256, 0, q->dev->stream>>>((const float4 *)dst, ksplit, n4,
                                                                                       (float4 *)y);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

template <int T, int NTERM, int WN, int FN, int FM>
static fh_status qmm_launch_tile2(const fh_qmatrix *q, const _Float16 *xh, const _Float16 *xl, const float *rs, int m,
                                  float *y, int ksplit = 1) {
    constexpr int TM = (8 / WN) * FM * 32;
    constexpr size_t lds = 2 * (size_t)(2 * 128 * 32 + NTERM * TM * 32) * 2;
    FH_TRY(fh_kernel_lds(q->dev, (const void *)k_qmm_tile2<T, NTERM, WN, FN, FM>, (int)lds));
    dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + TM - 1) / TM), (unsigned)ksplit);
    if (TM == 256 && ksplit == 1 && q->k % 128 == 0) { // split the tiles of a short last round along k
        fh_device *dev = q->dev;
        const int tiles = (int)(grid.x * grid.y), tail = qmm_tail_tiles(dev, tiles);
        if (tail) {
            FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)2 * tail * 256 * 128 * 4));
            k_qmm_tile2<T, NTERM, WN, FN, FM><<<dim3((unsigned)(tiles + tail)), 512, lds, dev->stream>>>(
                fh_view(q), xh, xl, rs, m, y, (int)grid.x, tiles - tail, tail, dev->ksplit_buf);
            FH_HIP(hipGetLastError());
            k_qmm_tail_sum<<<dim3((unsigned)(tail * 16)), 512, 0, dev->stream>>>(dev->ksplit_buf, tail, tiles - tail, (int)grid.x, m,
                                                                                q->n, y);
            FH_HIP(hipGetLastError());
            return FH_OK;
        }
    }
    float *dst = y;
    if (ksplit > 1) {
        fh_device *dev = q->dev;
        FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, (size_t)ksplit * m * q->n * 4));
        dst = dev->ksplit_buf;
    }
    k_qmm_tile2<T, NTERM, WN, FN, FM><<<grid, 512, lds, q->dev->stream>>>(fh_view(q), xh, xl, rs, m, dst);
    FH_HIP(hipGetLastError());
    if (ksplit > 1) {
        const int64_t n4 = (int64_t)m * q->n / 4;
        k_qmm_sum_planes<<<dim3((unsigned)((n4 + 255) / 256)), 256, 0, q->dev->stream>>>((const float4 *)dst, ksplit, n4,
                                                                                       (float4 *)y);
        FH_HIP(hipGetLastError());
    }
    return FH_OK;
}

template <int T, int NTERM>
static fh_status qmm_launch_t(const fh_qmatrix *q, const _Float16 *xh, const _Float16 *xl, const float *rs, int m,
                              float *y, const _Float16 *xs) {
    hipStream_t s = q->dev->stream;
    QView v = fh_view(q);
    // the pipelined kernel with the tallest activation tile (256, 128, 64 rows) that still fills most of the device
    // (opt_matmul_kernel = 3: never, 4: always 256)
    const int64_t tn = (q->n + 127) / 128, cus = q->dev->compute_units;
    const int64_t mk = q->dev->opt_matmul_kernel;
    if (mk == 4 || mk == 8 || mk == 9 || mk == 10 || (m > 128 && tn * ((m + 255) / 256) * 5 >= cus * 4 && mk != 3)) { // 8, 9, 10: as 4, integer codes
        // one scale per 32 weights: integer codes and the scale after the MFMA (matmul_kernel = 6 keeps the split form)
        if constexpr (T == FH_Q8_0 || T == FH_Q4_0) {
            // (matmul_kernel = 7: four wavefronts and 128 activation rows per workgroup, two workgroups per compute unit:
            // measured slower, 596 against 496 µs for 2048 x 14336 x 4096)
            if (mk == 7) return qmm_launch_tile2i<T, NTERM, 2>(q, xh, xl, rs, m, y);
            if constexpr (NTERM == 1) // (matmul_kernel = 9: one block of 32 per step also for one activation plane)
                if (mk != 6 && mk != 4 && mk != 9 && q->k % 64 == 0)
                    return qmm_launch_tile2j<T, 4>(q, xh, rs, m, y);
            if (mk != 6 && mk != 4) return qmm_launch_tile2i<T, NTERM, 4>(q, xh, xl, rs, m, y);
        }
        // Q6_K with one activation plane: two exact integer-code terms, the 256-block's d after the MFMAs
        if constexpr (T == FH_Q6_K && NTERM == 1)
            if (mk != 6 && mk != 4) return qmm_launch_tile2q(q, xh, rs, m, y, mk == 10 && (q->k / 256) % 2 == 0 && (q->n & 3) == 0 ? 2 : 1);
        // Q4_K: integer codes sc * q, the 256-block's d after the MFMAs, the offsets as one more MFMA per block
        if constexpr (T == FH_Q4_K)
            if (mk != 6 && mk != 4 && xs) // (matmul_kernel = 10: k split in two where k allows it)
                return qmm_launch_tile2k<NTERM>(q, xh, xl, xs, rs, m, y, mk == 10 && (q->k / 256) % 2 == 0 && (q->n & 3) == 0 ? 2 : 1);
        return qmm_launch_tile2<T, NTERM, 2, 2, 2>(q, xh, xl, rs, m, y);
    }
    if (m > 64 && mk != 3 && mk != 5) {
        // too few tiles for the device: split k over workgroups rather than shrink the tile (every tile row of
        // workgroups decodes the weights again), as long as a split keeps 16 steps; the partial planes are summed
        // by a second launch
        const int ksteps = (int)(q->k / 32);
        auto split_for = [&](int64_t tiles) {
            int ks = 1;
            while (tiles * ks * 5 < cus * 4 && ks < 8 && ksteps % (ks * 4) == 0 && ksteps / (ks * 2) >= 16 &&
                   (q->n & 3) == 0)
                ks *= 2;
            return ks;
        };
        if (m > 128) {
            const int ks = split_for(tn * ((m + 255) / 256));
            if (tn * ((m + 255) / 256) * ks * 5 >= cus * 4) {
                if constexpr (T == FH_Q4_K)
                    if (mk != 6 && xs && (q->k / 256) % ks == 0) return qmm_launch_tile2k<NTERM>(q, xh, xl, xs, rs, m, y, ks);
                if constexpr (T == FH_Q6_K && NTERM == 1)
                    if (mk != 6 && (q->k / 256) % ks == 0) return qmm_launch_tile2q(q, xh, rs, m, y, ks);
                return qmm_launch_tile2<T, NTERM, 2, 2, 2>(q, xh, xl, rs, m, y, ks);
            }
        }
        const int ks = split_for(tn * ((m + 127) / 128));
        if (tn * ((m + 127) / 128) * ks * 5 >= cus * 4) return qmm_launch_tile2<T, NTERM, 2, 2, 1>(q, xh, xl, rs, m, y, ks);
        return qmm_launch_tile2<T, NTERM, 4, 1, 1>(q, xh, xl, rs, m, y, split_for(tn * ((m + 63) / 64)));
    }
    if (m <= 32) {
        dim3 grid((unsigned)((q->n + 127) / 128), 1);
        k_qmm_tile<T, NTERM, 4, 1, 1, 1><<<grid, 256, 0, s>>>(v, xh, xl, rs, m, y);
    } else if (m <= 64) {
        dim3 grid((unsigned)((q->n + 127) / 128), 1);
        k_qmm_tile<T, NTERM, 2, 2, 2, 1><<<grid, 256, 0, s>>>(v, xh, xl, rs, m, y);
    } else if (((q->n + 127) / 128) * ((m + 127) / 128) < (int64_t)q->dev->compute_units && mk != 5) {
        // too few 128 x 128 tiles to fill the device: 128 x 64 tiles (the weight slab is decoded twice as often)
        dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + 63) / 64));
        k_qmm_tile<T, NTERM, 2, 2, 2, 1><<<grid, 256, 0, s>>>(v, xh, xl, rs, m, y);
    } else {
        dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + 127) / 128));
        k_qmm_tile<T, NTERM, 2, 2, 2, 2><<<grid, 256, 0, s>>>(v, xh, xl, rs, m, y);
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// dense f16 / f32 weight rows: the plain tile kernel (its weight "decode" is a load), tile shape by row count
template <int T, int NTERM>
static fh_status qmm_launch_dense(const fh_qmatrix *q, const _Float16 *xh, const _Float16 *xl, const float *rs, int m,
                                  float *y, const float *cs = nullptr) {
    hipStream_t s = q->dev->stream;
    QView v = fh_view(q);
    const unsigned gn = (unsigned)((q->n + 127) / 128);
    FH_REQUIRE((m + 63) / 64 <= 65535, "m = %d too large for one launch", m);
    if (m <= 32) k_qmm_tile<T, NTERM, 4, 1, 1, 1><<<dim3(gn, 1), 256, 0, s>>>(v, xh, xl, rs, m, y, cs);
    else if (m <= 64 || (int64_t)gn * ((m + 127) / 128) < (int64_t)q->dev->compute_units)
        k_qmm_tile<T, NTERM, 2, 2, 2, 1><<<dim3(gn, (unsigned)((m + 63) / 64)), 256, 0, s>>>(v, xh, xl, rs, m, y, cs);
    else k_qmm_tile<T, NTERM, 2, 2, 2, 2><<<dim3(gn, (unsigned)((m + 127) / 128)), 256, 0, s>>>(v, xh, xl, rs, m, y, cs);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_launch_qmatmul_tile(const fh_qmatrix *q, const void *x, int x_is_bf16, int m, float *y) {
    fh_device *dev = q->dev;
    const int64_t K = q->k;
    if (fh_is_plain(q->type) && K % 32 != 0)
        FH_FAIL(FH_ERR_UNSUPPORTED, "type %u with k = %lld has no matrix-core matmul (it runs through fh_qmatmul)", q->type,
                (long long)K);
    FH_REQUIRE((m + 127) / 128 <= 65535, "m = %d too large for one launch", m);
    // planes: xh | xl | rs | (Q4_K: sums of the 32-groups, hi and lo)
    const size_t plane = ((size_t)m * K * 2 + 255) & ~(size_t)255;
    const size_t rs_bytes = ((size_t)m * 4 + 255) & ~(size_t)255;
    const bool sums = q->type == FH_Q4_K && K % 256 == 0;
    const size_t need = plane * (x_is_bf16 ? 1 : 2) + rs_bytes + (sums ? 2 * (size_t)m * (K / 32) * 2 : 0) + 256;
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, need));
    _Float16 *xh = (_Float16 *)dev->act_buf;
    _Float16 *xl = x_is_bf16 ? nullptr : (_Float16 *)((uint8_t *)dev->act_buf + plane);
    float *rs = (float *)((uint8_t *)dev->act_buf + plane * (x_is_bf16 ? 1 : 2));
    _Float16 *xs = sums ? (_Float16 *)((uint8_t *)rs + rs_bytes) : nullptr;
    const bool rows = K % 32 == 0 && K <= 16384 && ((uintptr_t)x & 15) == 0 && dev->opt_matmul_kernel != 12; // (12: the general kernel)
    if (rows && x_is_bf16) k_act_split_rows<1><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(x, (int)K, xh, xl, rs, xs);
    else if (rows) k_act_split_rows<0><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(x, (int)K, xh, xl, rs, xs);
    else if (x_is_bf16) k_act_split<1><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(x, K, 1, (int)K, (int)K, xh, xl, rs, xs);
    else k_act_split<0><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(x, K, 1, (int)K, (int)K, xh, xl, rs, xs);
    FH_HIP(hipGetLastError());
#define QMM_GO(T_)                                                              \
    return x_is_bf16 ? qmm_launch_t<T_, 1>(q, xh, xl, rs, m, y, xs) : qmm_launch_t<T_, 2>(q, xh, xl, rs, m, y, xs)
    switch (q->type) {
    case FH_Q4_0: QMM_GO(FH_Q4_0);
    case FH_Q8_0: QMM_GO(FH_Q8_0);
    case FH_Q4_K: QMM_GO(FH_Q4_K);
    case FH_Q6_K: QMM_GO(FH_Q6_K);
    case FH_Q5_0: QMM_GO(FH_Q5_0);
    case FH_Q5_K: QMM_GO(FH_Q5_K);
    case FH_W_F16: return x_is_bf16 ? qmm_launch_dense<FH_W_F16, 1>(q, xh, xl, rs, m, y) : qmm_launch_dense<FH_W_F16, 2>(q, xh, xl, rs, m, y);
    case FH_W_F32: return x_is_bf16 ? qmm_launch_dense<FH_W_F32, 1>(q, xh, xl, rs, m, y) : qmm_launch_dense<FH_W_F32, 2>(q, xh, xl, rs, m, y);
    }
#undef QMM_GO
    FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported type %u", q->type);
}

// ------------------------------------------------------------------------------ dense matmul
// largest |w| of a dense f32 weight -> the power of two that brings it into [2^14, 2^15)
__global__ __launch_bounds__(256) void k_amax_bits(const float *__restrict__ w, int64_t count, uint32_t *__restrict__ out) {
    uint32_t a = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
        a = max(a, __float_as_uint(w[i]) & 0x7FFFFFFFu);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) a = max(a, (uint32_t)__shfl_xor((int)a, o, 64));
    if ((threadIdx.x & 63) == 0) atomicMax(out, a); // integer maximum: the order does not matter
}

fh_status fh_dense_wscale(fh_device *dev, const float *w_dev, int64_t count, float *wscale) {
    uint32_t *slot = (uint32_t *)dev->small_buf;
    FH_TRY(fh_memset(dev, slot, 0, 4));
    const int64_t blocks = (count + 255) / 256;
    k_amax_bits<<<dim3((unsigned)(blocks > 1024 ? 1024 : blocks)), dim3(256), 0, dev->stream>>>(w_dev, count, slot);
    FH_HIP(hipGetLastError());
    uint32_t bits = 0;
    FH_TRY(fh_download(dev, &bits, slot, 4));
    int e = 141 - (int)((bits >> 23) & 0xFFu);
    e = e > 100 ? 100 : (e < -100 ? -100 : e);
    const uint32_t sb = (uint32_t)(e + 127) << 23;
    __builtin_memcpy(wscale, &sb, 4);
    return FH_OK;
}

// Tensor::matmul (fusor-ml/fusor/src/lib.rs:1094-1103; CPU form fusor-ml/cpu/src/matmul.rs:226-352, f16 form :159-179):
// C[b] = A[b] . B[b] for strided views A [batch, m, k] and B [batch, k, n].  Both operands become exact two-term
// f16 splits of values normalised per row of A and per column of B (as the reference copies non-contiguous operands to
// scratch first, :299-328), the product runs on the matrix cores with f32 accumulation, f16 results are rounded once.
extern "C" fh_status fh_matmul(fh_device *dev, int32_t dtype, const void *a_dev, int64_t a_sb, int64_t a_sr, int64_t a_sc,
                               const void *b_dev, int64_t b_sb, int64_t b_sr, int64_t b_sc, int32_t batch, int32_t m,
                               int32_t k, int32_t n, void *c_dev) {
    FH_REQUIRE(dev && a_dev && b_dev && c_dev, "NULL argument");
    FH_REQUIRE(dtype == FH_F32 || dtype == FH_F16, "dtype must be FH_F32 or FH_F16");
    FH_REQUIRE(batch > 0 && m > 0 && k > 0 && n > 0, "empty matmul operand [%d, %d, %d] @ [.., %d, %d]", batch, m, k, k, n);
    const bool h16 = dtype == FH_F16;
    const int kp = (k + 31) / 32 * 32;
    const size_t plane = ((size_t)m * kp * 2 + 255) & ~(size_t)255;
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, 2 * plane + (size_t)m * 4 + 256));
    const size_t bt = ((size_t)n * kp * 4 + 255) & ~(size_t)255, csb = ((size_t)n * 4 + 255) & ~(size_t)255;
    FH_TRY(fh_dev_scratch(dev, (void **)&dev->ksplit_buf, &dev->ksplit_cap, bt + csb + (h16 ? (size_t)m * n * 4 : 0)));
    _Float16 *xh = (_Float16 *)dev->act_buf, *xl = (_Float16 *)((uint8_t *)dev->act_buf + plane);
    float *rs = (float *)((uint8_t *)dev->act_buf + 2 * plane);
    float *btp = dev->ksplit_buf, *cs = (float *)((uint8_t *)dev->ksplit_buf + bt);
    float *c32 = (float *)((uint8_t *)dev->ksplit_buf + bt + csb);
    const size_t esz = h16 ? 2 : 4;
    fh_qmatrix qt; // the packed right-hand side viewed as dense f32 weight rows [n, kp]
    qt.dev = dev;
    qt.type = FH_W_F32;
    qt.n = n;
    qt.k = kp;
    qt.n_pad = n;
    qt.kb = kp;
    qt.rec_bytes = 4;
    qt.data = (uint8_t *)btp;
    for (int bi = 0; bi < batch; bi++) {
        const uint8_t *ab = (const uint8_t *)a_dev + (size_t)bi * a_sb * esz, *bb = (const uint8_t *)b_dev + (size_t)bi * b_sb * esz;
        if (h16) {
            k_act_split<2><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(ab, a_sr, a_sc, k, kp, xh, xl, rs);
            k_dense_rows<true><<<dim3((unsigned)n), dim3(256), 0, dev->stream>>>(bb, b_sc, b_sr, k, kp, btp, cs);
        } else {
            k_act_split<0><<<dim3((unsigned)m), dim3(256), 0, dev->stream>>>(ab, a_sr, a_sc, k, kp, xh, xl, rs);
            k_dense_rows<false><<<dim3((unsigned)n), dim3(256), 0, dev->stream>>>(bb, b_sc, b_sr, k, kp, btp, cs);
        }
        FH_HIP(hipGetLastError());
        float *dst = h16 ? c32 : (float *)c_dev + (size_t)bi * m * n;
        FH_TRY((qmm_launch_dense<FH_W_F32, 2>(&qt, xh, xl, rs, m, dst, cs)));
        if (h16) FH_TRY(fh_cast_f32_f16(dev, c32, (_Float16 *)c_dev + (size_t)bi * m * n, (int64_t)m * n));
    }
    return FH_OK;
}

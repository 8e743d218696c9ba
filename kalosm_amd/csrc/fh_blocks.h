// Device-side accessors of the tiled weight layouts (see fh_internal.h) and the bit-exact
// block decode of the four GGUF formats.  The arithmetic follows GgufBlock::dequantize
// (fusor-ml/gguf/src/lib.rs:828-846, :1284-1288, :1526-1556, :2034-2085) operation for
// operation; the library is built with -ffp-contract=off so `a*b - c` is never fused.
#pragma once
#include "fh_internal.h"

typedef _Float16 fh_half;

__device__ __forceinline__ float fh_h2f(uint16_t bits) {
    fh_half h;
    __builtin_memcpy(&h, &bits, 2);
    return (float)h;
}

// ---- byte addresses inside a tile record -------------------------------------------------
// Q4_K: record 2304 B
__device__ __host__ __forceinline__ int q4k_hdr_off(int j) { return 16 * j; }
__device__ __host__ __forceinline__ int q4k_qs_off(int j, int i) { // i: byte 0..127 of the block's qs
    int p = i >> 6, w = i & 63, c2 = w >> 5, o = w & 31, g = o >> 3, r = o & 7;
    return 256 + p * 1024 + (g * 16 + j) * 16 + c2 * 8 + r;
}
// Q6_K: record 3360 B.  Element e (0..255, dequantised order) of row j: step t = e/32, lane group
// g = (e/8)%4, value v = e%8 of lane (g*16 + j).  The 6-bit code is stored as a low nibble in an L word
// (one per lane and step) and two high bits in an H word (one per lane and step pair), placed so that
// the f16 operand pair (v = 2p, v = 2p+1) of MFMA operand dword p comes out of one shift+AND each:
//   L word  = byte offset (t/4)*1024 + (g*16+j)*16 + (t%4)*4; nibble p + 4*(v%2)
//   H word  = byte offset 2048 + (g*16+j)*16 + (t/2)*4; bit position q6k_hbit(t, p) + 16*(v%2)
//   scales  = byte 3072 + ((G%8)/2*16 + j)*4 + 2*(G/8) + (G%2) for 16-element group G = e/16
//   d       = byte 3328 + 2*j
__device__ __host__ __forceinline__ int q6k_lword_off(int j, int t, int g) {
    return (t >> 2) * 1024 + (g * 16 + j) * 16 + (t & 3) * 4;
}
__device__ __host__ __forceinline__ int q6k_hword_off(int j, int t, int g) {
    return 2048 + (g * 16 + j) * 16 + (t >> 1) * 4;
}
__device__ __host__ __forceinline__ int q6k_hbit(int t, int p) {
    // even step of the pair: (H >> 2p) & 0x00300030;  odd step: (H << 4), (H << 2), (H >> 8), (H >> 10)
    return (t & 1) ? (p < 2 ? 2 * p : 8 + 2 * p) : 4 + 2 * p;
}
__device__ __host__ __forceinline__ int q6k_sc_off(int j, int G) {
    return 3072 + (((G & 7) >> 1) * 16 + j) * 4 + 2 * (G >> 3) + (G & 1);
}
__device__ __host__ __forceinline__ int q6k_d_off(int j) { return 3328 + 2 * j; }
// Q8_0: record 1088 B = two blocks
__device__ __host__ __forceinline__ int q80_q_off(int j, int u, int i) { // u: block in record, i: 0..31
    int g = i >> 3, r = i & 7;
    return (g * 16 + j) * 16 + u * 8 + r;
}
__device__ __host__ __forceinline__ int q80_d_off(int j, int u) { return 1024 + 4 * j + 2 * u; }
// Q4_0: record 1152 B = four blocks
__device__ __host__ __forceinline__ int q40_q_off(int j, int u, int i) { // i: byte 0..15
    int g = i >> 2, r = i & 3;
    return (g * 16 + j) * 16 + u * 4 + r;
}
__device__ __host__ __forceinline__ int q40_d_off(int j, int u) { return 1024 + 8 * j + 2 * u; }

__device__ __forceinline__ uint16_t fh_ld16(const uint8_t *p) { return *(const uint16_t *)p; }

// ---- one dequantised element -------------------------------------------------------------
__device__ __forceinline__ float deq_elem_q4_0(const QView &q, int64_t row, int64_t k) {
    int64_t b = k >> 5;
    int e = (int)(k & 31);
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + (b >> 2)) * (int64_t)q.rec_bytes;
    int j = (int)(row & 15), u = (int)(b & 3);
    float d = fh_h2f(fh_ld16(rec + q40_d_off(j, u)));
    uint8_t byte = rec[q40_q_off(j, u, e & 15)];
    int v = (e < 16 ? (byte & 0x0F) : (byte >> 4)) - 8;
    return (float)v * d;
}

__device__ __forceinline__ float deq_elem_q8_0(const QView &q, int64_t row, int64_t k) {
    int64_t b = k >> 5;
    int e = (int)(k & 31);
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + (b >> 1)) * (int64_t)q.rec_bytes;
    int j = (int)(row & 15), u = (int)(b & 1);
    float d = fh_h2f(fh_ld16(rec + q80_d_off(j, u)));
    int v = (int)(int8_t)rec[q80_q_off(j, u, e)];
    return (float)v * d;
}

__device__ __forceinline__ void q4k_scale_min(const uint8_t *p, int s, int &sc, int &mn) {
    if (s < 4) {
        sc = p[s] & 63;
        mn = p[4 + s] & 63;
    } else {
        sc = (p[4 + s] & 0x0F) | ((p[s - 4] >> 6) << 4);
        mn = (p[4 + s] >> 4) | ((p[s] >> 6) << 4);
    }
}

__device__ __forceinline__ float deq_elem_q4_k(const QView &q, int64_t row, int64_t k) {
    int64_t b = k >> 8;
    int e = (int)(k & 255);
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + b) * (int64_t)q.rec_bytes;
    int j = (int)(row & 15);
    const uint8_t *h = rec + q4k_hdr_off(j);
    float d = fh_h2f(fh_ld16(h)), dmin = fh_h2f(fh_ld16(h + 2));
    int s = e >> 5; // sub-block 0..7
    int sc, mn;
    q4k_scale_min(h + 4, s, sc, mn);
    int c = e >> 6, l = e & 31;
    uint8_t byte = rec[q4k_qs_off(j, 32 * c + l)];
    int v = (s & 1) ? (byte >> 4) : (byte & 0x0F);
    float scale = (float)sc * d;
    float off = (float)mn * dmin;
    float prod = scale * (float)v;
    return prod - off;
}

__device__ __forceinline__ float deq_elem_q6_k(const QView &q, int64_t row, int64_t k) {
    int64_t b = k >> 8;
    int e = (int)(k & 255);
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + b) * (int64_t)q.rec_bytes;
    int j = (int)(row & 15);
    int t = e >> 5, g = (e >> 3) & 3, vv = e & 7, p = vv >> 1, odd = vv & 1;
    uint32_t lw = *(const uint32_t *)(rec + q6k_lword_off(j, t, g));
    uint32_t hw = *(const uint32_t *)(rec + q6k_hword_off(j, t, g));
    int nib = (int)((lw >> (4 * (p + 4 * odd))) & 15u);
    int hb = (int)((hw >> (q6k_hbit(t, p) + 16 * odd)) & 3u);
    int v = ((hb << 4) | nib) - 32;
    int sc = (int)(int8_t)rec[q6k_sc_off(j, e >> 4)];
    float d = fh_h2f(fh_ld16(rec + q6k_d_off(j)));
    float ds = d * (float)sc;
    return ds * (float)v;
}

// ---- the 5-bit formats: the Q4_0 / Q4_K record followed by a plane of fifth bits
// Q5_K: record 2816 B; byte l (0..31) of the block's qh
__device__ __host__ __forceinline__ int q5k_qh_off(int j, int l) { return 2304 + ((l >> 3) * 16 + j) * 8 + (l & 7); }
// Q5_0: record 1408 B; the byte of block u that holds the fifth bits of the lane group g = (e % 16) / 4 of row j
__device__ __host__ __forceinline__ int q50_qh_off(int j, int u, int g) { return 1152 + (g * 16 + j) * 4 + u; }

// BlockQ5_0::dequantize, gguf/src/lib.rs:1046-1073: f16 d | 32 high bits | 16 bytes of nibbles;
// element i < 16: low nibble of byte i with bit i, element i + 16: high nibble with bit i + 16; (code - 16) * d
__device__ __forceinline__ float deq_elem_q5_0(const QView &q, int64_t row, int64_t k) {
    const int64_t b = k >> 5;
    const int e = (int)(k & 31), j = (int)(row & 15), u = (int)(b & 3);
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + (b >> 2)) * (int64_t)q.rec_bytes;
    const float d = fh_h2f(fh_ld16(rec + q40_d_off(j, u)));
    const uint8_t byte = rec[q40_q_off(j, u, e & 15)];
    const uint8_t hb = rec[q50_qh_off(j, u, (e & 15) >> 2)];
    const int nib = e < 16 ? (byte & 0x0F) : (byte >> 4);
    const int bit = (hb >> ((e & 3) + (e < 16 ? 0 : 4))) & 1;
    const int v = (nib | (bit << 4)) - 16;
    return (float)v * d;
}
// BlockQ5K::dequantize, gguf/src/lib.rs:1819-1861: f16 d | f16 dmin | 12 scale bytes | qh[32] | qs[128];
// sub-block s (32 elements): nibble of qs[32 (s / 2) + l] (low for even s) + 16 * bit s of qh[l];
// (sc * d) * code - mn * dmin
__device__ __forceinline__ float deq_elem_q5_k(const QView &q, int64_t row, int64_t k) {
    const uint8_t *rec = q.data + ((row >> 4) * q.recs + (k >> 8)) * (int64_t)q.rec_bytes;
    const int e = (int)(k & 255), s = e >> 5, l = e & 31, j = (int)(row & 15);
    const uint8_t *h = rec + q4k_hdr_off(j);
    const float d = fh_h2f(fh_ld16(h)), dmin = fh_h2f(fh_ld16(h + 2));
    int sc, mn;
    q4k_scale_min(h + 4, s, sc, mn);
    const uint8_t ql = rec[q4k_qs_off(j, 32 * (s >> 1) + l)], qh = rec[q5k_qh_off(j, l)];
    const int v = ((s & 1) ? (ql >> 4) : (ql & 0x0F)) + (((qh >> s) & 1) ? 16 : 0);
    const float scale = (float)sc * d;
    const float off = (float)mn * dmin;
    const float prod = scale * (float)v;
    return prod - off;
}
// ---- dense rows in the file's order
__device__ __forceinline__ float deq_elem_f16(const QView &q, int64_t row, int64_t k) {
    return fh_h2f(((const uint16_t *)q.data)[row * q.k + k]);
}
__device__ __forceinline__ float deq_elem_f32(const QView &q, int64_t row, int64_t k) {
    return ((const float *)q.data)[row * q.k + k];
}

template <int T>
__device__ __forceinline__ float deq_elem(const QView &q, int64_t row, int64_t k) {
    if (T == FH_Q5_0) return deq_elem_q5_0(q, row, k);
    if (T == FH_Q5_K) return deq_elem_q5_k(q, row, k);
    if (T == 0) return deq_elem_f32(q, row, k);
    if (T == 1) return deq_elem_f16(q, row, k);
    if (T == FH_Q4_0) return deq_elem_q4_0(q, row, k);
    if (T == FH_Q8_0) return deq_elem_q8_0(q, row, k);
    if (T == FH_Q4_K) return deq_elem_q4_k(q, row, k);
    return deq_elem_q6_k(q, row, k);
}

/*
 * fusor_cpu_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the CPU semantics of floneum/kalosm's Fusor
 * quantized-inference path (the Rust crates fusor-ml/gguf, fusor-ml/cpu,
 * fusor-ml/fusor and the decoder math of models/kalosm-llama).  The Rust
 * reference cannot be built where this repository is developed (no Rust
 * toolchain, un-vendored crates), so this file is the checker the HIP kernels
 * are compared with.  Only tests, the smoke check and the CPU-baseline leg of
 * the benchmark may link or call it; the product library never does.
 *
 * Every function cites the reference file:line it follows.  Build with
 *   gcc -O3 -mavx2 -mfma -ffp-contract=off
 * The contraction switch matters: Rust never fuses `a*b - c`, and the
 * dequantised values are compared bit for bit.  `fmaf()` below is an explicit
 * fused multiply-add wherever the reference calls `mul_add`.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   f16 conversion ........ exhaustive 65536-value round trip vs numpy.float16
 *   dequantize (4 formats)  reference known answers (+528/-528, nibble identity),
 *                           an independent numpy restatement, brute-force scale unpack
 *   dequantize Q5_0 / Q5_K  reference known answers (+528/-528, 32896, nibble identity, all high
 *                           bits -> 16), an independent numpy restatement, and the special case
 *                           qh = 0 where a Q5_K block must equal the Q4_K block bit for bit
 *   dense f16 / f32 rows .. the stored values; their product goes through the reference's dense
 *                           matmul (gemm crate): accumulation order UNPINNED, tolerance only
 *   q_mat_mul ............. one-hot / zero / linearity invariants, float64 dense product
 *   q8_0 quantize/vec_dot . closed form, exact integer sums, round trip < 0.02
 *   attention ............. float64 textbook form and torch CPU scaled_dot_product_attention (none, causal,
 *                           additive and per-batch key masks, grouped heads), causal row 0 = v_0, equal keys ->
 *                           mean of V, grouped heads == repeated KV heads (tests/test_oracle_ops.py)
 *   attention, f16 form ... one key -> v bit for bit, equal scores -> n * f16(1/n) * v, agreement with the f32
 *                           form on short rows, and the stall of the f16 running sum on long rows
 *   rms_norm .............. float64 formula of the reference's host check, residual and bias forms, zero row
 *   rope rotation ......... complex multiplication in float64 (both pairings, start positions), unit vectors
 *                           (signs and partner element), bit equality with the f32 host forms of the
 *                           reference's conformance suite
 *   rope tables ........... RoPE golden sextets; inverse-frequency closed form; composition of positions;
 *                           long-context scaling and rope_freqs weights against numpy
 *   silu / swiglu / add3 .. float64 closed form, fixed points, operand order
 *   embed_rows ............ rows of the independently dequantised table, bit for bit
 *   causal mask ........... numpy triu with the cache offset
 *   argmax ................ tie and non-finite cases from the reference's rule
 *   samplers .............. the reference's stored answers (flat logits: Mirostat 2 with random 0.8 -> id 0, top_p 0.5
 *                           with random 0.8 -> id 2, min_p 0.1 -> id 3, processed order -> id 0), the processor
 *                           case of its test (temperature 0.5, penalty 2, previous {0, 3, 9}) worked by hand,
 *                           sampled frequencies against the softmax probabilities, and the Mirostat update
 *                           against the closed form on two-candidate cases
 *   decoder ............... PARITY UNPINNED in the reference (no stored logits); pinned here by an independent
 *                           float64 numpy decoder (textbook ops on independently dequantised weights: prefill,
 *                           decode steps and a second chunk against the cache, groups of 1, 2 and 3 query heads
 *                           per KV head) on a two-layer configuration (tests/test_oracle_ops.py)
 *   Committed vectors: tests/golden/fusor_golden.npz (written by tests/golden/make_golden.py) holds edge blocks,
 *   [64, 512] matvecs, attention / rope / rms_norm / swiglu cases, a tiny decoder's logits and the values the
 *   reference's tests store; tests/test_golden.py holds this file to them.
 *   q_mat_mul summation order, attention dot order, expf/sinf/cosf/powf are
 *   machine/library dependent in the reference itself (pulp lane width, gemm
 *   crate, platform libm) and are held to tolerance, never to bit equality.
 */
#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FO_F32 0
#define FO_F16 1
#define FO_Q4_0 2
#define FO_Q5_0 6
#define FO_Q8_0 8
#define FO_Q4_K 12
#define FO_Q5_K 13
#define FO_Q6_K 14

/* ---------------------------------------------------------------- f16 <-> f32
 * The reference uses the `half` crate (IEEE binary16, round-to-nearest-even):
 * fusor-ml/gguf/src/lib.rs:766 (`half::f16` fields), conformance
 * common/quantized.rs:23-25 (`half::f16::from_f32`). */
float fo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t fo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
    if (ax < 0x33000001u) return (uint16_t)sign;               /* rounds to zero (<= 2^-25) */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q)); /* carry into the exponent is correct by construction */
}

void fo_f16_to_f32_array(const uint16_t *h, float *f, size_t n) {
    for (size_t i = 0; i < n; i++) f[i] = fo_f16_to_f32(h[i]);
}
void fo_f32_to_f16_array(const float *f, uint16_t *h, size_t n) {
    for (size_t i = 0; i < n; i++) h[i] = fo_f32_to_f16(f[i]);
}

/* ------------------------------------------------------------- block layouts
 * gguf/src/lib.rs:764-769 (Q4_0, 18 B), :1122-1127 (Q8_0, 34 B),
 * :1425-1432 (Q4_K, 144 B), :1933-1944 (Q6_K, 210 B; the f16 scale is LAST). */
int fo_block_elems(int t) {
    switch (t) {
    case FO_F32: case FO_F16: return 1;
    case FO_Q4_0: case FO_Q8_0: case FO_Q5_0: return 32;
    case FO_Q4_K: case FO_Q6_K: case FO_Q5_K: return 256;
    default: return 0;
    }
}
int fo_block_bytes(int t) {
    switch (t) {
    case FO_F32: return 4;
    case FO_F16: return 2;
    case FO_Q4_0: return 18;
    case FO_Q5_0: return 22;  /* gguf/src/lib.rs:958-966 */
    case FO_Q8_0: return 34;
    case FO_Q4_K: return 144;
    case FO_Q5_K: return 176; /* gguf/src/lib.rs:1703-1711 */
    case FO_Q6_K: return 210;
    default: return 0;
    }
}

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* gguf/src/lib.rs:828-846 */
static void deq_q4_0(const uint8_t *b, float *out) {
    float d = fo_f16_to_f32(rd16(b));
    const uint8_t *qs = b + 2;
    for (int i = 0; i < 16; i++) {
        int lo = (int)(qs[i] & 0x0F) - 8;
        int hi = (int)(qs[i] >> 4) - 8;
        out[i] = (float)lo * d;
        out[i + 16] = (float)hi * d;
    }
}

/* gguf/src/lib.rs:1284-1288 */
static void deq_q8_0(const uint8_t *b, float *out) {
    float d = fo_f16_to_f32(rd16(b));
    const int8_t *qs = (const int8_t *)(b + 2);
    for (int i = 0; i < 32; i++) out[i] = (float)qs[i] * d;
}

/* gguf/src/lib.rs:2138-2208 (first_scales_min_k4 / second_scales_min_k4) */
void fo_unpack_k4_scales(const uint8_t *p, uint8_t *sc, uint8_t *mn) {
    for (int j = 0; j < 4; j++) {
        sc[j] = p[j] & 63;
        mn[j] = p[4 + j] & 63;
        sc[4 + j] = (uint8_t)((p[8 + j] & 0x0F) | ((p[j] >> 6) << 4));
        mn[4 + j] = (uint8_t)((p[8 + j] >> 4) | ((p[4 + j] >> 6) << 4));
    }
}

/* gguf/src/lib.rs:1526-1556: (sc*d)*q - (m*dmin), the two products rounded separately */
static void deq_q4_k(const uint8_t *b, float *out) {
    float d = fo_f16_to_f32(rd16(b));
    float dmin = fo_f16_to_f32(rd16(b + 2));
    uint8_t sc[8], mn[8];
    fo_unpack_k4_scales(b + 4, sc, mn);
    const uint8_t *qs = b + 16;
    for (int c = 0; c < 4; c++) {
        float ls = (float)sc[2 * c] * d;
        float lo = (float)mn[2 * c] * dmin;
        float hs = (float)sc[2 * c + 1] * d;
        float ho = (float)mn[2 * c + 1] * dmin;
        for (int l = 0; l < 32; l++) {
            uint8_t w = qs[32 * c + l];
            out[64 * c + l] = ls * (float)(w & 0xF) - lo;
            out[64 * c + 32 + l] = hs * (float)(w >> 4) - ho;
        }
    }
}

/* gguf/src/lib.rs:2034-2085: scale * sc as f32 * q as f32, evaluated left to right */
static void deq_q6_k(const uint8_t *b, float *out) {
    const uint8_t *ql = b;
    const uint8_t *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    float d = fo_f16_to_f32(rd16(b + 208));
    for (int n = 0; n < 2; n++) {
        for (int l = 0; l < 32; l++) {
            int is = 8 * n + l / 16;
            uint8_t h = qh[32 * n + l];
            uint8_t a = ql[64 * n + l];
            uint8_t c = ql[64 * n + l + 32];
            int q1 = (int)(int8_t)(((h & 3) << 4) | (a & 0xF)) - 32;
            int q2 = (int)(int8_t)((((h >> 2) & 3) << 4) | (c & 0xF)) - 32;
            int q3 = (int)(int8_t)((((h >> 4) & 3) << 4) | (a >> 4)) - 32;
            int q4 = (int)(int8_t)((((h >> 6) & 3) << 4) | (c >> 4)) - 32;
            out[128 * n + l] = d * (float)sc[is] * (float)q1;
            out[128 * n + l + 32] = d * (float)sc[is + 2] * (float)q2;
            out[128 * n + l + 64] = d * (float)sc[is + 4] * (float)q3;
            out[128 * n + l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
    }
}

/* gguf/src/lib.rs:1046-1073 (BlockQ5_0): f16 scale, 32 high bits (little-endian u32), 16 nibble bytes.
 * element i takes bit i, element i + 16 bit i + 16; codes are centred at 16. */
static void deq_q5_0(const uint8_t *b, float *out) {
    float d = fo_f16_to_f32(rd16(b));
    uint32_t hb = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
    for (int i = 0; i < 16; i++) {
        uint8_t byte = b[6 + i];
        uint8_t low = byte & 0x0F, high = byte >> 4;
        uint8_t low_bit = (uint8_t)(((hb >> i) << 4) & 0x10);
        uint8_t high_bit = (uint8_t)((hb >> (i + 12)) & 0x10);
        int8_t lo = (int8_t)((low | low_bit) - 16), hi = (int8_t)((high | high_bit) - 16);
        out[i] = (float)lo * d;
        out[i + 16] = (float)hi * d;
    }
}

/* gguf/src/lib.rs:1819-1861 (BlockQ5K): d, dmin, 12 packed scale bytes (the Q4_K packing), qh[32], qs[128].
 * chunk c: d1 = sc[2c] * d, m1 = mn[2c] * dmin; low nibbles + 16 * bit 2c of qh[l], then high nibbles + bit 2c+1. */
static void deq_q5_k(const uint8_t *b, float *out) {
    float d = fo_f16_to_f32(rd16(b)), dmin = fo_f16_to_f32(rd16(b + 2));
    uint8_t sc[8], mn[8];
    fo_unpack_k4_scales(b + 4, sc, mn);
    const uint8_t *qh = b + 16, *qs = b + 48;
    uint8_t u1 = 1, u2 = 2;
    for (int c = 0; c < 4; c++) {
        float d1 = (float)sc[2 * c] * d, m1 = (float)mn[2 * c] * dmin;
        float d2 = (float)sc[2 * c + 1] * d, m2 = (float)mn[2 * c + 1] * dmin;
        for (int l = 0; l < 32; l++) {
            uint8_t q = (uint8_t)((qs[32 * c + l] & 0xF) + ((qh[l] & u1) ? 16 : 0));
            float p = d1 * (float)q;
            out[64 * c + l] = p - m1;
        }
        for (int l = 0; l < 32; l++) {
            uint8_t q = (uint8_t)((qs[32 * c + l] >> 4) + ((qh[l] & u2) ? 16 : 0));
            float p = d2 * (float)q;
            out[64 * c + 32 + l] = p - m2;
        }
        u1 = (uint8_t)(u1 << 2);
        u2 = (uint8_t)(u2 << 2);
    }
}

static void deq_block(int t, const uint8_t *b, float *out) {
    switch (t) {
    case FO_F32: memcpy(out, b, 4); break;
    case FO_F16: out[0] = fo_f16_to_f32(rd16(b)); break;
    case FO_Q5_0: deq_q5_0(b, out); break;
    case FO_Q5_K: deq_q5_k(b, out); break;
    case FO_Q4_0: deq_q4_0(b, out); break;
    case FO_Q8_0: deq_q8_0(b, out); break;
    case FO_Q4_K: deq_q4_k(b, out); break;
    case FO_Q6_K: deq_q6_k(b, out); break;
    }
}

/* cpu/src/quantized.rs:130-146 (QuantizedTensor::dequantize: block order = row-major) */
int fo_dequantize(int t, const uint8_t *bytes, size_t nblocks, float *out) {
    int e = fo_block_elems(t), bb = fo_block_bytes(t);
    if (!e) return -1;
    for (size_t i = 0; i < nblocks; i++) deq_block(t, bytes + i * bb, out + i * e);
    return 0;
}

/* ------------------------------------------------------------------ q_mat_mul
 * cpu/src/quantized.rs:641-675 (compute_dot_product) and :562-637
 * (process_row_simd_tiled).  Both evaluate, per output element, the same
 * sequence: lane l of an L-wide accumulator takes elements == l (mod L) of
 * every dequantised block in K order with a fused multiply-add, and the result
 * is the left fold of the lanes starting from 0.0 (cpu/src/reduce.rs:166-172).
 * The 4-column tiling only interleaves independent columns, so it is not
 * restated.  L is pulp's run-time SIMD width: 8 on an AVX2 host. */
#define FO_MAX_LANES 16
static float dot_row(int t, const float *x, const uint8_t *wrow, int blocks, int lanes) {
    int e = fo_block_elems(t), bb = fo_block_bytes(t);
    float acc[FO_MAX_LANES];
    float deq[256];
    for (int l = 0; l < lanes; l++) acc[l] = 0.0f;
    if (e == 1) {
        /* dense f32 / f16 rows: the reference multiplies them with its dense matmul (fusor/src/lib.rs:1183-1215 ->
         * gemm crate, accumulation order not pinned); here the same lane fold over the row with a scalar tail */
        int i = 0;
        for (; i + lanes <= blocks; i += lanes)
            for (int l = 0; l < lanes; l++) {
                deq_block(t, wrow + (size_t)(i + l) * bb, deq);
                acc[l] = fmaf(x[i + l], deq[0], acc[l]);
            }
        float s1 = 0.0f;
        for (int l = 0; l < lanes; l++) s1 = s1 + acc[l];
        for (; i < blocks; i++) {
            deq_block(t, wrow + (size_t)i * bb, deq);
            s1 = fmaf(x[i], deq[0], s1);
        }
        return s1;
    }
    for (int b = 0; b < blocks; b++) {
        deq_block(t, wrow + (size_t)b * bb, deq);
        const float *xb = x + (size_t)b * e;
        if (lanes == 8) {
            for (int i = 0; i < e; i += 8)
                for (int l = 0; l < 8; l++) acc[l] = fmaf(xb[i + l], deq[i + l], acc[l]);
        } else {
            for (int i = 0; i < e; i += lanes)
                for (int l = 0; l < lanes; l++) acc[l] = fmaf(xb[i + l], deq[i + l], acc[l]);
        }
    }
    float s = 0.0f;
    for (int l = 0; l < lanes; l++) s = s + acc[l];
    return s + 0.0f; /* `+ scalar_acc` with an empty tail (block sizes are multiples of L) */
}

typedef struct {
    int t, m, k, n, lanes;
    const float *x;
    const uint8_t *w;
    float *y;
    /* work slice */
    int row0, row1; /* activation rows   (m >= 4 split, cpu/src/quantized.rs:462-521) */
    int col0, col1; /* weight rows / output columns (m == 1 split, :404-461) */
} qmm_job;

static void *qmm_worker(void *arg) {
    qmm_job *j = (qmm_job *)arg;
    int e = fo_block_elems(j->t), bb = fo_block_bytes(j->t);
    int blocks = j->k / e;
    size_t rowbytes = (size_t)blocks * bb;
    for (int r = j->row0; r < j->row1; r++)
        for (int c = j->col0; c < j->col1; c++)
            j->y[(size_t)r * j->n + c] =
                dot_row(j->t, j->x + (size_t)r * j->k, j->w + (size_t)c * rowbytes, blocks, j->lanes);
    return NULL;
}

/* cpu/src/quantized.rs:246-365 + :389-537.  x is [m,k] contiguous f32, w is the raw
 * GGUF block stream of an [n,k] weight, y is [m,n].  nthreads <= 0 means one thread.
 * Threading follows the reference's static split: m == 1 splits output columns in
 * multiples of 32 (only when n >= 64), m >= 4 splits activation rows, m in {2,3} is
 * sequential.  The result does not depend on the thread count. */
int fo_q_mat_mul(int t, const float *x, int m, int k, const uint8_t *w, int n, float *y,
                 int lanes, int nthreads) {
    int e = fo_block_elems(t);
    if (!e || k % e != 0) return -1; /* cpu/src/quantized.rs:54-59 */
    if (lanes != 4 && lanes != 8 && lanes != 16) return -2;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    qmm_job jobs[256];
    pthread_t th[256];
    int nj = 0;
    qmm_job base = {t, m, k, n, lanes, x, w, y, 0, m, 0, n};
    if (m == 1 && n >= 64 && nthreads > 1) {
        int total_chunks = (n + 31) / 32;
        int per = (total_chunks + nthreads - 1) / nthreads * 32;
        for (int s = 0; s < n && nj < nthreads; s += per) {
            jobs[nj] = base;
            jobs[nj].col0 = s;
            jobs[nj].col1 = (nj == nthreads - 1 || s + per > n) ? n : s + per;
            if (nj == nthreads - 1) { nj++; break; }
            nj++;
        }
    } else if (m >= 4 && nthreads > 1) {
        int per = (m + nthreads - 1) / nthreads;
        for (int s = 0; s < m && nj < nthreads; s += per) {
            jobs[nj] = base;
            jobs[nj].row0 = s;
            jobs[nj].row1 = (nj == nthreads - 1 || s + per > m) ? m : s + per;
            if (nj == nthreads - 1) { nj++; break; }
            nj++;
        }
    } else {
        jobs[nj++] = base;
    }
    if (nj == 1) {
        qmm_worker(&jobs[0]);
        return 0;
    }
    for (int i = 0; i < nj; i++) pthread_create(&th[i], NULL, qmm_worker, &jobs[i]);
    for (int i = 0; i < nj; i++) pthread_join(th[i], NULL);
    return 0;
}

/* Same arithmetic per output element as fo_q_mat_mul, but each weight row is
 * dequantised once and reused for all m activation rows (the reference
 * re-dequantises per activation row, cpu/src/quantized.rs:467-477; the values it
 * produces are identical).  Used only so the checker finishes quickly at
 * prefill sizes; the timed CPU baseline uses fo_q_mat_mul. */
typedef struct {
    int t, m, k, n, lanes, c0, c1;
    const float *x;
    const uint8_t *w;
    float *y;
} qmm_fast_job;

static void *qmm_fast_worker(void *arg) {
    qmm_fast_job *j = (qmm_fast_job *)arg;
    int e = fo_block_elems(j->t), bb = fo_block_bytes(j->t);
    int blocks = j->k / e, L = j->lanes;
    float *deq = (float *)malloc((size_t)j->k * sizeof(float));
    for (int c = j->c0; c < j->c1; c++) {
        const uint8_t *wrow = j->w + (size_t)c * blocks * bb;
        for (int b = 0; b < blocks; b++) deq_block(j->t, wrow + (size_t)b * bb, deq + (size_t)b * e);
        for (int r = 0; r < j->m; r++) {
            const float *xr = j->x + (size_t)r * j->k;
            float acc[FO_MAX_LANES];
            for (int l = 0; l < L; l++) acc[l] = 0.0f;
            int i = 0;
            if (L == 8) {
                for (; i + 8 <= j->k; i += 8)
                    for (int l = 0; l < 8; l++) acc[l] = fmaf(xr[i + l], deq[i + l], acc[l]);
            } else {
                for (; i + L <= j->k; i += L)
                    for (int l = 0; l < L; l++) acc[l] = fmaf(xr[i + l], deq[i + l], acc[l]);
            }
            float s = 0.0f;
            for (int l = 0; l < L; l++) s = s + acc[l];
            s = s + 0.0f;
            for (; i < j->k; i++) s = fmaf(xr[i], deq[i], s); /* dense rows whose length is no multiple of L */
            j->y[(size_t)r * j->n + c] = s;
        }
    }
    free(deq);
    return NULL;
}

int fo_q_mat_mul_fast(int t, const float *x, int m, int k, const uint8_t *w, int n, float *y,
                      int lanes, int nthreads) {
    int e = fo_block_elems(t);
    if (!e || k % e != 0) return -1;
    if (lanes != 4 && lanes != 8 && lanes != 16) return -2;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    if (nthreads > n) nthreads = n > 0 ? n : 1;
    qmm_fast_job jobs[256];
    pthread_t th[256];
    int per = (n + nthreads - 1) / nthreads, nj = 0;
    for (int s = 0; s < n; s += per) {
        qmm_fast_job jb = {t, m, k, n, lanes, s, s + per > n ? n : s + per, x, w, y};
        jobs[nj++] = jb;
    }
    if (nj == 1) { qmm_fast_worker(&jobs[0]); return 0; }
    for (int i = 0; i < nj; i++) pthread_create(&th[i], NULL, qmm_fast_worker, &jobs[i]);
    for (int i = 0; i < nj; i++) pthread_join(th[i], NULL);
    return 0;
}

/* ------------------------------------------------- int8 activation path (Q8_0)
 * gguf/src/lib.rs:1150-1164 (quantize_scalar: `.round()` = half away from zero)
 * and :1166-1230 (quantize_avx2: `_mm256_cvtps_epi32` = half to even under the
 * default MXCSR).  `Self::quantize` picks the AVX2 form on any x86-64 host with
 * AVX2 (:1137-1147), so mode 0 (half-even) is what the reference computes on the
 * benchmark host; mode 1 is the scalar form.  They differ on exact ties only. */
void fo_q8_0_quantize(const float *x, size_t nblocks, uint8_t *out, int round_half_away) {
    for (size_t b = 0; b < nblocks; b++) {
        const float *v = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float a = fabsf(v[i]);
            amax = a > amax ? a : amax; /* f32::max / _mm256_max_ps on non-NaN input */
        }
        float scale = amax / 127.0f;
        float inv = amax != 0.0f ? 127.0f / amax : 0.0f;
        uint16_t h = fo_f32_to_f16(scale);
        uint8_t *o = out + b * 34;
        o[0] = (uint8_t)(h & 0xFF);
        o[1] = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; i++) {
            float p = v[i] * inv;
            float r;
            if (round_half_away) { /* .round().clamp(-127, 127) */
                r = roundf(p);
                r = r > 127.0f ? 127.0f : (r < -127.0f ? -127.0f : r);
            } else { /* cvtps_epi32 then two saturating packs: [-128, 127] */
                r = nearbyintf(p);
                r = r > 127.0f ? 127.0f : (r < -128.0f ? -128.0f : r);
            }
            o[2 + i] = (uint8_t)(int8_t)r;
        }
    }
}

/* gguf/src/lib.rs:1315-1358: (sum_i32 as f32) * (d_w * d_a) */
float fo_vec_dot_q8_0_q8_0(const uint8_t *w, const uint8_t *a) {
    int32_t s = 0;
    for (int i = 0; i < 32; i++) s += (int32_t)(int8_t)w[2 + i] * (int32_t)(int8_t)a[2 + i];
    float scale = fo_f16_to_f32(rd16(w)) * fo_f16_to_f32(rd16(a));
    return (float)s * scale;
}

/* gguf/src/lib.rs:927-938 (Q4_0 weights x Q8_0 activations) */
float fo_vec_dot_q4_0_q8_0(const uint8_t *w, const uint8_t *a) {
    int32_t s = 0;
    for (int i = 0; i < 16; i++) {
        int lo = (int)(w[2 + i] & 0x0F) - 8, hi = (int)(w[2 + i] >> 4) - 8;
        s += lo * (int32_t)(int8_t)a[2 + i];
        s += hi * (int32_t)(int8_t)a[2 + i + 16];
    }
    float scale = fo_f16_to_f32(rd16(w)) * fo_f16_to_f32(rd16(a));
    return (float)s * scale;
}

/* The Q8_0 x Q8 matmul variant: activations quantised per 32 along K, each output
 * is the f32 sum over K-blocks (in K order) of vec_dot.  The reference defines the
 * per-block product (above); the block-sum order is this build's choice and is
 * therefore held to tolerance.  isums (optional, [m,n,k/32]) receives the exact
 * integer block sums, which the GPU int8 path must reproduce bit for bit. */
int fo_q8_0_matmul_q8(const float *x, int m, int k, const uint8_t *w, int n, float *y,
                      int32_t *isums, int round_half_away) {
    if (k % 32) return -1;
    int kb = k / 32;
    uint8_t *aq = (uint8_t *)malloc((size_t)m * kb * 34);
    fo_q8_0_quantize(x, (size_t)m * kb, aq, round_half_away);
    for (int r = 0; r < m; r++)
        for (int c = 0; c < n; c++) {
            float acc = 0.0f;
            for (int b = 0; b < kb; b++) {
                const uint8_t *wb = w + ((size_t)c * kb + b) * 34;
                const uint8_t *ab = aq + ((size_t)r * kb + b) * 34;
                if (isums) {
                    int32_t s = 0;
                    for (int i = 0; i < 32; i++) s += (int32_t)(int8_t)wb[2 + i] * (int32_t)(int8_t)ab[2 + i];
                    isums[((size_t)r * n + c) * kb + b] = s;
                }
                acc = acc + fo_vec_dot_q8_0_q8_0(wb, ab);
            }
            y[(size_t)r * n + c] = acc;
        }
    free(aq);
    return 0;
}

/* ------------------------------------------------------------------ attention
 * fusor/src/composite/flash_attention.rs:113-236: expand K/V over the GQA groups
 * (kv head = h / groups), S = Q.K^T, * scale, + mask, row max, subtract, exp, row
 * sum, divide, . V.  Every step in f32 with libm expf (cpu/src/elementwise.rs:157).
 * mask_kind: 0 none, 1 causal generated here as attention_mask.rs:46-66 with the
 * cache offset of mask_cache.rs:73-88 (query i sees keys j <= i + (skv - sq)),
 * 2 additive [sq, skv] mask supplied by the caller (MaskKind::QKMask), 3 additive [b, skv] mask
 * broadcast over heads and queries (MaskKind::BatchKeyMask, flash_attention.rs:199-213).
 * Layout: q [b,h,sq,d], k/v [b,hkv,skv,d], out [b,h,sq,d], all contiguous.
 * One score row is materialised at a time; the arithmetic per row is that of the
 * reference. */
typedef struct {
    const float *q, *k, *v, *mask;
    float *out;
    int b, h, hkv, sq, skv, d, mask_kind;
    float scale;
    int bh0, bh1;
} att_job;

static void *att_worker(void *arg) {
    att_job *j = (att_job *)arg;
    int groups = j->h / j->hkv;
    float *s = (float *)malloc((size_t)j->skv * sizeof(float));
    float ninf = -INFINITY;
    for (int bh = j->bh0; bh < j->bh1; bh++) {
        int bi = bh / j->h, hi = bh % j->h, kh = hi / groups;
        const float *qh = j->q + ((size_t)bi * j->h + hi) * j->sq * j->d;
        const float *kk = j->k + ((size_t)bi * j->hkv + kh) * j->skv * j->d;
        const float *vv = j->v + ((size_t)bi * j->hkv + kh) * j->skv * j->d;
        float *oh = j->out + ((size_t)bi * j->h + hi) * j->sq * j->d;
        for (int i = 0; i < j->sq; i++) {
            const float *qi = qh + (size_t)i * j->d;
            float mx = ninf;
            for (int t = 0; t < j->skv; t++) {
                float acc = 0.0f;
                for (int c = 0; c < j->d; c++) acc += qi[c] * kk[(size_t)t * j->d + c];
                acc = acc * j->scale;
                if (j->mask_kind == 1) {
                    if (t > i + (j->skv - j->sq)) acc = acc + ninf;
                } else if (j->mask_kind == 2) {
                    acc = acc + j->mask[(size_t)i * j->skv + t];
                } else if (j->mask_kind == 3) {
                    acc = acc + j->mask[(size_t)bi * j->skv + t];
                }
                s[t] = acc;
                mx = acc > mx ? acc : mx;
            }
            float sum = 0.0f;
            for (int t = 0; t < j->skv; t++) {
                s[t] = expf(s[t] - mx);
                sum += s[t];
            }
            for (int t = 0; t < j->skv; t++) s[t] = s[t] / sum;
            for (int c = 0; c < j->d; c++) oh[(size_t)i * j->d + c] = 0.0f;
            for (int t = 0; t < j->skv; t++) {
                float p = s[t];
                const float *vt = vv + (size_t)t * j->d;
                for (int c = 0; c < j->d; c++) oh[(size_t)i * j->d + c] += p * vt[c];
            }
        }
    }
    free(s);
    return NULL;
}

int fo_flash_attention(const float *q, const float *k, const float *v, int b, int h, int hkv,
                       int sq, int skv, int d, float scale, int mask_kind, const float *mask,
                       float *out, int nthreads) {
    if (hkv <= 0 || h % hkv) return -1; /* flash_attention.rs:131-136 */
    if ((mask_kind == 2 || mask_kind == 3) && !mask) return -2;
    int total = b * h;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > total) nthreads = total;
    if (nthreads > 256) nthreads = 256;
    att_job jobs[256];
    pthread_t th[256];
    int per = (total + nthreads - 1) / nthreads, nj = 0;
    for (int s = 0; s < total; s += per) {
        att_job jb = {q, k, v, mask, out, b, h, hkv, sq, skv, d, mask_kind, scale, s,
                      s + per > total ? total : s + per};
        jobs[nj++] = jb;
    }
    if (nj == 1) { att_worker(&jobs[0]); return 0; }
    for (int i = 0; i < nj; i++) pthread_create(&th[i], NULL, att_worker, &jobs[i]);
    for (int i = 0; i < nj; i++) pthread_join(th[i], NULL);
    return 0;
}

/* The reference's f16 instantiation of the same composite: every tensor op yields f16, i.e. the value is
 * computed in f32 and rounded to f16 after EVERY op.  matmul: f32 sum over k, one rounding per output
 * (cpu/src/matmul.rs:159-179); mul_scalar / + mask / - max / exp / div: one rounding each
 * (cpu/src/pairwise.rs:157-160, cpu/src/elementwise.rs:222); the row sum folds left to right with a rounding
 * to f16 after every add (cpu/src/reduce.rs:228-237), so once the running sum's f16 spacing exceeds twice an
 * addend the addend is lost; max is exact.  q, k, v and out are f16 bit patterns; mask_kind 0 or 1 (the causal
 * mask holds 0 / -inf, exact in f16).  Single-threaded: it exists to show what the f16 CPU path yields on small cases. */
static float fo_r16(float x) { return fo_f16_to_f32(fo_f32_to_f16(x)); }
int fo_flash_attention_f16(const uint16_t *q, const uint16_t *k, const uint16_t *v, int b, int h, int hkv, int sq,
                           int skv, int d, float scale, int mask_kind, uint16_t *out) {
    if (hkv <= 0 || h % hkv) return -1;
    if (mask_kind != 0 && mask_kind != 1) return -2;
    int groups = h / hkv;
    float sc16 = fo_r16(scale); /* D::from_f32(scale) */
    float *s = (float *)malloc((size_t)skv * sizeof(float));
    for (int bh = 0; bh < b * h; bh++) {
        int bi = bh / h, hi = bh % h, kh = hi / groups;
        const uint16_t *qh = q + ((size_t)bi * h + hi) * sq * d;
        const uint16_t *kk = k + ((size_t)bi * hkv + kh) * skv * d;
        const uint16_t *vv = v + ((size_t)bi * hkv + kh) * skv * d;
        uint16_t *oh = out + ((size_t)bi * h + hi) * sq * d;
        for (int i = 0; i < sq; i++) {
            float mx = -INFINITY;
            for (int t = 0; t < skv; t++) {
                float acc = 0.0f;
                for (int c = 0; c < d; c++)
                    acc += fo_f16_to_f32(qh[(size_t)i * d + c]) * fo_f16_to_f32(kk[(size_t)t * d + c]);
                acc = fo_r16(acc);
                acc = fo_r16(acc * sc16);
                if (mask_kind == 1) acc = fo_r16(acc + ((t > i + (skv - sq)) ? -INFINITY : 0.0f));
                s[t] = acc;
                mx = acc > mx ? acc : mx;
            }
            float sum = 0.0f;
            for (int t = 0; t < skv; t++) {
                s[t] = fo_r16(expf(fo_r16(s[t] - mx)));
                sum = fo_r16(sum + s[t]);
            }
            for (int t = 0; t < skv; t++) s[t] = fo_r16(s[t] / sum);
            for (int c = 0; c < d; c++) {
                float acc = 0.0f;
                for (int t = 0; t < skv; t++) acc += s[t] * fo_f16_to_f32(vv[(size_t)t * d + c]);
                oh[(size_t)i * d + c] = fo_f32_to_f16(acc);
            }
        }
    }
    free(s);
    return 0;
}

/* fusor/src/cache/attention_mask.rs:46-66 with the zero left padding of
 * mask_cache.rs:73-88: mask is [s, p + s]. */
void fo_causal_mask(int s, int p, float *mask) {
    for (int i = 0; i < s; i++)
        for (int t = 0; t < p + s; t++) mask[(size_t)i * (p + s) + t] = (t > i + p) ? -INFINITY : 0.0f;
}

/* ------------------------------------------------------------------- rms_norm
 * fusor/src/composite/normalization.rs:404-460: x^2 -> sum/len -> +eps -> sqrt ->
 * x / rms -> * w (+ bias); the residual form first adds x + residual (:394-397).
 * The row sum follows the reference's SIMD reduction only to tolerance. */
void fo_rms_norm(const float *x, const float *residual, const float *w, const float *bias,
                 float eps, int rows, int cols, float *y) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * cols;
        const float *rr = residual ? residual + (size_t)r * cols : NULL;
        float *yr = y + (size_t)r * cols;
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int c = 0;
        for (; c + 8 <= cols; c += 8)
            for (int l = 0; l < 8; l++) {
                float t = rr ? xr[c + l] + rr[c + l] : xr[c + l];
                acc[l] = acc[l] + t * t;
            }
        float s = 0.0f;
        for (int l = 0; l < 8; l++) s = s + acc[l];
        for (; c < cols; c++) {
            float t = rr ? xr[c] + rr[c] : xr[c];
            s = s + t * t;
        }
        float mean = s / (float)cols;
        float rms = sqrtf(mean + eps);
        for (c = 0; c < cols; c++) {
            float t = rr ? xr[c] + rr[c] : xr[c];
            float o = (t / rms) * w[c];
            yr[c] = bias ? o + bias[c] : o;
        }
    }
}

/* ----------------------------------------------------------------------- rope
 * fusor/src/composite/rope.rs:241-246 (inverse frequency, f32 powf) and
 * models/kalosm-llama/src/raw/rope.rs:63-85 (outer product position * inv in f32,
 * then f32 sin / cos).  cos and sin are [ctx, dim/2]. */
void fo_rope_inverse_frequency(int dim, float theta, float *inv) {
    for (int i = 0; i < dim; i += 2) inv[i / 2] = 1.0f / powf(theta, (float)i / (float)dim);
}
/* freq_weight (optional, dim/2 values): the `rope_freqs.weight` tensor of a model file; the inverse
 * frequencies are MULTIPLIED by it (models/kalosm-llama/src/raw/rope.rs:41-48). */
/* scaling (optional): {factor, high_freq_factor, low_freq_factor, original_max_position_embeddings as float},
 * models/kalosm-llama/src/raw/rope.rs:20-38.  Note the `==` of the smooth branch (:32), kept as written. */
void fo_rope_scale_inverse_frequency(float *inv, int half, const float *scaling) {
    float factor = scaling[0], high = scaling[1], low = scaling[2], orig = scaling[3];
    float low_wavelen = orig / low, high_wavelen = orig / high;
    for (int i = 0; i < half; i++) {
        float wavelen = 2.0f * 3.14159265358979323846f / inv[i];
        if (wavelen > low_wavelen) inv[i] = inv[i] / factor;
        else if (wavelen == high_wavelen) {
            float smooth = (orig / wavelen - low) / (high - low);
            inv[i] = (1.0f - smooth) * inv[i] / factor + smooth * inv[i];
        }
    }
}
void fo_rope_tables_scaled(int dim, int ctx, float theta, const float *scaling, const float *freq_weight, float *cosv,
                           float *sinv);
void fo_rope_tables_weighted(int dim, int ctx, float theta, const float *freq_weight, float *cosv, float *sinv) {
    fo_rope_tables_scaled(dim, ctx, theta, NULL, freq_weight, cosv, sinv);
}
void fo_rope_tables_scaled(int dim, int ctx, float theta, const float *scaling, const float *freq_weight, float *cosv,
                           float *sinv) {
    int half = dim / 2;
    float *inv = (float *)malloc((size_t)half * sizeof(float));
    fo_rope_inverse_frequency(dim, theta, inv);
    if (scaling) fo_rope_scale_inverse_frequency(inv, half, scaling);
    if (freq_weight)
        for (int i = 0; i < half; i++) inv[i] = inv[i] * freq_weight[i];
    for (int p = 0; p < ctx; p++)
        for (int i = 0; i < half; i++) {
            float a = (float)p * inv[i];
            cosv[(size_t)p * half + i] = cosf(a);
            sinv[(size_t)p * half + i] = sinf(a);
        }
    free(inv);
}
void fo_rope_tables(int dim, int ctx, float theta, float *cosv, float *sinv) {
    fo_rope_tables_weighted(dim, ctx, theta, NULL, cosv, sinv);
}

/* fusor/src/composite/rope.rs:77-108 (interleaved: pairs (2i, 2i+1)) and :46-68
 * (half split: pairs (i, i + d/2), out = x*cos + rotate_half(x)*sin); rows
 * [start_pos, start_pos + s) of the tables (:309-329).  x is [b,h,s,d] contiguous
 * and is rotated into y.  Each product is rounded before the add/sub. */
void fo_rope(const float *x, int b, int h, int s, int d, const float *cosv, const float *sinv,
             int start_pos, int interleaved, float *y) {
    int half = d / 2;
    for (int bh = 0; bh < b * h; bh++)
        for (int t = 0; t < s; t++) {
            const float *xr = x + ((size_t)bh * s + t) * d;
            float *yr = y + ((size_t)bh * s + t) * d;
            const float *c = cosv + (size_t)(start_pos + t) * half;
            const float *sn = sinv + (size_t)(start_pos + t) * half;
            for (int i = 0; i < half; i++) {
                if (interleaved) {
                    float x0 = xr[2 * i], x1 = xr[2 * i + 1];
                    float ac = x0 * c[i], bs = x1 * sn[i];
                    float as = x0 * sn[i], bc = x1 * c[i];
                    yr[2 * i] = ac - bs;
                    yr[2 * i + 1] = as + bc;
                } else {
                    float x0 = xr[i], x1 = xr[i + half];
                    float a0 = x0 * c[i], r0 = (-x1) * sn[i];
                    float a1 = x1 * c[i], r1 = x0 * sn[i];
                    yr[i] = a0 + r0;
                    yr[i + half] = a1 + r1;
                }
            }
        }
}

/* --------------------------------------------------------------- activations
 * fusor/src/composite/activations.rs:47-65: silu(x) = x / (exp(-x) + 1);
 * models/kalosm-llama/src/raw/attention_layer.rs:186-196: silu(gate) * up. */
void fo_silu(const float *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = x[i] / (expf(-x[i]) + 1.0f);
}
void fo_swiglu(const float *gate, const float *up, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = (gate[i] / (expf(-gate[i]) + 1.0f)) * up[i];
}
/* raw/attention_layer.rs:168-173 and raw/mod.rs:1036: (a + b) + c */
void fo_add3(const float *a, const float *b, const float *c, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = (a[i] + b[i]) + c[i];
}

/* fusor/src/lib.rs:416-447 with k = 1: largest finite logit, ties to the LARGER
 * token id, non-finite values skipped.  Returns -1 when nothing is finite. */
int64_t fo_argmax(const float *x, size_t n) {
    int64_t best = -1;
    float bv = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float v = x[i];
        if (!isfinite(v)) continue;
        if (best < 0 || v > bv || v == bv) {
            best = (int64_t)i;
            bv = v;
        }
    }
    return best;
}

/* fusor/src/lib.rs:416-447 for any k: the insertion loop as written (a sorted list of at most k pairs; a new
 * finite logit replaces the last one when it is larger, or equal with a larger token id).  Returns the count. */
int fo_top_k(const float *x, size_t n, int k, uint32_t *ids, float *vals) {
    int len = 0;
    if (k <= 0) return 0;
    for (size_t t = 0; t < n; t++) {
        float v = x[t];
        if (!isfinite(v)) continue;
        if (len == k) {
            float lv = vals[len - 1];
            uint32_t li = ids[len - 1];
            if (v > lv || (v == lv && (uint32_t)t > li)) len = k - 1;
            else continue;
        }
        int at = 0; /* partition point: entries that stay in front of the new one */
        while (at < len && (vals[at] > v || (vals[at] == v && ids[at] > (uint32_t)t))) at++;
        for (int i = len; i > at; i--) { vals[i] = vals[i - 1]; ids[i] = ids[i - 1]; }
        vals[at] = v;
        ids[at] = (uint32_t)t;
        len++;
    }
    return len;
}

/* Device sampling of fusor-ml/core/src/sampling, restated step by step.
 * Processors (row_kernels.rs:150-205; host form process_logit, models/kalosm-llama/src/sampler.rs:275-307): a
 * non-finite logit is dropped; one whose id is among `prev` is multiplied (<= 0) or divided (> 0) by a repetition
 * penalty above 1; a non-zero temperature divides; a non-finite result is dropped.
 * Top-k: descending, ties to the larger id (better_candidate, row_kernels.rs:85-87); slots past the finite
 * candidates read as value -FLT_MAX / id 0xFFFFFFFF (sampler_top_value / sampler_top_id, :484-497).
 * Standard sampler: row_kernels.rs:799-919.  Mirostat 2: :672-797.  weighted_pick: :609-660.
 * result = [status, token]: 1 sampled, 2 no finite logit (emit_sampler_guards, :518-545).
 * *margin (optional) = the smallest relative gap of any comparison that decided the outcome; a caller comparing
 * against another exp / log2 implementation can set cases with a tiny margin aside. */
typedef struct {
    uint32_t kind, top_k;
    float temperature, repetition_penalty, top_p, min_p, tau, eta, random;
} fo_sampler_params;

static void fo_gap(float *margin, float a, float b) {
    if (!margin) return;
    float m = fmaxf(fmaxf(fabsf(a), fabsf(b)), 1e-30f);
    float g = fabsf(a - b) / m;
    if (g < *margin) *margin = g;
}

int fo_process_logits(const float *x, size_t n, float temperature, float penalty, const uint32_t *prev, uint32_t n_prev,
                      float *out) {
    for (size_t t = 0; t < n; t++) {
        float v = x[t];
        if (isfinite(v)) {
            int repeated = 0;
            for (uint32_t j = 0; j < n_prev; j++) repeated |= prev[j] == (uint32_t)t;
            if (repeated && penalty > 1.0f) v = v <= 0.0f ? v * penalty : v / penalty;
            if (temperature != 0.0f) v = v / temperature;
        }
        out[t] = v; /* what is not finite here is skipped by the top-k */
    }
    return 0;
}

int fo_sample_token(const float *logits, size_t n, const fo_sampler_params *p, const uint32_t *prev, uint32_t n_prev,
                    float *mu_state, uint32_t *result, uint32_t *ids, float *vals, float *margin) {
    const float eps = 1.0e-20f;
    int k = (int)p->top_k;
    if (k < 1 || k > 256) return -1;
    float *proc = (float *)malloc(n * sizeof(float));
    if (!proc) return -2;
    fo_process_logits(logits, n, p->temperature, p->repetition_penalty, prev, n_prev, proc);
    int found = fo_top_k(proc, n, k, ids, vals);
    free(proc);
    for (int i = found; i < k; i++) { ids[i] = 0xFFFFFFFFu; vals[i] = -FLT_MAX; }
    if (margin) *margin = 1.0f;
    if (ids[0] == 0xFFFFFFFFu) { result[0] = 2; result[1] = 0; return 0; }
    float w[256] = {0};
    for (int i = 0; i < k; i++) w[i] = expf(vals[i] - vals[0]);
    int cutoff = k;
    float cutoff_sum = 0.f, mu = 0.f;
    if (p->kind == 1) {
        float total = 0.f;
        for (int i = 0; i < k; i++) total += w[i];
        total = fmaxf(total, eps);
        mu = *mu_state;
        for (int i = 0; i < k; i++) {
            float pr = fmaxf(w[i] / total, eps);
            float surprise = log2f(pr) * -1.0f;
            fo_gap(margin, surprise, mu);
            if (surprise > mu) { cutoff = i > 1 ? i : 1; break; }
        }
        for (int i = 0; i < cutoff; i++) cutoff_sum += w[i];
    } else {
        float filtered = 0.f;
        for (int i = 0; i < k; i++) {
            fo_gap(margin, w[i], p->min_p);
            if (w[i] >= p->min_p) filtered += w[i];
        }
        float target = fmaxf(filtered, eps) * p->top_p;
        for (int i = 0; i < k; i++) {
            if (w[i] >= p->min_p) {
                cutoff_sum += w[i];
                fo_gap(margin, cutoff_sum, target);
                if (cutoff_sum >= target) { cutoff = i + 1; break; }
            } else { cutoff = i; break; }
        }
        if (cutoff == 0) { cutoff = 1; cutoff_sum = w[0]; }
    }
    cutoff_sum = fmaxf(cutoff_sum, eps);
    float threshold = p->random * cutoff_sum;
    uint32_t token = ids[0];
    float prob = w[0] / cutoff_sum, cum = 0.f;
    for (int i = 0; i < cutoff; i++) {
        cum += w[i];
        fo_gap(margin, cum, threshold);
        if (cum >= threshold) { token = ids[i]; prob = w[i] / cutoff_sum; break; }
    }
    if (p->kind == 1) {
        float surprise = log2f(fmaxf(prob, eps)) * -1.0f;
        float error = surprise - p->tau;
        float correction = p->eta * error;
        *mu_state = mu - correction;
    }
    result[0] = 1;
    result[1] = token;
    return 0;
}

/* fusor/src/layers/embedding.rs:43-89: out[t,:] = dequantize(W)[id[t],:] */
int fo_embed_rows(int t, const uint8_t *w, int n, int k, const uint32_t *ids, int count, float *out) {
    int e = fo_block_elems(t), bb = fo_block_bytes(t);
    if (!e || k % e) return -1;
    size_t rowbytes = (size_t)(k / e) * bb;
    for (int i = 0; i < count; i++) {
        if ((int)ids[i] >= n) return -2;
        fo_dequantize(t, w + (size_t)ids[i] * rowbytes, (size_t)(k / e), out + (size_t)i * k);
    }
    return 0;
}

/* -------------------------------------------------------------------- decoder
 * models/kalosm-llama/src/raw/mod.rs:925-1049 with the Separate attention variant
 * (raw/attention_layer.rs:281-426, :514-573, :659-694) and the Llama feed-forward
 * (:130-237); interleaved RoPE (raw/mod.rs:488-490); f32 KV cache
 * (raw/cache.rs:18).  One call runs `s` new tokens at position `pos` and returns
 * the logits of the last one (raw/mod.rs:851-865, :1045-1046). */
typedef struct {
    int n_layers, d_model, n_heads, n_kv_heads, head_dim, ffn, vocab, ctx;
    float eps, theta;
    int type_attn, type_ffn_gate_up, type_ffn_down, type_embd, type_output;
} fo_llama_config;

typedef struct {
    const uint8_t *wq, *wk, *wv, *wo, *gate, *up, *down;
    const float *attn_norm, *ffn_norm;
    int tq, tk, tv, to, tgate, tup, tdown; /* block type of each weight (model files mix them per layer) */
} fo_llama_layer;

typedef struct {
    fo_llama_config c;
    fo_llama_layer *layers;
    const uint8_t *embd, *output;
    const float *out_norm;
    float *cosv, *sinv;
    float **kc, **vc; /* per layer [n_kv_heads, ctx, head_dim] */
    int len;
    int nthreads;
} fo_llama;

fo_llama *fo_llama_create(const fo_llama_config *c, int nthreads) {
    fo_llama *m = (fo_llama *)calloc(1, sizeof(fo_llama));
    m->c = *c;
    m->layers = (fo_llama_layer *)calloc((size_t)c->n_layers, sizeof(fo_llama_layer));
    m->cosv = (float *)malloc((size_t)c->ctx * (c->head_dim / 2) * sizeof(float));
    m->sinv = (float *)malloc((size_t)c->ctx * (c->head_dim / 2) * sizeof(float));
    fo_rope_tables(c->head_dim, c->ctx, c->theta, m->cosv, m->sinv);
    m->kc = (float **)calloc((size_t)c->n_layers, sizeof(float *));
    m->vc = (float **)calloc((size_t)c->n_layers, sizeof(float *));
    for (int l = 0; l < c->n_layers; l++) {
        m->kc[l] = (float *)calloc((size_t)c->n_kv_heads * c->ctx * c->head_dim, sizeof(float));
        m->vc[l] = (float *)calloc((size_t)c->n_kv_heads * c->ctx * c->head_dim, sizeof(float));
    }
    m->nthreads = nthreads < 1 ? 1 : nthreads;
    return m;
}
void fo_llama_set_layer(fo_llama *m, int l, const uint8_t *wq, const uint8_t *wk, const uint8_t *wv,
                        const uint8_t *wo, const uint8_t *gate, const uint8_t *up,
                        const uint8_t *down, const float *attn_norm, const float *ffn_norm) {
    fo_llama_layer *y = &m->layers[l];
    y->wq = wq; y->wk = wk; y->wv = wv; y->wo = wo;
    y->gate = gate; y->up = up; y->down = down;
    y->attn_norm = attn_norm; y->ffn_norm = ffn_norm;
    y->tq = y->tk = y->tv = y->to = m->c.type_attn;
    y->tgate = y->tup = m->c.type_ffn_gate_up;
    y->tdown = m->c.type_ffn_down;
}
/* types: q, k, v, o, gate, up, down -- call after fo_llama_set_layer */
void fo_llama_set_layer_types(fo_llama *m, int l, const int *types) {
    fo_llama_layer *y = &m->layers[l];
    y->tq = types[0]; y->tk = types[1]; y->tv = types[2]; y->to = types[3];
    y->tgate = types[4]; y->tup = types[5]; y->tdown = types[6];
}
void fo_llama_set_rope_freq_weight(fo_llama *m, const float *w) {
    fo_rope_tables_weighted(m->c.head_dim, m->c.ctx, m->c.theta, w, m->cosv, m->sinv);
}
/* scaling = {factor, high_freq_factor, low_freq_factor, original_max_position_embeddings} or NULL; w or NULL */
void fo_llama_set_rope(fo_llama *m, const float *scaling, const float *w) {
    fo_rope_tables_scaled(m->c.head_dim, m->c.ctx, m->c.theta, scaling, w, m->cosv, m->sinv);
}
void fo_llama_set_globals(fo_llama *m, const uint8_t *embd, const float *out_norm, const uint8_t *output) {
    m->embd = embd; m->out_norm = out_norm; m->output = output;
}
void fo_llama_reset(fo_llama *m) { m->len = 0; }
void fo_llama_destroy(fo_llama *m) {
    if (!m) return;
    for (int l = 0; l < m->c.n_layers; l++) { free(m->kc[l]); free(m->vc[l]); }
    free(m->kc); free(m->vc); free(m->cosv); free(m->sinv); free(m->layers); free(m);
}

static void to_heads(const float *x, int s, int h, int d, float *y) { /* [s,h,d] -> [h,s,d] */
    for (int t = 0; t < s; t++)
        for (int i = 0; i < h; i++)
            memcpy(y + ((size_t)i * s + t) * d, x + ((size_t)t * h + i) * d, (size_t)d * sizeof(float));
}
static void from_heads(const float *x, int s, int h, int d, float *y) { /* [h,s,d] -> [s,h,d] */
    for (int t = 0; t < s; t++)
        for (int i = 0; i < h; i++)
            memcpy(y + ((size_t)t * h + i) * d, x + ((size_t)i * s + t) * d, (size_t)d * sizeof(float));
}

/* hidden_out (optional) receives the final-norm hidden state of the last token. */
int fo_llama_forward(fo_llama *m, const uint32_t *tokens, int s, float *logits, float *hidden_out) {
    const fo_llama_config *c = &m->c;
    int D = c->d_model, H = c->n_heads, HK = c->n_kv_heads, hd = c->head_dim, F = c->ffn;
    int pos = m->len, nt = m->nthreads, L = 8;
    if (pos + s > c->ctx) return -1;
    size_t sd = (size_t)s * D;
    float *x = (float *)malloc(sd * 4), *xn = (float *)malloc(sd * 4), *att = (float *)malloc(sd * 4);
    float *q = (float *)malloc((size_t)s * H * hd * 4), *qh = (float *)malloc((size_t)s * H * hd * 4);
    float *qr = (float *)malloc((size_t)s * H * hd * 4);
    float *k = (float *)malloc((size_t)s * HK * hd * 4), *kh = (float *)malloc((size_t)s * HK * hd * 4);
    float *kr = (float *)malloc((size_t)s * HK * hd * 4);
    float *v = (float *)malloc((size_t)s * HK * hd * 4), *vh = (float *)malloc((size_t)s * HK * hd * 4);
    float *ao = (float *)malloc((size_t)s * H * hd * 4), *ao2 = (float *)malloc((size_t)s * H * hd * 4);
    float *g = (float *)malloc((size_t)s * F * 4), *u = (float *)malloc((size_t)s * F * 4);
    float *act = (float *)malloc((size_t)s * F * 4), *ff = (float *)malloc(sd * 4);
    int len = pos + s;
    float *kall = (float *)malloc((size_t)HK * len * hd * 4), *vall = (float *)malloc((size_t)HK * len * hd * 4);
    int rc = fo_embed_rows(c->type_embd, m->embd, c->vocab, D, tokens, s, x);
    if (rc) goto done;
    for (int l = 0; l < c->n_layers; l++) {
        fo_llama_layer *y = &m->layers[l];
        /* residual = x; x = attention_norm(x)                      raw/mod.rs:961-964 */
        fo_rms_norm(x, NULL, y->attn_norm, NULL, c->eps, s, D, xn);
        fo_q_mat_mul_fast(y->tq, xn, s, D, y->wq, H * hd, q, L, nt);
        fo_q_mat_mul_fast(y->tk, xn, s, D, y->wk, HK * hd, k, L, nt);
        fo_q_mat_mul_fast(y->tv, xn, s, D, y->wv, HK * hd, v, L, nt);
        to_heads(q, s, H, hd, qh);      /* reshape + transpose(1,2), attention_layer.rs:371-374 */
        to_heads(k, s, HK, hd, kh);
        to_heads(v, s, HK, hd, vh);
        fo_rope(qh, 1, H, s, hd, m->cosv, m->sinv, pos, 1, qr);
        fo_rope(kh, 1, HK, s, hd, m->cosv, m->sinv, pos, 1, kr);
        for (int i = 0; i < HK; i++) {  /* KvCache::append, fusor/src/cache/kv_cache.rs:49-63 */
            memcpy(m->kc[l] + ((size_t)i * c->ctx + pos) * hd, kr + (size_t)i * s * hd, (size_t)s * hd * 4);
            memcpy(m->vc[l] + ((size_t)i * c->ctx + pos) * hd, vh + (size_t)i * s * hd, (size_t)s * hd * 4);
            memcpy(kall + (size_t)i * len * hd, m->kc[l] + (size_t)i * c->ctx * hd, (size_t)len * hd * 4);
            memcpy(vall + (size_t)i * len * hd, m->vc[l] + (size_t)i * c->ctx * hd, (size_t)len * hd * 4);
        }
        /* mask only when seq_len > 1 (raw/mod.rs:969-972) */
        fo_flash_attention(qr, kall, vall, 1, H, HK, s, len, hd, (float)(1.0 / sqrt((double)hd)),
                           s > 1 ? 1 : 0, NULL, ao, nt);
        from_heads(ao, s, H, hd, ao2);  /* transpose(1,2) + reshape, attention_layer.rs:689-691 */
        fo_q_mat_mul_fast(y->to, ao2, s, H * hd, y->wo, D, att, L, nt);
        /* x2 = ffn_norm(att + residual)                            raw/mod.rs:1017 */
        fo_rms_norm(att, x, y->ffn_norm, NULL, c->eps, s, D, xn);
        fo_q_mat_mul_fast(y->tgate, xn, s, D, y->gate, F, g, L, nt);
        fo_q_mat_mul_fast(y->tup, xn, s, D, y->up, F, u, L, nt);
        fo_swiglu(g, u, act, (size_t)s * F);
        fo_q_mat_mul_fast(y->tdown, act, s, F, y->down, D, ff, L, nt);
        fo_add3(ff, att, x, x, sd);     /* (ffn + attn) + residual, raw/mod.rs:1036 */
    }
    fo_rms_norm(x + (size_t)(s - 1) * D, NULL, m->out_norm, NULL, c->eps, 1, D, xn);
    if (hidden_out) memcpy(hidden_out, xn, (size_t)D * 4);
    if (logits) fo_q_mat_mul_fast(c->type_output, xn, 1, D, m->output, c->vocab, logits, L, nt);
    m->len = len;
done:
    free(x); free(xn); free(att); free(q); free(qh); free(qr); free(k); free(kh); free(kr);
    free(v); free(vh); free(ao); free(ao2); free(g); free(u); free(act); free(ff);
    free(kall); free(vall);
    return rc;
}

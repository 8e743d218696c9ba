// Q8_0 weights x Q8_0-quantised activations on the integer matrix cores.
// Reference: fusor-ml/gguf/src/lib.rs:1150-1230 (BlockQ8_0::quantize: per-32 scale amax / 127 stored as f16, codes
// round(x * 127 / amax)), :1315-1358 (vec_dot: exact i32 sum of the 32 code products, times d_w * d_a), accumulated
// over the blocks of a row in k order in f32 (the Q8-activation matmul of fusor-ml/cpu/src/quantized.rs).
//
// One v_mfma_i32_32x32x32_i8 is exactly one 32-element block of 32 weight rows against 32 activation rows: the
// integer block sums are exact (the reference fixes nothing else: the order in which the f32 block terms are scaled
// and added is the caller's).  A block term is added as  acc = fma(f32(isum) * d_a, d_w, acc):  three vector
// operations per accumulator element and block (convert, multiply, fused multiply-add) with the MFMA result in
// vector registers, where  acc + f32(isum) * (d_w * d_a)  with separate roundings took five (accumulator-register
// read, convert, two multiplies, add).
// Workgroup: 128 weight rows x 128 activation rows, 4 wavefronts of 64 x 64 (2 x 2 MFMA tiles), two blocks (one
// device record) per barrier round through LDS.  The kernel is bound by the per-block scaling (48 vector
// instructions per MFMA, i.e. 192 cycles against the 32 of the MFMA), not by the matrix cores.
#include "fh_blocks.h"

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));

// Activation quantisation into the layout the kernel reads: codes [m][k] (a block = 32 aligned bytes) and the
// f16-rounded block scales as f32 [m][k / 32].  Same arithmetic as k_q8_0_quantize.
__global__ void k_q8_split_quantize(const float *__restrict__ x, int64_t nblocks, int8_t *__restrict__ codes,
                                    float *__restrict__ scales) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *v = x + b * 32;
    float amax = 0.f;
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    const float scale = amax / 127.0f;
    const float inv = amax != 0.f ? 127.0f / amax : 0.f;
    scales[b] = (float)(_Float16)scale;
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t u = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float r = rintf(v[4 * i + e] * inv);
            r = fminf(127.f, fmaxf(-128.f, r));
            u |= (uint32_t)(uint8_t)(int8_t)(int)r << (8 * e);
        }
        w[i] = u;
    }
    uint4 *o = (uint4 *)(codes + b * 32);
    o[0] = make_uint4(w[0], w[1], w[2], w[3]);
    o[1] = make_uint4(w[4], w[5], w[6], w[7]);
}

#define Q8M_ROW 80 // LDS bytes per row and round: 2 blocks x 32 codes + 16 padding

// (at least two wavefronts per SIMD: with at most 256 registers per lane the MFMA results stay in vector registers)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_qmm_q8_mfma(QView q, const int8_t *__restrict__ xc, const float *__restrict__ xs,
                                                      int m, float *__restrict__ y) {
    __shared__ __attribute__((aligned(16))) uint8_t sA[128 * Q8M_ROW], sB[128 * Q8M_ROW];
    __shared__ __attribute__((aligned(16))) float sAs[2][128], sBs[2][128];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
    const int wn = wave >> 1, wm = wave & 1;
    const int64_t n0 = (int64_t)blockIdx.x * 128;
    const int m0 = blockIdx.y * 128;
    const int kb = (int)q.kb, rounds = (kb + 1) / 2;
    const int64_t K = q.k, tiles16 = (q.n + 15) / 16;
    float acc[2][2][16];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    for (int rr = 0; rr < rounds; rr++) {
        __syncthreads(); // the previous round is consumed
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int item = tid + 256 * i, row = item >> 2, blk = (item >> 1) & 1, half = item & 1;
            // weights: record rr of the row's 16-row tile holds blocks 2 rr and 2 rr + 1 (k padded with zero blocks)
            int64_t t16 = (n0 + row) >> 4;
            if (t16 >= tiles16) t16 = tiles16 - 1; // rows past the end read a valid tile and are never stored
            const int j = row & 15;
            const uint8_t *rec = q.data + (t16 * q.recs + rr) * 1088;
            const uint2 p0 = *(const uint2 *)(rec + ((2 * half) * 16 + j) * 16 + 8 * blk);
            const uint2 p1 = *(const uint2 *)(rec + ((2 * half + 1) * 16 + j) * 16 + 8 * blk);
            *(uint4 *)(sA + row * Q8M_ROW + blk * 32 + half * 16) = make_uint4(p0.x, p0.y, p1.x, p1.y);
            if (half == 0) sAs[blk][row] = fh_h2f(fh_ld16(rec + 1024 + 4 * j + 2 * blk));
            // activations
            const int mm = m0 + row, b = 2 * rr + blk;
            uint4 c = make_uint4(0, 0, 0, 0);
            float s = 0.f;
            if (mm < m && b < kb) {
                c = *(const uint4 *)(xc + (int64_t)mm * K + (int64_t)b * 32 + 16 * half);
                s = xs[(int64_t)mm * kb + b];
            }
            *(uint4 *)(sB + row * Q8M_ROW + blk * 32 + half * 16) = c;
            if (half == 0) sBs[blk][row] = s;
        }
        __syncthreads();
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            intx4 av[2], bv[2];
            float dx[2];
#pragma unroll
            for (int f = 0; f < 2; f++) {
                av[f] = *(const intx4 *)(sA + (wn * 64 + f * 32 + li) * Q8M_ROW + blk * 32 + 16 * g);
                bv[f] = *(const intx4 *)(sB + (wm * 64 + f * 32 + li) * Q8M_ROW + blk * 32 + 16 * g);
                dx[f] = sBs[blk][wm * 64 + f * 32 + li];
            }
#pragma unroll
            for (int fn = 0; fn < 2; fn++) {
                float dw[16]; // scales of the lane's 16 weight rows: n = 8 (r / 4) + 4 g + r % 4
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    const float4 t = *(const float4 *)(&sAs[blk][wn * 64 + fn * 32 + 8 * r4 + 4 * g]);
                    dw[4 * r4] = t.x; dw[4 * r4 + 1] = t.y; dw[4 * r4 + 2] = t.z; dw[4 * r4 + 3] = t.w;
                }
#pragma unroll
                for (int fm = 0; fm < 2; fm++) {
                    intx16 d;
#pragma unroll
                    for (int r = 0; r < 16; r++) d[r] = 0;
                    d = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[fn], bv[fm], d, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[fn][fm][r] = fmaf((float)d[r] * dx[fm], dw[r], acc[fn][fm][r]);
                }
            }
        }
    }
    const bool vec = (q.n & 3) == 0;
#pragma unroll
    for (int fm = 0; fm < 2; fm++) {
        const int mm = m0 + wm * 64 + fm * 32 + li;
        if (mm >= m) continue;
#pragma unroll
        for (int fn = 0; fn < 2; fn++) {
            const int64_t nb = n0 + wn * 64 + fn * 32 + 4 * g;
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const int64_t nn = nb + 8 * r4;
                const float *a = &acc[fn][fm][4 * r4];
                float *dst = y + (int64_t)mm * q.n + nn;
                if (vec && nn + 3 < q.n) {
                    *(float4 *)dst = make_float4(a[0], a[1], a[2], a[3]);
                } else {
                    if (nn < q.n) dst[0] = a[0];
                    if (nn + 1 < q.n) dst[1] = a[1];
                    if (nn + 2 < q.n) dst[2] = a[2];
                    if (nn + 3 < q.n) dst[3] = a[3];
                }
            }
        }
    }
}

fh_status fh_launch_qmm_q8_mfma(const fh_qmatrix *q, const float *x, int m, float *y) {
    fh_device *dev = q->dev;
    FH_REQUIRE(q->type == FH_Q8_0, "Q8_0 weights expected");
    FH_REQUIRE((m + 127) / 128 <= 65535, "m = %d too large for one launch", m);
    const int64_t nb = (int64_t)m * q->kb;
    const size_t codes = ((size_t)m * q->k + 255) & ~(size_t)255;
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, codes + (size_t)nb * 4));
    int8_t *xc = (int8_t *)dev->act_buf;
    float *xs = (float *)((uint8_t *)dev->act_buf + codes);
    k_q8_split_quantize<<<dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, dev->stream>>>(x, nb, xc, xs);
    FH_HIP(hipGetLastError());
    dim3 grid((unsigned)((q->n + 127) / 128), (unsigned)((m + 127) / 128));
    k_qmm_q8_mfma<<<grid, 256, 0, dev->stream>>>(fh_view(q), xc, xs, m, y);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// Prefill-side quantized matmul (m > 16 activation rows), the bf16-activation form, and the
// Q8_0 x Q8 integer variant.
// Reference: fusor-ml/cpu/src/quantized.rs:246-675 (f32 product),
// fusor-ml/gguf/src/lib.rs:1150-1230 (BlockQ8_0::quantize), :1315-1358 (vec_dot).
#include "fh_blocks.h"

extern "C" fh_status fh_qmatmul_bf16(const fh_qmatrix *q, const uint16_t *x_bf16_dev, int32_t m, float *y_dev) {
    FH_REQUIRE(q && x_bf16_dev && y_dev, "NULL argument");
    FH_REQUIRE(m >= 1, "m = %d", m);
    return fh_launch_qmatmul_tile(q, x_bf16_dev, 1, m, y_dev);
}

// ------------------------------------------------------------------------------ Q8_0 activations
// One thread per 32-block: amax, scale = amax / 127 stored as f16, q = rint(x * (127 / amax))
// (round half to even, the result of _mm256_cvtps_epi32 in quantize_avx2), saturated to [-128, 127].
__global__ void k_q8_0_quantize(const float *__restrict__ x, int64_t nblocks, uint8_t *__restrict__ out) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *v = x + b * 32;
    float amax = 0.f;
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
    float scale = amax / 127.0f;
    float inv = amax != 0.f ? 127.0f / amax : 0.f;
    uint8_t *o = out + b * 34;
    _Float16 h = (_Float16)scale;
    uint16_t hb;
    __builtin_memcpy(&hb, &h, 2);
    o[0] = (uint8_t)(hb & 0xFF);
    o[1] = (uint8_t)(hb >> 8);
    for (int i = 0; i < 32; i++) {
        float r = rintf(v[i] * inv);
        r = fminf(127.f, fmaxf(-128.f, r));
        o[2 + i] = (uint8_t)(int8_t)(int)r;
    }
}

extern "C" fh_status fh_q8_0_quantize(fh_device *dev, const float *x_dev, int64_t count, void *out_dev) {
    FH_REQUIRE(dev && x_dev && out_dev, "NULL argument");
    FH_REQUIRE(count > 0 && count % 32 == 0, "count %lld is not a positive multiple of 32", (long long)count);
    int64_t nb = count / 32;
    k_q8_0_quantize<<<dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, dev->stream>>>(x_dev, nb, (uint8_t *)out_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// y[r, c] = sum_b (sum_i w_q * a_q) as f32 * (d_w * d_a); one thread per output, blocks in k order.
template <int T>
__global__ void k_qmm_q8(QView q, const uint8_t *__restrict__ aq, int m, float *__restrict__ y,
                         int32_t *__restrict__ isums) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)m * q.n) return;
    int r = (int)(idx / q.n);
    int64_t c = idx % q.n;
    int kb = (int)q.kb;
    int j = (int)(c & 15);
    float acc = 0.f;
    for (int b = 0; b < kb; b++) {
        const uint8_t *ab = aq + ((int64_t)r * kb + b) * 34;
        float da = fh_h2f((uint16_t)(ab[0] | (ab[1] << 8)));
        int32_t s = 0;
        float dw;
        if (T == FH_Q8_0) {
            const uint8_t *rec = q.data + ((c >> 4) * q.recs + (b >> 1)) * (int64_t)q.rec_bytes;
            int u = b & 1;
            dw = fh_h2f(fh_ld16(rec + q80_d_off(j, u)));
            for (int i = 0; i < 32; i++) s += (int)(int8_t)rec[q80_q_off(j, u, i)] * (int)(int8_t)ab[2 + i];
        } else {
            const uint8_t *rec = q.data + ((c >> 4) * q.recs + (b >> 2)) * (int64_t)q.rec_bytes;
            int u = b & 3;
            dw = fh_h2f(fh_ld16(rec + q40_d_off(j, u)));
            for (int i = 0; i < 16; i++) {
                uint8_t byte = rec[q40_q_off(j, u, i)];
                s += ((int)(byte & 0x0F) - 8) * (int)(int8_t)ab[2 + i];
                s += ((int)(byte >> 4) - 8) * (int)(int8_t)ab[2 + i + 16];
            }
        }
        if (isums) isums[idx * kb + b] = s;
        float scale = dw * da;
        float term = (float)s * scale;
        acc = acc + term;
    }
    y[idx] = acc;
}

extern "C" fh_status fh_qmatmul_q8(const fh_qmatrix *q, const float *x_dev, int32_t m, float *y_dev,
                                   int32_t *isums_dev) {
    FH_REQUIRE(q && x_dev && y_dev, "NULL argument");
    FH_REQUIRE(m >= 1, "m = %d", m);
    if (q->type != FH_Q8_0 && q->type != FH_Q4_0)
        FH_FAIL(FH_ERR_UNSUPPORTED, "the Q8 activation path exists for Q8_0 and Q4_0 weights only (type %u)", q->type);
    fh_device *dev = q->dev;
    // Q8_0 weights without a request for the integer block sums: the integer matrix-core kernel
    if (q->type == FH_Q8_0 && !isums_dev && dev->opt_matmul_kernel != 1) return fh_launch_qmm_q8_mfma(q, x_dev, m, y_dev);
    int64_t nb = (int64_t)m * q->kb;
    FH_TRY(fh_dev_scratch(dev, &dev->act_buf, &dev->act_cap, (size_t)nb * 34 + 64));
    k_q8_0_quantize<<<dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, dev->stream>>>(x_dev, nb, (uint8_t *)dev->act_buf);
    FH_HIP(hipGetLastError());
    int64_t total = (int64_t)m * q->n;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    QView v = fh_view(q);
    if (q->type == FH_Q8_0)
        k_qmm_q8<FH_Q8_0><<<grid, block, 0, dev->stream>>>(v, (const uint8_t *)dev->act_buf, m, y_dev, isums_dev);
    else
        k_qmm_q8<FH_Q4_0><<<grid, block, 0, dev->stream>>>(v, (const uint8_t *)dev->act_buf, m, y_dev, isums_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

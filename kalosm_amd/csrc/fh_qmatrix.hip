// QMatrix: ingest of raw GGUF block streams into the tiled device layouts, bit-exact
// dequantisation, embedding row gather and row concatenation.
// Reference: fusor-ml/fusor/src/quantized.rs:80-279, fusor-ml/fusor/src/layers/embedding.rs:43-89.
#include "fh_blocks.h"

// ------------------------------------------------------------------------------ repack
// One thread per (row, source block).  The source is the GGUF stream ([n][kb] blocks); the
// destination is the tile record.  Upload-time only.
__global__ void k_repack_q4_k(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 144;
    uint8_t *rec = dst + ((row >> 4) * recs + b) * 2304;
    int j = (int)(row & 15);
    for (int i = 0; i < 16; i++) rec[q4k_hdr_off(j) + i] = s[i];
    for (int i = 0; i < 128; i++) rec[q4k_qs_off(j, i)] = s[16 + i];
}
__global__ void k_repack_q6_k(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 210;
    uint8_t *rec = dst + ((row >> 4) * recs + b) * 3360;
    int j = (int)(row & 15);
    // 6-bit codes in dequantised element order (fusor-ml/gguf/src/lib.rs:2034-2085), then re-packed
    for (int t = 0; t < 8; t++)
        for (int g = 0; g < 4; g++) {
            uint32_t lw = 0, hbits = 0;
            for (int vv = 0; vv < 8; vv++) {
                int e = 32 * t + 8 * g + vv;
                int n = e >> 7, jj = (e >> 5) & 3, l = e & 31;
                uint8_t lo = s[64 * n + l + ((jj & 1) ? 32 : 0)];
                uint8_t hi = s[128 + 32 * n + l];
                uint32_t nib = (jj & 2) ? (lo >> 4) : (lo & 0x0F);
                uint32_t hb = (hi >> (2 * jj)) & 3u;
                int p = vv >> 1, odd = vv & 1;
                lw |= nib << (4 * (p + 4 * odd));
                hbits |= hb << (q6k_hbit(t, p) + 16 * odd);
            }
            *(uint32_t *)(rec + q6k_lword_off(j, t, g)) = lw;
            uint32_t *hw = (uint32_t *)(rec + q6k_hword_off(j, t, g));
            if (t & 1) *hw |= hbits; // steps 2u and 2u+1 share a word; this thread owns the whole word
            else *hw = hbits;
        }
    for (int G = 0; G < 16; G++) rec[q6k_sc_off(j, G)] = s[192 + G];
    rec[q6k_d_off(j)] = s[208];
    rec[q6k_d_off(j) + 1] = s[209];
}
__global__ void k_repack_q8_0(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 34;
    uint8_t *rec = dst + ((row >> 4) * recs + (b >> 1)) * 1088;
    int j = (int)(row & 15), u = (int)(b & 1);
    rec[q80_d_off(j, u)] = s[0];
    rec[q80_d_off(j, u) + 1] = s[1];
    for (int i = 0; i < 32; i++) rec[q80_q_off(j, u, i)] = s[2 + i];
}
__global__ void k_repack_q4_0(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 18;
    uint8_t *rec = dst + ((row >> 4) * recs + (b >> 2)) * 1152;
    int j = (int)(row & 15), u = (int)(b & 3);
    rec[q40_d_off(j, u)] = s[0];
    rec[q40_d_off(j, u) + 1] = s[1];
    for (int i = 0; i < 16; i++) rec[q40_q_off(j, u, i)] = s[2 + i];
}

__global__ void k_repack_q5_k(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 176; // d, dmin, 12 scale bytes | qh[32] | qs[128]
    uint8_t *rec = dst + ((row >> 4) * recs + b) * 2816;
    int j = (int)(row & 15);
    for (int i = 0; i < 16; i++) rec[q4k_hdr_off(j) + i] = s[i];
    for (int i = 0; i < 32; i++) rec[q5k_qh_off(j, i)] = s[16 + i];
    for (int i = 0; i < 128; i++) rec[q4k_qs_off(j, i)] = s[48 + i];
}
__global__ void k_repack_q5_0(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n, int64_t kb,
                              int64_t recs) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n * kb) return;
    int64_t row = idx / kb, b = idx % kb;
    const uint8_t *s = src + idx * 22; // f16 d | 32 high bits | qs[16]
    uint8_t *rec = dst + ((row >> 4) * recs + (b >> 2)) * 1408;
    int j = (int)(row & 15), u = (int)(b & 3);
    rec[q40_d_off(j, u)] = s[0];
    rec[q40_d_off(j, u) + 1] = s[1];
    const uint32_t qh = (uint32_t)s[2] | ((uint32_t)s[3] << 8) | ((uint32_t)s[4] << 16) | ((uint32_t)s[5] << 24);
    for (int g = 0; g < 4; g++)
        rec[q50_qh_off(j, u, g)] = (uint8_t)(((qh >> (4 * g)) & 0xFu) | (((qh >> (16 + 4 * g)) & 0xFu) << 4));
    for (int i = 0; i < 16; i++) rec[q40_q_off(j, u, i)] = s[6 + i];
}

static fh_status qm_alloc(fh_device *dev, uint32_t type, int64_t n, int64_t k, fh_qmatrix **out) {
    int e = fh_block_elems(type);
    if (!e)
        FH_FAIL(FH_ERR_UNSUPPORTED, "unsupported ggml type %u (supported: F32=0, F16=1, Q4_0=2, Q5_0=6, Q8_0=8, Q4_K=12, "
                                    "Q5_K=13, Q6_K=14)", type);
    FH_REQUIRE(n > 0 && k > 0, "empty weight [%lld, %lld]", (long long)n, (long long)k);
    FH_REQUIRE(k % e == 0, "k=%lld is not a multiple of the block size %d", (long long)k, e);
    FH_REQUIRE(n < (1ll << 31) && k < (1ll << 31), "weight too large");
    fh_qmatrix *q = new fh_qmatrix();
    q->dev = dev;
    q->type = type;
    q->n = n;
    q->k = k;
    q->n_pad = (n + 15) / 16 * 16;
    q->kb = k / e;
    int rb = fh_rec_blocks(type);
    q->recs = (q->kb + rb - 1) / rb;
    q->rec_bytes = fh_rec_bytes(type);
    q->bytes = (size_t)(q->n_pad / 16) * (size_t)q->recs * (size_t)q->rec_bytes;
    if (fh_is_plain(type)) { // the file's own layout: rows of kb blocks
        q->recs = 0;
        q->rec_bytes = fh_block_bytes(type);
        q->bytes = (size_t)n * (size_t)q->kb * (size_t)fh_block_bytes(type);
    }
    hipError_t err = hipMalloc((void **)&q->data, q->bytes + 256); // slack: kernels may prefetch one record ahead
    if (err != hipSuccess) {
        delete q;
        FH_FAIL(err == hipErrorOutOfMemory ? FH_ERR_OOM : FH_ERR_HIP, "hipMalloc(%zu) failed: %s", q->bytes,
                hipGetErrorString(err));
    }
    *out = q;
    return FH_OK;
}

extern "C" fh_status fh_qmatrix_from_gguf_bytes(fh_device *dev, uint32_t ggml_type, int64_t n, int64_t k,
                                                const void *bytes, size_t len, fh_qmatrix **out) {
    FH_REQUIRE(dev && bytes && out, "NULL argument");
    *out = nullptr;
    FH_HIP(hipSetDevice(dev->ordinal));
    fh_qmatrix *q = nullptr;
    FH_TRY(qm_alloc(dev, ggml_type, n, k, &q));
    size_t want = (size_t)n * (size_t)q->kb * (size_t)fh_block_bytes(ggml_type);
    if (len != want) {
        fh_qmatrix_free(q);
        FH_FAIL(FH_ERR_INVALID, "byte length %zu does not match [%lld, %lld] of type %u (%zu expected)", len,
                (long long)n, (long long)k, ggml_type, want);
    }
    if (fh_is_plain(ggml_type)) {
        hipError_t e = hipMemcpyAsync(q->data, bytes, len, hipMemcpyHostToDevice, dev->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(dev->stream);
        if (e != hipSuccess) {
            fh_qmatrix_free(q);
            FH_FAIL(FH_ERR_HIP, "upload of a [%lld, %lld] type-%u weight failed: %s", (long long)n, (long long)k, ggml_type,
                    hipGetErrorString(e));
        }
        if (ggml_type == FH_W_F32) { // for the matrix-core path of dense f32 rows
            fh_status ws = fh_dense_wscale(dev, (const float *)q->data, n * k, &q->wscale);
            if (ws != FH_OK) {
                fh_qmatrix_free(q);
                return ws;
            }
        }
        *out = q;
        return FH_OK;
    }
    uint8_t *staging = nullptr;
    hipError_t err = hipMalloc((void **)&staging, len);
    if (err != hipSuccess) {
        fh_qmatrix_free(q);
        FH_FAIL(FH_ERR_OOM, "hipMalloc(%zu) for staging failed: %s", len, hipGetErrorString(err));
    }
    fh_status st = FH_OK;
    do {
        if (hipMemsetAsync(q->data, 0, q->bytes + 256, dev->stream) != hipSuccess) { st = FH_ERR_HIP; break; }
        if (hipMemcpyAsync(staging, bytes, len, hipMemcpyHostToDevice, dev->stream) != hipSuccess) { st = FH_ERR_HIP; break; }
        int64_t total = n * q->kb;
        dim3 grid((unsigned)((total + 255) / 256)), block(256);
        switch (ggml_type) {
        case FH_Q4_K: k_repack_q4_k<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        case FH_Q6_K: k_repack_q6_k<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        case FH_Q8_0: k_repack_q8_0<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        case FH_Q4_0: k_repack_q4_0<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        case FH_Q5_K: k_repack_q5_k<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        case FH_Q5_0: k_repack_q5_0<<<grid, block, 0, dev->stream>>>(staging, q->data, n, q->kb, q->recs); break;
        }
        if (hipGetLastError() != hipSuccess) { st = FH_ERR_HIP; break; }
        if (hipStreamSynchronize(dev->stream) != hipSuccess) { st = FH_ERR_HIP; break; }
    } while (0);
    (void)hipFree(staging);
    if (st != FH_OK) {
        fh_qmatrix_free(q);
        FH_FAIL(st, "upload/repack of a [%lld, %lld] type-%u weight failed", (long long)n, (long long)k, ggml_type);
    }
    *out = q;
    return FH_OK;
}

extern "C" fh_status fh_qmatrix_free(fh_qmatrix *q) {
    if (!q) return FH_OK;
    if (q->data) {
        (void)hipStreamSynchronize(q->dev->stream);
        (void)hipFree(q->data);
    }
    delete q;
    return FH_OK;
}

extern "C" fh_status fh_qmatrix_info(const fh_qmatrix *q, uint32_t *ggml_type, int64_t *n, int64_t *k,
                                     uint64_t *device_bytes) {
    FH_REQUIRE(q, "q is NULL");
    if (ggml_type) *ggml_type = q->type;
    if (n) *n = q->n;
    if (k) *k = q->k;
    if (device_bytes) *device_bytes = q->bytes;
    return FH_OK;
}

// Row concatenation works tile-wise, so every part but the last must hold a multiple of 16 rows.
extern "C" fh_status fh_qmatrix_concat_rows(fh_device *dev, const fh_qmatrix *const *parts, int32_t count,
                                            fh_qmatrix **out) {
    FH_REQUIRE(dev && parts && out && count > 0, "bad argument");
    *out = nullptr;
    int64_t n = 0;
    for (int i = 0; i < count; i++) {
        FH_REQUIRE(parts[i], "part %d is NULL", i);
        // Option::None in the reference (fusor-ml/core/src/quantized/mod.rs:329-337)
        if (parts[i]->type != parts[0]->type || parts[i]->k != parts[0]->k)
            FH_FAIL(FH_ERR_UNSUPPORTED, "concat_rows needs one type and one k (part %d differs)", i);
        if (i + 1 < count && parts[i]->n % 16 != 0 && !fh_is_plain(parts[0]->type))
            FH_FAIL(FH_ERR_UNSUPPORTED, "concat_rows: part %d has %lld rows, not a multiple of 16", i,
                    (long long)parts[i]->n);
        n += parts[i]->n;
    }
    fh_qmatrix *q = nullptr;
    FH_TRY(qm_alloc(dev, parts[0]->type, n, parts[0]->k, &q));
    size_t off = 0;
    for (int i = 0; i < count; i++) {
        hipError_t e = hipMemcpyAsync(q->data + off, parts[i]->data, parts[i]->bytes, hipMemcpyDeviceToDevice, dev->stream);
        if (e != hipSuccess) {
            fh_qmatrix_free(q);
            FH_FAIL(FH_ERR_HIP, "hipMemcpyAsync failed: %s", hipGetErrorString(e));
        }
        off += parts[i]->bytes;
        if (i == 0 || parts[i]->wscale < q->wscale) q->wscale = parts[i]->wscale; // the largest |w| decides
    }
    *out = q;
    return FH_OK;
}

// ------------------------------------------------------------------------------ dequantize
template <int T>
__global__ void k_dequantize(QView q, float *__restrict__ out) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = q.n * q.k;
    if (idx >= total) return;
    int64_t row = idx / q.k, k = idx % q.k;
    out[idx] = deq_elem<T>(q, row, k);
}

extern "C" fh_status fh_qmatrix_dequantize(const fh_qmatrix *q, float *out_dev) {
    FH_REQUIRE(q && out_dev, "NULL argument");
    int64_t total = q->n * q->k;
    FH_REQUIRE((total + 255) / 256 < (1ll << 31), "weight too large for one launch");
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    QView v = fh_view(q);
    hipStream_t s = q->dev->stream;
    switch (q->type) {
    case FH_Q4_0: k_dequantize<FH_Q4_0><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_Q8_0: k_dequantize<FH_Q8_0><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_Q4_K: k_dequantize<FH_Q4_K><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_Q6_K: k_dequantize<FH_Q6_K><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_Q5_0: k_dequantize<FH_Q5_0><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_Q5_K: k_dequantize<FH_Q5_K><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_W_F32: k_dequantize<FH_W_F32><<<grid, block, 0, s>>>(v, out_dev); break;
    case FH_W_F16: k_dequantize<FH_W_F16><<<grid, block, 0, s>>>(v, out_dev); break;
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

// ------------------------------------------------------------------------------ embedding
template <int T>
__global__ void k_embed_rows(QView q, const uint32_t *__restrict__ ids, int count, float *__restrict__ out) {
    int t = blockIdx.y;
    int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= count || k >= q.k) return;
    uint32_t id = ids[t];
    // an id outside the table cannot be reported from here; it reads row 0 of the padding-free
    // range instead of faulting, and the host-side check is the defined error path
    int64_t row = id < (uint32_t)q.n ? (int64_t)id : 0;
    out[(int64_t)t * q.k + k] = deq_elem<T>(q, row, k);
}

extern "C" fh_status fh_embed_rows(const fh_qmatrix *q, const uint32_t *ids_dev, const uint32_t *ids_host,
                                   int32_t count, float *out_dev) {
    FH_REQUIRE(q && ids_dev && out_dev, "NULL argument");
    FH_REQUIRE(count > 0 && count <= 65535, "count %d out of range", count);
    if (ids_host)
        for (int i = 0; i < count; i++)
            FH_REQUIRE((int64_t)ids_host[i] < q->n, "token id %u at %d is outside the table of %lld rows", ids_host[i],
                       i, (long long)q->n);
    dim3 grid((unsigned)((q->k + 255) / 256), (unsigned)count), block(256);
    QView v = fh_view(q);
    hipStream_t s = q->dev->stream;
    switch (q->type) {
    case FH_Q4_0: k_embed_rows<FH_Q4_0><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_Q8_0: k_embed_rows<FH_Q8_0><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_Q4_K: k_embed_rows<FH_Q4_K><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_Q6_K: k_embed_rows<FH_Q6_K><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_Q5_0: k_embed_rows<FH_Q5_0><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_Q5_K: k_embed_rows<FH_Q5_K><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_W_F32: k_embed_rows<FH_W_F32><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    case FH_W_F16: k_embed_rows<FH_W_F16><<<grid, block, 0, s>>>(v, ids_dev, count, out_dev); break;
    }
    FH_HIP(hipGetLastError());
    return FH_OK;
}

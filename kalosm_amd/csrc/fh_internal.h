// Internal declarations shared by the translation units of libfusor_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <string>
#include <utility>
#include <vector>

#include "../../include/fusor_hip.h"

// ---------------------------------------------------------------- errors
void fh_set_error(const char *fmt, ...);
#define FH_FAIL(code, ...)            \
    do {                              \
        fh_set_error(__VA_ARGS__);    \
        return (code);                \
    } while (0)
#define FH_REQUIRE(cond, ...)                         \
    do {                                              \
        if (!(cond)) FH_FAIL(FH_ERR_INVALID, __VA_ARGS__); \
    } while (0)
#define FH_HIP(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            fh_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return e_ == hipErrorOutOfMemory ? FH_ERR_OOM : FH_ERR_HIP;                       \
        }                                                                                     \
    } while (0)
#define FH_TRY(call)                  \
    do {                              \
        fh_status s_ = (call);        \
        if (s_ != FH_OK) return s_;   \
    } while (0)

// ---------------------------------------------------------------- device
struct fh_device {
    int ordinal = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int compute_units = 0;
    bool capturing = false;          // between fh_graph_begin and fh_graph_end
    // activation staging for the MFMA decode kernels (grown on demand)
    void *act_buf = nullptr;
    size_t act_cap = 0;
    // split-K partial sums
    float *part_buf = nullptr;
    size_t part_cap = 0;
    float *ksplit_buf = nullptr; // partial planes of a k-split prefill matmul
    size_t ksplit_cap = 0;
    // 64 KB that never moves: partial results of small reductions (argmax)
    void *small_buf = nullptr;
    // Counts the reallocations of act_buf / part_buf / ksplit_buf.  A captured graph holds their addresses as
    // kernel arguments, so whoever keeps a graph records the value at capture and must not replay it after
    // the value has changed.
    uint64_t scratch_gen = 0;
    // this GPU's copy of the library's file-scope scratch array (fh_attention_decode.hip), for the entry point that
    // must not allocate
    void *static_scratch = nullptr;
    size_t static_scratch_bytes = 0;
    // kernels whose dynamic LDS limit was raised on this device, with the limit (fh_kernel_lds)
    std::vector<std::pair<const void *, size_t>> lds_raised;
    // options (fh_set_option)
    int64_t opt_matvec_kernel = 0;   // 0 auto, 1 generic VALU, 2 MFMA, 3 first-generation Q4_K MFMA, 4 batch MFMA
    int64_t opt_matvec_splitk = 0;   // 0 auto, else forced split count
    int64_t opt_matvec_waves = 0;    // 0 auto
    int64_t opt_matvec_tiles = 0;    // 0 auto, else 1 / 2 / 4 row tiles per workgroup
    int64_t opt_matvec_per = 0;      // 0 auto, else 1 / 2 / 4 blocks per wavefront
    int64_t opt_matvec_rowsplit = 0; // 0 auto, else 1 / 2 / 4 workgroups per row tile of the single-row Q4_K kernel
    int64_t opt_attn_splits = 0;     // 0 auto
    int64_t opt_attn_kernel = 0;     // 0 auto, 1 first-generation kernels only, 2 matrix-core prefill for f32 too
    int64_t opt_down_splitk = 0;     // 0: decode steps split k of a Q6_K down projection (atomic adds), 1: never, 3: and SwiGLU in its staging
    int64_t opt_down_tiles = 0;      // row tiles per wavefront of the accumulating Q6_K down projection (0: 1; 1, 2, 4)
    int64_t opt_attn_heads = 0;      // query heads per workgroup of the decode attention (0: automatic; 1, 2, 4, 8)
    int64_t opt_attn_waves = 0;      // wavefronts per workgroup of the decode attention (0: 16; 8)
    int64_t opt_matvec_rows = 0;     // 1: 2 .. 4 activation rows never through the single-row Q4_K kernel's row variant
    int64_t opt_matvec_direct = 0; // 1: 5 .. 16 rows never through the unstaged kernel, 2: 2 .. 4 rows through it as well
    int64_t opt_wo_tiles = 0;        // row tiles per wavefront of the accumulating output projection (0: 4; 1, 2, 4)
    int64_t opt_wo_acc = 0;          // 0: decode steps accumulate the output projection into the residual stream, 1: never
    int64_t opt_fuse_norm = 0;       // 0: decode steps fold rms_norm into the consuming matvec, 1: separate launches
    int64_t opt_deterministic = 0;   // 1: decode steps never accumulate k-split partial sums with float atomics (run-to-run bit-equal)
    int64_t opt_trace_nan = 0;       // 1: fh_llama_forward probes the residual stream of every layer for NaN / inf
    int64_t opt_trace_timing = 0;    // 1: fh_llama_forward times its layer loop, 2: and every stage of every layer
    int64_t opt_trace_stderr = 0;    // 1: trace lines go to stderr as well as into the decoder's trace text
    uint64_t opt_gen = 0;            // bumped by every fh_set_option: captured decode steps are recorded again after a change
    int64_t opt_matmul_kernel = 0;   // 0 auto, 1 generic for every m, 2 MFMA tile kernels for every m, 3 / 4 and never / always the 128 x 256 one
};

fh_status fh_dev_scratch(fh_device *dev, void **buf, size_t *cap, size_t need);
// Allows the kernel `bytes` of dynamic LDS on this device (hipFuncSetAttribute, once per kernel and device).
fh_status fh_kernel_lds(fh_device *dev, const void *kernel, size_t bytes);
fh_status fh_static_scratch_init(fh_device *dev); // with dev->ordinal current

// ---------------------------------------------------------------- weights
// Device layouts.  All of them hold exactly the bits of the GGUF block stream,
// re-ordered so that a 64-lane wavefront reads them with 16-byte loads.
//
// Rows are grouped in tiles of 16 (the N extent of one MFMA); a matrix whose row
// count is not a multiple of 16 is padded with all-zero blocks.  kb = k / block
// elements.  For tile t and record r the record lives at
//   base + (t * records_per_tile + r) * record_bytes.
//
// FH_Q4_K (record = one 256-block of 16 rows, 2304 B)
//   [0,256)      header: row j at 16*j: d f16, dmin f16, 12 packed scale bytes (as in GGUF)
//   [256,2304)   quants: for p in {0,1}, lane l = g*16 + j (g in 0..3):
//                16 B at 256 + p*1024 + l*16 = qs_j[64p + 8g .. +8] ++ qs_j[64p + 32 + 8g .. +8]
// FH_Q6_K (record = one 256-block of 16 rows, 3360 B)
//   element e of row j belongs to MFMA step t = e/32, lane l = ((e/8)%4)*16 + j, value v = e%8
//   [0,2048)     low nibbles: lane l holds 16 B at (t/4)*1024 + l*16, one 32-bit word per step t%4; value v
//                sits in nibble v/2 + 4*(v%2), so (word >> 4p) & 0x000F000F is the f16 pair (v=2p, v=2p+1)
//   [2048,3072)  high 2 bits: lane l holds 16 B at 2048 + l*16, one word per step PAIR; bit positions chosen
//                so that one shift and one AND with 0x00300030 drop them onto bits 4-5 of the same pair
//   [3072,3328)  scales: lane l holds 4 x i8 at 3072 + l*4: groups 2g, 2g+1 of each half block (g = l/16)
//   [3328,3360)  d: row j at 3328 + 2*j (f16)
// FH_Q8_0 (record = two 32-blocks of 16 rows, 1088 B; kb padded to even with zero blocks)
//   [0,1024)     quants: lane l = g*16 + j: 16 B at l*16 = q_j[blk 2r][8g .. +8] ++ q_j[blk 2r+1][8g .. +8]
//   [1024,1088)  d: row j at 1024 + 4*j: d[blk 2r], d[blk 2r+1] (f16 x2)
// FH_Q4_0 (record = four 32-blocks of 16 rows, 1152 B; kb padded to a multiple of 4)
//   [0,1024)     quants: lane l = g*16 + j: 16 B at l*16 = for u in 0..3: qs_j[blk 4r+u][4g .. +4]
//   [1024,1152)  d: row j at 1024 + 8*j: d[blk 4r .. 4r+3] (f16 x4)
// FH_Q5_K (record = one 256-block of 16 rows, 2816 B): the FH_Q4_K record followed by
//   [2304,2816)  fifth bits: lane l = g*16 + j: 8 B at 2304 + l*8 = qh_j[8g .. +8] (bit s of byte e: element 8g+e of sub-block s)
// FH_Q5_0 (record = four 32-blocks of 16 rows, 1408 B): the FH_Q4_0 record followed by
//   [1152,1408)  fifth bits: lane l = g*16 + j: 4 B at 1152 + l*4, byte u for block 4r+u: bits 0-3 = qh bits 4g .. 4g+3
//                (elements of the low nibbles of the lane's four bytes), bits 4-7 = qh bits 16+4g .. 16+4g+3 (high nibbles)
struct fh_qmatrix {
    fh_device *dev = nullptr;
    uint32_t type = 0;
    int64_t n = 0, k = 0;
    int64_t n_pad = 0;       // rows padded to a multiple of 16
    int64_t kb = 0;          // blocks per row (unpadded)
    int64_t recs = 0;        // records per tile
    int rec_bytes = 0;
    uint8_t *data = nullptr; // device
    size_t bytes = 0;
    // dense f32 rows on the matrix cores: a power of two that brings the largest |w| into [2^14, 2^15), so that the
    // f16 pair hi + lo of w * wscale keeps 22 bits for every value that matters next to the largest one
    float wscale = 1.f;
};

// Weight types kept in the file's own row-major order (no tiled re-layout): dense f32 / f16 rows.
enum { FH_W_F32 = 0, FH_W_F16 = 1 };
static inline bool fh_is_plain(uint32_t t) { return t == FH_W_F32 || t == FH_W_F16; }
// Types without kernels for several activation rows (batch, row and tile kernels): those go row by row or element by
// element.  The 5-bit formats have the single-row matrix-core kernel only.
static inline bool fh_single_row_only(uint32_t t) { return fh_is_plain(t) || t == FH_Q5_0 || t == FH_Q5_K; }
static inline int fh_block_elems(uint32_t t) {
    switch (t) {
    case FH_W_F32: case FH_W_F16: return 1;
    case FH_Q4_0: case FH_Q8_0: case FH_Q5_0: return 32;
    case FH_Q4_K: case FH_Q6_K: case FH_Q5_K: return 256;
    default: return 0;
    }
}
static inline int fh_block_bytes(uint32_t t) { // gguf/src/lib.rs:109-121
    switch (t) {
    case FH_W_F32: return 4;
    case FH_W_F16: return 2;
    case FH_Q4_0: return 18;
    case FH_Q5_0: return 22;
    case FH_Q8_0: return 34;
    case FH_Q4_K: return 144;
    case FH_Q5_K: return 176;
    case FH_Q6_K: return 210;
    default: return 0;
    }
}
static inline int fh_rec_blocks(uint32_t t) {   // blocks per record (per row)
    switch (t) {
    case FH_Q4_0: case FH_Q5_0: return 4;
    case FH_Q8_0: return 2;
    default: return 1;
    }
}
static inline int fh_rec_bytes(uint32_t t) { return 16 * fh_rec_blocks(t) * fh_block_bytes(t); }

// A plain-data view passed to kernels by value.
struct QView {
    const uint8_t *data;
    int64_t n, k, kb, recs;
    int rec_bytes;
    float wscale = 1.f, winv = 1.f; // dense f32 rows: decode multiplies by wscale, the store by winv
};
static inline QView fh_view(const fh_qmatrix *q) {
    QView v{q->data, q->n, q->k, q->kb, q->recs, q->rec_bytes, q->wscale, 1.f / q->wscale};
    return v;
}

// ---------------------------------------------------------------- launches implemented per file
fh_status fh_launch_qmatvec(const fh_qmatrix *q, const float *x, int m, float *y, int epilogue,
                            const float *a, const float *b);
bool fh_qmatvec_batch_supports(const fh_qmatrix *q, int m, int epi);
fh_status fh_launch_qmatvec_batch(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a,
                                  const float *b);
fh_status fh_launch_qmm_q8_mfma(const fh_qmatrix *q, const float *x, int m, float *y);
fh_status fh_launch_qmatmul_tile(const fh_qmatrix *q, const void *x, int x_is_bf16, int m, float *y);
// power of two for fh_qmatrix::wscale from the largest |w| of `count` f32 values on the device (blocking)
fh_status fh_dense_wscale(fh_device *dev, const float *w_dev, int64_t count, float *wscale);
enum { FH_EPI_NONE = 0, FH_EPI_ADD2 = 1, FH_EPI_SWIGLU = 2, FH_EPI_ROPEKV = 3, FH_EPI_ACC = 4 };
fh_status fh_launch_kparts_reduce(fh_device *dev, const float *part, int parts, int m, int64_t n, float *y, int epi,
                                  const float *a, const float *b);
fh_status fh_launch_q4k_rows(const fh_qmatrix *q, const float *x, int m, float *y, int epi, const float *a, const float *b);
fh_status fh_launch_q4k_m1(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b);
fh_status fh_launch_q4k_m1_norm(const fh_qmatrix *q, const float *x, const float *xres, const float *nw, float eps,
                                float *y, int epi, const float *a, const float *b);
fh_status fh_launch_q4k_m1_attn(const fh_qmatrix *q, const float *part, int nsplit, float *y);
fh_status fh_launch_q4k_m1_attn_acc(const fh_qmatrix *q, const float *part, int nsplit, float *y_inout);
fh_status fh_attention_combine_dl(fh_device *dev, int hq, int splits, float *out);
fh_status fh_attention_combine_parts(fh_device *dev, const float *part, int hq, int splits, void *out, bool out_f16);
fh_status fh_attention_decode_mfma(fh_device *dev, const void *q, bool q_f16, const void *k, const void *v,
                                   int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale, int skv,
                                   int splits, float *part);
fh_status fh_attention_decode_hostlen(fh_device *dev, int kv_dtype, const void *q, bool q_f16, const void *k,
                                      const void *v, int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale,
                                      int skv, void *out, bool out_f16);
fh_status fh_attention_prefill_mfma(fh_device *dev, int q_dtype, int kv_dtype, const void *q, int64_t q_sb,
                                    int64_t q_sh, int64_t q_st, const void *k, const void *v, int64_t kv_sb,
                                    int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int sq, int skv, int d,
                                    float scale, int mask_kind, void *out);
fh_status fh_launch_q6k_m1_acc(const fh_qmatrix *q, const float *x, const float *xup, float *y_inout, const float *add);
fh_status fh_launch_q6k_m1(const fh_qmatrix *q, const float *x, float *y, int epi, const float *a, const float *b);

struct fh_kvcache {
    fh_device *dev = nullptr;
    int layers = 0, kv_heads = 0, head_dim = 0, max_len = 0, dtype = FH_F32;
    int len = 0, capacity = 0;
    bool sliding = false;            // past max_len: keep the last max_len positions instead of failing
    void *k = nullptr, *v = nullptr; // [layers][kv_heads][capacity][head_dim]
    int *len_dev = nullptr;          // device copy of len (for graph-replayed decode steps)
};
size_t fh_dtype_size(int dtype);
fh_status fh_kvcache_reserve(fh_kvcache *c, int required);
// append reading the write position from c->len_dev (graph friendly), s == 1
fh_status fh_kvcache_append_devpos(fh_kvcache *c, int layer, const float *k, const float *v, int64_t sh);
fh_status fh_launch_q4k_m1_ropekv(const fh_qmatrix *q, const float *x, const float *nw, float eps, fh_kvcache *c,
                                  int layer, int hq, const float *cos_t, const float *sin_t, int table_rows,
                                  float *q_out);
fh_status fh_rope_kv_decode(fh_kvcache *c, int layer, const float *q, const float *k, const float *v, int hq,
                            const float *cos_t, const float *sin_t, int table_rows, float *q_out);
fh_status fh_kvcache_append_kv(fh_kvcache *c, int layer, const float *k, int64_t k_sh, int64_t k_st, const float *v,
                               int64_t v_sh, int64_t v_st, int s, int pos);
fh_status fh_kvcache_set_len_dev(fh_kvcache *c, int len);
fh_status fh_swiglu_rows(fh_device *dev, const float *gu, int rows, int f, float *y);
// decode attention reading the KV length from a device int (graph friendly)
fh_status fh_attention_decode_devlen_v1(fh_device *dev, int kv_dtype, const float *q, const void *k,
                                     const void *v, int64_t kv_sh, int64_t kv_st, int hq, int hkv,
                                     int d, float scale, const int *len_dev, int max_len, float *out);
fh_status fh_attention_decode_devlen(fh_device *dev, int kv_dtype, const float *q, const void *k, const void *v,
                                     int64_t kv_sh, int64_t kv_st, int hq, int hkv, int d, float scale,
                                     const int *len_dev, int max_len, float *out, int *splits_out);
fh_status fh_rope_pair_devpos(fh_device *dev, const float *q, const float *k, int hq, int hk, int d,
                              const float *cos_t, const float *sin_t, int table_rows,
                              const int *pos_dev, float *q_out, float *k_out);
// End of a device-side decode step, done by the last stage of the greedy pick (all pointers device memory).
struct FhStepTail {
    uint32_t *ids = nullptr;        // next step's input id
    uint32_t *out_tokens = nullptr; // the step's output list
    int *step = nullptr;            // its fill count
    int *kv_len = nullptr;          // KV cache length
};
fh_status fh_argmax_step(fh_device *dev, const float *x_dev, int64_t count, uint32_t *id_dev, FhStepTail tail);
// Sampler with every per-step input in device memory (fh_elementwise.hip); fh_sample_token is its host-input form.
fh_status fh_sample_token_dev(fh_device *dev, const float *logits_dev, int64_t count, const fh_sampler_params *p,
                              const uint32_t *prev_dev, const uint32_t *prev_len_dev, uint32_t n_prev,
                              const float *randoms_dev, const int *step_dev, float *mu_dev, uint32_t *result_dev,
                              uint32_t *ids_dev, float *values_dev);


// Device, memory, error and timing entry points of libfusor_hip.so.
#include "fh_internal.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

static thread_local char g_err[512] = "";

void fh_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *fh_last_error(void) { return g_err; }
extern "C" const char *fh_version(void) { return "fusor-hip 0.1 (gfx950)"; }

extern "C" fh_status fh_device_count(int32_t *count) {
    FH_REQUIRE(count, "count is NULL");
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        c = 0;
    }
    *count = c;
    return FH_OK;
}

extern "C" fh_status fh_device_create(int32_t ordinal, fh_device **out) {
    FH_REQUIRE(out, "out is NULL");
    *out = nullptr;
    int c = 0;
    if (hipGetDeviceCount(&c) != hipSuccess || c <= 0) {
        (void)hipGetLastError();
        FH_FAIL(FH_ERR_NO_DEVICE, "no HIP device available");
    }
    FH_REQUIRE(ordinal >= 0 && ordinal < c, "device ordinal %d out of range (have %d)", ordinal, c);
    FH_HIP(hipSetDevice(ordinal));
    hipDeviceProp_t p;
    FH_HIP(hipGetDeviceProperties(&p, ordinal));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        FH_FAIL(FH_ERR_NO_DEVICE, "device %d is %s; this library holds gfx950 code only", ordinal, p.gcnArchName);
    fh_device *d = new fh_device();
    d->ordinal = ordinal;
    d->compute_units = p.multiProcessorCount;
    FH_HIP(hipStreamCreate(&d->stream));
    FH_HIP(hipEventCreate(&d->ev_start));
    FH_HIP(hipEventCreate(&d->ev_stop));
    FH_HIP(hipMalloc(&d->small_buf, 64 * 1024));
    // the reference's trace switches (models/kalosm-llama/src/raw/mod.rs:943-955, fusor-ml/core/src/compute_graph/
    // resolve/run.rs:141): present in the environment = on, lines on stderr
    if (getenv("KALOSM_TRACE_LAYER_NAN")) d->opt_trace_nan = d->opt_trace_stderr = 1;
    if (getenv("KALOSM_TRACE_FORWARD_TIMING")) d->opt_trace_timing = d->opt_trace_stderr = 1;
    if (getenv("FUSOR_TRACE_GPU_KERNELS")) d->opt_trace_timing = 2, d->opt_trace_stderr = 1;
    fh_status st = fh_static_scratch_init(d);
    if (st != FH_OK) {
        (void)fh_device_destroy(d);
        return st;
    }
    *out = d;
    return FH_OK;
}

extern "C" fh_status fh_device_destroy(fh_device *dev) {
    if (!dev) return FH_OK;
    (void)hipSetDevice(dev->ordinal);
    (void)hipStreamSynchronize(dev->stream);
    if (dev->act_buf) (void)hipFree(dev->act_buf);
    if (dev->part_buf) (void)hipFree(dev->part_buf);
    if (dev->ksplit_buf) (void)hipFree(dev->ksplit_buf);
    if (dev->small_buf) (void)hipFree(dev->small_buf);
    (void)hipEventDestroy(dev->ev_start);
    (void)hipEventDestroy(dev->ev_stop);
    (void)hipStreamDestroy(dev->stream);
    delete dev;
    return FH_OK;
}

extern "C" fh_status fh_device_sync(fh_device *dev) {
    FH_REQUIRE(dev, "dev is NULL");
    FH_HIP(hipStreamSynchronize(dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_device_info(fh_device *dev, char *name, size_t name_cap, int32_t *compute_units,
                                    uint64_t *total_mem_bytes) {
    FH_REQUIRE(dev, "dev is NULL");
    hipDeviceProp_t p;
    FH_HIP(hipGetDeviceProperties(&p, dev->ordinal));
    if (name && name_cap) snprintf(name, name_cap, "%s (%s)", p.name, p.gcnArchName);
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (total_mem_bytes) *total_mem_bytes = (uint64_t)p.totalGlobalMem;
    return FH_OK;
}

extern "C" fh_status fh_malloc(fh_device *dev, size_t bytes, void **out_dev) {
    FH_REQUIRE(dev && out_dev, "NULL argument");
    *out_dev = nullptr;
    if (bytes == 0) bytes = 16;
    FH_HIP(hipSetDevice(dev->ordinal));
    FH_HIP(hipMalloc(out_dev, bytes));
    return FH_OK;
}

extern "C" fh_status fh_free(fh_device *dev, void *ptr_dev) {
    FH_REQUIRE(dev, "dev is NULL");
    if (!ptr_dev) return FH_OK;
    FH_HIP(hipStreamSynchronize(dev->stream));
    FH_HIP(hipFree(ptr_dev));
    return FH_OK;
}

// A fill kernel rather than hipMemsetAsync, so the call can be recorded into a graph.
__global__ void k_fill_bytes(uint8_t *p, uint8_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

extern "C" fh_status fh_memset(fh_device *dev, void *ptr_dev, int32_t byte, size_t bytes) {
    FH_REQUIRE(dev && ptr_dev, "NULL argument");
    if (!bytes) return FH_OK;
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    k_fill_bytes<<<dim3((unsigned)blocks), dim3(256), 0, dev->stream>>>((uint8_t *)ptr_dev, (uint8_t)byte, bytes);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_upload(fh_device *dev, void *dst_dev, const void *src_host, size_t bytes) {
    FH_REQUIRE(dev && dst_dev && (src_host || bytes == 0), "NULL argument");
    if (!bytes) return FH_OK;
    FH_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, dev->stream));
    FH_HIP(hipStreamSynchronize(dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_download(fh_device *dev, void *dst_host, const void *src_dev, size_t bytes) {
    FH_REQUIRE(dev && src_dev && (dst_host || bytes == 0), "NULL argument");
    if (!bytes) return FH_OK;
    FH_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, dev->stream));
    FH_HIP(hipStreamSynchronize(dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_copy(fh_device *dev, void *dst_dev, const void *src_dev, size_t bytes) {
    FH_REQUIRE(dev && dst_dev && src_dev, "NULL argument");
    if (!bytes) return FH_OK;
    FH_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_timer_start(fh_device *dev) {
    FH_REQUIRE(dev, "dev is NULL");
    FH_HIP(hipEventRecord(dev->ev_start, dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_timer_stop(fh_device *dev, float *elapsed_ms) {
    FH_REQUIRE(dev && elapsed_ms, "NULL argument");
    FH_HIP(hipEventRecord(dev->ev_stop, dev->stream));
    FH_HIP(hipEventSynchronize(dev->ev_stop));
    FH_HIP(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
    return FH_OK;
}

// ---------------------------------------------------------------- measurement probes
// What a launch costs on this device before any arithmetic: an empty kernel, and a plain streaming read (16 bytes
// per lane and request, 4 KB per wavefront, four requests in flight per lane).  The matvec kernels are priced
// against these, not only against the nominal HBM peak.
__global__ void k_probe_empty(uint32_t *p) {
    if (p && threadIdx.x == 9999) *p = 1;
}
__global__ __launch_bounds__(256) void k_probe_read(const uint4 *__restrict__ src, uint32_t *out) {
    const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint4 *p = src + wave * 256 + (threadIdx.x & 63);
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = p[u * 64];
    uint32_t a = 0;
#pragma unroll
    for (int u = 0; u < 4; u++) a ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (a == 0x12345678u) out[0] = a; // keeps the loads alive; practically never true
}

// What the device sustains under three access patterns the kernels are built from (each call measures itself):
//   dense v_mfma_f32_32x32x16_f16 (four independent accumulators per wavefront),
//   ds_read_b128 with eight reads in flight per wavefront, by address pattern,
//   L2 hits of some wavefronts of a compute unit next to an HBM stream of the others.
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void k_probe_mfma(int iters, float *out) {
    probe_half8 a, b;
    for (int i = 0; i < 8; i++) a[i] = (_Float16)(threadIdx.x * 0.001f + i), b[i] = (_Float16)(1.0f - i * 0.01f);
    probe_floatx16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
    }
    float s = 0;
    for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 12345.f) out[0] = s; // keeps the products alive; practically never true
}
// pattern 0: lane l reads 16 bytes at 16 l.  1 .. 3: MFMA operand addressing - lane l reads row l % 32 (128 bytes per row),
// 16-byte piece (l / 32) ^ swizzle(row): 1 none, 2 row & 7, 3 the tile kernels' ((row >> 1) & 1) << 2 | ((row >> 2) & 3)
__global__ __launch_bounds__(1024) void k_probe_lds(int iters, int pattern, uint32_t *out, long long *clk) {
    extern __shared__ __attribute__((aligned(16))) unsigned char probe_lds[];
    for (int i = threadIdx.x; i < 65536 / 4; i += blockDim.x) ((uint32_t *)probe_lds)[i] = i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int off = lane * 16;
    if (pattern != 0) {
        const int row = lane & 31, piece = lane >> 5;
        const int sw = pattern == 1 ? 0 : pattern == 2 ? (row & 7) : (((row >> 1) & 1) << 2 | ((row >> 2) & 3));
        off = row * 128 + 16 * (piece ^ sw);
    }
    off += (wave & 3) * 4096;
    uint32_t acc = 0;
    const long long t0 = clock64();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const probe_u32x4 v = *(const probe_u32x4 *)(probe_lds + off + ((u * 8192 + i * 64) & 0xE000));
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
        }
    }
    const long long t1 = clock64();
    if (acc == 0x12345u) out[0] = acc;
    if (threadIdx.x == 0 && blockIdx.x == 0) clk[0] = t1 - t0;
}
// One workgroup of 16 wavefronts per compute unit.  mode 0: every wavefront reads the shared 256 KB at `l2` `reps` times;
// 1: every wavefront streams its own `per_wave16` x 16 bytes of `hbm`; 2: even wavefronts the first, odd ones the second.
// clk[workgroup * 16 + wavefront] = the wavefront's duration in ticks of the 100 MHz wall clock.
__global__ __launch_bounds__(1024) void k_probe_mix(const probe_u32x4 *l2, const probe_u32x4 *hbm, size_t per_wave16, int reps,
                                                    int mode, long long *clk, uint32_t *out) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool l2wave = mode == 0 ? true : mode == 1 ? false : (wave & 1) == 0;
    probe_u32x4 acc = {0, 0, 0, 0};
    const long long t0 = wall_clock64();
    if (l2wave) {
        for (int r = 0; r < reps; r++)
            for (int i = 0; i < 16384 / 256; i++) {
                const probe_u32x4 *p = l2 + i * 256 + lane;
                acc ^= p[0] ^ p[64] ^ p[128] ^ p[192];
            }
    } else {
        const probe_u32x4 *base = hbm + ((size_t)blockIdx.x * 16 + wave) * per_wave16;
        for (size_t i = 0; i < per_wave16 / 256; i++) {
            const probe_u32x4 *p = base + i * 256 + lane;
            acc ^= __builtin_nontemporal_load(p) ^ __builtin_nontemporal_load(p + 64) ^ __builtin_nontemporal_load(p + 128) ^
                   __builtin_nontemporal_load(p + 192);
        }
    }
    const long long t1 = wall_clock64();
    if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345u) out[0] = 1;
}

extern "C" fh_status fh_probe_device(fh_device *dev, int32_t kind, int32_t a, int32_t b, const void *src_dev, size_t src_bytes,
                                     double *out4) {
    FH_REQUIRE(dev && out4, "NULL argument");
    out4[0] = out4[1] = out4[2] = out4[3] = 0.0;
    const int cus = dev->compute_units;
    uint32_t *sink = (uint32_t *)dev->small_buf;
    long long *clk = (long long *)((uint8_t *)dev->small_buf + 256); // up to 256 x 16 durations
    float ms = 0;
    if (kind == 0) { // a = wavefronts per SIMD (1, 2), b = iterations: out = TFLOP/s, microseconds
        FH_REQUIRE((a == 1 || a == 2) && b > 0, "mfma probe: wavefronts per SIMD 1 or 2, iterations > 0");
        k_probe_mfma<<<dim3((unsigned)cus), dim3(256 * a), 0, dev->stream>>>(b, (float *)sink); // warm
        FH_TRY(fh_timer_start(dev));
        k_probe_mfma<<<dim3((unsigned)cus), dim3(256 * a), 0, dev->stream>>>(b, (float *)sink);
        FH_HIP(hipGetLastError());
        FH_TRY(fh_timer_stop(dev, &ms));
        out4[0] = (double)cus * 4 * a * b * 4 * 32768.0 / (ms * 1e-3) / 1e12;
        out4[1] = ms * 1e3;
        return FH_OK;
    }
    if (kind == 1) { // a = wavefronts per workgroup (4, 8, 16), b = pattern 0 .. 3: out = bytes per ns, bytes per shader clock (per CU)
        FH_REQUIRE((a == 4 || a == 8 || a == 16) && b >= 0 && b <= 3, "lds probe: 4, 8 or 16 wavefronts, pattern 0 .. 3");
        const int iters = 2000;
        static bool attr_done = false;
        if (!attr_done) {
            FH_HIP(hipFuncSetAttribute((const void *)k_probe_lds, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
            attr_done = true;
        }
        k_probe_lds<<<dim3((unsigned)cus), dim3(64 * a), 65536, dev->stream>>>(iters, b, sink, clk);
        FH_TRY(fh_timer_start(dev));
        k_probe_lds<<<dim3((unsigned)cus), dim3(64 * a), 65536, dev->stream>>>(iters, b, sink, clk);
        FH_HIP(hipGetLastError());
        FH_TRY(fh_timer_stop(dev, &ms));
        long long ticks = 0;
        FH_TRY(fh_download(dev, &ticks, clk, 8));
        const double bytes = (double)a * 64 * 16 * 8 * iters;
        out4[0] = bytes / (ms * 1e6); // the launch includes filling the LDS: a lower bound
        out4[1] = ticks > 0 ? bytes / (double)ticks : 0.0;
        return FH_OK;
    }
    if (kind == 2) { // a = mode 0 .. 2; src: 256 KB + compute units x 16 x 512 KB: out = L2 bytes per ns and CU, HBM bytes per ns and CU
        const size_t per_wave = 512 << 10, need = (256 << 10) + (size_t)cus * 16 * per_wave;
        FH_REQUIRE(a >= 0 && a <= 2 && src_dev && src_bytes >= need && cus <= 256, "mix probe: mode 0 .. 2 and a buffer of %zu bytes",
                   need);
        const probe_u32x4 *l2 = (const probe_u32x4 *)src_dev, *hbm = l2 + (256 << 10) / 16;
        const int reps = 8;
        for (int it = 0; it < 2; it++) k_probe_mix<<<dim3((unsigned)cus), dim3(1024), 0, dev->stream>>>(l2, hbm, per_wave / 16, reps, a, clk, sink);
        FH_HIP(hipGetLastError());
        std::vector<long long> h((size_t)cus * 16);
        FH_TRY(fh_download(dev, h.data(), clk, h.size() * 8));
        double tl = 0, th = 0;
        int nl = 0, nh = 0;
        for (size_t i = 0; i < h.size(); i++) {
            const bool l2wave = a == 0 ? true : a == 1 ? false : ((i & 15) & 1) == 0;
            if (l2wave) tl += (double)h[i], nl++;
            else th += (double)h[i], nh++;
        }
        // ticks of 10 ns; wavefronts of a kind per compute unit: 16 or 8
        if (nl) out4[0] = (nl / cus) * (256.0 * 1024 * reps) / (tl / nl * 10.0);
        if (nh) out4[1] = (nh / cus) * (double)per_wave / (th / nh * 10.0);
        return FH_OK;
    }
    FH_FAIL(FH_ERR_INVALID, "unknown probe kind %d", kind);
}

extern "C" fh_status fh_probe_empty(fh_device *dev, int32_t workgroups, int32_t threads) {
    FH_REQUIRE(dev && workgroups > 0 && threads > 0 && threads <= 1024, "bad probe launch");
    k_probe_empty<<<dim3((unsigned)workgroups), dim3((unsigned)threads), 0, dev->stream>>>((uint32_t *)dev->small_buf);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_probe_read(fh_device *dev, const void *src_dev, size_t bytes) {
    FH_REQUIRE(dev && src_dev, "NULL argument");
    FH_REQUIRE(bytes >= 16384 && bytes % 16384 == 0 && bytes / 16384 <= 0x7FFFFFFFu, "bytes must be a multiple of 16384");
    k_probe_read<<<dim3((unsigned)(bytes / 16384)), dim3(256), 0, dev->stream>>>((const uint4 *)src_dev,
                                                                              (uint32_t *)dev->small_buf);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

fh_status fh_dev_scratch(fh_device *dev, void **buf, size_t *cap, size_t need) {
    if (*cap >= need) return FH_OK;
    if (dev->capturing)
        FH_FAIL(FH_ERR_INVALID, "a captured call needs %zu bytes of scratch but only %zu are allocated: run the "
                                "sequence once eagerly before capturing it", need, *cap);
    if (*buf) {
        FH_HIP(hipStreamSynchronize(dev->stream));
        FH_HIP(hipFree(*buf));
        *buf = nullptr;
        *cap = 0;
    }
    size_t want = need < (1u << 20) ? (1u << 20) : need;
    FH_HIP(hipMalloc(buf, want));
    *cap = want;
    dev->scratch_gen++;
    return FH_OK;
}

extern "C" fh_status fh_set_option(fh_device *dev, const char *key, int64_t value) {
    FH_REQUIRE(dev && key, "NULL argument");
    if (!strcmp(key, "matvec_kernel")) dev->opt_matvec_kernel = value;
    else if (!strcmp(key, "matvec_splitk")) dev->opt_matvec_splitk = value;
    else if (!strcmp(key, "matvec_waves")) dev->opt_matvec_waves = value;
    else if (!strcmp(key, "matvec_tiles")) dev->opt_matvec_tiles = value;
    else if (!strcmp(key, "matvec_per")) dev->opt_matvec_per = value;
    else if (!strcmp(key, "attn_splits")) dev->opt_attn_splits = value;
    else if (!strcmp(key, "attn_kernel")) dev->opt_attn_kernel = value;
    else if (!strcmp(key, "matmul_kernel")) dev->opt_matmul_kernel = value;
    else if (!strcmp(key, "fuse_norm")) dev->opt_fuse_norm = value;
    else if (!strcmp(key, "down_splitk")) dev->opt_down_splitk = value;
    else if (!strcmp(key, "wo_acc")) dev->opt_wo_acc = value;
    else if (!strcmp(key, "wo_tiles")) dev->opt_wo_tiles = value;
    else if (!strcmp(key, "matvec_rows")) dev->opt_matvec_rows = value;
    else if (!strcmp(key, "matvec_direct")) dev->opt_matvec_direct = value;
    else if (!strcmp(key, "attn_waves")) dev->opt_attn_waves = value;
    else if (!strcmp(key, "attn_heads")) dev->opt_attn_heads = value;
    else if (!strcmp(key, "down_tiles")) dev->opt_down_tiles = value;
    else if (!strcmp(key, "deterministic")) dev->opt_deterministic = value;
    else if (!strcmp(key, "trace_nan")) dev->opt_trace_nan = value;
    else if (!strcmp(key, "trace_timing")) dev->opt_trace_timing = value;
    else if (!strcmp(key, "trace_stderr")) dev->opt_trace_stderr = value;
    else FH_FAIL(FH_ERR_INVALID, "unknown option '%s'", key);
    dev->opt_gen++;
    return FH_OK;
}

struct fh_graph {
    fh_device *dev = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint64_t scratch_gen = 0; // dev->scratch_gen when the capture ended
};

extern "C" fh_status fh_graph_begin(fh_device *dev) {
    FH_REQUIRE(dev, "dev is NULL");
    FH_REQUIRE(!dev->capturing, "a capture is already in progress");
    FH_HIP(hipStreamSynchronize(dev->stream));
    FH_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
    dev->capturing = true;
    return FH_OK;
}

extern "C" fh_status fh_graph_end(fh_device *dev, fh_graph **out) {
    FH_REQUIRE(dev && out, "NULL argument");
    FH_REQUIRE(dev->capturing, "no capture in progress");
    *out = nullptr;
    dev->capturing = false;
    hipGraph_t g = nullptr;
    FH_HIP(hipStreamEndCapture(dev->stream, &g));
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        FH_FAIL(FH_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    fh_graph *r = new fh_graph();
    r->dev = dev;
    r->graph = g;
    r->exec = ex;
    r->scratch_gen = dev->scratch_gen;
    *out = r;
    return FH_OK;
}

extern "C" fh_status fh_graph_launch(fh_graph *g) {
    FH_REQUIRE(g && g->exec, "NULL graph");
    if (g->scratch_gen != g->dev->scratch_gen)
        FH_FAIL(FH_ERR_INVALID, "the device's scratch buffers were reallocated by a larger call since this graph was "
                                "captured; its kernels hold the old addresses: capture it again");
    FH_HIP(hipGraphLaunch(g->exec, g->dev->stream));
    return FH_OK;
}

extern "C" fh_status fh_graph_free(fh_graph *g) {
    if (!g) return FH_OK;
    (void)hipStreamSynchronize(g->dev->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return FH_OK;
}

size_t fh_dtype_size(int dtype) { return dtype == FH_F16 ? 2 : 4; }

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

fh_status fh_kernel_lds(fh_device *dev, const void *kernel, size_t bytes) {
    for (auto &e : dev->lds_raised)
        if (e.first == kernel) {
            if (e.second >= bytes) return FH_OK;
            FH_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
            e.second = bytes;
            return FH_OK;
        }
    FH_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    dev->lds_raised.emplace_back(kernel, bytes);
    return FH_OK;
}

extern "C" fh_status fh_set_option(fh_device *dev, const char *key, int64_t value) {
    FH_REQUIRE(dev && key, "NULL argument");
    if (!strcmp(key, "matvec_kernel")) dev->opt_matvec_kernel = value;
    else if (!strcmp(key, "matvec_splitk")) dev->opt_matvec_splitk = value;
    else if (!strcmp(key, "matvec_waves")) dev->opt_matvec_waves = value;
    else if (!strcmp(key, "matvec_tiles")) dev->opt_matvec_tiles = value;
    else if (!strcmp(key, "matvec_per")) dev->opt_matvec_per = value;
    else if (!strcmp(key, "matvec_rowsplit")) dev->opt_matvec_rowsplit = value;
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

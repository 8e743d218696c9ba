// Measurement probes (include/fusor_hip_probe.h): what a launch and a plain streaming read cost on this device, and
// what the matrix cores, the LDS and the L2 next to an HBM stream sustain.  Not part of the operator boundary.
#include "fh_internal.h"
#include "../../include/fusor_hip_probe.h"

#include <vector>

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
            // inside the 64 KB allocation whatever the wavefront's offset
            const probe_u32x4 v = *(const probe_u32x4 *)(probe_lds + ((off + ((u * 8192 + i * 64) & 0xE000)) & 0xFFFF));
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
        FH_TRY(fh_kernel_lds(dev, (const void *)k_probe_lds, 65536));
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

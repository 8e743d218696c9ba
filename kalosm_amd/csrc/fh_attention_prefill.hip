// Prefill attention on the matrix cores: softmax(Q . K^T * scale [causal]) . V for many query rows, grouped-query
// heads, head_dim 64 or 128.
// Reference: fusor-ml/fusor/src/composite/flash_attention.rs:58-236 (semantics; causal mask as MaskKind::Causal
// with the queries aligned to the END of the keys), fusor-ml/core/src/row_program.rs:1210-1382 (the fused kernel).
//
// grid (q heads / HW, query blocks of 128, batch); 4 x HW wavefronts, each owning 32 query rows of one head: the HW
// (1 or 2) heads of a workgroup share a KV head, so a KV tile is fetched and staged once for 128 x HW query rows.
// KV tiles of 64 keys go through LDS as f16, both as [key][d] rows written with 16-byte stores; the V^T operand
// of the second product is read with the transposing LDS load of gfx950 (ds_read_b64_tr_b16: the 16 lanes of a
// group supply 4 keys x 16 dims and receive, per lane, one dim of the 4 keys).  Two LDS buffers and one barrier per
// tile: tile t+1 is written to the other buffer right after the first product of tile t (its LDS writes and the
// request for tile t+2 then run under the softmax arithmetic).
// KS = 2 (short prompts: fewer workgroups than the device holds, and the launch lasts as long as the workgroup of the
// last query block): eight wavefronts per query block, the second four take every other key tile with running
// statistics of their own, and the two halves are merged through LDS at the end - half the tile steps per workgroup.
// QW = 2 (shorter still: every workgroup of 64 query rows finds a compute unit of its own): two wavefronts per key
// group, so a SIMD runs one wavefront's chain of a step instead of two.
// What bounds the loop (measured per stage): the first product is matrix-core bound, the softmax vector-ALU bound
// (both wavefronts of a SIMD are in it together) and the second product bound by the transposing LDS loads, which
// run at half the rate of plain 16-byte loads.
// Both products are computed TRANSPOSED with
// v_mfma_f32_32x32x16_f16 so that a lane always stands for ONE query (the accumulator column):
//   S^T (keys x queries) = K . Q^T      A = K rows, B = Q^T kept in registers for the whole kernel
//   O^T (d x queries)    = V^T . P^T    A = V^T rows, B = P^T = the S^T accumulator, exponentiated, as f16
// The online-softmax statistics (running max, running sum, rescale factor) are then per-lane scalars, and the row
// maximum is a reduction over the lane's own registers plus one exchange with lane + 32.  MFMA row i of the K
// operand reads key 16*(i/16) + 8*((i/4)%2) + 4*((i/8)%2) + i%4 of the tile: with that order the 16 accumulator
// registers of a lane are keys 8g .. 8g+7 and 16 + 8g .. 16 + 8g+7 (g = lane / 32), which is exactly the k-slot
// order of the B operand of the second product - P^T never leaves the registers.
// Inputs may be f32 or f16; operands are rounded to f16, all accumulation and the softmax are f32.
// SPLIT (f32 Q, K and V): every operand is the exact two-term f16 split hi + lo of the f32 value (2^-22 relative;
// the values must lie within the f16 range of +-65504) and both products are the three MFMAs
// hi.hi + lo.hi + hi.lo, so the result keeps f32 accuracy at three times the matrix-core work.
#include "fh_internal.h"

typedef _Float16 fh_half;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void ap_load8(const float *p, fh_half *o) {
    const float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
    o[0] = (fh_half)a.x; o[1] = (fh_half)a.y; o[2] = (fh_half)a.z; o[3] = (fh_half)a.w;
    o[4] = (fh_half)b.x; o[5] = (fh_half)b.y; o[6] = (fh_half)b.z; o[7] = (fh_half)b.w;
}
__device__ __forceinline__ void ap_load8(const fh_half *p, fh_half *o) {
    const uint4 r = *(const uint4 *)p;
    __builtin_memcpy(o, &r, 16);
}
__device__ __forceinline__ float ap_swap32_max(float v) {
    const uint32_t u = __float_as_uint(v);
    auto s = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(s[0]), __uint_as_float(s[1]));
}
__device__ __forceinline__ float ap_swap32_sum(float v) {
    const uint32_t u = __float_as_uint(v);
    auto s = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}
__device__ __forceinline__ void ap_store4(float *p, float a, float b, float c, float d) {
    *(float4 *)p = make_float4(a, b, c, d);
}
__device__ __forceinline__ void ap_store4(fh_half *p, float a, float b, float c, float d) {
    const fh_half h[4] = {(fh_half)a, (fh_half)b, (fh_half)c, (fh_half)d};
    uint2 u;
    __builtin_memcpy(&u, h, 8);
    *(uint2 *)p = u;
}

__device__ __forceinline__ void ap_split8(const float *x, fh_half *hi, fh_half *lo) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        hi[e] = (fh_half)x[e];
        lo[e] = (fh_half)(x[e] - (float)hi[e]);
    }
}

typedef short short4v __attribute__((ext_vector_type(4)));
// Eight halfs of the V^T operand: keys k .. k+7 of the dim this lane stands for (two transposing loads of 4 keys).
__device__ __forceinline__ half8 ap_vt8(const fh_half *p, int row_stride) {
    const short4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p);
    const short4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(uintptr_t)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)(p + 4 * row_stride));
    half8 r;
    __builtin_memcpy(&r, &a, 8);
    __builtin_memcpy((char *)&r + 8, &b, 8);
    return r;
}

template <typename TQ, typename TKV, int D, bool SPLIT = false, int HW = 1, int KS = 1, int QW = 4>
__global__ __launch_bounds__(64 * QW * HW * KS) __attribute__((amdgpu_waves_per_eu(QW == 4 ? 2 : 1, 2))) void k_attn_prefill(const TQ *__restrict__ q, int64_t q_sb, int64_t q_sh, int64_t q_st,
                                                       const TKV *__restrict__ k, const TKV *__restrict__ v,
                                                       int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int hq, int hkv,
                                                       int sq, int skv, float scale, int causal, TQ *__restrict__ out) {
    constexpr int BN = 64, KS_ = D + 8, VS = D + 16, DT = D / 32, KSTEPS = D / 16, CH = D / 8; // CH: 8-element chunks per row
    constexpr int NP = SPLIT ? 2 : 1; // operand planes: hi (, lo)
    static_assert(HW * KS <= 2 && !(SPLIT && KS == 2), "eight wavefronts at most; split operands leave no room for two tiles");
    static_assert(QW == 4 || (QW == 2 && HW == 1 && KS == 2), "query blocks of 128 rows, or of 64 with two key groups");
    constexpr int QB = 32 * QW; // query rows of a workgroup: QW wavefronts of 32
    constexpr int NTH = 64 * QW * HW * KS, KBUF = NP * BN * KS_, VBUF = NP * BN * VS, TILE = KBUF + VBUF; // halfs per staged tile
    extern __shared__ __attribute__((aligned(16))) fh_half ap_lds[]; // [2 buffers][K planes | V planes]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
    const int kset = KS == 2 ? wave / QW : 0; // which key tiles of a step this wavefront multiplies
    const int h = (int)blockIdx.x * HW + (HW == 2 ? wave >> 2 : 0), bi = blockIdx.z, kh = h / (hq / hkv);
    // causal: the last query blocks see the most keys; with the block index on the slow grid axis ALL heads of the
    // longest block are dispatched first and the short blocks fill the tail
    const int qb0 = (causal ? (int)(gridDim.y - 1 - blockIdx.y) : (int)blockIdx.y) * QB;
    const int qi = qb0 + (wave % QW) * 32 + li; // this lane's query row (KS = 2: both groups have the same rows)
    const int off = skv - sq;                  // causal: query i sees keys 0 .. i + off
    const TKV *kb = k + bi * kv_sb + kh * kv_sh, *vb = v + bi * kv_sb + kh * kv_sh;

    // Q^T operand, once: lane (query li, k-slots 8g .. 8g+7 of every 16-wide step of d)
    half8 qf[KSTEPS], ql[SPLIT ? KSTEPS : 1];
    {
        const TQ *qp = q + bi * q_sb + h * q_sh + (int64_t)(qi < sq ? qi : sq - 1) * q_st + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            fh_half t[8];
            if constexpr (SPLIT) {
                const float4 a = *(const float4 *)(qp + 16 * ks), b = *(const float4 *)(qp + 16 * ks + 4);
                const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                fh_half lo[8];
                ap_split8(x, t, lo);
                __builtin_memcpy(&ql[ks], lo, 16);
            } else {
                ap_load8(qp + 16 * ks, t);
            }
            __builtin_memcpy(&qf[ks], t, 16);
        }
    }
    const int prow = 16 * (li >> 4) + 8 * ((li >> 2) & 1) + 4 * ((li >> 3) & 1) + (li & 3); // key read by MFMA row li
    const float sc2 = scale * 1.4426950408889634f;                                        // scores in the log2 domain
    float m_run = -INFINITY, l_run = 0.f;
    floatx16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[dt][r] = 0.f;

    int kend = skv;
    if (causal) {
        const int last = (qb0 + QB - 1 < sq ? qb0 + QB - 1 : sq - 1) + off + 1;
        kend = last < skv ? last : skv;
    }
    // A KV tile waits in registers (as f16; SPLIT: as the f32 values) from one tile before it is written to LDS.
    // Piece c = tid + NTH i of a tile: key c / CH, d chunk c % CH - consecutive threads along d, K and V alike.
    constexpr int NCH = KS * BN * CH / NTH;
    uint4 kreg[SPLIT ? 1 : NCH], vreg[SPLIT ? 1 : NCH];
    float4 kraw[SPLIT ? 2 * NCH : 1], vraw[SPLIT ? 2 * NCH : 1];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + NTH * i, key = c / CH, dc = c % CH; // key 0 .. KS * BN - 1: the KS tiles of a step
            // rows past the end repeat the last one (no branch): their scores are masked and their P is 0
            const int64_t row = (int64_t)(t0 + key < skv ? t0 + key : skv - 1) * kv_st + 8 * dc;
            if constexpr (SPLIT) {
                const float *kp = (const float *)kb + row, *vp = (const float *)vb + row;
                kraw[2 * i] = *(const float4 *)kp;
                kraw[2 * i + 1] = *(const float4 *)(kp + 4);
                vraw[2 * i] = *(const float4 *)vp;
                vraw[2 * i + 1] = *(const float4 *)(vp + 4);
            } else {
                fh_half t[8];
                ap_load8(kb + row, t);
                __builtin_memcpy(&kreg[i], t, 16);
                ap_load8(vb + row, t);
                __builtin_memcpy(&vreg[i], t, 16);
            }
        }
    };
    auto stash = [&](int buf) { // K tile -> sK[key][d], V tile -> sV[key][d]
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + NTH * i, kk = c / CH, key = kk % BN, dc = c % CH;
            fh_half *sK = ap_lds + (buf * KS + kk / BN) * TILE, *sV = sK + KBUF;
            if constexpr (SPLIT) {
                const float kx[8] = {kraw[2 * i].x, kraw[2 * i].y, kraw[2 * i].z, kraw[2 * i].w,
                                     kraw[2 * i + 1].x, kraw[2 * i + 1].y, kraw[2 * i + 1].z, kraw[2 * i + 1].w};
                fh_half hi[8], lo[8];
                ap_split8(kx, hi, lo);
                uint4 uh, ul;
                __builtin_memcpy(&uh, hi, 16);
                __builtin_memcpy(&ul, lo, 16);
                *(uint4 *)(sK + key * KS_ + 8 * dc) = uh;
                *(uint4 *)(sK + BN * KS_ + key * KS_ + 8 * dc) = ul;
                const float vx[8] = {vraw[2 * i].x, vraw[2 * i].y, vraw[2 * i].z, vraw[2 * i].w,
                                     vraw[2 * i + 1].x, vraw[2 * i + 1].y, vraw[2 * i + 1].z, vraw[2 * i + 1].w};
                ap_split8(vx, hi, lo);
                __builtin_memcpy(&uh, hi, 16);
                __builtin_memcpy(&ul, lo, 16);
                *(uint4 *)(sV + key * VS + 8 * dc) = uh;
                *(uint4 *)(sV + BN * VS + key * VS + 8 * dc) = ul;
            } else {
                *(uint4 *)(sK + key * KS_ + 8 * dc) = kreg[i];
                *(uint4 *)(sV + key * VS + 8 * dc) = vreg[i];
            }
        }
    };
    // V^T operand addressing: the 16 lanes of a group supply keys (8 g + s / 4) and dims (16 * (group & 1) + 4 * (s % 4))
    // .. +3 and receive dim 16 * (group & 1) + s of keys 8 g .. 8 g + 3
    const int vt_off = (8 * g + ((lane & 15) >> 2)) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    // The Q loads must have landed before the loop: a wait for them inside the loop would also wait, every tile, for
    // the KV loads issued after them (the memory counter is in order).
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
        asm volatile("" ::"v"(qf[ks]));
        if constexpr (SPLIT) asm volatile("" ::"v"(ql[ks]));
    }
    const int lim = causal ? (qi + off < skv - 1 ? qi + off : skv - 1) : skv - 1; // this query's last visible key
    if (kend > 0) {
        fetch(0);
        stash(0);
        if (KS * BN < kend) fetch(KS * BN);
    }
    __syncthreads();

    const float ninf = -INFINITY;
    for (int ts = 0, it = 0; ts < kend; ts += KS * BN, it++) { // a step: KS tiles, one per group of four wavefronts
        const int t0 = ts + kset * BN;
        // a group without a tile in the last step multiplies the staged rows (clamped, finite) with every key masked
        const int lim_t = (KS == 1 || t0 < kend) ? lim : -1;
        const fh_half *sK = ap_lds + ((it & 1) * KS + kset) * TILE, *sV = sK + KBUF;
        // ---- S^T = K . Q^T for the two 32-key halves of the tile
        floatx16 st[2];
#pragma unroll
        for (int r = 0; r < 16; r++) st[0][r] = st[1][r] = 0.f;
        if constexpr (!SPLIT) {
            // product i: key half i % 2, d step i / 2; the K operands are requested eight products ahead
            const fh_half *ap = sK + prow * KS_ + 8 * g;
            constexpr int NI = 2 * KSTEPS, AHEAD = 8;
            half8 ka[AHEAD];
#pragma unroll
            for (int i = 0; i < AHEAD; i++) ka[i] = *(const half8 *)(ap + (i & 1) * 32 * KS_ + 16 * (i >> 1));
#pragma unroll
            for (int i = 0; i < NI; i++) {
                st[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[i % AHEAD], qf[i >> 1], st[i & 1], 0, 0, 0);
                if (i + AHEAD < NI) ka[i % AHEAD] = *(const half8 *)(ap + (i & 1) * 32 * KS_ + 16 * ((i + AHEAD) >> 1));
            }
            __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
            for (int i = 0; i < NI - AHEAD; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
        } else {
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
                const fh_half *ap = sK + (kt * 32 + prow) * KS_ + 8 * g;
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ks++) {
                    const half8 a = *(const half8 *)(ap + 16 * ks);
                    st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], st[kt], 0, 0, 0);
                    const half8 al = *(const half8 *)(ap + BN * KS_ + 16 * ks);
                    st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, qf[ks], st[kt], 0, 0, 0);
                    st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ql[ks], st[kt], 0, 0, 0);
                }
            }
        }
        // ---- tile t+1 goes into the other buffer (last read before the barrier that ended the previous tile) and
        // tile t+2 is requested: the LDS writes and the loads run under the softmax arithmetic
        // (the scheduler may not mix the stages: the operands prefetched for one product and the tile in flight would
        // otherwise be live together with the scores)
        __builtin_amdgcn_sched_barrier(0);
        if (ts + KS * BN < kend) stash((it + 1) & 1);
        if (ts + 2 * KS * BN < kend) fetch(ts + 2 * KS * BN);
        __builtin_amdgcn_sched_barrier(0);
        // ---- mask, running max: register r of half kt is key t0 + 32 kt + 16 (r / 8) + 8 g + r % 8
        // Only a tile that reaches past some query's last visible key pays for the compares (one branch for the
        // wavefront); the select works in place, so the common path has no register copies at the join.
        if (__any(t0 + BN - 1 > lim_t)) {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = t0 + 32 * kt + 16 * (r >> 3) + 8 * g + (r & 7);
                    asm volatile("v_cmp_le_i32 vcc, %1, %2\n\tv_cndmask_b32 %0, %3, %0, vcc"
                                 : "+v"(st[kt][r])
                                 : "v"(key), "v"(lim_t), "v"(ninf)
                                 : "vcc");
                }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[kt][r]);
        // the scale (> 0) is applied inside the exponent: p = 2^(s * sc2 - m), one multiply-add per score
        mx = ap_swap32_max(mx) * sc2;
        const float m_new = fmaxf(m_run, mx);
        const bool dead = m_new == -INFINITY; // nothing visible yet (only queries past the end)
        const float alpha = dead ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
        const float m_sub = dead ? 0.f : -m_new; // dead rows: 2^(-inf - 0) = 0
        float ps = 0.f;
        half8 pb[2][2], pl[SPLIT ? 2 : 1][2];
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                fh_half t[8], tl[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(st[kt][8 * s2 + e], sc2, m_sub)); // arguments <= 0
                    ps += p;
                    t[e] = (fh_half)p;
                    if constexpr (SPLIT) tl[e] = (fh_half)(p - (float)t[e]);
                }
                __builtin_memcpy(&pb[kt][s2], t, 16);
                if constexpr (SPLIT) __builtin_memcpy(&pl[kt][s2], tl, 16);
            }
        l_run = l_run * alpha + ap_swap32_sum(ps);
        m_run = m_new;
        // ---- O^T = O^T * alpha + V^T . P^T (once the maxima have settled no lane of the wavefront rescales)
        __builtin_amdgcn_sched_barrier(0);
        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[dt][r] *= alpha;
        }
        if constexpr (!SPLIT) {
            // product j: d tile j % DT, key step j / DT (= 2 kt + s2): consecutive products go to different
            // accumulators; the V^T operand is requested eight products ahead
            const fh_half *vp = sV + vt_off;
            constexpr int NJ = 4 * DT, AHEAD = 8;
            half8 va[AHEAD];
#pragma unroll
            for (int j = 0; j < AHEAD; j++) va[j] = ap_vt8(vp + 32 * (j % DT) + 16 * (j / DT) * VS, VS);
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int c = j / DT;
                acc[j % DT] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[j % AHEAD], pb[c >> 1][c & 1], acc[j % DT], 0, 0, 0);
                if (j + AHEAD < NJ) va[j % AHEAD] = ap_vt8(vp + 32 * ((j + AHEAD) % DT) + 16 * ((j + AHEAD) / DT) * VS, VS);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
            for (int j = 0; j < NJ - AHEAD; j++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
        } else {
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                const fh_half *vp = sV + vt_off + 32 * dt;
#pragma unroll
                for (int kt = 0; kt < 2; kt++)
#pragma unroll
                    for (int s2 = 0; s2 < 2; s2++) {
                        const half8 a = ap_vt8(vp + (32 * kt + 16 * s2) * VS, VS);
                        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[kt][s2], acc[dt], 0, 0, 0);
                        const half8 al = ap_vt8(vp + BN * VS + (32 * kt + 16 * s2) * VS, VS);
                        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, pb[kt][s2], acc[dt], 0, 0, 0);
                        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pl[kt][s2], acc[dt], 0, 0, 0);
                    }
            }
        }
        __syncthreads(); // tile t+1 is staged, and nobody reads this tile's buffer any more
    }
    if constexpr (KS == 2) {
        // ---- the second group hands its statistics and output over: [value][query wavefront][lane] floats in the
        // tile buffers (the barrier that ended the last step has passed: nobody reads them any more)
        float *sm = (float *)ap_lds;
        constexpr int NQ = 64 * QW;
        const int slot = (wave % QW) * 64 + lane;
        if (kset == 1) {
            sm[slot] = m_run;
            sm[NQ + slot] = l_run;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) sm[(2 + dt * 16 + r) * NQ + slot] = acc[dt][r];
        }
        __syncthreads();
        if (kset == 1) return;
        const float m1 = sm[slot], l1 = sm[NQ + slot];
        const float mm = fmaxf(m_run, m1), ref = mm == -INFINITY ? 0.f : mm;
        const float f0 = __builtin_amdgcn_exp2f(m_run - ref), f1 = __builtin_amdgcn_exp2f(m1 - ref);
        l_run = l_run * f0 + l1 * f1;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[dt][r] = acc[dt][r] * f0 + sm[(2 + dt * 16 + r) * NQ + slot] * f1;
    }
    // ---- store: lane = query, register r of d-tile dt is d = 32 dt + 8 (r / 4) + 4 g + r % 4
    if (qi < sq) {
        const float inv = 1.0f / l_run;
        TQ *op = out + (((int64_t)bi * hq + h) * sq + qi) * D;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++)
                ap_store4(op + 32 * dt + 8 * r4 + 4 * g, acc[dt][4 * r4] * inv, acc[dt][4 * r4 + 1] * inv,
                          acc[dt][4 * r4 + 2] * inv, acc[dt][4 * r4 + 3] * inv);
    }
}

template <typename TQ, typename TKV, int D, bool SPLIT, int HW, int KS = 1, int QW = 4>
static fh_status ap_launch_k(fh_device *dev, const void *q, int64_t q_sb, int64_t q_sh, int64_t q_st, const void *k,
                             const void *v, int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int sq,
                             int skv, float scale, int causal, void *out) {
    constexpr int LDS = 2 * KS * (SPLIT ? 2 : 1) * 64 * (D + 8 + D + 16) * 2; // two buffers of KS tiles (K and V planes), bytes
    static_assert(KS == 1 || LDS >= (2 + (D / 32) * 16) * 256 * 4, "the merge of the key groups reuses the tile buffers");
    static_assert(LDS <= 160 * 1024, "KV tiles exceed the LDS of a compute unit");
    auto kern = k_attn_prefill<TQ, TKV, D, SPLIT, HW, KS, QW>;
    FH_TRY(fh_kernel_lds(dev, (const void *)kern, LDS)); // allow more than 64 KB of dynamic LDS
    dim3 grid((unsigned)(hq / HW), (unsigned)((sq + 32 * QW - 1) / (32 * QW)), (unsigned)b);
    kern<<<grid, 64 * QW * HW * KS, LDS, dev->stream>>>((const TQ *)q, q_sb, q_sh, q_st, (const TKV *)k, (const TKV *)v, kv_sb,
                                               kv_sh, kv_st, hq, hkv, sq, skv, scale, causal, (TQ *)out);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

template <typename TQ, typename TKV, bool SPLIT = false>
static fh_status ap_launch(fh_device *dev, const void *q, int64_t q_sb, int64_t q_sh, int64_t q_st, const void *k,
                           const void *v, int64_t kv_sb, int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int sq,
                           int skv, int d, float scale, int causal, void *out) {
    // Two heads of one KV group share the staged tiles when the launch still has enough workgroups without the
    // split: short prompts are bound by the longest workgroup and by how many compute units have one at all.
    const long wgs = (long)hq * ((sq + 127) / 128) * b;
    // attn_kernel = 6 / 7 / 8 / 9 force the workgroup shape (two heads / two key groups / plain / 64-row query blocks
    // with two key groups) whatever the size: tests
    const int64_t force = dev->opt_attn_kernel;
    const bool pair = (hq / hkv) % 2 == 0 && (force == 6 || (force != 7 && force != 8 && wgs >= 1024));
#define FH_AP(D, HW, KS) ap_launch_k<TQ, TKV, D, SPLIT, HW, KS>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, scale, causal, out)
    if constexpr (!SPLIT) {
        // short prompts: every workgroup is resident at once (two of four wavefronts per compute unit) and the launch
        // lasts as long as the last query block's - its key tiles are shared out over two groups of wavefronts
        const bool halves = force == 7 || force == 9 || (force != 6 && force != 8 && wgs <= 2L * dev->compute_units && skv > 128);
        // shorter still: query blocks of 64 rows, four wavefronts, while one workgroup per compute unit holds (nearly) all
        // of them - a SIMD then runs one wavefront's chain of a step instead of two (512 tokens: 15.0 against 16.8 us)
        const long wgs64 = (long)hq * ((sq + 63) / 64) * b;
        const bool rows64 = force == 9 || (force == 0 && halves && 4 * wgs64 <= 5L * dev->compute_units);
        if (rows64) return d == 128 ? ap_launch_k<TQ, TKV, 128, SPLIT, 1, 2, 2>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, scale, causal, out)
                                    : ap_launch_k<TQ, TKV, 64, SPLIT, 1, 2, 2>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, scale, causal, out);
        if (halves) return d == 128 ? FH_AP(128, 1, 2) : FH_AP(64, 1, 2);
    }
    if (d == 128) return pair ? FH_AP(128, 2, 1) : FH_AP(128, 1, 1);
    return pair ? FH_AP(64, 2, 1) : FH_AP(64, 1, 1);
#undef FH_AP
}

// FH_ERR_UNSUPPORTED when the shape is not one this kernel is written for (the caller keeps the generic kernel).
fh_status fh_attention_prefill_mfma(fh_device *dev, int q_dtype, int kv_dtype, const void *q, int64_t q_sb,
                                    int64_t q_sh, int64_t q_st, const void *k, const void *v, int64_t kv_sb,
                                    int64_t kv_sh, int64_t kv_st, int b, int hq, int hkv, int sq, int skv, int d,
                                    float scale, int mask_kind, void *out) {
    if ((d != 128 && d != 64) || hq % hkv || (mask_kind != FH_MASK_NONE && mask_kind != FH_MASK_CAUSAL)) return FH_ERR_UNSUPPORTED;
    if (q_st % 8 || q_sh % 8 || q_sb % 8 || kv_st % 8 || kv_sh % 8 || kv_sb % 8 || (sq + 127) / 128 > 65535 || b > 65535) return FH_ERR_UNSUPPORTED;
    if (mask_kind == FH_MASK_CAUSAL && skv < sq) return FH_ERR_UNSUPPORTED;
    const int causal = mask_kind == FH_MASK_CAUSAL;
    if (q_dtype == FH_F16 && kv_dtype == FH_F16)
        return ap_launch<fh_half, fh_half>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, d, scale, causal, out);
    if (q_dtype == FH_F32 && kv_dtype == FH_F16)
        return ap_launch<float, fh_half>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, d, scale, causal, out);
    if (q_dtype == FH_F32 && kv_dtype == FH_F32 && dev->opt_attn_kernel != 2) // all f32: split operands, f32 accuracy
        return ap_launch<float, float, true>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, d, scale, causal, out);
    if (q_dtype == FH_F32 && kv_dtype == FH_F32)
        return ap_launch<float, float>(dev, q, q_sb, q_sh, q_st, k, v, kv_sb, kv_sh, kv_st, b, hq, hkv, sq, skv, d, scale, causal, out);
    return FH_ERR_UNSUPPORTED;
}

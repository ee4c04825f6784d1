// Batch-1 HLQ bit-serial LUT GEMV for gfx950 (MI355X), replacing
// MultiThread_arm_gemv_w_lowbit_activation_fp_impl (C++/ops/src/arm/arm_gemm.cpp:312-360)
// and t_mac_g4_float_update_impl (C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469).
//
//   y[n] = sum_g ( z[n,g] * sum_{k in g} x[k]  +  sum_b s[b,n,g] * sum_{k in g} B_b[n,k] x[k] ) + bias[n]
//
// Design (memory bound: 0.30 B per weight at w2g128, so the budget is ~0.8 VALU
// lane-ops per plane bit at 6 TB/s):
//  * lane = output column, wave = 64 columns; every lane of a wave instruction looks up
//    the same 4-activation chunk, so all 64 LDS reads fall in one 64-byte table and are
//    conflict free (broadcast), and the per-column sums need no cross-lane reduction;
//  * the activation tables hold the 16 subset sums of each chunk as int32 fixed point
//    with a per-unit power-of-two scale chosen from max|x| of the unit: sums are exact
//    integers (no LUT rounding unless |x_k| < 2^-13 max|x|, then <= 2^-24 max|x|), two
//    lookups retire with one v_add3_u32;
//  * the plane dwords are stored rotated so that `byte & 0x3C` is already the byte offset
//    into the table; one SDWA v_and per lookup writes that offset into byte 0 of a
//    register whose upper bytes keep the table base (dst_unused:UNUSED_PRESERVE), the
//    chunk index rides in the ds_read immediate;
//  * a workgroup owns one column block and a slice of K, builds only that slice's
//    tables, its waves split the slice; slices are combined through a workspace by the
//    last workgroup to arrive (fixed summation order, so results are deterministic).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"

namespace {

constexpr int TBL_BYTES = 64;                    // 16 int32 entries
constexpr int UNIT_LUT_BYTES = 32 * TBL_BYTES;   // 32 chunks per unit

struct GemvArgs {
    const uint4 *planes;
    const uint32_t *scales;
    const uint32_t *zeros;
    const uint16_t *bias;    // fp16 or null
    const uint16_t *x;       // fp16 [K]
    uint16_t *y;             // fp16 [N]
    float *partial;          // [ksplit][ncb*64]   (ksplit > 1)
    unsigned *counters;      // [ncb], zero between calls
    int N, U, NT, ncb;
    int ksplit, tps;         // slices per column block, tasks per slice
};

typedef __attribute__((address_space(3))) const int lds_cint;

__device__ __forceinline__ int lds_ld(uint32_t addr, int imm)
{
    return *(lds_cint *)(uintptr_t)(addr + (uint32_t)imm);
}

__device__ __forceinline__ float h2f_lo(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v & 0xffffu)); }
__device__ __forceinline__ float h2f_hi(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v >> 16)); }

// a.byte0 = mask & src.byte<SEL>; bytes 1..3 of `a` are kept (they hold the table base).
#define HLQ_SDWA_AND(a, mask, src, SEL)                                                        \
    asm("v_and_b32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD "  \
        "src1_sel:BYTE_" #SEL                                                                  \
        : "+v"(a)                                                                              \
        : "v"(mask), "v"(src))

// Eight lookups for one plane dword (32 k): chunks 8*D .. 8*D+7 of the unit.
template <int D>
__device__ __forceinline__ int lookup_dword(uint32_t w, uint32_t (&a)[8], uint32_t mask, int acc)
{
    const uint32_t r = __builtin_amdgcn_alignbit(w, w, 4);
    HLQ_SDWA_AND(a[0], mask, w, 0);
    HLQ_SDWA_AND(a[1], mask, r, 0);
    HLQ_SDWA_AND(a[2], mask, w, 1);
    HLQ_SDWA_AND(a[3], mask, r, 1);
    HLQ_SDWA_AND(a[4], mask, w, 2);
    HLQ_SDWA_AND(a[5], mask, r, 2);
    HLQ_SDWA_AND(a[6], mask, w, 3);
    HLQ_SDWA_AND(a[7], mask, r, 3);
    constexpr int base = D * 8 * TBL_BYTES;
    const int v0 = lds_ld(a[0], base + 0 * TBL_BYTES);
    const int v1 = lds_ld(a[1], base + 1 * TBL_BYTES);
    const int v2 = lds_ld(a[2], base + 2 * TBL_BYTES);
    const int v3 = lds_ld(a[3], base + 3 * TBL_BYTES);
    const int v4 = lds_ld(a[4], base + 4 * TBL_BYTES);
    const int v5 = lds_ld(a[5], base + 5 * TBL_BYTES);
    const int v6 = lds_ld(a[6], base + 6 * TBL_BYTES);
    const int v7 = lds_ld(a[7], base + 7 * TBL_BYTES);
    acc = acc + v0 + v1;
    acc = acc + v2 + v3;
    acc = acc + v4 + v5;
    acc = acc + v6 + v7;
    return acc;
}

template <int BITS, bool G64>
struct Task {
    static constexpr int UPT = G64 ? 1 : 2;
    uint4 w[UPT][BITS];
    uint32_t sc[BITS];
    uint32_t zz;
};

template <int BITS, bool G64>
__device__ __forceinline__ void load_task(Task<BITS, G64> &t, const GemvArgs &a, int cb, int task, int lane)
{
    constexpr int UPT = Task<BITS, G64>::UPT;
#pragma unroll
    for (int ul = 0; ul < UPT; ul++) {
        const int u = task * UPT + ul;
        if (u < a.U) {
            const uint4 *p = a.planes + (((size_t)cb * a.U + u) * BITS) * HLQ_CB + lane;
#pragma unroll
            for (int b = 0; b < BITS; b++) t.w[ul][b] = p[b * HLQ_CB];
        } else {
#pragma unroll
            for (int b = 0; b < BITS; b++) t.w[ul][b] = make_uint4(0, 0, 0, 0);
        }
    }
    const size_t m = (size_t)cb * a.NT + task;
#pragma unroll
    for (int b = 0; b < BITS; b++) t.sc[b] = a.scales[(m * BITS + b) * HLQ_CB + lane];
    t.zz = a.zeros[m * HLQ_CB + lane];
}

// One unit (128 k of 64 columns, all planes).  `lu` = unit index inside the slice.
template <int BITS, bool G64, int HALF>
__device__ __forceinline__ float process_unit(const uint4 (&w)[BITS], const uint32_t (&sc)[BITS], uint32_t zz,
                                              int lu, uint32_t lut_base, const float *xs, const float *invs,
                                              uint32_t mask, float acc)
{
    uint32_t a[8];
    const uint32_t ub = lut_base + (uint32_t)lu * UNIT_LUT_BYTES;
#pragma unroll
    for (int j = 0; j < 8; j++) a[j] = ub;
    const float inv = invs[lu];
    if (G64) {
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int b = 0; b < BITS; b++) {
            int i0 = lookup_dword<0>(w[b].x, a, mask, 0);
            i0 = lookup_dword<1>(w[b].y, a, mask, i0);
            int i1 = lookup_dword<2>(w[b].z, a, mask, 0);
            i1 = lookup_dword<3>(w[b].w, a, mask, i1);
            p0 = fmaf((float)i0, h2f_lo(sc[b]), p0);
            p1 = fmaf((float)i1, h2f_hi(sc[b]), p1);
        }
        acc = fmaf(inv, p0 + p1, acc);
        acc = fmaf(h2f_lo(zz), xs[2 * lu], acc);
        acc = fmaf(h2f_hi(zz), xs[2 * lu + 1], acc);
    } else {
        float p = 0.f;
#pragma unroll
        for (int b = 0; b < BITS; b++) {
            int i0 = lookup_dword<0>(w[b].x, a, mask, 0);
            i0 = lookup_dword<1>(w[b].y, a, mask, i0);
            i0 = lookup_dword<2>(w[b].z, a, mask, i0);
            i0 = lookup_dword<3>(w[b].w, a, mask, i0);
            p = fmaf((float)i0, HALF ? h2f_hi(sc[b]) : h2f_lo(sc[b]), p);
        }
        acc = fmaf(inv, p, acc);
        acc = fmaf(HALF ? h2f_hi(zz) : h2f_lo(zz), xs[lu], acc);
    }
    return acc;
}

// Subset-sum tables of the slice's units, as int32 fixed point; xs = group sums of x
// (fp32), invs = 2^-p per unit.  32 consecutive threads build one unit.
template <bool G64>
__device__ __forceinline__ void build_luts(const uint16_t *x, int u0, int nU, unsigned char *lut, float *xs,
                                           float *invs, int tid, int nthreads)
{
    const int nchunks = nU * 32;
    for (int ci = tid; ci < nchunks; ci += nthreads) {
        const int lu = ci >> 5, c = ci & 31;
        const uint2 raw = *(const uint2 *)(x + (size_t)(u0 + lu) * HLQ_UNIT + c * 4);
        const float x0 = h2f_lo(raw.x), x1 = h2f_hi(raw.x), x2 = h2f_lo(raw.y), x3 = h2f_hi(raw.y);
        float amax = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3)));
        float s = (x0 + x1) + (x2 + x3);
#pragma unroll
        for (int o = 1; o <= 8; o <<= 1) {
            s += __shfl_xor(s, o, 32);
            amax = fmaxf(amax, __shfl_xor(amax, o, 32));
        }
        const float s16 = s;
        s += __shfl_xor(s, 16, 32);
        amax = fmaxf(amax, __shfl_xor(amax, 16, 32));
        // amax < 2^(eb-126): scale by 2^(149-eb) so |x * scale| < 2^23, a 4-subset < 2^25,
        // 32 lookups < 2^30.
        const uint32_t eb = (__float_as_uint(amax) >> 23) & 0xffu;
        const float scale = eb ? __uint_as_float((276u - eb) << 23) : 1.0f;
        const float inv = eb ? __uint_as_float((eb - 22u) << 23) : 1.0f;
        const int i0 = __float2int_rn(x0 * scale), i1 = __float2int_rn(x1 * scale);
        const int i2 = __float2int_rn(x2 * scale), i3 = __float2int_rn(x3 * scale);
        const int e3 = i0 + i1, e5 = i0 + i2, e6 = i1 + i2, e7 = e3 + i2;
        int4 *dst = (int4 *)(lut + (size_t)ci * TBL_BYTES);
        dst[0] = make_int4(0, i0, i1, e3);
        dst[1] = make_int4(i2, e5, e6, e7);
        dst[2] = make_int4(i3, i3 + i0, i3 + i1, i3 + e3);
        dst[3] = make_int4(i3 + i2, i3 + e5, i3 + e6, i3 + e7);
        if (c == 0) invs[lu] = inv;
        if (G64) {
            if ((c & 15) == 0) xs[2 * lu + (c >> 4)] = s16;
        } else {
            if (c == 0) xs[lu] = s;
        }
    }
}

template <int BITS, bool G64>
__global__ __launch_bounds__(1024) void hlq_gemv_kernel(const GemvArgs a)
{
    extern __shared__ __align__(256) unsigned char smem[];
    constexpr int UPT = G64 ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const int cb = blockIdx.x / a.ksplit, slice = blockIdx.x - cb * a.ksplit;
    const int t0 = slice * a.tps, t1 = min(t0 + a.tps, a.NT);
    const int u0 = t0 * UPT, nU = min(t1 * UPT, a.U) - u0;
    const int maxU = a.tps * UPT;

    unsigned char *lut = smem;
    float *xs = (float *)(smem + (size_t)maxU * UNIT_LUT_BYTES);   // [maxU * (G64 ? 2 : 1)]
    float *invs = xs + maxU * 2;                                     // [maxU]
    float *red = invs + maxU;                                        // [nw][64]
    int *flag = (int *)(red + nw * HLQ_CB);
    const uint32_t lut_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lut;

    // Issue the first task's loads before the tables are built: HBM latency overlaps the build.
    Task<BITS, G64> cur;
    int t = t0 + wave;
    bool have = t < t1;
    if (have) load_task<BITS, G64>(cur, a, cb, t, lane);

    build_luts<G64>(a.x, u0, nU, lut, xs, invs, tid, blockDim.x);
    __syncthreads();

    const uint32_t mask = 0x3Cu;
    float acc = 0.f;
    while (have) {
        const int tn = t + nw;
        const bool hn = tn < t1;
        Task<BITS, G64> nxt;
        if (hn) load_task<BITS, G64>(nxt, a, cb, tn, lane);
        const int lu = (t - t0) * UPT;
        acc = process_unit<BITS, G64, 0>(cur.w[0], cur.sc, cur.zz, lu, lut_base, xs, invs, mask, acc);
        if (!G64) {
            if (t * UPT + 1 < a.U)
                acc = process_unit<BITS, G64, 1>(cur.w[UPT - 1], cur.sc, cur.zz, lu + 1, lut_base, xs, invs, mask, acc);
        }
        if (hn) cur = nxt;
        t = tn;
        have = hn;
    }

    // Combine the waves of this workgroup, then the slices of this column block.
    red[wave * HLQ_CB + lane] = acc;
    __syncthreads();
    const int n = cb * HLQ_CB + lane;
    float total = 0.f;
    if (wave == 0) {
        for (int w = 0; w < nw; w++) total += red[w * HLQ_CB + lane];
    }
    if (a.ksplit == 1) {
        if (wave == 0 && n < a.N) {
            if (a.bias) total += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
        }
        return;
    }
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    if (wave == 0) {
        a.partial[(size_t)slice * npad + n] = total;
        __threadfence();
    }
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(&a.counters[cb], 1u);
        *flag = (ticket == (unsigned)a.ksplit - 1u);
    }
    __syncthreads();
    if (*flag && wave == 0) {
        __threadfence();
        float sum = 0.f;
        for (int s = 0; s < a.ksplit; s++) sum += __builtin_nontemporal_load(&a.partial[(size_t)s * npad + n]);
        if (n < a.N) {
            if (a.bias) sum += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)sum);
        }
        if (lane == 0) a.counters[cb] = 0u;
    }
}

size_t gemv_lds_bytes(int tps, int upt, int waves)
{
    const int maxU = tps * upt;
    return (size_t)maxU * UNIT_LUT_BYTES + (size_t)maxU * 3 * sizeof(float) + (size_t)waves * HLQ_CB * sizeof(float) + 16;
}

template <int BITS, bool G64>
int launch_gemv(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    auto kern = hlq_gemv_kernel<BITS, G64>;
    if (lds > 64 * 1024) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return ELUTQ_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, dim3(a.ncb * a.ksplit), dim3(waves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

int dispatch_gemv(const GemvArgs &a, int bits, int group, int waves, size_t lds, hipStream_t stream)
{
    const bool g64 = group == 64;
    switch (bits) {
    case 1: return g64 ? launch_gemv<1, true>(a, waves, lds, stream) : launch_gemv<1, false>(a, waves, lds, stream);
    case 2: return g64 ? launch_gemv<2, true>(a, waves, lds, stream) : launch_gemv<2, false>(a, waves, lds, stream);
    case 3: return g64 ? launch_gemv<3, true>(a, waves, lds, stream) : launch_gemv<3, false>(a, waves, lds, stream);
    case 4: return g64 ? launch_gemv<4, true>(a, waves, lds, stream) : launch_gemv<4, false>(a, waves, lds, stream);
    }
    return ELUTQ_ERR_BITS;
}

int check_shape(int K, int N, int bits, int group)
{
    if (bits < 1 || bits > 4) return ELUTQ_ERR_BITS;
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (K < HLQ_UNIT || N < 1 || K % HLQ_UNIT != 0 || K % group != 0) return ELUTQ_ERR_SHAPE;
    return ELUTQ_OK;
}

constexpr int MAX_LDS = 160 * 1024;
constexpr int WS_COUNTER_BYTES = 64 * 1024;   // one arrival counter per column block, N <= 2^20
constexpr int NUM_CU = 256;

// Launch shape: enough workgroups to cover every CU a few times over, slices no
// smaller than one task per wave.
void choose_shape(const HlqGeo &g, int &ksplit, int &waves)
{
    if (waves <= 0) waves = 4;
    if (ksplit <= 0) {
        const int want = (4 * NUM_CU + g.ncb - 1) / g.ncb;              // slices for ~4 workgroups per CU
        const int most = (g.NT + waves - 1) / waves;                    // at least one task per wave
        ksplit = want < 1 ? 1 : want;
        if (ksplit > most) ksplit = most;
        if (ksplit < 1) ksplit = 1;
    }
}

}  // namespace

extern "C" {

size_t elutq_hlq_workspace_bytes(int K, int N, int bits, int group, int M)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK || M < 1) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    // arrival counters (fixed region, so layers of any shape can share one workspace) +
    // partial sums for the finest split (one task per slice)
    return (size_t)WS_COUNTER_BYTES + (size_t)g.NT * g.ncb * HLQ_CB * sizeof(float);
}

int elutq_hlq_workspace_init(void *d_workspace, size_t workspace_bytes, void *stream)
{
    if (!d_workspace) return ELUTQ_ERR_NULL;
    return hipMemsetAsync(d_workspace, 0, workspace_bytes, (hipStream_t)stream) == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

int elutq_hlq_gemv_f16_tuned(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                             const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                             size_t workspace_bytes, void *stream, int ksplit, int waves)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.NT) return ELUTQ_ERR_TUNING;
    choose_shape(g, ksplit, waves);
    int tps = (g.NT + ksplit - 1) / ksplit;
    // shrink the slice count so that no slice is empty, and the slice so its tables fit in LDS
    while (gemv_lds_bytes(tps, g.UPT, waves) > (size_t)MAX_LDS) tps = (tps + 1) / 2;
    ksplit = (g.NT + tps - 1) / tps;

    GemvArgs a;
    a.planes = (const uint4 *)d_planes;
    a.scales = (const uint32_t *)d_scales;
    a.zeros = (const uint32_t *)d_zeros;
    a.bias = (const uint16_t *)d_bias;
    a.x = (const uint16_t *)d_x;
    a.y = (uint16_t *)d_y;
    a.N = N; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb;
    a.ksplit = ksplit; a.tps = tps;
    a.partial = nullptr; a.counters = nullptr;
    if (ksplit > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ksplit * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        a.counters = (unsigned *)d_workspace;
        a.partial = (float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
    }
    return dispatch_gemv(a, bits, group, waves, gemv_lds_bytes(tps, g.UPT, waves), (hipStream_t)stream);
}

int elutq_hlq_gemv_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                       const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                       size_t workspace_bytes, void *stream)
{
    return elutq_hlq_gemv_f16_tuned(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                                    workspace_bytes, stream, 0, 0);
}

}  // extern "C"

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

constexpr int MAX_LDS = HLQ_MAX_LDS;
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
    int ksplit, ups;         // slices per column block, units per slice
    // optional fusion with the ops around the projection in a decoder layer
    int prologue;            // 0: x as is; 1: rmsnorm(x) * norm_w; 2: silu(x[0:K]) * x[K:2K]
    float eps;
    const uint16_t *norm_w;  // fp16 [K]      (prologue 1)
    const uint16_t *residual;  // fp16 [N] added to the output, or null
};

#ifdef HLQ_TIMING
// Profiling builds only: per-stage wall-clock stamps (100 MHz) of wave 0 of every workgroup.
__device__ unsigned long long *g_hlq_stamps = nullptr;
#define HLQ_STAMP(i)                                                                              \
    do {                                                                                          \
        if (g_hlq_stamps && threadIdx.x == 0) g_hlq_stamps[(size_t)blockIdx.x * 8 + (i)] = wall_clock64(); \
    } while (0)
#else
#define HLQ_STAMP(i) do { } while (0)
#endif

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

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// A sub-task is one unit of one plane: 128 k of 64 columns = one dwordx4 per lane, plus the
// meta dword(s) that scale it.
struct Sub {
    uint4 w;
    uint32_t sc;   // fp16 scales of the group pair this unit belongs to (this plane)
    uint32_t zz;   // fp16 zeros of the pair; loaded for plane 0 only, which folds the zero point
};

template <int BITS, bool G64>
__device__ __forceinline__ void load_sub(Sub &t, const GemvArgs &a, int cb, int u, int b, int lane)
{
    const u32x4 v = __builtin_nontemporal_load((const u32x4 *)(a.planes + (((size_t)cb * a.U + u) * BITS + b) * HLQ_CB + lane));
    t.w = make_uint4(v.x, v.y, v.z, v.w);
    const size_t m = (size_t)cb * a.NT + (G64 ? u : (u >> 1));
    t.sc = a.scales[(m * BITS + b) * HLQ_CB + lane];
    t.zz = 0;
    if (b == 0) t.zz = a.zeros[m * HLQ_CB + lane];
}

// The two 64-k halves of a unit have their own table scale (2^-p) and activation sum; at
// G = 64 they are also two quantization groups (lo / hi half of the meta dwords), at G = 128
// one group (the half of the meta dwords selected by the unit's parity).
template <bool G64>
__device__ __forceinline__ float process_sub(const Sub &t, int lu, int b, int odd, uint32_t lut_base,
                                             const float2 *xs_inv, uint32_t mask, float acc)
{
    uint32_t a[8];
    const uint32_t ub = lut_base + (uint32_t)lu * UNIT_LUT_BYTES;
#pragma unroll
    for (int j = 0; j < 8; j++) a[j] = ub;
    const float2 h0 = xs_inv[2 * lu], h1 = xs_inv[2 * lu + 1];      // .x = sum of x, .y = 2^-p
    int i0 = lookup_dword<0>(t.w.x, a, mask, 0);
    i0 = lookup_dword<1>(t.w.y, a, mask, i0);
    int i1 = lookup_dword<2>(t.w.z, a, mask, 0);
    i1 = lookup_dword<3>(t.w.w, a, mask, i1);
    const uint32_t sc = G64 ? t.sc : (odd ? (t.sc >> 16) * 0x10001u : (t.sc & 0xffffu) * 0x10001u);
    acc = fmaf((float)i0 * h0.y, h2f_lo(sc), acc);
    acc = fmaf((float)i1 * h1.y, h2f_hi(sc), acc);
    if (b == 0) {
        const uint32_t zz = G64 ? t.zz : (odd ? (t.zz >> 16) * 0x10001u : (t.zz & 0xffffu) * 0x10001u);
        acc = fmaf(h2f_lo(zz), h0.x, acc);
        acc = fmaf(h2f_hi(zz), h1.x, acc);
    }
    return acc;
}

// DPP lane exchanges inside a row of 16 lanes (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// all-reduce over the 16 lanes of a row: xor 1, xor 2 (quad_perm), then half-row and row mirrors
#define HLQ_ROW_REDUCE(v, OP)             \
    v = OP(v, dpp_f<0xB1>(v));            \
    v = OP(v, dpp_f<0x4E>(v));            \
    v = OP(v, dpp_f<0x141>(v));           \
    v = OP(v, dpp_f<0x140>(v))
__device__ __forceinline__ float op_add(float a, float b) { return a + b; }
__device__ __forceinline__ float op_max(float a, float b) { return fmaxf(a, b); }

// The four activations of a chunk after the optional prologue, as fp32 values that are
// exactly representable in fp16 (the fused ops round to fp16 where the unfused pipeline
// would have stored fp16: RMSNorm output, arm_rmsnorm.cpp:25-84; SiLU(gate)*up,
// arm_activation.cpp:36-49).
__device__ __forceinline__ void chunk_values(int prologue, uint2 raw, uint2 raw2, float rstd, float (&v)[4])
{
    v[0] = h2f_lo(raw.x); v[1] = h2f_hi(raw.x); v[2] = h2f_lo(raw.y); v[3] = h2f_hi(raw.y);
    if (prologue == 0) return;
    const float w[4] = {h2f_lo(raw2.x), h2f_hi(raw2.x), h2f_lo(raw2.y), h2f_hi(raw2.y)};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float t;
        if (prologue == 1) t = v[i] * rstd * w[i];
        else t = v[i] / (1.0f + __expf(-v[i])) * w[i];
        v[i] = (float)(_Float16)t;
    }
}

__device__ __forceinline__ void load_chunk(const GemvArgs &a, int K, size_t k, uint2 &raw, uint2 &raw2)
{
    raw = *(const uint2 *)(a.x + k);
    if (a.prologue == 1) raw2 = *(const uint2 *)(a.norm_w + k);
    else if (a.prologue == 2) raw2 = *(const uint2 *)(a.x + (size_t)K + k);
}

// Subset-sum tables of the slice's units as int32 fixed point.  One thread per chunk of
// 4 activations; the 16 threads of a DPP row cover one 64-k half unit, whose max|x| sets
// the power-of-two table scale and whose sum feeds the zero-point fold.  `raw`/`raw2` hold
// the chunk of the first pass (loaded by the caller ahead of the weight loads).
__device__ __forceinline__ void build_luts(const GemvArgs &a, int K, size_t k0, uint2 raw, uint2 raw2, float rstd,
                                           int nchunks, unsigned char *lut, float2 *xs_inv, int tid, int nthreads)
{
    for (int ci = tid; ci < nchunks; ci += nthreads) {
        if (ci != tid) load_chunk(a, K, k0 + (size_t)ci * 4, raw, raw2);
        float v[4];
        chunk_values(a.prologue, raw, raw2, rstd, v);
        const float x0 = v[0], x1 = v[1], x2 = v[2], x3 = v[3];
        float amax = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3)));
        float s = (x0 + x1) + (x2 + x3);
        HLQ_ROW_REDUCE(s, op_add);
        HLQ_ROW_REDUCE(amax, op_max);
        // amax < 2^(eb-126): scale by 2^(149-eb) so |x * scale| < 2^23, a 4-subset < 2^25 and
        // the 16 lookups of a half unit < 2^29.
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
        if ((ci & 15) == 0) xs_inv[ci >> 4] = make_float2(s, inv);
    }
}

// 1 / rms of the whole activation vector (every workgroup computes it for itself: 2K bytes
// from cache), for the fused RMSNorm prologue.  `red` is LDS scratch of >= 64 floats.
__device__ __forceinline__ float block_rstd(const GemvArgs &a, int K, float *red, int tid, int nthreads)
{
    float ssq = 0.f;
    for (int i = tid; i < K / 4; i += nthreads) {
        const uint2 r = *(const uint2 *)(a.x + (size_t)i * 4);
        const float x0 = h2f_lo(r.x), x1 = h2f_hi(r.x), x2 = h2f_lo(r.y), x3 = h2f_hi(r.y);
        ssq += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
    }
    HLQ_ROW_REDUCE(ssq, op_add);
    if ((tid & 15) == 0) red[tid >> 4] = ssq;
    __syncthreads();
    if (tid < 64) {
        float v = tid < (nthreads >> 4) ? red[tid] : 0.f;
        HLQ_ROW_REDUCE(v, op_add);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (tid == 0) red[64] = v;
    }
    __syncthreads();
    return rsqrtf(red[64] / (float)K + a.eps);
}

constexpr int DEPTH = 4;    // sub-tasks a wave keeps in flight

template <int BITS, bool G64>
__global__ __launch_bounds__(1024) void hlq_gemv_kernel(const GemvArgs a)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const int cb = blockIdx.x / a.ksplit, slice = blockIdx.x - cb * a.ksplit;
    const int u0 = slice * a.ups, nU = min(u0 + a.ups, a.U) - u0;
    const int nst = nU * BITS;                                             // sub-tasks of this workgroup

    unsigned char *lut = smem;
    float2 *xs_inv = (float2 *)(smem + (size_t)a.ups * UNIT_LUT_BYTES);   // [2 * ups]
    float *red = (float *)(xs_inv + 2 * a.ups);                            // [nw][64]
    const uint32_t lut_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lut;

    HLQ_STAMP(0);
    // Activations first (they are needed first and come from cache), then the weight
    // stream: its HBM latency overlaps the table build.
    const int K = a.U * HLQ_UNIT;
    const size_t k0 = (size_t)u0 * HLQ_UNIT;
    const int nchunks = nU * 32;
    uint2 raw = make_uint2(0, 0), raw2 = make_uint2(0, 0);
    if (tid < nchunks) load_chunk(a, K, k0 + (size_t)tid * 4, raw, raw2);

    Sub slot[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
        const int st = wave + d * nw;
        if (st < nst) load_sub<BITS, G64>(slot[d], a, cb, u0 + st / BITS, st % BITS, lane);
    }

    float rstd = 1.f;
    if (a.prologue == 1) rstd = block_rstd(a, K, red, tid, blockDim.x);
    build_luts(a, K, k0, raw, raw2, rstd, nchunks, lut, xs_inv, tid, blockDim.x);
    HLQ_STAMP(1);
    __syncthreads();
    HLQ_STAMP(2);

    const uint32_t mask = 0x3Cu;
    float acc = 0.f;
    for (int base = wave; base < nst; base += DEPTH * nw) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            const int st = base + d * nw;
            if (st < nst) {
                const int lu = st / BITS, b = st % BITS;
                acc = process_sub<G64>(slot[d], lu, b, (u0 + lu) & 1, lut_base, xs_inv, mask, acc);
                const int sn = st + DEPTH * nw;
                if (sn < nst) load_sub<BITS, G64>(slot[d], a, cb, u0 + sn / BITS, sn % BITS, lane);
            }
        }
    }

    HLQ_STAMP(3);
    // Combine the waves of this workgroup, then the slices of this column block.
    const int n = cb * HLQ_CB + lane;
    float total = acc;
    if (nw > 1) {
        red[wave * HLQ_CB + lane] = acc;
        __syncthreads();
        if (wave == 0) {
            total = 0.f;
            for (int w = 0; w < nw; w++) total += red[w * HLQ_CB + lane];
        }
    }
    HLQ_STAMP(4);
    if (a.ksplit == 1) {
        if (wave == 0 && n < a.N) {
            if (a.bias) total += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            if (a.residual) total += (float)__builtin_bit_cast(_Float16, a.residual[n]);
            a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
        }
        return;
    }
    // Slices meet through device memory.  Partial sums are written and read with
    // agent-scope atomics (they bypass the per-XCD L2s' non-coherent lines), the writer
    // waits for its stores to be acknowledged before it takes a ticket, and the reader's
    // loads depend on the ticket it drew -- so no cache write-back / invalidate is needed.
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    if (wave == 0) {
        __hip_atomic_store(&a.partial[(size_t)slice * npad + n], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        HLQ_STAMP(5);
        unsigned ticket = 0;
        if (lane == 0)
            ticket = __hip_atomic_fetch_add(&a.counters[cb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        HLQ_STAMP(6);
        if (ticket == (unsigned)a.ksplit - 1u) {
            // eight independent loads in flight at a time, summed in slice order
            float sum = 0.f;
            for (int s0 = 0; s0 < a.ksplit; s0 += 8) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int s = min(s0 + j, a.ksplit - 1);
                    v[j] = __hip_atomic_load(&a.partial[(size_t)s * npad + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (s0 + j < a.ksplit) sum += v[j];
            }
            if (n < a.N) {
                if (a.bias) sum += (float)__builtin_bit_cast(_Float16, a.bias[n]);
                if (a.residual) sum += (float)__builtin_bit_cast(_Float16, a.residual[n]);
                a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)sum);
            }
            if (lane == 0) __hip_atomic_store(&a.counters[cb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            HLQ_STAMP(7);
        }
    }
}

size_t gemv_lds_bytes(int ups, int waves)
{
    const int red = waves * HLQ_CB > 80 ? waves * HLQ_CB : 80;      // cross-wave sums; >= 65 floats for block_rstd
    return (size_t)ups * UNIT_LUT_BYTES + (size_t)ups * 2 * sizeof(float2) + (size_t)red * sizeof(float) + 16;
}

template <int BITS, bool G64>
int launch_gemv(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    auto kern = hlq_gemv_kernel<BITS, G64>;
    static bool big_lds_enabled = false;      // per template instance; the setting is sticky
    if (lds > 64 * 1024 && !big_lds_enabled) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS) != hipSuccess)
            return ELUTQ_ERR_HIP;
        big_lds_enabled = true;
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

constexpr int WS_COUNTER_BYTES = HLQ_WS_COUNTER_BYTES;   // one arrival counter per column block, N <= 2^20
constexpr int NUM_CU = HLQ_NUM_CU;

// Launch shape (measured on MI355X): about one workgroup per CU, as few K slices as that
// allows (every slice adds a trip through device memory to the tail of the kernel), and
// 16 waves per workgroup so that every SIMD has several waves to hide LDS latency with.
void choose_shape(const HlqGeo &g, int &ksplit, int &waves)
{
    if (ksplit <= 0) {
        ksplit = NUM_CU / g.ncb;
        if (ksplit > 4) ksplit = 4;
        if (ksplit < 1) ksplit = 1;
        if (ksplit > g.U) ksplit = g.U;
    }
    if (waves <= 0) waves = g.ncb * ksplit > 300 ? 8 : 16;
}

}  // namespace

extern "C" {

#ifdef HLQ_TIMING
int elutq_debug_set_stamps(void *d_buf)
{
    return hipMemcpyToSymbol(HIP_SYMBOL(g_hlq_stamps), &d_buf, sizeof(d_buf)) == hipSuccess ? 0 : -1;
}
#endif

size_t elutq_hlq_workspace_bytes(int K, int N, int bits, int group, int M)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK || M < 1) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    // arrival counters (fixed region, so layers of any shape can share one workspace) +
    // partial sums: GEMV at its finest split (one unit per slice), GEMM at the split it uses
    const size_t gemv = (size_t)WS_COUNTER_BYTES + (size_t)g.U * g.ncb * HLQ_CB * sizeof(float);
    const size_t gemm = M > 1 ? hlq_gemm_ws_bytes(g, M > 64 ? 64 : M) : 0;
    return gemv > gemm ? gemv : gemm;
}

int elutq_hlq_workspace_init(void *d_workspace, size_t workspace_bytes, void *stream)
{
    if (!d_workspace) return ELUTQ_ERR_NULL;
    return hipMemsetAsync(d_workspace, 0, workspace_bytes, (hipStream_t)stream) == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

int elutq_hlq_gemv_fused_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                             const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                             size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion, int ksplit,
                             int waves)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.U) return ELUTQ_ERR_TUNING;
    choose_shape(g, ksplit, waves);
    int ups = (g.U + ksplit - 1) / ksplit;
    // shrink the slice so its tables fit in LDS, then the slice count so that no slice is empty
    while (gemv_lds_bytes(ups, waves) > (size_t)MAX_LDS) ups = (ups + 1) / 2;
    ksplit = (g.U + ups - 1) / ups;

    GemvArgs a;
    a.planes = (const uint4 *)d_planes;
    a.scales = (const uint32_t *)d_scales;
    a.zeros = (const uint32_t *)d_zeros;
    a.bias = (const uint16_t *)d_bias;
    a.x = (const uint16_t *)d_x;
    a.y = (uint16_t *)d_y;
    a.N = N; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb;
    a.ksplit = ksplit; a.ups = ups;
    a.partial = nullptr; a.counters = nullptr;
    a.prologue = 0; a.eps = 0.f; a.norm_w = nullptr; a.residual = nullptr;
    if (fusion) {
        if (fusion->prologue < 0 || fusion->prologue > 2) return ELUTQ_ERR_TUNING;
        if (fusion->prologue == 1 && !fusion->d_norm_weight) return ELUTQ_ERR_NULL;
        a.prologue = fusion->prologue;
        a.eps = fusion->eps;
        a.norm_w = (const uint16_t *)fusion->d_norm_weight;
        a.residual = (const uint16_t *)fusion->d_residual;
    }
    if (ksplit > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ksplit * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        a.counters = (unsigned *)d_workspace;
        a.partial = (float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
    }
    return dispatch_gemv(a, bits, group, waves, gemv_lds_bytes(ups, waves), (hipStream_t)stream);
}

int elutq_hlq_gemv_f16_tuned(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                             const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                             size_t workspace_bytes, void *stream, int ksplit, int waves)
{
    return elutq_hlq_gemv_fused_f16(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                                    workspace_bytes, stream, nullptr, ksplit, waves);
}

int elutq_hlq_gemv_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                       const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                       size_t workspace_bytes, void *stream)
{
    return elutq_hlq_gemv_fused_f16(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                                    workspace_bytes, stream, nullptr, 0, 0);
}

}  // extern "C"

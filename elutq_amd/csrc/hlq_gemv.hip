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
//    with a power-of-two scale per 64-k half unit chosen from max|x| of that half: sums are
//    exact integers (no LUT rounding unless |x_k| < 2^-13 max|x|, then <= 2^-24 max|x|), two
//    lookups retire with one v_add3_u32;
//  * the plane dwords are stored rotated so that `byte & 0x3C` is already the byte offset
//    into the table; one SDWA v_and per lookup writes that offset into byte 0 of a
//    register whose upper bytes keep the table base (dst_unused:UNUSED_PRESERVE), the
//    chunk index rides in the ds_read immediate;
//  * a workgroup owns one column block and a slice of K; its (unit, plane) sub-tasks are
//    dealt to the waves in contiguous runs, and each wave builds the tables of the units of
//    its own run in its own LDS region, so no wave waits for another before its lookups;
//  * loads are unconditional and ordered (activations, first sub-task, table build, rest of
//    the run) so that the in-order vector-memory counter can be waited on precisely;
//  * slices are combined through a workspace by the last workgroup to arrive (fixed
//    summation order, so results are deterministic).
#include <hip/hip_runtime.h>
#include <type_traits>
#include <vector>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"
#include "hlq_gemv_index.h"

namespace {

constexpr int MAX_LDS = HLQ_MAX_LDS;
constexpr int TBL_BYTES = HLQ_TBL_BYTES;             // 16 int32 entries
constexpr int UNIT_LUT_BYTES = HLQ_UNIT_LUT_BYTES;   // 32 chunks per unit

// Device pointers are declared in the global address space for the device pass: a pointer that a
// kernel reads out of a struct in memory (the grouped launch) would otherwise be generic, and
// generic loads count on the LDS counter too, which serialises them with the table lookups.
#if defined(__HIP_DEVICE_COMPILE__)
#define HLQ_GLOBAL __attribute__((address_space(1)))
#else
#define HLQ_GLOBAL
#endif

struct GemvArgs {
    const HLQ_GLOBAL uint4 *planes;
    const HLQ_GLOBAL uint32_t *scales;
    const HLQ_GLOBAL uint32_t *zeros;
    const HLQ_GLOBAL uint16_t *bias;    // fp16 or null
    const HLQ_GLOBAL uint16_t *x;       // fp16 [K]
    HLQ_GLOBAL uint16_t *y;             // fp16 [N]
    HLQ_GLOBAL float *partial;          // [ksplit][ncb*64]   (ksplit > 1)
    HLQ_GLOBAL unsigned *counters;      // [ncb], zero between calls
    int N, U, NT, ncb;
    int ksplit, ups;         // slices per column block, units per slice
    int spw;                 // sub-tasks per wave (contiguous run)
    int nuw_max, wave_lds;   // units a wave's run can touch, bytes of its LDS region
    // optional fusion with the ops around the projection in a decoder layer
    int prologue;            // 0: x as is; 1: rmsnorm(x) * norm_w; 2: silu(x[0:K]) * x[K:2K]
    float eps;
    const HLQ_GLOBAL uint16_t *norm_w;  // fp16 [K]      (prologue 1)
    const HLQ_GLOBAL uint16_t *residual;  // fp16 [N] added to the output, or null
    const HLQ_GLOBAL float *extra;        // fp32 [N] added to the output before it is rounded, or null
    // K slices handed to the next launch instead of being summed here, and the consuming side
    int defer;                            // 1: write the slices' partial sums to `partial` and nothing else
    int n_slices_in;                      // > 0: x = fp16(sum of slices_in in order + x), prologue 1 only
    const HLQ_GLOBAL float *slices_in;    // fp32 [n_slices_in][K]
    HLQ_GLOBAL uint16_t *x_out;           // fp16 [K] or null: the combined x, written by workgroup (0, 0)
};

#ifdef HLQ_TIMING
// Profiling builds only: per-stage wall-clock stamps (100 MHz) of every wave (up to 16) of every
// workgroup, kept in registers and written once when the tile is done.
__device__ unsigned long long *g_hlq_stamps = nullptr;
#define HLQ_STAMP_DECL unsigned long long hlq_t[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define HLQ_STAMP(i) hlq_t[i] = wall_clock64()
#define HLQ_STAMP_FLUSH                                                                           \
    do {                                                                                          \
        if (g_hlq_stamps && (threadIdx.x & 63) == 0)                                              \
            for (int hlq_i = 0; hlq_i < 8; hlq_i++)                                               \
                g_hlq_stamps[(((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + (threadIdx.x >> 6)) * 8 + hlq_i] = hlq_t[hlq_i]; \
    } while (0)
#else
#define HLQ_STAMP_DECL do { } while (0)
#define HLQ_STAMP(i) do { } while (0)
#define HLQ_STAMP_FLUSH do { } while (0)
#endif

typedef __attribute__((address_space(3))) const int lds_cint;

__device__ __forceinline__ int lds_ld(uint32_t addr, int imm)
{
    return *(lds_cint *)(uintptr_t)(addr + (uint32_t)imm);
}

__device__ __forceinline__ float h2f_lo(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v & 0xffffu)); }
__device__ __forceinline__ float h2f_hi(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v >> 16)); }

// dst = base | src.byte<SEL>: the table address of one lookup.  `src` is a plane dword (or its
// rotation by 4) masked to bits 2..5 of every byte, i.e. 4 * nibble; `base` (wave-uniform, a
// multiple of 256) is the LDS address of the unit's tables.
#define HLQ_SDWA_OR(dst, base, src, SEL)                                                       \
    asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD "         \
        "src1_sel:BYTE_" #SEL                                                                  \
        : "=v"(dst)                                                                            \
        : "s"(base), "v"(src))

// Eight lookups for one plane dword (32 k): chunks 8*D .. 8*D+7 of the unit.  Issue and sum are
// separate so that the lookups of the next dword are on their way to LDS before the wave waits
// for the results of this one (LDS returns a wave's reads in order).
template <int D>
__device__ __forceinline__ void lookup_issue(uint32_t w, uint32_t base, int (&v)[8])
{
    const uint32_t wm = w & 0x3C3C3C3Cu;
    const uint32_t rm = __builtin_amdgcn_alignbit(w, w, 4) & 0x3C3C3C3Cu;
    uint32_t a[8];
    HLQ_SDWA_OR(a[0], base, wm, 0);
    HLQ_SDWA_OR(a[1], base, rm, 0);
    HLQ_SDWA_OR(a[2], base, wm, 1);
    HLQ_SDWA_OR(a[3], base, rm, 1);
    HLQ_SDWA_OR(a[4], base, wm, 2);
    HLQ_SDWA_OR(a[5], base, rm, 2);
    HLQ_SDWA_OR(a[6], base, wm, 3);
    HLQ_SDWA_OR(a[7], base, rm, 3);
    constexpr int off = D * 8 * TBL_BYTES;
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = lds_ld(a[j], off + j * TBL_BYTES);
}

__device__ __forceinline__ int lookup_sum(const int (&v)[8], int acc)
{
    acc = acc + v[0] + v[1];
    acc = acc + v[2] + v[3];
    acc = acc + v[4] + v[5];
    acc = acc + v[6] + v[7];
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

// Byte addresses of one column block's data, uniform over the wave: every load of a sub-task
// is one of these (scalar registers) plus a 32-bit offset, so the per-load address arithmetic
// stays short -- the scalar unit is shared by the four SIMDs of a CU and the index arithmetic
// of sixteen waves would otherwise hold up the start of the weight stream.
struct CbBase {
    const HLQ_GLOBAL unsigned char *planes;   // sub-task 0 of the slice
    const HLQ_GLOBAL unsigned char *scales;   // meta row 0 of the column block
    const HLQ_GLOBAL unsigned char *zeros;    // meta row 0 of the column block
};

template <int BITS>
__device__ __forceinline__ CbBase cb_base(const GemvArgs &a, int cb, int u0)
{
    CbBase p;
    p.planes = (const HLQ_GLOBAL unsigned char *)a.planes + ((size_t)cb * a.U + u0) * (size_t)(BITS * HLQ_CB * 16);
    p.scales = (const HLQ_GLOBAL unsigned char *)a.scales + (size_t)cb * a.NT * (size_t)(BITS * HLQ_CB * 4);
    p.zeros = (const HLQ_GLOBAL unsigned char *)a.zeros + (size_t)cb * a.NT * (size_t)(HLQ_CB * 4);
    return p;
}

// st = sub-task index inside the slice (unit u0 + st / BITS, plane st % BITS); planes of a
// slice are contiguous in st.
template <int BITS, bool G64, bool SC = true, bool ZZ = true>
__device__ __forceinline__ void load_sub(Sub &t, const CbBase &p, int u0, int st, int lane)
{
    const uint32_t u = (uint32_t)(u0 + st / BITS), b = (uint32_t)(st % BITS);
    const uint32_t row = G64 ? u : (u >> 1);
    const u32x4 v = __builtin_nontemporal_load(
        (const HLQ_GLOBAL u32x4 *)(p.planes + ((uint32_t)st * (uint32_t)(HLQ_CB * 16) + (uint32_t)lane * 16u)));
    t.w = make_uint4(v.x, v.y, v.z, v.w);
    if (SC) t.sc = *(const HLQ_GLOBAL uint32_t *)(p.scales + ((row * BITS + b) * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u));
    if (ZZ) t.zz = *(const HLQ_GLOBAL uint32_t *)(p.zeros + (row * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u));
}

// Sub-tasks that share scale / zero dwords form a meta group: the planes of one unit at
// G = 64, of a unit pair at G = 128.  When every wave's run starts on a group boundary and the
// slots hold whole groups (`PAIRED`), position d of a pass is a compile-time (unit, plane) of
// its group: only the first unit's positions load the scale dword of their plane, only position 0
// the zero dword -- 7 loads instead of 12 for the four sub-tasks of a w2g128 pair -- and the
// later positions reuse the values.  Otherwise every sub-task loads both (3 loads each, so
// that the load count behind any point is still a compile-time constant).
template <int BITS, bool G64>
struct MetaGroup {
    static constexpr int SIZE = G64 ? BITS : 2 * BITS;           // sub-tasks per group
    static constexpr bool fits(int nslot) { return nslot % SIZE == 0; }
    static constexpr bool sc_at(int d) { return d % SIZE < BITS; }
    static constexpr bool zz_at(int d) { return d % SIZE == 0; }
};

template <int BITS, bool G64, bool PAIRED, int D>
__device__ __forceinline__ void load_slot(Sub &t, const CbBase &p, int u0, int st, int lane)
{
    using MG = MetaGroup<BITS, G64>;
    load_sub<BITS, G64, !PAIRED || MG::sc_at(D), !PAIRED || MG::zz_at(D)>(t, p, u0, st, lane);
}

// The two 64-k halves of a unit have their own table scale (2^-p) and activation sum; at
// G = 64 they are also two quantization groups (lo / hi half of the meta dwords), at G = 128
// one group (the half of the meta dwords selected by the unit's parity).
template <bool G64>
__device__ __forceinline__ float process_sub(const uint4 &w, uint32_t sc_raw, uint32_t zz_raw, int lu, int b, int odd,
                                             uint32_t lut_base, const float2 *xs_inv, float acc)
{
    int v0[8], v1[8];
    const uint32_t ub = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lut_base + (uint32_t)lu * UNIT_LUT_BYTES));
    const float2 h0 = xs_inv[2 * lu], h1 = xs_inv[2 * lu + 1];      // .x = sum of x, .y = 2^-p
    lookup_issue<0>(w.x, ub, v0);
    lookup_issue<1>(w.y, ub, v1);
    __builtin_amdgcn_sched_barrier(0);
    int i0 = lookup_sum(v0, 0);
    lookup_issue<2>(w.z, ub, v0);
    __builtin_amdgcn_sched_barrier(0);
    i0 = lookup_sum(v1, i0);
    lookup_issue<3>(w.w, ub, v1);
    __builtin_amdgcn_sched_barrier(0);
    int i1 = lookup_sum(v0, 0);
    i1 = lookup_sum(v1, i1);
    const uint32_t sc = G64 ? sc_raw : (odd ? (sc_raw >> 16) * 0x10001u : (sc_raw & 0xffffu) * 0x10001u);
    acc = fmaf((float)i0 * h0.y, h2f_lo(sc), acc);
    acc = fmaf((float)i1 * h1.y, h2f_hi(sc), acc);
    if (b == 0) {
        const uint32_t zz = G64 ? zz_raw : (odd ? (zz_raw >> 16) * 0x10001u : (zz_raw & 0xffffu) * 0x10001u);
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

// Always two loads (without a prologue the second one re-reads the chunk): a fixed number
// of loads lets the compiler wait for these with an exact vector-memory count while the
// weight loads issued after them are still in flight.
template <bool PLAIN>
__device__ __forceinline__ void load_chunk(const GemvArgs &a, int prologue, int K, size_t k, uint2 &raw, uint2 &raw2)
{
    raw = *(const HLQ_GLOBAL uint2 *)(a.x + k);
    if (PLAIN) {            // no prologue at compile time: one load
        raw2 = raw;
        return;
    }
    const HLQ_GLOBAL uint16_t *second = prologue == 1 ? a.norm_w + k : (prologue == 2 ? a.x + (size_t)K + k : a.x + k);
    raw2 = *(const HLQ_GLOBAL uint2 *)second;
}

// Subset-sum table of one chunk of 4 activations as int32 fixed point, 64 bytes at `tbl`.
// The 16 lanes of a DPP row cover one 64-k half unit, whose max|x| sets the power-of-two
// table scale and whose sum feeds the zero-point fold (row leader stores both in *half).
__device__ __forceinline__ void build_chunk(int prologue, uint2 raw, uint2 raw2, float rstd, unsigned char *tbl,
                                            float2 *half, bool leader)
{
    float v[4];
    chunk_values(prologue, raw, raw2, rstd, v);
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
    int4 *dst = (int4 *)tbl;
    dst[0] = make_int4(0, i0, i1, e3);
    dst[1] = make_int4(i2, e5, e6, e7);
    dst[2] = make_int4(i3, i3 + i0, i3 + i1, i3 + e3);
    dst[3] = make_int4(i3 + i2, i3 + e5, i3 + e6, i3 + e7);
    if (leader) *half = make_float2(s, inv);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load of the wave (its fence covers all address spaces), which here would
// be the weight loads that are meant to stay in flight across the barrier.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 1 / rms of the whole activation vector for the fused RMSNorm prologue: the workgroup sums
// the squares together (one chunk per thread and pass), two barriers.  `scratch` is LDS of
// HLQ_RSTD_SCRATCH floats (at hlq_lds_map().rstd).  Every workgroup does this for itself (2K bytes from cache).

// Activations that arrive as a base vector plus the unsummed K slices of the launch that
// produced them (its `defer` mode): element k is fp16(((s0[k] + s1[k]) + ...) + x[k]), the same
// operations in the same order as that launch's own output stage would have used.
constexpr int GEMV_MAX_SLICES_IN = HLQ_GEMV_MAX_SLICES_IN;

struct SliceChunk {
    float4 p[GEMV_MAX_SLICES_IN];
};

__device__ __forceinline__ void load_slice_chunk(const GemvArgs &a, int K, int chunk, SliceChunk &c)
{
#pragma unroll
    for (int s = 0; s < GEMV_MAX_SLICES_IN; s++)     // always GEMV_MAX_SLICES_IN loads: a fixed count
        c.p[s] = *(const HLQ_GLOBAL float4 *)(a.slices_in + (size_t)hlq_slice_row(s, a.n_slices_in) * K + (size_t)chunk * 4);
}

__device__ __forceinline__ uint2 combine_chunk(const GemvArgs &a, uint2 base, const SliceChunk &c)
{
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < GEMV_MAX_SLICES_IN; s++)
        if (s < a.n_slices_in) { v[0] += c.p[s].x; v[1] += c.p[s].y; v[2] += c.p[s].z; v[3] += c.p[s].w; }
    v[0] += h2f_lo(base.x); v[1] += h2f_hi(base.x); v[2] += h2f_lo(base.y); v[3] += h2f_hi(base.y);
    auto pack = [](float lo, float hi) __attribute__((always_inline)) {
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
    };
    return make_uint2(pack(v[0], v[1]), pack(v[2], v[3]));
}

// The chunk of x this thread squares first; issued ahead of the other loads of the tile so that
// the reduction below overlaps with them.
__device__ __forceinline__ uint2 rstd_first_load(const GemvArgs &a, int K, int tid)
{
    return *(const HLQ_GLOBAL uint2 *)(a.x + (size_t)min(tid, K / 4 - 1) * 4);
}

// With slices (`sliced`) every chunk of the combined x is formed here once, kept in
// `stage` (LDS, fp16 [K]) for the table builds and, by the first workgroup, written to a.x_out.
__device__ __forceinline__ float block_rstd(const GemvArgs &a, int K, float *scratch, int tid, int nthreads, uint2 first,
                                            const SliceChunk &sfirst, bool sliced, uint2 *stage, bool write_out)
{
    auto sq4 = [](uint2 r) __attribute__((always_inline)) {
        const float x0 = h2f_lo(r.x), x1 = h2f_hi(r.x), x2 = h2f_lo(r.y), x3 = h2f_hi(r.y);
        return (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
    };
    float ssq = 0.f;
    if (sliced) {
        for (int i = tid; i < K / 4; i += nthreads) {
            uint2 r;
            if (i == tid) r = combine_chunk(a, first, sfirst);
            else {
                SliceChunk c;
                load_slice_chunk(a, K, i, c);
                r = combine_chunk(a, *(const HLQ_GLOBAL uint2 *)(a.x + (size_t)i * 4), c);
            }
            stage[i] = r;
            if (write_out) *(HLQ_GLOBAL uint2 *)(a.x_out + (size_t)i * 4) = r;
            ssq += sq4(r);
        }
    } else {
        ssq = tid < K / 4 ? sq4(first) : 0.f;
        for (int i = tid + nthreads; i < K / 4; i += nthreads) ssq += sq4(*(const HLQ_GLOBAL uint2 *)(a.x + (size_t)i * 4));
    }
    HLQ_ROW_REDUCE(ssq, op_add);
    if ((tid & 15) == 0) scratch[tid >> 4] = ssq;
    lds_barrier();
    if (tid < 64) {
        float v = tid < (nthreads >> 4) ? scratch[tid] : 0.f;
        HLQ_ROW_REDUCE(v, op_add);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (tid == 0) scratch[64] = v;
    }
    lds_barrier();
    return rsqrtf(scratch[64] / (float)K + a.eps);
}

// A SIMD issues from its oldest wave first, so the waves of a workgroup finish their runs one
// after the other and the last one works alone at the end.  Every wave therefore lowers its own
// priority as it gets on with its run (3 at the start, 0 in the last quarter): the waves that are
// behind are served first and all finish together.
__device__ __forceinline__ void progress_prio(int done, int total)
{
    const int d4 = done * 4;                 // quarter of the run the wave is in, without a division
    if (d4 < total) __builtin_amdgcn_s_setprio(3);
    else if (d4 < 2 * total) __builtin_amdgcn_s_setprio(2);
    else if (d4 < 3 * total) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Sub-tasks a wave keeps in flight at most.  Three planes get six slots and four planes eight: a
// unit pair (one meta group at G = 128) is that many sub-tasks, and K = 4096 gives a wave exactly
// that run -- so a layer with more column blocks than CUs can run as column-block runs (which need
// the whole run in slots) without slicing K.
constexpr int depth_of(int bits) { return bits == 3 ? 6 : (bits == 4 ? 8 : 4); }

// One workgroup = one column block x one K slice.  Its (unit, plane) sub-tasks are dealt to
// the waves in contiguous runs of `spw`; every wave builds the activation tables of the
// (one or two) units its run touches in its own LDS region and goes on to its lookups
// without waiting for the other waves -- the only workgroup barrier is the one in front of
// the final cross-wave sum.
//
// `red_sel` picks one of two cross-wave buffers so that a caller that runs tiles
// back to back needs no barrier between them: waves other than wave 0 may start the next
// tile while wave 0 still sums and stores this one.
//
// MULTI: the tile covers `ncb_run` consecutive column blocks of the same slice.  The tables are
// built once; while a wave looks up its sub-tasks of one column block, each slot it has
// consumed is refilled with the same sub-task of the next block, so the weight stream never
// stops between blocks.  Needs runs of at most NSLOT sub-tasks per wave.
// VAR: which optional inputs the instance reads, known when the kernel is compiled.
//   GEMV_FUSED  prologue and residual as `a` says (the decode step's launches)
//   GEMV_PLAIN  none of them (their fields of `a` are not read)
//   GEMV_EXTRA  plain, plus the fp32 term `a.extra` added before the output is rounded
enum { GEMV_FUSED = 0, GEMV_PLAIN = 1, GEMV_EXTRA = 2 };
template <int BITS, bool G64, int NSLOT, bool MULTI, int VAR, bool PAIRED>
__device__ __forceinline__ void gemv_tile(const GemvArgs &a, int cb, int slice, int ncb_run, unsigned char *smem, int &red_sel)
{
    HLQ_STAMP_DECL;
#ifdef HLQ_TIMING_ENTRY
    HLQ_STAMP(7);
    asm volatile("" ::: "memory");
#endif
    constexpr bool PLAIN = VAR != GEMV_FUSED;
    const int prologue = PLAIN ? 0 : a.prologue;
    const HLQ_GLOBAL uint16_t *residual = PLAIN ? nullptr : a.residual;
    const HLQ_GLOBAL float *extra = VAR == GEMV_EXTRA ? a.extra : nullptr;
    const int tid = threadIdx.x, lane = tid & 63, nw = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int u0 = slice * a.ups, nU = min(u0 + a.ups, a.U) - u0;
    const int nst = nU * BITS;                                             // sub-tasks of this workgroup
    const HlqWaveRun wr = hlq_wave_run(wave, a.spw, nst, BITS);
    const int s_begin = wr.s_begin, s_end = wr.s_end;
    const int ub = wr.ub;                                                  // first unit (in the slice) of this wave
    const int nuw = wr.nuw;                                                // units this wave touches
    const int s_last = wr.s_last;                                          // clamp target for loads past the run

    const HlqLdsMap lm = hlq_lds_map(nw, a.wave_lds);
    unsigned char *lut = smem + (size_t)wave * a.wave_lds;                 // this wave's tables [nuw][32][16] int32
    float2 *xs_inv = (float2 *)(lut + (size_t)a.nuw_max * UNIT_LUT_BYTES); // [2 * nuw_max]
    float *red0 = (float *)(smem + lm.red);                                // [2][nw][64]
    float *rstd_scratch = (float *)(smem + lm.rstd);                       // [HLQ_RSTD_SCRATCH]
    const uint32_t lut_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lut;

    __builtin_amdgcn_s_setprio(3);
    HLQ_STAMP(0);
    // Activations first, then the weight stream.  Every load below is unconditional (a wave
    // whose run is shorter than NSLOT re-reads its last sub-task), so the number of loads
    // behind the activations is a compile-time constant and the table build waits for the
    // activations only (vmcnt(3 * NSLOT)), with the weights still in flight.
    const int K = a.U * HLQ_UNIT;
    const size_t k0 = (size_t)(u0 + ub) * HLQ_UNIT;
    const int nchunks = nuw * 32;
    float rstd = 1.f;
    // what the last step adds to the output is fetched first of all, so that its latency is not
    // left at the end of the kernel (wave 0 finishes a tile; a run of column blocks loads it there)
    uint16_t pre_bias = 0, pre_res = 0;
    if (!MULTI && wave == 0 && cb * HLQ_CB + lane < a.N) {
        if (a.bias) pre_bias = a.bias[cb * HLQ_CB + lane];
        if (residual) pre_res = residual[cb * HLQ_CB + lane];
    }
    uint2 rfirst = make_uint2(0, 0);
    if (prologue == 1) rfirst = rstd_first_load(a, K, tid);
    const bool sliced = !PLAIN && a.n_slices_in > 0;                       // host: only with prologue 1
    SliceChunk sfirst = {};
    // fp16 [K] behind the reduction scratch when `sliced` (not selected against a null pointer: the
    // accesses must stay LDS instructions, a generic access would also count as a vector-memory one
    // and wait behind the weight loads in flight)
    uint2 *stage = (uint2 *)(smem + lm.stage);
    if (sliced) load_slice_chunk(a, K, min(tid, K / 4 - 1), sfirst);
    uint2 raw, raw2;
    // lanes past the run (and waves without one, whose k0 is the end of the slice) re-read a valid chunk
    load_chunk<PLAIN>(a, prologue, K, hlq_x_first_k(k0, nchunks, lane), raw, raw2);
    asm volatile("" ::: "memory");      // keep both activation loads ahead of the weight loads

    float acc = 0.f;
    Sub slot[NSLOT];
    const CbBase here = cb_base<BITS>(a, cb, u0);
    {   // the first sub-task's loads start the weight stream ...
        load_slot<BITS, G64, PAIRED, 0>(slot[0], here, u0, min(s_begin, s_last), lane);
    }
    asm volatile("" ::: "memory");
    if (prologue == 1)
        rstd = block_rstd(a, K, rstd_scratch, tid, blockDim.x, rfirst, sfirst, sliced, stage,
                          sliced && a.x_out && blockIdx.x == 0 && blockIdx.y == 0);
    // the combined chunk replaces the base's (a wave without a run sits at the end of the slice: clamped)
    if (sliced) raw = stage[hlq_stage_first_index(k0, nchunks, lane, K)];

    // ... the tables are built as soon as the activations are in (a wave that first queued all
    // its weight loads would sit in the memory pipeline's back-pressure instead) ...
    if (lane < nchunks)
        build_chunk(prologue, raw, raw2, rstd, lut + (size_t)lane * TBL_BYTES, xs_inv + (lane >> 4), (lane & 15) == 0);
    asm volatile("" ::: "memory");

    // ... and the rest of the run's loads follow.
    static_for<1, NSLOT>([&](auto dc) __attribute__((always_inline)) {
        constexpr int d = decltype(dc)::value;
        load_slot<BITS, G64, PAIRED, d>(slot[d], here, u0, min(s_begin + d, s_last), lane);
    });
    for (int ci = lane + 64; ci < nchunks; ci += 64) {      // runs of more than two units (not the common case)
        load_chunk<PLAIN>(a, prologue, K, k0 + (size_t)ci * 4, raw, raw2);
        if (sliced) raw = stage[(k0 >> 2) + ci];
        build_chunk(prologue, raw, raw2, rstd, lut + (size_t)ci * TBL_BYTES, xs_inv + (ci >> 4), (ci & 15) == 0);
    }
    HLQ_STAMP(1);
    // The tables were written by this wave and are read by this wave: LDS executes a wave's
    // operations in order, so no barrier -- only keep the compiler from reordering.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    HLQ_STAMP(2);

    // Combine the waves of this workgroup, then the slices of this column block.  The wave that
    // does it waits for its partial-sum stores to be acknowledged, and that wait covers every load
    // it has in flight: in a run of column blocks those are the next block's weights, fetched a
    // moment ago.  Where the last wave has no sub-tasks (a slice of 28 units at 2 planes keeps 14
    // waves busy) it loads nothing inside the run and takes this part over.
    const int fin = (MULTI && a.ksplit > 1 && (nw - 1) * a.spw >= nst) ? nw - 1 : 0;
    auto finish = [&](int cbf, float accf) __attribute__((always_inline)) {
        float *red = red0 + red_sel * nw * HLQ_CB;
        red_sel ^= 1;
        const int n = cbf * HLQ_CB + lane;
        float total = accf;
        if (nw > 1) {
            red[wave * HLQ_CB + lane] = accf;
            lds_barrier();
            if (wave == fin) {
                total = 0.f;
                for (int w = 0; w < nw; w++) total += red[w * HLQ_CB + lane];
            }
        }
        HLQ_STAMP(4);
        if (a.ksplit == 1) {
            if (wave == fin && n < a.N) {
                if (a.bias) total += (float)__builtin_bit_cast(_Float16, MULTI ? a.bias[n] : pre_bias);
                if (residual) total += (float)__builtin_bit_cast(_Float16, MULTI ? residual[n] : pre_res);
                if (extra) total += extra[n];
                a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
            }
            return;
        }
        // Slices meet through device memory.  Partial sums are written and read with
        // agent-scope atomics (they bypass the per-XCD L2s' non-coherent lines), the writer
        // waits for its stores to be acknowledged before it takes a ticket, and the reader's
        // loads depend on the ticket it drew -- so no cache write-back / invalidate is needed.
        const size_t npad = (size_t)a.ncb * HLQ_CB;
        if (!PLAIN && a.defer) {
            // the consumer is a later launch on the same stream: an ordinary store, no meeting
            if (wave == fin) a.partial[(size_t)slice * npad + n] = total;
            return;
        }
        if (wave == fin) {
            __hip_atomic_store(&a.partial[(size_t)slice * npad + n], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            HLQ_STAMP(5);
            unsigned ticket = 0;
            if (lane == 0)
                ticket = __hip_atomic_fetch_add(&a.counters[cbf], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ticket = __builtin_amdgcn_readfirstlane(ticket);
            HLQ_STAMP(6);
            if (ticket == (unsigned)a.ksplit - 1u) {
                // eight independent loads in flight at a time, summed in slice order
                float sum = 0.f;
                for (int s0 = 0; s0 < a.ksplit; s0 += 8) {
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const int sl = min(s0 + j, a.ksplit - 1);
                        v[j] = __hip_atomic_load(&a.partial[(size_t)sl * npad + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        if (s0 + j < a.ksplit) sum += v[j];
                }
                if (n < a.N) {
                    if (a.bias) sum += (float)__builtin_bit_cast(_Float16, MULTI ? a.bias[n] : pre_bias);
                    if (residual) sum += (float)__builtin_bit_cast(_Float16, MULTI ? residual[n] : pre_res);
                    if (extra) sum += extra[n];
                    a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)sum);
                }
                if (lane == 0) __hip_atomic_store(&a.counters[cbf], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                HLQ_STAMP(7);
            }
        }
    };

    // Position d of a pass over the slots: the sub-task's plane and unit parity are compile-time
    // in PAIRED mode, where the scale / zero dwords are taken over from the positions that loaded them.
    using MG = MetaGroup<BITS, G64>;
    uint32_t sc_keep[BITS] = {}, zz_keep = 0;
    auto run_slot = [&](auto dc, int st, float accv) __attribute__((always_inline)) -> float {
        constexpr int d = decltype(dc)::value;
        const int u = st / BITS;
        if constexpr (PAIRED) {
            constexpr int pos = d % MG::SIZE, b = pos % BITS, odd = pos / BITS;     // odd only matters at G = 128
            if (MG::sc_at(d)) sc_keep[b] = slot[d].sc;
            if (MG::zz_at(d)) zz_keep = slot[d].zz;
            return process_sub<G64>(slot[d].w, sc_keep[b], zz_keep, u - ub, b, odd, lut_base, xs_inv, accv);
        } else {
            return process_sub<G64>(slot[d].w, slot[d].sc, slot[d].zz, u - ub, st % BITS, (u0 + u) & 1, lut_base, xs_inv, accv);
        }
    };

    if (MULTI) {
        for (int c = 0; c < ncb_run; c++) {
            const CbBase next = cb_base<BITS>(a, min(cb + c + 1, cb + ncb_run - 1), u0);   // past the run: a reload nobody reads
            float accc = 0.f;
            HLQ_STAMP(2);
            if (s_begin < s_end)                              // wave-uniform; a wave without sub-tasks loads nothing here
                static_for<0, NSLOT>([&](auto dc) __attribute__((always_inline)) {
                    constexpr int d = decltype(dc)::value;
                    const int st = s_begin + d;
                    progress_prio(d, a.spw);
                    if (st < s_end) accc = run_slot(dc, st, accc);
                    load_slot<BITS, G64, PAIRED, d>(slot[d], next, u0, min(st, s_last), lane);
                });
            HLQ_STAMP(3);
            finish(cb + c, accc);
            HLQ_STAMP(6);
        }
        HLQ_STAMP_FLUSH;
        return;
    }

    // Slot d holds sub-task base + d; it is refilled with sub-task base + d + NSLOT as soon as
    // it has been consumed (past the end of the run: a reload nobody reads).
    for (int base = s_begin; base < s_end; base += NSLOT) {
        static_for<0, NSLOT>([&](auto dc) __attribute__((always_inline)) {
            constexpr int d = decltype(dc)::value;
            const int st = base + d;
            progress_prio(st - s_begin, a.spw);
            if (st < s_end) acc = run_slot(dc, st, acc);
            if (base + NSLOT < s_end)                      // wave-uniform: only runs longer than NSLOT refill
                load_slot<BITS, G64, PAIRED, d>(slot[d], here, u0, min(st + NSLOT, s_last), lane);
        });
    }
    HLQ_STAMP(3);
    finish(cb, acc);
    HLQ_STAMP_FLUSH;
}

template <int BITS, bool G64, int NSLOT, bool PAIRED, int VAR>
__global__ __launch_bounds__(1024) void hlq_gemv_kernel(const GemvArgs a)
{
    extern __shared__ __align__(256) unsigned char smem[];
    int sel = 0;
    gemv_tile<BITS, G64, NSLOT, false, VAR, PAIRED>(a, blockIdx.y, blockIdx.x, 1, smem, sel);      // grid = (slices, column blocks)
}

// One GEMV with more column blocks than the chip has CUs: every workgroup takes a run of
// consecutive column blocks (tables built once, weights prefetched across the blocks) instead
// of the launch holding two workgroups per CU that each build the same tables.
template <int BITS, bool G64, int NSLOT, bool PAIRED, bool PLAIN>
__global__ __launch_bounds__(1024) void hlq_gemv_run_kernel(const GemvArgs a, int run)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const int cb0 = blockIdx.y * run;               // grid = (slices, runs of column blocks)
    int sel = 0;
    gemv_tile<BITS, G64, NSLOT, true, PLAIN ? GEMV_PLAIN : GEMV_FUSED, PAIRED>(a, cb0, blockIdx.x, min(run, a.ncb - cb0), smem, sel);
}

// Many independent GEMVs in one launch: the tiles of all of them form one list that the
// workgroups walk with stride gridDim.x (tiles of one GEMV are neighbours in the list, so its
// activations stay in cache and the slices of a column block run at about the same time).
// Nothing waits for another workgroup -- slices still meet through tickets -- so the launch,
// the first memory round trips and the tail of a GEMV are paid once per list instead of once
// per GEMV, and with two workgroups per CU the sum-and-store of one tile hides under the
// lookups of another.
struct GroupItem {
    int problem, cb, slice;  // first column block and K slice
    int ncb_run;             // consecutive column blocks of that slice
};

template <int BITS, bool G64, int NSLOT, bool PAIRED>
__global__ __launch_bounds__(1024) void hlq_gemv_group_kernel(const GemvArgs *__restrict__ problems,
                                                              const GroupItem *__restrict__ items, int n_items)
{
    extern __shared__ __align__(256) unsigned char smem[];
    int sel = 0;
    for (int i = blockIdx.x; i < n_items; i += gridDim.x) {
        const GroupItem it = items[i];
        const GemvArgs a = problems[it.problem];
        gemv_tile<BITS, G64, NSLOT, true, GEMV_PLAIN, PAIRED>(a, it.cb, it.slice, it.ncb_run, smem, sel);
    }
}

// Per-wave LDS region and run length for a slice of `ups` units handled by `waves` waves, and the dynamic
// LDS of the workgroup: hlq_gemv_index.h (shared with the CPU audit of the tile's index arithmetic).
using WavePlan = HlqWavePlan;
WavePlan wave_plan(int ups, int bits, int waves) { return hlq_wave_plan(ups, bits, waves); }
size_t gemv_lds_bytes(int ups, int bits, int waves) { return hlq_gemv_lds_bytes(ups, bits, waves); }

constexpr int NUM_CU_RUN = HLQ_NUM_CU;

// Kernels that need more than 64 KiB of dynamic LDS must be told so once per device (the
// setting is sticky); `done` is the caller's per-kernel table of devices already set.
inline bool allow_big_lds(const void *kern, size_t lds, int limit, bool (&done)[64])
{
    if (lds <= 64 * 1024) return true;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    if (!done[dev]) {
        if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, limit) != hipSuccess) return false;
        done[dev] = true;
    }
    return true;
}


// Every wave's run starts on a meta-group boundary, the slots hold whole groups and (at G = 128)
// every slice starts on an even unit: the conditions of the PAIRED load pattern.
template <int BITS, bool G64, int NSLOT>
bool paired_ok(int spw, int ups, int ksplit)
{
    using MG = MetaGroup<BITS, G64>;
    return MG::fits(NSLOT) && spw % MG::SIZE == 0 && (G64 || ksplit == 1 || ups % 2 == 0);
}

template <int BITS, bool G64, int NSLOT, bool PAIRED, int VAR>
int launch_gemv_pp(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    constexpr bool PLAIN = VAR == GEMV_PLAIN;
    auto kern = hlq_gemv_kernel<BITS, G64, NSLOT, PAIRED, VAR>;
    static bool big_lds_done[64] = {};        // per template instance
    if (!allow_big_lds((const void *)kern, lds, MAX_LDS, big_lds_done)) return ELUTQ_ERR_HIP;
    // more tiles than CUs and runs that fit the slots: runs of column blocks, one workgroup per CU
    const int run = (a.ncb * a.ksplit + NUM_CU_RUN - 1) / NUM_CU_RUN;
    if (VAR != GEMV_EXTRA && run > 1 && a.spw <= NSLOT && waves == 16) {       // (the extra term has no run instances)
        auto kern_run = hlq_gemv_run_kernel<BITS, G64, NSLOT, PAIRED, PLAIN>;
        static bool big_lds_run_done[64] = {};
        if (!allow_big_lds((const void *)kern_run, lds, MAX_LDS, big_lds_run_done)) return ELUTQ_ERR_HIP;
        const int groups = (a.ncb + run - 1) / run;
        hipLaunchKernelGGL(kern_run, dim3(a.ksplit, groups), dim3(waves * 64), lds, stream, a, run);
        return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, dim3(a.ksplit, a.ncb), dim3(waves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64, int NSLOT, bool PAIRED>
int launch_gemv_p(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    if (a.extra) {
        if (a.prologue != 0 || a.residual) return ELUTQ_ERR_TUNING;     // no instance reads both
        return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_EXTRA>(a, waves, lds, stream);
    }
    if (a.prologue == 0 && !a.residual && !a.defer && a.n_slices_in == 0)      // the plain instances read none of these fields
        return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_PLAIN>(a, waves, lds, stream);
    return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_FUSED>(a, waves, lds, stream);
}

template <int BITS, bool G64, int NSLOT>
int launch_gemv_n(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    if constexpr (MetaGroup<BITS, G64>::fits(NSLOT)) {
        if (paired_ok<BITS, G64, NSLOT>(a.spw, a.ups, a.ksplit)) return launch_gemv_p<BITS, G64, NSLOT, true>(a, waves, lds, stream);
    }
    return launch_gemv_p<BITS, G64, NSLOT, false>(a, waves, lds, stream);
}

// NSLOT = sub-tasks a wave keeps in flight: its whole run when that is at most depth_of(BITS).
template <int BITS, bool G64>
int launch_gemv(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    constexpr int DEPTH = depth_of(BITS);
    switch (a.spw < DEPTH ? a.spw : DEPTH) {
    case 1: return launch_gemv_n<BITS, G64, 1>(a, waves, lds, stream);
    case 2: return launch_gemv_n<BITS, G64, 2>(a, waves, lds, stream);
    case 3: return launch_gemv_n<BITS, G64, 3>(a, waves, lds, stream);
    case 4: return launch_gemv_n<BITS, G64, 4>(a, waves, lds, stream);
    default:
        if constexpr (DEPTH >= 6) {
            if (a.spw == 5) return launch_gemv_n<BITS, G64, 5>(a, waves, lds, stream);
            if (a.spw == 6 || DEPTH == 6) return launch_gemv_n<BITS, G64, 6>(a, waves, lds, stream);
        }
        if constexpr (DEPTH == 8) {
            if (a.spw == 7) return launch_gemv_n<BITS, G64, 7>(a, waves, lds, stream);
            return launch_gemv_n<BITS, G64, 8>(a, waves, lds, stream);
        }
        return launch_gemv_n<BITS, G64, 4>(a, waves, lds, stream);
    }
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

// grid < 0: no launch, returns the number of workgroups of this shape a CU holds at once
template <int BITS, bool G64, int NSLOT, bool PAIRED>
int launch_group_p(const GemvArgs *d_problems, const GroupItem *d_items, int n_items, int grid, int waves, size_t lds,
                   hipStream_t stream)
{
    auto kern = hlq_gemv_group_kernel<BITS, G64, NSLOT, PAIRED>;
    static bool big_lds_done[64] = {};
    if (!allow_big_lds((const void *)kern, lds, MAX_LDS, big_lds_done)) return ELUTQ_ERR_HIP;
    if (grid < 0) {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)kern, waves * 64, lds) != hipSuccess || per_cu < 1)
            return 1;
        return per_cu;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * 64), lds, stream, d_problems, d_items, n_items);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

// paired: every problem of the group meets paired_ok for this slot count
template <int BITS, bool G64, int NSLOT>
int launch_group_n(bool paired, const GemvArgs *p, const GroupItem *it, int n, int grid, int waves, size_t lds, hipStream_t st)
{
    if constexpr (MetaGroup<BITS, G64>::fits(NSLOT)) {
        if (paired) return launch_group_p<BITS, G64, NSLOT, true>(p, it, n, grid, waves, lds, st);
    }
    return launch_group_p<BITS, G64, NSLOT, false>(p, it, n, grid, waves, lds, st);
}

template <int BITS, bool G64>
int launch_group(int nslot, bool paired, const GemvArgs *p, const GroupItem *it, int n, int grid, int waves, size_t lds,
                 hipStream_t st)
{
    switch (nslot) {
    case 1: return launch_group_n<BITS, G64, 1>(paired, p, it, n, grid, waves, lds, st);
    case 2: return launch_group_n<BITS, G64, 2>(paired, p, it, n, grid, waves, lds, st);
    case 3: return launch_group_n<BITS, G64, 3>(paired, p, it, n, grid, waves, lds, st);
    case 4: return launch_group_n<BITS, G64, 4>(paired, p, it, n, grid, waves, lds, st);
    default:
        if constexpr (depth_of(BITS) >= 6) {
            if (nslot == 5) return launch_group_n<BITS, G64, 5>(paired, p, it, n, grid, waves, lds, st);
            if (nslot == 6 || depth_of(BITS) == 6) return launch_group_n<BITS, G64, 6>(paired, p, it, n, grid, waves, lds, st);
        }
        if constexpr (depth_of(BITS) == 8) {
            if (nslot == 7) return launch_group_n<BITS, G64, 7>(paired, p, it, n, grid, waves, lds, st);
            return launch_group_n<BITS, G64, 8>(paired, p, it, n, grid, waves, lds, st);
        }
        return launch_group_n<BITS, G64, 4>(paired, p, it, n, grid, waves, lds, st);
    }
}

int dispatch_group(int bits, bool g64, int nslot, bool paired, const GemvArgs *p, const GroupItem *it, int n, int grid,
                   int waves, size_t lds, hipStream_t st)
{
    switch (bits) {
    case 1: return g64 ? launch_group<1, true>(nslot, paired, p, it, n, grid, waves, lds, st) : launch_group<1, false>(nslot, paired, p, it, n, grid, waves, lds, st);
    case 2: return g64 ? launch_group<2, true>(nslot, paired, p, it, n, grid, waves, lds, st) : launch_group<2, false>(nslot, paired, p, it, n, grid, waves, lds, st);
    case 3: return g64 ? launch_group<3, true>(nslot, paired, p, it, n, grid, waves, lds, st) : launch_group<3, false>(nslot, paired, p, it, n, grid, waves, lds, st);
    case 4: return g64 ? launch_group<4, true>(nslot, paired, p, it, n, grid, waves, lds, st) : launch_group<4, false>(nslot, paired, p, it, n, grid, waves, lds, st);
    }
    return ELUTQ_ERR_BITS;
}

// paired_ok for run-time plane count / group size / slot count
bool paired_ok_rt(int bits, bool g64, int nslot, int spw, int ups, int ksplit)
{
    const int size = g64 ? bits : 2 * bits;
    return nslot % size == 0 && spw % size == 0 && (g64 || ksplit == 1 || ups % 2 == 0);
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

// Launch shape (measured on MI355X): 16 waves per workgroup so that every SIMD has several
// waves to hide LDS latency with; K is sliced only where it has to be -- when the column
// blocks alone leave most CUs idle (N < 4096), or when a slice longer than 32 units would
// give a wave a run of more than four sub-tasks at w2 (every slice adds partial-sum
// traffic and three dependent trips through device memory to the tail of the kernel).
void choose_shape(const HlqGeo &g, int &ksplit, int &waves)
{
    if (ksplit <= 0) {
        ksplit = g.ncb >= 64 ? 1 : NUM_CU / g.ncb;
        // more than four sub-tasks per wave (3 and 4 planes at K = 4096): slice while that still leaves
        // at most one workgroup per CU
        const int by_slots = (g.U * g.bits + 16 * depth_of(g.bits) - 1) / (16 * depth_of(g.bits));
        if (g.U * g.bits > 16 * 4 && g.ncb < 128) {
            const int fill = NUM_CU / g.ncb > by_slots ? NUM_CU / g.ncb : by_slots;
            if (ksplit < fill) ksplit = fill;
        }
        if (ksplit > 4) ksplit = 4;
        // slices of at most 32 units (one table-build pass of 1024 lanes); with workgroups to spare anyway
        // a slice of up to 48 units in two passes beats a second slice and its exchange (K = 5120: 9.5 -> 8.9 us)
        const int max_ups = g.ncb >= 128 ? 48 : 32;
        const int by_len = (g.U + max_ups - 1) / max_ups;
        if (ksplit < by_len) ksplit = by_len;
        if (ksplit > g.U) ksplit = g.U;
    }
    if (waves <= 0) waves = 16;
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
    return hlq_gemv_with_extra(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                               workspace_bytes, stream, fusion, ksplit, waves, nullptr);
}

}  // extern "C"

// The fused GEMV with an fp32 vector [N] added to every output before it is rounded to fp16
// (the block-sparse extra plane of a use_sparse layer, computed by another kernel on the same stream).
int hlq_gemv_with_extra(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                        const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                        size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion, int ksplit,
                        int waves, const float *d_extra)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.U) return ELUTQ_ERR_TUNING;
    const bool auto_waves = waves <= 0;
    choose_shape(g, ksplit, waves);
    int ups = (g.U + ksplit - 1) / ksplit;
    // shrink the slice so its tables fit in LDS, then the slice count so that no slice is empty
    while (gemv_lds_bytes(ups, bits, waves) > (size_t)MAX_LDS) ups = (ups + 1) / 2;
    ksplit = (g.U + ups - 1) / ups;
    // a slice of at most 16 sub-tasks: eight waves with two each start sooner than sixteen with one
    if (auto_waves && ups * bits <= 16) waves = 8;

    GemvArgs a;
    a.planes = (const HLQ_GLOBAL uint4 *)d_planes;
    a.scales = (const HLQ_GLOBAL uint32_t *)d_scales;
    a.zeros = (const HLQ_GLOBAL uint32_t *)d_zeros;
    a.bias = (const HLQ_GLOBAL uint16_t *)d_bias;
    a.x = (const HLQ_GLOBAL uint16_t *)d_x;
    a.y = (HLQ_GLOBAL uint16_t *)d_y;
    a.N = N; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb;
    a.ksplit = ksplit; a.ups = ups;
    const WavePlan wp = wave_plan(ups, bits, waves);
    a.spw = wp.spw; a.nuw_max = wp.nuw_max; a.wave_lds = wp.wave_lds;
    a.partial = nullptr; a.counters = nullptr;
    a.prologue = 0; a.eps = 0.f; a.norm_w = nullptr; a.residual = nullptr; a.extra = nullptr;
    a.defer = 0; a.n_slices_in = 0; a.slices_in = nullptr; a.x_out = nullptr;
    if (fusion) {
        if (fusion->prologue < 0 || fusion->prologue > 2) return ELUTQ_ERR_TUNING;
        if (fusion->prologue == 1 && !fusion->d_norm_weight) return ELUTQ_ERR_NULL;
        a.prologue = fusion->prologue;
        a.eps = fusion->eps;
        a.norm_w = (const HLQ_GLOBAL uint16_t *)fusion->d_norm_weight;
        a.residual = (const HLQ_GLOBAL uint16_t *)fusion->d_residual;
    }
    a.extra = (const HLQ_GLOBAL float *)d_extra;
    size_t stage_bytes = 0;
    if (fusion && fusion->n_slices_in != 0) {
        // x arrives as a base vector plus the unsummed K slices of the launch that produced it
        if (fusion->n_slices_in < 0 || fusion->n_slices_in > GEMV_MAX_SLICES_IN || fusion->prologue != 1) return ELUTQ_ERR_TUNING;
        if (!fusion->d_slices_in) return ELUTQ_ERR_NULL;
        a.n_slices_in = fusion->n_slices_in;
        a.slices_in = (const HLQ_GLOBAL float *)fusion->d_slices_in;
        if (fusion->d_x_out == d_x) return ELUTQ_ERR_TUNING;       // other workgroups still read the base
        // only launches of one tile per workgroup take slices: the instances that walk a run of column
        // blocks (more tiles than compute units) have not been validated as consumers
        if ((long long)g.ncb * ksplit > NUM_CU) return ELUTQ_ERR_TUNING;
        a.x_out = (HLQ_GLOBAL uint16_t *)fusion->d_x_out;
        stage_bytes = (size_t)K * sizeof(uint16_t);
        if (gemv_lds_bytes(ups, bits, waves) + stage_bytes > (size_t)MAX_LDS) return ELUTQ_ERR_SHAPE;
    }
    if (fusion && fusion->d_slices_out) {
        // the K slices stay unsummed for the next launch: nothing else may be due in the output stage
        if (ksplit < 2 || d_bias || a.residual || d_extra || N % HLQ_CB != 0) return ELUTQ_ERR_TUNING;
        a.defer = 1;
        a.partial = (HLQ_GLOBAL float *)fusion->d_slices_out;
    } else if (ksplit > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ksplit * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        a.counters = (HLQ_GLOBAL unsigned *)d_workspace;
        a.partial = (HLQ_GLOBAL float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
    }
    return dispatch_gemv(a, bits, group, waves, gemv_lds_bytes(ups, bits, waves) + stage_bytes, (hipStream_t)stream);
}

// Whether a launch of this shape (ksplit / waves as the call would pass them) takes `n_slices` handed-over
// K slices in its RMSNorm prologue: the same steps and limits as the launch itself.
extern "C" int elutq_hlq_gemv_accepts_slices(int K, int N, int bits, int group, int ksplit, int waves, int n_slices)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK) return 0;
    if (n_slices < 1 || n_slices > GEMV_MAX_SLICES_IN) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.U) return 0;
    choose_shape(g, ksplit, waves);
    int ups = (g.U + ksplit - 1) / ksplit;
    while (gemv_lds_bytes(ups, bits, waves) > (size_t)MAX_LDS) ups = (ups + 1) / 2;
    ksplit = (g.U + ups - 1) / ups;
    if ((long long)g.ncb * ksplit > NUM_CU) return 0;
    return gemv_lds_bytes(ups, bits, waves) + (size_t)K * sizeof(uint16_t) <= (size_t)MAX_LDS ? 1 : 0;
}

extern "C" int elutq_hlq_gemv_slices(int K, int N, int bits, int group, int ksplit, int waves)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.U) return 0;
    choose_shape(g, ksplit, waves);                      // the same steps as the launch itself
    int ups = (g.U + ksplit - 1) / ksplit;
    while (gemv_lds_bytes(ups, bits, waves) > (size_t)MAX_LDS) ups = (ups + 1) / 2;
    return (g.U + ups - 1) / ups;
}

extern "C" {

// ---- grouped launch of independent GEMVs --------------------------------------------------
struct GroupShape {                      // tile shape of one problem inside a group
    HlqGeo g;
    int ksplit, ups;
    WavePlan wp;
};

static int group_shape(const elutq_gemv_problem &p, int bits, int group, GroupShape &sh)
{
    int rc = check_shape(p.K, p.N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!p.d_planes || !p.d_scales || !p.d_zeros || !p.d_x || !p.d_y) return ELUTQ_ERR_NULL;
    sh.g = hlq_geo(p.K, p.N, bits, group);
    // the list supplies the parallelism: slice K only as far as LDS and the run length ask for
    // (a wave's run must fit its slots: at most 16 * depth_of(bits) sub-tasks per slice)
    const int DEPTH = depth_of(bits);
    int ksplit = (sh.g.U * bits + 16 * DEPTH - 1) / (16 * DEPTH);
    int ups = (sh.g.U + ksplit - 1) / ksplit;
    while (ups > 1 && (gemv_lds_bytes(ups, bits, 16) > (size_t)MAX_LDS / 2 ||            // two workgroups per CU
                       wave_plan(ups, bits, 16).spw > DEPTH))                            // whole units per wave may round the run up
        ups--;
    sh.ups = ups;
    sh.ksplit = (sh.g.U + ups - 1) / ups;
    sh.wp = wave_plan(ups, bits, 16);
    return ELUTQ_OK;
}

struct GemvGroupPlan {
    int bits, group, nslot, n_items, grid;
    bool paired;
    size_t lds;
    GemvArgs *d_problems;
    GroupItem *d_items;
};

static size_t group_layout(const elutq_gemv_problem *problems, int count, int bits, int group,
                           std::vector<GroupShape> *shapes, std::vector<size_t> *counter_off, std::vector<size_t> *partial_off,
                           int *rc_out)
{
    size_t counters = 0, partials = 0;
    *rc_out = ELUTQ_OK;
    for (int i = 0; i < count; i++) {
        GroupShape sh;
        const int rc = group_shape(problems[i], bits, group, sh);
        if (rc != ELUTQ_OK) { *rc_out = rc; return 0; }
        if (shapes) shapes->push_back(sh);
        if (counter_off) counter_off->push_back(counters);
        if (partial_off) partial_off->push_back(partials);
        if (sh.ksplit > 1) {
            counters += (size_t)sh.g.ncb * sizeof(unsigned);
            partials += (size_t)sh.ksplit * sh.g.ncb * HLQ_CB * sizeof(float);
        }
    }
    counters = (counters + 255) & ~(size_t)255;
    if (partial_off)
        for (auto &o : *partial_off) o += counters;
    return counters + partials + 256;
}

size_t elutq_hlq_gemv_group_workspace_bytes(const elutq_gemv_problem *problems, int count, int bits, int group)
{
    if (!problems || count < 1) return 0;
    int rc;
    const size_t n = group_layout(problems, count, bits, group, nullptr, nullptr, nullptr, &rc);
    return rc == ELUTQ_OK ? n : 0;
}

int elutq_hlq_gemv_group_create(const elutq_gemv_problem *problems, int count, int bits, int group, void *d_workspace,
                                size_t workspace_bytes, void **plan_out)
{
    if (!problems || !plan_out) return ELUTQ_ERR_NULL;
    if (count < 1) return ELUTQ_ERR_SHAPE;
    *plan_out = nullptr;
    std::vector<GroupShape> shapes;
    std::vector<size_t> coff, poff;
    int rc;
    const size_t need = group_layout(problems, count, bits, group, &shapes, &coff, &poff, &rc);
    if (rc != ELUTQ_OK) return rc;
    bool any_split = false;
    for (auto &sh : shapes) any_split |= sh.ksplit > 1;
    if (any_split) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if (workspace_bytes < need) return ELUTQ_ERR_WORKSPACE;
    }
    std::vector<GemvArgs> args(count);
    std::vector<GroupItem> items;
    // column blocks per tile: long runs amortise the table build, as long as every CU still gets a tile
    long total_cbs = 0;
    for (auto &sh : shapes) total_cbs += (long)sh.g.ncb * sh.ksplit;
    int cbs_per_item = (int)((total_cbs + NUM_CU - 1) / NUM_CU);
    if (cbs_per_item > 16) cbs_per_item = 16;
    if (cbs_per_item < 1) cbs_per_item = 1;
    int nslot = 1;
    size_t lds = 0;
    for (int i = 0; i < count; i++) {
        const GroupShape &sh = shapes[i];
        GemvArgs &a = args[i];
        a.planes = (const HLQ_GLOBAL uint4 *)problems[i].d_planes;
        a.scales = (const HLQ_GLOBAL uint32_t *)problems[i].d_scales;
        a.zeros = (const HLQ_GLOBAL uint32_t *)problems[i].d_zeros;
        a.bias = (const HLQ_GLOBAL uint16_t *)problems[i].d_bias;
        a.x = (const HLQ_GLOBAL uint16_t *)problems[i].d_x;
        a.y = (HLQ_GLOBAL uint16_t *)problems[i].d_y;
        a.N = problems[i].N; a.U = sh.g.U; a.NT = sh.g.NT; a.ncb = sh.g.ncb;
        a.ksplit = sh.ksplit; a.ups = sh.ups;
        a.spw = sh.wp.spw; a.nuw_max = sh.wp.nuw_max; a.wave_lds = sh.wp.wave_lds;
        a.partial = nullptr; a.counters = nullptr;
        if (sh.ksplit > 1) {
            a.counters = (HLQ_GLOBAL unsigned *)((unsigned char *)d_workspace + coff[i]);
            a.partial = (HLQ_GLOBAL float *)((unsigned char *)d_workspace + poff[i]);
        }
        a.prologue = 0; a.eps = 0.f; a.norm_w = nullptr; a.residual = nullptr; a.extra = nullptr;
        a.defer = 0; a.n_slices_in = 0; a.slices_in = nullptr; a.x_out = nullptr;
        const int ns = a.spw < depth_of(bits) ? a.spw : depth_of(bits);
        if (ns > nslot) nslot = ns;
        const size_t l = gemv_lds_bytes(sh.ups, bits, 16);
        if (l > lds) lds = l;
        // runs of column blocks share one table build
        for (int sl = 0; sl < sh.ksplit; sl++)
            for (int cb0 = 0; cb0 < sh.g.ncb; cb0 += cbs_per_item) {
                const int len = sh.g.ncb - cb0 < cbs_per_item ? sh.g.ncb - cb0 : cbs_per_item;
                items.push_back(GroupItem{i, cb0, sl, len});
            }
    }
    GemvGroupPlan *pl = new GemvGroupPlan();
    pl->bits = bits; pl->group = group; pl->nslot = nslot; pl->n_items = (int)items.size(); pl->lds = lds;
    pl->paired = true;
    for (auto &sh : shapes) pl->paired = pl->paired && paired_ok_rt(bits, group == 64, nslot, sh.wp.spw, sh.ups, sh.ksplit);
    // as many workgroups as the chip holds at once: each walks the list with that stride
    int per_cu = dispatch_group(bits, group == 64, nslot, pl->paired, nullptr, nullptr, 0, -1, 16, lds, nullptr);
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 2) per_cu = 2;
    const int slots = NUM_CU * per_cu;
    pl->grid = pl->n_items < slots ? pl->n_items : slots;
    pl->d_problems = nullptr; pl->d_items = nullptr;
    if (hipMalloc((void **)&pl->d_problems, args.size() * sizeof(GemvArgs)) != hipSuccess ||
        hipMalloc((void **)&pl->d_items, items.size() * sizeof(GroupItem)) != hipSuccess ||
        hipMemcpy(pl->d_problems, args.data(), args.size() * sizeof(GemvArgs), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(pl->d_items, items.data(), items.size() * sizeof(GroupItem), hipMemcpyHostToDevice) != hipSuccess) {
        if (pl->d_problems) (void)hipFree(pl->d_problems);
        if (pl->d_items) (void)hipFree(pl->d_items);
        delete pl;
        return ELUTQ_ERR_HIP;
    }
    *plan_out = pl;
    return ELUTQ_OK;
}

int elutq_hlq_gemv_group_run(void *plan, void *stream)
{
    if (!plan) return ELUTQ_ERR_NULL;
    const GemvGroupPlan *pl = (const GemvGroupPlan *)plan;
    return dispatch_group(pl->bits, pl->group == 64, pl->nslot, pl->paired, pl->d_problems, pl->d_items, pl->n_items, pl->grid, 16,
                          pl->lds, (hipStream_t)stream);
}

int elutq_hlq_gemv_group_destroy(void *plan)
{
    if (!plan) return ELUTQ_ERR_NULL;
    GemvGroupPlan *pl = (GemvGroupPlan *)plan;
    const bool ok = hipFree(pl->d_problems) == hipSuccess && hipFree(pl->d_items) == hipSuccess;
    delete pl;
    return ok ? ELUTQ_OK : ELUTQ_ERR_HIP;
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

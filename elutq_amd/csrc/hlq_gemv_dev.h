// Device-side building blocks shared by the batch-1 GEMV kernels (hlq_gemv.hip: the LUT kernel,
// hlq_gemv_mfma.hip: the matrix-core kernel): the kernel argument block, activation loads with the
// optional RMSNorm / SiLU*up prologues, the per-chunk lookup tables, barriers that order LDS traffic
// only, and the combination of handed-over K slices.  Everything lives in an anonymous namespace of
// the including source file.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
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
    HLQ_GLOBAL unsigned *counters;      // [ncb], zero between calls (meet_slots == 0)
    int meet_slots;                     // 1: `partial` [ksplit - 1][ncb*64] is all-zero bits between calls and the slices
                                        // meet by filling and emptying it (slices_meet); 0: arrival counters
    int N, U, NT, ncb;
    int K;                   // activations: 128 U, or 64 fewer where K ends half way through the last unit (G = 64)
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
    int lut_int8;                         // host side only: launch the instance whose tables are quantized to int8 (GEMV_INT8)
    // the slot meeting's bounded wait (meet_slots == 1)
    HLQ_GLOBAL unsigned *fault;           // the library's count of meetings that gave up (never null when meet_slots)
    int spin_limit;                       // polls before a waiting wave gives up
    int drop_slice;                       // -1; tests only: this slice leaves without storing its sums, so that the wait runs out
    // block-sparse extra plane looked up in the tables the tile has built anyway (GEMV_SPARSE instances; hlq_layout.h:
    // the inline form of a sparse plane): record index per (column block, unit) or -1, and the records
    const HLQ_GLOBAL int32_t *sp_cells;        // [ncb][U]
    const HLQ_GLOBAL unsigned char *sp_recs;   // [records][HLQ_SP_REC_BYTES]
    int sp_nrec;                               // records behind sp_recs: a number outside [0, sp_nrec) counts as "no block"
};

// One tile of a grouped launch (many independent GEMVs in one launch): a run of consecutive column blocks of one
// K slice of one problem of the list.
struct GroupItem {
    int problem, cb, slice;  // first column block and K slice
    int ncb_run;             // consecutive column blocks of that slice
};

typedef __attribute__((address_space(3))) const int lds_cint;

__device__ __forceinline__ int lds_ld(uint32_t addr, int imm)
{
    return *(lds_cint *)(uintptr_t)(addr + (uint32_t)imm);
}

__device__ __forceinline__ float h2f_lo(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v & 0xffffu)); }
__device__ __forceinline__ float h2f_hi(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(v >> 16)); }

// dst = base | src.byte<SEL>: the table address of one lookup.  `src` is a plane dword (or its
// rotation by 4) masked to bits 2..5 of every byte, i.e. 4 * nibble; `base` (a multiple of 64) is the
// LDS address of the unit's tables: wave-uniform where all lanes of a wave work on the same unit
// (HLQ_SDWA_OR), a vector register where they do not (HLQ_SDWA_OR_V).
#define HLQ_SDWA_OR(dst, base, src, SEL)                                                       \
    asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD "         \
        "src1_sel:BYTE_" #SEL                                                                  \
        : "=v"(dst)                                                                            \
        : "s"(base), "v"(src))
#define HLQ_SDWA_OR_V(dst, base, src, SEL)                                                     \
    asm("v_or_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD "         \
        "src1_sel:BYTE_" #SEL                                                                  \
        : "=v"(dst)                                                                            \
        : "v"(base), "v"(src))

// Eight lookups for one plane dword (32 k): chunks 8*D .. 8*D+7 of the unit.  Issue and sum are
// separate so that the lookups of the next dword are on their way to LDS before the wave waits
// for the results of this one (LDS returns a wave's reads in order).  VBASE: `base` differs between lanes.
template <int D, bool VBASE = false>
__device__ __forceinline__ void lookup_issue(uint32_t w, uint32_t base, int (&v)[8])
{
    const uint32_t wm = w & 0x3C3C3C3Cu;
    const uint32_t rm = __builtin_amdgcn_alignbit(w, w, 4) & 0x3C3C3C3Cu;
    uint32_t a[8];
    if constexpr (VBASE) {
        HLQ_SDWA_OR_V(a[0], base, wm, 0);
        HLQ_SDWA_OR_V(a[1], base, rm, 0);
        HLQ_SDWA_OR_V(a[2], base, wm, 1);
        HLQ_SDWA_OR_V(a[3], base, rm, 1);
        HLQ_SDWA_OR_V(a[4], base, wm, 2);
        HLQ_SDWA_OR_V(a[5], base, rm, 2);
        HLQ_SDWA_OR_V(a[6], base, wm, 3);
        HLQ_SDWA_OR_V(a[7], base, rm, 3);
    } else {
        HLQ_SDWA_OR(a[0], base, wm, 0);
        HLQ_SDWA_OR(a[1], base, rm, 0);
        HLQ_SDWA_OR(a[2], base, wm, 1);
        HLQ_SDWA_OR(a[3], base, rm, 1);
        HLQ_SDWA_OR(a[4], base, wm, 2);
        HLQ_SDWA_OR(a[5], base, rm, 2);
        HLQ_SDWA_OR(a[6], base, wm, 3);
        HLQ_SDWA_OR(a[7], base, rm, 3);
    }
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
__device__ __forceinline__ float prologue_value(int prologue, float v, float w, float rstd)
{
    float t;
    if (prologue == 1) t = v * rstd * w;
    else t = v / (1.0f + __expf(-v)) * w;
    return (float)(_Float16)t;
}

__device__ __forceinline__ void chunk_values(int prologue, uint2 raw, uint2 raw2, float rstd, float (&v)[4])
{
    v[0] = h2f_lo(raw.x); v[1] = h2f_hi(raw.x); v[2] = h2f_lo(raw.y); v[3] = h2f_hi(raw.y);
    if (prologue == 0) return;
    const float w[4] = {h2f_lo(raw2.x), h2f_hi(raw2.x), h2f_lo(raw2.y), h2f_hi(raw2.y)};
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = prologue_value(prologue, v[i], w[i], rstd);
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
                                            float2 *half, bool leader, int rot_lane)
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
    // Entry e = b0 + 2 b1 + 4 b2 + 8 b3 holds b0 i0 + b1 i1 + b2 i2 + b3 i3; quarter qq = (b2, b3) of the table is one
    // 16-byte store.  A table is 64 bytes at a 64-byte lane stride, so lanes two apart would hit the same banks with
    // the same quarter: every lane therefore starts with quarter (lane / 2) % 4 and goes round from there, and the
    // stores of any eight neighbouring lanes fall into 32 different banks.
    const int e3 = i0 + i1;
    int4 *dst = (int4 *)tbl;
    const int rot = (rot_lane >> 1) & 3;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int qq = (q + rot) & 3;
        const int base = ((qq & 1) ? i2 : 0) + ((qq & 2) ? i3 : 0);
        dst[qq] = make_int4(base, base + i0, base + i1, base + e3);
    }
    if (leader) *half = make_float2(s, inv);
}

// The same table with the entries quantized as the reference's int8-LUT variant quantizes them
// (t_mac_g4_groupsize32_calculate_lut_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:15-93): every entry is the fp16
// sum of its activations added in ascending order (:22-48), the quantization group's scale is
// fp16(max|entry| / 127) (:50) and an entry becomes round-to-nearest-even(fp16(entry / scale)), saturated to int8
// (:59-90).  The entries are stored as int32 like the exact ones, so the lookups and their integer sums are the
// same code; *half gets the scale in place of the exact tables' power of two.  A group of zeros has scale 0 and
// zero entries.  The 16 lanes of a DPP row cover 64 activations: one group at G = 64, half of one at G = 128,
// where the rows of a unit's two halves exchange their maxima.
template <bool G64>
__device__ __forceinline__ void build_chunk_int8(uint2 raw, unsigned char *tbl, float2 *half, bool leader)
{
    const _Float16 a[4] = {__builtin_bit_cast(_Float16, (uint16_t)(raw.x & 0xffffu)), __builtin_bit_cast(_Float16, (uint16_t)(raw.x >> 16)),
                           __builtin_bit_cast(_Float16, (uint16_t)(raw.y & 0xffffu)), __builtin_bit_cast(_Float16, (uint16_t)(raw.y >> 16))};
    float s = ((float)a[0] + (float)a[1]) + ((float)a[2] + (float)a[3]);
    HLQ_ROW_REDUCE(s, op_add);
    _Float16 e[16];
    e[0] = (_Float16)0.f;
    float m = 0.f;
#pragma unroll
    for (int g = 1; g < 16; g++) {
        const int top = g >= 8 ? 3 : (g >= 4 ? 2 : (g >= 2 ? 1 : 0));          // the activation added last
        e[g] = (g & ~(1 << top)) ? (_Float16)(e[g & ~(1 << top)] + a[top]) : a[top];
        m = fmaxf(m, fabsf((float)e[g]));
    }
    HLQ_ROW_REDUCE(m, op_max);
    if (!G64) m = fmaxf(m, __shfl_xor(m, 16, 64));
    const float scale = (float)(_Float16)(m / 127.0f);
    int q[16];
#pragma unroll
    for (int g = 0; g < 16; g++) {
        const float r = rintf((float)(_Float16)((float)e[g] / scale));
        q[g] = scale != 0.f ? (int)fminf(fmaxf(r, -128.f), 127.f) : 0;
    }
    // (the quarters go out in table order: picking them by the lane's rotation, as build_chunk does to spread the
    // stores over the banks, would cost a chain of selects per entry here)
    int4 *dst = (int4 *)tbl;
#pragma unroll
    for (int i = 0; i < 4; i++) dst[i] = make_int4(q[4 * i], q[4 * i + 1], q[4 * i + 2], q[4 * i + 3]);
    if (leader) *half = make_float2(s, scale);
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

// The K slices of a column block meet in device memory without an arrival counter.  A slot of `partial`
// holds all-zero bits while it is empty (the workspace starts zero-filled); a slice stores its sum with an
// agent-scope store (+0.0 goes in as -0.0, which adds the same) and leaves.  The workgroup of the last slice
// keeps its own sum in registers, reads the other slots until none is empty, adds them in slice order and puts
// the zeros back.  One trip through memory lies between the last store and the result (the counter needed
// three dependent ones: store acknowledged, ticket drawn, slots read).
//
// Who waits is fixed, so the others must be certain to run.  The last slice has the highest workgroup index of its
// column block (slices are the fastest grid dimension).  Workgroups go to the eight XCDs of the chip round robin by
// index and every XCD places its own in index order, so with 2, 4 or 8 slices -- the only counts the launcher uses
// slots for -- waiting workgroups sit on XCDs 1, 3, 5, 7 only and each waits for XCDs with lower numbers: XCD 0
// never holds a waiter and drains whatever else shares the GPU, then XCD 1's waiters have what they wait for, and so
// on up (tests/test_slot_meeting_model.py replays that placement for several launches sharing the chip, and shows
// the cycle that three slices allow).  The argument rests on how the dispatcher places workgroups, which no document
// promises, so the wait is bounded all the same (GemvArgs.spin_limit polls, about a second by default).  A wave that
// gives up does not pass a partial result off as a sum: it counts the event in the library's fault word
// (elutq_hlq_gemv_fault_count), makes its 64 outputs NaN, and empties the slots it can see; a slice that arrives
// later still dirties its slot, so after a fault the workspace must be zero-filled again before it is reused.
constexpr int SLICE_SPIN_LIMIT = 1 << 20;

// Called by one whole wave (lane = column n of the block); true in the wave that holds the complete sum.
__device__ __forceinline__ bool slices_meet_slots(const GemvArgs &a, int slice, size_t npad, int n, float total, float &sum)
{
    HLQ_GLOBAL float *mine = a.partial + (size_t)slice * npad + n;
    if (slice != a.ksplit - 1) {
        if (slice == a.drop_slice) return false;        // (tests of the give-up path)
        const float v = __float_as_uint(total) == 0u ? -0.0f : total;
        __hip_atomic_store(mine, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    sum = 0.f;
    const int others = a.ksplit - 1;
    int spins = 0;
    bool gave_up = false;
    for (int s0 = 0; s0 < others; s0 += 8) {            // eight independent loads in flight at a time
        float v[8];
        for (;;) {
            bool here = true;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int sl = min(s0 + j, others - 1);
                v[j] = __hip_atomic_load(&a.partial[(size_t)sl * npad + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                here = here && __float_as_uint(v[j]) != 0u;
            }
            if (__all(here)) break;
            if (++spins > a.spin_limit) { gave_up = true; break; }
            __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (s0 + j < others) {
                sum += v[j];
                __hip_atomic_store(&a.partial[(size_t)(s0 + j) * npad + n], 0.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
    }
    sum += total;
    if (gave_up) {                                      // wave-uniform
        sum = __builtin_nanf("");
        if ((n & (HLQ_CB - 1)) == 0) __hip_atomic_fetch_add(a.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// The same meeting with an arrival counter per column block, for launches whose slots would not fit the
// zero-kept head of the workspace and for grouped launches: partial sums are written and read with agent-scope atomics (they bypass the
// per-XCD L2s' non-coherent lines), the writer waits for its stores to be acknowledged before it takes a
// ticket, and the reader's loads depend on the ticket it drew -- so no cache write-back / invalidate is
// needed.  The last workgroup to arrive sums in slice order.  Nothing waits for another workgroup.
__device__ __forceinline__ bool slices_meet_ticket(const GemvArgs &a, int cb, int slice, size_t npad, int n, int lane,
                                                   float total, float &sum)
{
    __hip_atomic_store(&a.partial[(size_t)slice * npad + n], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(&a.counters[cb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __builtin_amdgcn_readfirstlane(ticket);
    if (ticket != (unsigned)a.ksplit - 1u) return false;
    sum = 0.f;
    for (int s0 = 0; s0 < a.ksplit; s0 += 8) {          // eight independent loads in flight at a time
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
    if (lane == 0) __hip_atomic_store(&a.counters[cb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

__device__ __forceinline__ bool slices_meet(const GemvArgs &a, int cb, int slice, size_t npad, int n, int lane, float total,
                                            float &sum)
{
    if (a.meet_slots) return slices_meet_slots(a, slice, npad, n, total, sum);
    return slices_meet_ticket(a, cb, slice, npad, n, lane, total, sum);
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

// Which optional inputs a kernel instance reads, known when it is compiled:
//   GEMV_FUSED  prologue, residual and the fp32 term `extra` as the argument block says (the decode step's launches)
//   GEMV_PLAIN  none of them (their fields are not read)
//   GEMV_EXTRA  plain, plus the fp32 term `extra` added before the output is rounded
//   GEMV_INT8   plain, with the tables quantized to int8 per group (build_chunk_int8)
//   GEMV_SPARSE fused, plus the blocks of a block-sparse extra plane looked up in the unit's tables (sp_cells, sp_recs)
enum { GEMV_FUSED = 0, GEMV_PLAIN = 1, GEMV_EXTRA = 2, GEMV_INT8 = 3, GEMV_SPARSE = 4 };

// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

}  // namespace

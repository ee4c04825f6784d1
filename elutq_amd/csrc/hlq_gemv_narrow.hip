// Batch-1 HLQ LUT GEMV for layers with fewer column blocks than the chip has compute units
// (same computation, layout and tables as hlq_gemv.hip; replaces the same reference functions,
// C++/ops/src/arm/arm_gemm.cpp:312-360 and C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469).
//
// The wide-tile kernel gives a wave 64 columns of one unit (128 k) per instruction, so a layer of
// N columns has N / 64 independent tiles; with fewer tiles than compute units it has to cut K across
// workgroups, and the slices then meet through device memory -- three dependent round trips at the
// end of a launch that is only a few microseconds long.  Here a wave instruction covers CW = 16 or 32
// columns of 64 / CW units at once (lane = column c + CW * unit lane), and a workgroup owns CW columns
// over the whole of K: four or two times as many workgroups, no meeting.  Lanes of one instruction
// then read the tables of different units, so a wave keeps the tables of its units 16 banks apart
// (one spare table between units) and the lookups stay free of bank conflicts.  The per-column sums
// of the unit lanes meet in the final cross-wave sum through LDS.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"

#include "hlq_gemv_dev.h"

namespace {

constexpr int UNIT_STRIDE = HLQ_NARROW_UNIT_STRIDE;           // tables of a unit plus the spare one

template <int CW, int R>
struct NarrowGeo {
    static constexpr int UL = 64 / CW;           // units one wave instruction covers (unit lanes)
    static constexpr int NU = UL * R;            // units of a wave: R rounds
    static constexpr int PASSES = NU / 2;        // table-build passes of 64 chunks
    // tables [NU][33][16] int32, then the half-unit records float2 [2 * NU] (hlq_narrow_wave_lds)
    static constexpr int WAVE_LDS = (NU * UNIT_STRIDE + 2 * NU * 8 + 255) & ~255;
};

// dynamic LDS: [waves][WAVE_LDS] | float [waves][64] cross-wave sums | float [HLQ_RSTD_SCRATCH] | gap |
// fp16 [K] staged activations (launches that take handed-over slices only)
template <int CW, int R>
size_t narrow_lds_bytes(int waves)
{
    static_assert(NarrowGeo<CW, R>::WAVE_LDS == (NarrowGeo<CW, R>::NU * HLQ_NARROW_UNIT_STRIDE + 2 * NarrowGeo<CW, R>::NU * 8 + 255) / 256 * 256, "");
    return hlq_narrow_lds(NarrowGeo<CW, R>::NU, waves).stage;
}

// The lookups of one sub-task (128 k of one plane) where every lane has its own unit: `ub` is the LDS
// address of the lane's unit tables, `xs` its two half-unit records.  Same arithmetic as process_sub.
template <bool G64>
__device__ __forceinline__ float process_sub_lane(const uint4 &w, uint32_t sc_raw, uint32_t zz_raw, uint32_t ub,
                                                  const float2 *xs, int b, int odd, float acc)
{
    int v0[8], v1[8];
    const float2 h0 = xs[0], h1 = xs[1];      // .x = sum of x, .y = 2^-p
    lookup_issue<0, true>(w.x, ub, v0);
    lookup_issue<1, true>(w.y, ub, v1);
    __builtin_amdgcn_sched_barrier(0);
    // (the empty statements pin each sum in front of the scheduling barrier that follows it: a pure integer add
    // has no place of its own in the instruction order, and the lookups of a whole round piled up in registers)
    int i0 = lookup_sum(v0, 0);
    asm volatile("" : "+v"(i0));
    lookup_issue<2, true>(w.z, ub, v0);
    __builtin_amdgcn_sched_barrier(0);
    i0 = lookup_sum(v1, i0);
    asm volatile("" : "+v"(i0));
    lookup_issue<3, true>(w.w, ub, v1);
    __builtin_amdgcn_sched_barrier(0);
    int i1 = lookup_sum(v0, 0);
    i1 = lookup_sum(v1, i1);
    asm volatile("" : "+v"(i1));
    const uint32_t sh = odd ? 16u : 0u;
    const uint32_t sc = G64 ? sc_raw : ((sc_raw >> sh) & 0xffffu) * 0x10001u;
    acc = fmaf((float)i0 * h0.y, h2f_lo(sc), acc);
    acc = fmaf((float)i1 * h1.y, h2f_hi(sc), acc);
    if (b == 0) {
        const uint32_t zz = G64 ? zz_raw : ((zz_raw >> sh) & 0xffffu) * 0x10001u;
        acc = fmaf(h2f_lo(zz), h0.x, acc);
        acc = fmaf(h2f_hi(zz), h1.x, acc);
    }
    return acc;
}

// grid = ceil(N / 64) * (64 / CW) workgroups of ceil(U / NU) waves; workgroup nb owns columns
// 64 * (nb / UL) + CW * (nb % UL) + [0, CW) over all of K.
// VAR: GEMV_PLAIN (no prologue, residual or extra term), GEMV_FUSED (as the argument block says), GEMV_SPARSE (fused, plus
// the blocks of a block-sparse extra plane in its inline form: every lane looks its own unit's record up in that unit's tables).
template <int BITS, bool G64, int CW, int R, int VAR>
__global__ __launch_bounds__(1024) void hlq_gemv_narrow_kernel(const GemvArgs a)
{
    using Geo = NarrowGeo<CW, R>;
    constexpr int UL = Geo::UL, NU = Geo::NU, PASSES = Geo::PASSES;
    constexpr bool PLAIN = VAR == GEMV_PLAIN, SPARSE = VAR == GEMV_SPARSE;
    extern __shared__ __align__(256) unsigned char smem[];
    const int prologue = PLAIN ? 0 : a.prologue;
    const HLQ_GLOBAL uint16_t *residual = PLAIN ? nullptr : a.residual;
    const HLQ_GLOBAL float *extra = PLAIN ? nullptr : a.extra;      // fp32 term added before the rounding (a sparse extra plane)
    const int tid = threadIdx.x, lane = tid & 63, nw = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = a.K;
    const int cb = blockIdx.x / UL, part = blockIdx.x % UL;
    const int col = part * CW + (lane % CW);                    // column inside the column block
    const int ul = lane / CW;                                   // this lane's unit inside a round
    const int ub = wave * NU;                                   // first unit of the wave

    unsigned char *lut = smem + (size_t)wave * Geo::WAVE_LDS;
    float2 *xs_inv = (float2 *)(lut + NU * UNIT_STRIDE);
    const HlqNarrowLds lm = hlq_narrow_lds(NU, nw);
    float *red = (float *)(smem + lm.red);                      // [nw][64]
    float *rstd_scratch = (float *)(smem + lm.rstd);
    const uint32_t lut_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lut;

    // what the last step adds to the output, fetched first so that its latency is not left at the end
    const int n_out = cb * HLQ_CB + part * CW + lane;           // lanes < CW of wave 0 store
    uint16_t pre_bias = 0, pre_res = 0;
    float pre_extra = 0.f;
    if (wave == 0 && lane < CW && n_out < a.N) {
        if (a.bias) pre_bias = a.bias[n_out];
        if (residual) pre_res = residual[n_out];
        if (extra) pre_extra = extra[n_out];
    }
    // activations: chunk p * 64 + lane of the wave's NU units (clamped to K: units past the end are masked below)
    uint2 rfirst = make_uint2(0, 0);
    if (prologue == 1) rfirst = rstd_first_load(a, K, tid);
    // x as a base vector plus the unsummed K slices of the launch that produced it (host: prologue 1 only):
    // block_rstd forms every chunk once, into `stage`
    const bool sliced = !PLAIN && a.n_slices_in > 0;
    SliceChunk sfirst = {};
    uint2 *stage = (uint2 *)(smem + lm.stage);
    if (sliced) load_slice_chunk(a, K, min(tid, K / 4 - 1), sfirst);
    uint2 raw[PASSES], raw2[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        load_chunk<PLAIN>(a, prologue, K, (size_t)hlq_narrow_x_chunk(ub, p * 64 + lane, K) * 4, raw[p], raw2[p]);
    }
    // the record of this lane's unit in every round (-1: no block on its column block and unit), with the activations
    int cell[R];
    if constexpr (SPARSE) {
#pragma unroll
        for (int r = 0; r < R; r++) cell[r] = a.sp_cells[(size_t)cb * a.U + hlq_narrow_unit(ub, r, UL, ul, a.U)];
    }
    asm volatile("" ::: "memory");      // the activation loads stay ahead of the weight loads

    // every weight load of the wave, unconditional (units past the end re-read the last one)
    uint4 w[R][BITS];
    uint32_t sc[R][BITS], zz[R];
    const HLQ_GLOBAL unsigned char *pl = (const HLQ_GLOBAL unsigned char *)a.planes + (size_t)cb * a.U * (size_t)(BITS * HLQ_CB * 16);
    const HLQ_GLOBAL unsigned char *ps = (const HLQ_GLOBAL unsigned char *)a.scales + (size_t)cb * a.NT * (size_t)(BITS * HLQ_CB * 4);
    const HLQ_GLOBAL unsigned char *pz = (const HLQ_GLOBAL unsigned char *)a.zeros + (size_t)cb * a.NT * (size_t)(HLQ_CB * 4);
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t u = (uint32_t)hlq_narrow_unit(ub, r, UL, ul, a.U);
        const uint32_t row = G64 ? u : (u >> 1);
#pragma unroll
        for (int b = 0; b < BITS; b++) {
            const u32x4 v = __builtin_nontemporal_load(
                (const HLQ_GLOBAL u32x4 *)(pl + ((u * BITS + b) * (uint32_t)(HLQ_CB * 16) + (uint32_t)col * 16u)));
            w[r][b] = make_uint4(v.x, v.y, v.z, v.w);
            sc[r][b] = *(const HLQ_GLOBAL uint32_t *)(ps + ((row * BITS + b) * (uint32_t)(HLQ_CB * 4) + (uint32_t)col * 4u));
        }
        zz[r] = *(const HLQ_GLOBAL uint32_t *)(pz + (row * (uint32_t)(HLQ_CB * 4) + (uint32_t)col * 4u));
    }
    asm volatile("" ::: "memory");

    float rstd = 1.f;
    if (prologue == 1)
        rstd = block_rstd(a, K, rstd_scratch, tid, blockDim.x, rfirst, sfirst, sliced, stage, sliced && a.x_out && blockIdx.x == 0);
    if (sliced) {
#pragma unroll
        for (int p = 0; p < PASSES; p++) raw[p] = stage[hlq_narrow_x_chunk(ub, p * 64 + lane, K)];
    }
    // chunks past K (the absent half of a last unit, units no wave lane owns) count as zeros
#pragma unroll
    for (int p = 0; p < PASSES; p++)
        if ((ub * 32 + p * 64 + lane) * 4 >= K) raw[p] = make_uint2(0u, 0u);

    // the records of the units that have blocks: requested before the tables are built, looked up after the dense planes
    uint4 spw[R];
    uint32_t spsc[R];
    bool sp_any[R];
    if constexpr (SPARSE) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const bool has = cell[r] >= 0 && cell[r] < a.sp_nrec && ub + r * UL + ul < a.U;
            sp_any[r] = __builtin_amdgcn_ballot_w64(has) != 0;              // wave-uniform
            spw[r] = make_uint4(0u, 0u, 0u, 0u);
            spsc[r] = 0u;
            if (has) {
                const HLQ_GLOBAL unsigned char *rec = a.sp_recs + (size_t)cell[r] * HLQ_SP_REC_BYTES;
                const u32x4 v = *(const HLQ_GLOBAL u32x4 *)(rec + (uint32_t)col * 16u);
                spw[r] = make_uint4(v.x, v.y, v.z, v.w);
                spsc[r] = *(const HLQ_GLOBAL uint32_t *)(rec + 1024u + (uint32_t)col * 4u);
            }
        }
    }
    // the wave's own tables: chunk ci of the wave belongs to unit ci / 32, half unit ci / 16
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        const int ci = p * 64 + lane;
        build_chunk(prologue, raw[p], raw2[p], rstd, lut + hlq_narrow_table_off(ci), xs_inv + hlq_narrow_half_index(ci),
                    (lane & 15) == 0, lane);
    }
    // written by this wave, read by this wave: LDS executes a wave's operations in order
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();

    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int lu = r * UL + ul;
        const uint32_t base = lut_base + (uint32_t)lu * (uint32_t)UNIT_STRIDE;
        float t = 0.f;
#pragma unroll
        for (int b = 0; b < BITS; b++)
            t = process_sub_lane<G64>(w[r][b], sc[r][b], zz[r], base, xs_inv + 2 * lu, b, ul & 1, t);
        if constexpr (SPARSE) {
            // lanes without a block look up entry 0 of every table (the empty subset: 0) with scale 0
            if (sp_any[r]) t = process_sub_lane<true>(spw[r], spsc[r], 0u, base, xs_inv + 2 * lu, 1, 0, t);
        }
        acc += ub + lu < a.U ? t : 0.f;
    }

    // all waves and unit lanes of a column, summed in a fixed order
    red[wave * 64 + lane] = acc;
    lds_barrier();
    if (wave == 0) {
        float total = 0.f;
        for (int i = 0; i < nw; i++) total += red[i * 64 + lane];
#pragma unroll
        for (int off = CW; off < 64; off <<= 1) total += __shfl_xor(total, off, 64);
        if (lane < CW && n_out < a.N) {
            if (a.bias) total += (float)__builtin_bit_cast(_Float16, pre_bias);
            if (residual) total += (float)__builtin_bit_cast(_Float16, pre_res);
            if (extra) total += pre_extra;
            a.y[n_out] = __builtin_bit_cast(uint16_t, (_Float16)total);
        }
    }
}

template <int BITS, bool G64, int CW, int R, int VAR>
int launch_narrow_v(const GemvArgs &a, size_t stage_bytes, hipStream_t stream)
{
    using Geo = NarrowGeo<CW, R>;
    const int waves = (a.U + Geo::NU - 1) / Geo::NU;
    const size_t lds = narrow_lds_bytes<CW, R>(waves) + stage_bytes;
    if (waves < 1 || waves > 16) return ELUTQ_ERR_TUNING;
    if (lds > (size_t)MAX_LDS) return ELUTQ_ERR_SHAPE;
    auto kern = hlq_gemv_narrow_kernel<BITS, G64, CW, R, VAR>;
    static bool big_lds_done[64] = {};        // per template instance
    if (lds > 64 * 1024) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ELUTQ_ERR_HIP;
        if (!big_lds_done[dev]) {
            if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS) != hipSuccess)
                return ELUTQ_ERR_HIP;
            big_lds_done[dev] = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(a.ncb * Geo::UL), dim3(waves * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64, int CW, int R>
int launch_narrow_r(const GemvArgs &a, size_t stage_bytes, hipStream_t stream)
{
    if constexpr (BITS <= 3) {        // a layer with the extra plane has at most four planes in all
        if (a.sp_cells) return launch_narrow_v<BITS, G64, CW, R, GEMV_SPARSE>(a, stage_bytes, stream);
    }
    if (a.sp_cells) return ELUTQ_ERR_BITS;
    if (a.prologue == 0 && !a.residual && !a.extra) return launch_narrow_v<BITS, G64, CW, R, GEMV_PLAIN>(a, stage_bytes, stream);
    return launch_narrow_v<BITS, G64, CW, R, GEMV_FUSED>(a, stage_bytes, stream);
}

template <int BITS, bool G64>
int launch_narrow(const GemvArgs &a, int cw, size_t stage_bytes, hipStream_t stream)
{
    const int rounds = hlq_gemv_narrow_rounds(a.U, cw);
    if (cw == 16 && rounds == 1) return launch_narrow_r<BITS, G64, 16, 1>(a, stage_bytes, stream);
    if (cw == 32 && rounds == 1) return launch_narrow_r<BITS, G64, 32, 1>(a, stage_bytes, stream);
    if (cw == 32 && rounds == 2) return launch_narrow_r<BITS, G64, 32, 2>(a, stage_bytes, stream);
    return ELUTQ_ERR_TUNING;
}

}  // namespace

int hlq_gemv_narrow_rounds(int U, int cw)
{
    if (cw == 16) return U >= 1 && U <= 64 ? 1 : 0;
    if (cw == 32) return U >= 1 && U <= 32 ? 1 : (U <= 64 ? 2 : 0);
    return 0;
}

size_t hlq_gemv_narrow_lds_bytes(int U, int cw)
{
    const int rounds = hlq_gemv_narrow_rounds(U, cw);
    if (cw == 16 && rounds == 1) return narrow_lds_bytes<16, 1>((U + 3) / 4);
    if (cw == 32 && rounds == 1) return narrow_lds_bytes<32, 1>((U + 1) / 2);
    if (cw == 32 && rounds == 2) return narrow_lds_bytes<32, 2>((U + 3) / 4);
    return 0;
}

int hlq_gemv_narrow_launch(const void *gemv_args, size_t args_bytes, int bits, int group, int cw, size_t stage_bytes,
                           void *stream)
{
    if (args_bytes != sizeof(GemvArgs)) return ELUTQ_ERR_HIP;
    const GemvArgs &a = *(const GemvArgs *)gemv_args;
    if (a.defer) return ELUTQ_ERR_TUNING;                 // slices are left behind by the wide-tile kernel only
    const bool g64 = group == 64;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
    case 1: return g64 ? launch_narrow<1, true>(a, cw, stage_bytes, st) : launch_narrow<1, false>(a, cw, stage_bytes, st);
    case 2: return g64 ? launch_narrow<2, true>(a, cw, stage_bytes, st) : launch_narrow<2, false>(a, cw, stage_bytes, st);
    case 3: return g64 ? launch_narrow<3, true>(a, cw, stage_bytes, st) : launch_narrow<3, false>(a, cw, stage_bytes, st);
    case 4: return g64 ? launch_narrow<4, true>(a, cw, stage_bytes, st) : launch_narrow<4, false>(a, cw, stage_bytes, st);
    }
    return ELUTQ_ERR_BITS;
}

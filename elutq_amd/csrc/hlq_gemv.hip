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
#include <mutex>
#include <type_traits>
#include <vector>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"
#include "hlq_gemv_index.h"

#include "hlq_gemv_dev.h"

namespace {
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
//   GEMV_FUSED  prologue, residual and the fp32 term `a.extra` as `a` says (the decode step's launches)
//   GEMV_PLAIN  none of them (their fields of `a` are not read)
//   GEMV_EXTRA  plain, plus `a.extra`, added before the output is rounded
//   GEMV_INT8   plain, tables quantized to int8 per group as the reference's int8-LUT variant does
template <int BITS, bool G64, int NSLOT, bool MULTI, int VAR, bool PAIRED>
__device__ __forceinline__ void gemv_tile(const GemvArgs &a, int cb, int slice, int ncb_run, unsigned char *smem, int &red_sel)
{
    constexpr bool SPARSE = VAR == GEMV_SPARSE;
    constexpr bool PLAIN = VAR != GEMV_FUSED && !SPARSE;
    const int prologue = PLAIN ? 0 : a.prologue;
    const HLQ_GLOBAL uint16_t *residual = PLAIN ? nullptr : a.residual;
    const HLQ_GLOBAL float *extra = (VAR == GEMV_FUSED || VAR == GEMV_EXTRA || SPARSE) ? a.extra : nullptr;
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
    // Activations first, then the weight stream.  Every load below is unconditional (a wave
    // whose run is shorter than NSLOT re-reads its last sub-task), so the number of loads
    // behind the activations is a compile-time constant and the table build waits for the
    // activations only (vmcnt(3 * NSLOT)), with the weights still in flight.
    const int K = a.K;
    const size_t k0 = (size_t)(u0 + ub) * HLQ_UNIT;
    const int nchunks = nuw * 32;
    float rstd = 1.f;
    // what the last step adds to the output is fetched first of all, so that its latency is not
    // left at the end of the kernel (wave 0 finishes a tile; a run of column blocks loads it there)
    uint16_t pre_bias = 0, pre_res = 0;
    float pre_extra = 0.f;
    if (!MULTI && wave == 0 && cb * HLQ_CB + lane < a.N) {
        if (a.bias) pre_bias = a.bias[cb * HLQ_CB + lane];
        if (residual) pre_res = residual[cb * HLQ_CB + lane];
        if (extra) pre_extra = extra[cb * HLQ_CB + lane];
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
    // (where K ends half way through the last unit, the chunks of the absent half re-read the last one and count as zeros)
    const size_t kfirst = hlq_x_first_k(k0, nchunks, lane);
    load_chunk<PLAIN>(a, prologue, K, hlq_x_load_k(kfirst, K), raw, raw2);
    // Block-sparse extra plane: a unit's blocks are looked up by the wave that has the unit's plane 0 in its run, in the
    // tables it builds anyway.  The record numbers of the first two units of the run come in with the activations, the
    // records themselves are requested once the tables stand and arrive while the dense planes are looked up.
    // (Dealing the units that have blocks evenly to the waves, whichever wave built their tables, was measured: the
    // barrier it needs in front of the lookups costs more than the uneven work -- 8.1 against 7.5 us at 4096 x 14336.)
    int scell[2] = {-1, -1};
    bool sown[2] = {false, false};
    Sub sp[2];
    auto sp_cells_load = [&](int cbx, int (&out)[2]) __attribute__((always_inline)) {
        const HLQ_GLOBAL int32_t *row = a.sp_cells + ((size_t)cbx * a.U + u0);
#pragma unroll
        for (int j = 0; j < 2; j++) out[j] = row[min(ub + j, nU - 1)];
    };
    auto sp_recs_load = [&](int (&cell)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            cell[j] = sown[j] ? __builtin_amdgcn_readfirstlane(cell[j]) : -1;
            if (cell[j] >= a.sp_nrec) cell[j] = -1;
            if (cell[j] >= 0) {                                            // wave-uniform
                const HLQ_GLOBAL unsigned char *r = a.sp_recs + (size_t)cell[j] * HLQ_SP_REC_BYTES;
                const u32x4 v = __builtin_nontemporal_load((const HLQ_GLOBAL u32x4 *)(r + (uint32_t)lane * 16u));
                sp[j].w = make_uint4(v.x, v.y, v.z, v.w);
                sp[j].sc = *(const HLQ_GLOBAL uint32_t *)(r + 1024u + (uint32_t)lane * 4u);
            }
        }
    };
    if constexpr (SPARSE) {
#pragma unroll
        for (int j = 0; j < 2; j++) sown[j] = j < nuw && s_begin <= (ub + j) * BITS && (ub + j) * BITS < s_end;
        sp_cells_load(cb, scell);
    }
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
    if (kfirst >= (size_t)K) raw = make_uint2(0u, 0u);
    if constexpr (SPARSE) sp_recs_load(scell);      // (the record numbers came in with the activations)

    // ... the tables are built as soon as the activations are in (a wave that first queued all
    // its weight loads would sit in the memory pipeline's back-pressure instead) ...
    if (lane < nchunks) {
        if constexpr (VAR == GEMV_INT8)
            build_chunk_int8<G64>(raw, lut + (size_t)lane * TBL_BYTES, xs_inv + (lane >> 4), (lane & 15) == 0);
        else
            build_chunk(prologue, raw, raw2, rstd, lut + (size_t)lane * TBL_BYTES, xs_inv + (lane >> 4), (lane & 15) == 0, lane);
    }
    asm volatile("" ::: "memory");

    // ... and the rest of the run's loads follow.
    static_for<1, NSLOT>([&](auto dc) __attribute__((always_inline)) {
        constexpr int d = decltype(dc)::value;
        load_slot<BITS, G64, PAIRED, d>(slot[d], here, u0, min(s_begin + d, s_last), lane);
    });
    for (int ci = lane + 64; ci < nchunks; ci += 64) {      // runs of more than two units (not the common case)
        const size_t kc = k0 + (size_t)ci * 4;
        load_chunk<PLAIN>(a, prologue, K, hlq_x_load_k(kc, K), raw, raw2);
        if (sliced) raw = stage[hlq_stage_index(k0, ci, K)];
        if (kc >= (size_t)K) raw = make_uint2(0u, 0u);
        if constexpr (VAR == GEMV_INT8)
            build_chunk_int8<G64>(raw, lut + (size_t)ci * TBL_BYTES, xs_inv + (ci >> 4), (ci & 15) == 0);
        else
            build_chunk(prologue, raw, raw2, rstd, lut + (size_t)ci * TBL_BYTES, xs_inv + (ci >> 4), (ci & 15) == 0, lane);
    }
    // The tables were written by this wave and are read by this wave: LDS executes a wave's
    // operations in order, so no barrier -- only keep the compiler from reordering.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();

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
        if (a.ksplit == 1) {
            if (wave == fin && n < a.N) {
                if (a.bias) total += (float)__builtin_bit_cast(_Float16, MULTI ? a.bias[n] : pre_bias);
                if (residual) total += (float)__builtin_bit_cast(_Float16, MULTI ? residual[n] : pre_res);
                if (extra) total += MULTI ? extra[n] : pre_extra;
                a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
            }
            return;
        }
        const size_t npad = (size_t)a.ncb * HLQ_CB;
        if (!PLAIN && a.defer) {
            // the consumer is a later launch on the same stream: an ordinary store, no meeting
            if (wave == fin) a.partial[(size_t)slice * npad + n] = total;
            return;
        }
        // the slices meet through device memory (slices_meet): all but the last store and leave
        if (wave == fin) {
            float sum;
            if (slices_meet(a, cbf, slice, npad, n, lane, total, sum)) {
                if (n < a.N) {
                    if (a.bias) sum += (float)__builtin_bit_cast(_Float16, MULTI ? a.bias[n] : pre_bias);
                    if (residual) sum += (float)__builtin_bit_cast(_Float16, MULTI ? residual[n] : pre_res);
                    if (extra) sum += MULTI ? extra[n] : pre_extra;
                    a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)sum);
                }
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

    // the blocks of column block `cbx`: records in `sp` for the first two units of the run, the (rare) further units
    // of a long run fetched here
    auto sp_process = [&](int cbx, const int (&cell)[2], float accv) __attribute__((always_inline)) -> float {
#pragma unroll
        for (int j = 0; j < 2; j++)
            if (cell[j] >= 0) accv = process_sub<true>(sp[j].w, sp[j].sc, 0u, j, 1, 0, lut_base, xs_inv, accv);
        for (int j = 2; j < nuw; j++) {
            if (!(s_begin <= (ub + j) * BITS && (ub + j) * BITS < s_end)) continue;
            const int cj = __builtin_amdgcn_readfirstlane(a.sp_cells[(size_t)cbx * a.U + u0 + ub + j]);
            if (cj < 0 || cj >= a.sp_nrec) continue;
            const HLQ_GLOBAL unsigned char *r = a.sp_recs + (size_t)cj * HLQ_SP_REC_BYTES;
            const u32x4 v = *(const HLQ_GLOBAL u32x4 *)(r + (uint32_t)lane * 16u);
            const uint32_t scj = *(const HLQ_GLOBAL uint32_t *)(r + 1024u + (uint32_t)lane * 4u);
            accv = process_sub<true>(make_uint4(v.x, v.y, v.z, v.w), scj, 0u, j, 1, 0, lut_base, xs_inv, accv);
        }
        return accv;
    };

    if (MULTI) {
        for (int c = 0; c < ncb_run; c++) {
            const CbBase next = cb_base<BITS>(a, min(cb + c + 1, cb + ncb_run - 1), u0);   // past the run: a reload nobody reads
            int ncell[2] = {-1, -1};
            if constexpr (SPARSE) {
                if (c > 0) sp_recs_load(scell);
                sp_cells_load(min(cb + c + 1, cb + ncb_run - 1), ncell);
            }
            float accc = 0.f;
            if (s_begin < s_end)                              // wave-uniform; a wave without sub-tasks loads nothing here
                static_for<0, NSLOT>([&](auto dc) __attribute__((always_inline)) {
                    constexpr int d = decltype(dc)::value;
                    const int st = s_begin + d;
                    progress_prio(d, a.spw);
                    if (st < s_end) accc = run_slot(dc, st, accc);
                    load_slot<BITS, G64, PAIRED, d>(slot[d], next, u0, min(st, s_last), lane);
                });
            if constexpr (SPARSE) {
                accc = sp_process(cb + c, scell, accc);
                scell[0] = ncell[0]; scell[1] = ncell[1];
            }
            finish(cb + c, accc);
        }
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
    if constexpr (SPARSE) acc = sp_process(cb, scell, acc);
    finish(cb, acc);
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
template <int BITS, bool G64, int NSLOT, bool PAIRED, int VAR>
__global__ __launch_bounds__(1024) void hlq_gemv_run_kernel(const GemvArgs a, int run)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const int cb0 = blockIdx.y * run;               // grid = (slices, runs of column blocks)
    int sel = 0;
    gemv_tile<BITS, G64, NSLOT, true, VAR, PAIRED>(a, cb0, blockIdx.x, min(run, a.ncb - cb0), smem, sel);
}

// Many independent GEMVs in one launch: the tiles of all of them form one list that the
// workgroups walk with stride gridDim.x (tiles of one GEMV are neighbours in the list, so its
// activations stay in cache and the slices of a column block run at about the same time).
// Nothing waits for another workgroup -- slices still meet through tickets -- so the launch,
// the first memory round trips and the tail of a GEMV are paid once per list instead of once
// per GEMV, and with two workgroups per CU the sum-and-store of one tile hides under the
// lookups of another.
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
    constexpr int RUN_VAR = VAR == GEMV_PLAIN ? GEMV_PLAIN : (VAR == GEMV_SPARSE ? GEMV_SPARSE : GEMV_FUSED);
    auto kern = hlq_gemv_kernel<BITS, G64, NSLOT, PAIRED, VAR>;
    static bool big_lds_done[64] = {};        // per template instance
    if (!allow_big_lds((const void *)kern, lds, MAX_LDS, big_lds_done)) return ELUTQ_ERR_HIP;
    // more tiles than CUs and runs that fit the slots: runs of column blocks, one workgroup per CU
    const int run = (a.ncb * a.ksplit + NUM_CU_RUN - 1) / NUM_CU_RUN;
    if (VAR != GEMV_EXTRA && VAR != GEMV_INT8 && run > 1 && a.spw <= NSLOT && waves == 16) {       // (plain plus extra term, int8 tables: no run instances)
        auto kern_run = hlq_gemv_run_kernel<BITS, G64, NSLOT, PAIRED, RUN_VAR>;
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
    if constexpr (BITS <= 3) {     // a layer with the extra plane has at most four planes in all
        if (a.sp_cells) return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_SPARSE>(a, waves, lds, stream);
    }
    if (a.sp_cells) return ELUTQ_ERR_BITS;
    if (a.extra && a.prologue == 0 && !a.residual)
        return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_EXTRA>(a, waves, lds, stream);
    if (a.prologue == 0 && !a.residual && !a.extra && !a.defer && a.n_slices_in == 0)      // the plain instances read none of these fields
        return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_PLAIN>(a, waves, lds, stream);
    return launch_gemv_pp<BITS, G64, NSLOT, PAIRED, GEMV_FUSED>(a, waves, lds, stream);
}

template <int BITS, bool G64, int NSLOT>
int launch_gemv_n(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    if (a.lut_int8) {        // plain calls only, one load pattern
        if (a.prologue != 0 || a.residual || a.extra || a.defer || a.n_slices_in != 0) return ELUTQ_ERR_TUNING;
        return launch_gemv_pp<BITS, G64, NSLOT, false, GEMV_INT8>(a, waves, lds, stream);
    }
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
    if (N < 1 || !hlq_k_ok(K, group)) return ELUTQ_ERR_SHAPE;
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
        // 3 -> 4 and 5..7 -> 8 slices where the slots of the meeting then fit the head of a workspace: slots are used
        // for 2, 4 or 8 slices only (slices_meet_slots), and they cost one trip through memory where counters cost three
        const int up = ksplit == 3 ? 4 : (ksplit > 4 && ksplit < 8 ? 8 : ksplit);
        if (up != ksplit && up <= g.U && (size_t)(up - 1) * g.ncb * HLQ_CB * sizeof(float) <= (size_t)HLQ_WS_COUNTER_BYTES &&
            g.ncb * up <= NUM_CU) ksplit = up;
        if (ksplit > g.U) ksplit = g.U;
    }
    if (waves <= 0) waves = 16;
}

int g_gemv_engine = ELUTQ_GEMV_ENGINE_AUTO;

// Count of slot meetings whose bounded wait ran out (slices_meet_slots), one word per GPU, held until the process ends.
// The name is a host-side stand-in: the device address is looked up once per device.
static __device__ unsigned g_gemv_fault_word[4];
std::mutex g_fault_lock;
unsigned *g_fault_ptr[64] = {};

int fault_address(unsigned **out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ELUTQ_ERR_HIP;
    std::lock_guard<std::mutex> hold(g_fault_lock);
    if (!g_fault_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_gemv_fault_word)) != hipSuccess || !p) return ELUTQ_ERR_HIP;
        g_fault_ptr[dev] = (unsigned *)p;
    }
    *out = g_fault_ptr[dev];
    return ELUTQ_OK;
}

// Test hook (elutq_test_gemv_meeting): a slice that leaves without storing, and the poll limit of the waiting wave.
int g_test_drop_slice = -1, g_test_spin_limit = SLICE_SPIN_LIMIT;

// The launch shape of a batch-1 GEMV: which kernel, K slices, units per slice, waves per workgroup.  One
// function for the launch itself and for the queries about it (elutq_hlq_gemv_slices, _accepts_slices).
struct LaunchShape {
    bool mfma;
    int narrow;              // 0, or the columns per wave of the narrow-tile kernel (16 / 32)
    int ksplit, ups, waves;
};

// `allow_narrow`: the call has nothing the narrow-tile kernel lacks (extra term, handed-over slices).
int plan_launch(const HlqGeo &g, int bits, int ksplit, int waves, bool allow_narrow, LaunchShape &sh, bool lut_only = false)
{
    sh.mfma = false;
    sh.narrow = 0;
    if (ksplit == ELUTQ_GEMV_WIDE) {
        ksplit = 0;
        allow_narrow = false;
    }
    if (ksplit == ELUTQ_GEMV_NARROW16 || ksplit == ELUTQ_GEMV_NARROW32) {
        // the caller's choice of the narrow-tile kernel
        const int cw = ksplit == ELUTQ_GEMV_NARROW16 ? 16 : 32;
        const int rounds = hlq_gemv_narrow_rounds(g.U, cw);
        if (!allow_narrow || waves != 0 || rounds == 0) return ELUTQ_ERR_TUNING;
        sh.narrow = cw;
    } else if (allow_narrow && ksplit == 0 && waves == 0 && g_gemv_engine != ELUTQ_GEMV_ENGINE_MFMA) {
        // Fewer column blocks than compute units: tiles of 16 (32) columns give four (two) times the
        // workgroups without cutting K, where the tables of all of K fit one workgroup's LDS (measured on
        // MI355X: 4096x4096 5.1 -> 3.x us, where K slices only trade lookups for their meeting).
        if (g.ncb * 4 <= NUM_CU && hlq_gemv_narrow_rounds(g.U, 16)) sh.narrow = 16;
        else if (g.ncb * 2 <= NUM_CU && hlq_gemv_narrow_rounds(g.U, 32)) sh.narrow = 32;
    }
    if (sh.narrow) {
        const int per_wave = 64 / sh.narrow;         // units a wave covers per round
        sh.ksplit = 1; sh.ups = g.U; sh.waves = g.U < 16 * per_wave ? (g.U + per_wave - 1) / per_wave : 16;
        return ELUTQ_OK;
    }
    if (ksplit < 0 || waves < 0 || waves > 16 || ksplit > g.U) return ELUTQ_ERR_TUNING;
    const bool auto_waves = waves <= 0;
    // measured on MI355X: the matrix-core kernel streams large layers as fast as the LUT kernel but a launch of one
    // tile per workgroup takes 0.5-1 us longer (its A operands cost more to build than the tables), so the
    // library's own choice is the LUT kernel throughout
    sh.mfma = !lut_only && g_gemv_engine == ELUTQ_GEMV_ENGINE_MFMA;
    if (sh.mfma && g.K % HLQ_UNIT != 0) return ELUTQ_ERR_TUNING;      // the matrix-core kernel takes whole units only
    choose_shape(g, ksplit, waves);
    int ups = (g.U + ksplit - 1) / ksplit;
    if (sh.mfma) {
        // slices start on a unit pair (at G = 128 a pair shares its scale / zero dwords), and a wave holds the A
        // operands of at most two pairs: 16 waves x 2 pairs x 256 k = 8192 k per slice
        if (ksplit > 1 && (ups & 1)) ups++;
        while ((ups + 1) / 2 > 2 * 16) ups = ((ups + 1) / 2 + 1) & ~1;
        ksplit = (g.U + ups - 1) / ups;
        const int npairs = (ups + 1) / 2;
        if (auto_waves) waves = npairs < 16 ? npairs : 16;
        if ((npairs + waves - 1) / waves > 2) {
            if (g_gemv_engine == ELUTQ_GEMV_ENGINE_MFMA) return ELUTQ_ERR_TUNING;      // the caller's wave count is too small
            sh.mfma = false;
        }
    }
    if (!sh.mfma) {
        // shrink the slice so its tables fit in LDS, then the slice count so that no slice is empty
        ups = (g.U + ksplit - 1) / ksplit;
        while (gemv_lds_bytes(ups, bits, waves) > (size_t)MAX_LDS) ups = (ups + 1) / 2;
        ksplit = (g.U + ups - 1) / ups;
        // a slice of at most 16 sub-tasks: eight waves with two each start sooner than sixteen with one
        if (auto_waves && ups * bits <= 16) waves = 8;
    }
    sh.ksplit = ksplit; sh.ups = ups; sh.waves = waves;
    return ELUTQ_OK;
}

size_t shape_lds_bytes(const LaunchShape &sh, int bits)
{
    if (sh.narrow) return hlq_gemv_narrow_lds_bytes(sh.ups, sh.narrow);
    return sh.mfma ? hlq_gemv_mfma_lds_bytes(sh.ups, sh.waves) : gemv_lds_bytes(sh.ups, bits, sh.waves);
}

}  // namespace

extern "C" {

size_t elutq_hlq_workspace_bytes(int K, int N, int bits, int group, int M)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK || M < 1) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    // arrival counters (fixed region, so layers of any shape can share one workspace) +
    // partial sums: GEMV at its finest split (one unit per slice), GEMM at the split it uses
    const size_t gemv = (size_t)WS_COUNTER_BYTES + (size_t)g.U * g.ncb * HLQ_CB * sizeof(float);
    const size_t gemm = M > 1 ? hlq_gemm_ws_bytes(g, M) : 0;
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
// `lut_int8`: the wide-tile LUT kernel's instance with int8 tables (plain calls only).
static int gemv_launch(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                       const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                       size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion, int ksplit,
                       int waves, const float *d_extra, bool lut_int8, const void *d_sp_inline = nullptr, size_t sp_inline_bytes = 0)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    LaunchShape sh;
    // (a block-sparse plane held in its inline form is looked up by the LUT kernels)
    const bool allow_narrow = !(fusion && fusion->d_slices_out) && !lut_int8;
    const bool own_shape = ksplit == 0 && waves == 0;              // the library chooses the launch shape
    rc = plan_launch(g, bits, ksplit, waves, allow_narrow, sh, lut_int8 || d_sp_inline != nullptr);
    if (rc != ELUTQ_OK) return rc;
    if (lut_int8 && (sh.mfma || sh.narrow || fusion || d_extra)) return ELUTQ_ERR_TUNING;
    ksplit = sh.ksplit; waves = sh.waves;
    const int ups = sh.ups;

    // A plain call on a layer with more column blocks than the chip has compute units and K > 4096: the streaming
    // matrix-core kernel, every workgroup an equal share of the column blocks over all of K (no slices, no workspace).
    // Measured on MI355X against the LUT kernel's runs of column blocks with K slices: 8192 x 28672 17.7 against
    // 21.2 us, 14336 x 32768 29.2 against 51.8 us; at K = 4096, where the LUT kernel needs no slices, the two are level
    // (4096 x 128256: 31.0 against 30.6 us) and the LUT kernel stays.
    const bool wide = g_gemv_engine != ELUTQ_GEMV_ENGINE_LUT && !lut_int8 && !fusion && !d_extra && !d_sp_inline && own_shape &&
                      g.K % HLQ_UNIT == 0 && g.ncb > NUM_CU && (g.U > 32 || g_gemv_engine == ELUTQ_GEMV_ENGINE_MFMA);
    if (wide) sh.ksplit = 1;
    ksplit = sh.ksplit;
    GemvArgs a;
    a.planes = (const HLQ_GLOBAL uint4 *)d_planes;
    a.scales = (const HLQ_GLOBAL uint32_t *)d_scales;
    a.zeros = (const HLQ_GLOBAL uint32_t *)d_zeros;
    a.bias = (const HLQ_GLOBAL uint16_t *)d_bias;
    a.x = (const HLQ_GLOBAL uint16_t *)d_x;
    a.y = (HLQ_GLOBAL uint16_t *)d_y;
    a.N = N; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb; a.K = K;
    a.ksplit = ksplit; a.ups = ups;
    const WavePlan wp = wave_plan(ups, bits, waves);
    a.spw = wp.spw; a.nuw_max = wp.nuw_max; a.wave_lds = wp.wave_lds;
    a.partial = nullptr; a.counters = nullptr; a.meet_slots = 0;
    a.prologue = 0; a.eps = 0.f; a.norm_w = nullptr; a.residual = nullptr; a.extra = nullptr;
    a.defer = 0; a.n_slices_in = 0; a.slices_in = nullptr; a.x_out = nullptr; a.lut_int8 = 0;
    a.fault = nullptr; a.spin_limit = SLICE_SPIN_LIMIT; a.drop_slice = -1; a.sp_cells = nullptr; a.sp_recs = nullptr; a.sp_nrec = 0;
    if (fusion) {
        if (fusion->prologue < 0 || fusion->prologue > 2) return ELUTQ_ERR_TUNING;
        if (fusion->prologue == 1 && !fusion->d_norm_weight) return ELUTQ_ERR_NULL;
        a.prologue = fusion->prologue;
        a.eps = fusion->eps;
        a.norm_w = (const HLQ_GLOBAL uint16_t *)fusion->d_norm_weight;
        a.residual = (const HLQ_GLOBAL uint16_t *)fusion->d_residual;
    }
    a.extra = (const HLQ_GLOBAL float *)d_extra;
    a.lut_int8 = lut_int8 ? 1 : 0;
    if (d_sp_inline) {
        // the form's size is the caller's word for how many records lie behind the cell table: a record number beyond
        // them is treated as "no block", and a buffer too small for the layer's cell table is refused
        const size_t recs_off = hlq_sp_recs_offset(g.ncb, g.U);
        if (sp_inline_bytes < recs_off) return ELUTQ_ERR_WORKSPACE;
        a.sp_cells = (const HLQ_GLOBAL int32_t *)((const unsigned char *)d_sp_inline + HLQ_SP_HEAD_BYTES);
        a.sp_recs = (const HLQ_GLOBAL unsigned char *)d_sp_inline + recs_off;
        const size_t nrec = (sp_inline_bytes - recs_off) / HLQ_SP_REC_BYTES;
        a.sp_nrec = nrec > 0x7fffffffu ? 0x7fffffff : (int)nrec;
    }
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
        if (!sh.narrow && (long long)g.ncb * ksplit > NUM_CU) return ELUTQ_ERR_TUNING;
        a.x_out = (HLQ_GLOBAL uint16_t *)fusion->d_x_out;
        stage_bytes = (size_t)K * sizeof(uint16_t);
        if (shape_lds_bytes(sh, bits) + stage_bytes > (size_t)MAX_LDS) return ELUTQ_ERR_SHAPE;
        if (fusion->slices_in_bytes < (size_t)fusion->n_slices_in * K * sizeof(float)) return ELUTQ_ERR_WORKSPACE;
    }
    if (fusion && fusion->d_slices_out) {
        // the K slices stay unsummed for the next launch: nothing else may be due in the output stage
        if (ksplit < 2 || d_bias || a.residual || d_extra || N % HLQ_CB != 0) return ELUTQ_ERR_TUNING;
        // every slice writes a row of N floats: the buffer's size is the caller's word, checked here because a row
        // too many would land on whatever lies behind the buffer
        if (fusion->slices_out_bytes < (size_t)ksplit * N * sizeof(float)) return ELUTQ_ERR_WORKSPACE;
        a.defer = 1;
        a.partial = (HLQ_GLOBAL float *)fusion->d_slices_out;
    } else if (ksplit > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ksplit * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        // slots that fit the head of the workspace, which every kernel leaves zero-filled, are filled and emptied
        // instead of counted (slices_meet_slots); else arrival counters there and the partial sums behind it
        // -- with 2, 4 or 8 slices only: the fixed waiter must not share an XCD with a slice it waits for (slices_meet_slots)
        if ((size_t)(ksplit - 1) * g.ncb * HLQ_CB * sizeof(float) <= (size_t)WS_COUNTER_BYTES &&
            (ksplit == 2 || ksplit == 4 || ksplit == 8)) {
            a.meet_slots = 1;
            a.partial = (HLQ_GLOBAL float *)d_workspace;
            unsigned *fault = nullptr;
            rc = fault_address(&fault);
            if (rc != ELUTQ_OK) return rc;
            a.fault = (HLQ_GLOBAL unsigned *)fault;
            a.spin_limit = g_test_spin_limit;
            a.drop_slice = g_test_drop_slice;
        } else {
            a.counters = (HLQ_GLOBAL unsigned *)d_workspace;
            a.partial = (HLQ_GLOBAL float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
        }
    }
    if (wide) return hlq_gemv_mfma_wide_launch(&a, sizeof(a), bits, group, stream);
    if (sh.narrow) return hlq_gemv_narrow_launch(&a, sizeof(a), bits, group, sh.narrow, stage_bytes, stream);
    if (sh.mfma) return hlq_gemv_mfma_launch(&a, sizeof(a), bits, group, waves, stage_bytes, stream);
    return dispatch_gemv(a, bits, group, waves, gemv_lds_bytes(ups, bits, waves) + stage_bytes, (hipStream_t)stream);
}

int hlq_gemv_with_extra(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                        const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                        size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion, int ksplit,
                        int waves, const float *d_extra)
{
    return gemv_launch(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace, workspace_bytes,
                       stream, fusion, ksplit, waves, d_extra, false);
}

int hlq_gemv_with_inline_sparse(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                const void *d_sp_inline, size_t sp_inline_bytes, const void *d_x, void *d_y, int K, int N, int bits, int group,
                                void *d_workspace, size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion,
                                int ksplit, int waves)
{
    if (!d_sp_inline) return ELUTQ_ERR_NULL;
    return gemv_launch(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace, workspace_bytes,
                       stream, fusion, ksplit, waves, nullptr, false, d_sp_inline, sp_inline_bytes);
}

extern "C" int elutq_hlq_gemv_int8lut_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                          const void *d_x, void *d_y, int K, int N, int bits, int group,
                                          void *d_workspace, size_t workspace_bytes, void *stream)
{
    // the library's own launch shape on wide tiles, whatever engine is selected for the exact GEMV
    return gemv_launch(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace, workspace_bytes,
                       stream, nullptr, ELUTQ_GEMV_WIDE, 0, nullptr, true);
}

extern "C" int elutq_hlq_set_gemv_engine(int engine)
{
    if (engine != ELUTQ_GEMV_ENGINE_AUTO && engine != ELUTQ_GEMV_ENGINE_LUT && engine != ELUTQ_GEMV_ENGINE_MFMA)
        return ELUTQ_ERR_TUNING;
    g_gemv_engine = engine;
    return ELUTQ_OK;
}

extern "C" int elutq_hlq_get_gemv_engine(void) { return g_gemv_engine; }

extern "C" int elutq_hlq_gemv_fault_count(int clear)
{
    unsigned *p = nullptr;
    const int rc = fault_address(&p);
    if (rc != ELUTQ_OK) return rc;
    unsigned h = 0;
    if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(&h, p, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) return ELUTQ_ERR_HIP;
    if (clear && h && hipMemset(p, 0, sizeof(h)) != hipSuccess) return ELUTQ_ERR_HIP;
    return h > 0x7fffffffu ? 0x7fffffff : (int)h;
}

// Not part of the C ABI (no declaration in include/elutq_hip.h): lets a test force the give-up path of the slot meeting
// from the host with every kernel still ending normally.  drop_slice >= 0: that K slice of the following slot-meeting
// launches leaves without storing its sums; spin_limit: polls before the waiting wave gives up (<= 0: the default).
// elutq_test_gemv_meeting(-1, 0) restores normal operation.
extern "C" int elutq_test_gemv_meeting(int drop_slice, int spin_limit)
{
    g_test_drop_slice = drop_slice < 0 ? -1 : drop_slice;
    g_test_spin_limit = spin_limit > 0 ? spin_limit : SLICE_SPIN_LIMIT;
    return ELUTQ_OK;
}

// Whether a launch of this shape (ksplit / waves as the call would pass them) takes `n_slices` handed-over
// K slices in its RMSNorm prologue: the same steps and limits as the launch itself.
extern "C" int elutq_hlq_gemv_accepts_slices(int K, int N, int bits, int group, int ksplit, int waves, int n_slices)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK) return 0;
    if (n_slices < 1 || n_slices > GEMV_MAX_SLICES_IN) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    LaunchShape sh;
    if (plan_launch(g, bits, ksplit, waves, true, sh) != ELUTQ_OK) return 0;
    if (!sh.narrow && (long long)g.ncb * sh.ksplit > NUM_CU) return 0;
    return shape_lds_bytes(sh, bits) + (size_t)K * sizeof(uint16_t) <= (size_t)MAX_LDS ? 1 : 0;
}

extern "C" int elutq_hlq_gemv_slices(int K, int N, int bits, int group, int ksplit, int waves)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK) return 0;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    LaunchShape sh;
    // the wide-tile kernel's figure (a producer of handed-over slices runs on it), unless the caller names the narrow one
    if (plan_launch(g, bits, ksplit, waves, ksplit == ELUTQ_GEMV_NARROW16 || ksplit == ELUTQ_GEMV_NARROW32, sh) != ELUTQ_OK) return 0;
    return sh.ksplit;
}

extern "C" {

// ---- grouped launch of independent GEMVs --------------------------------------------------
struct GroupShape {                      // tile shape of one problem inside a group
    HlqGeo g;
    int ksplit, ups;
    WavePlan wp;
};

static int group_shape(const elutq_gemv_problem &p, int bits, int group, bool mfma, GroupShape &sh)
{
    int rc = check_shape(p.K, p.N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!p.d_planes || !p.d_scales || !p.d_zeros || !p.d_x || !p.d_y) return ELUTQ_ERR_NULL;
    sh.g = hlq_geo(p.K, p.N, bits, group);
    if (mfma) {
        // a tile of the matrix-core kernel covers all of K: no slices, nothing to meet in the workspace
        sh.ups = sh.g.U;
        sh.ksplit = 1;
        sh.wp = wave_plan(1, bits, 16);              // (the wave-run fields are not read by the matrix-core kernel)
        return ELUTQ_OK;
    }
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
    bool paired, mfma;
    size_t lds;
    GemvArgs *d_problems;
    void *d_items;           // GroupItem array, or the tile blob of the matrix-core kernel
};

// The grouped launch runs on the matrix cores where that engine is selected and every layer has whole units.
static bool group_on_mfma(const elutq_gemv_problem *problems, int count)
{
    if (g_gemv_engine == ELUTQ_GEMV_ENGINE_LUT) return false;          // (the library's own choice: measured 6.3 against 5.6 TB/s)
    for (int i = 0; i < count; i++)
        if (problems[i].K % HLQ_UNIT != 0) return false;
    return true;
}

static size_t group_layout(const elutq_gemv_problem *problems, int count, int bits, int group,
                           std::vector<GroupShape> *shapes, std::vector<size_t> *counter_off, std::vector<size_t> *partial_off,
                           int *rc_out)
{
    size_t counters = 0, partials = 0;
    *rc_out = ELUTQ_OK;
    const bool mfma = group_on_mfma(problems, count);
    for (int i = 0; i < count; i++) {
        GroupShape sh;
        const int rc = group_shape(problems[i], bits, group, mfma, sh);
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
    const bool mfma = group_on_mfma(problems, count);
    for (int i = 0; i < count; i++) {
        const GroupShape &sh = shapes[i];
        GemvArgs &a = args[i];
        a.planes = (const HLQ_GLOBAL uint4 *)problems[i].d_planes;
        a.scales = (const HLQ_GLOBAL uint32_t *)problems[i].d_scales;
        a.zeros = (const HLQ_GLOBAL uint32_t *)problems[i].d_zeros;
        a.bias = (const HLQ_GLOBAL uint16_t *)problems[i].d_bias;
        a.x = (const HLQ_GLOBAL uint16_t *)problems[i].d_x;
        a.y = (HLQ_GLOBAL uint16_t *)problems[i].d_y;
        a.N = problems[i].N; a.U = sh.g.U; a.NT = sh.g.NT; a.ncb = sh.g.ncb; a.K = problems[i].K;
        a.ksplit = sh.ksplit; a.ups = sh.ups;
        a.spw = sh.wp.spw; a.nuw_max = sh.wp.nuw_max; a.wave_lds = sh.wp.wave_lds;
        a.partial = nullptr; a.counters = nullptr; a.meet_slots = 0;
        if (sh.ksplit > 1) {
            // Arrival counters, not slots: in this launch a workgroup walks a list of tiles, so the workgroup a
            // waiting one depends on can have a higher index -- and if two such launches share the GPU, neither
            // need be resident in full.  With counters nothing ever waits for another workgroup.
            a.counters = (HLQ_GLOBAL unsigned *)((unsigned char *)d_workspace + coff[i]);
            a.partial = (HLQ_GLOBAL float *)((unsigned char *)d_workspace + poff[i]);
        }
        a.prologue = 0; a.eps = 0.f; a.norm_w = nullptr; a.residual = nullptr; a.extra = nullptr;
        a.defer = 0; a.n_slices_in = 0; a.slices_in = nullptr; a.x_out = nullptr; a.lut_int8 = 0;
        a.fault = nullptr; a.spin_limit = SLICE_SPIN_LIMIT; a.drop_slice = -1; a.sp_cells = nullptr; a.sp_recs = nullptr; a.sp_nrec = 0;
        const int ns = a.spw < depth_of(bits) ? a.spw : depth_of(bits);
        if (ns > nslot) nslot = ns;
        if (mfma) continue;                          // its tile list is made below, over all layers at once
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
    pl->mfma = mfma;
    for (auto &sh : shapes) pl->paired = pl->paired && paired_ok_rt(bits, group == 64, nslot, sh.wp.spw, sh.ups, sh.ksplit);
    std::vector<unsigned char> blob;
    const void *h_items = items.data();
    size_t items_bytes = items.size() * sizeof(GroupItem);
    if (mfma) {
        // one workgroup per compute unit, each with its own contiguous share of the layers' column blocks
        std::vector<int> units(count), ncbs(count);
        for (int i = 0; i < count; i++) { units[i] = shapes[i].g.U; ncbs[i] = shapes[i].g.ncb; }
        pl->grid = total_cbs < NUM_CU ? (int)total_cbs : NUM_CU;
        blob.resize(hlq_gemv_mfma_group_plan(units.data(), ncbs.data(), count, pl->grid, nullptr));
        hlq_gemv_mfma_group_plan(units.data(), ncbs.data(), count, pl->grid, blob.data());
        h_items = blob.data();
        items_bytes = blob.size();
    } else {
        // as many workgroups as the chip holds at once: each walks the list with that stride
        int per_cu = dispatch_group(bits, group == 64, nslot, pl->paired, nullptr, nullptr, 0, -1, 16, lds, nullptr);
        if (per_cu < 1) per_cu = 1;
        if (per_cu > 2) per_cu = 2;
        const int slots = NUM_CU * per_cu;
        pl->grid = pl->n_items < slots ? pl->n_items : slots;
    }
    pl->d_problems = nullptr; pl->d_items = nullptr;
    if (hipMalloc((void **)&pl->d_problems, args.size() * sizeof(GemvArgs)) != hipSuccess ||
        hipMalloc((void **)&pl->d_items, items_bytes) != hipSuccess ||
        hipMemcpy(pl->d_problems, args.data(), args.size() * sizeof(GemvArgs), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(pl->d_items, h_items, items_bytes, hipMemcpyHostToDevice) != hipSuccess) {
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
    if (pl->mfma) return hlq_gemv_mfma_group_launch(pl->bits, pl->group, pl->d_problems, pl->d_items, pl->grid, stream);
    return dispatch_group(pl->bits, pl->group == 64, pl->nslot, pl->paired, pl->d_problems, (const GroupItem *)pl->d_items, pl->n_items, pl->grid, 16,
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

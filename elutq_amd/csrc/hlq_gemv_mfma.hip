// Batch-1 HLQ GEMV on the matrix cores of gfx950 (MI355X): the bit planes go into
// v_mfma_f32_32x32x64_f8f6f4 as they lie in memory, read as fp4 (e2m1) nibbles, with no expansion.
// Same computation, buffers and launch structure as the LUT kernel of hlq_gemv.hip (the counterpart of
// MultiThread_arm_gemv_w_lowbit_activation_fp_impl, C++/ops/src/arm/arm_gemm.cpp:312-360, and
// t_mac_g4_float_update_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469); what changes is how
// sum_k B[n,k] x[k] is formed.
//
//  * A nibble of a plane dword holds four plane bits.  Masked to one bit position p it is the fp4 number
//    0.5 (p = 0), 1.0 (p = 1) or 2.0 (p = 2) where the bit is set and 0 where it is not; bit 3 is the sign
//    bit, so it is shifted to position 2 first.  Four masked copies ("features") of a register of plane
//    bits are four B operands, one VALU instruction each per 32 plane bits, and the four MFMAs accumulate
//    into one tile.
//  * The A operand holds the activations as fp8 (e4m3) terms: per 64-k half unit x is scaled by a power of two
//    that puts max|x| in [64, 128), divided by the feature's value v_p, and written as the sum of three fp8
//    numbers (round to nearest, subtract, round the remainder: 3 x 4 significant bits hold an fp16 value
//    exactly unless it lies more than 2^-15 below the half unit's maximum).  Row (half unit h, term t) of A holds
//    term t of the activations of half unit h and zeros elsewhere, so tile element D[(h, t)][n] = sum over the
//    half unit of term_t(k) * B[n,k] * v_p, exact in fp32; sum_t D[(h, t)][n] / scale is the half unit's sum for
//    column n.  The rows of a tile that a GEMM would spend on other tokens carry the terms and the four half
//    units of a unit pair.
//  * The K dimension of one MFMA is a unit pair (2 x 128 k): lanes 0-31 hold the first unit of 32
//    columns, lanes 32-63 the second.  The layout in memory has lane = column for one unit, so two loads
//    (units u, u + 1 of 64 columns) are turned into two B operands (columns 0-31 / 32-63, both units) with
//    v_permlane32_swap.
//  * Scale / zero fold per (half unit, plane) in fp32 as in the LUT kernel; K slices, the cross-wave sum,
//    prologues and epilogues are the LUT kernel's.
//
// No LDS lookups and about half the vector instructions per plane bit of the LUT kernel: the matrix pipe
// takes 8 MFMAs (64 cycles each with an fp8 operand) per 2 KiB of plane data and wave.
#include "hlq_gemv_dev.h"
#include "hlq_internal.h"

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

// K index of v_mfma_f32_32x32x64_f8f6f4 (measured on gfx950): an fp4 operand's lane l holds K = 32 (l / 32) + v in
// nibble v % 8 of register v / 8; an fp8 operand's lane l holds K = 16 (l / 32) + 4 i + j in byte j of register
// i < 4 and K = 32 + 16 (l / 32) + 4 (i - 4) + j in register i >= 4.  With the B operand (fp4) = plane bits of unit u
// in lanes 0-31 and of unit u + 1 in lanes 32-63, the A operand's (fp8) lane half h therefore faces half unit h of
// both units: registers 0-3 the first unit's, registers 4-7 the second unit's.
constexpr int MF_TERMS = 3;                                   // fp8 terms per activation: 3 x 4 significant bits >= fp16's 11
constexpr int MF_REC = 32;                                    // one A row of one lane half: 8 registers
constexpr int MF_IMG_BYTES = 4 * 2 * 2 * MF_TERMS * MF_REC;   // A image of a pair: [feature][unit][half][term][32 bytes]
constexpr int MF_META_FLOATS = 8;                             // per pair: 1 / scale [unit][half], sum of x [unit][half]
constexpr int MF_PAIR_LDS = (MF_IMG_BYTES + MF_REC + MF_META_FLOATS * 4 + 255) & ~255;   // image, a zero record, meta

// Activations of one unit pair (256 k, lane = chunk of 4 k of unit lane / 32) as the A operand images of the four
// features, and the pair's half-unit records (1 / scale, sum of x).  Every activation becomes MF_TERMS fp8 (e4m3)
// numbers that add up to x * scale / v_p exactly (scale: a power of two per half unit that puts max|x| in [64, 128);
// v_p = 0.5, 1, 2, 2: the fp4 value of a set plane bit of feature p): round to nearest, subtract, round the rest.
// A record is the 32 bytes one lane of the A operand holds: the half unit's 16 slots at offset 16 * unit, zeros in
// the other half (they are written once per kernel and never overwritten).
__device__ __forceinline__ void build_pair(const float (&v)[4], unsigned char *img, float *meta, int lane)
{
    const int unit = lane >> 5, d = (lane & 31) >> 3, j = lane & 7, half = d >> 1;
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    float s = (v[0] + v[1]) + (v[2] + v[3]);
    HLQ_ROW_REDUCE(s, op_add);
    HLQ_ROW_REDUCE(amax, op_max);
    // amax in [2^(eb-127), 2^(eb-126)): times 2^(133-eb) it lies in [64, 128)
    const uint32_t eb = (__float_as_uint(amax) >> 23) & 0xffu;
    const float scale = eb ? __uint_as_float((260u - eb) << 23) : 1.0f;
    const float inv = eb ? __uint_as_float((eb - 6u) << 23) : 1.0f;
    // value i of the chunk sits at bit i + 2 of the chunk's field in the rotated dword: features 2, 3 (v_p = 2) in
    // nibble slot j, features 0 (v_p = 0.5) and 1 (v_p = 1) in slot j + 1 (the last chunk of a dword wraps to slot 0)
    float r[4] = {v[0] * scale * 0.5f, v[1] * scale * 0.5f, v[2] * scale * 2.0f, v[3] * scale};
    uint32_t term[MF_TERMS];
#pragma unroll
    for (int t = 0; t < MF_TERMS; t++) {
        int pk = __builtin_amdgcn_cvt_pk_fp8_f32(r[0], r[1], 0, false);
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(r[2], r[3], pk, true);
        term[t] = (uint32_t)pk;
        if (t + 1 < MF_TERMS) {
            r[0] -= __builtin_amdgcn_cvt_f32_fp8(pk, 0);
            r[1] -= __builtin_amdgcn_cvt_f32_fp8(pk, 1);
            r[2] -= __builtin_amdgcn_cvt_f32_fp8(pk, 2);
            r[3] -= __builtin_amdgcn_cvt_f32_fp8(pk, 3);
        }
    }
    // record (feature p, unit, half, term): byte 16 * unit + 8 * (d & 1) + slot
    unsigned char *base = img + (size_t)((unit * 2 + half) * MF_TERMS) * MF_REC + 16 * unit + 8 * (d & 1);
    const int s01 = j, s23 = (j + 1) & 7;
    constexpr int FSTRIDE = 2 * 2 * MF_TERMS * MF_REC;        // bytes per feature
#pragma unroll
    for (int t = 0; t < MF_TERMS; t++) {
        base[2 * FSTRIDE + t * MF_REC + s01] = (unsigned char)(term[t] & 0xffu);          // value 0 -> feature 2
        base[3 * FSTRIDE + t * MF_REC + s01] = (unsigned char)((term[t] >> 8) & 0xffu);   // value 1 -> feature 3
        base[0 * FSTRIDE + t * MF_REC + s23] = (unsigned char)((term[t] >> 16) & 0xffu);  // value 2 -> feature 0
        base[1 * FSTRIDE + t * MF_REC + s23] = (unsigned char)(term[t] >> 24);            // value 3 -> feature 1
    }
    if ((lane & 15) == 0) {
        const int h4 = lane >> 4;                             // (unit, half) 0..3
        meta[h4] = inv;
        meta[4 + h4] = s;
    }
}

// A operands of a pair from its images: lane L supplies row L & 31 for lane half L >> 5.  Row r = term + 4 unit +
// 16 half (term < MF_TERMS; rows with bit 3 set are unused): with that assignment lanes 0-31 of the result tile hold
// the terms of the first unit's two half units in registers 0.. / 8.., lanes 32-63 those of the second unit.  A row
// is live only in the lane half that faces its half unit; every other lane reads the zero record.
struct PairA {
    uint32_t a[4][8];
};

__device__ __forceinline__ void load_pair_a(PairA &pa, const unsigned char *img, int lane)
{
    const int row = lane & 31, kh = lane >> 5;
    const int unit = (row >> 2) & 1, half = row >> 4, term = row & 3;
    const bool live = half == kh && term < MF_TERMS && (row & 8) == 0;
    const int rec = live ? ((unit * 2 + half) * MF_TERMS + term) * MF_REC : MF_IMG_BYTES;     // MF_IMG_BYTES: the zero record
    constexpr int FSTRIDE = 2 * 2 * MF_TERMS * MF_REC;
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const uint4 lo = *(const uint4 *)(img + (live ? p * FSTRIDE : 0) + rec);
        const uint4 hi = *(const uint4 *)(img + (live ? p * FSTRIDE : 0) + rec + 16);
        pa.a[p][0] = lo.x; pa.a[p][1] = lo.y; pa.a[p][2] = lo.z; pa.a[p][3] = lo.w;
        pa.a[p][4] = hi.x; pa.a[p][5] = hi.y; pa.a[p][6] = hi.z; pa.a[p][7] = hi.w;
    }
}

// One plane of one unit pair for 32 columns: four features into one tile, then the terms of each half unit added up.
// A tile element is a sum of products (fp8 term) x (0.5, 1 or 2): exact in the fp32 accumulator.
__device__ __forceinline__ void pair_plane(const PairA &pa, const uint32_t (&b)[4], float &half0, float &half1)
{
    v16f d = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 4; p++) {
        v8i av = {(int)pa.a[p][0], (int)pa.a[p][1], (int)pa.a[p][2], (int)pa.a[p][3],
                  (int)pa.a[p][4], (int)pa.a[p][5], (int)pa.a[p][6], (int)pa.a[p][7]};
        v8i bv = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t m = p == 0 ? 0x11111111u : (p == 1 ? 0x22222222u : 0x44444444u);
            bv[i] = (int)((p == 3 ? b[i] >> 1 : b[i]) & m);
        }
        d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, d, 0, 4, 0, 0, 0, 0);
    }
    float h0 = d[0], h1 = d[8];
#pragma unroll
    for (int t = 1; t < MF_TERMS; t++) {
        h0 += d[t];
        h1 += d[8 + t];
    }
    half0 = h0;
    half1 = h1;
}

// Sub-tasks a wave has in registers or in flight (12 registers each): four (8 KiB per wave, 128 KiB per compute
// unit) for a wave with one pair, two where the wave also holds the fold constants of a second pair.
#ifdef MF_NS_OVERRIDE
constexpr int mf_slots(int bits, bool g64, int maxp) { return MF_NS_OVERRIDE; }
#else
constexpr int mf_slots(int bits, bool g64, int maxp) { return maxp == 1 ? 4 : 2; }
#endif
constexpr int mf_gcd(int a, int b) { return b == 0 ? a : mf_gcd(b, a % b); }

// Plane data of one (unit pair, plane) sub-task for the 64 columns of a block, as loaded (lane = column).
struct PairLoad {
    uint4 w0, w1;          // units u and u + 1
    uint32_t sc0, sc1;     // scale dwords (G = 128: sc0 only, the pair's dword; G = 64: one per unit)
    uint32_t zz0, zz1;     // zero dwords, plane 0 only
};

template <int BITS, bool G64, int b>
__device__ __forceinline__ void load_pair(PairLoad &t, const GemvArgs &a, int cb, int u, int u_last, int lane)
{
    const uint32_t u1 = (uint32_t)min(u + 1, u_last);
    const HLQ_GLOBAL unsigned char *pl = (const HLQ_GLOBAL unsigned char *)a.planes + (size_t)cb * a.U * (size_t)(BITS * HLQ_CB * 16);
    const HLQ_GLOBAL unsigned char *sc = (const HLQ_GLOBAL unsigned char *)a.scales + (size_t)cb * a.NT * (size_t)(BITS * HLQ_CB * 4);
    const HLQ_GLOBAL unsigned char *zz = (const HLQ_GLOBAL unsigned char *)a.zeros + (size_t)cb * a.NT * (size_t)(HLQ_CB * 4);
    const u32x4 v0 = __builtin_nontemporal_load((const HLQ_GLOBAL u32x4 *)(pl + (((uint32_t)u * BITS + b) * (uint32_t)(HLQ_CB * 16) + (uint32_t)lane * 16u)));
    const u32x4 v1 = __builtin_nontemporal_load((const HLQ_GLOBAL u32x4 *)(pl + ((u1 * BITS + b) * (uint32_t)(HLQ_CB * 16) + (uint32_t)lane * 16u)));
    t.w0 = make_uint4(v0.x, v0.y, v0.z, v0.w);
    t.w1 = make_uint4(v1.x, v1.y, v1.z, v1.w);
    const uint32_t r0 = G64 ? (uint32_t)u : (uint32_t)u >> 1, r1 = G64 ? u1 : u1 >> 1;
    t.sc0 = *(const HLQ_GLOBAL uint32_t *)(sc + ((r0 * BITS + b) * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u));
    t.sc1 = G64 ? *(const HLQ_GLOBAL uint32_t *)(sc + ((r1 * BITS + b) * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u)) : t.sc0;
    if (b == 0) {
        t.zz0 = *(const HLQ_GLOBAL uint32_t *)(zz + (r0 * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u));
        t.zz1 = G64 ? *(const HLQ_GLOBAL uint32_t *)(zz + (r1 * (uint32_t)(HLQ_CB * 4) + (uint32_t)lane * 4u)) : t.zz0;
    } else {
        t.zz0 = t.zz1 = 0;
    }
}

// Lanes 0-31 keep `lo`'s lower half and lanes 32-63 receive `hi`'s lower half (columns 0-31 of both
// units); the second result is the same for the upper halves (columns 32-63).
__device__ __forceinline__ void split32(uint32_t lo, uint32_t hi, uint32_t &c0, uint32_t &c1)
{
    const auto r = __builtin_amdgcn_permlane32_swap(lo, hi, false, false);
    c0 = r[0];
    c1 = r[1];
}

// Per-lane constants of a pair for the fold: the lane's unit is lane >> 5.
struct PairFold {
    float inv0, inv1;      // 2^-F of the unit's two half units
    float xs0, xs1;        // sums of x over them
};

// The sub-task's contribution to the two column halves (accx: columns 0-31, accy: 32-63; lanes 0-31 carry
// the first unit's share, lanes 32-63 the second unit's).
template <bool G64>
__device__ __forceinline__ void process_pair(const PairLoad &t, const PairA &pa, const PairFold &pf, bool plane0, int lane,
                                             float &accx, float &accy)
{
    const bool second = lane >= 32;
    uint32_t bx[4], by[4];
    split32(t.w0.x, t.w1.x, bx[0], by[0]);
    split32(t.w0.y, t.w1.y, bx[1], by[1]);
    split32(t.w0.z, t.w1.z, bx[2], by[2]);
    split32(t.w0.w, t.w1.w, bx[3], by[3]);
    uint32_t scx, scy, zzx, zzy;
    split32(t.sc0, t.sc1, scx, scy);
    split32(t.zz0, t.zz1, zzx, zzy);
    float x0, x1, y0, y1;
    pair_plane(pa, bx, x0, x1);
    pair_plane(pa, by, y0, y1);
    // G = 64: the unit's dword holds the scales of its two half units; G = 128: the pair's dword holds the
    // scales of its two units, one group each
    const float sx0 = G64 ? h2f_lo(scx) : (second ? h2f_hi(scx) : h2f_lo(scx)), sx1 = G64 ? h2f_hi(scx) : sx0;
    const float sy0 = G64 ? h2f_lo(scy) : (second ? h2f_hi(scy) : h2f_lo(scy)), sy1 = G64 ? h2f_hi(scy) : sy0;
    accx = fmaf(x0 * pf.inv0, sx0, accx);
    accx = fmaf(x1 * pf.inv1, sx1, accx);
    accy = fmaf(y0 * pf.inv0, sy0, accy);
    accy = fmaf(y1 * pf.inv1, sy1, accy);
    if (plane0) {
        const float zx0 = G64 ? h2f_lo(zzx) : (second ? h2f_hi(zzx) : h2f_lo(zzx)), zx1 = G64 ? h2f_hi(zzx) : zx0;
        const float zy0 = G64 ? h2f_lo(zzy) : (second ? h2f_hi(zzy) : h2f_lo(zzy)), zy1 = G64 ? h2f_hi(zzy) : zy0;
        accx = fmaf(zx0, pf.xs0, accx);
        accx = fmaf(zx1, pf.xs1, accx);
        accy = fmaf(zy0, pf.xs0, accy);
        accy = fmaf(zy1, pf.xs1, accy);
    }
}

// Cross-wave sum of a column block and the meeting of its K slices: the LUT kernel's output stage.
template <bool MULTI, bool PLAIN>
__device__ __forceinline__ void mf_finish(const GemvArgs &a, int cbf, int slice, float accf, float *red0, int &red_sel, int nw,
                                          int wave, int lane, int fin, const HLQ_GLOBAL uint16_t *residual,
                                          const HLQ_GLOBAL float *extra)
{
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
            if (a.bias) total += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            if (residual) total += (float)__builtin_bit_cast(_Float16, residual[n]);
            if (extra) total += extra[n];
            a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
        }
        return;
    }
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    if (!PLAIN && a.defer) {
        if (wave == fin) a.partial[(size_t)slice * npad + n] = total;
        return;
    }
    if (wave == fin) {
        float sum;
        if (slices_meet(a, cbf, slice, npad, n, lane, total, sum) && n < a.N) {
            if (a.bias) sum += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            if (residual) sum += (float)__builtin_bit_cast(_Float16, residual[n]);
            if (extra) sum += extra[n];
            a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)sum);
        }
    }
}

// One workgroup = `ncb_run` consecutive column blocks x one K slice.  The unit pairs of the slice are
// dealt to the waves in contiguous runs of at most MAXP; a wave builds the A operands of its pairs once
// (own LDS region, no workgroup barrier) and keeps them in registers over all column blocks of the run,
// while the plane data of the next sub-task is in flight.
template <int BITS, bool G64, int MAXP, int VAR>
__device__ __forceinline__ void mfma_tile(const GemvArgs &a, int cb, int slice, int ncb_run, unsigned char *smem, int &red_sel)
{
    HLQ_STAMP_DECL;
    HLQ_STAMP(0);
    constexpr bool PLAIN = VAR != GEMV_FUSED;
    const int prologue = PLAIN ? 0 : a.prologue;
    const HLQ_GLOBAL uint16_t *residual = PLAIN ? nullptr : a.residual;
    const HLQ_GLOBAL float *extra = VAR == GEMV_EXTRA ? a.extra : nullptr;
    const int tid = threadIdx.x, lane = tid & 63, nw = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = a.K;                                                      // (host: whole units only)
    const int u0 = slice * a.ups, nU = min(u0 + a.ups, a.U) - u0;
    const int npairs = (nU + 1) >> 1;
    const int ppw = (npairs + nw - 1) / nw;                                 // <= MAXP (host)
    const int p_begin = min(wave * ppw, npairs), p_end = min(p_begin + ppw, npairs);
    const int u_last = u0 + nU - 1;

    const HlqLdsMap lm = hlq_lds_map(nw, MAXP * MF_PAIR_LDS);
    unsigned char *wlds = smem + (size_t)wave * (MAXP * MF_PAIR_LDS);
    float *red0 = (float *)(smem + lm.red);
    float *rstd_scratch = (float *)(smem + lm.rstd);
    uint2 *stage = (uint2 *)(smem + lm.stage);

    // activations of the wave's pairs first (one chunk of 4 k per lane and pair), then the weight stream
    float rstd = 1.f;
    uint2 rfirst = make_uint2(0, 0);
    if (prologue == 1) rfirst = rstd_first_load(a, K, tid);
    const bool sliced = !PLAIN && a.n_slices_in > 0;
    SliceChunk sfirst = {};
    if (sliced) load_slice_chunk(a, K, min(tid, K / 4 - 1), sfirst);
    uint2 raw[MAXP], raw2[MAXP];
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        const int p = min(p_begin + i, max(p_end - 1, 0));
        const int ku = u0 + 2 * p + (lane >> 5);                            // the lane's unit; past the slice: re-read the last one
        const size_t k = (size_t)min(ku, u_last) * HLQ_UNIT + (size_t)(lane & 31) * 4;
        load_chunk<PLAIN>(a, prologue, K, k, raw[i], raw2[i]);
    }
    asm volatile("" ::: "memory");
    // The wave's sub-tasks form one stream over the run: position q = (column block, pair, plane), plane fastest.
    // NS of them are in registers or on their way at any time; slot q % NS is refilled with position q + NS as soon as
    // position q has been worked on (past the end: a reload nobody reads), so the weight stream never stops.
    constexpr int NS = mf_slots(BITS, G64, MAXP);
    const int npw = p_end - p_begin;                                        // pairs of this wave: 0..MAXP
    const int steps = ncb_run * npw;                                        // (column block, pair) steps of the stream
    PairLoad slot[NS];
    auto load_at = [&](auto bc, PairLoad &t, int ps) __attribute__((always_inline)) {
        constexpr int b = decltype(bc)::value;
        const int psc = min(ps, max(steps - 1, 0));
        const int c = (MAXP > 1 && npw == 2) ? psc >> 1 : psc, i = (MAXP > 1 && npw == 2) ? psc & 1 : 0;
        const int p = min(p_begin + i, max(npairs - 1, 0));
        load_pair<BITS, G64, b>(t, a, cb + c, u0 + 2 * p, u_last, lane);
    };
    // the first sub-task's loads start the weight stream; the others follow the A operands (a wave that queued all
    // its loads first would sit in the memory pipeline's back-pressure instead of building them)
    load_at(std::integral_constant<int, 0>{}, slot[0], 0);
    asm volatile("" ::: "memory");
    if (prologue == 1)
        rstd = block_rstd(a, K, rstd_scratch, tid, blockDim.x, rfirst, sfirst, sliced, stage,
                          sliced && a.x_out && blockIdx.x == 0 && blockIdx.y == 0);

    HLQ_STAMP(1);
    // the halves of the A records that no activation is ever written to, and the zero record
    for (int o = lane * 16; o < MAXP * MF_PAIR_LDS; o += 64 * 16) *(uint4 *)(wlds + o) = make_uint4(0, 0, 0, 0);
    // one pair per wave: its A operands stay in registers over all column blocks; two pairs: they are read back
    // from the wave's LDS region at the head of each pair's planes (32 registers instead of 64)
    constexpr int NPA = MAXP == 1 ? 1 : 0;
    PairA pa[1];
    PairFold pf[MAXP];
#pragma unroll
    for (int i = 0; i < MAXP; i++) {
        if (p_begin + i < p_end) {                                          // wave-uniform
            const int ku = u0 + 2 * (p_begin + i) + (lane >> 5);
            uint2 r = raw[i];
            if (sliced) r = stage[(size_t)min(ku, u_last) * 32 + (lane & 31)];
            float v[4];
            chunk_values(prologue, r, raw2[i], rstd, v);
            if (ku > u_last) v[0] = v[1] = v[2] = v[3] = 0.f;               // the odd unit out of a slice has no partner
            unsigned char *img = wlds + i * MF_PAIR_LDS;
            float *meta = (float *)(img + MF_IMG_BYTES + MF_REC);
            build_pair(v, img, meta, lane);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();                                // written and read by this wave: LDS keeps a wave's order
            if (NPA) load_pair_a(pa[0], img, lane);
            const int unit = lane >> 5;
            pf[i].inv0 = meta[unit * 2];
            pf[i].inv1 = meta[unit * 2 + 1];
            pf[i].xs0 = meta[4 + unit * 2];
            pf[i].xs1 = meta[4 + unit * 2 + 1];
        }
    }
    asm volatile("" ::: "memory");
    static_for<1, NS>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        load_at(std::integral_constant<int, j % BITS>{}, slot[j], j / BITS);
    });
    HLQ_STAMP(2);

    // where the last wave has no pair it takes the meeting of the K slices (its wait for the stores'
    // acknowledgement then covers no weight loads)
    const int fin = (a.ksplit > 1 && (nw - 1) * ppw >= npairs) ? nw - 1 : 0;
    auto finish_cb = [&](int cbf, float accx, float accy) __attribute__((always_inline)) {
        // both lane halves of a column half hold shares (first / second unit of each pair): add them, then lane l
        // carries column l of the block
        accx += __shfl_xor(accx, 32, 64);
        accy += __shfl_xor(accy, 32, 64);
        mf_finish<true, PLAIN>(a, cbf, slice, lane < 32 ? accx : accy, red0, red_sel, nw, wave, lane, fin, residual, extra);
    };
    if (npw == 0) {                                                         // a wave without a pair only takes part in the sums
        for (int c = 0; c < ncb_run; c++) finish_cb(cb + c, 0.f, 0.f);
        HLQ_STAMP_FLUSH;
        return;
    }
    constexpr int UNROLL = NS * BITS / mf_gcd(NS, BITS);                    // slot and plane of a position are compile-time
    float accx = 0.f, accy = 0.f;
    for (int q0 = 0; q0 < steps * BITS; q0 += UNROLL) {
        static_for<0, UNROLL>([&](auto jc) __attribute__((always_inline)) {
            constexpr int j = decltype(jc)::value, b = j % BITS, sl = j % NS, nb = (j + NS) % BITS;
            const int ps = q0 / BITS + j / BITS;
            if (ps < steps) {                                               // wave-uniform
                const int c = (MAXP > 1 && npw == 2) ? ps >> 1 : ps, i = (MAXP > 1 && npw == 2) ? ps & 1 : 0;
                if (!NPA && b == 0) load_pair_a(pa[0], wlds + i * MF_PAIR_LDS, lane);
                PairFold f = pf[0];
                if constexpr (MAXP > 1) {
                    if (i) f = pf[1];
                }
                process_pair<G64>(slot[sl], pa[0], f, b == 0, lane, accx, accy);
                load_at(std::integral_constant<int, nb>{}, slot[sl], q0 / BITS + (j + NS) / BITS);
                if (b == BITS - 1 && i == npw - 1) {
                    HLQ_STAMP(3);
                    finish_cb(cb + c, accx, accy);
                    accx = accy = 0.f;
                    HLQ_STAMP(4);
                }
            }
        });
    }
    HLQ_STAMP_FLUSH;
}

// grid = (K slices, runs of column blocks)
template <int BITS, bool G64, int MAXP, int VAR>
__global__ __launch_bounds__(1024) void hlq_gemv_mfma_kernel(const GemvArgs a, int run)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const int cb0 = blockIdx.y * run;
    int sel = 0;
    mfma_tile<BITS, G64, MAXP, VAR>(a, cb0, blockIdx.x, min(run, a.ncb - cb0), smem, sel);
}

template <int BITS, bool G64, int MAXP, int VAR>
int launch_mfma(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    auto kern = hlq_gemv_mfma_kernel<BITS, G64, MAXP, VAR>;
    static bool big_lds_done[64] = {};
    if (lds > 64 * 1024) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ELUTQ_ERR_HIP;
        if (!big_lds_done[dev]) {
            if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, HLQ_MAX_LDS) != hipSuccess)
                return ELUTQ_ERR_HIP;
            big_lds_done[dev] = true;
        }
    }
    // more tiles than compute units: every workgroup walks a run of column blocks with the same A operands
    const int run = (a.ncb * a.ksplit + HLQ_NUM_CU - 1) / HLQ_NUM_CU;
    const int groups = (a.ncb + run - 1) / run;
    hipLaunchKernelGGL(kern, dim3(a.ksplit, groups), dim3(waves * 64), lds, stream, a, run);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64, int MAXP>
int launch_mfma_v(const GemvArgs &a, int waves, size_t lds, hipStream_t stream)
{
    if (a.extra) return launch_mfma<BITS, G64, MAXP, GEMV_EXTRA>(a, waves, lds, stream);
    if (a.prologue == 0 && !a.residual && !a.defer && a.n_slices_in == 0)
        return launch_mfma<BITS, G64, MAXP, GEMV_PLAIN>(a, waves, lds, stream);
    return launch_mfma<BITS, G64, MAXP, GEMV_FUSED>(a, waves, lds, stream);
}

template <int BITS, bool G64>
int launch_mfma_p(const GemvArgs &a, int maxp, int waves, size_t lds, hipStream_t stream)
{
    return maxp == 1 ? launch_mfma_v<BITS, G64, 1>(a, waves, lds, stream) : launch_mfma_v<BITS, G64, 2>(a, waves, lds, stream);
}

}  // namespace

#ifdef HLQ_TIMING
extern "C" int elutq_debug_set_mfma_stamps(void *d_buf)
{
    return hipMemcpyToSymbol(HIP_SYMBOL(g_hlq_stamps), &d_buf, sizeof(d_buf)) == hipSuccess ? 0 : -1;
}
#endif

size_t hlq_gemv_mfma_lds_bytes(int ups, int waves)
{
    const int npairs = (ups + 1) / 2, ppw = (npairs + waves - 1) / waves;
    const int maxp = ppw <= 1 ? 1 : 2;
    return hlq_lds_map(waves, maxp * MF_PAIR_LDS).end_plain;
}

// `gemv_args` is the launcher's argument block (GemvArgs, filled as for the LUT kernel: ups, ksplit and the
// pointers are read; the wave-run fields are not).  ELUTQ_ERR_TUNING: a slice too long for two pairs per wave.
int hlq_gemv_mfma_launch(const void *gemv_args, size_t args_bytes, int bits, int group, int waves, size_t stage_bytes,
                         void *stream)
{
    if (args_bytes != sizeof(GemvArgs)) return ELUTQ_ERR_HIP;
    const GemvArgs &a = *(const GemvArgs *)gemv_args;
    const int npairs = (a.ups + 1) / 2, ppw = (npairs + waves - 1) / waves;
    if (ppw > 2 || waves < 1 || waves > 16) return ELUTQ_ERR_TUNING;
    if (a.extra && (a.prologue != 0 || a.residual)) return ELUTQ_ERR_TUNING;
    const int maxp = ppw <= 1 ? 1 : 2;
    const size_t lds = hlq_gemv_mfma_lds_bytes(a.ups, waves) + stage_bytes;
    if (lds > (size_t)HLQ_MAX_LDS) return ELUTQ_ERR_SHAPE;
    const bool g64 = group == 64;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
    case 1: return g64 ? launch_mfma_p<1, true>(a, maxp, waves, lds, st) : launch_mfma_p<1, false>(a, maxp, waves, lds, st);
    case 2: return g64 ? launch_mfma_p<2, true>(a, maxp, waves, lds, st) : launch_mfma_p<2, false>(a, maxp, waves, lds, st);
    case 3: return g64 ? launch_mfma_p<3, true>(a, maxp, waves, lds, st) : launch_mfma_p<3, false>(a, maxp, waves, lds, st);
    case 4: return g64 ? launch_mfma_p<4, true>(a, maxp, waves, lds, st) : launch_mfma_p<4, false>(a, maxp, waves, lds, st);
    }
    return ELUTQ_ERR_BITS;
}

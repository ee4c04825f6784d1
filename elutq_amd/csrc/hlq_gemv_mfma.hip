// Batch-1 HLQ GEMV on the matrix cores of gfx950 (MI355X): the bit planes go into
// v_mfma_f32_32x32x64_f8f6f4 as they lie in memory, read as fp4 (e2m1) nibbles, with no expansion, against
// fp4 digits of the activations (fp4 x fp4: 32 cycles per MFMA).
// Same computation, buffers and launch structure as the LUT kernel of hlq_gemv.hip (the counterpart of
// MultiThread_arm_gemv_w_lowbit_activation_fp_impl, C++/ops/src/arm/arm_gemm.cpp:312-360, and
// t_mac_g4_float_update_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469); what changes is how
// sum_k B[n,k] x[k] is formed.
//
//  * B operand.  A nibble of a plane dword holds four plane bits.  Masked to one bit position p it is the fp4
//    number v_p = 0.5 (p = 0), 1.0 (p = 1) or 2.0 (p = 2) where the bit is set and 0 where it is not; bit 3 is the
//    sign bit, so it is shifted to position 2 first.  Four masked copies ("features") of a register of plane
//    bits are four B operands, one VALU instruction each per 32 plane bits, and the four MFMAs accumulate
//    into one tile.
//  * A operand.  Per 64-k half unit the activations are scaled by a power of two that puts max|x| in
//    [2^17, 2^18) and rounded to integers (an fp16 value is kept exactly unless it lies more than seven binades
//    below the half unit's maximum; the rounding error is at most 2^-19 of that maximum), and every integer is
//    written in balanced base 7: x_int = sum_t 7^t d_t with seven digits d_t in {-3 .. 3}.  Row (half unit h,
//    digit t, unit j) of A holds d_t / v_p of the activations of that half unit and zeros elsewhere -- 2 d, d and
//    d / 2 are all fp4 numbers -- so tile element D[(h, t, j)][n] = sum over the half unit of d_t(k) B[n,k],
//    an exact integer in fp32, and sum_t 7^t D[(h, t, j)][n] is the half unit's sum for column n.  The rows
//    of a tile that a GEMM would spend on other tokens carry the digits and the four half units of a unit
//    pair.
//  * The K dimension of one MFMA is a unit pair (2 x 128 k): lanes 0-31 hold the first unit of 32
//    columns, lanes 32-63 the second.  The layout in memory has lane = column for one unit, so two loads
//    (units u, u + 1 of 64 columns) are turned into two B operands (columns 0-31 / 32-63, both units) with
//    v_permlane32_swap.
//  * Scale / zero fold per (half unit, plane) in fp32 as in the LUT kernel; K slices, the cross-wave sum,
//    prologues and epilogues are the LUT kernel's.
//
// No LDS lookups and about a third of the vector instructions per plane bit of the LUT kernel: the matrix pipe
// takes 8 MFMAs of 32 cycles per 2 KiB of plane data and wave.
#include "hlq_gemv_dev.h"
#include "hlq_internal.h"

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));

// Operand layout of v_mfma_f32_32x32x64_f8f6f4 with fp4 operands (measured on gfx950): lane l of A holds row
// l % 32, lane l of B column l % 32, both for K = 32 (l / 32) + v in nibble v % 8 of register v / 8 (v < 32);
// result register i of lane l is row 8 (i / 4) + 4 (l / 32) + i % 4 of column l % 32.  With the B operand = plane
// bits of unit u in lanes 0-31 and of unit u + 1 in lanes 32-63, row r = 16 h + 8 (t / 4) + 4 j + t % 4 (half unit
// h, digit t, unit j) is live in lane half j only, and lane half j finds the digits' tiles of its own unit in
// result registers 8 h + t.
constexpr int MF_TERMS = 7;                                   // balanced base-7 digits per activation: 3 (7^7 - 1) / 6 >= 2^18
constexpr int MF_SPLIT = 3;                                   // digits taken from the low part x_int - 7^MF_SPLIT hi
constexpr int MF_XBITS = 18;                                  // |x_int| < 2^MF_XBITS
static_assert(MF_TERMS <= 8 && MF_TERMS - MF_SPLIT <= 4, "a lane half holds eight digit rows per half unit; hi < 2048");
constexpr int MF_IMG_BYTES = 4 * 64 * 16;                     // A operands of a pair: [feature][lane][16 bytes]
constexpr int MF_STAGE_BYTES = 64 * 8;                        // the pair's 256 activations as fp16, chunk by chunk
constexpr int MF_META_FLOATS = 8;                             // per pair: 1 / scale [unit][half], sum of x [unit][half]
constexpr int MF_WAVE_LDS = (MF_IMG_BYTES + MF_STAGE_BYTES + MF_META_FLOATS * 4 + 255) & ~255;

// A operands of one unit pair in registers: [feature][register]
struct PairA {
    uint32_t a[4][4];
};

// Per-lane constants of a pair for the fold: the lane's unit is lane >> 5.
struct PairFold {
    float inv0, inv1;      // 1 / scale of the unit's two half units
    float xs0, xs1;        // sums of x over them
};

// Activations of one unit pair (256 k; on entry lane = chunk of 4 k of unit lane / 32, `v` exactly representable in
// fp16) -> the A operands of the four features and the fold constants.  The wave's LDS region is used as
// [image | staged fp16 activations | half-unit records]; the image's bytes that no digit is ever written to are zero
// (the caller zero-fills it once).
//
// After the staging every lane owns one byte of every (feature, digit) row: two neighbouring K positions (nibbles
// 2 b, 2 b + 1 of plane dword dd of unit j) of two features -- lane = 32 j + 8 dd + 2 b + g, g = 0: features 2 and 3
// (plane bits 2, 3 of a nibble: values 0 and 1 of chunks 2 b and 2 b + 1 of the dword), g = 1: features 0 and 1
// (values 2 and 3 of chunks 2 b - 1 and 2 b; the dword's last chunk wraps to nibble 0, as the rotated layout has it).
__device__ __forceinline__ void build_pair(const float (&v)[4], unsigned char *region, int lane, PairA &pa, PairFold &pf)
{
    unsigned char *img = region;
    uint32_t *stage = (uint32_t *)(region + MF_IMG_BYTES);
    float *meta = (float *)(region + MF_IMG_BYTES + MF_STAGE_BYTES);
    auto pack = [](float lo, float hi) __attribute__((always_inline)) {
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
    };
    *(uint2 *)(stage + 2 * lane) = make_uint2(pack(v[0], v[1]), pack(v[2], v[3]));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();                          // written and read by this wave: LDS keeps a wave's order
    const int j = lane >> 5, dd = (lane >> 3) & 3, b = (lane >> 1) & 3, g = lane & 1;
    const int ca = dd * 8 + ((2 * b + (g ? 7 : 0)) & 7), cb = dd * 8 + 2 * b + (g ? 0 : 1);
    const uint32_t ra = stage[(j * 32 + ca) * 2 + g], rb = stage[(j * 32 + cb) * 2 + g];
    // x[0], x[1]: the lower feature of the lane (value 0 or 2 of the chunk) at the two K positions; x[2], x[3]: the upper
    const float x[4] = {h2f_lo(ra), h2f_lo(rb), h2f_hi(ra), h2f_hi(rb)};
    float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
    float s = (x[0] + x[1]) + (x[2] + x[3]);
    HLQ_ROW_REDUCE(s, op_add);                                // the 16 lanes of a DPP row hold one half unit
    HLQ_ROW_REDUCE(amax, op_max);
    // amax in [2^(eb-127), 2^(eb-126)): times 2^(126+MF_XBITS-eb) it lies in [2^(MF_XBITS-1), 2^MF_XBITS)
    const uint32_t eb = (__float_as_uint(amax) >> 23) & 0xffu;
    const float scale = eb ? __uint_as_float((253u + MF_XBITS - eb) << 23) : 1.0f;
    const float inv = eb ? __uint_as_float((eb + 1u - MF_XBITS) << 23) : 1.0f;
    // x_int = lo + 343 hi with |lo| <= 171, |hi| <= 765: three and four balanced base-7 digits, in packed fp16
    // arithmetic (all values are integers below 2048, so every operation is exact; q = rint(x / 7) by a fused
    // multiply-add with 1536 and its subtraction, which is safe because x / 7 is never within 1/14 of a half integer
    // and 765 |fp16(1/7) - 1/7| < 0.03)
    constexpr float P7 = MF_SPLIT == 3 ? 343.0f : 2401.0f;
    float lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float xi = rintf(x[i] * scale);
        hi[i] = rintf(xi * (1.0f / P7));
        lo[i] = fmaf(-P7, hi[i], xi);
    }
    h2v dig[2][MF_TERMS];                                      // [feature of the lane][digit], .x / .y = the two K positions
    const h2v c7 = {(_Float16)(1.0f / 7.0f), (_Float16)(1.0f / 7.0f)}, big = {(_Float16)1536.0f, (_Float16)1536.0f};
    const h2v m7 = {(_Float16)-7.0f, (_Float16)-7.0f};
#pragma unroll
    for (int f = 0; f < 2; f++) {
#pragma unroll
        for (int part = 0; part < 2; part++) {
            h2v X = __builtin_bit_cast(h2v, part ? __builtin_amdgcn_cvt_pkrtz(hi[2 * f], hi[2 * f + 1])
                                                 : __builtin_amdgcn_cvt_pkrtz(lo[2 * f], lo[2 * f + 1]));
            const int t0 = part ? MF_SPLIT : 0, nd = part ? MF_TERMS - MF_SPLIT : MF_SPLIT;
#pragma unroll
            for (int t = 0; t < nd - 1; t++) {
                const h2v q = __builtin_elementwise_fma(X, c7, big) - big;
                dig[f][t0 + t] = __builtin_elementwise_fma(q, m7, X);
                X = q;
            }
            dig[f][t0 + nd - 1] = X;
        }
    }
    // the byte of row (h, t, j) of feature p: image[p][r + 32 j][4 dd + b], r = 16 h + 8 (t / 4) + 4 j + t % 4; the A
    // operand is digit / v_p: v_0 = 0.5, v_1 = 1, v_2 = v_3 = 2 (the conversion divides by its scale operand)
    const int p_lo = g ? 0 : 2;
    const float sc_lo = g ? 0.5f : 2.0f, sc_hi = g ? 1.0f : 2.0f;
    unsigned char *dst = img + p_lo * 1024 + ((dd >> 1) * 16 + 36 * j) * 16 + 4 * dd + b;
#pragma unroll
    for (int t = 0; t < MF_TERMS; t++) {
        constexpr int dummy = 0;
        (void)dummy;
        const int roff = (8 * (t / 4) + t % 4) * 16;
        dst[roff] = (unsigned char)__builtin_amdgcn_cvt_scalef32_pk_fp4_f16(0u, dig[0][t], sc_lo, 0);
        dst[1024 + roff] = (unsigned char)__builtin_amdgcn_cvt_scalef32_pk_fp4_f16(0u, dig[1][t], sc_hi, 0);
    }
    if ((lane & 15) == 0) {
        const int h4 = lane >> 4;                             // (unit, half) 0..3
        meta[h4] = inv;
        meta[4 + h4] = s;
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const uint4 r = *(const uint4 *)(img + p * 1024 + lane * 16);
        pa.a[p][0] = r.x; pa.a[p][1] = r.y; pa.a[p][2] = r.z; pa.a[p][3] = r.w;
    }
    pf.inv0 = meta[j * 2];
    pf.inv1 = meta[j * 2 + 1];
    pf.xs0 = meta[4 + j * 2];
    pf.xs1 = meta[4 + j * 2 + 1];
}

// One plane of one unit pair for 32 columns: four features into one tile, then the digits of each half unit weighted
// by their powers of 7.  A tile element is a sum of at most 64 products of |digit| <= 3 and 1: exact in fp32, and so is
// every partial sum of the Horner chain (< 2^24).
__device__ __forceinline__ void pair_plane(const PairA &pa, const uint32_t (&b)[4], float &half0, float &half1)
{
    v16f d = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 4; p++) {
        v8i av = {(int)pa.a[p][0], (int)pa.a[p][1], (int)pa.a[p][2], (int)pa.a[p][3], 0, 0, 0, 0};
        v8i bv = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t m = p == 0 ? 0x11111111u : (p == 1 ? 0x22222222u : 0x44444444u);
            bv[i] = (int)((p == 3 ? b[i] >> 1 : b[i]) & m);
        }
        d = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, d, 4, 4, 0, 0, 0, 0);
    }
    float h0 = d[MF_TERMS - 1], h1 = d[8 + MF_TERMS - 1];
#pragma unroll
    for (int t = MF_TERMS - 2; t >= 0; t--) {
        h0 = fmaf(h0, 7.0f, d[t]);
        h1 = fmaf(h1, 7.0f, d[8 + t]);
    }
    half0 = h0;
    half1 = h1;
}

// Sub-tasks a wave has in registers or in flight (10 to 12 registers each).  Two: measured on MI355X, a deeper ring
// streams slower (the sixteen waves of a compute unit then crowd its memory pipeline with requests that are far
// from being consumed).
#ifdef MF_NS_OVERRIDE
constexpr int mf_slots(int bits, bool g64, int maxp) { return MF_NS_OVERRIDE; }
#else
constexpr int mf_slots(int bits, bool g64, int maxp) { return 2; }
#endif
constexpr int mf_gcd(int a, int b) { return b == 0 ? a : mf_gcd(b, a % b); }

// Plane data of one (unit pair, plane) sub-task for the 64 columns of a block, as loaded (lane = column).
struct PairLoad {
    uint4 w0, w1;          // units u and u + 1
    uint32_t sc0, sc1;     // scale dwords (G = 128: sc0 only, the pair's dword; G = 64: one per unit)
    uint32_t zz0, zz1;     // zero dwords, plane 0 only
};

// The buffers of a layer as the loads need them.
struct LayerRef {
    const HLQ_GLOBAL unsigned char *planes, *scales, *zeros;
    int U, NT;
};

template <int BITS, bool G64, int b>
__device__ __forceinline__ void load_pair(PairLoad &t, const LayerRef &a, int cb, int u, int u_last, int lane)
{
    const uint32_t u1 = (uint32_t)min(u + 1, u_last);
    const HLQ_GLOBAL unsigned char *pl = a.planes + (size_t)cb * a.U * (size_t)(BITS * HLQ_CB * 16);
    const HLQ_GLOBAL unsigned char *sc = a.scales + (size_t)cb * a.NT * (size_t)(BITS * HLQ_CB * 4);
    const HLQ_GLOBAL unsigned char *zz = a.zeros + (size_t)cb * a.NT * (size_t)(HLQ_CB * 4);
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
// (own LDS region, no workgroup barrier) and keeps them in registers (16 per pair) over all column blocks of the
// run, while the plane data of the next sub-task is in flight.
__device__ __forceinline__ LayerRef layer_ref(const GemvArgs &a)
{
    LayerRef r;
    r.planes = (const HLQ_GLOBAL unsigned char *)a.planes;
    r.scales = (const HLQ_GLOBAL unsigned char *)a.scales;
    r.zeros = (const HLQ_GLOBAL unsigned char *)a.zeros;
    r.U = a.U; r.NT = a.NT;
    return r;
}

template <int BITS, bool G64, int MAXP, int VAR>
__device__ __forceinline__ void mfma_tile(const GemvArgs &a, int cb, int slice, int ncb_run, unsigned char *smem, int &red_sel)
{
    const LayerRef lref = layer_ref(a);
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

    const HlqLdsMap lm = hlq_lds_map(nw, MF_WAVE_LDS);
    unsigned char *wlds = smem + (size_t)wave * MF_WAVE_LDS;
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
        load_pair<BITS, G64, b>(t, lref, cb + c, u0 + 2 * p, u_last, lane);
    };
    // the first sub-task's loads start the weight stream; the others follow the A operands (a wave that queued all
    // its loads first would sit in the memory pipeline's back-pressure instead of building them)
    load_at(std::integral_constant<int, 0>{}, slot[0], 0);
    asm volatile("" ::: "memory");
    if (prologue == 1)
        rstd = block_rstd(a, K, rstd_scratch, tid, blockDim.x, rfirst, sfirst, sliced, stage,
                          sliced && a.x_out && blockIdx.x == 0 && blockIdx.y == 0);

    // the bytes of the operand image that no digit is ever written to (rows of digits that do not exist, the lane
    // half that does not face a row's unit)
    for (int o = lane * 16; o < MF_IMG_BYTES; o += 64 * 16) *(uint4 *)(wlds + o) = make_uint4(0, 0, 0, 0);
    PairA pa[MAXP];
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
            build_pair(v, wlds, lane, pa[i], pf[i]);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();                                // the next pair reuses the region
        }
    }
    asm volatile("" ::: "memory");
    static_for<1, NS>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        load_at(std::integral_constant<int, j % BITS>{}, slot[j], j / BITS);
    });

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
                if constexpr (MAXP > 1) {
                    if (i) process_pair<G64>(slot[sl], pa[1], pf[1], b == 0, lane, accx, accy);     // wave-uniform
                    else process_pair<G64>(slot[sl], pa[0], pf[0], b == 0, lane, accx, accy);
                } else {
                    process_pair<G64>(slot[sl], pa[0], pf[0], b == 0, lane, accx, accy);
                }
                load_at(std::integral_constant<int, nb>{}, slot[sl], q0 / BITS + (j + NS) / BITS);
                if (b == BITS - 1 && i == npw - 1) {
                    finish_cb(cb + c, accx, accy);
                    accx = accy = 0.f;
                }
            }
        });
    }
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

// ---- grouped launch: many independent GEMVs, every workgroup streams its own contiguous share of all the bytes ----
//
// A tile is up to MF_ITEM_CBS consecutive column blocks of one layer over ALL of K: nothing meets in device memory.
// The work units (unit pair, column block), pair-major, are dealt to the sixteen waves in equal contiguous shares,
// whatever the number of pairs; a wave rebuilds its A operands when its share moves on to another pair (the
// activations of that pair were requested while the previous one was being streamed) and adds what a unit
// contributes to a column block into its own row of a per-workgroup table in LDS.  One barrier per tile, after
// which wave c sums the sixteen rows of column block c in wave order and stores its 64 outputs while the others are
// already in the next tile (the table alternates between two copies).  The ring of plane loads runs on across tile
// boundaries: the last positions of a tile are refilled with the first ones of the next.
constexpr int MF_ITEM_CBS = HLQ_MFMA_ITEM_CBS;
typedef HlqMfmaItem MfmaItem;
typedef HlqMfmaShare ItemShare;

// A tile's layer: what the kernel reads of its argument block, in registers.
struct TileLayer {
    LayerRef w;
    const HLQ_GLOBAL uint16_t *x, *bias;
    HLQ_GLOBAL uint16_t *y;
    int N;
};

__device__ __forceinline__ TileLayer tile_layer(const GemvArgs *__restrict__ problems, int i)
{
    const GemvArgs *a = problems + i;
    TileLayer t;
    t.w.planes = (const HLQ_GLOBAL unsigned char *)a->planes;
    t.w.scales = (const HLQ_GLOBAL unsigned char *)a->scales;
    t.w.zeros = (const HLQ_GLOBAL unsigned char *)a->zeros;
    t.w.U = a->U; t.w.NT = a->NT;
    t.x = a->x; t.bias = a->bias; t.y = a->y; t.N = a->N;
    return t;
}

__device__ __forceinline__ void unit_of(const ItemShare &v, int m, int &p, int &c) { hlq_mfma_unit_of(v, m, p, c); }

// Where a workgroup's tiles come from: the plan of a grouped launch ...
struct PlannedTiles {
    const GemvArgs *__restrict__ problems;
    const MfmaItem *__restrict__ items;
    int i_begin, i_end;
    __device__ __forceinline__ int count() const { return i_end - i_begin; }
    __device__ __forceinline__ MfmaItem item(int i) const { return items[i_begin + i]; }
    __device__ __forceinline__ TileLayer layer(const MfmaItem &it) const { return tile_layer(problems, it.problem); }
};

// ... or, for one wide layer, the workgroup's equal share of its column blocks cut into tiles on the fly.
struct LayerTiles {
    TileLayer l;
    int cb_begin, cb_end;
    __device__ __forceinline__ int count() const { return (cb_end - cb_begin + MF_ITEM_CBS - 1) / MF_ITEM_CBS; }
    __device__ __forceinline__ MfmaItem item(int i) const
    {
        const int cb0 = cb_begin + i * MF_ITEM_CBS, len = min(MF_ITEM_CBS, cb_end - cb0);
        return MfmaItem{0, cb0, len, (int)(((1u << 20) + (unsigned)len - 1u) / (unsigned)len)};
    }
    __device__ __forceinline__ TileLayer layer(const MfmaItem &) const { return l; }
};

template <int BITS, bool G64, typename Tiles>
__device__ __forceinline__ void mfma_stream_tiles(const Tiles &tiles, unsigned char *smem)
{
    constexpr int NW = 16, NS = 2;
    constexpr int UNROLL = NS * BITS / mf_gcd(NS, BITS);                   // slot and plane of a position are compile-time
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned char *wlds = smem + (size_t)wave * MF_WAVE_LDS;
    typedef __attribute__((address_space(3))) float lds_float;
    lds_float *accl0 = (lds_float *)(smem + (size_t)NW * MF_WAVE_LDS);     // [2][MF_ITEM_CBS][NW][64]
    // the bytes of the operand image that no digit is ever written to stay zero for the whole launch
    for (int o = lane * 16; o < MF_IMG_BYTES; o += 64 * 16) *(uint4 *)(wlds + o) = make_uint4(0, 0, 0, 0);

    const int n_tiles = tiles.count();
    if (n_tiles <= 0) return;
    MfmaItem it = tiles.item(0);
    TileLayer a = tiles.layer(it);
    ItemShare v = hlq_mfma_share(a.w.U, it, wave, BITS, UNROLL);

    // activations of unit pair p of a layer (lane = chunk of 4 k of unit lane / 32); past the layer: its last unit, zeroed later
    auto load_x = [&](const HLQ_GLOBAL uint16_t *x, const ItemShare &sv, int p, uint2 &raw) __attribute__((always_inline)) {
        const int ku = min(2 * min(p, sv.npairs - 1) + (lane >> 5), sv.u_last);
        raw = *(const HLQ_GLOBAL uint2 *)(x + ((size_t)ku * HLQ_UNIT + (size_t)(lane & 31) * 4));
    };
    auto load_pos = [&](auto bc, PairLoad &t, const LayerRef &g, const ItemShare &sv, int pos) __attribute__((always_inline)) {
        constexpr int b = decltype(bc)::value;
        int p, c;
        hlq_mfma_load_target(sv, pos, BITS, p, c);
        load_pair<BITS, G64, b>(t, g, sv.cb0 + c, 2 * p, sv.u_last, lane);
    };

    uint2 raw_next;
    const HLQ_GLOBAL uint16_t *raw_x = a.x;       // raw_next = the activations of pair raw_p of the layer whose x is raw_x
    int raw_p;
    { int c; unit_of(v, v.m_lo, raw_p, c); }
    load_x(a.x, v, raw_p, raw_next);
    asm volatile("" ::: "memory");
    PairLoad slot[NS];
    static_for<0, NS>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        load_pos(std::integral_constant<int, j % BITS>{}, slot[j], a.w, v, j);
    });
    PairA pa;
    PairFold pf;
    const HLQ_GLOBAL uint16_t *cur_x = nullptr;   // pa / pf: pair cur_p of the layer whose x is cur_x
    int cur_p = -1;
    int buf = 0;
    for (int i = 0; i < n_tiles; i++) {
        MfmaItem itn = it;
        TileLayer an = a;
        ItemShare vn = v;
        if (i + 1 < n_tiles) {                     // (no next tile: the ring is refilled with reloads nobody reads)
            itn = tiles.item(i + 1);
            an = tiles.layer(itn);
            vn = hlq_mfma_share(an.w.U, itn, wave, BITS, UNROLL);
        }
        lds_float *accl = accl0 + buf * (MF_ITEM_CBS * NW * HLQ_CB);
        for (int c = 0; c < v.ncb; c++) accl[(c * NW + wave) * HLQ_CB + lane] = 0.f;
        int p_last, c_last;
        unit_of(v, v.m_lo + max(v.nt / BITS - 1, 0), p_last, c_last);
        int pn_first, cn_first;
        unit_of(vn, vn.m_lo, pn_first, cn_first);
        float accx = 0.f, accy = 0.f;
        for (int q0 = 0; q0 < v.nt_pad; q0 += UNROLL) {
            static_for<0, UNROLL>([&](auto jc) __attribute__((always_inline)) {
                constexpr int j = decltype(jc)::value, b = j % BITS, sl = j % NS, nb = (j + NS) % BITS;
                const int pos = q0 + j;
                int p, c;
                unit_of(v, v.m_lo + q0 / BITS + j / BITS, p, c);
                if (pos < v.nt) {                                           // wave-uniform
                    if (b == 0 && (p != cur_p || a.x != cur_x)) {           // wave-uniform: the share moves on to another pair
                        if (raw_p != p || raw_x != a.x) load_x(a.x, v, p, raw_next);    // (not requested ahead: the first tile of a share)
                        float xv[4];
                        chunk_values(0, raw_next, raw_next, 1.f, xv);
                        if (2 * p + (lane >> 5) > v.u_last) xv[0] = xv[1] = xv[2] = xv[3] = 0.f;   // the odd unit out has no partner
                        // the pair this wave builds next: the following one of this tile, else the first of the next tile
                        if (p < p_last) { raw_p = p + 1; raw_x = a.x; load_x(a.x, v, raw_p, raw_next); }
                        else { raw_p = pn_first; raw_x = an.x; load_x(an.x, vn, raw_p, raw_next); }
                        build_pair(xv, wlds, lane, pa, pf);
                        cur_p = p;
                        cur_x = a.x;
                    }
                    process_pair<G64>(slot[sl], pa, pf, b == 0, lane, accx, accy);
                }
                // refill: the position NS further on, in the next tile where this one ends
                if (pos + NS < v.nt_pad) load_pos(std::integral_constant<int, nb>{}, slot[sl], a.w, v, pos + NS);
                else load_pos(std::integral_constant<int, nb>{}, slot[sl], an.w, vn, pos + NS - v.nt_pad);
                if (b == BITS - 1 && pos < v.nt) {
                    // both lane halves of a column half hold shares (first / second unit of the pair)
                    accx += __shfl_xor(accx, 32, 64);
                    accy += __shfl_xor(accy, 32, 64);
                    __hip_atomic_fetch_add(&accl[(c * NW + wave) * HLQ_CB + lane], lane < 32 ? accx : accy, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
                    accx = accy = 0.f;
                }
            });
        }
        if (v.nt == 0) {                           // a wave without a share in this tile still primes the ring for the next
            static_for<0, NS>([&](auto jc) __attribute__((always_inline)) {
                constexpr int j = decltype(jc)::value;
                load_pos(std::integral_constant<int, j % BITS>{}, slot[j], an.w, vn, j);
            });
        }
        lds_barrier();
        if (wave < v.ncb) {
            float total = 0.f;
            for (int w = 0; w < NW; w++) total += accl[(wave * NW + w) * HLQ_CB + lane];
            const int n = (v.cb0 + wave) * HLQ_CB + lane;
            if (n < a.N) {
                if (a.bias) total += (float)__builtin_bit_cast(_Float16, a.bias[n]);
                a.y[n] = __builtin_bit_cast(uint16_t, (_Float16)total);
            }
        }
        buf ^= 1;
        it = itn; a = an; v = vn;
    }
}

template <int BITS, bool G64>
__global__ __launch_bounds__(1024) void hlq_gemv_mfma_group_kernel(const GemvArgs *__restrict__ problems,
                                                                   const int *__restrict__ wg_begin,
                                                                   const MfmaItem *__restrict__ items)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const PlannedTiles tiles = {problems, items, wg_begin[blockIdx.x], wg_begin[blockIdx.x + 1]};
    mfma_stream_tiles<BITS, G64>(tiles, smem);
}

// One layer with (many) more column blocks than compute units, plain call: every workgroup streams an equal share of
// the column blocks over all of K.
template <int BITS, bool G64>
__global__ __launch_bounds__(1024) void hlq_gemv_mfma_wide_kernel(const GemvArgs a)
{
    extern __shared__ __align__(256) unsigned char smem[];
    const int g = blockIdx.x, ng = gridDim.x;
    TileLayer l;
    l.w = layer_ref(a);
    l.x = a.x; l.bias = a.bias; l.y = a.y; l.N = a.N;
    const LayerTiles tiles = {l, (int)((long long)g * a.ncb / ng), (int)((long long)(g + 1) * a.ncb / ng)};
    mfma_stream_tiles<BITS, G64>(tiles, smem);
}

template <int BITS, bool G64>
int launch_mfma_group(const GemvArgs *p, const int *wg_begin, const MfmaItem *it, int grid, size_t lds, hipStream_t stream)
{
    auto kern = hlq_gemv_mfma_group_kernel<BITS, G64>;
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
    hipLaunchKernelGGL(kern, dim3(grid), dim3(1024), lds, stream, p, wg_begin, it);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64>
int launch_mfma_wide(const GemvArgs &a, size_t lds, hipStream_t stream)
{
    auto kern = hlq_gemv_mfma_wide_kernel<BITS, G64>;
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
    const int grid = a.ncb < HLQ_NUM_CU ? a.ncb : HLQ_NUM_CU;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(1024), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
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

size_t hlq_gemv_mfma_lds_bytes(int ups, int waves)
{
    (void)ups;
    return hlq_lds_map(waves, MF_WAVE_LDS).end_plain;
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

// ---- host side of the grouped launch ----------------------------------------------------------------------------
size_t hlq_gemv_mfma_group_plan(const int *units, const int *ncbs, int count, int grid, void *h_blob)
{
    return hlq_mfma_group_plan(units, ncbs, count, grid, h_blob);
}

size_t hlq_gemv_mfma_group_lds_bytes(void)
{
    return (size_t)16 * MF_WAVE_LDS + (size_t)2 * MF_ITEM_CBS * 16 * HLQ_CB * sizeof(float);
}

// `d_problems`: device array of GemvArgs (pointers, N, U, K, NT, ncb are read); `d_blob`: the plan's blob on the device.
int hlq_gemv_mfma_group_launch(int bits, int group, const void *d_problems, const void *d_blob, int grid, void *stream)
{
    const GemvArgs *p = (const GemvArgs *)d_problems;
    const int *wg_begin = (const int *)d_blob;
    const MfmaItem *it = (const MfmaItem *)((const unsigned char *)d_blob + (((size_t)(grid + 1) * sizeof(int) + 15) & ~(size_t)15));
    const size_t lds = hlq_gemv_mfma_group_lds_bytes();
    const bool g64 = group == 64;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
    case 1: return g64 ? launch_mfma_group<1, true>(p, wg_begin, it, grid, lds, st) : launch_mfma_group<1, false>(p, wg_begin, it, grid, lds, st);
    case 2: return g64 ? launch_mfma_group<2, true>(p, wg_begin, it, grid, lds, st) : launch_mfma_group<2, false>(p, wg_begin, it, grid, lds, st);
    case 3: return g64 ? launch_mfma_group<3, true>(p, wg_begin, it, grid, lds, st) : launch_mfma_group<3, false>(p, wg_begin, it, grid, lds, st);
    case 4: return g64 ? launch_mfma_group<4, true>(p, wg_begin, it, grid, lds, st) : launch_mfma_group<4, false>(p, wg_begin, it, grid, lds, st);
    }
    return ELUTQ_ERR_BITS;
}

// One plain GEMV (no prologue, residual, extra term or slices: only pointers, N, U, K, NT, ncb of the argument block are
// read) of a layer with whole units, every workgroup streaming an equal share of its column blocks over all of K.
int hlq_gemv_mfma_wide_launch(const void *gemv_args, size_t args_bytes, int bits, int group, void *stream)
{
    if (args_bytes != sizeof(GemvArgs)) return ELUTQ_ERR_HIP;
    const GemvArgs &a = *(const GemvArgs *)gemv_args;
    const size_t lds = hlq_gemv_mfma_group_lds_bytes();
    const bool g64 = group == 64;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
    case 1: return g64 ? launch_mfma_wide<1, true>(a, lds, st) : launch_mfma_wide<1, false>(a, lds, st);
    case 2: return g64 ? launch_mfma_wide<2, true>(a, lds, st) : launch_mfma_wide<2, false>(a, lds, st);
    case 3: return g64 ? launch_mfma_wide<3, true>(a, lds, st) : launch_mfma_wide<3, false>(a, lds, st);
    case 4: return g64 ? launch_mfma_wide<4, true>(a, lds, st) : launch_mfma_wide<4, false>(a, lds, st);
    }
    return ELUTQ_ERR_BITS;
}

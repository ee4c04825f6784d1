// Small-batch HLQ GEMM for gfx950 (MI355X): y[M][N] = x[M][K] W^T + bias, 2 <= M <= 64 per
// launch, replacing MultiThread_arm_gemm_w_lowbit_activation_fp_impl
// (C++/ops/src/arm/arm_gemm.cpp:362-387), which re-runs the GEMV once per row.
//
// With M rows the contraction is dense enough for the matrix cores, bit-serially.  With
// c[n,g] = z[n,g] + sum_b s[b,n,g]/2 (the centre of the group's value range),
//
//   y[m][n] = sum_g ( c[n,g] * (sum_{k in g} x[m][k])  +  sum_b sum_{k in g} x[m][k] * (+-s[b,n,g]/2) )
//
// where the sign is + for a set plane bit.  The B operand of v_mfma_f32_32x32x16_f16 is
// built in registers from the packed planes: one shift (a rotation where the bits wrap) moves two
// plane bits (k and k + 16 of a 32-k dword) onto the sign bits of a packed fp16 pair, one v_bfi merges them
// with |s|/2 -- so every B element is exactly +-s/2, every product exact in fp32, and the
// fp32 accumulator of the MFMA sums planes and groups alike; nothing is rounded before the
// final fp16 store.  The centre term uses per-row sums of x over 64-k halves, taken while
// the activations are staged in LDS (in the element order the B operand uses) as A operand.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int GW = HLQ_GEMM_WAVES;             // waves per workgroup
constexpr int GEMM_THREADS = GW * 64;
constexpr int WS_COUNTER_BYTES = HLQ_WS_COUNTER_BYTES;

struct GemmArgs {
    const uint4 *planes;
    const uint32_t *scales;
    const uint32_t *zeros;
    const uint16_t *bias;
    const uint16_t *x;      // fp16 [M][K]
    uint16_t *y;            // fp16 [M][N]
    const float *extra;     // fp32 [M][N] added to the output before it is rounded, or null
    float *partial;         // [ksplit][MR][ncb*64]
    unsigned *counters;     // one per workgroup column (super block)
    int M, N, K, U, NT, ncb;
    int ksplit, ups;        // K slices per super block, units per slice (multiple of KW)
};

#ifdef HLQ_TIMING
// Profiling builds only: wall-clock stamps (100 MHz) of thread 0 of every workgroup.
__device__ unsigned long long *g_gemm_stamps = nullptr;
#define GEMM_STAMP(i)                                                                                  \
    do {                                                                                               \
        if (g_gemm_stamps && threadIdx.x == 0 && (i) < 16) {                                           \
            g_gemm_stamps[(size_t)blockIdx.x * 16 + (i)] = wall_clock64();                             \
            g_gemm_stamps[(size_t)(2048 + blockIdx.x) * 16 + (i)] = clock64();                         \
        }                                                                                              \
    } while (0)
#else
#define GEMM_STAMP(i) do { } while (0)
#endif

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Staging of x[:, u0*128 .. (u0+KW)*128) into LDS.  Inside every 32-k block the fp16 values
// are stored in operand order: position 8s + 2q + r holds k = 4s + q + 16r, so the 16 bytes
// at 8s are the A operand of MFMA step s and pair q = (k, k + 16) lines up with what one
// shift extracts from a plane dword.  One task = one such 16-byte slot of one row, built
// from two 8-byte loads (k = 4s..4s+3 and k + 16); consecutive lanes write consecutive
// slots, so the LDS stores are conflict-free.  xs[(ul*2 + half) * MR + m] receives the
// fp32 sum of x[m] over 64-k half `half` of unit ul (eight consecutive lanes).  MR = rows staged
// (16, 32 or 64).
template <int MR, int KW>
struct StageRegs {
    static constexpr int SLOTS = KW * 16;                            // 16-byte slots per row
    static constexpr int TASKS = MR * SLOTS;
    static constexpr int TPT = TASKS / GEMM_THREADS;
    static_assert(TASKS % GEMM_THREADS == 0, "whole waves of staging tasks");
    uint2 lo[TPT], hi[TPT];
};

template <int MR, int KW>
__device__ __forceinline__ void stage_load(StageRegs<MR, KW> &r, const GemmArgs &a, int u0, int u_end, int tid)
{
    constexpr int SLOTS = StageRegs<MR, KW>::SLOTS;
#pragma unroll
    for (int t = 0; t < StageRegs<MR, KW>::TPT; t++) {
        const int idx = tid + t * GEMM_THREADS;
        const int m = idx / SLOTS, o = idx % SLOTS, ul = o >> 4, blk = (o >> 2) & 3, sq = o & 3;
        const int mm = m < a.M ? m : a.M - 1, uu = u0 + ul < u_end ? u0 + ul : u_end - 1;
        const uint16_t *src = a.x + (size_t)mm * a.K + (size_t)uu * HLQ_UNIT + blk * 32 + sq * 4;
        r.lo[t] = *(const uint2 *)src;
        r.hi[t] = *(const uint2 *)(src + 16);
    }
}

template <int MR, int KW>
__device__ __forceinline__ void stage_store(const StageRegs<MR, KW> &r, _Float16 *xl, float *xs, int tid)
{
    constexpr int SLOTS = StageRegs<MR, KW>::SLOTS;
    constexpr int ROW_HALFS = KW * HLQ_UNIT + 8;
    const half2v ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
    for (int t = 0; t < StageRegs<MR, KW>::TPT; t++) {
        const int idx = tid + t * GEMM_THREADS;
        const int m = idx / SLOTS, o = idx % SLOTS;
        float sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.lo[t].x), ones, 0.f, false);
        sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.lo[t].y), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.hi[t].x), ones, sum, false);
        sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.hi[t].y), ones, sum, false);
        sum += dpp_f<0xB1>(sum);                 // lanes of a quad: the four slots of a 32-k block
        sum += dpp_f<0x4E>(sum);
        sum += dpp_f<0x141>(sum);                // the other 32-k block of the same 64-k half
        if ((o & 7) == 0) xs[(o >> 3) * MR + m] = sum;
        uint4 v;
        v.x = __builtin_amdgcn_perm(r.hi[t].x, r.lo[t].x, 0x05040100u);
        v.y = __builtin_amdgcn_perm(r.hi[t].x, r.lo[t].x, 0x07060302u);
        v.z = __builtin_amdgcn_perm(r.hi[t].y, r.lo[t].y, 0x05040100u);
        v.w = __builtin_amdgcn_perm(r.hi[t].y, r.lo[t].y, 0x07060302u);
        *(uint4 *)(xl + (size_t)m * ROW_HALFS + o * 8) = v;
    }
}

// Everything a wave needs from HBM for one unit of its column block.
template <int BITS>
struct UnitData {
    uint4 w[BITS];
    uint32_t sc[BITS];
    uint32_t zz;
};

template <int BITS, bool G64>
__device__ __forceinline__ void load_unit(UnitData<BITS> &d, const GemmArgs &a, int cb, int u, int u_end, int lane)
{
    const int uu = u < u_end ? u : u_end - 1;          // past the slice: reload a valid unit nobody uses
    const size_t meta = (size_t)cb * a.NT + (G64 ? uu : (uu >> 1));
#pragma unroll
    for (int b = 0; b < BITS; b++) {
        d.w[b] = a.planes[(((size_t)cb * a.U + uu) * BITS + b) * HLQ_CB + lane];
        d.sc[b] = a.scales[(meta * BITS + b) * HLQ_CB + lane];
    }
    d.zz = a.zeros[meta * HLQ_CB + lane];
}

// Lanes 0..31 keep `lo_src`'s lower half, lanes 32..63 receive `hi_src`'s lower half (tile 0);
// the second result is the same for the upper halves (tile 1).
__device__ __forceinline__ void split_tiles(uint32_t lo_src, uint32_t hi_src, uint32_t &t0, uint32_t &t1)
{
    const auto r = __builtin_amdgcn_permlane32_swap(lo_src, hi_src, false, false);
    t0 = r[0];
    t1 = r[1];
}

__device__ __forceinline__ float h2f(uint32_t v, bool hi)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? v >> 16 : v & 0xffffu));
}

// MR = activation rows of the launch, rounded up to 16, 32 or 64.  The MFMA tile has 32 rows; with
// MR = 16 only rows 0..15 are staged (lanes of rows 16..31 read rows 0..15 again) and only the
// accumulator registers of those rows (0..7 of 16) are reduced and stored.
template <int BITS, bool G64, int MR, int KW>
__global__ __launch_bounds__(GEMM_THREADS) void hlq_gemm_kernel(const GemmArgs a)
{
    constexpr int MT = (MR + 31) / 32;              // 32-row MFMA tiles
    constexpr int REGS = MR == 16 ? 8 : 16;         // accumulator registers per tile that hold real rows
    extern __shared__ __align__(256) unsigned char smem[];
    constexpr int CBW = GW / KW;                    // column blocks per workgroup
    constexpr int ROW_HALFS = KW * HLQ_UNIT + 8;    // 16 B pad: conflict-free b128 reads
    constexpr int TILES = MT * 2;
    constexpr int VALS = TILES * REGS * 64;         // fp32 results per wave
    constexpr int MROWS = MR;
    constexpr int XBUF = MROWS * ROW_HALFS * 2 + KW * 2 * MROWS * 4;    // bytes of one staged chunk: x, then row sums
    float *red = (float *)smem;                     // reused after the last step
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int ci = wave % CBW, kp = wave / CBW;
    const int sb = blockIdx.x / a.ksplit, slice = blockIdx.x - sb * a.ksplit;
    const int cb = sb * CBW + ci;
    const bool cb_ok = cb < a.ncb;
    const int cbc = cb_ok ? cb : a.ncb - 1;
    const int u_begin = slice * a.ups, u_end = min(u_begin + a.ups, a.U);

    float16v acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][j][i] = 0.f;

    GEMM_STAMP(0);
    int stamp_i = 1;
    (void)stamp_i;
    // Two chunk buffers in LDS alternate: while the waves compute on one, the next chunk (its
    // global loads were issued a step earlier) is written to the other, and the loads of the
    // chunk after that are issued.  One barrier per step.
    UnitData<BITS> ua, ub;
    StageRegs<MR, KW> xr;
    load_unit<BITS, G64>(ua, a, cbc, u_begin + kp, u_end, lane);
    stage_load<MR, KW>(xr, a, u_begin, u_end, tid);
    stage_store<MR, KW>(xr, (_Float16 *)smem, (float *)(smem + MROWS * ROW_HALFS * 2), tid);
    if (u_begin + KW < u_end) {
        load_unit<BITS, G64>(ub, a, cbc, u_begin + KW + kp, u_end, lane);
        stage_load<MR, KW>(xr, a, u_begin + KW, u_end, tid);
    }
    __syncthreads();

    // One step: compute on `cur` (the unit of this step), then refill it with the unit two steps
    // ahead; the caller alternates the two register sets, so no set is ever copied.
    auto step = [&](UnitData<BITS> &cur, int u0, int par) __attribute__((always_inline)) {
        GEMM_STAMP(stamp_i); stamp_i++;
        const _Float16 *xl = (const _Float16 *)(smem + par * XBUF);
        const float *xs = (const float *)(smem + par * XBUF + MROWS * ROW_HALFS * 2);
        if (u0 + KW < u_end) {
            unsigned char *nb = smem + (par ^ 1) * XBUF;
            stage_store<MR, KW>(xr, (_Float16 *)nb, (float *)(nb + MROWS * ROW_HALFS * 2), tid);
            if (u0 + 2 * KW < u_end) stage_load<MR, KW>(xr, a, u0 + 2 * KW, u_end, tid);
        }
        GEMM_STAMP(stamp_i); stamp_i++;
        const int u = u0 + kp;
        if (cb_ok && u < u_end) {
            // Lane (col, h) of tile j works on column 32j + col of the block: bring that column's
            // scale / zero dwords and its plane dwords (k half h of each 64-k pair) into the lane.
            uint32_t scj[BITS][2], zzj[2], tw[BITS][2][2];
#pragma unroll
            for (int b = 0; b < BITS; b++) {
                split_tiles(cur.sc[b], cur.sc[b], scj[b][0], scj[b][1]);
                split_tiles(cur.w[b].x, cur.w[b].y, tw[b][0][0], tw[b][1][0]);
                split_tiles(cur.w[b].z, cur.w[b].w, tw[b][0][1], tw[b][1][1]);
            }
            split_tiles(cur.zz, cur.zz, zzj[0], zzj[1]);
            // A operands are read two MFMA steps ahead of their use (three rotating registers sets);
            // scheduling barriers between the steps keep the compiler from sinking the reads
            const _Float16 *arow = xl + (size_t)(MR == 16 ? (col & 15) : col) * ROW_HALFS + kp * HLQ_UNIT + h * 32;
            half8 aop[3][MT];
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    aop[st][mt] = *(const half8 *)(arow + (size_t)mt * 32 * ROW_HALFS + (st >> 2) * 64 + (st & 3) * 8);
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {          // 64-k pair of dwords: k = 64pr + 32h + ...
                const bool hi = G64 ? pr == 1 : (u & 1) != 0;       // fp16 of the meta dwords this pair belongs to
                uint32_t mag[BITS][2], bits[BITS][2];
                float cen[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    cen[j] = h2f(zzj[j], hi);
#pragma unroll
                    for (int b = 0; b < BITS; b++) {
                        const float sf = h2f(scj[b][j], hi);
                        cen[j] = fmaf(0.5f, sf, cen[j]);
                        const uint32_t m16 = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(0.5f * fabsf(sf)));
                        mag[b][j] = m16 | (m16 << 16);
                        // the sign of a B element is the plane bit, inverted unless the scale is negative
                        bits[b][j] = sf < 0.f ? tw[b][j][pr] : ~tw[b][j][pr];
                    }
                }
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const int st = pr * 4 + s;        // step 0..7 of the unit
                    if (st < 6) {
                        const int nx = st + 2;
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
                            aop[nx % 3][mt] = *(const half8 *)(arow + (size_t)mt * 32 * ROW_HALFS + (nx >> 2) * 64 + (nx & 3) * 8);
                    }
                    // planes outermost: consecutive MFMAs then go to different accumulators
#pragma unroll
                    for (int b = 0; b < BITS; b++)
#pragma unroll
                        for (int j = 0; j < 2; j++) {
                            uint32_t o[4];
#pragma unroll
                            for (int q = 0; q < 4; q++) {
                                // stored dwords are rotated left by HLQ_ROT: bit k = 4s + q goes to the sign of
                                // the low fp16, bit k + 16 to the sign of the high one
                                // (positions k + HLQ_ROT and k + 16 + HLQ_ROT move to 15 and 31).  Without a wrap a plain
                                // shift does it -- a 32-bit-encoded instruction, which the SIMD retires in 2.4
                                // cycles where v_alignbit (64-bit encoding) takes 4.25
                                const int mv = 15 - (4 * s + q + HLQ_ROT);       // left shift that is needed (compile time)
                                const uint32_t src = bits[b][j];
                                const uint32_t rot = mv > 0 ? src << mv : (mv == 0 ? src : __builtin_amdgcn_alignbit(src, src, (uint32_t)-mv));
                                o[q] = (rot & 0x80008000u) | (mag[b][j] & 0x7fff7fffu);
                            }
                            const half8 bop = __builtin_bit_cast(half8, make_uint4(o[0], o[1], o[2], o[3]));
#pragma unroll
                            for (int mt = 0; mt < MT; mt++)
                                acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[st % 3][mt], bop, acc[mt][j], 0, 0, 0);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // centre term: c[n, g] * sum_{k in g} x[m, k]; C rows of register i: 8*(i/4) + 4h + i%4
                if (G64 || pr == 1) {
#pragma unroll
                    for (int mt = 0; mt < MT; mt++)
#pragma unroll
                        for (int i4 = 0; i4 < REGS / 4; i4++) {
                            const int m0 = mt * 32 + 8 * i4 + 4 * h;
                            float4 sx = *(const float4 *)(xs + (kp * 2 + pr) * MROWS + m0);
                            if (!G64) {
                                const float4 s0 = *(const float4 *)(xs + (kp * 2) * MROWS + m0);
                                sx.x += s0.x; sx.y += s0.y; sx.z += s0.z; sx.w += s0.w;
                            }
#pragma unroll
                            for (int j = 0; j < 2; j++) {
                                acc[mt][j][4 * i4 + 0] = fmaf(cen[j], sx.x, acc[mt][j][4 * i4 + 0]);
                                acc[mt][j][4 * i4 + 1] = fmaf(cen[j], sx.y, acc[mt][j][4 * i4 + 1]);
                                acc[mt][j][4 * i4 + 2] = fmaf(cen[j], sx.z, acc[mt][j][4 * i4 + 2]);
                                acc[mt][j][4 * i4 + 3] = fmaf(cen[j], sx.w, acc[mt][j][4 * i4 + 3]);
                            }
                        }
                }
            }
        }
        GEMM_STAMP(stamp_i); stamp_i++;
        if (u0 + 2 * KW < u_end) load_unit<BITS, G64>(cur, a, cbc, u0 + 2 * KW + kp, u_end, lane);
        __syncthreads();
    };
    for (int u0 = u_begin; u0 < u_end; u0 += 2 * KW) {
        step(ua, u0, 0);
        if (u0 + KW < u_end) step(ub, u0 + KW, 1);
    }

    GEMM_STAMP(13);
    // Sum of the KW parts of every column block through LDS: red[wave][tile = mt*2+j][reg][lane].
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < REGS; i++) red[((wave * TILES + mt * 2 + j) * REGS + i) * 64 + lane] = acc[mt][j][i];
    __syncthreads();

    constexpr int NV = CBW * VALS / GEMM_THREADS;    // results per thread
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    const int mpad = MROWS;
    // value v = (column block, tile, reg, lane); C layout of the 32x32 MFMA: column = lane % 32,
    // row = 8 * (reg / 4) + 4 * (lane / 32) + reg % 4.
    auto decode = [&](int v, int &m, int &n) {
        const int c = v / VALS, r = v % VALS;
        const int ln = r & 63, reg = (r >> 6) % REGS, tile = r / (64 * REGS);
        const int mt = tile >> 1, j = tile & 1;
        m = mt * 32 + 8 * (reg >> 2) + 4 * (ln >> 5) + (reg & 3);
        n = (sb * CBW + c) * HLQ_CB + j * 32 + (ln & 31);
    };
    float outv[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int v = tid + it * GEMM_THREADS;
        const int c = v / VALS, r = v % VALS;
        float s = 0.f;
#pragma unroll
        for (int p = 0; p < KW; p++) s += red[(p * CBW + c) * VALS + r];
        outv[it] = s;
    }
    if (a.ksplit == 1) {
#pragma unroll
        for (int it = 0; it < NV; it++) {
            int m, n;
            decode(tid + it * GEMM_THREADS, m, n);
            if (m < a.M && n < a.N) {
                float s = outv[it];
                if (a.bias) s += (float)__builtin_bit_cast(_Float16, a.bias[n]);
                if (a.extra) s += a.extra[(size_t)m * a.N + n];
                a.y[(size_t)m * a.N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
            }
        }
        return;
    }
    // Slices meet through device memory, as in the GEMV: agent-scope stores, wait for their
    // acknowledgement, take a ticket; the last workgroup sums the slices in order.
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        if ((size_t)n < npad)
            __hip_atomic_store(&a.partial[((size_t)slice * mpad + m) * npad + n], outv[it], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    GEMM_STAMP(14);
    __syncthreads();
    __shared__ unsigned s_ticket;
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&a.counters[sb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)a.ksplit - 1u) return;
    // a thread's loads for QB slices are in flight together; summed in slice order
    constexpr int QB = NV <= 8 ? 4 : (NV <= 16 ? 2 : 1);
    float sum[NV];
    size_t off[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        off[it] = (size_t)n < npad ? (size_t)m * npad + n : 0;
        sum[it] = 0.f;
    }
    for (int s0 = 0; s0 < a.ksplit; s0 += QB) {
        float v[QB][NV];
#pragma unroll
        for (int q = 0; q < QB; q++) {
            const int sl = min(s0 + q, a.ksplit - 1);
#pragma unroll
            for (int it = 0; it < NV; it++)
                v[q][it] = __hip_atomic_load(&a.partial[(size_t)sl * mpad * npad + off[it]], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int q = 0; q < QB; q++)
            if (s0 + q < a.ksplit) {
#pragma unroll
                for (int it = 0; it < NV; it++) sum[it] += v[q][it];
            }
    }
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        if (m < a.M && n < a.N) {
            float s = sum[it];
            if (a.bias) s += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            if (a.extra) s += a.extra[(size_t)m * a.N + n];
            a.y[(size_t)m * a.N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
        }
    }
    if (tid == 0) __hip_atomic_store(&a.counters[sb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    GEMM_STAMP(15);
}

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

template <int MR, int KW>
size_t gemm_lds_bytes()
{
    constexpr int MT = (MR + 31) / 32, REGS = MR == 16 ? 8 : 16;
    const size_t x = 2 * ((size_t)MR * (KW * HLQ_UNIT + 8) * 2 + (size_t)KW * 2 * MR * sizeof(float));
    const size_t r = (size_t)GW * MT * 2 * REGS * 64 * 4;
    return (x > r ? x : r) + 256;
}

template <int BITS, bool G64, int MR, int KW>
int launch_gemm(const GemmArgs &a, hipStream_t stream)
{
    auto kern = hlq_gemm_kernel<BITS, G64, MR, KW>;
    const size_t lds = gemm_lds_bytes<MR, KW>();
    static bool big_lds_done[64] = {};        // per template instance
    if (!allow_big_lds((const void *)kern, lds, (int)lds, big_lds_done)) return ELUTQ_ERR_HIP;
    const int cbw = GW / KW, nsb = (a.ncb + cbw - 1) / cbw;
    hipLaunchKernelGGL(kern, dim3(nsb * a.ksplit), dim3(GEMM_THREADS), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64, int MR>
int launch_gemm_kw(const GemmArgs &a, int kw, hipStream_t stream)
{
    switch (kw) {
    case 2: return launch_gemm<BITS, G64, MR, 2>(a, stream);
    case 4: return launch_gemm<BITS, G64, MR, 4>(a, stream);
    }
    return ELUTQ_ERR_TUNING;
}

template <int BITS, bool G64>
int launch_gemm_mt(const GemmArgs &a, int kw, hipStream_t stream)
{
    if (a.M <= 16) return launch_gemm_kw<BITS, G64, 16>(a, kw, stream);
    return a.M <= 32 ? launch_gemm_kw<BITS, G64, 32>(a, kw, stream) : launch_gemm_kw<BITS, G64, 64>(a, kw, stream);
}

int dispatch_gemm(const GemmArgs &a, int bits, bool g64, int kw, hipStream_t stream)
{
    switch (bits) {
    case 1: return g64 ? launch_gemm_mt<1, true>(a, kw, stream) : launch_gemm_mt<1, false>(a, kw, stream);
    case 2: return g64 ? launch_gemm_mt<2, true>(a, kw, stream) : launch_gemm_mt<2, false>(a, kw, stream);
    case 3: return g64 ? launch_gemm_mt<3, true>(a, kw, stream) : launch_gemm_mt<3, false>(a, kw, stream);
    case 4: return g64 ? launch_gemm_mt<4, true>(a, kw, stream) : launch_gemm_mt<4, false>(a, kw, stream);
    }
    return ELUTQ_ERR_BITS;
}

}  // namespace

extern "C" {

#ifdef HLQ_TIMING
int elutq_debug_set_gemm_stamps(void *d_buf)
{
    return hipMemcpyToSymbol(HIP_SYMBOL(g_gemm_stamps), &d_buf, sizeof(d_buf)) == hipSuccess ? 0 : -1;
}
#endif

// y[M][N] = x[M][K] W^T + bias.  M == 1 goes to the LUT GEMV; larger M to the MFMA kernel in
// chunks of up to 64 rows.
int elutq_hlq_gemm_f16_tuned(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                             const void *d_x, void *d_y, int M, int K, int N, int bits, int group, void *d_workspace,
                             size_t workspace_bytes, void *stream, int kparts, int ksplit)
{
    if (M < 1) return ELUTQ_ERR_SHAPE;
    if (M == 1)
        return elutq_hlq_gemv_f16(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                                  workspace_bytes, stream);
    for (int m0 = 0; m0 < M; m0 += HLQ_GEMM_MAX_M) {
        const int mc = M - m0 < HLQ_GEMM_MAX_M ? M - m0 : HLQ_GEMM_MAX_M;
        int rc = hlq_gemm_chunk_with_extra(d_planes, d_scales, d_zeros, d_bias, (const uint16_t *)d_x + (size_t)m0 * K,
                                           (uint16_t *)d_y + (size_t)m0 * N, mc, K, N, bits, group, d_workspace,
                                           workspace_bytes, stream, kparts, ksplit, nullptr);
        if (rc != ELUTQ_OK) return rc;
    }
    return ELUTQ_OK;
}

}  // extern "C"

// One launch of the MFMA kernel: 1 <= M <= 64 rows, with an optional fp32 [M][N] term added to
// every output before it is rounded to fp16 (the block-sparse extra plane of a use_sparse layer).
int hlq_gemm_chunk_with_extra(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_x, void *d_y, int M, int K, int N, int bits, int group, void *d_workspace,
                              size_t workspace_bytes, void *stream, int kparts, int ksplit, const float *d_extra)
{
    if (M < 1 || M > HLQ_GEMM_MAX_M) return ELUTQ_ERR_SHAPE;
    if (bits < 1 || bits > 4) return ELUTQ_ERR_BITS;
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (K < HLQ_UNIT || N < 1 || K % HLQ_UNIT != 0 || K % group != 0) return ELUTQ_ERR_SHAPE;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    if (kparts != 0 && kparts != 2 && kparts != 4) return ELUTQ_ERR_TUNING;
    if (ksplit < 0 || ksplit > K / HLQ_UNIT) return ELUTQ_ERR_TUNING;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    int kw = kparts, ks = ksplit, ups;
    hlq_gemm_shape(g, kw, ks, ups);

    GemmArgs a;
    a.planes = (const uint4 *)d_planes;
    a.scales = (const uint32_t *)d_scales;
    a.zeros = (const uint32_t *)d_zeros;
    a.bias = (const uint16_t *)d_bias;
    a.x = (const uint16_t *)d_x;
    a.y = (uint16_t *)d_y;
    a.extra = d_extra;
    a.M = M; a.N = N; a.K = K; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb;
    a.ksplit = ks; a.ups = ups;
    a.partial = nullptr; a.counters = nullptr;
    if (ks > 1) {
        const int mpad = M <= 32 ? 32 : 64;
        const int cbw = GW / kw, nsb = (g.ncb + cbw - 1) / cbw;
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)nsb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ks * mpad * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        a.counters = (unsigned *)d_workspace;
        a.partial = (float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
    }
    return dispatch_gemm(a, bits, group == 64, kw, (hipStream_t)stream);
}

extern "C" {

int elutq_hlq_gemm_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                       const void *d_x, void *d_y, int M, int K, int N, int bits, int group, void *d_workspace,
                       size_t workspace_bytes, void *stream)
{
    return elutq_hlq_gemm_f16_tuned(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, M, K, N, bits, group, d_workspace,
                                    workspace_bytes, stream, 0, 0);
}

}  // extern "C"

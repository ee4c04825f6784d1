// Small-batch HLQ GEMM for gfx950 (MI355X): y[M][N] = x[M][K] W^T + bias, 2 <= M <= 64 per
// launch, replacing MultiThread_arm_gemm_w_lowbit_activation_fp_impl
// (C++/ops/src/arm/arm_gemm.cpp:362-387), which re-runs the GEMV once per row.
//
// With M rows the contraction is dense enough for the matrix cores, bit-serially:
//
//   y[m][n] = sum_g ( z[n,g] * (sum_{k in g} x[m][k])  +  sum_b s[b,n,g] * (sum_{k in g} x[m][k] * B_b[n][k]) )
//
// The inner sum over one group and one plane is a chain of v_mfma_f32_32x32x16_f16 (up to 16 rows:
// v_mfma_f32_16x16x32_f16) whose B operand is the plane itself as fp16 zeros and ones.  That operand is not computed: every byte of a plane dword (8 k of
// one column) indexes a 256-row table in LDS whose row v holds the eight fp16 values of v's bits, so one
// address instruction and one ds_read_b128 deliver the operand of one MFMA.  Every product is x or 0, the
// chain accumulates in fp32 from zero, and its result is scaled once by the fp32 value of the group's
// fp16 scale -- nothing else is rounded before the final fp16 store.  The zero term uses per-row sums of
// x over 64-k halves, taken while the activations are staged in LDS as A operand.
//
// A workgroup is one column block (64 columns) x one K slice; its eight waves take the units of the slice
// in turn (wave w: units w, w + 8, ...).  Every wave stages the activations of its own unit in
// its own LDS region, so the waves never wait for each other until the final sum: while one wave of a SIMD
// stages, the other one keeps the matrix core busy.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef const half8 __attribute__((address_space(3))) *lds_half8_ptr;

constexpr int GW = HLQ_GEMM_WAVES;             // waves per workgroup = K parts
constexpr int WS_COUNTER_BYTES = HLQ_WS_COUNTER_BYTES;
#ifndef HLQ_GEMM_LA
#define HLQ_GEMM_LA 2                          // MFMA steps between an operand read and its use
#endif

struct GemmArgs {
    const uint4 *planes;
    const uint32_t *scales;
    const uint32_t *zeros;
    const uint16_t *bias;
    const uint16_t *x;      // fp16 [M][K]
    uint16_t *y;            // fp16 [M][N]
    const float *extra;     // fp32 [M][N] added to the output before it is rounded, or null
    float *partial;         // [ksplit][mpad][ncb*64]
    unsigned *counters;     // one per column block
    int M, N, K, U, NT, ncb;
    int ksplit, ups;        // K slices per column block, units per slice
    int mpad;               // rows of `partial`: 32 or 64
};

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Staging of x[0 .. MR, k0 .. k0 + KS) by one wave into its LDS region, rows in their natural k order:
// the 16 bytes at k = 8t are the A operand of the MFMA step whose B operand comes from plane byte t.
// KS = 128 (a whole unit) for up to 32 rows, 64 (half a unit at a time: `half` = 0, 1) for 64 rows, so that
// a round always fits 32 registers per lane and 9 KiB of LDS per wave.  One task = one 16-byte slot of one
// row; consecutive lanes write consecutive slots, so the LDS stores are conflict-free.  xs[half * MR + m]
// receives the fp32 sum of x[m] over 64-k half `half` of the unit (eight consecutive lanes).
template <int MR>
struct StageRegs {
    static constexpr int KS = MR <= 32 ? HLQ_UNIT : HLQ_UNIT / 2;    // k per round
    static constexpr int SLOTS = KS / 8;                             // 16-byte slots per row
    static constexpr int TPT = MR * SLOTS / 64;                      // tasks per lane
    static constexpr int ROW_BYTES = KS * 2 + 16;                    // padded row: conflict-free b128 reads
    uint4 v[TPT];
};

template <int MR>
__device__ __forceinline__ void stage_load(StageRegs<MR> &r, const GemmArgs &a, int u, int half, int lane)
{
    using S = StageRegs<MR>;
    // The lane number passes through an empty statement so that the offsets below are recomputed for
    // every round (two instructions per task) instead of being kept in registers for the whole kernel.
    asm volatile("" : "+v"(lane));
    const uint32_t row_bytes = (uint32_t)a.K * 2;
    // where K ends half way through the last unit, the slots of the absent half read the row's last slot and count as zeros
    const uint32_t kcol = (uint32_t)u * HLQ_UNIT + half * S::KS + (lane & (S::SLOTS - 1)) * 8;
    const bool absent = kcol >= (uint32_t)a.K;
    const uint32_t col_off = (absent ? (uint32_t)a.K - 8u : kcol) * 2;
    const uint32_t last = (uint32_t)(a.M - 1) * row_bytes + col_off;         // rows past M read row M - 1 again
    uint32_t off = (uint32_t)(lane / S::SLOTS) * row_bytes + col_off;
#pragma unroll
    for (int t = 0; t < S::TPT; t++) {
        r.v[t] = *(const uint4 *)((const unsigned char *)a.x + (off < last ? off : last));
        off += (64 / S::SLOTS) * row_bytes;
        asm volatile("" : "+v"(off));            // one add per task: keeps the compiler from re-deriving every offset with a multiply
    }
    if (absent) {
#pragma unroll
        for (int t = 0; t < S::TPT; t++) r.v[t] = make_uint4(0u, 0u, 0u, 0u);
    }
}

template <int MR>
__device__ __forceinline__ void stage_store(const StageRegs<MR> &r, unsigned char *xw, float *xs, int half, int lane)
{
    using S = StageRegs<MR>;
    const half2v ones = {(_Float16)1.f, (_Float16)1.f};
    float sum[S::TPT];
    // the reduction steps of all tasks side by side: no instruction waits for the one just before it
#pragma unroll
    for (int t = 0; t < S::TPT; t++) {
        sum[t] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.v[t].x), ones, 0.f, false);
        sum[t] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.v[t].y), ones, sum[t], false);
    }
#pragma unroll
    for (int t = 0; t < S::TPT; t++) {
        sum[t] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.v[t].z), ones, sum[t], false);
        sum[t] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, r.v[t].w), ones, sum[t], false);
    }
#pragma unroll
    for (int t = 0; t < S::TPT; t++) sum[t] += dpp_f<0xB1>(sum[t]);      // the eight slots of a 64-k half: quad,
#pragma unroll
    for (int t = 0; t < S::TPT; t++) sum[t] += dpp_f<0x4E>(sum[t]);      // quad pair,
#pragma unroll
    for (int t = 0; t < S::TPT; t++) sum[t] += dpp_f<0x141>(sum[t]);     // both quad pairs
    const int m0 = lane / S::SLOTS, o = lane % S::SLOTS;
#pragma unroll
    for (int t = 0; t < S::TPT; t++) {
        const int m = m0 + (64 / S::SLOTS) * t;
        if ((o & 7) == 0) xs[((o >> 3) + half) * MR + m] = sum[t];
        *(uint4 *)(xw + m * S::ROW_BYTES + o * 16) = r.v[t];
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
__device__ __forceinline__ void load_unit(UnitData<BITS> &d, const GemmArgs &a, int cb, int u, int lane)
{
    const size_t meta = (size_t)cb * a.NT + (G64 ? u : (u >> 1));
#pragma unroll
    for (int b = 0; b < BITS; b++) {
        d.w[b] = a.planes[(((size_t)cb * a.U + u) * BITS + b) * HLQ_CB + lane];
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

// The wave as four rows of 16 lanes.  transpose_rows: out[j] in lane row r = in[r] of lane row j, same position in
// the row (a 4 x 4 transposition between register index and lane row in four swaps).  bcast_rows: out[j] in every
// lane row = v of lane row j.
__device__ __forceinline__ void transpose_rows(const uint32_t (&in)[4], uint32_t (&out)[4])
{
    const auto p02 = __builtin_amdgcn_permlane32_swap(in[0], in[2], false, false);     // [0] = in0.r0 in0.r1 in2.r0 in2.r1
    const auto p13 = __builtin_amdgcn_permlane32_swap(in[1], in[3], false, false);     // [1] = the same of rows 2, 3
    const auto lo = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
    const auto hi = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
    out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}

__device__ __forceinline__ void bcast_rows(uint32_t v, uint32_t (&out)[4])
{
    const auto q = __builtin_amdgcn_permlane32_swap(v, v, false, false);               // [0] = r0 r1 r0 r1, [1] = r2 r3 r2 r3
    const auto lo = __builtin_amdgcn_permlane16_swap(q[0], q[0], false, false);
    const auto hi = __builtin_amdgcn_permlane16_swap(q[1], q[1], false, false);
    out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}

// out[j] in lane rows 0, 1 = a of lane row j, in lane rows 2, 3 = b of lane row j.
__device__ __forceinline__ void bcast_row_pairs(uint32_t a, uint32_t b, uint32_t (&out)[4])
{
    const auto q = __builtin_amdgcn_permlane32_swap(a, b, false, false);               // [0] = a.r0 a.r1 b.r0 b.r1, [1] = a.r2 a.r3 b.r2 b.r3
    const auto lo = __builtin_amdgcn_permlane16_swap(q[0], q[0], false, false);
    const auto hi = __builtin_amdgcn_permlane16_swap(q[1], q[1], false, false);
    out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}

__device__ __forceinline__ float h2f(uint32_t v, bool hi)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? v >> 16 : v & 0xffffu));
}

// Byte offset of the operand-table row for byte S of w.  The table holds TREP = 16 copies of every row
// side by side (row stride 256 bytes) and a lane reads copy lane % 16 (`lanepart` = 16 * that): the lanes
// of one ds_read_b128 then fall on different banks whatever their bytes are.  One v_perm_b32 puts byte S
// into bits 8..15 above the lane part.  A compiler builtin on purpose: the compiler knows which registers
// a pending MFMA is still going to write and keeps other writes away from them for long enough, which it
// does not do for instructions inside inline assembly.
template <int TREP>
__device__ __forceinline__ uint32_t row_addr(uint32_t w, int S, uint32_t lanepart)
{
    if (TREP == 16) return __builtin_amdgcn_perm(w, lanepart, 0x0c0c0000u | ((4u + S) << 8));
    return ((w >> (8 * S)) & 0xffu) * (16u * TREP) + lanepart;
}

// Emits no instruction.  `chain` is the 16-register result of a chain of MFMAs of which only some
// registers are read, `first_use` a value computed from one of them.  Tying the two together keeps all 16
// registers allocated to the chain until that value exists, i.e. until the last MFMA has written them;
// otherwise the registers nobody reads are free from the moment that MFMA is issued and could be handed
// to another value while the MFMA is still going to write them.
// Operand-table row at LDS address `addr`.  The kernel has no static LDS, so its dynamic LDS -- the table
// first -- starts at address 0 and the offset formed by row_addr is the address itself; going through the
// generic `smem + offset` form would cost one more vector instruction per operand (an add of the base).
__device__ __forceinline__ half8 table_row(uint32_t addr)
{
    return *(lds_half8_ptr)(uintptr_t)addr;
}

__device__ __forceinline__ float hold_until_read(float first_use, const float16v &chain)
{
    asm volatile("" : "+v"(first_use) : "v"(chain));
    return first_use;
}

// LDS of a workgroup: the operand table, then one region per wave (a staged unit, or half unit, of MR rows
// and the row sums of both halves); the cross-wave reduction reuses the space after the last unit.
template <int MR>
struct GemmLds {
    static constexpr int NW = GW;                                    // waves
    static constexpr int TREP = 16;                                  // copies of the operand table
    static constexpr int ROW_BYTES = StageRegs<MR>::ROW_BYTES;
    static constexpr int MT = (MR + 31) / 32;                        // 32-row MFMA tiles
    static constexpr int REGS = MR == 16 ? 8 : 16;
    static constexpr int TAB_BYTES = 256 * 16 * TREP;
    static constexpr int WAVE_BYTES = MR * ROW_BYTES + 2 * MR * 4;
    static constexpr int RED_BYTES = NW * MT * 2 * REGS * 64 * 4;
    static constexpr int TICKET_OFF = TAB_BYTES + NW * WAVE_BYTES;   // arrival ticket of a K-sliced launch
    static constexpr int BYTES = TICKET_OFF + 16;                    // no static LDS: the table starts at address 0
    static_assert(RED_BYTES <= TICKET_OFF, "the reduction reuses the table and the regions");
    static_assert(WAVE_BYTES % 16 == 0, "aligned regions");
};

// MR = activation rows of the launch rounded up to 16, 32 or 64.  With MR = 16 the MFMA tile is 16 rows x 16
// columns x 32 k (four column tiles per wave, four result registers each); otherwise 32 x 32 x 16.  With MR = 64 every B
// operand serves two MFMAs (rows 0..31 and 32..63) and the activations are staged half a unit at a time.
// grid = column blocks * K slices.
template <int BITS, bool G64, int MR>
__global__ __launch_bounds__(GemmLds<MR>::NW * 64) void hlq_gemm_kernel(const GemmArgs a)
{
    using L = GemmLds<MR>;
    constexpr int REGS = L::REGS, MT = L::MT, NW = L::NW, THREADS = NW * 64, TREP = L::TREP, ROW_BYTES = L::ROW_BYTES;
    constexpr int VALS = MT * 2 * REGS * 64;        // fp32 results per wave
    extern __shared__ __align__(256) unsigned char smem[];
    float *red = (float *)smem;                     // reused after the last unit
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;
    const int cb = blockIdx.x / a.ksplit, slice = blockIdx.x - cb * a.ksplit;
    const int u_begin = slice * a.ups, u_end = min(u_begin + a.ups, a.U);

    // Up to 16 rows: v_mfma_f32_16x16x32_f16 on four 16-column tiles (no idle rows in the matrix core, four result
    // registers per tile).  The 32 k of a step must lie in one quantization group: at G = 128 lane row r takes k
    // quarter r of the unit and step s byte s of it; at G = 64 lane row r takes 16 k of the step's group (k = 64 g +
    // 16 r + 8 s).
    constexpr bool T16 = MR == 16;
    float4v acc4[4];
#pragma unroll
    for (int j = 0; j < 4; j++) acc4[j] = float4v{0.f, 0.f, 0.f, 0.f};
    float16v acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][j][i] = 0.f;

    // The plane data of two of the wave's units is in registers at any time (two alternating sets, so no
    // set is ever copied); the activations of the next unit wait in registers while the wave computes on
    // the staged ones.
    UnitData<BITS> ua, ub;
    StageRegs<MR> xr;
    const int u_first = u_begin + wave;
    if (u_first < u_end) {
        load_unit<BITS, G64>(ua, a, cb, u_first, lane);
        stage_load<MR>(xr, a, u_first, 0, lane);
    }
    if (u_first + NW < u_end) load_unit<BITS, G64>(ub, a, cb, u_first + NW, lane);
    // operand table: row v holds the eight fp16 values (0 or 1) of the bits of v, TREP copies side by side
#pragma unroll
    for (int e = tid; e < 256 * TREP; e += THREADS) {
        const int v = e / TREP;
        uint4 row;
        row.x = ((v & 1) ? 0x3C00u : 0u) | ((v & 2) ? 0x3C000000u : 0u);
        row.y = ((v & 4) ? 0x3C00u : 0u) | ((v & 8) ? 0x3C000000u : 0u);
        row.z = ((v & 16) ? 0x3C00u : 0u) | ((v & 32) ? 0x3C000000u : 0u);
        row.w = ((v & 64) ? 0x3C00u : 0u) | ((v & 128) ? 0x3C000000u : 0u);
        *(uint4 *)(smem + e * 16) = row;
    }
    __syncthreads();
    const uint32_t lanepart = (uint32_t)(lane % TREP) * 16u;
    unsigned char *xw = smem + L::TAB_BYTES + wave * L::WAVE_BYTES;
    float *xs = (float *)(xw + MR * ROW_BYTES);
    const unsigned char *arow = T16 ? xw + (lane & 15) * ROW_BYTES + (lane >> 4) * (G64 ? 32 : 64)
                                    : xw + col * ROW_BYTES + h * 64;

    // One unit: stage its activations (LDS operations of one wave execute in order, so the wave reads
    // what it has just written without a barrier), refill `cur` with the unit two turns ahead, compute.
    auto unit = [&](UnitData<BITS> &cur, int u) __attribute__((always_inline)) {
        if constexpr (MT == 1) {
            stage_store<MR>(xr, xw, xs, 0, lane);
            if (u + NW < u_end) stage_load<MR>(xr, a, u + NW, 0, lane);
        }
        if constexpr (T16) {
            // Lane (c, r) of tile j works on column 16 j + c of the block: the scale / zero dwords of that column in
            // every lane row, and the plane bits of its k (rotation undone).  G = 128: plane dword r, bit i = k 32 r + i,
            // step s = byte s.  G = 64: per group g plane dword 2 g + r / 2 (bit i = k 64 g + 32 (r / 2) + i), step s =
            // byte 2 (r % 2) + s -- the byte's place in the dword differs between lanes, so the v_perm selector is a
            // register.
            constexpr int NG = G64 ? 2 : 1, NQ = G64 ? 2 : 4;          // groups per unit, steps per chain
            uint32_t sc4[BITS][4], zz4[4], tq[BITS][NG][4];
#pragma unroll
            for (int b = 0; b < BITS; b++) {
                bcast_rows(cur.sc[b], sc4[b]);
                if constexpr (G64) {
                    bcast_row_pairs(cur.w[b].x, cur.w[b].y, tq[b][0]);
                    bcast_row_pairs(cur.w[b].z, cur.w[b].w, tq[b][1]);
                } else {
                    const uint32_t dw[4] = {cur.w[b].x, cur.w[b].y, cur.w[b].z, cur.w[b].w};
                    transpose_rows(dw, tq[b][0]);
                }
#pragma unroll
                for (int g = 0; g < NG; g++)
#pragma unroll
                    for (int j = 0; j < 4; j++) tq[b][g][j] = __builtin_amdgcn_alignbit(tq[b][g][j], tq[b][g][j], HLQ_ROT);
            }
            bcast_rows(cur.zz, zz4);
            if (u + 2 * NW < u_end) load_unit<BITS, G64>(cur, a, cb, u + 2 * NW, lane);
            // the A operands of the unit's four (group, step) pairs serve every plane
            half8 aop[4];
#pragma unroll
            for (int q = 0; q < 4; q++) aop[q] = *(const half8 *)(arow + (G64 ? (q >> 1) * 128 + (q & 1) * 16 : q * 16));
            const uint32_t sel0 = 0x0c0c0000u | ((4u + 2u * ((uint32_t)(lane >> 4) & 1u)) << 8);      // G = 64: byte 2 (r % 2) + s
            constexpr int LA = HLQ_GEMM_LA, RING = LA + 1, NSTEP = 4 * BITS;
            half8 bop[RING][4];
            float4v tmp[4];
            auto issue = [&](int t) __attribute__((always_inline)) {
                const int g = t / (BITS * NQ), b = (t / NQ) % BITS, sq = t % NQ;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if constexpr (G64) bop[t % RING][j] = table_row(__builtin_amdgcn_perm(tq[b][g][j], lanepart, sel0 + ((uint32_t)sq << 8)));
                    else bop[t % RING][j] = table_row(row_addr<TREP>(tq[b][0][j], sq, lanepart));
                }
            };
#pragma unroll
            for (int t = 0; t < LA && t < NSTEP; t++) issue(t);
#pragma unroll
            for (int t = 0; t < NSTEP; t++) {
                const int g = t / (BITS * NQ), b = (t / NQ) % BITS, sq = t % NQ;
                if (t + LA < NSTEP) issue(t + LA);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    tmp[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop[G64 ? 2 * g + sq : sq], bop[t % RING][j],
                                                                    sq == 0 ? float4v{0.f, 0.f, 0.f, 0.f} : tmp[j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (sq == NQ - 1) {
                    const bool hi = G64 ? g == 1 : (u & 1) != 0;      // fp16 of the meta dwords this group belongs to
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const float sf = h2f(sc4[b][j], hi);
#pragma unroll
                        for (int i = 0; i < 4; i++) acc4[j][i] = fmaf(sf, tmp[j][i], acc4[j][i]);
                    }
                    if (b == BITS - 1) {
                        // zero term of the group: z[n, g] * sum_{k in g} x[m, k]; C rows of register i: 4 * (lane / 16) + i
                        float4 sx = *(const float4 *)(xs + (G64 ? g : 1) * MR + 4 * (lane >> 4));
                        if (!G64) {
                            const float4 s0 = *(const float4 *)(xs + 4 * (lane >> 4));
                            sx.x += s0.x; sx.y += s0.y; sx.z += s0.z; sx.w += s0.w;
                        }
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float zf = h2f(zz4[j], hi);
                            acc4[j][0] = fmaf(zf, sx.x, acc4[j][0]);
                            acc4[j][1] = fmaf(zf, sx.y, acc4[j][1]);
                            acc4[j][2] = fmaf(zf, sx.z, acc4[j][2]);
                            acc4[j][3] = fmaf(zf, sx.w, acc4[j][3]);
                        }
                    }
                }
            }
            return;
        }
        // Lane (col, h) of tile j works on column 32j + col of the block: bring that column's
        // scale / zero dwords and its plane dwords (k half h of each 64-k pair, rotation undone:
        // bit i of tw[b][j][pr] is k = 64 pr + 32 h + i) into the lane.
        uint32_t scj[BITS][2], zzj[2], tw[BITS][2][2];
#pragma unroll
        for (int b = 0; b < BITS; b++) {
            split_tiles(cur.sc[b], cur.sc[b], scj[b][0], scj[b][1]);
            split_tiles(cur.w[b].x, cur.w[b].y, tw[b][0][0], tw[b][1][0]);
            split_tiles(cur.w[b].z, cur.w[b].w, tw[b][0][1], tw[b][1][1]);
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int pr = 0; pr < 2; pr++) tw[b][j][pr] = __builtin_amdgcn_alignbit(tw[b][j][pr], tw[b][j][pr], HLQ_ROT);
        }
        split_tiles(cur.zz, cur.zz, zzj[0], zzj[1]);
        if (u + 2 * NW < u_end) load_unit<BITS, G64>(cur, a, cb, u + 2 * NW, lane);
        // zero term of group g: z[n, g] * sum_{k in g} x[m, k]; C rows of register i: 8*(i/4) + 4h + i%4
        auto zero_term = [&](int g, bool hi) __attribute__((always_inline)) {
            const float zf[2] = {h2f(zzj[0], hi), h2f(zzj[1], hi)};
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int i4 = 0; i4 < REGS / 4; i4++) {
                    const int mr = mt * 32 + 8 * i4 + 4 * h;
                    float4 sx = *(const float4 *)(xs + (G64 ? g : 1) * MR + mr);
                    if (!G64) {
                        const float4 s0 = *(const float4 *)(xs + mr);
                        sx.x += s0.x; sx.y += s0.y; sx.z += s0.z; sx.w += s0.w;
                    }
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        acc[mt][j][4 * i4 + 0] = fmaf(zf[j], sx.x, acc[mt][j][4 * i4 + 0]);
                        acc[mt][j][4 * i4 + 1] = fmaf(zf[j], sx.y, acc[mt][j][4 * i4 + 1]);
                        acc[mt][j][4 * i4 + 2] = fmaf(zf[j], sx.z, acc[mt][j][4 * i4 + 2]);
                        acc[mt][j][4 * i4 + 3] = fmaf(zf[j], sx.w, acc[mt][j][4 * i4 + 3]);
                    }
                }
        };
        constexpr int LA = HLQ_GEMM_LA, RING = LA + 1;
        if constexpr (MT == 1) {
            // The unit is a list of MFMA steps: for every group of the unit, for every plane, the NQ 16-k
            // steps of the group.  Step t uses the A operand of its 16 k and one B operand per column
            // tile; they are read from LDS LA steps before their use, into rotating register sets, so that
            // the reads are not waited for.  Every (group, plane, column tile) is a chain that starts from
            // zero; its result is scaled by the group's scale and added to the accumulator (16 or 8
            // multiply-adds per chain).
            constexpr int NG = G64 ? 2 : 1, NQ = G64 ? 4 : 8, NSTEP = NG * BITS * NQ;
            half8 aopr[RING], bopr[RING][2];
            float16v tmp[2];
            auto issue = [&](int t) __attribute__((always_inline)) {
                const int g = t / (BITS * NQ), b = (t / NQ) % BITS, q = t % NQ;
                const int pr = G64 ? g : q / 4, sq = q % 4;
                aopr[t % RING] = *(const half8 *)(arow + pr * 128 + sq * 16);
#pragma unroll
                for (int j = 0; j < 2; j++) bopr[t % RING][j] = table_row(row_addr<TREP>(tw[b][j][pr], sq, lanepart));
            };
#pragma unroll
            for (int t = 0; t < LA && t < NSTEP; t++) issue(t);
#pragma unroll
            for (int t = 0; t < NSTEP; t++) {
                const int g = t / (BITS * NQ), b = (t / NQ) % BITS, q = t % NQ;
                if (t + LA < NSTEP) issue(t + LA);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    if (q == 0) {
                        float16v zero;
#pragma unroll
                        for (int i = 0; i < 16; i++) zero[i] = 0.f;
                        tmp[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aopr[t % RING], bopr[t % RING][j], zero, 0, 0, 0);
                    } else {
                        tmp[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aopr[t % RING], bopr[t % RING][j], tmp[j], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (q == NQ - 1) {
                    const bool hi = G64 ? g == 1 : (u & 1) != 0;      // fp16 of the meta dwords this group belongs to
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const float sf = h2f(scj[b][j], hi);
#pragma unroll
                        for (int i = 0; i < REGS; i++) acc[0][j][i] = fmaf(sf, tmp[j][i], acc[0][j][i]);
                        if (REGS < 16) acc[0][j][REGS - 1] = hold_until_read(acc[0][j][REGS - 1], tmp[j]);
                    }
                    if (b == BITS - 1) zero_term(g, hi);
                }
            }
        } else {
            // Two row tiles: a B operand serves two MFMAs, which pays for scaling the operand itself (four
            // packed fp16 multiplications, exact: the operand is 0 or 1) and accumulating straight into the
            // result, with neither chain registers nor multiply-adds afterwards.  The unit is worked on half
            // by half (one 64-k pair of every plane dword at a time); a step is (16 k, plane): the two A
            // operands of 16 k are read once for all planes.
            constexpr int NSTEP = 4 * BITS;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                stage_store<MR>(xr, xw, xs, half, lane);
                if (half == 0) stage_load<MR>(xr, a, u, 1, lane);
                else if (u + NW < u_end) stage_load<MR>(xr, a, u + NW, 0, lane);
                const bool hi = G64 ? half == 1 : (u & 1) != 0;
                half2v s2[BITS][2];
#pragma unroll
                for (int b = 0; b < BITS; b++)
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const uint32_t sc = scj[b][j];
                        s2[b][j] = __builtin_bit_cast(half2v, hi ? __builtin_amdgcn_perm(sc, sc, 0x03020302u)
                                                                 : __builtin_amdgcn_perm(sc, sc, 0x01000100u));
                    }
                half8 aopr[3][MT], bopr[RING][2];
                auto issue = [&](int t) __attribute__((always_inline)) {
                    const int q = t / BITS, b = t % BITS;
                    if (b == 0) {
#pragma unroll
                        for (int mt = 0; mt < MT; mt++) aopr[q % 3][mt] = *(const half8 *)(arow + mt * 32 * ROW_BYTES + q * 16);
                    }
#pragma unroll
                    for (int j = 0; j < 2; j++) bopr[t % RING][j] = table_row(row_addr<TREP>(tw[b][j][half], q, lanepart));
                };
#pragma unroll
                for (int t = 0; t < LA && t < NSTEP; t++) issue(t);
#pragma unroll
                for (int t = 0; t < NSTEP; t++) {
                    const int q = t / BITS, b = t % BITS;
                    if (t + LA < NSTEP) issue(t + LA);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        half8 bs;
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const half2v v = {bopr[t % RING][j][2 * i], bopr[t % RING][j][2 * i + 1]};
                            const half2v p = v * s2[b][j];
                            bs[2 * i] = p[0];
                            bs[2 * i + 1] = p[1];
                        }
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
                            acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aopr[q % 3][mt], bs, acc[mt][j], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (G64 || half == 1) zero_term(half, hi);
            }
        }
    };
    for (int u = u_first; u < u_end; u += 2 * NW) {
        unit(ua, u);
        if (u + NW < u_end) unit(ub, u + NW);
    }

    // Sum of the K parts through LDS: red[wave][tile = mt*2+j][reg][lane].
    __syncthreads();
    if constexpr (T16) {
        static_assert(VALS == 4 * 4 * 64, "four tiles of four registers");
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[((wave * 4 + j) * 4 + i) * 64 + lane] = acc4[j][i];
    } else {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < REGS; i++) red[((wave * MT * 2 + mt * 2 + j) * REGS + i) * 64 + lane] = acc[mt][j][i];
    }
    __syncthreads();

    constexpr int NV = VALS / THREADS;               // results per thread
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    // value v = (tile, reg, lane); C layout of the 32x32 MFMA: column = lane % 32,
    // row = 8 * (reg / 4) + 4 * (lane / 32) + reg % 4.
    // (16x16 tiles: column = lane % 16, row = 4 * (lane / 16) + reg.)
    auto decode = [&](int v, int &m, int &n) {
        if constexpr (T16) {
            const int ln = v & 63, reg = (v >> 6) & 3, tile = v >> 8;
            m = 4 * (ln >> 4) + reg;
            n = cb * HLQ_CB + tile * 16 + (ln & 15);
            return;
        }
        const int ln = v & 63, reg = (v >> 6) % REGS, tile = v / (64 * REGS);
        m = (tile >> 1) * 32 + 8 * (reg >> 2) + 4 * (ln >> 5) + (reg & 3);
        n = cb * HLQ_CB + (tile & 1) * 32 + (ln & 31);
    };
    float outv[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int v = tid + it * THREADS;
        float s = 0.f;
#pragma unroll
        for (int p = 0; p < NW; p++) s += red[p * VALS + v];
        outv[it] = s;
    }
    if (a.ksplit == 1) {
#pragma unroll
        for (int it = 0; it < NV; it++) {
            int m, n;
            decode(tid + it * THREADS, m, n);
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
        decode(tid + it * THREADS, m, n);
        __hip_atomic_store(&a.partial[((size_t)slice * a.mpad + m) * npad + n], outv[it], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    unsigned *s_ticket = (unsigned *)(smem + L::TICKET_OFF);
    unsigned *counter = a.counters + cb;
    if (tid == 0) *s_ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*s_ticket != (unsigned)a.ksplit - 1u) return;
    // a thread's loads for QB slices are in flight together; summed in slice order
    constexpr int QB = NV <= 8 ? 4 : 2;
    float sum[NV];
    size_t off[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * THREADS, m, n);
        off[it] = (size_t)m * npad + n;
        sum[it] = 0.f;
    }
    for (int s0 = 0; s0 < a.ksplit; s0 += QB) {
        float v[QB][NV];
#pragma unroll
        for (int q = 0; q < QB; q++) {
            const int sl = min(s0 + q, a.ksplit - 1);
#pragma unroll
            for (int it = 0; it < NV; it++)
                v[q][it] = __hip_atomic_load(&a.partial[(size_t)sl * a.mpad * npad + off[it]], __ATOMIC_RELAXED,
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
        decode(tid + it * THREADS, m, n);
        if (m < a.M && n < a.N) {
            float s = sum[it];
            if (a.bias) s += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            if (a.extra) s += a.extra[(size_t)m * a.N + n];
            a.y[(size_t)m * a.N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
        }
    }
    if (tid == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

template <int BITS, bool G64, int MR>
int launch_gemm(const GemmArgs &a, hipStream_t stream)
{
    auto kern = hlq_gemm_kernel<BITS, G64, MR>;
    const size_t lds = GemmLds<MR>::BYTES;
    static_assert(GemmLds<MR>::BYTES <= HLQ_MAX_LDS, "LDS of one workgroup");
    static bool big_lds_done[64] = {};        // per template instance
    if (!allow_big_lds((const void *)kern, lds, (int)lds, big_lds_done)) return ELUTQ_ERR_HIP;
    // table_row() takes LDS offsets for addresses: true only while the kernel has no static LDS in front of
    // its dynamic LDS
    static int static_lds = -1;
    if (static_lds < 0) {
        hipFuncAttributes attr;
        if (hipFuncGetAttributes(&attr, (const void *)kern) != hipSuccess) return ELUTQ_ERR_HIP;
        static_lds = (int)attr.sharedSizeBytes;
    }
    if (static_lds != 0) return ELUTQ_ERR_HIP;
    hipLaunchKernelGGL(kern, dim3(a.ncb * a.ksplit), dim3(GemmLds<MR>::NW * 64), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64>
int launch_gemm_rows(const GemmArgs &a, hipStream_t stream)
{
    if (a.M <= 16) return launch_gemm<BITS, G64, 16>(a, stream);
    return a.M <= 32 ? launch_gemm<BITS, G64, 32>(a, stream) : launch_gemm<BITS, G64, 64>(a, stream);
}

int dispatch_gemm(const GemmArgs &a, int bits, bool g64, hipStream_t stream)
{
    switch (bits) {
    case 1: return g64 ? launch_gemm_rows<1, true>(a, stream) : launch_gemm_rows<1, false>(a, stream);
    case 2: return g64 ? launch_gemm_rows<2, true>(a, stream) : launch_gemm_rows<2, false>(a, stream);
    case 3: return g64 ? launch_gemm_rows<3, true>(a, stream) : launch_gemm_rows<3, false>(a, stream);
    case 4: return g64 ? launch_gemm_rows<4, true>(a, stream) : launch_gemm_rows<4, false>(a, stream);
    }
    return ELUTQ_ERR_BITS;
}

}  // namespace

extern "C" {

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
    if (N < 1 || !hlq_k_ok(K, group)) return ELUTQ_ERR_SHAPE;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    if (kparts != 0 && kparts != HLQ_GEMM_WAVES) return ELUTQ_ERR_TUNING;
    if (ksplit < 0 || ksplit > (K + HLQ_UNIT - 1) / HLQ_UNIT) return ELUTQ_ERR_TUNING;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    int ks = ksplit, ups;
    hlq_gemm_shape(g, M, ks, ups);

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
    a.mpad = M <= 32 ? 32 : 64;
    if (ks > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ks * a.mpad * g.ncb * HLQ_CB * sizeof(float))
            return ELUTQ_ERR_WORKSPACE;
        a.counters = (unsigned *)d_workspace;
        a.partial = (float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
    }
    return dispatch_gemm(a, bits, group == 64, (hipStream_t)stream);
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

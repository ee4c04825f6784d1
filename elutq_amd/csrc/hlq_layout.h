// Device-side layout of a repacked HLQ layer, shared by the host repack and the kernels.
//
// A "unit" is 128 consecutive k of one output column in one bit-plane: 128 bits = one
// dwordx4 per lane.  Output columns are tiled in blocks of 64 (one wavefront, lane =
// column), so a wave-wide dwordx4 load covers one unit of 64 columns = 1 KiB contiguous.
//
//   planes  uint4    [ncb][U][bits][64]        U = ceil(K/128), ncb = ceil(N/64)
//   scales  uint32   [ncb][NT][bits][64]       one dword = fp16 scales of groups 2t, 2t+1
//   zeros   uint32   [ncb][NT][64]             one dword = fp16 zeros  of groups 2t, 2t+1
//
// NT = ceil(NG/2) with NG = K/G groups per column ("task" t = the groups one meta dword
// covers: two units at G = 128, one unit at G = 64).  Columns >= N and the odd group of
// an odd NG are zero-filled.  K is a multiple of the group size and at least 128: at G = 64 it may
// end half way through the last unit (K % 128 == 64, which the reference accepts, arm_gemm.cpp:249);
// the plane bits of that unit's second half are zero like the scales and zero of its absent group, and
// the kernels read the activations of that half as zeros.
//
// Inside a unit, dword d holds k = 32d .. 32d+31 LSB-first (bit i <-> k = 32d + i, the
// byte order of the reference's w_quant.bin read as little-endian dwords), rotated left
// by HLQ_ROT bits.  After the rotation the 4-bit field of chunk c (k = 4c..4c+3) sits at
// bits 4c+2 .. 4c+5, so `byte_j & 0x3C` is 4 * (nibble of chunk 2j) -- a ready-made byte
// offset into a table of 16 int32 entries -- and the same holds for chunk 2j+1 after a
// further rotate right by 4.
#pragma once
#include <stddef.h>
#include <stdint.h>

#define HLQ_CB 64
#define HLQ_UNIT 128
#define HLQ_ROT 2
#define HLQ_NUM_CU 256                 /* MI355X */
#define HLQ_MAX_LDS (160 * 1024)       /* per workgroup on gfx950 */
#define HLQ_WS_COUNTER_BYTES (64 * 1024) /* head of every workspace: one arrival counter per column block */
#define HLQ_GEMM_WAVES 8               /* waves per GEMM workgroup */
#define HLQ_GEMM_MAX_M 64              /* rows per GEMM launch; more rows run in chunks of this many (weights re-streamed) */

// Inline form of a block-sparse extra plane (blocks of 32 output channels x G inputs on the group grid, at most one per
// cell): what a GEMV tile needs to look the blocks up in the activation tables it has built for the dense planes.
//   header   int32 [8]          magic, K, N, group, U, ncb, records, 0
//   cells    int32 [ncb][U]     record of (column block, unit), or -1             at HLQ_SP_HEAD_BYTES
//   records  [records][1280 B]  uint4 [64]: lane n's 128 plane bits of the unit, laid out and rotated like a dense plane's,
//                               zero where n's half of the column block (or, at G = 64, a 64-k half) has no block;
//                               uint32 [64]: fp16 scales of n for the unit's two 64-k halves (0 where there is no block)
//                                                                                   at hlq_sp_recs_offset(ncb, U)
#define HLQ_SP_MAGIC 0x53504c31
#define HLQ_SP_HEAD_BYTES 32
#define HLQ_SP_REC_BYTES 1280
static inline size_t hlq_sp_recs_offset(int ncb, int U)
{
    return ((size_t)HLQ_SP_HEAD_BYTES + (size_t)ncb * U * sizeof(int32_t) + 255) & ~(size_t)255;
}

struct HlqGeo {
    int K, N, bits, group;
    int U;      // units per column
    int NG;     // groups per column
    int NT;     // tasks (meta dwords) per column
    int UPT;    // units per task: 2 at G=128, 1 at G=64
    int ncb;    // column blocks
};

// K >= 128, a multiple of the group size and -- except for half a unit at G = 64 -- of 128.
static inline bool hlq_k_ok(int K, int group)
{
    if (K < HLQ_UNIT || (group != 64 && group != 128)) return false;
    return K % HLQ_UNIT == 0 || (group == 64 && K % HLQ_UNIT == 64);
}

static inline HlqGeo hlq_geo(int K, int N, int bits, int group)
{
    HlqGeo g;
    g.K = K; g.N = N; g.bits = bits; g.group = group;
    g.U = (K + HLQ_UNIT - 1) / HLQ_UNIT;
    g.NG = K / group;
    g.NT = (g.NG + 1) / 2;
    g.UPT = group == 64 ? 1 : 2;
    g.ncb = (N + HLQ_CB - 1) / HLQ_CB;
    return g;
}

static inline size_t hlq_planes_bytes(const HlqGeo &g) { return (size_t)g.ncb * g.U * g.bits * HLQ_CB * 16; }
static inline size_t hlq_scales_bytes(const HlqGeo &g) { return (size_t)g.ncb * g.NT * g.bits * HLQ_CB * 4; }
static inline size_t hlq_zeros_bytes(const HlqGeo &g) { return (size_t)g.ncb * g.NT * HLQ_CB * 4; }

// Launch shape of the small-batch GEMM.  A workgroup is one column block x one K slice; its
// HLQ_GEMM_WAVES waves take the units of the slice in turn.  K is cut
// into ksplit slices of ups units handled by different workgroups that meet through device memory.  That
// meeting costs about as much as two units per wave, so K is cut only where the units saved outweigh it,
// and never into more workgroups than the chip has CUs.
static inline void hlq_gemm_shape(const HlqGeo &g, int M, int &ksplit, int &ups)
{
    const int waves = HLQ_GEMM_WAVES;
    const int turns = (g.U + waves - 1) / waves;        // units per wave over all of K
    int ks = ksplit;
    if (ks <= 0) {
        const int turn_cost = M <= 32 ? 24 : 16, meet_cost = 40;       // tenths of a microsecond
        int most = HLQ_NUM_CU / g.ncb;
        if (most > turns) most = turns;
        ks = 1;
        int best = turns * turn_cost;
        for (int k = 2; k <= most; k++) {
            const int cost = (turns + k - 1) / k * turn_cost + meet_cost;
            if (cost < best) { best = cost; ks = k; }
        }
    }
    if (ks > g.U) ks = g.U;
    if (ks < 1) ks = 1;
    ups = (g.U + ks - 1) / ks;
    ksplit = (g.U + ups - 1) / ups;
}

static inline size_t hlq_gemm_ws_rows(const HlqGeo &g, int M)
{
    int ks = 0, ups;
    hlq_gemm_shape(g, M, ks, ups);
    const int mpad = M <= 32 ? 32 : 64;
    return (size_t)HLQ_WS_COUNTER_BYTES + (ks > 1 ? (size_t)ks * mpad * g.ncb * HLQ_CB * sizeof(float) : 0);
}

// Workspace of a GEMM call with M rows: launches take up to HLQ_GEMM_MAX_M rows, the last one the rest.
static inline size_t hlq_gemm_ws_bytes(const HlqGeo &g, int M)
{
    size_t w = hlq_gemm_ws_rows(g, M > HLQ_GEMM_MAX_M ? HLQ_GEMM_MAX_M : M);
    if (M > HLQ_GEMM_MAX_M) {
        const size_t r = hlq_gemm_ws_rows(g, 32);
        if (r > w) w = r;
    }
    return w;
}

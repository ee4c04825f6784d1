// Index arithmetic of the batch-1 GEMV tile (hlq_gemv.hip: gemv_tile, block_rstd, load_slice_chunk), in
// a form that compiles for the device and for the host: the kernel computes every run boundary, LDS
// offset and staging index with these functions, and a CPU program can replay them for every workgroup
// and wave of a launch and check each access against the sizes the launcher allocates
// (tests/gemv_index_audit.cpp).
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define HLQ_HD __host__ __device__ __forceinline__
#else
#define HLQ_HD inline
#endif

#define HLQ_TBL_BYTES 64                          /* one chunk's table: 16 int32 entries */
#define HLQ_UNIT_LUT_BYTES (32 * HLQ_TBL_BYTES)   /* 32 chunks per unit of 128 k */
#define HLQ_RSTD_SCRATCH 80                       /* floats of reduction scratch of the RMSNorm prologue */
#define HLQ_STAGE_GAP 4                           /* floats between that scratch and the staged activations */
#define HLQ_GEMV_MAX_SLICES_IN 4

// Per-wave LDS region and run length for a slice of `ups` units handled by `waves` waves.
struct HlqWavePlan {
    int spw;        // sub-tasks (unit, plane) per wave: a contiguous run
    int nuw_max;    // units a wave's run can touch
    int wave_lds;   // bytes of a wave's LDS region: tables [nuw_max][32][16] int32, then float2 [2 * nuw_max]
};

HLQ_HD HlqWavePlan hlq_wave_plan(int ups, int bits, int waves)
{
    HlqWavePlan p;
    const int nst = ups * bits;
    p.spw = (nst + waves - 1) / waves;
    if (p.spw > bits && p.spw % bits) p.spw += bits - p.spw % bits;     // whole units per wave when it has several
    if (p.spw == 1) p.nuw_max = 1;
    else if (p.spw % bits == 0) p.nuw_max = p.spw / bits;
    else p.nuw_max = (p.spw + bits - 2) / bits + 1;
    p.wave_lds = (p.nuw_max * (HLQ_UNIT_LUT_BYTES + 2 * 8) + 255) & ~255;
    return p;
}

// Dynamic LDS of a workgroup, in bytes from its start:
//   [waves][wave_lds] tables and half-unit records | [2][waves][64] float cross-wave sums |
//   [HLQ_RSTD_SCRATCH] float | gap | fp16 [K] staged activations (launches that take handed-over slices only)
struct HlqLdsMap {
    uint32_t red, rstd, stage, end_plain;
};

HLQ_HD HlqLdsMap hlq_lds_map(int waves, int wave_lds)
{
    HlqLdsMap m;
    m.red = (uint32_t)waves * (uint32_t)wave_lds;
    m.rstd = m.red + 2u * (uint32_t)waves * 64u * 4u;
    m.stage = m.rstd + (HLQ_RSTD_SCRATCH + HLQ_STAGE_GAP) * 4u;
    m.end_plain = m.stage;                        // == hlq_gemv_lds_bytes(): what a launch without staging allocates
    return m;
}

HLQ_HD size_t hlq_gemv_lds_bytes(int ups, int bits, int waves)
{
    const HlqWavePlan p = hlq_wave_plan(ups, bits, waves);
    return hlq_lds_map(waves, p.wave_lds).end_plain;
}

// The run of one wave inside a workgroup that owns `nst` sub-tasks (units of the slice x planes).
struct HlqWaveRun {
    int s_begin, s_end;   // sub-tasks [s_begin, s_end) of the slice
    int ub;               // first unit (in the slice) the run touches
    int nuw;              // units it touches (0: a wave without a run)
    int s_last;           // clamp target of loads past the run
};

HLQ_HD HlqWaveRun hlq_wave_run(int wave, int spw, int nst, int bits)
{
    HlqWaveRun r;
    const int b = wave * spw;
    r.s_begin = b < nst ? b : nst;
    const int e = r.s_begin + spw;
    r.s_end = e < nst ? e : nst;
    r.ub = r.s_begin / bits;
    r.nuw = r.s_end > r.s_begin ? (r.s_end - 1) / bits - r.ub + 1 : 0;
    r.s_last = r.s_end - 1 > 0 ? r.s_end - 1 : 0;
    return r;
}

// Chunk (4 activations) of the whole K that lane `lane` of a wave builds its first table from, as an index
// into the staged activations uint2 [K/4]: k0 = first k of the run, nchunks = 32 * nuw.  `clamp` = the
// upper clamp a wave without a run needs (its k0 is the end of the slice, for the last slice the end of K).
HLQ_HD int hlq_stage_first_index(size_t k0, int nchunks, int lane, int K, bool clamp = true)
{
    const int within = nchunks ? (lane < nchunks - 1 ? lane : nchunks - 1) : 0;
    const int i = (int)(k0 >> 2) + within;
    return clamp && i > K / 4 - 1 ? K / 4 - 1 : i;
}

// Element offset (in k) of the activation chunk the same lane loads from global memory first.
HLQ_HD size_t hlq_x_first_k(size_t k0, int nchunks, int lane)
{
    return nchunks ? k0 + (size_t)(lane < nchunks - 1 ? lane : nchunks - 1) * 4 : 0;
}

// K may end half way through the last unit (G = 64): the chunks of the absent half are read from the last
// chunk of x -- and counted as zeros by the caller -- in global memory and in the staged copy alike.
HLQ_HD size_t hlq_x_load_k(size_t k, int K) { return k < (size_t)(K - 4) ? k : (size_t)(K - 4); }
HLQ_HD int hlq_stage_index(size_t k0, int ci, int K)
{
    const int i = (int)(k0 >> 2) + ci;
    return i < K / 4 - 1 ? i : K / 4 - 1;
}

// Row of the handed-over slices a fixed-count load reads for position s (rows past the count re-read the last).
HLQ_HD int hlq_slice_row(int s, int n_slices_in) { return s < n_slices_in - 1 ? s : n_slices_in - 1; }

// ---- narrow tiles (hlq_gemv_narrow.hip): a wave instruction covers cw = 16 / 32 columns of 64 / cw units ----------
// LDS of one wave: the tables of its nu = (64 / cw) * rounds units, one spare table behind each unit's 32 (so that
// units looked up side by side start 16 banks apart), then float2 [2 * nu] half-unit records; rounded up to 256 bytes.
#define HLQ_NARROW_UNIT_STRIDE (HLQ_UNIT_LUT_BYTES + HLQ_TBL_BYTES)
HLQ_HD int hlq_narrow_wave_lds(int nu) { return (nu * HLQ_NARROW_UNIT_STRIDE + 2 * nu * 8 + 255) & ~255; }
// Dynamic LDS of a workgroup: [waves][wave_lds] | float [waves][64] cross-wave sums | float [HLQ_RSTD_SCRATCH] | gap |
// fp16 [K] staged activations (launches that take handed-over slices only).
struct HlqNarrowLds {
    uint32_t red, rstd, stage;      // byte offsets; `stage` == what a launch without staging allocates
};
HLQ_HD HlqNarrowLds hlq_narrow_lds(int nu, int waves)
{
    HlqNarrowLds m;
    m.red = (uint32_t)waves * (uint32_t)hlq_narrow_wave_lds(nu);
    m.rstd = m.red + (uint32_t)waves * 64u * 4u;
    m.stage = m.rstd + (HLQ_RSTD_SCRATCH + HLQ_STAGE_GAP) * 4u;
    return m;
}
// Chunk `ci` (0 .. 32 nu) of a wave: byte offset of its table inside the wave's region, index of its half-unit record.
HLQ_HD uint32_t hlq_narrow_table_off(int ci) { return (uint32_t)(ci >> 5) * HLQ_NARROW_UNIT_STRIDE + (uint32_t)(ci & 31) * HLQ_TBL_BYTES; }
HLQ_HD int hlq_narrow_half_index(int ci) { return ci >> 4; }
// Global chunk index of x a lane loads for chunk `ci` of its wave (first unit `ub`), clamped to the last chunk of x.
HLQ_HD int hlq_narrow_x_chunk(int ub, int ci, int K) { const int c = ub * 32 + ci; return c < K / 4 - 1 ? c : K / 4 - 1; }
// Unit whose weights a lane loads in round r (clamped to the last unit; past it the lane's sum is masked).
HLQ_HD int hlq_narrow_unit(int ub, int r, int ul_count, int ul, int U) { const int u = ub + r * ul_count + ul; return u < U - 1 ? u : U - 1; }

// ---- grouped launch of the matrix-core GEMV (hlq_gemv_mfma.hip) ---------------------------------------------------
// A tile is up to HLQ_MFMA_ITEM_CBS consecutive column blocks of one layer over all of K.  Its work units (unit pair,
// column block), pair-major, are dealt to the sixteen waves of the workgroup in equal contiguous shares.
#define HLQ_MFMA_ITEM_CBS 8

struct HlqMfmaItem {
    int problem, cb0;      // layer and first column block
    int ncb, magic;        // column blocks (1..HLQ_MFMA_ITEM_CBS), ceil(2^20 / ncb)
};

// What one wave does of a tile.
struct HlqMfmaShare {
    int npairs, u_last;    // unit pairs and last unit of the layer
    int cb0, ncb, magic;
    int m_lo, nt, nt_pad;  // first work unit of the wave's share, positions (unit, plane) in it, the same rounded up to `unroll`
};

HLQ_HD HlqMfmaShare hlq_mfma_share(int U, const HlqMfmaItem &it, int wave, int bits, int unroll)
{
    HlqMfmaShare v;
    v.npairs = (U + 1) >> 1;
    v.u_last = U - 1;
    v.cb0 = it.cb0; v.ncb = it.ncb; v.magic = it.magic;
    const int n_units = v.npairs * it.ncb;
    v.m_lo = wave * n_units / 16;
    v.nt = ((wave + 1) * n_units / 16 - v.m_lo) * bits;
    v.nt_pad = (v.nt + unroll - 1) / unroll * unroll;
    return v;
}

// work unit m of a tile -> unit pair and column block inside the tile (exact for m < 2^17, ncb <= 8)
HLQ_HD void hlq_mfma_unit_of(const HlqMfmaShare &v, int m, int &p, int &c)
{
    p = (int)(((unsigned)m * (unsigned)v.magic) >> 20);
    c = m - p * v.ncb;
}

// The unit pair and column block whose plane data a wave loads for position `pos` of its share (positions past the
// share re-read its last one; a wave without a share reads a valid block of the tile).
HLQ_HD void hlq_mfma_load_target(const HlqMfmaShare &v, int pos, int bits, int &p, int &c)
{
    const int last = v.nt - 1 > 0 ? v.nt - 1 : 0;
    hlq_mfma_unit_of(v, v.m_lo + (pos < last ? pos : last) / bits, p, c);
    if (p > v.npairs - 1) p = v.npairs - 1;
    if (c > v.ncb - 1) c = v.ncb - 1;
}

// The tile list: the column blocks of all layers, in order, are cut into `grid` contiguous shares of equal weight (a
// column block weighs its layer's unit count, i.e. its bytes), one per workgroup, and every share into tiles of at most
// HLQ_MFMA_ITEM_CBS column blocks of one layer.  Blob layout: int wg_begin[grid + 1] (padded to 16 bytes), then the
// tiles.  h_blob null: only the size is returned.
static inline size_t hlq_mfma_group_plan(const int *units, const int *ncbs, int count, int grid, void *h_blob)
{
    long long total = 0;
    for (int i = 0; i < count; i++) total += (long long)units[i] * ncbs[i];
    const size_t head = ((size_t)(grid + 1) * sizeof(int) + 15) & ~(size_t)15;
    int *wg_begin = (int *)h_blob;
    HlqMfmaItem *items = h_blob ? (HlqMfmaItem *)((unsigned char *)h_blob + head) : nullptr;
    size_t n_items = 0;
    int layer = 0, cb = 0;
    long long done = 0;
    for (int g = 0; g < grid; g++) {
        if (wg_begin) wg_begin[g] = (int)n_items;
        const long long goal = total * (g + 1) / grid;       // cumulative weight at the end of this share
        while (layer < count) {
            if (cb >= ncbs[layer]) { layer++; cb = 0; continue; }
            // column blocks of this layer that still belong to the share (at least half of a block's weight inside it)
            long long room = (goal - done + units[layer] / 2) / units[layer];
            if (g == grid - 1) room = ncbs[layer] - cb;
            if (room <= 0) break;
            int take = (int)(room < ncbs[layer] - cb ? room : ncbs[layer] - cb);
            done += (long long)take * units[layer];
            while (take > 0) {
                const int len = take < HLQ_MFMA_ITEM_CBS ? take : HLQ_MFMA_ITEM_CBS;
                if (items) items[n_items] = HlqMfmaItem{layer, cb, len, (int)(((1u << 20) + len - 1) / len)};
                n_items++;
                cb += len;
                take -= len;
            }
        }
    }
    if (wg_begin) wg_begin[grid] = (int)n_items;
    return head + n_items * sizeof(HlqMfmaItem);
}

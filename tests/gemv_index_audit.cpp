// CPU audit of the index arithmetic of the batch-1 GEMV tiles (elutq_amd/csrc/hlq_gemv.hip: gemv_tile,
// block_rstd, load_slice_chunk; elutq_amd/csrc/hlq_gemv_narrow.hip: the narrow-tile kernel).  The kernel computes its run boundaries, LDS offsets and staging indices
// with the functions of elutq_amd/csrc/hlq_gemv_index.h; this program replays them for every slice and
// every wave -- waves without a run included -- of a superset of the launch shapes the library can choose,
// and checks the highest byte each access can touch against what the launcher allocates (dynamic LDS =
// hlq_gemv_lds_bytes + the fp16 [K] staging area of a slice-taking launch) and against the buffers the
// C ABI documents.  Built and run by tests/test_gemv_index_audit.py (g++, no GPU).
//
//   gemv_index_audit [--unclamped-stage]     prints "violations <n>" and per-category counts
//
// --unclamped-stage replays the staged-chunk read without its upper clamp (the kernel as it was before the
// clamp was added): the audit must then report violations, which shows that it looks at that access.
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "hlq_gemv_index.h"
#include "hlq_layout.h"

namespace {

constexpr int MAX_LDS = 160 * 1024;
constexpr int CB = 64, UNIT = 128;

int depth_of(int bits) { return bits == 3 ? 6 : (bits == 4 ? 8 : 4); }

std::map<std::string, long> g_viol;
long g_checked = 0;

void check(bool ok, const char *what, int bits, int g64, int waves, int U, int ups, int slice, int wave, int nsl, int multi)
{
    g_checked++;
    if (ok) return;
    if (g_viol[what]++ < 3)
        std::printf("VIOLATION %-14s bits=%d G=%d waves=%d U=%d ups=%d slice=%d wave=%d slices_in=%d run_kernel=%d\n", what, bits,
                    g64 ? 64 : 128, waves, U, ups, slice, wave, nsl, multi);
}

// One launch shape: U units of K, ncb column blocks, slices of `ups` units, `waves` waves per workgroup,
// n_slices_in handed-over slices (0 = none), MULTI = the instances that walk runs of column blocks.
// `ragged`: K ends half way through the last unit (G = 64 only).
void audit(int bits, bool g64, int waves, int U, int ups, int ncb, int n_slices_in, bool multi, bool clamp_stage, bool ragged)
{
    const int K = U * UNIT - (ragged ? UNIT / 2 : 0);
    const HlqWavePlan wp = hlq_wave_plan(ups, bits, waves);
    const size_t lds_alloc = hlq_gemv_lds_bytes(ups, bits, waves) + (n_slices_in ? (size_t)K * 2 : 0);
    if (lds_alloc > (size_t)MAX_LDS) return;                       // the launcher halves the slice or refuses
    const int nslot = wp.spw < depth_of(bits) ? wp.spw : depth_of(bits);
    if (multi && (wp.spw > nslot || waves != 16)) return;          // the condition of the run kernels
    const int ksplit = (U + ups - 1) / ups;
    const HlqLdsMap lm = hlq_lds_map(waves, wp.wave_lds);
    const int NT = ((g64 ? K / 64 : U) + 1) / 2;
    const size_t planes_bytes = (size_t)ncb * U * bits * CB * 16;
    const size_t scale_bytes = (size_t)ncb * NT * bits * CB * 4, zero_bytes = (size_t)ncb * NT * CB * 4;
    const size_t npad = (size_t)ncb * CB;
#define CHECK(ok, what) check((ok), what, bits, g64, waves, U, ups, slice, wave, n_slices_in, multi)
    for (int slice = 0; slice < ksplit; slice++) {
        const int u0 = slice * ups, nU = (u0 + ups < U ? u0 + ups : U) - u0, nst = nU * bits;
        for (int wave = 0; wave < waves; wave++) {
            const HlqWaveRun r = hlq_wave_run(wave, wp.spw, nst, bits);
            const uint32_t lut = (uint32_t)wave * wp.wave_lds, xs = lut + (uint32_t)wp.nuw_max * HLQ_UNIT_LUT_BYTES;
            const size_t k0 = (size_t)(u0 + r.ub) * UNIT;
            const int nchunks = r.nuw * 32;
            CHECK(r.nuw <= wp.nuw_max && r.ub + r.nuw <= nU && r.s_begin <= r.s_end && r.s_last < (nst > 0 ? nst : 1), "run");
            // table build: chunk ci writes 64 bytes at lut + ci * 64 and, as a row leader, float2 xs[ci >> 4]
            for (int ci = 0; ci < nchunks; ci++) {
                CHECK(lut + (uint32_t)ci * 64 + 64 <= xs, "lds-table");
                CHECK(xs + (uint32_t)(ci >> 4) * 8 + 8 <= lut + (uint32_t)wp.wave_lds, "lds-half");
                CHECK(hlq_x_load_k(k0 + (size_t)ci * 4, K) + 4 <= (size_t)K, "x");
                if (n_slices_in && ci >= 64) CHECK(lm.stage + (uint32_t)hlq_stage_index(k0, ci, K) * 8 + 8 <= lm.stage + (uint32_t)K * 2, "lds-stage");
            }
            for (int lane = 0; lane < 64; lane++) {
                CHECK(hlq_x_load_k(hlq_x_first_k(k0, nchunks, lane), K) + 4 <= (size_t)K, "x");
                if (n_slices_in) {
                    const int i = hlq_stage_first_index(k0, nchunks, lane, K, clamp_stage);
                    CHECK(i >= 0 && lm.stage + (uint32_t)i * 8 + 8 <= lds_alloc, "lds-stage");
                }
            }
            // lookups of the wave's sub-tasks: 32 reads of 4 bytes inside the unit's tables, two half-unit records
            for (int st = r.s_begin; st < r.s_end; st++) {
                const int lu = st / bits - r.ub;
                CHECK(lu >= 0 && lut + (uint32_t)lu * HLQ_UNIT_LUT_BYTES + 3 * 8 * 64 + 7 * 64 + 60 + 4 <= xs, "lds-lookup");
                CHECK(xs + (uint32_t)(2 * lu + 1) * 8 + 8 <= lut + (uint32_t)wp.wave_lds, "lds-half");
            }
            // weight stream: slot d holds min(s_begin + d, s_last), refills hold min(st + NSLOT, s_last); every
            // load is (column block base) + st * 1 KiB + lane * 16, scale / zero rows from the absolute unit
            for (int d = 0; d < (r.s_end - r.s_begin > nslot ? r.s_end - r.s_begin : nslot) + nslot; d++) {
                const int st = r.s_begin + d < r.s_last ? r.s_begin + d : r.s_last;
                for (int cb = 0; cb < ncb; cb += (ncb > 1 ? ncb - 1 : 1)) {
                    const size_t off = (((size_t)cb * U + u0) * bits + st) * (CB * 16) + 63 * 16 + 16;
                    CHECK(st >= 0 && off <= planes_bytes, "planes");
                    const int u = u0 + st / bits, b = st % bits, row = g64 ? u : (u >> 1);
                    CHECK(row < NT && ((size_t)cb * NT * bits + (size_t)row * bits + b) * (CB * 4) + 63 * 4 + 4 <= scale_bytes, "scales");
                    CHECK(((size_t)cb * NT + row) * (CB * 4) + 63 * 4 + 4 <= zero_bytes, "zeros");
                }
            }
            // inline sparse plane: record numbers of the run's first two units (fetched by every wave, clamped into the
            // slice), of its further units only where the wave has their plane 0; the lookups use the unit's own tables
            for (int cb = 0; cb < ncb; cb += (ncb > 1 ? ncb - 1 : 1)) {
                for (int j = 0; j < 2; j++) {
                    const int uj = r.ub + j < nU - 1 ? r.ub + j : nU - 1;
                    CHECK(uj >= 0 && (size_t)cb * U + u0 + uj < (size_t)ncb * U, "sparse-cell");
                    const bool own = j < r.nuw && r.s_begin <= (r.ub + j) * bits && (r.ub + j) * bits < r.s_end;
                    if (own) CHECK(lut + (uint32_t)j * HLQ_UNIT_LUT_BYTES + 3 * 8 * 64 + 7 * 64 + 60 + 4 <= xs, "sparse-lookup");
                }
                for (int j = 2; j < r.nuw; j++) {
                    if (!(r.s_begin <= (r.ub + j) * bits && (r.ub + j) * bits < r.s_end)) continue;
                    CHECK(r.ub + j < nU && (size_t)cb * U + u0 + r.ub + j < (size_t)ncb * U, "sparse-cell");
                    CHECK(lut + (uint32_t)j * HLQ_UNIT_LUT_BYTES + 3 * 8 * 64 + 7 * 64 + 60 + 4 <= xs, "sparse-lookup");
                }
            }
            // cross-wave sums (two alternating buffers), reduction scratch of the RMSNorm prologue
            for (int sel = 0; sel < 2; sel++)
                CHECK(lm.red + ((uint32_t)(sel * waves + wave) * 64 + 63) * 4 + 4 <= lm.rstd, "lds-red");
            CHECK(lm.rstd + (uint32_t)((waves * 64 - 1) >> 4) * 4 + 4 <= lm.rstd + 64 * 4 && lm.rstd + 64 * 4 + 4 <= lm.stage, "lds-rstd");
            // partial sums of the slice and handed-over slices
            CHECK((size_t)slice * npad + (size_t)(ncb - 1) * CB + 63 < (size_t)ksplit * npad, "partial");
        }
        // block_rstd: thread tid stages chunks tid, tid + nthreads, ... of the whole K and reads 4 slice rows per chunk
        if (n_slices_in) {
            const int wave = -1;
            for (int i = 0; i < K / 4; i++) CHECK(lm.stage + (uint32_t)i * 8 + 8 <= lds_alloc, "lds-stage");
            for (int s = 0; s < HLQ_GEMV_MAX_SLICES_IN; s++) {
                const int row = hlq_slice_row(s, n_slices_in);
                CHECK(row >= 0 && row < n_slices_in && (size_t)row * K + (size_t)(K / 4 - 1) * 4 + 4 <= (size_t)n_slices_in * K, "slices-in");
            }
            const int first = (waves * 64 - 1 < K / 4 - 1 ? waves * 64 - 1 : K / 4 - 1);
            CHECK(first >= 0 && first < K / 4, "slices-in");
        }
    }
#undef CHECK
}

// The narrow-tile kernel (hlq_gemv_narrow.hip): workgroups of cw = 16 / 32 columns over all of K, `rounds` units per
// unit lane of a wave, waves = ceil(U / nu).  Every wave and lane: table stores and half-unit records inside the wave's
// region, lookups inside the unit's tables, activation chunks inside x and the staged copy, weight / scale / zero loads
// inside the layer's buffers, cross-wave sums and reduction scratch inside the allocation.
void audit_narrow(int bits, bool g64, int cw, int rounds, int U, int ncb, bool ragged, bool staged)
{
    const int K = U * UNIT - (ragged ? UNIT / 2 : 0);
    const int ul_count = 64 / cw, nu = ul_count * rounds, waves = (U + nu - 1) / nu;
    if (waves > 16) return;
    const HlqNarrowLds lm = hlq_narrow_lds(nu, waves);
    const size_t lds_alloc = lm.stage + (staged ? (size_t)K * 2 : 0);
    if (lds_alloc > (size_t)MAX_LDS) return;
    const int wave_lds = hlq_narrow_wave_lds(nu);
    const int NT = ((g64 ? K / 64 : U) + 1) / 2;
    const size_t planes_bytes = (size_t)ncb * U * bits * CB * 16;
    const size_t scale_bytes = (size_t)ncb * NT * bits * CB * 4, zero_bytes = (size_t)ncb * NT * CB * 4;
    const int slice = 0, n_slices_in = staged ? 4 : 0, multi = 0, ups = U;
#define CHECK(ok, what) check((ok), what, bits, g64, waves, U, ups, slice, wave, n_slices_in, multi)
    for (int wave = 0; wave < waves; wave++) {
        const uint32_t lut = (uint32_t)wave * wave_lds, xs = lut + (uint32_t)nu * HLQ_NARROW_UNIT_STRIDE;
        const int ub = wave * nu;
        for (int ci = 0; ci < 32 * nu; ci++) {
            CHECK(lut + hlq_narrow_table_off(ci) + 64 <= xs, "n-lds-table");
            CHECK(xs + (uint32_t)hlq_narrow_half_index(ci) * 8 + 8 <= lut + (uint32_t)wave_lds, "n-lds-half");
            const int xc = hlq_narrow_x_chunk(ub, ci, K);
            CHECK(xc >= 0 && (size_t)xc * 4 + 4 <= (size_t)K, "n-x");
            if (staged) CHECK(lm.stage + (uint32_t)xc * 8 + 8 <= lds_alloc, "n-lds-stage");
        }
        for (int r = 0; r < rounds; r++)
            for (int ul = 0; ul < ul_count; ul++) {
                const int lu = r * ul_count + ul;
                CHECK(lut + (uint32_t)lu * HLQ_NARROW_UNIT_STRIDE + 3 * 8 * 64 + 7 * 64 + 60 + 4 <= xs, "n-lds-lookup");
                CHECK(xs + (uint32_t)(2 * lu + 1) * 8 + 8 <= lut + (uint32_t)wave_lds, "n-lds-half");
                const int u = hlq_narrow_unit(ub, r, ul_count, ul, U), row = g64 ? u : (u >> 1);
                for (int cb = 0; cb < ncb; cb += (ncb > 1 ? ncb - 1 : 1))
                    for (int b = 0; b < bits; b++) {
                        CHECK(u >= 0 && (((size_t)cb * U + u) * bits + b) * (CB * 16) + 63 * 16 + 16 <= planes_bytes, "n-planes");
                        CHECK(row < NT && ((size_t)cb * NT * bits + (size_t)row * bits + b) * (CB * 4) + 63 * 4 + 4 <= scale_bytes, "n-scales");
                        CHECK(((size_t)cb * NT + row) * (CB * 4) + 63 * 4 + 4 <= zero_bytes, "n-zeros");
                    }
                // inline sparse plane: the record number of the lane's unit, the lane's 20 bytes of a 1280-byte record
                for (int cb = 0; cb < ncb; cb += (ncb > 1 ? ncb - 1 : 1)) CHECK((size_t)cb * U + u < (size_t)ncb * U, "n-sparse-cell");
                for (int part = 0; part < ul_count; part++)
                    CHECK((size_t)(part * cw + cw - 1) * 16 + 16 <= 1024 && 1024 + (size_t)(part * cw + cw - 1) * 4 + 4 <= HLQ_SP_REC_BYTES, "n-sparse-rec");
            }
        CHECK(lm.red + ((uint32_t)wave * 64 + 63) * 4 + 4 <= lm.rstd, "n-lds-red");
        CHECK(lm.rstd + (uint32_t)((waves * 64 - 1) >> 4) * 4 + 4 <= lm.rstd + 64 * 4 && lm.rstd + 64 * 4 + 4 <= lm.stage, "n-lds-rstd");
    }
#undef CHECK
}

// The grouped launch of the matrix-core kernel (hlq_gemv_mfma.hip: hlq_gemv_mfma_group_kernel): the plan's shares and
// tiles must cover every column block of every layer exactly once, every work unit (unit pair, column block) of a tile
// must fall to exactly one wave, and every plane / scale / zero / activation load -- the positions past a wave's share
// and the ring refills that reach into the next tile included -- must stay inside the layer's buffers.
void audit_mfma_group(const std::vector<int> &units, const std::vector<int> &ncbs, int grid, int bits, bool g64)
{
    const int count = (int)units.size();
    std::vector<unsigned char> blob(hlq_mfma_group_plan(units.data(), ncbs.data(), count, grid, nullptr));
    hlq_mfma_group_plan(units.data(), ncbs.data(), count, grid, blob.data());
    const int *wg_begin = (const int *)blob.data();
    const HlqMfmaItem *items = (const HlqMfmaItem *)(blob.data() + (((size_t)(grid + 1) * sizeof(int) + 15) & ~(size_t)15));
    const int slice = 0, n_slices_in = 0, multi = 2, waves = 16;
    const int unroll = bits % 2 ? 2 * bits : bits;
    std::vector<std::vector<int>> seen(count);
    for (int i = 0; i < count; i++) seen[i].assign(ncbs[i], 0);
    long long total = 0, heaviest = 0;
    for (int i = 0; i < count; i++) total += (long long)units[i] * ncbs[i];
    int wave = 0, U = 0, ups = 0;
#define CHECK(ok, what) check((ok), what, bits, g64, waves, U, ups, slice, wave, n_slices_in, multi)
    CHECK(wg_begin[0] == 0, "g-plan");
    for (int g = 0; g < grid; g++) {
        long long weight = 0;
        CHECK(wg_begin[g] <= wg_begin[g + 1], "g-plan");
        for (int i = wg_begin[g]; i < wg_begin[g + 1]; i++) {
            const HlqMfmaItem &it = items[i];
            CHECK(it.problem >= 0 && it.problem < count && it.ncb >= 1 && it.ncb <= HLQ_MFMA_ITEM_CBS && it.cb0 >= 0 &&
                  it.cb0 + it.ncb <= ncbs[it.problem] && it.magic == (int)(((1u << 20) + it.ncb - 1) / it.ncb), "g-item");
            U = units[it.problem]; ups = it.ncb;
            for (int c = 0; c < it.ncb; c++) seen[it.problem][it.cb0 + c]++;
            weight += (long long)U * it.ncb;
            const int npairs = (U + 1) / 2;
            std::vector<int> unit_seen(npairs * it.ncb, 0);
            const int K = U * UNIT, NT = ((g64 ? K / 64 : U) + 1) / 2, ncb_layer = ncbs[it.problem];
            const size_t planes_bytes = (size_t)ncb_layer * U * bits * CB * 16;
            const size_t scale_bytes = (size_t)ncb_layer * NT * bits * CB * 4, zero_bytes = (size_t)ncb_layer * NT * CB * 4;
            for (wave = 0; wave < 16; wave++) {
                const HlqMfmaShare v = hlq_mfma_share(U, it, wave, bits, unroll);
                CHECK(v.nt >= 0 && v.nt % bits == 0 && v.nt_pad >= v.nt && v.nt_pad % unroll == 0, "g-share");
                for (int pos = 0; pos < v.nt; pos += bits) {
                    int p, c;
                    hlq_mfma_unit_of(v, v.m_lo + pos / bits, p, c);
                    CHECK(p >= 0 && p < npairs && c >= 0 && c < it.ncb, "g-unit");
                    if (p >= 0 && p < npairs && c >= 0 && c < it.ncb) unit_seen[p * it.ncb + c]++;
                }
                // loads: every position of the share, the refills past it, and what a wave without a share reads
                for (int pos = -2; pos < v.nt_pad + 4; pos++) {
                    int p, c;
                    hlq_mfma_load_target(v, pos < 0 ? 0 : pos, bits, p, c);
                    CHECK(p >= 0 && p < npairs && c >= 0 && c < it.ncb, "g-load");
                    const int cb = it.cb0 + c, u = 2 * p, u1 = u + 1 < U - 1 ? u + 1 : U - 1;
                    for (int b = 0; b < bits; b++)
                        for (int uu : {u, u1}) {
                            CHECK(uu >= 0 && uu < U && (((size_t)cb * U + uu) * bits + b) * (CB * 16) + 63 * 16 + 16 <= planes_bytes, "g-planes");
                            const int row = g64 ? uu : (uu >> 1);
                            CHECK(row < NT && ((size_t)cb * NT * bits + (size_t)row * bits + b) * (CB * 4) + 63 * 4 + 4 <= scale_bytes, "g-scales");
                            CHECK(((size_t)cb * NT + row) * (CB * 4) + 63 * 4 + 4 <= zero_bytes, "g-zeros");
                        }
                    // the activations of the pair (and of the one requested ahead): unit min(2 p + 1, U - 1), 128 k each
                    for (int pp : {p, p + 1 < npairs ? p + 1 : npairs - 1}) {
                        const int ku = 2 * pp + 1 < U - 1 ? 2 * pp + 1 : U - 1;
                        CHECK((size_t)ku * UNIT + 31 * 4 + 4 <= (size_t)K, "g-x");
                    }
                }
            }
            wave = -1;
            for (int x : unit_seen) CHECK(x == 1, "g-cover");
        }
        if (weight > heaviest) heaviest = weight;
    }
    wave = -1; U = 0; ups = 0;
    for (int i = 0; i < count; i++)
        for (int x : seen[i]) CHECK(x == 1, "g-blocks");
    // balance: no share exceeds the mean by more than one column block of the heaviest layer
    int umax = 0;
    for (int u : units) umax = u > umax ? u : umax;
    CHECK(heaviest <= total / grid + umax + 1, "g-balance");
#undef CHECK
}

}  // namespace

int main(int argc, char **argv)
{
    const bool clamp_stage = !(argc > 1 && std::strcmp(argv[1], "--unclamped-stage") == 0);
    long shapes = 0;
    const int Us[] = {1, 2, 3, 5, 8, 16, 28, 32, 40, 43, 108, 112};     // K = 128 .. 14336 (4096, 5120, 13824 among them)
    const int wave_counts[] = {1, 2, 3, 4, 5, 7, 8, 12, 15, 16};
    for (int bits = 1; bits <= 4; bits++)
        for (int g64 = 0; g64 < 2; g64++)
            for (int waves : wave_counts)
                for (int U : Us)
                    for (int ups = 1; ups <= U; ups++)
                        for (int nsl = 0; nsl <= HLQ_GEMV_MAX_SLICES_IN; nsl++)
                            for (int multi = 0; multi < 2; multi++) {
                                for (int ragged = 0; ragged <= (g64 && U > 1 ? 1 : 0); ragged++) {
                                    audit(bits, g64 != 0, waves, U, ups, multi ? 448 : 3, nsl, multi != 0, clamp_stage, ragged != 0);
                                    shapes++;
                                }
                            }
    // narrow tiles: the instances the launcher has (16 columns x 1 round, 32 x 1, 32 x 2), every unit count they take
    const int narrow[3][2] = {{16, 1}, {32, 1}, {32, 2}};
    for (int bits = 1; bits <= 4; bits++)
        for (int g64 = 0; g64 < 2; g64++)
            for (auto &cr : narrow)
                for (int U = 1; U <= 64; U++)
                    for (int ragged = 0; ragged <= (g64 && U > 1 ? 1 : 0); ragged++)
                        for (int staged = 0; staged < 2; staged++) {
                            audit_narrow(bits, g64 != 0, cr[0], cr[1], U, 3, ragged != 0, staged != 0);
                            shapes++;
                        }
    // grouped launch of the matrix-core kernel: the LLaMA-3-8B sweep, one wide layer, mixed odd shapes, fewer blocks than shares
    {
        std::vector<int> su, sn;
        for (int layer = 0; layer < 32; layer++) {
            const int kn[7][2] = {{32, 64}, {32, 16}, {32, 16}, {32, 64}, {32, 224}, {32, 224}, {112, 64}};
            for (auto &x : kn) { su.push_back(x[0]); sn.push_back(x[1]); }
        }
        for (int bits = 1; bits <= 4; bits++)
            for (int g64 = 0; g64 < 2; g64++) {
                audit_mfma_group(su, sn, 256, bits, g64 != 0);
                audit_mfma_group({32}, {2004}, 256, bits, g64 != 0);
                audit_mfma_group({4, 8, 32, 64, 1, 72, 5}, {2, 2, 4, 1, 1, 3, 3}, 16, bits, g64 != 0);
                audit_mfma_group({1, 3, 224, 7}, {1, 300, 5, 9}, 256, bits, g64 != 0);
                audit_mfma_group({40, 108}, {80, 216}, 256, bits, g64 != 0);
                audit_mfma_group({2}, {1}, 1, bits, g64 != 0);
                shapes += 6;
            }
    }
    long total = 0;
    for (auto &kv : g_viol) {
        std::printf("category %s %ld\n", kv.first.c_str(), kv.second);
        total += kv.second;
    }
    std::printf("shapes %ld checks %ld\nviolations %ld\n", shapes, g_checked, total);
    return total ? 1 : 0;
}

// Block-sparse extra plane of a `use_sparse` layer.
//
// Beside its dense planes such a layer has one more binary plane that exists only on listed
// blocks of 32 output channels x G input channels, each block with 32 fp16 scales of its own and
// no zero term.  The reference reads the list from weight_mask.bin (uint32 pairs: channel start,
// k start), the block bits and scales from the tails of w_quant.bin / w_scale.bin
// (C++/ops/src/arm/parameters.cpp:19-64), permutes the bits for its NEON kernel
// (t_mac_g4_rearrange_weight_sparse_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:554-647) and adds the
// plane to the output after the dense planes (t_mac_g4_float_update_sparse_impl, :678-788, called
// from C++/ops/src/arm/arm_gemm.cpp:779-790).
//
// The plane's contribution is computed first, in fp32, into the tail of the call's workspace; the
// dense GEMV / GEMM kernel then adds it to its own fp32 sum before the one rounding to fp16, so a
// sparse layer's output is as exact as a dense layer's.
//
// In a decode step the projection's input may only exist inside the launch that reads it (the fused GEMV forms
// RMSNorm(x) or SiLU(gate) * up in its prologue): the batch-1 plane kernel then forms the same values itself, with
// the same operations (prologue_value), from the same stored vectors.
//
// The block bits and scales stay exactly as the files hold them -- [block][32 channels][G/8
// bytes] is already what a wave wants: consecutive lanes own consecutive parts of one channel's k, so a
// block is one contiguous 32*G/8-byte read -- and the pair list becomes an index by channel tile.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <vector>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"
#include "hlq_gemv_dev.h"

namespace {

constexpr int SP_TILE = 32;        // channels per block
constexpr int SP_PARTS = 8;        // lanes that share a channel: each owns G/8 consecutive k
constexpr int SP_THREADS = SP_TILE * SP_PARTS;
constexpr int SP_HEAD = 16;        // k starts per tile that the batch-1 kernel finds without knowing the tile's block range

inline int sp_tiles(int N) { return (N + SP_TILE - 1) / SP_TILE; }

struct SparseArgs {
    const uint8_t *blocks;         // [nblk][32][G/8]
    const uint16_t *blk_scales;    // fp16 [nblk][32]
    const int32_t *tile_ptr;       // [tiles + 1]: blocks of tile t are tile_ptr[t] .. tile_ptr[t+1]-1
    const int32_t *blk_k;          // [nblk] k start
    const int32_t *head;           // [tiles][SP_HEAD]: k starts of a tile's first SP_HEAD blocks again (-1: no such block)
    const uint16_t *x;             // fp16 [M][K]
    float *extra;                  // fp32 [M][N], written for every (m, n)
    uint16_t *w;                   // fp16 [N][K] (dequantisation only)
    int M, K, N, nblk;
    // M == 1 only: the activations pass through the prologue of the fused GEMV first
    int prologue;                  // 0: x as is; 1: rmsnorm(x) * norm_w; 2: silu(x[0:K]) * x[K:2K]
    float eps;
    const uint16_t *norm_w;        // fp16 [K] (prologue 1)
};

__device__ __forceinline__ float hf(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
__device__ __forceinline__ uint16_t fh(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

// v where bit `pos` of `bits` is set, else +0: the sums below add every activation, masked, rather than branch on
// the bits (the compiler turns `if (bit) sum += v` into a branch around each load).
__device__ __forceinline__ float bit_select(float v, uint32_t bits, int pos)
{
    const uint32_t mask = (uint32_t)__builtin_amdgcn_sbfe((int)bits, pos, 1);      // the bit, sign-extended
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) & mask);
}

// Thread (channel, part) of a block: its G/8 bits, LSB = lowest k.
template <int G>
__device__ __forceinline__ uint32_t block_bits(const uint8_t *blocks, int blk, int ch, int part)
{
    const uint8_t *p = blocks + ((size_t)blk * SP_TILE + ch) * (G / 8) + part * (G / 64);
    if (G == 64) return p[0];
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8);
}

// extra[m][c0 + ch] = sum over the tile's blocks of scale[blk][ch] * sum_{k in block, bit set} x[m][k]
// (0 for a tile without blocks).  grid (tiles, ceil(M / ROWS)); every sum in fp32 in a fixed order.
// NB blocks are in flight at a time: the k start, bits, scale and activations of one block depend on
// each other only through addresses, so the loads of NB blocks overlap and a tile costs about
// three memory round trips per NB blocks instead of per block.
template <int G, int ROWS, int NB>
__global__ __launch_bounds__(SP_THREADS) void hlq_sparse_plane_kernel(const SparseArgs a)
{
    constexpr int KP = G / SP_PARTS;                 // k per thread and block: 8 or 16
    const int tile = blockIdx.x, m0 = blockIdx.y * ROWS;
    const int b0 = a.tile_ptr[tile], b1 = a.tile_ptr[tile + 1];
    const int tid = threadIdx.x, ch = tid / SP_PARTS, part = tid % SP_PARTS;
    float tot[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) tot[r] = 0.f;
    for (int blk0 = b0; blk0 < b1; blk0 += NB) {
        int k0[NB];
        uint32_t bits[NB];
        float s[NB];
        uint2 xv[NB][ROWS][KP / 4];
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int blk = min(blk0 + i, b1 - 1);   // past the end: the last block again, its result dropped
            k0[i] = a.blk_k[blk];
            bits[i] = block_bits<G>(a.blocks, blk, ch, part);
            s[i] = hf(a.blk_scales[(size_t)blk * SP_TILE + ch]);
        }
#pragma unroll
        for (int i = 0; i < NB; i++) {
            // the index is validated on the host; a bad k start still never reads outside x
            const bool ok = k0[i] >= 0 && k0[i] + G <= a.K && blk0 + i < b1;
            if (!ok) { k0[i] = 0; s[i] = 0.f; bits[i] = 0; }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const int m = min(m0 + r, a.M - 1);
                const uint2 *xp = (const uint2 *)(a.x + (size_t)m * a.K + k0[i] + part * KP);   // k0 % 4 == 0: 8-byte aligned
#pragma unroll
                for (int q = 0; q < KP / 4; q++) xv[i][r][q] = xp[q];
            }
        }
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                float sum = 0.f;
#pragma unroll
                for (int q = 0; q < KP / 4; q++) {
                    const uint2 v = xv[i][r][q];
                    const uint16_t h[4] = {(uint16_t)(v.x & 0xffffu), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xffffu),
                                           (uint16_t)(v.y >> 16)};
#pragma unroll
                    for (int j = 0; j < 4; j++) sum += bit_select(hf(h[j]), bits[i], 4 * q + j);
                }
                // the 8 parts of a channel sit in 8 consecutive lanes
                sum += __shfl_xor(sum, 1);
                sum += __shfl_xor(sum, 2);
                sum += __shfl_xor(sum, 4);
                tot[r] = fmaf(s[i], sum, tot[r]);
            }
    }
    const int n = tile * SP_TILE + ch;
    if (part == 0 && n < a.N) {
#pragma unroll
        for (int r = 0; r < ROWS; r++)
            if (m0 + r < a.M) a.extra[(size_t)(m0 + r) * a.N + n] = tot[r];
    }
}

// Batch 1: one workgroup of up to sixteen waves per channel tile; wave w takes the tile's blocks w, w + 16, ... and
// works on a block alone (a tile's blocks cost a chain of dependent memory round trips -- block range, k starts,
// activations -- whatever their number, so as many as possible go through it side by side).  The G activations of a
// block are the same for its 32 channels, so the wave forms them once (two per lane, through the prologue if there
// is one), parks them in LDS as fp32 and every lane (channel, half of the block's k) adds up the ones its bits
// select: LDS reads of one address per half, no bank conflicts.  NB blocks of a wave are in flight at a time (their
// k starts, bits, scales and activations depend on each other only through addresses).  The waves' sums meet in LDS
// in wave order: the result does not depend on timing.
constexpr int SPV_WAVES = 16;                    // at most; the launch decides (blockDim.x / 64)

template <int G, bool PRO, int NB>
__global__ __launch_bounds__(SPV_WAVES * 64) void hlq_sparse_plane_gemv_kernel(const SparseArgs a)
{
    constexpr int HALF = G / 2;                      // k per lane and block
    __shared__ __align__(16) float xs[SPV_WAVES][NB][G];
    __shared__ float red[SPV_WAVES][SP_TILE];
    __shared__ float part_ssq[SPV_WAVES];
    const int tile = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nw = blockDim.x >> 6;
    const int ch = lane >> 1, part = lane & 1;
    const int prologue = PRO ? a.prologue : 0;
    // block `wave` of the tile is this wave's first: its k start comes in with the tile's block range, not after it
    // (one memory round trip fewer in front of the activations)
    const int k_head = a.head[(size_t)tile * SP_HEAD + wave];
    const int b0 = a.tile_ptr[tile], b1 = a.tile_ptr[tile + 1];
    const int n = tile * SP_TILE + ch;
    if (b0 >= b1) {                                  // the same for every thread of the workgroup
        if (wave == 0 && part == 0 && n < a.N) a.extra[n] = 0.f;
        return;
    }
    const uint16_t *second = prologue == 1 ? a.norm_w : (prologue == 2 ? a.x + a.K : a.x);
    const int xl = G == 128 ? lane : (lane & 31);    // the pair of activations this lane forms (G = 64: both halves of the wave the same)
    int k0[NB];
    uint32_t raw[NB], raw2[NB], bits[NB][HALF / 32];
    float s[NB];
    // everything a round of NB blocks reads from memory (nothing of it depends on 1 / rms): first what depends on
    // the block numbers alone, then the activations at the k starts that came in
    auto load_meta = [&](int base, bool first) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int blk = base + i * nw;
            const int blkc = min(blk, b1 - 1);       // past the end: the last block again, its result dropped
            k0[i] = first && i == 0 ? k_head : a.blk_k[blkc];
            const uint32_t *bp = (const uint32_t *)(a.blocks + ((size_t)blkc * SP_TILE + ch) * (G / 8) + part * (HALF / 8));
#pragma unroll
            for (int q = 0; q < HALF / 32; q++) bits[i][q] = bp[q];
            s[i] = hf(a.blk_scales[(size_t)blkc * SP_TILE + ch]);
            // the index is validated on the host; a bad k start still never reads outside x
            if (!(blk < b1 && k0[i] >= 0 && k0[i] + G <= a.K)) {
                k0[i] = 0; s[i] = 0.f;
#pragma unroll
                for (int q = 0; q < HALF / 32; q++) bits[i][q] = 0;
            }
        }
    };
    auto load_x = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            raw[i] = *(const uint32_t *)(a.x + k0[i] + 2 * xl);          // k0 % 4 == 0: 4-byte aligned
            raw2[i] = PRO ? *(const uint32_t *)(second + k0[i] + 2 * xl) : raw[i];
        }
    };
    load_meta(b0 + wave, true);                      // in flight while the workgroup sums the squares
    float rstd = 1.f;
    if (PRO && prologue == 1) {
        float ssq = 0.f;
        for (int i = tid; i < a.K / 4; i += nw * 64) {
            const uint2 r = *(const uint2 *)(a.x + (size_t)i * 4);
            const float x0 = h2f_lo(r.x), x1 = h2f_hi(r.x), x2 = h2f_lo(r.y), x3 = h2f_hi(r.y);
            ssq += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
        }
        load_x();
#pragma unroll
        for (int d = 1; d < 64; d *= 2) ssq += __shfl_xor(ssq, d, 64);
        if (lane == 0) part_ssq[wave] = ssq;
        __syncthreads();
        float all = 0.f;
        for (int w = 0; w < nw; w++) all += part_ssq[w];
        rstd = rsqrtf(all / (float)a.K + a.eps);
    } else {
        load_x();
    }
    float tot = 0.f;
    for (int base = b0 + wave; base < b1; base += nw * NB) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            float v0 = h2f_lo(raw[i]), v1 = h2f_hi(raw[i]);
            if (PRO && prologue != 0) {
                v0 = prologue_value(prologue, v0, h2f_lo(raw2[i]), rstd);
                v1 = prologue_value(prologue, v1, h2f_hi(raw2[i]), rstd);
            }
            if (G == 128 || lane < 32) *(float2 *)&xs[wave][i][2 * xl] = make_float2(v0, v1);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");          // this wave's LDS stores before its loads below
        __builtin_amdgcn_wave_barrier();
        float sums[NB];
#pragma unroll
        for (int i = 0; i < NB; i++) {
            sums[i] = 0.f;
            if (base + i * nw >= b1) continue;       // no such block (the same for the whole wave)
            const float4 *xp = (const float4 *)&xs[wave][i][part * HALF];
            float sum = 0.f;
#pragma unroll
            for (int q = 0; q < HALF / 4; q++) {
                // an activation or +0, chosen by an all-ones / all-zeros mask made of its bit: no branches, and the
                // reads of a block go out together
                const float4 v = xp[q];
                const uint32_t w = bits[i][q / 8];
                sum += bit_select(v.x, w, 4 * (q % 8));
                sum += bit_select(v.y, w, 4 * (q % 8) + 1);
                sum += bit_select(v.z, w, 4 * (q % 8) + 2);
                sum += bit_select(v.w, w, 4 * (q % 8) + 3);
            }
            sums[i] = sum + __shfl_xor(sum, 1, 64);  // the two halves of a channel sit in neighbouring lanes
        }
#pragma unroll
        for (int i = 0; i < NB; i++) tot = fmaf(s[i], sums[i], tot);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");          // ... and those loads before the next round's stores
        __builtin_amdgcn_wave_barrier();
        if (base + nw * NB < b1) {
            load_meta(base + nw * NB, false);
            load_x();
        }
    }
    if (part == 0) red[wave][ch] = tot;
    __syncthreads();
    if (wave == 0 && part == 0 && n < a.N) {
        float sum = red[0][ch];
        for (int w = 1; w < nw; w++) sum += red[w][ch];
        a.extra[n] = sum;
    }
}

// W[c0 + ch][k0 + j] += scale[blk][ch] where the block's bit is set.  One workgroup per channel
// tile walks the tile's blocks in list order with a barrier between them, so blocks that overlap in
// k (the format does not forbid it) add up as they do in the GEMV.
template <int G>
__global__ __launch_bounds__(SP_THREADS) void hlq_sparse_dequant_kernel(const SparseArgs a)
{
    constexpr int KP = G / SP_PARTS;
    const int tile = blockIdx.x;
    const int b0 = a.tile_ptr[tile], b1 = a.tile_ptr[tile + 1];
    const int tid = threadIdx.x, ch = tid / SP_PARTS, part = tid % SP_PARTS;
    const int n = tile * SP_TILE + ch;
    for (int blk = b0; blk < b1; blk++) {
        const int k0 = a.blk_k[blk];
        if (k0 >= 0 && k0 + G <= a.K && n < a.N) {
            const uint32_t bits = block_bits<G>(a.blocks, blk, ch, part);
            const float s = hf(a.blk_scales[(size_t)blk * SP_TILE + ch]);
            uint16_t *wp = a.w + (size_t)n * a.K + k0 + part * KP;
#pragma unroll
            for (int j = 0; j < KP; j++)
                if (bits >> j & 1u) wp[j] = fh(hf(wp[j]) + s);
        }
        __syncthreads();
    }
}

int check_sparse_call(int K, int N, int group, int nblk)
{
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (N < 1 || !hlq_k_ok(K, group) || nblk < 0) return ELUTQ_ERR_SHAPE;
    return ELUTQ_OK;
}

SparseArgs sparse_args(const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk, int K, int N)
{
    SparseArgs a = {};
    a.blocks = (const uint8_t *)d_blocks;
    a.blk_scales = (const uint16_t *)d_blk_scales;
    a.tile_ptr = (const int32_t *)d_index;
    a.blk_k = a.tile_ptr + sp_tiles(N) + 1;
    a.head = a.blk_k + nblk;
    a.K = K; a.N = N; a.nblk = nblk;
    return a;
}

// The plane's term for rows x[0..M) into extra[M][N].
int launch_sparse_plane(SparseArgs a, const void *d_x, float *d_extra, int M, int group, hipStream_t stream)
{
    a.x = (const uint16_t *)d_x;
    a.extra = d_extra;
    a.M = M;
    if (M == 1) {
        // the kernel reads block bits as dwords and activations as fp16 pairs
        if (((uintptr_t)a.blocks & 3) != 0 || ((uintptr_t)d_x & 3) != 0 || ((uintptr_t)a.norm_w & 3) != 0) return ELUTQ_ERR_SHAPE;
        // as many waves per tile as leave all tiles resident at once (32 waves per compute unit)
        const int tiles = sp_tiles(a.N);
        const int waves = tiles * 16 <= HLQ_NUM_CU * 32 ? 16 : (tiles * 8 <= HLQ_NUM_CU * 32 ? 8 : 4);
        const dim3 grid(tiles), block(waves * 64);
        if (a.prologue != 0) {
            if (group == 64) hipLaunchKernelGGL((hlq_sparse_plane_gemv_kernel<64, true, 2>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((hlq_sparse_plane_gemv_kernel<128, true, 2>), grid, block, 0, stream, a);
        } else {
            if (group == 64) hipLaunchKernelGGL((hlq_sparse_plane_gemv_kernel<64, false, 2>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((hlq_sparse_plane_gemv_kernel<128, false, 2>), grid, block, 0, stream, a);
        }
    } else {
        if (a.prologue != 0) return ELUTQ_ERR_TUNING;
        const dim3 grid(sp_tiles(a.N), (M + 3) / 4);
        if (group == 64) hipLaunchKernelGGL((hlq_sparse_plane_kernel<64, 4, 2>), grid, dim3(SP_THREADS), 0, stream, a);
        else hipLaunchKernelGGL((hlq_sparse_plane_kernel<128, 4, 2>), grid, dim3(SP_THREADS), 0, stream, a);
    }
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

size_t elutq_hlq_sparse_index_bytes(int N, int nblk)
{
    if (N < 1 || nblk < 0) return 0;
    return sizeof(int32_t) * ((size_t)sp_tiles(N) + 1 + (size_t)nblk + (size_t)sp_tiles(N) * SP_HEAD);
}

int elutq_hlq_sparse_index_host(const uint32_t *h_mask, int mask_len, int K, int N, int group, void *h_index_out)
{
    if (mask_len < 0 || mask_len % 2) return ELUTQ_ERR_SPARSE;
    const int nblk = mask_len / 2;
    int rc = check_sparse_call(K, N, group, nblk);
    if (rc != ELUTQ_OK) return rc;
    if ((!h_mask && nblk) || !h_index_out) return ELUTQ_ERR_NULL;
    const int tiles = sp_tiles(N);
    int32_t *tile_ptr = (int32_t *)h_index_out, *blk_k = tile_ptr + tiles + 1;
    for (int t = 0; t <= tiles; t++) tile_ptr[t] = 0;
    uint32_t prev = 0;
    for (int i = 0; i < nblk; i++) {
        const uint32_t c = h_mask[2 * i], k = h_mask[2 * i + 1];
        if (c % SP_TILE || c >= (uint32_t)N || k % 4 || (uint64_t)k + (uint32_t)group > (uint32_t)K || c < prev)
            return ELUTQ_ERR_SPARSE;
        prev = c;
        tile_ptr[c / SP_TILE + 1]++;
        blk_k[i] = (int32_t)k;
    }
    for (int t = 0; t < tiles; t++) tile_ptr[t + 1] += tile_ptr[t];
    int32_t *head = blk_k + nblk;
    for (int t = 0; t < tiles; t++)
        for (int j = 0; j < SP_HEAD; j++)
            head[(size_t)t * SP_HEAD + j] = tile_ptr[t] + j < tile_ptr[t + 1] ? blk_k[tile_ptr[t] + j] : -1;
    return ELUTQ_OK;
}

size_t elutq_hlq_sparse_workspace_bytes(int K, int N, int bits, int group, int M)
{
    const size_t dense = elutq_hlq_workspace_bytes(K, N, bits, group, M);
    if (!dense || M < 1) return 0;
    const int rows = M < HLQ_GEMM_MAX_M ? M : HLQ_GEMM_MAX_M;
    return align256(dense) + (size_t)rows * N * sizeof(float);
}

int elutq_hlq_sparse_gemm_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                              const void *d_x, void *d_y, int M, int K, int N, int bits, int group,
                              void *d_workspace, size_t workspace_bytes, void *stream)
{
    int rc = check_sparse_call(K, N, group, nblk);
    if (rc != ELUTQ_OK) return rc;
    if (M < 1) return ELUTQ_ERR_SHAPE;
    if (!d_index || !d_x || !d_y || !d_workspace || (nblk && (!d_blocks || !d_blk_scales))) return ELUTQ_ERR_NULL;
    const size_t dense = elutq_hlq_workspace_bytes(K, N, bits, group, M);
    if (!dense) return bits < 1 || bits > 4 ? ELUTQ_ERR_BITS : ELUTQ_ERR_SHAPE;
    if (workspace_bytes < elutq_hlq_sparse_workspace_bytes(K, N, bits, group, M)) return ELUTQ_ERR_WORKSPACE;
    float *extra = (float *)((unsigned char *)d_workspace + align256(dense));
    const SparseArgs a = sparse_args(d_blocks, d_blk_scales, d_index, nblk, K, N);
    const hipStream_t st = (hipStream_t)stream;
    if (M == 1) {
        rc = launch_sparse_plane(a, d_x, extra, 1, group, st);
        if (rc != ELUTQ_OK) return rc;
        return hlq_gemv_with_extra(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace, dense,
                                   stream, nullptr, 0, 0, extra);
    }
    // chunks of up to HLQ_GEMM_MAX_M rows share the staging area: the stream orders them
    for (int m0 = 0; m0 < M;) {
        const int mc = M - m0 < HLQ_GEMM_MAX_M ? M - m0 : HLQ_GEMM_MAX_M;
        const uint16_t *xc = (const uint16_t *)d_x + (size_t)m0 * K;
        rc = launch_sparse_plane(a, xc, extra, mc, group, st);
        if (rc != ELUTQ_OK) return rc;
        rc = hlq_gemm_chunk_with_extra(d_planes, d_scales, d_zeros, d_bias, xc, (uint16_t *)d_y + (size_t)m0 * N, mc, K, N,
                                       bits, group, d_workspace, dense, stream, 0, 0, extra);
        if (rc != ELUTQ_OK) return rc;
        m0 += mc;
    }
    return ELUTQ_OK;
}

int elutq_hlq_sparse_gemv_fused_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                    const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                                    const void *d_x, void *d_y, int K, int N, int bits, int group,
                                    void *d_workspace, size_t workspace_bytes, void *stream,
                                    const elutq_gemv_fusion *fusion, int ksplit, int waves)
{
    int rc = check_sparse_call(K, N, group, nblk);
    if (rc != ELUTQ_OK) return rc;
    if (!d_index || !d_x || !d_y || !d_workspace || (nblk && (!d_blocks || !d_blk_scales))) return ELUTQ_ERR_NULL;
    const size_t dense = elutq_hlq_workspace_bytes(K, N, bits, group, 1);
    if (!dense) return bits < 1 || bits > 4 ? ELUTQ_ERR_BITS : ELUTQ_ERR_SHAPE;
    if (workspace_bytes < elutq_hlq_sparse_workspace_bytes(K, N, bits, group, 1)) return ELUTQ_ERR_WORKSPACE;
    SparseArgs a = sparse_args(d_blocks, d_blk_scales, d_index, nblk, K, N);
    if (fusion) {
        // the plane reads the projection's input from the vectors the call names: K slices handed over by another
        // launch, or left to one, are not among them
        if (fusion->d_slices_out || fusion->n_slices_in != 0 || fusion->d_slices_in) return ELUTQ_ERR_TUNING;
        if (fusion->prologue < 0 || fusion->prologue > 2) return ELUTQ_ERR_TUNING;
        if (fusion->prologue == 1 && !fusion->d_norm_weight) return ELUTQ_ERR_NULL;
        a.prologue = fusion->prologue;
        a.eps = fusion->eps;
        a.norm_w = (const uint16_t *)fusion->d_norm_weight;
    }
    float *extra = (float *)((unsigned char *)d_workspace + align256(dense));
    rc = launch_sparse_plane(a, d_x, extra, 1, group, (hipStream_t)stream);
    if (rc != ELUTQ_OK) return rc;
    return hlq_gemv_with_extra(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace, dense,
                               stream, fusion, ksplit, waves, extra);
}

// ---- the inline form of a plane: blocks looked up inside the dense GEMV launch ------------------------------------
size_t elutq_hlq_sparse_inline_bytes(int K, int N, int group, int nblk)
{
    if (check_sparse_call(K, N, group, nblk) != ELUTQ_OK) return 0;
    const HlqGeo g = hlq_geo(K, N, 1, group);
    return hlq_sp_recs_offset(g.ncb, g.U) + (size_t)nblk * HLQ_SP_REC_BYTES;
}

int elutq_hlq_sparse_inline_host(const uint32_t *h_mask, int mask_len, const void *h_blocks, const void *h_blk_scales,
                                 int K, int N, int group, void *h_out, size_t *bytes_used)
{
    if (mask_len < 0 || mask_len % 2) return ELUTQ_ERR_SPARSE;
    const int nblk = mask_len / 2;
    int rc = check_sparse_call(K, N, group, nblk);
    if (rc != ELUTQ_OK) return rc;
    if (!h_out || (nblk && (!h_mask || !h_blocks || !h_blk_scales))) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, 1, group);
    const size_t recs_off = hlq_sp_recs_offset(g.ncb, g.U);
    int32_t *head = (int32_t *)h_out, *cells = (int32_t *)((unsigned char *)h_out + HLQ_SP_HEAD_BYTES);
    unsigned char *recs = (unsigned char *)h_out + recs_off;
    memset(h_out, 0, recs_off);
    for (size_t i = 0; i < (size_t)g.ncb * g.U; i++) cells[i] = -1;
    std::vector<unsigned char> taken;                 // per record: which (channel half, 64-k half) quarters hold a block
    const int bpr = group / 8;                        // bytes per channel of a block
    int nrec = 0;
    for (int i = 0; i < nblk; i++) {
        const uint32_t c = h_mask[2 * i], k = h_mask[2 * i + 1];
        // the inline form needs the blocks on the grid of the quantization groups: anything else keeps the block form
        if (c % SP_TILE || c >= (uint32_t)N || k % (uint32_t)group || (uint64_t)k + (uint32_t)group > (uint32_t)K)
            return ELUTQ_ERR_SPARSE;
        const int cb = (int)(c / HLQ_CB), half = (int)(c / SP_TILE) & 1, u = (int)(k / HLQ_UNIT), g2 = (int)(k % HLQ_UNIT) / 64;
        int32_t &cell = cells[(size_t)cb * g.U + u];
        if (cell < 0) {
            cell = nrec++;
            memset(recs + (size_t)cell * HLQ_SP_REC_BYTES, 0, HLQ_SP_REC_BYTES);
            taken.push_back(0);
        }
        const unsigned char quarters = group == 128 ? (unsigned char)(3u << (2 * half)) : (unsigned char)(1u << (2 * half + g2));
        if (taken[cell] & quarters) return ELUTQ_ERR_SPARSE;          // two blocks on one cell
        taken[cell] |= quarters;
        uint32_t *w = (uint32_t *)(recs + (size_t)cell * HLQ_SP_REC_BYTES);
        uint32_t *sc = w + HLQ_CB * 4;
        for (int r = 0; r < SP_TILE; r++) {
            const int lane = SP_TILE * half + r;
            const unsigned char *src = (const unsigned char *)h_blocks + ((size_t)i * SP_TILE + r) * bpr;
            for (int d = 0; d < bpr / 4; d++) {
                uint32_t v;
                memcpy(&v, src + 4 * d, 4);                            // little-endian dword: bit j <-> k = 32 d + j of the block
                v = (v << HLQ_ROT) | (v >> (32 - HLQ_ROT));
                w[lane * 4 + (group == 128 ? d : 2 * g2 + d)] = v;
            }
            const uint32_t s = ((const uint16_t *)h_blk_scales)[(size_t)i * SP_TILE + r];
            if (group == 128) sc[lane] = s | (s << 16);
            else sc[lane] |= s << (16 * g2);
        }
    }
    head[0] = HLQ_SP_MAGIC; head[1] = K; head[2] = N; head[3] = group; head[4] = g.U; head[5] = g.ncb; head[6] = nrec; head[7] = 0;
    if (bytes_used) *bytes_used = recs_off + (size_t)nrec * HLQ_SP_REC_BYTES;
    return ELUTQ_OK;
}

int elutq_hlq_sparse_gemv_inline_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                     const void *d_inline, size_t inline_bytes, const void *d_x, void *d_y, int K, int N,
                                     int bits, int group, void *d_workspace, size_t workspace_bytes, void *stream,
                                     const elutq_gemv_fusion *fusion, int ksplit, int waves)
{
    if (bits > 3) return ELUTQ_ERR_BITS;              // the extra plane is the layer's fourth at most
    return hlq_gemv_with_inline_sparse(d_planes, d_scales, d_zeros, d_bias, d_inline, inline_bytes, d_x, d_y, K, N, bits, group,
                                       d_workspace, workspace_bytes, stream, fusion, ksplit, waves);
}

int elutq_hlq_sparse_gemv_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                              const void *d_x, void *d_y, int K, int N, int bits, int group,
                              void *d_workspace, size_t workspace_bytes, void *stream)
{
    return elutq_hlq_sparse_gemm_f16(d_planes, d_scales, d_zeros, d_bias, d_blocks, d_blk_scales, d_index, nblk, d_x, d_y,
                                     1, K, N, bits, group, d_workspace, workspace_bytes, stream);
}

int elutq_hlq_sparse_dequant_add_f16(const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                                     void *d_w, int K, int N, int group, void *stream)
{
    int rc = check_sparse_call(K, N, group, nblk);
    if (rc != ELUTQ_OK) return rc;
    if (!d_index || !d_w || (nblk && (!d_blocks || !d_blk_scales))) return ELUTQ_ERR_NULL;
    if (nblk == 0) return ELUTQ_OK;
    SparseArgs a = sparse_args(d_blocks, d_blk_scales, d_index, nblk, K, N);
    a.w = (uint16_t *)d_w;
    if (group == 64)
        hipLaunchKernelGGL(hlq_sparse_dequant_kernel<64>, dim3(sp_tiles(N)), dim3(SP_THREADS), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL(hlq_sparse_dequant_kernel<128>, dim3(sp_tiles(N)), dim3(SP_THREADS), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

}  // extern "C"

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
// The block bits and scales stay exactly as the files hold them -- [block][32 channels][G/8
// bytes] is already what a wave wants: 8 consecutive lanes own the 8 k-eighths of one channel, so a
// block is one contiguous 32*G/8-byte read -- and the pair list becomes an index by channel tile.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"

namespace {

constexpr int SP_TILE = 32;        // channels per block
constexpr int SP_PARTS = 8;        // lanes that share a channel: each owns G/8 consecutive k
constexpr int SP_THREADS = SP_TILE * SP_PARTS;

inline int sp_tiles(int N) { return (N + SP_TILE - 1) / SP_TILE; }

struct SparseArgs {
    const uint8_t *blocks;         // [nblk][32][G/8]
    const uint16_t *blk_scales;    // fp16 [nblk][32]
    const int32_t *tile_ptr;       // [tiles + 1]: blocks of tile t are tile_ptr[t] .. tile_ptr[t+1]-1
    const int32_t *blk_k;          // [nblk] k start
    const uint16_t *x;             // fp16 [M][K]
    float *extra;                  // fp32 [M][N], written for every (m, n)
    uint16_t *w;                   // fp16 [N][K] (dequantisation only)
    int M, K, N, nblk;
};

__device__ __forceinline__ float hf(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
__device__ __forceinline__ uint16_t fh(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

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
                    for (int j = 0; j < 4; j++)
                        if (bits[i] >> (4 * q + j) & 1u) sum += hf(h[j]);
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
    a.K = K; a.N = N; a.nblk = nblk;
    return a;
}

// The plane's term for rows x[0..M) into extra[M][N].
int launch_sparse_plane(SparseArgs a, const void *d_x, float *d_extra, int M, int group, hipStream_t stream)
{
    a.x = (const uint16_t *)d_x;
    a.extra = d_extra;
    a.M = M;
    const int rows = M == 1 ? 1 : 4;
    const dim3 grid(sp_tiles(a.N), (M + rows - 1) / rows);
    if (M == 1) {
        if (group == 64) hipLaunchKernelGGL((hlq_sparse_plane_kernel<64, 1, 4>), grid, dim3(SP_THREADS), 0, stream, a);
        else hipLaunchKernelGGL((hlq_sparse_plane_kernel<128, 1, 4>), grid, dim3(SP_THREADS), 0, stream, a);
    } else {
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
    return sizeof(int32_t) * ((size_t)sp_tiles(N) + 1 + (size_t)nblk);
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

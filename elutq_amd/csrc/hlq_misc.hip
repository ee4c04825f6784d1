// Version / status strings and the dense dequantisation kernel
// (dequantize_with_scales, GPTQ/quant.py:176-183) on the repacked layout.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_gemv_dev.h"

namespace {

struct DequantArgs {
    const uint4 *planes;
    const uint32_t *scales;
    const uint32_t *zeros;
    uint16_t *w;     // fp16 [N][K]
    int N, K, U, NT, bits, g64;
};

__device__ __forceinline__ float h2f(uint32_t v, int hi) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? v >> 16 : v & 0xffffu)); }

// One wave per (column block, unit): lane = column, writes 128 fp16 of its row.
__global__ __launch_bounds__(64) void hlq_dequant_kernel(const DequantArgs a)
{
    const int lane = threadIdx.x;
    const int u = blockIdx.x % a.U, cb = blockIdx.x / a.U;
    const int n = cb * HLQ_CB + lane;
    if (n >= a.N) return;
    uint32_t bitsw[4][4];
    for (int b = 0; b < a.bits; b++) {
        const uint4 v = a.planes[(((size_t)cb * a.U + u) * a.bits + b) * HLQ_CB + lane];
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
        for (int i = 0; i < 4; i++) bitsw[b][i] = (d[i] >> HLQ_ROT) | (d[i] << (32 - HLQ_ROT));
    }
    uint16_t *dst = a.w + (size_t)n * a.K + (size_t)u * HLQ_UNIT;
    const int nk = min(HLQ_UNIT, a.K - u * HLQ_UNIT);             // 64 in a last unit that K ends half way through
    for (int i = 0; i < nk; i++) {
        // group of this k and where its scale sits: task t = g / 2, half = g & 1
        const int g = a.g64 ? 2 * u + (i >> 6) : u;
        const int t = g >> 1, hi = g & 1;
        float v = h2f(a.zeros[((size_t)cb * a.NT + t) * HLQ_CB + lane], hi);
        for (int b = 0; b < a.bits; b++)
            if (bitsw[b][i >> 5] >> (i & 31) & 1u)
                v += h2f(a.scales[(((size_t)cb * a.NT + t) * a.bits + b) * HLQ_CB + lane], hi);
        dst[i] = __builtin_bit_cast(uint16_t, (_Float16)v);
    }
}

// Measurement aid: every wave does nothing but 16-entry table lookups (ds_read_b32, one table per read, the 16 entries
// on 16 banks, equal entries broadcast -- the access pattern of the LUT GEMV), 16 per loop pass, so that the time of a
// launch divided by the wave instructions of one compute unit is the rate at which a compute unit retires them.
__global__ __launch_bounds__(1024) void lds_lookup_rate_kernel(int passes, uint32_t *out)
{
    __shared__ uint32_t tbl[16 * 16 * 16];                 // 16 waves x 16 tables x 16 entries
    for (int i = threadIdx.x; i < 16 * 16 * 16; i += blockDim.x) tbl[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // one address register per pass (entry (7 lane + wave) % 16 of the wave's first table), the 16 tables by
    // instruction offset: a pass is 16 reads and 8 three-operand adds, so that the reads are what the time is made of
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t *)tbl +
                          (uint32_t)(wave * 16 * 16 + ((lane * 7 + wave) & 15)) * 4u;
    uint32_t acc = 0;
    for (int p = 0; p < passes; p++) {
        uint32_t v[16];
        asm volatile("ds_read_b32 %0, %16\n\tds_read_b32 %1, %16 offset:64\n\tds_read_b32 %2, %16 offset:128\n\t"
                     "ds_read_b32 %3, %16 offset:192\n\tds_read_b32 %4, %16 offset:256\n\tds_read_b32 %5, %16 offset:320\n\t"
                     "ds_read_b32 %6, %16 offset:384\n\tds_read_b32 %7, %16 offset:448\n\tds_read_b32 %8, %16 offset:512\n\t"
                     "ds_read_b32 %9, %16 offset:576\n\tds_read_b32 %10, %16 offset:640\n\tds_read_b32 %11, %16 offset:704\n\t"
                     "ds_read_b32 %12, %16 offset:768\n\tds_read_b32 %13, %16 offset:832\n\tds_read_b32 %14, %16 offset:896\n\t"
                     "ds_read_b32 %15, %16 offset:960\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]),
                       "=&v"(v[8]), "=&v"(v[9]), "=&v"(v[10]), "=&v"(v[11]), "=&v"(v[12]), "=&v"(v[13]), "=&v"(v[14]), "=&v"(v[15])
                     : "v"(addr)
                     : "memory");
#pragma unroll
        for (int j = 0; j < 16; j += 2) acc += v[j] + v[j + 1];
    }
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// The same measurement on the LUT GEMV's own instruction sequence: process_sub (address formation by SDWA, 32 lookups,
// integer sums, conversion and two multiply-adds per sub-task) on plane words held in registers and tables that are
// already in LDS -- what the sequence reaches when it never waits for memory.  16 lookups per pass, like the kernel above.
__global__ __launch_bounds__(1024) void lut_sequence_rate_kernel(int passes, uint32_t *out)
{
    __shared__ __align__(16) unsigned char smem[16 * 2 * UNIT_LUT_BYTES + 64 * sizeof(float2)];
    for (int i = threadIdx.x; i < 16 * 2 * UNIT_LUT_BYTES / 4; i += blockDim.x) ((int *)smem)[i] = i & 1023;
    float2 *xs_inv = (float2 *)(smem + 16 * 2 * UNIT_LUT_BYTES);
    if (threadIdx.x < 64) xs_inv[threadIdx.x] = make_float2(1.f, 1.f);
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lut_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem + wave * 2 * UNIT_LUT_BYTES;
    uint4 w = make_uint4(lane * 2654435761u, lane * 40503u + 7u, lane * 69069u + 1u, lane * 1103515245u);
    float acc = 0.f;
    for (int p = 0; p < passes; p += 2) {           // a sub-task is 32 lookups = two passes
        acc = process_sub<false>(w, 0x3c003c00u, 0x3c003c00u, (p >> 1) & 1, (p >> 1) & 1, 0, lut_base, xs_inv + 4 * wave, acc);
        w.x += 0x01010101u; w.y ^= w.x; w.z += 0x11111111u; w.w ^= w.z;
    }
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = __float_as_uint(acc);
}

}  // namespace

extern "C" {

int elutq_diag_lds_lookup_rate(int sequence, int waves, int passes, void *d_out, void *stream)
{
    if (waves < 1 || (waves > 16 && waves != 32) || passes < 2 || passes % 2 || sequence < 0 || sequence > 1) return ELUTQ_ERR_TUNING;
    if (!d_out) return ELUTQ_ERR_NULL;
    // 32: two workgroups of 16 wavefronts per compute unit
    const int per_cu = waves == 32 ? 2 : 1;
    const dim3 grid(HLQ_NUM_CU * per_cu), block(waves / per_cu * 64);
    if (sequence) hipLaunchKernelGGL(lut_sequence_rate_kernel, grid, block, 0, (hipStream_t)stream, passes, (uint32_t *)d_out);
    else hipLaunchKernelGGL(lds_lookup_rate_kernel, grid, block, 0, (hipStream_t)stream, passes, (uint32_t *)d_out);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

int elutq_version(void) { return 100; }

const char *elutq_status_string(int status)
{
    switch (status) {
    case ELUTQ_OK: return "ok";
    case ELUTQ_ERR_NULL: return "a required pointer is NULL";
    case ELUTQ_ERR_SHAPE: return "unsupported shape: need K >= 128, K % group == 0 and K % 128 == 0 (or 64 at group 64), N >= 1, M >= 1";
    case ELUTQ_ERR_BITS: return "bits must be 1..4";
    case ELUTQ_ERR_GROUP: return "group must be 64 or 128";
    case ELUTQ_ERR_WORKSPACE: return "workspace smaller than elutq_hlq_workspace_bytes()";
    case ELUTQ_ERR_HIP: return "a HIP runtime call failed";
    case ELUTQ_ERR_TUNING: return "ksplit / waves out of range";
    case ELUTQ_ERR_SPARSE:
        return "malformed sparse block list: need (channel start, k start) pairs, channel start a multiple of 32 below N "
               "and ascending, k start a multiple of 4 with k + group <= K";
    case ELUTQ_ERR_STATIC_LIMIT:
        return "the shape needs more partial-sum scratch than the static buffer holds (ELUTQ_STATIC_PARTIAL_BYTES): "
               "use elutq_hlq_gemv_f16 with a workspace";
    }
    return "unknown status";
}

int elutq_hlq_dequant_f16(const void *d_planes, const void *d_scales, const void *d_zeros, void *d_w_out, int K, int N,
                          int bits, int group, void *stream)
{
    if (bits < 1 || bits > 4) return ELUTQ_ERR_BITS;
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (N < 1 || !hlq_k_ok(K, group)) return ELUTQ_ERR_SHAPE;
    if (!d_planes || !d_scales || !d_zeros || !d_w_out) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    DequantArgs a;
    a.planes = (const uint4 *)d_planes;
    a.scales = (const uint32_t *)d_scales;
    a.zeros = (const uint32_t *)d_zeros;
    a.w = (uint16_t *)d_w_out;
    a.N = N; a.K = K; a.U = g.U; a.NT = g.NT; a.bits = bits; a.g64 = group == 64;
    hipLaunchKernelGGL(hlq_dequant_kernel, dim3(g.ncb * g.U), dim3(64), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

}  // extern "C"

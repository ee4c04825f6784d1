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

}  // namespace

extern "C" {

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

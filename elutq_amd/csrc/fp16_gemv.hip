// Dense fp16 GEMV for gfx950: y[n] = sum_k W[n][k] x[k] (+ bias[n]), the bit == 16 branch of arm_gemm
// (C++/ops/src/arm/arm_gemm.cpp:883-886; MultiThreadGemvFP::Run, :586-626, thread split :630-660) -- in a
// decode step the lm_head of an export whose lm_head was not quantized (lm_head.bin,
// C++/examples/models/llama.cpp:78; W is [vocab][hidden], 1 GB for LLaMA-3-8B).  Purely HBM bound: 2 bytes
// per multiply-add.
//
//  * a wave takes two rows at a time; a lane owns the same eight consecutive k of every 512-k stretch
//    (one dwordx4 per row and stretch), so a row is read in whole 1 KiB wave loads, and the sixteen loads of a
//    row pair over 4096 k are all issued before the first is used;
//  * the activations are staged once per workgroup in LDS (optionally through the RMSNorm of the decode
//    step's tail, launch_pre_rms_norm, C++/ops/src/arm/arm_rmsnorm.cpp:25-84: fp32 statistics, rounded to
//    fp16 as the unfused operator would store them) and read from there per stretch for both rows;
//  * products in fp32 (v_dot2_f32_f16), one wave-wide sum per row, one rounding to fp16.  The reference
//    accumulates in fp16 (eight partial sums per row); this is closer to the exact result.
//  * workgroups walk the row pairs with stride gridDim.x * waves, so neighbouring waves stream
//    neighbouring rows.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#if defined(__HIP_DEVICE_COMPILE__)
#define FP16_GLOBAL __attribute__((address_space(1)))
#else
#define FP16_GLOBAL
#endif

constexpr int DG_WAVES = 16;
constexpr int DG_SEG = 8;                       // stretches of 512 k a wave has in flight per row: 4096 k
constexpr int DG_MAX_K = 32768;                 // activations staged in LDS: 64 KiB

struct DenseArgs {
    const FP16_GLOBAL uint16_t *w;      // fp16 [N][K]
    const FP16_GLOBAL uint16_t *bias;   // fp16 [N] or null
    const FP16_GLOBAL uint16_t *x;      // fp16 [K]
    const FP16_GLOBAL uint16_t *norm_w; // fp16 [K] or null: x <- fp16(x * rsqrt(mean(x^2) + eps) * norm_w)
    FP16_GLOBAL uint16_t *y;            // fp16 [N]
    int N, K;
    float eps;
};

__device__ __forceinline__ float h2f(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f<0xB1>(v);            // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);            // quad_perm [2,3,0,1]
    v += dpp_f<0x141>(v);           // row_half_mirror
    v += dpp_f<0x140>(v);           // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float dot8(const uint4 &a, const uint4 &b, float acc)
{
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a.x), __builtin_bit_cast(half2v, b.x), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a.y), __builtin_bit_cast(half2v, b.y), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a.z), __builtin_bit_cast(half2v, b.z), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a.w), __builtin_bit_cast(half2v, b.w), acc, false);
    return acc;
}

__global__ __launch_bounds__(DG_WAVES * 64) void fp16_gemv_kernel(const DenseArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    uint16_t *xs = (uint16_t *)smem;                              // fp16 [K8]: the (normalised) activations, zero past K
    __shared__ float part[DG_WAVES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = a.K;
    const int stretches = (K + 511) / 512;                        // 512 k = one dwordx4 per lane
    const int K8 = stretches * 512;

    // activations into LDS, through the RMSNorm if there is one
    float rstd = 1.f;
    if (a.norm_w) {
        float ssq = 0.f;
        for (int i = tid; i < K; i += DG_WAVES * 64) {
            const float v = h2f(a.x[i]);
            ssq = fmaf(v, v, ssq);
        }
        ssq = wave_sum(ssq);
        if (lane == 0) part[wave] = ssq;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < DG_WAVES; i++) tot += part[i];
        rstd = rsqrtf(tot / (float)K + a.eps);
    }
    for (int i = tid; i < K8; i += DG_WAVES * 64) {
        uint16_t v = 0;
        if (i < K) {
            v = a.x[i];
            if (a.norm_w) v = __builtin_bit_cast(uint16_t, (_Float16)(h2f(v) * rstd * h2f(a.norm_w[i])));
        }
        xs[i] = v;
    }
    __syncthreads();

    const int pairs = (a.N + 1) / 2;
    const size_t row_bytes = (size_t)K * 2;
    const FP16_GLOBAL unsigned char *wb = (const FP16_GLOBAL unsigned char *)a.w;
    for (int p = blockIdx.x * DG_WAVES + wave; p < pairs; p += gridDim.x * DG_WAVES) {
        const int r0 = 2 * p, r1 = min(2 * p + 1, a.N - 1);      // an odd N: the last pair reads its row twice
        const FP16_GLOBAL unsigned char *w0 = wb + (size_t)r0 * row_bytes, *w1 = wb + (size_t)r1 * row_bytes;
        float acc0 = 0.f, acc1 = 0.f;
        for (int s0 = 0; s0 < stretches; s0 += DG_SEG) {
            u32x4 v0[DG_SEG], v1[DG_SEG];
            // every load of the segment before the first use; past K: the row's last 16 bytes again (x is zero there)
#pragma unroll
            for (int j = 0; j < DG_SEG; j++) {
                const uint32_t k = min((uint32_t)((s0 + j) * 512 + lane * 8), (uint32_t)(K - 8));
                v0[j] = __builtin_nontemporal_load((const FP16_GLOBAL u32x4 *)(w0 + k * 2));
                v1[j] = __builtin_nontemporal_load((const FP16_GLOBAL u32x4 *)(w1 + k * 2));
            }
#pragma unroll
            for (int j = 0; j < DG_SEG; j++) {
                const int st = min(s0 + j, stretches - 1);
                uint4 xv = *(const uint4 *)(xs + st * 512 + lane * 8);
                if (s0 + j >= stretches) xv = make_uint4(0u, 0u, 0u, 0u);
                acc0 = dot8(make_uint4(v0[j].x, v0[j].y, v0[j].z, v0[j].w), xv, acc0);
                acc1 = dot8(make_uint4(v1[j].x, v1[j].y, v1[j].z, v1[j].w), xv, acc1);
            }
        }
        acc0 = wave_sum(acc0);
        acc1 = wave_sum(acc1);
        if (lane == 0) {
            if (a.bias) { acc0 += h2f(a.bias[r0]); acc1 += h2f(a.bias[r1]); }
            a.y[r0] = __builtin_bit_cast(uint16_t, (_Float16)acc0);
            if (2 * p + 1 < a.N) a.y[r1] = __builtin_bit_cast(uint16_t, (_Float16)acc1);
        }
    }
}

}  // namespace

extern "C" int elutq_fp16_gemv_f16(const void *d_weight, const void *d_bias, const void *d_x, void *d_y, int K, int N,
                                   const void *d_norm_weight, float eps, void *stream)
{
    if (!d_weight || !d_x || !d_y) return ELUTQ_ERR_NULL;
    if (K < 8 || K % 8 != 0 || K > DG_MAX_K || N < 1 || ((uintptr_t)d_weight & 15) != 0) return ELUTQ_ERR_SHAPE;
    DenseArgs a;
    a.w = (const FP16_GLOBAL uint16_t *)d_weight;
    a.bias = (const FP16_GLOBAL uint16_t *)d_bias;
    a.x = (const FP16_GLOBAL uint16_t *)d_x;
    a.norm_w = (const FP16_GLOBAL uint16_t *)d_norm_weight;
    a.y = (FP16_GLOBAL uint16_t *)d_y;
    a.N = N; a.K = K; a.eps = eps;
    const int pairs = (N + 1) / 2;
    const size_t lds = (size_t)((K + 511) / 512) * 512 * 2;
    // as many workgroups as the chip holds at once walk the rows
    int per_cu = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)fp16_gemv_kernel, DG_WAVES * 64, lds) != hipSuccess ||
        per_cu < 1)
        per_cu = 1;
    int grid = (pairs + DG_WAVES - 1) / DG_WAVES;
    if (grid > per_cu * HLQ_NUM_CU) grid = per_cu * HLQ_NUM_CU;
    hipLaunchKernelGGL(fp16_gemv_kernel, dim3(grid), dim3(DG_WAVES * 64), lds, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

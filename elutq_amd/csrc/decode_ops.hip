// Glue of a batch-1 decode step around the HLQ projections, as one kernel per layer:
// RoPE on q and k, KV-cache append, single-token GQA attention.  Counterparts in the
// reference runtime: launch_llama_qkv_apply_rotary (C++/ops/src/arm/arm_rotary.cpp:4-89,
// half-split pairs (j, j + d/2), theta = pos * base^(-2j/d), no frequency rescaling),
// arm_cache (C++/ops/src/arm/arm_cache.cpp:17-22, cache [pos][kv head][d] fp16) and the
// single-token branch of arm_attention (C++/ops/src/arm/arm_attention.cpp:162-316: fp32
// softmax, GQA map h_kv = h * n_kv / n_q).  Scores and the P.V sum are kept in fp32 here.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"

namespace {

struct AttnArgs {
    const uint16_t *qkv;     // fp16 [nq*d | nkv*d | nkv*d]
    uint16_t *kc, *vc;       // fp16 [max_seq][nkv][d]
    const long long *pos;    // device scalar: index of the token being decoded
    uint16_t *out;           // fp16 [nq*d]
    int nq, nkv, d, max_seq;
    float log2_base;
};

__device__ __forceinline__ float h2f(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
__device__ __forceinline__ uint16_t f2h(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ float r16(float v) { return (float)(_Float16)v; }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

constexpr int ATTN_WAVES = 4;
constexpr int ATTN_UNROLL = 4;

// One workgroup per query head; lane j owns the rotary pair (j, j + d/2); the waves split
// the cached positions and are merged with the usual running-max softmax algebra.
__global__ __launch_bounds__(ATTN_WAVES * 64) void rope_attn_kernel(const AttnArgs a)
{
    __shared__ float sm_m[ATTN_WAVES], sm_l[ATTN_WAVES];
    __shared__ float sm_o[ATTN_WAVES][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.x, grp = a.nq / a.nkv, g = h / grp;
    const int d = a.d, half = d >> 1;
    const int j = lane < half ? lane : 0;
    const bool active = lane < half;
    const int pos = (int)*a.pos;
    if (pos < 0 || pos >= a.max_seq) return;      // outside the cache: nothing is read or written

    const float inv_freq = exp2f(-(float)(2 * j) / (float)d * a.log2_base);
    float sn, cs;
    sincosf((float)pos * inv_freq, &sn, &cs);
    const uint16_t *qp = a.qkv + (size_t)h * d, *kp = a.qkv + (size_t)a.nq * d + (size_t)g * d;
    const uint16_t *vp = a.qkv + (size_t)(a.nq + a.nkv) * d + (size_t)g * d;
    const float qa = h2f(qp[j]), qb = h2f(qp[j + half]), ka = h2f(kp[j]), kb = h2f(kp[j + half]);
    const float scale = rsqrtf((float)d);
    const float q0 = active ? r16(qa * cs - qb * sn) * scale : 0.f, q1 = active ? r16(qb * cs + qa * sn) * scale : 0.f;
    const uint16_t k0h = f2h(ka * cs - kb * sn), k1h = f2h(kb * cs + ka * sn);
    const uint16_t v0h = vp[j], v1h = vp[j + half];
    if (h % grp == 0 && wave == 0 && active) {
        const size_t row = ((size_t)pos * a.nkv + g) * d;
        a.kc[row + j] = k0h; a.kc[row + j + half] = k1h;
        a.vc[row + j] = v0h; a.vc[row + j + half] = v1h;
    }

    float m = -INFINITY, l = 0.f, o0 = 0.f, o1 = 0.f;
    for (int p = wave * ATTN_UNROLL; p < pos; p += ATTN_WAVES * ATTN_UNROLL) {
        float s[ATTN_UNROLL], va[ATTN_UNROLL], vb[ATTN_UNROLL];
#pragma unroll
        for (int u = 0; u < ATTN_UNROLL; u++) {
            const int pp = min(p + u, pos - 1);
            const size_t row = ((size_t)pp * a.nkv + g) * d;
            s[u] = q0 * h2f(a.kc[row + j]) + q1 * h2f(a.kc[row + j + half]);
            va[u] = h2f(a.vc[row + j]);
            vb[u] = h2f(a.vc[row + j + half]);
        }
        float mx = m;
#pragma unroll
        for (int u = 0; u < ATTN_UNROLL; u++) {
            s[u] = wave_sum(s[u]);
            if (p + u >= pos) s[u] = -INFINITY;
            mx = fmaxf(mx, s[u]);
        }
        const float corr = __expf(m - mx);
        l *= corr; o0 *= corr; o1 *= corr;
#pragma unroll
        for (int u = 0; u < ATTN_UNROLL; u++) {
            const float e = __expf(s[u] - mx);
            l += e; o0 = fmaf(e, va[u], o0); o1 = fmaf(e, vb[u], o1);
        }
        m = mx;
    }
    if (wave == 0) {                         // the token being decoded attends to itself from registers
        const float s = wave_sum(q0 * h2f(k0h) + q1 * h2f(k1h));
        const float mx = fmaxf(m, s), corr = __expf(m - mx), e = __expf(s - mx);
        l = l * corr + e;
        o0 = fmaf(e, h2f(v0h), o0 * corr);
        o1 = fmaf(e, h2f(v1h), o1 * corr);
        m = mx;
    }
    if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    if (active) { sm_o[wave][j] = o0; sm_o[wave][j + half] = o1; }
    __syncthreads();
    if (wave == 0 && active) {
        float M = sm_m[0];
#pragma unroll
        for (int w = 1; w < ATTN_WAVES; w++) M = fmaxf(M, sm_m[w]);
        float L = 0.f, r0 = 0.f, r1 = 0.f;
#pragma unroll
        for (int w = 0; w < ATTN_WAVES; w++) {
            const float f = __expf(sm_m[w] - M);
            L = fmaf(sm_l[w], f, L);
            r0 = fmaf(sm_o[w][j], f, r0);
            r1 = fmaf(sm_o[w][j + half], f, r1);
        }
        a.out[(size_t)h * d + j] = f2h(r0 / L);
        a.out[(size_t)h * d + j + half] = f2h(r1 / L);
    }
}

}  // namespace

extern "C" int elutq_decode_rope_attn_f16(const void *d_qkv, void *d_k_cache, void *d_v_cache, const void *d_pos,
                                          void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                          float rope_base, void *stream)
{
    if (!d_qkv || !d_k_cache || !d_v_cache || !d_pos || !d_out) return ELUTQ_ERR_NULL;
    if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || head_dim < 2 || head_dim > 128 ||
        head_dim % 2 != 0 || max_seq < 1 || !(rope_base > 1.f))
        return ELUTQ_ERR_SHAPE;
    AttnArgs a;
    a.qkv = (const uint16_t *)d_qkv;
    a.kc = (uint16_t *)d_k_cache;
    a.vc = (uint16_t *)d_v_cache;
    a.pos = (const long long *)d_pos;
    a.out = (uint16_t *)d_out;
    a.nq = n_heads; a.nkv = n_kv_heads; a.d = head_dim; a.max_seq = max_seq;
    a.log2_base = log2f(rope_base);
    hipLaunchKernelGGL(rope_attn_kernel, dim3(n_heads), dim3(ATTN_WAVES * 64), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

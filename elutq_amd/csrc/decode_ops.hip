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
    __sincosf((float)pos * inv_freq, &sn, &cs);
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


// ---------------------------------------------------------------------------------------
// head_dim 128: coalesced variant.  A wave instruction covers 4 cache rows x 16 segments of
// 8 dims (one dwordx4 per lane, 1 KiB contiguous per kv head row group); the 16 lanes of a
// DPP row reduce their partial dot products among themselves, so no LDS permutes are
// needed, and every (wave, row) pair runs its own running-max softmax stream over the
// positions it sees.  Batches of FAST_BATCH row groups are loaded before any is used.
// ---------------------------------------------------------------------------------------
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
constexpr int FAST_WAVES = 8;
constexpr int FAST_BATCH = 8;
constexpr int FAST_D = 128;

__device__ __forceinline__ float dot8(const uint4 &q, const uint4 &k)
{
    float s = 0.f;
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, q.x), __builtin_bit_cast(half2v, k.x), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, q.y), __builtin_bit_cast(half2v, k.y), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, q.z), __builtin_bit_cast(half2v, k.z), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, q.w), __builtin_bit_cast(half2v, k.w), s, false);
    s += dpp_f<0xB1>(s);
    s += dpp_f<0x4E>(s);
    s += dpp_f<0x141>(s);
    s += dpp_f<0x140>(s);
    return s;
}

__device__ __forceinline__ void stream_update(float s, bool valid, const uint4 &v, float &m, float &l, float (&acc)[8])
{
    const float mx = valid ? fmaxf(m, s) : m;
    const float corr = (m == mx) ? 1.f : __expf(m - mx);
    const float e = valid ? __expf(s - mx) : 0.f;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    l = fmaf(l, corr, e);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        acc[2 * i] = fmaf(e, h2f((uint16_t)(w[i] & 0xffffu)), acc[2 * i] * corr);
        acc[2 * i + 1] = fmaf(e, h2f((uint16_t)(w[i] >> 16)), acc[2 * i + 1] * corr);
    }
    m = mx;
}

__global__ __launch_bounds__(FAST_WAVES * 64) void rope_attn_d128_kernel(const AttnArgs a)
{
    constexpr int D = FAST_D, HALF = D / 2, STREAMS = FAST_WAVES * 4;
    __shared__ __align__(16) uint16_t sq[D], sk[D], sv[D];
    __shared__ float sm_m[STREAMS], sm_l[STREAMS];
    __shared__ float sm_o[STREAMS][D];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = blockIdx.x, grp = a.nq / a.nkv, g = h / grp;
    const int pos = (int)*a.pos;
    if (pos < 0 || pos >= a.max_seq) return;

    if (tid < HALF) {                                    // rotary pair (tid, tid + 64) of q and of the new k
        const int j = tid;
        const float inv_freq = exp2f(-(float)(2 * j) / (float)D * a.log2_base);
        float sn, cs;
        __sincosf((float)pos * inv_freq, &sn, &cs);
        const uint16_t *qp = a.qkv + (size_t)h * D, *kp = a.qkv + (size_t)a.nq * D + (size_t)g * D;
        const uint16_t *vp = a.qkv + (size_t)(a.nq + a.nkv) * D + (size_t)g * D;
        const float qa = h2f(qp[j]), qb = h2f(qp[j + HALF]), ka = h2f(kp[j]), kb = h2f(kp[j + HALF]);
        sq[j] = f2h(qa * cs - qb * sn); sq[j + HALF] = f2h(qb * cs + qa * sn);
        sk[j] = f2h(ka * cs - kb * sn); sk[j + HALF] = f2h(kb * cs + ka * sn);
        sv[j] = vp[j]; sv[j + HALF] = vp[j + HALF];
    }
    __syncthreads();
    if (h % grp == 0 && tid < D / 8) {                   // one workgroup per kv head appends the new row
        const size_t row = ((size_t)pos * a.nkv + g) * D;
        ((uint4 *)(a.kc + row))[tid] = ((const uint4 *)sk)[tid];
        ((uint4 *)(a.vc + row))[tid] = ((const uint4 *)sv)[tid];
    }

    const int seg = lane & 15, r = lane >> 4;
    const uint4 qv = ((const uint4 *)sq)[seg];
    const float scale = rsqrtf((float)D);
    const int ngroups = (pos + 3) >> 2;                  // row groups of the cached positions 0..pos-1
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;

    for (int gb = wave; gb < ngroups; gb += FAST_WAVES * FAST_BATCH) {
        uint4 kk[FAST_BATCH], vv[FAST_BATCH];
        bool ok[FAST_BATCH];
#pragma unroll
        for (int b = 0; b < FAST_BATCH; b++) {
            const int p = (gb + FAST_WAVES * b) * 4 + r;
            ok[b] = p < pos;
            const size_t row = ((size_t)(ok[b] ? p : 0) * a.nkv + g) * D;
            kk[b] = ((const uint4 *)(a.kc + row))[seg];
            vv[b] = ((const uint4 *)(a.vc + row))[seg];
        }
        // keep the whole batch of loads ahead of the first use (the scheduler would otherwise
        // sink each load to its consumer and serialise the memory round trips)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < FAST_BATCH; b++) {
            const float s = dot8(qv, kk[b]) * scale;
            stream_update(s, ok[b], vv[b], m, l, acc);
        }
    }
    if (wave == 0) {                                     // the token being decoded, from LDS (row 0 only)
        const float s = dot8(qv, ((const uint4 *)sk)[seg]) * scale;
        stream_update(s, r == 0, ((const uint4 *)sv)[seg], m, l, acc);
    }
    const int stream = wave * 4 + r;
    if (seg == 0) { sm_m[stream] = m; sm_l[stream] = l; }
#pragma unroll
    for (int i = 0; i < 8; i++) sm_o[stream][seg * 8 + i] = acc[i];
    __syncthreads();
    if (tid < D) {
        float M = -INFINITY;
#pragma unroll
        for (int s = 0; s < STREAMS; s++) M = fmaxf(M, sm_m[s]);
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS; s++) {
            const float f = __expf(sm_m[s] - M);
            L = fmaf(sm_l[s], f, L);
            o = fmaf(sm_o[s][tid], f, o);
        }
        a.out[(size_t)h * D + tid] = f2h(o / L);
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
    if (head_dim == FAST_D)
        hipLaunchKernelGGL(rope_attn_d128_kernel, dim3(n_heads), dim3(FAST_WAVES * 64), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL(rope_attn_kernel, dim3(n_heads), dim3(ATTN_WAVES * 64), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

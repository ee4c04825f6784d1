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
#include "hlq_layout.h"

namespace {

struct AttnArgs {
    const uint16_t *qkv;     // fp16 [nq*d | nkv*d | nkv*d]
    uint16_t *kc, *vc;       // fp16 [max_seq][nkv][d]
    const long long *pos;    // device scalar: index of the token being decoded
    uint16_t *out;           // fp16 [nq*d]
    int nq, nkv, d, max_seq;
    float log2_base;
    int splits;              // workgroups per query head (head_dim 128 only)
    float *partial;          // [nq][splits][d + 2] unnormalised output, running max, running sum
    unsigned *counters;      // [nq] arrival counters, zero between launches
    const float *qkv_slices; // fp32 [n_qkv_slices][qkv_stride]: the q|k|v projection's K slices, unsummed, or null
    int n_qkv_slices, qkv_stride;
};

constexpr int ATTN_MAX_SPLITS = 8;
constexpr int ATTN_MAX_QKV_SLICES = 4;

// The six q|k|v elements a lane needs (indices idx[]): as stored (fp16), or fp16(((s0[i] + s1[i]) + ...))
// where the projection left its K slices unsummed -- the value its own output stage would have stored.
// One branch, then all loads of the taken side before the first use (ATTN_MAX_QKV_SLICES per element in
// the second case, the last slice repeated, none of them conditional).
__device__ __forceinline__ void qkv_elems(const AttnArgs &a, const int (&idx)[6], bool needed, uint16_t (&out)[6])
{
    if (a.n_qkv_slices == 0) {
#pragma unroll
        for (int e = 0; e < 6; e++) out[e] = a.qkv[idx[e]];
        return;
    }
    if (!needed) {                                       // wave-uniform: only the wave that rotates q and k sums slices
#pragma unroll
        for (int e = 0; e < 6; e++) out[e] = 0;
        return;
    }
    float v[6][ATTN_MAX_QKV_SLICES];
#pragma unroll
    for (int s = 0; s < ATTN_MAX_QKV_SLICES; s++) {
        const float *row = a.qkv_slices + (size_t)min(s, a.n_qkv_slices - 1) * a.qkv_stride;
#pragma unroll
        for (int e = 0; e < 6; e++) v[e][s] = row[idx[e]];
    }
#pragma unroll
    for (int e = 0; e < 6; e++) {
        float sum = v[e][0];
#pragma unroll
        for (int s = 1; s < ATTN_MAX_QKV_SLICES; s++)
            if (s < a.n_qkv_slices) sum += v[e][s];
        out[e] = __builtin_bit_cast(uint16_t, (_Float16)sum);
    }
}

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
    if (pos < 0 || pos >= a.max_seq) {            // outside the cache: nothing is read, the output says so (NaN)
        if (wave == 0 && active) {
            a.out[(size_t)h * d + j] = 0x7e00u;
            a.out[(size_t)h * d + j + half] = 0x7e00u;
        }
        return;
    }

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
// positions it sees (one running-max update per batch); the four streams of a wave are
// merged with wave shuffles, the waves through LDS.  Batches of FAST_BATCH row groups are
// loaded before any is used, the first one before the position is even known (4 * FAST_WAVES *
// FAST_BATCH = 256 rows).
// ---------------------------------------------------------------------------------------
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
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

// WAVES x BATCH x 4 rows form a block; split sp of S takes blocks sp, sp + S, ... of the cached
// positions.  S > 1: the splits of a head meet in device memory (unnormalised fp32 output,
// running max and sum per split; agent-scope stores, arrival ticket, the last workgroup of the
// head merges the splits in order), as the K slices of the GEMV do.
template <int WAVES, int BATCH>
__global__ __launch_bounds__(WAVES * 64) void rope_attn_d128_kernel(const AttnArgs a)
{
    constexpr int D = FAST_D, HALF = D / 2, BLOCK_ROWS = WAVES * BATCH * 4;
    __shared__ __align__(16) uint16_t sq[D], sk[D], sv[D];
    __shared__ float sm_m[WAVES], sm_l[WAVES];
    __shared__ float sm_o[WAVES][D];
    __shared__ unsigned s_ticket;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int SL = a.splits;                             // splits launched; S below = splits that take part
    const int h = blockIdx.x / SL, sp = blockIdx.x - h * SL, grp = a.nq / a.nkv, g = h / grp;
    const int seg = lane & 15, r = lane >> 4;

    // Everything the kernel needs from memory first is requested before anything is waited for:
    // the first block of cache rows (row numbers clamped by the cache size, not by the position,
    // so the addresses do not depend on *pos; rows at or beyond it are masked later), q and the
    // new k / v, and the position itself.  One memory round trip instead of three dependent ones.
    const long long pos64 = *a.pos;
    uint4 kk[BATCH], vv[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; b++) {
        const int p = min(sp * BLOCK_ROWS + (wave + WAVES * b) * 4 + r, a.max_seq - 1);
        const size_t row = ((size_t)p * a.nkv + g) * D;
        kk[b] = ((const uint4 *)(a.kc + row))[seg];
        vv[b] = ((const uint4 *)(a.vc + row))[seg];
    }
    // every wave loads the rotary pair (lane, lane + 64) of q, k and v (only wave 0 uses it):
    // unconditional, so that nothing is converted -- and therefore waited for -- in between
    const int qi = h * D, ki = a.nq * D + g * D, vi = (a.nq + a.nkv) * D + g * D;
    const int idx[6] = {qi + lane, qi + lane + HALF, ki + lane, ki + lane + HALF, vi + lane, vi + lane + HALF};
    uint16_t el[6];
    qkv_elems(a, idx, wave == 0, el);
    const uint16_t qa16 = el[0], qb16 = el[1], ka16 = el[2], kb16 = el[3], va16 = el[4], vb16 = el[5];
    asm volatile("" ::: "memory");
    const int pos = (int)pos64;
    if (pos64 < 0 || pos64 >= a.max_seq) {          // outside the cache: nothing is read, the output says so (NaN)
        if (sp == 0 && tid < D) a.out[(size_t)h * D + tid] = 0x7e00u;
        return;
    }
    // How many of the launched workgroups take part follows the context: meeting in device memory
    // costs about 2 us plus 0.1-0.2 us per partial result, a further 64-row block about 0.6 us.  So a
    // context of at most SHORT_BLOCKS blocks is one workgroup's work, up to 12 blocks are shared by
    // at most four, longer contexts by all.  Every workgroup of the head derives the same S from
    // *pos; those beyond it leave at once.
    constexpr int SHORT_BLOCKS = 3;
    const int nblocks = (pos + BLOCK_ROWS - 1) / BLOCK_ROWS;
    const int S = nblocks <= SHORT_BLOCKS ? 1 : min(SL, nblocks <= 12 ? min(nblocks, 4) : ATTN_MAX_SPLITS);
    if (sp >= S) return;

    if (tid < HALF) {                                    // rotary pair (tid, tid + 64) of q and of the new k
        const int j = tid;
        const float inv_freq = exp2f(-(float)(2 * j) / (float)D * a.log2_base);
        float sn, cs;
        __sincosf((float)pos * inv_freq, &sn, &cs);
        const float qa = h2f(qa16), qb = h2f(qb16), ka = h2f(ka16), kb = h2f(kb16);
        sq[j] = f2h(qa * cs - qb * sn); sq[j + HALF] = f2h(qb * cs + qa * sn);
        sk[j] = f2h(ka * cs - kb * sn); sk[j + HALF] = f2h(kb * cs + ka * sn);
        sv[j] = va16; sv[j + HALF] = vb16;
    }
    __syncthreads();
    if (h % grp == 0 && sp == 0 && tid < D / 8) {        // one workgroup per kv head appends the new row
        const size_t row = ((size_t)pos * a.nkv + g) * D;
        ((uint4 *)(a.kc + row))[tid] = ((const uint4 *)sk)[tid];
        ((uint4 *)(a.vc + row))[tid] = ((const uint4 *)sv)[tid];
    }

    const uint4 qv = ((const uint4 *)sq)[seg];
    const float scale = rsqrtf((float)D);
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;

    // The rows of the next block are requested before the current block is worked on, so that a
    // block's memory round trip lies under the arithmetic of the one before.  The loads are
    // unconditional (rows clamped to the last cached one: past the end every lane re-reads one row,
    // which costs next to nothing), so they can be waited for by count.
    const int last_row = max(pos - 1, 0);        // rows below pos do not change during the launch
    for (int blk = sp; blk * BLOCK_ROWS < pos; blk += S) {
        const int base = blk * BLOCK_ROWS;
        uint4 kn[BATCH], vn[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            const int p = min(base + S * BLOCK_ROWS + (wave + WAVES * b) * 4 + r, last_row);
            const size_t row = ((size_t)p * a.nkv + g) * D;
            kn[b] = ((const uint4 *)(a.kc + row))[seg];
            vn[b] = ((const uint4 *)(a.vc + row))[seg];
        }
        // keep the whole batch of loads ahead of the arithmetic (the scheduler would otherwise
        // sink each load to its consumer and serialise the memory round trips)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // one running-max update per batch: scores first, then a single rescale of the stream
        float sc[BATCH], mx = m;
#pragma unroll
        for (int b = 0; b < BATCH; b++) {
            const bool ok = base + (wave + WAVES * b) * 4 + r < pos;
            sc[b] = ok ? dot8(qv, kk[b]) * scale : -INFINITY;
            mx = fmaxf(mx, sc[b]);
        }
        if (mx > -INFINITY) {                            // uniform per 16-lane stream; false only if no row was valid yet
            const float corr = __expf(m - mx);
            l *= corr;
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] *= corr;
#pragma unroll
            for (int b = 0; b < BATCH; b++) {
                const float e = __expf(sc[b] - mx);
                const uint32_t w[4] = {vv[b].x, vv[b].y, vv[b].z, vv[b].w};
                l += e;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    acc[2 * i] = fmaf(e, h2f((uint16_t)(w[i] & 0xffffu)), acc[2 * i]);
                    acc[2 * i + 1] = fmaf(e, h2f((uint16_t)(w[i] >> 16)), acc[2 * i + 1]);
                }
            }
            m = mx;
        }
#pragma unroll
        for (int b = 0; b < BATCH; b++) { kk[b] = kn[b]; vv[b] = vn[b]; }
    }
    if (wave == 0 && sp == 0) {                          // the token being decoded, from LDS (row 0 only)
        const float s = dot8(qv, ((const uint4 *)sk)[seg]) * scale;
        stream_update(s, r == 0, ((const uint4 *)sv)[seg], m, l, acc);
    }
    // merge the four row streams of the wave (lanes 16 and 32 apart), then the waves through LDS
#pragma unroll
    for (int sh = 16; sh <= 32; sh <<= 1) {
        const float m2 = __shfl_xor(m, sh, 64), l2 = __shfl_xor(l, sh, 64);
        const float mx = fmaxf(m, m2);
        const float f1 = (m == mx) ? 1.f : __expf(m - mx), f2 = (m2 == mx) ? 1.f : __expf(m2 - mx);
        l = l * f1 + l2 * f2;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = acc[i] * f1 + __shfl_xor(acc[i], sh, 64) * f2;
        m = mx;
    }
    if (lane == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    if (r == 0) {
#pragma unroll
        for (int i = 0; i < 8; i++) sm_o[wave][seg * 8 + i] = acc[i];
    }
    __syncthreads();
    float M = -INFINITY, L = 0.f, o = 0.f;               // this split's result for dimension tid
    if (tid < D) {
#pragma unroll
        for (int s = 0; s < WAVES; s++) M = fmaxf(M, sm_m[s]);
#pragma unroll
        for (int s = 0; s < WAVES; s++) {
            const float f = (sm_m[s] == M) ? 1.f : __expf(sm_m[s] - M);
            L = fmaf(sm_l[s], f, L);
            o = fmaf(sm_o[s][tid], f, o);
        }
    }
    if (S == 1) {
        if (tid < D) a.out[(size_t)h * D + tid] = f2h(o / L);
        return;
    }
    float *po = a.partial + ((size_t)h * SL + sp) * (D + 2);
    if (tid < D) __hip_atomic_store(&po[tid], o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(&po[D], M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&po[D + 1], L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&a.counters[h], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)S - 1u) return;
    if (tid < D) {
        // all loads of the merge are issued before the first is used
        float pm[ATTN_MAX_SPLITS], pl[ATTN_MAX_SPLITS], pv[ATTN_MAX_SPLITS];
#pragma unroll
        for (int s = 0; s < ATTN_MAX_SPLITS; s++) {
            const float *ps = a.partial + ((size_t)h * SL + min(s, S - 1)) * (D + 2);
            pv[s] = __hip_atomic_load(&ps[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pm[s] = __hip_atomic_load(&ps[D], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pl[s] = __hip_atomic_load(&ps[D + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        float MM = -INFINITY;
#pragma unroll
        for (int s = 0; s < ATTN_MAX_SPLITS; s++)
            if (s < S) MM = fmaxf(MM, pm[s]);
        float LL = 0.f, oo = 0.f;
#pragma unroll
        for (int s = 0; s < ATTN_MAX_SPLITS; s++)
            if (s < S) {
                const float f = (pm[s] == MM) ? 1.f : __expf(pm[s] - MM);
                LL = fmaf(pl[s], f, LL);
                oo = fmaf(pv[s], f, oo);
            }
        a.out[(size_t)h * D + tid] = f2h(oo / LL);
    }
    if (tid == 0) __hip_atomic_store(&a.counters[h], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------
// Tail of the decode step: final RMSNorm in front of the lm_head and the greedy pick behind
// it (launch_pre_rms_norm, C++/ops/src/arm/arm_rmsnorm.cpp:25-84: fp32 statistics, fp16
// output; arm_argmax_last, C++/ops/src/arm/arm_argmax.cpp:3-30: first index of the strict
// maximum).  One workgroup each: the vectors are a few KiB to a few hundred KiB.
// ---------------------------------------------------------------------------------------
constexpr int TAIL_THREADS = 1024;

__global__ __launch_bounds__(TAIL_THREADS) void rmsnorm_kernel(const uint16_t *x, const uint16_t *w, uint16_t *out, int n,
                                                               float eps)
{
    __shared__ float part[TAIL_THREADS / 64];
    const int tid = threadIdx.x;
    float ssq = 0.f;
    for (int i = tid; i < n; i += TAIL_THREADS) {
        const float v = h2f(x[i]);
        ssq = fmaf(v, v, ssq);
    }
    ssq = wave_sum(ssq);
    if ((tid & 63) == 0) part[tid >> 6] = ssq;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < TAIL_THREADS / 64; i++) tot += part[i];
    const float rstd = rsqrtf(tot / (float)n + eps);
    for (int i = tid; i < n; i += TAIL_THREADS) out[i] = f2h(h2f(x[i]) * rstd * h2f(w[i]));
}

// Embedding gather of the current token (arm_embedding, C++/ops/src/arm/arm_embedding.cpp:4-20: a row copy).
// The token is a device scalar; one outside [0, vocab) yields a zero row instead of a read outside the table.
__global__ __launch_bounds__(256) void embed_kernel(const uint16_t *embed, const long long *token, uint16_t *out, int hidden,
                                                    int vocab)
{
    const long long t = *token;
    const bool ok = t >= 0 && t < (long long)vocab;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;             // 8 values per thread
    if (i * 8 + 8 <= hidden) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (ok) v = *(const uint4 *)(embed + (size_t)t * hidden + (size_t)i * 8);
        *(uint4 *)(out + (size_t)i * 8) = v;
    } else {
        for (int j = i * 8; j < hidden; j++) out[j] = ok ? embed[(size_t)t * hidden + j] : (uint16_t)0;
    }
}

// (value, index) order of the greedy pick: larger value first, lower index among equals.
__device__ __forceinline__ void pick(float &v, int &i, float v2, int i2)
{
    if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
}

__global__ __launch_bounds__(TAIL_THREADS) void argmax_kernel(const uint16_t *logits, int n, long long *token, long long *pos)
{
    __shared__ float sv[TAIL_THREADS / 64];
    __shared__ int si[TAIL_THREADS / 64];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    const bool aligned = ((uintptr_t)logits & 15) == 0;
    const int nvec = aligned ? n / 8 : 0;
    for (int c = tid; c < nvec; c += TAIL_THREADS) {     // 8 values per load; indices rise within a thread
        const uint4 q = ((const uint4 *)logits)[c];
        const uint32_t wd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float lo = h2f((uint16_t)(wd[j] & 0xffffu)), hi = h2f((uint16_t)(wd[j] >> 16));
            if (lo > best) { best = lo; idx = c * 8 + 2 * j; }
            if (hi > best) { best = hi; idx = c * 8 + 2 * j + 1; }
        }
    }
    for (int i = nvec * 8 + tid; i < n; i += TAIL_THREADS) {
        const float v = h2f(logits[i]);
        if (v > best) { best = v; idx = i; }
    }
#pragma unroll
    for (int sh = 1; sh < 64; sh <<= 1) pick(best, idx, __shfl_xor(best, sh, 64), __shfl_xor(idx, sh, 64));
    if ((tid & 63) == 0) { sv[tid >> 6] = best; si[tid >> 6] = idx; }
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int i = 1; i < TAIL_THREADS / 64; i++) pick(best, idx, sv[i], si[i]);
        *token = idx == 0x7fffffff ? 0 : idx;            // nothing compared greater than -inf: the reference's initial 0
        if (pos) *pos += 1;
    }
}

// The same pick over a long vector by ARGMAX_WGS workgroups that meet in device memory like the splits
// of the attention kernel: each takes a contiguous range of 8-value groups, stores its (value, index)
// with agent-scope stores, waits for their acknowledgement and draws a ticket; the last one merges the
// pairs (ties go to the lower index, so the result is that of one scan).  One workgroup takes in a
// vocabulary's logits no faster than about 50 KB/us; the vector needs 16-byte alignment here.
constexpr int ARGMAX_WGS = 64, ARGMAX_THREADS = 256;

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_split_kernel(const uint16_t *logits, int n, long long *token,
                                                                      long long *pos, float *pval, int *pidx,
                                                                      unsigned *counter)
{
    __shared__ float sv[ARGMAX_THREADS / 64];
    __shared__ int si[ARGMAX_THREADS / 64];
    __shared__ unsigned s_ticket;
    const int tid = threadIdx.x, wg = blockIdx.x;
    const int nvec = n / 8, per = (nvec + ARGMAX_WGS - 1) / ARGMAX_WGS;
    const int c_begin = wg * per, c_end = min(c_begin + per, nvec);
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int c = c_begin + tid; c < c_end; c += ARGMAX_THREADS) {       // indices rise within a thread
        const uint4 q = ((const uint4 *)logits)[c];
        const uint32_t wd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float lo = h2f((uint16_t)(wd[j] & 0xffffu)), hi = h2f((uint16_t)(wd[j] >> 16));
            if (lo > best) { best = lo; idx = c * 8 + 2 * j; }
            if (hi > best) { best = hi; idx = c * 8 + 2 * j + 1; }
        }
    }
    if (wg == ARGMAX_WGS - 1)                                             // the last n % 8 values
        for (int i = nvec * 8 + tid; i < n; i += ARGMAX_THREADS) {
            const float v = h2f(logits[i]);
            if (v > best) { best = v; idx = i; }
        }
#pragma unroll
    for (int sh = 1; sh < 64; sh <<= 1) pick(best, idx, __shfl_xor(best, sh, 64), __shfl_xor(idx, sh, 64));
    if ((tid & 63) == 0) { sv[tid >> 6] = best; si[tid >> 6] = idx; }
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int i = 1; i < ARGMAX_THREADS / 64; i++) pick(best, idx, sv[i], si[i]);
        __hip_atomic_store(&pval[wg], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&pidx[wg], idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        s_ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (s_ticket != (unsigned)ARGMAX_WGS - 1u || tid >= 64) return;
    best = __hip_atomic_load(&pval[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);      // ARGMAX_WGS == 64: one pair per lane
    idx = __hip_atomic_load(&pidx[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int sh = 1; sh < 64; sh <<= 1) pick(best, idx, __shfl_xor(best, sh, 64), __shfl_xor(idx, sh, 64));
    if (tid == 0) {
        *token = idx == 0x7fffffff ? 0 : idx;
        if (pos) *pos += 1;
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace

extern "C" size_t elutq_decode_attn_workspace_bytes(int n_heads, int head_dim, int splits)
{
    if (n_heads < 1 || head_dim < 2 || splits < 0 || splits > ATTN_MAX_SPLITS) return 0;
    const int s = splits == 0 ? ATTN_MAX_SPLITS : splits;
    return (size_t)HLQ_WS_COUNTER_BYTES + (size_t)n_heads * s * (head_dim + 2) * sizeof(float);
}

// d_qkv_slices non-null: q|k|v arrives as n_qkv_slices unsummed K slices (fp32 rows of qkv_stride floats)
static int launch_rope_attn(const void *d_qkv, const void *d_qkv_slices, int n_qkv_slices, int qkv_stride,
                            void *d_k_cache, void *d_v_cache, const void *d_pos,
                            void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                            float rope_base, int splits, void *d_workspace, size_t workspace_bytes,
                            void *stream)
{
    if (d_qkv_slices) {
        if (head_dim != FAST_D || n_qkv_slices < 1 || n_qkv_slices > ATTN_MAX_QKV_SLICES ||
            qkv_stride < (n_heads + 2 * n_kv_heads) * head_dim)
            return ELUTQ_ERR_TUNING;
        d_qkv = d_qkv_slices;                            // (only checked against null below)
    }
    if (!d_qkv || !d_k_cache || !d_v_cache || !d_pos || !d_out) return ELUTQ_ERR_NULL;
    if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || head_dim < 2 || head_dim > 128 ||
        head_dim % 2 != 0 || max_seq < 1 || !(rope_base > 1.f))
        return ELUTQ_ERR_SHAPE;
    if (splits < 0 || splits > ATTN_MAX_SPLITS) return ELUTQ_ERR_TUNING;
    if (splits == 0) {                                   // default: about one workgroup per CU, if there is a workspace
        splits = d_workspace ? HLQ_NUM_CU / n_heads : 1;
        if (splits > ATTN_MAX_SPLITS) splits = ATTN_MAX_SPLITS;
        if (splits < 1) splits = 1;
    }
    if (head_dim != FAST_D) splits = 1;
    AttnArgs a;
    a.qkv = (const uint16_t *)d_qkv;
    a.kc = (uint16_t *)d_k_cache;
    a.vc = (uint16_t *)d_v_cache;
    a.pos = (const long long *)d_pos;
    a.out = (uint16_t *)d_out;
    a.nq = n_heads; a.nkv = n_kv_heads; a.d = head_dim; a.max_seq = max_seq;
    a.log2_base = log2f(rope_base);
    a.qkv_slices = (const float *)d_qkv_slices; a.n_qkv_slices = d_qkv_slices ? n_qkv_slices : 0; a.qkv_stride = qkv_stride;
    a.splits = splits; a.partial = nullptr; a.counters = nullptr;
    if (splits > 1) {
        if (!d_workspace) return ELUTQ_ERR_NULL;
        if ((size_t)n_heads * sizeof(unsigned) > (size_t)HLQ_WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
        if (workspace_bytes < elutq_decode_attn_workspace_bytes(n_heads, head_dim, splits)) return ELUTQ_ERR_WORKSPACE;
        a.counters = (unsigned *)d_workspace;
        a.partial = (float *)((unsigned char *)d_workspace + HLQ_WS_COUNTER_BYTES);
    }
    if (head_dim != FAST_D)
        hipLaunchKernelGGL(rope_attn_kernel, dim3(n_heads), dim3(ATTN_WAVES * 64), 0, (hipStream_t)stream, a);
    else if (splits == 1)
        hipLaunchKernelGGL((rope_attn_d128_kernel<8, 4>), dim3(n_heads), dim3(8 * 64), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((rope_attn_d128_kernel<4, 4>), dim3(n_heads * splits), dim3(4 * 64), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

extern "C" int elutq_decode_rope_attn_split_f16(const void *d_qkv, void *d_k_cache, void *d_v_cache, const void *d_pos,
                                                void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                                float rope_base, int splits, void *d_workspace, size_t workspace_bytes,
                                                void *stream)
{
    return launch_rope_attn(d_qkv, nullptr, 0, 0, d_k_cache, d_v_cache, d_pos, d_out, n_heads, n_kv_heads, head_dim, max_seq,
                            rope_base, splits, d_workspace, workspace_bytes, stream);
}

extern "C" int elutq_decode_rope_attn_sliced_f16(const void *d_qkv_slices, int n_slices, int slice_stride, void *d_k_cache,
                                                 void *d_v_cache, const void *d_pos, void *d_out, int n_heads,
                                                 int n_kv_heads, int head_dim, int max_seq, float rope_base, int splits,
                                                 void *d_workspace, size_t workspace_bytes, void *stream)
{
    if (!d_qkv_slices) return ELUTQ_ERR_NULL;
    return launch_rope_attn(nullptr, d_qkv_slices, n_slices, slice_stride, d_k_cache, d_v_cache, d_pos, d_out, n_heads,
                            n_kv_heads, head_dim, max_seq, rope_base, splits, d_workspace, workspace_bytes, stream);
}

extern "C" int elutq_decode_rope_attn_f16(const void *d_qkv, void *d_k_cache, void *d_v_cache, const void *d_pos,
                                          void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                          float rope_base, void *stream)
{
    return elutq_decode_rope_attn_split_f16(d_qkv, d_k_cache, d_v_cache, d_pos, d_out, n_heads, n_kv_heads, head_dim,
                                            max_seq, rope_base, 1, nullptr, 0, stream);
}

extern "C" int elutq_decode_embed_f16(const void *d_embed, const void *d_token, void *d_out, int hidden, int vocab, void *stream)
{
    if (!d_embed || !d_token || !d_out) return ELUTQ_ERR_NULL;
    if (hidden < 1 || vocab < 1 || hidden % 8 != 0) return ELUTQ_ERR_SHAPE;      // rows stay 16-byte aligned
    hipLaunchKernelGGL(embed_kernel, dim3((hidden / 8 + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)d_embed,
                       (const long long *)d_token, (uint16_t *)d_out, hidden, vocab);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

extern "C" int elutq_decode_rmsnorm_f16(const void *d_x, const void *d_weight, void *d_out, int n, float eps, void *stream)
{
    if (!d_x || !d_weight || !d_out) return ELUTQ_ERR_NULL;
    if (n < 1) return ELUTQ_ERR_SHAPE;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(TAIL_THREADS), 0, (hipStream_t)stream, (const uint16_t *)d_x,
                       (const uint16_t *)d_weight, (uint16_t *)d_out, n, eps);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

extern "C" int elutq_decode_argmax_ws_f16(const void *d_logits, int n, void *d_token, void *d_pos, void *d_workspace,
                                          size_t workspace_bytes, void *stream)
{
    if (!d_logits || !d_token) return ELUTQ_ERR_NULL;
    if (n < 1) return ELUTQ_ERR_SHAPE;
    const size_t need = (size_t)HLQ_WS_COUNTER_BYTES + (size_t)ARGMAX_WGS * (sizeof(float) + sizeof(int));
    // short or unaligned vectors, or no workspace: the single-workgroup kernel
    if (!d_workspace || n < 65536 || ((uintptr_t)d_logits & 15) != 0)
        return elutq_decode_argmax_f16(d_logits, n, d_token, d_pos, stream);
    if (workspace_bytes < need) return ELUTQ_ERR_WORKSPACE;
    float *pval = (float *)((unsigned char *)d_workspace + HLQ_WS_COUNTER_BYTES);
    hipLaunchKernelGGL(argmax_split_kernel, dim3(ARGMAX_WGS), dim3(ARGMAX_THREADS), 0, (hipStream_t)stream,
                       (const uint16_t *)d_logits, n, (long long *)d_token, (long long *)d_pos, pval,
                       (int *)(pval + ARGMAX_WGS), (unsigned *)d_workspace);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

extern "C" int elutq_decode_argmax_f16(const void *d_logits, int n, void *d_token, void *d_pos, void *stream)
{
    if (!d_logits || !d_token) return ELUTQ_ERR_NULL;
    if (n < 1) return ELUTQ_ERR_SHAPE;
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(TAIL_THREADS), 0, (hipStream_t)stream, (const uint16_t *)d_logits, n,
                       (long long *)d_token, (long long *)d_pos);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

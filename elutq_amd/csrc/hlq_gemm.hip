// Small-batch HLQ GEMM for gfx950 (MI355X): y[M][N] = x[M][K] W^T + bias, 2 <= M <= 64 per
// launch, replacing MultiThread_arm_gemm_w_lowbit_activation_fp_impl
// (C++/ops/src/arm/arm_gemm.cpp:362-387), which re-runs the GEMV once per row.
//
// With M rows the contraction is dense enough for the matrix cores, so the bit-planes are
// expanded in registers and fed to v_mfma_f32_32x32x16_f16, bit-serially:
//
//   y[m][n] = sum_g ( z[n,g] * (X 1)[m,g]  +  sum_b s[b,n,g] * (X B_b)[m,n,g] )
//
// Each plane (and an all-ones "plane" that carries the zero point) is a 0/1 matrix; one
// v_alignbit + v_and turns two plane bits into a packed pair of fp16 values 0 or 2^-14
// (a single exponent bit), eight such values are the B operand of one MFMA.  The plane
// sum of one quantization group is accumulated in fp32 by the MFMA, then folded into the
// running result with the column's scale (lane = output column in the MFMA's C layout, so
// the scale is one scalar per lane).  Only the weights stream from HBM; the activations
// are staged per workgroup in LDS, already in the element order the B operand uses.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int CH = HLQ_GEMM_CH;                // units staged per chunk = waves per workgroup
constexpr int ROW_HALFS = CH * HLQ_UNIT + 8;   // LDS row stride in fp16 (16 B pad: conflict-free b128 reads)
constexpr int GEMM_THREADS = CH * 64;
constexpr int WS_COUNTER_BYTES = HLQ_WS_COUNTER_BYTES;

struct GemmArgs {
    const uint4 *planes;
    const uint32_t *scales;
    const uint32_t *zeros;
    const uint16_t *bias;
    const uint16_t *x;      // fp16 [M][K]
    uint16_t *y;            // fp16 [M][N]
    float *partial;         // [ksplit][MT*32][ncb*64]
    unsigned *counters;     // [ncb]
    int M, N, K, U, NT, ncb;
    int ksplit, ups;        // slices per column block, units per slice (multiple of CH)
};

#ifdef HLQ_TIMING
// Profiling builds only: wall-clock stamps (100 MHz) of thread 0 of every workgroup.
__device__ unsigned long long *g_gemm_stamps = nullptr;
#define GEMM_STAMP(i)                                                                                  \
    do {                                                                                               \
        if (g_gemm_stamps && threadIdx.x == 0 && (i) < 16) g_gemm_stamps[(size_t)blockIdx.x * 16 + (i)] = wall_clock64(); \
    } while (0)
#else
#define GEMM_STAMP(i) do { } while (0)
#endif

__device__ __forceinline__ float h2f(uint32_t v, int hi)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? v >> 16 : v & 0xffffu));
}

// Element order of one 32-k dword inside the MFMA operands: step e (0/1), lane half h,
// element i = 2q + r  <->  k = 8e + 4h + q + 16r.  The B side gets it from
// (rotr(w, 8e + 4h + q - 10) & 0x04000400): bit k lands on the lowest exponent bit of the
// low fp16, bit k + 16 on that of the high fp16.
__device__ __forceinline__ half8 expand_bits(uint32_t w, int e, int h)
{
    uint32_t d[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const uint32_t sh = (uint32_t)(8 * e + 4 * h + q - 10 + HLQ_ROT) & 31u;   // stored dwords are rotated left by HLQ_ROT
        d[q] = __builtin_amdgcn_alignbit(w, w, sh) & 0x04000400u;
    }
    return __builtin_bit_cast(half8, make_uint4(d[0], d[1], d[2], d[3]));
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Staging of x[:, u0*128 .. (u0+CH)*128) into LDS in operand order: row m holds, for every
// unit ul, dword d, step e and half h, the eight fp16 { x[k(q,0)], x[k(q,1)] : q = 0..3 },
// and xs[(ul*2 + half) * MT*32 + m] the fp32 sum of x over each 64-k half unit (zero-point
// fold).  One task = (row, unit, 32-k dword); the four dwords of a unit sit in one DPP quad.
// Two phases so that the global loads of the next chunk fly while the current one computes;
// the loads are unconditional (clamped addresses) so the compiler can count them.
template <int MT>
struct StageRegs {
    static constexpr int TPT = MT * 32 * CH * 4 / GEMM_THREADS;     // tasks per thread
    uint4 v[TPT][4];
};

template <int MT>
__device__ __forceinline__ void stage_load(StageRegs<MT> &r, const GemmArgs &a, int u0, int u_end, int tid)
{
#pragma unroll
    for (int t = 0; t < StageRegs<MT>::TPT; t++) {
        const int idx = tid + t * GEMM_THREADS;
        const int m = idx / (CH * 4), rr = idx % (CH * 4), ul = rr >> 2, d = rr & 3;
        const int mm = m < a.M ? m : a.M - 1, uu = u0 + ul < u_end ? u0 + ul : u_end - 1;
        const uint4 *src = (const uint4 *)(a.x + (size_t)mm * a.K + (size_t)uu * HLQ_UNIT + d * 32);
#pragma unroll
        for (int i = 0; i < 4; i++) r.v[t][i] = src[i];
    }
}

template <int MT>
__device__ __forceinline__ void stage_store(const StageRegs<MT> &r, const GemmArgs &a, int u0, int u_end, _Float16 *xl,
                                            float *xs, int tid)
{
#pragma unroll
    for (int t = 0; t < StageRegs<MT>::TPT; t++) {
        const int idx = tid + t * GEMM_THREADS;
        const int m = idx / (CH * 4), rr = idx % (CH * 4), ul = rr >> 2, d = rr & 3;
        const bool live = m < a.M && u0 + ul < u_end;
        uint32_t v[16];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[4 * i] = live ? r.v[t][i].x : 0u; v[4 * i + 1] = live ? r.v[t][i].y : 0u;
            v[4 * i + 2] = live ? r.v[t][i].z : 0u; v[4 * i + 3] = live ? r.v[t][i].w : 0u;
        }
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) sum += h2f(v[i], 0) + h2f(v[i], 1);
        sum += dpp_f<0xB1>(sum);                 // dwords 0+1 and 2+3: the two 64-k halves of the unit
        if ((d & 1) == 0) xs[(ul * 2 + (d >> 1)) * (MT * 32) + m] = sum;
        // fp16 index j of the 32 sits in v[j/2], half j&1.  Output dword q of (e,h) pairs
        // x[8e+4h+q] (low) with x[8e+4h+q+16] (high).
        uint4 *dst = (uint4 *)(xl + (size_t)m * ROW_HALFS + (ul * 8 + 2 * d) * 16);
#pragma unroll
        for (int e = 0; e < 2; e++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                uint32_t o[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int j = 8 * e + 4 * h + q;
                    const uint32_t lo = (j & 1) ? (v[j / 2] >> 16) : (v[j / 2] & 0xffffu);
                    const uint32_t hi = (j & 1) ? (v[(j + 16) / 2] & 0xffff0000u) : (v[(j + 16) / 2] << 16);
                    o[q] = lo | hi;
                }
                dst[e * 2 + h] = make_uint4(o[0], o[1], o[2], o[3]);
            }
    }
}

// Everything a wave needs from HBM for one unit: the planes and, for each of the two
// 32-column tiles, the scale and zero dwords of its own column.
template <int BITS>
struct UnitData {
    uint4 w[BITS];
    uint32_t sc[BITS][2];
    uint32_t zz[2];
};

template <int BITS, bool G64>
__device__ __forceinline__ void load_unit(UnitData<BITS> &d, const GemmArgs &a, int cb, int u, int u_end, int lane)
{
    const int uu = u < u_end ? u : u_end - 1;          // past the slice: reload a valid unit nobody uses
    const int col = lane & 31;
    const size_t meta = (size_t)cb * a.NT + (G64 ? uu : (uu >> 1));
#pragma unroll
    for (int b = 0; b < BITS; b++) {
        d.w[b] = a.planes[(((size_t)cb * a.U + uu) * BITS + b) * HLQ_CB + lane];
        d.sc[b][0] = a.scales[(meta * BITS + b) * HLQ_CB + col];
        d.sc[b][1] = a.scales[(meta * BITS + b) * HLQ_CB + 32 + col];
    }
    d.zz[0] = a.zeros[meta * HLQ_CB + col];
    d.zz[1] = a.zeros[meta * HLQ_CB + 32 + col];
}

template <int BITS, bool G64, int MT>
__global__ __launch_bounds__(GEMM_THREADS) void hlq_gemm_kernel(const GemmArgs a)
{
    extern __shared__ __align__(256) unsigned char smem[];
    constexpr int MROWS = MT * 32;
    _Float16 *xl = (_Float16 *)smem;
    float *xs = (float *)(smem + (size_t)MROWS * ROW_HALFS * 2);      // [CH*2][MROWS]
    float *red = (float *)smem;                                          // reused after the last chunk
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int cb = blockIdx.x / a.ksplit, slice = blockIdx.x - cb * a.ksplit;
    const int u_begin = slice * a.ups, u_end = min(u_begin + a.ups, a.U);

    float16v acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][j][i] = 0.f;

    GEMM_STAMP(0);
    // Software pipeline over chunks of CH units: while chunk c computes, the planes / scales /
    // zeros of chunk c+1 (one unit per wave) and its slice of x are already in flight; two
    // register sets alternate so that nothing is copied while loads are pending.
    UnitData<BITS> bufA, bufB;
    StageRegs<MT> xr;
    load_unit<BITS, G64>(bufA, a, cb, u_begin + wave, u_end, lane);
    stage_load<MT>(xr, a, u_begin, u_end, tid);
    int stamp_i = 1;
    (void)stamp_i;
    auto step = [&](const UnitData<BITS> &cur, UnitData<BITS> &fill, int u0) __attribute__((always_inline)) {
        __syncthreads();                              // the previous chunk's operands are no longer read
        GEMM_STAMP(stamp_i); stamp_i++;
        stage_store<MT>(xr, a, u0, u_end, xl, xs, tid);
        load_unit<BITS, G64>(fill, a, cb, u0 + CH + wave, u_end, lane);
        stage_load<MT>(xr, a, u0 + CH, u_end, tid);
        GEMM_STAMP(stamp_i); stamp_i++;
        __syncthreads();
        GEMM_STAMP(stamp_i); stamp_i++;
        const int u = u0 + wave;
        if (u < u_end) {
            const int odd = u & 1;
            // JB column tiles share each A operand read (one ds_read_b128 per row tile and step
            // feeds JB * BITS MFMAs); limited by the accumulators that fit in registers.
            constexpr int JB = (BITS * MT <= 2) ? 2 : 1;
#pragma unroll
            for (int j0 = 0; j0 < 2; j0 += JB) {
                // columns 32j..32j+31 of the block live in lanes 32j..32j+31: give both lane halves a copy
                uint32_t wj[JB][BITS][4];
                float16v ct[JB][BITS][MT];
#pragma unroll
                for (int jj = 0; jj < JB; jj++)
#pragma unroll
                    for (int b = 0; b < BITS; b++) {
                        const uint32_t wd[4] = {cur.w[b].x, cur.w[b].y, cur.w[b].z, cur.w[b].w};
#pragma unroll
                        for (int d = 0; d < 4; d++) wj[jj][b][d] = (uint32_t)__shfl((int)wd[d], 32 * (j0 + jj) + col, 64);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
#pragma unroll
                            for (int i = 0; i < 16; i++) ct[jj][b][mt][i] = 0.f;
                    }
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    half8 aop[MT];
#pragma unroll
                    for (int mt = 0; mt < MT; mt++)
                        aop[mt] = *(const half8 *)(xl + (size_t)(mt * 32 + col) * ROW_HALFS + (wave * 8 + s) * 16 + h * 8);
#pragma unroll
                    for (int jj = 0; jj < JB; jj++)
#pragma unroll
                        for (int b = 0; b < BITS; b++) {
                            const half8 bop = expand_bits(wj[jj][b][s >> 1], s & 1, h);
#pragma unroll
                            for (int mt = 0; mt < MT; mt++)
                                ct[jj][b][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aop[mt], bop, ct[jj][b][mt], 0, 0, 0);
                        }
                    if (G64 && s == 3) {              // first 64 k = first group of the unit
#pragma unroll
                        for (int jj = 0; jj < JB; jj++)
#pragma unroll
                            for (int b = 0; b < BITS; b++) {
                                const float f = h2f(cur.sc[b][j0 + jj], 0) * 16384.f;
#pragma unroll
                                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                                    for (int i = 0; i < 16; i++) {
                                        acc[mt][j0 + jj][i] = fmaf(f, ct[jj][b][mt][i], acc[mt][j0 + jj][i]);
                                        ct[jj][b][mt][i] = 0.f;
                                    }
                            }
                    }
                }
#pragma unroll
                for (int jj = 0; jj < JB; jj++) {
                    const int j = j0 + jj;
#pragma unroll
                    for (int b = 0; b < BITS; b++) {
                        const float f = h2f(cur.sc[b][j], G64 ? 1 : odd) * 16384.f;
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
#pragma unroll
                            for (int i = 0; i < 16; i++) acc[mt][j][i] = fmaf(f, ct[jj][b][mt][i], acc[mt][j][i]);
                    }
                    // zero point: z[n, g] * sum_{k in g} x[m, k]; C rows of register i: 8*(i/4) + 4h + i%4
                    const float z0 = h2f(cur.zz[j], G64 ? 0 : odd), z1 = h2f(cur.zz[j], G64 ? 1 : odd);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++)
#pragma unroll
                        for (int i4 = 0; i4 < 4; i4++) {
                            const int m0 = mt * 32 + 8 * i4 + 4 * h;
                            const float4 s0 = *(const float4 *)(xs + (wave * 2 + 0) * MROWS + m0);
                            const float4 s1 = *(const float4 *)(xs + (wave * 2 + 1) * MROWS + m0);
                            acc[mt][j][4 * i4 + 0] += z0 * s0.x + z1 * s1.x;
                            acc[mt][j][4 * i4 + 1] += z0 * s0.y + z1 * s1.y;
                            acc[mt][j][4 * i4 + 2] += z0 * s0.z + z1 * s1.z;
                            acc[mt][j][4 * i4 + 3] += z0 * s0.w + z1 * s1.w;
                        }
                }
            }
        }
    };
    for (int u0 = u_begin; u0 < u_end; u0 += 2 * CH) {
        step(bufA, bufB, u0);
        if (u0 + CH < u_end) step(bufB, bufA, u0 + CH);
    }

    GEMM_STAMP(13);
    // Cross-wave sum through LDS: red[wave][tile = mt*2+j][reg][lane].
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) red[((wave * MT * 2 + mt * 2 + j) * 16 + i) * 64 + lane] = acc[mt][j][i];
    __syncthreads();

    constexpr int VALS = MT * 2 * 16 * 64;
    const size_t npad = (size_t)a.ncb * HLQ_CB;
    const int mpad = MT * 32;
    float outv[VALS / GEMM_THREADS];
#pragma unroll
    for (int it = 0; it < VALS / GEMM_THREADS; it++) {
        const int v = tid + it * GEMM_THREADS;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < CH; w++) s += red[w * VALS + v];
        outv[it] = s;
    }
    // value v = (tile, reg, lane): C layout of the 32x32 MFMA: column = lane % 32,
    // row = 8 * (reg / 4) + 4 * (lane / 32) + reg % 4.
    auto decode = [&](int v, int &m, int &n) {
        const int ln = v & 63, reg = (v >> 6) & 15, tile = v >> 10;
        const int mt = tile >> 1, j = tile & 1;
        m = mt * 32 + 8 * (reg >> 2) + 4 * (ln >> 5) + (reg & 3);
        n = cb * HLQ_CB + j * 32 + (ln & 31);
    };
    if (a.ksplit == 1) {
#pragma unroll
        for (int it = 0; it < VALS / GEMM_THREADS; it++) {
            int m, n;
            decode(tid + it * GEMM_THREADS, m, n);
            if (m < a.M && n < a.N) {
                float s = outv[it];
                if (a.bias) s += (float)__builtin_bit_cast(_Float16, a.bias[n]);
                a.y[(size_t)m * a.N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
            }
        }
        return;
    }
    // Slices meet through device memory, as in the GEMV: agent-scope stores, wait for their
    // acknowledgement, take a ticket; the last workgroup sums the slices in order.
#pragma unroll
    for (int it = 0; it < VALS / GEMM_THREADS; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        __hip_atomic_store(&a.partial[((size_t)slice * mpad + m) * npad + n], outv[it], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    GEMM_STAMP(14);
    __syncthreads();
    __shared__ unsigned s_ticket;
    if (tid == 0) s_ticket = __hip_atomic_fetch_add(&a.counters[cb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != (unsigned)a.ksplit - 1u) return;
    // all of a thread's loads for four slices are in flight together; summed in slice order
    constexpr int NV = VALS / GEMM_THREADS;
    float sum[NV];
    size_t off[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        off[it] = (size_t)m * npad + n;
        sum[it] = 0.f;
    }
    for (int s0 = 0; s0 < a.ksplit; s0 += 4) {
        float v[4][NV];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int sl = min(s0 + q, a.ksplit - 1);
#pragma unroll
            for (int it = 0; it < NV; it++)
                v[q][it] = __hip_atomic_load(&a.partial[(size_t)sl * mpad * npad + off[it]], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (s0 + q < a.ksplit) {
#pragma unroll
                for (int it = 0; it < NV; it++) sum[it] += v[q][it];
            }
    }
#pragma unroll
    for (int it = 0; it < NV; it++) {
        int m, n;
        decode(tid + it * GEMM_THREADS, m, n);
        if (m < a.M && n < a.N) {
            float s = sum[it];
            if (a.bias) s += (float)__builtin_bit_cast(_Float16, a.bias[n]);
            a.y[(size_t)m * a.N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
        }
    }
    if (tid == 0) __hip_atomic_store(&a.counters[cb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    GEMM_STAMP(15);
}

template <int MT>
size_t gemm_lds_bytes()
{
    const size_t x = (size_t)MT * 32 * ROW_HALFS * 2 + (size_t)CH * 2 * MT * 32 * sizeof(float);
    const size_t r = (size_t)CH * MT * 2 * 16 * 64 * 4;
    return (x > r ? x : r) + 256;
}

template <int BITS, bool G64, int MT>
int launch_gemm(const GemmArgs &a, hipStream_t stream)
{
    auto kern = hlq_gemm_kernel<BITS, G64, MT>;
    const size_t lds = gemm_lds_bytes<MT>();
    static bool big_lds_enabled = false;
    if (lds > 64 * 1024 && !big_lds_enabled) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return ELUTQ_ERR_HIP;
        big_lds_enabled = true;
    }
    hipLaunchKernelGGL(kern, dim3(a.ncb * a.ksplit), dim3(GEMM_THREADS), lds, stream, a);
    return hipGetLastError() == hipSuccess ? ELUTQ_OK : ELUTQ_ERR_HIP;
}

template <int BITS, bool G64>
int launch_gemm_mt(const GemmArgs &a, hipStream_t stream)
{
    return a.M <= 32 ? launch_gemm<BITS, G64, 1>(a, stream) : launch_gemm<BITS, G64, 2>(a, stream);
}

int dispatch_gemm(const GemmArgs &a, int bits, bool g64, hipStream_t stream)
{
    switch (bits) {
    case 1: return g64 ? launch_gemm_mt<1, true>(a, stream) : launch_gemm_mt<1, false>(a, stream);
    case 2: return g64 ? launch_gemm_mt<2, true>(a, stream) : launch_gemm_mt<2, false>(a, stream);
    case 3: return g64 ? launch_gemm_mt<3, true>(a, stream) : launch_gemm_mt<3, false>(a, stream);
    case 4: return g64 ? launch_gemm_mt<4, true>(a, stream) : launch_gemm_mt<4, false>(a, stream);
    }
    return ELUTQ_ERR_BITS;
}

}  // namespace

// Rows per launch; more rows are processed in chunks of this many (weights re-streamed).
#define HLQ_GEMM_MAX_M 64

extern "C" {

#ifdef HLQ_TIMING
int elutq_debug_set_gemm_stamps(void *d_buf)
{
    return hipMemcpyToSymbol(HIP_SYMBOL(g_gemm_stamps), &d_buf, sizeof(d_buf)) == hipSuccess ? 0 : -1;
}
#endif

// y[M][N] = x[M][K] W^T + bias.  M == 1 goes to the LUT GEMV; larger M to the MFMA kernel in
// chunks of up to 64 rows.
int elutq_hlq_gemm_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                       const void *d_x, void *d_y, int M, int K, int N, int bits, int group, void *d_workspace,
                       size_t workspace_bytes, void *stream)
{
    if (M < 1) return ELUTQ_ERR_SHAPE;
    if (M == 1)
        return elutq_hlq_gemv_f16(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, d_workspace,
                                  workspace_bytes, stream);
    if (bits < 1 || bits > 4) return ELUTQ_ERR_BITS;
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (K < HLQ_UNIT || N < 1 || K % HLQ_UNIT != 0 || K % group != 0) return ELUTQ_ERR_SHAPE;
    if (!d_planes || !d_scales || !d_zeros || !d_x || !d_y) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);

    for (int m0 = 0; m0 < M; m0 += HLQ_GEMM_MAX_M) {
        const int mc = M - m0 < HLQ_GEMM_MAX_M ? M - m0 : HLQ_GEMM_MAX_M;
        GemmArgs a;
        a.planes = (const uint4 *)d_planes;
        a.scales = (const uint32_t *)d_scales;
        a.zeros = (const uint32_t *)d_zeros;
        a.bias = (const uint16_t *)d_bias;
        a.x = (const uint16_t *)d_x + (size_t)m0 * K;
        a.y = (uint16_t *)d_y + (size_t)m0 * N;
        a.M = mc; a.N = N; a.K = K; a.U = g.U; a.NT = g.NT; a.ncb = g.ncb;
        int ks, ups;
        hlq_gemm_split(g, ks, ups);
        a.ksplit = ks; a.ups = ups;
        a.partial = nullptr; a.counters = nullptr;
        if (ks > 1) {
            const int mpad = mc <= 32 ? 32 : 64;
            if (!d_workspace) return ELUTQ_ERR_NULL;
            if ((size_t)g.ncb * sizeof(unsigned) > (size_t)WS_COUNTER_BYTES) return ELUTQ_ERR_SHAPE;
            if (workspace_bytes < (size_t)WS_COUNTER_BYTES + (size_t)ks * mpad * g.ncb * HLQ_CB * sizeof(float))
                return ELUTQ_ERR_WORKSPACE;
            a.counters = (unsigned *)d_workspace;
            a.partial = (float *)((unsigned char *)d_workspace + WS_COUNTER_BYTES);
        }
        int rc = dispatch_gemm(a, bits, group == 64, (hipStream_t)stream);
        if (rc != ELUTQ_OK) return rc;
    }
    return ELUTQ_OK;
}

}  // extern "C"

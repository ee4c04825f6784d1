/*
 * CPU restatement of the reference's live low-bit GEMV/GEMM path.
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed host
 * baseline.  Nothing in the shipped package links or loads this file.
 *
 * The reference (Nkniexin/ELUTQ, the .cpp files under C++/ops/src/arm) is ARM-NEON only and
 * cannot be compiled on x86, so its algorithm is restated here in portable C,
 * operation for operation, with the same fp16 rounding points:
 *
 *   elutq_ref_rearrange   arm_t_mac_kernal.cpp:472-552  (loader permutation)
 *   elutq_ref_lut         arm_t_mac_kernal.cpp:95-138   (fp16 subset-sum LUT)
 *   update_plane_scalar   arm_t_mac_kernal.cpp:364-469  (bit-plane update)
 *   run_chunk             arm_gemm.cpp:248-308          (zero fold, planes, bias)
 *   elutq_ref_gemv        arm_gemm.cpp:312-360          (N split over threads)
 *   elutq_ref_gemm        arm_gemm.cpp:362-387          (m > 1: row loop)
 *   elutq_ref_rearrange_sparse  arm_t_mac_kernal.cpp:554-647 (loader permutation, use_sparse)
 *   update_plane_sparse   arm_t_mac_kernal.cpp:678-788  (block-sparse extra plane)
 *   run_chunk_sparse      arm_gemm.cpp:725-808          (zero fold, dense planes, extra plane, bias)
 *   elutq_ref_gemv_sparse arm_gemm.cpp:811-868          (N split; blocks split by channel start)
 *   elutq_ref_gemv_fast   same data flow with AVX2 pshufb lookups (the x86
 *                         counterpart of vqtbl1q_u8) and fp32 accumulators; used
 *                         only as the timed CPU baseline, never as a checker.
 *
 * Every buffer the kernels index is in the reference's REARRANGED layout
 * (output of elutq_ref_rearrange), and is indexed with the reference's own
 * expressions, so that the permutation is exercised too.
 *
 * fp16 arithmetic: NEON fp16 add/mul round once to binary16.  Here a binary16
 * add or multiply is done in binary32 and rounded to binary16; that is the
 * correctly rounded result because 24 >= 2*11+2 (double rounding is innocuous).
 * A fused multiply-add is done in binary64 (product exact, one rounding of the
 * sum that is innocuous for the same reason) and rounded to binary16.
 * `fused` selects fmla semantics for `v += a*b`, which is what the reference's
 * -O3 build (default -ffp-contract=fast) emits for float16x8_t expressions.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <immintrin.h>

typedef uint16_t h16;

static inline float h2f(h16 h) { return _cvtsh_ss(h); }
static inline h16 f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }
static inline h16 d2h(double d)
{
    /* binary64 -> binary16 with a single rounding: go through binary32 only
     * when that conversion is exact enough; otherwise round by hand. */
    float f = (float)d;
    if ((double)f == d) return f2h(f);
    /* d is not representable in binary32: replace f by d rounded to odd
     * (truncate towards zero, then force the last bit), so the second rounding
     * cannot land on a tie that d itself does not sit on. */
    uint32_t u; memcpy(&u, &f, 4);
    double af = f < 0 ? -(double)f : (double)f, ad = d < 0 ? -d : d;
    if (af > ad) u -= 1u;         /* one ulp towards zero (same sign, magnitude bits) */
    u |= 1u;                      /* sticky bit, 13 places below binary16's last bit */
    memcpy(&f, &u, 4);
    return f2h(f);
}
static inline h16 hadd(h16 a, h16 b) { return f2h(h2f(a) + h2f(b)); }
static inline h16 hmul(h16 a, h16 b) { return f2h(h2f(a) * h2f(b)); }
static inline h16 hmac(h16 acc, h16 a, h16 b, int fused)
{
    if (fused) return d2h((double)h2f(acc) + (double)h2f(a) * (double)h2f(b));
    return hadd(acc, hmul(a, b));
}

#define MINI(a, b) ((a) < (b) ? (a) : (b))

/* arm_t_mac_kernal.cpp:472-552.  Returns 1 on success, 0 on a count mismatch
 * (the reference then calls exit(-1), parameters.cpp:68). */
int elutq_ref_rearrange(int out_channel, int in_channel, int bits, int Actk, int n_thread,
                        const uint8_t *weight, const h16 *w_scale, const h16 *w_zero,
                        uint8_t *weight_out, h16 *w_scale_out, h16 *w_zero_out)
{
    long index = 0;
    int chunk_size = (out_channel + n_thread - 1) / n_thread;
    for (int thread = 0; thread < n_thread; thread++) {
        int start = thread * chunk_size;
        int end = MINI(start + chunk_size, out_channel);
        for (int bit = 0; bit < bits; bit++) {
            const uint8_t *ws = weight + (long)bit * out_channel * in_channel / 8;
            for (int i = start; i < end; i += 32)
                for (int j = 0; j < in_channel / 8; j++)
                    for (int k = 0; k < 32; k++)
                        weight_out[index++] = ws[(long)(i + k) * in_channel / 8 + j];
        }
    }
    if (index != (long)in_channel * out_channel * bits / 8) return 0;

    index = 0;
    for (int thread = 0; thread < n_thread; thread++) {
        int start = thread * chunk_size;
        int end = MINI(start + chunk_size, out_channel);
        for (int bit = 0; bit < bits; bit++) {
            const h16 *ss = w_scale + (long)bit * out_channel * in_channel / Actk;
            for (int i = start; i < end; i += 32)
                for (int j = 0; j < in_channel; j += Actk)
                    for (int k = 0; k < 32; k++)
                        w_scale_out[index++] = ss[(long)(i + k) * in_channel / Actk + j / Actk];
        }
    }
    if (index != (long)bits * in_channel * out_channel / Actk) return 0;

    index = 0;
    for (int i = 0; i < out_channel; i += 32)
        for (int j = 0; j < in_channel; j += Actk)
            for (int k = 0; k < 32; k++)
                w_zero_out[index++] = w_zero[(long)(i + k) * in_channel / Actk + j / Actk];
    if (index != (long)in_channel * out_channel / Actk) return 0;
    return 1;
}

/* arm_t_mac_kernal.cpp:95-138: lut[c][g], g = 0..15, sequential fp16 adds in
 * ascending bit order. */
void elutq_ref_lut(int in_channel, const h16 *activation, h16 *lut)
{
    for (int i = 0; i < in_channel; i += 4) {
        h16 temp[16];
        memset(temp, 0, sizeof(temp));
        for (int g = 0; g < 16; g++) {
            if (g & 1) temp[g] = hadd(temp[g], activation[i]);
            if (g & 2) temp[g] = hadd(temp[g], activation[i + 1]);
            if (g & 4) temp[g] = hadd(temp[g], activation[i + 2]);
            if (g & 8) temp[g] = hadd(temp[g], activation[i + 3]);
        }
        memcpy(lut + (long)(i / 4) * 16, temp, sizeof(temp));
    }
}

/* arm_t_mac_kernal.cpp:364-469 for one plane of one thread chunk. */
static void update_plane_scalar(h16 *out, const uint8_t *weight, int in_channel, int out_channel,
                                const h16 *lut, const h16 *w_scale, int ActK, int fused)
{
    for (int i = 0; i < out_channel; i += 32) {
        h16 c[32];
        for (int j = 0; j < in_channel; j += ActK) {
            h16 acc[32];
            memset(acc, 0, sizeof(acc));
            for (int l = 0; l < ActK; l += 8) {
                const uint8_t *w = weight + ((long)i * in_channel) / 8 + (long)(j + l) * 4;
                const h16 *lut_lo = lut + (long)((j + l) / 4) * 16;
                const h16 *lut_hi = lut + (long)((j + l) / 4 + 1) * 16;
                for (int ch = 0; ch < 32; ch++) {
                    acc[ch] = hadd(acc[ch], lut_lo[w[ch] & 15]);
                    acc[ch] = hadd(acc[ch], lut_hi[w[ch] >> 4]);
                }
            }
            const h16 *s = w_scale + (long)i * in_channel / ActK + (long)32 * j / ActK;
            if (j == 0)
                for (int ch = 0; ch < 32; ch++) c[ch] = hmul(acc[ch], s[ch]);
            else
                for (int ch = 0; ch < 32; ch++) c[ch] = hmac(c[ch], acc[ch], s[ch], fused);
        }
        for (int ch = 0; ch < 32; ch++) out[i + ch] = hadd(out[i + ch], c[ch]);
    }
}

/* arm_gemm.cpp:248-308 (MultiThreadGemvW_lowbit_Activation_FP::Run). */
static void run_chunk(int k, int n, const h16 *input, const uint8_t *weight, const h16 *w_scale,
                      const h16 *w_zero, const h16 *bias, h16 *output, int Actk, int bit,
                      h16 *input_sum, h16 *lut, int fused)
{
    for (int i = 0; i < k; i += Actk) {
        h16 s = 0;
        for (int j = 0; j < Actk; j++) s = hadd(s, input[i + j]);
        input_sum[i / Actk] = s;
    }
    int cnt_per_row = k / Actk;
    for (int i = 0; i < n; i += 32) {
        h16 o[32];
        memset(o, 0, sizeof(o));
        for (int j = 0; j < cnt_per_row; j++) {
            const h16 *z = w_zero + (long)i * k / Actk + 32 * j;
            for (int ch = 0; ch < 32; ch++) o[ch] = hmac(o[ch], input_sum[j], z[ch], fused);
        }
        memcpy(output + i, o, sizeof(o));
    }
    elutq_ref_lut(k, input, lut);
    for (int i = 0; i < bit; i++) {
        long weight_bias = (long)i * k * n / 8;
        long w_scale_bias = (long)i * k * n / Actk;
        update_plane_scalar(output, weight + weight_bias, k, n, lut, w_scale + w_scale_bias, Actk, fused);
    }
    if (bias)
        for (int j = 0; j < n; j++) output[j] = hadd(output[j], bias[j]);
}

/* arm_gemm.cpp:312-360: N split into ceil(n/T) chunks, one per thread, on the
 * rearranged buffers.  Scratch per thread: k/Actk input sums + its own LUT
 * (the reference shares one LUT scratch between threads, each writing the same
 * values; private copies give the same results without the benign race).
 * Returns 0, or -1 if scratch allocation fails. */
int elutq_ref_gemv(int k, int n, const h16 *input, h16 *output, const uint8_t *weight,
                   const h16 *w_scale, const h16 *w_zero, const h16 *bias, int Actk, int bit,
                   int threadnum, int fused)
{
    int chunk_size = (n + threadnum - 1) / threadnum;
    int fail = 0;
#pragma omp parallel for num_threads(threadnum) schedule(static, 1)
    for (int i = 0; i < threadnum; i++) {
        int start = chunk_size * i;
        int end = MINI(start + chunk_size, n);
        if (start >= end) continue;
        h16 *input_sum = (h16 *)malloc(sizeof(h16) * (size_t)(k / Actk));
        h16 *lut = (h16 *)malloc(sizeof(h16) * (size_t)k * 4);
        if (!input_sum || !lut) { fail = 1; free(input_sum); free(lut); continue; }
        run_chunk(k, end - start, input, weight + (long)bit * start * k / 8,
                  w_scale + (long)bit * start * k / Actk, w_zero + (long)start * k / Actk,
                  bias ? bias + start : NULL, output + start, Actk, bit, input_sum, lut, fused);
        free(input_sum);
        free(lut);
    }
    return fail ? -1 : 0;
}

/* arm_gemm.cpp:362-387: one GEMV per row; weights are re-streamed m times. */
int elutq_ref_gemm(int m, int k, int n, const h16 *input, h16 *output, const uint8_t *weight,
                   const h16 *w_scale, const h16 *w_zero, const h16 *bias, int Actk, int bit,
                   int threadnum, int fused)
{
    for (int i = 0; i < m; i++) {
        int rc = elutq_ref_gemv(k, n, input + (long)i * k, output + (long)i * n, weight, w_scale,
                                w_zero, bias, Actk, bit, threadnum, fused);
        if (rc) return rc;
    }
    return 0;
}

/* ------------------------------------------------------------------------- *
 * use_sparse = true: `bits - 1` dense planes and one block-sparse extra plane.
 * mask_data holds mask_len uint32: pairs (channel start, k start) of blocks of
 * 32 channels x Actk inputs, grouped by ascending channel start.
 * ------------------------------------------------------------------------- */

/* arm_t_mac_kernal.cpp:554-647.  weight / w_scale hold the dense part followed
 * by the blocks' bits ([32][Actk/8] each) / scales ([32] each); the scale tail
 * is left as it is (the reference permutes the dense part in place). */
int elutq_ref_rearrange_sparse(int out_channel, int in_channel, int bits, int Actk,
                               const uint32_t *mask_data, uint32_t mask_len,
                               const uint8_t *weight, const h16 *w_scale, const h16 *w_zero,
                               uint8_t *weight_out, h16 *w_scale_out, h16 *w_zero_out)
{
    (void)mask_data;
    int base_bit = bits - 1;
    long index = 0;
    for (int bit = 0; bit < base_bit; bit++) {
        const uint8_t *ws = weight + (long)bit * out_channel * in_channel / 8;
        for (int i = 0; i < out_channel; i += 32)
            for (int j = 0; j < in_channel / 8; j++)
                for (int k = 0; k < 32; k++)
                    weight_out[index++] = ws[(long)(i + k) * in_channel / 8 + j];
    }
    long len = (long)mask_len;
    const uint8_t *wsp = weight + (long)base_bit * out_channel * in_channel / 8;
    for (long i = 0; i < len; i += 2)
        for (int j = 0; j < Actk / 8; j++)
            for (int k = 0; k < 32; k++)
                weight_out[index++] = wsp[i * 2 * Actk + (long)k * Actk / 8 + j];
    if (index != (long)in_channel * out_channel * base_bit / 8 + len * 2 * Actk) return 0;

    index = 0;
    for (int bit = 0; bit < base_bit; bit++) {
        const h16 *ss = w_scale + (long)bit * out_channel * in_channel / Actk;
        for (int i = 0; i < out_channel; i += 32)
            for (int j = 0; j < in_channel; j += Actk)
                for (int k = 0; k < 32; k++)
                    w_scale_out[index++] = ss[(long)(i + k) * in_channel / Actk + j / Actk];
    }
    if (index != (long)base_bit * in_channel * out_channel / Actk) return 0;
    memcpy(w_scale_out + index, w_scale + index, sizeof(h16) * (size_t)(len / 2 * 32));

    index = 0;
    for (int i = 0; i < out_channel; i += 32)
        for (int j = 0; j < in_channel; j += Actk)
            for (int k = 0; k < 32; k++)
                w_zero_out[index++] = w_zero[(long)(i + k) * in_channel / Actk + j / Actk];
    if (index != (long)in_channel * out_channel / Actk) return 0;
    return 1;
}

/* arm_t_mac_kernal.cpp:678-788.  `out` is the layer's whole output vector:
 * the channel start in the mask is absolute. */
static void update_plane_sparse(h16 *out, const uint8_t *weight, const h16 *lut, const h16 *w_scale,
                                const uint32_t *mask_data, int len, int ActK, int fused)
{
    h16 c[32];
    for (int i = 0; i < len; i += 2) {
        int x = (int)mask_data[i];
        int y = (int)mask_data[i + 1];
        h16 acc[32];
        memset(acc, 0, sizeof(acc));
        for (int l = 0; l < ActK; l += 8) {
            const uint8_t *w = weight + (long)i * 2 * ActK + 4 * l;
            const h16 *lut_lo = lut + (long)((y + l) / 4) * 16;
            const h16 *lut_hi = lut + (long)((y + l) / 4 + 1) * 16;
            for (int ch = 0; ch < 32; ch++) {
                acc[ch] = hadd(acc[ch], lut_lo[w[ch] & 15]);
                acc[ch] = hadd(acc[ch], lut_hi[w[ch] >> 4]);
            }
        }
        const h16 *s = w_scale + (long)(i / 2) * 32;
        if (i == 0 || x != (int)mask_data[i - 2])
            for (int ch = 0; ch < 32; ch++) c[ch] = hmul(acc[ch], s[ch]);
        else
            for (int ch = 0; ch < 32; ch++) c[ch] = hmac(c[ch], acc[ch], s[ch], fused);
        if (i == len - 2 || x != (int)mask_data[i + 2])
            for (int ch = 0; ch < 32; ch++) out[x + ch] = hadd(out[x + ch], c[ch]);
    }
}

/* arm_gemm.cpp:725-808 (MultiThreadGemvW_lowbit_Activation_FP_Sparse::Run): all
 * pointers are the layer's, the thread's share is channels [start, end) and
 * mask entries [mask_start, mask_end). */
static void run_chunk_sparse(int k, int n, int start, int end, int mask_start, int mask_end,
                             const h16 *input, const uint8_t *weight, const h16 *w_scale,
                             const h16 *w_zero, const h16 *bias, const uint32_t *mask_data,
                             h16 *output, int Actk, int bit, h16 *input_sum, h16 *lut, int fused)
{
    for (int i = 0; i < k; i += Actk) {
        h16 s = 0;
        for (int j = 0; j < Actk; j++) s = hadd(s, input[i + j]);
        input_sum[i / Actk] = s;
    }
    int cnt_per_row = k / Actk;
    for (int i = start; i < end; i += 32) {
        h16 o[32];
        memset(o, 0, sizeof(o));
        for (int j = 0; j < cnt_per_row; j++) {
            const h16 *z = w_zero + (long)i * k / Actk + 32 * j;
            for (int ch = 0; ch < 32; ch++) o[ch] = hmac(o[ch], input_sum[j], z[ch], fused);
        }
        memcpy(output + i, o, sizeof(o));
    }
    elutq_ref_lut(k, input, lut);
    for (int i = 0; i < bit; i++) {
        if (i == bit - 1) {
            long weight_bias = (long)i * k * n / 8 + 2L * mask_start * Actk;
            long w_scale_bias = (long)i * k * n / Actk + (long)mask_start * 16;
            update_plane_sparse(output, weight + weight_bias, lut, w_scale + w_scale_bias,
                                mask_data + mask_start, mask_end - mask_start, Actk, fused);
        } else {
            long weight_bias = (long)i * k * n / 8 + (long)start * k / 8;
            long w_scale_bias = (long)i * k * n / Actk + (long)start * k / Actk;
            update_plane_scalar(output + start, weight + weight_bias, k, end - start, lut,
                                w_scale + w_scale_bias, Actk, fused);
        }
    }
    if (bias)
        for (int j = start; j < end; j++) output[j] = hadd(output[j], bias[j]);
}

/* arm_gemm.cpp:811-868: channels split into ceil(n/T) chunks; a thread takes the
 * mask entries whose channel start falls into its chunk (linear scans over the
 * sorted list).  `bit` counts the extra plane.  Returns 0, or -1 if scratch
 * allocation fails. */
int elutq_ref_gemv_sparse(int k, int n, const h16 *input, h16 *output, const uint8_t *weight,
                          const h16 *w_scale, const h16 *w_zero, const h16 *bias,
                          const uint32_t *mask_data, uint32_t mask_len, int Actk, int bit,
                          int threadnum, int fused)
{
    int chunk_size = (n + threadnum - 1) / threadnum;
    int fail = 0;
#pragma omp parallel for num_threads(threadnum) schedule(static, 1)
    for (int i = 0; i < threadnum; i++) {
        int start = chunk_size * i;
        int end = MINI(start + chunk_size, n);
        if (start >= end) continue;
        uint32_t ms = 0, me = 0;
        while (ms < mask_len && mask_data[ms] < (uint32_t)start) ms += 2;
        while (me < mask_len && mask_data[me] < (uint32_t)end) me += 2;
        h16 *input_sum = (h16 *)malloc(sizeof(h16) * (size_t)(k / Actk));
        h16 *lut = (h16 *)malloc(sizeof(h16) * (size_t)k * 4);
        if (!input_sum || !lut) { fail = 1; free(input_sum); free(lut); continue; }
        run_chunk_sparse(k, n, start, end, (int)ms, (int)me, input, weight, w_scale, w_zero, bias,
                         mask_data, output, Actk, bit, input_sum, lut, fused);
        free(input_sum);
        free(lut);
    }
    return fail ? -1 : 0;
}

/* ------------------------------------------------------------------------- *
 * Timed baseline: the same loop nest with 32-channel AVX2 tiles.  vpshufb on
 * the low- and high-byte halves of a chunk's 16 fp16 entries stands in for
 * vqtbl1q_u8; the looked-up halves are widened to fp32 (F16C) and accumulated
 * in fp32 within a group, so it deviates from the fp16 chain by rounding only.
 * ------------------------------------------------------------------------- */
static void update_plane_avx2(float *out, const uint8_t *weight, int in_channel, int out_channel,
                              const uint8_t *lut_lohi, const h16 *w_scale, int ActK)
{
    const __m256i mask = _mm256_set1_epi8(0x0f);
    for (int i = 0; i < out_channel; i += 32) {
        __m256 c0 = _mm256_setzero_ps(), c1 = c0, c2 = c0, c3 = c0;
        for (int j = 0; j < in_channel; j += ActK) {
            __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
            for (int l = 0; l < ActK; l += 8) {
                __m256i w = _mm256_loadu_si256((const __m256i *)(weight + ((long)i * in_channel) / 8 + (long)(j + l) * 4));
                __m256i lo = _mm256_and_si256(w, mask);
                __m256i hi = _mm256_and_si256(_mm256_srli_epi16(w, 4), mask);
                for (int half = 0; half < 2; half++) {
                    const uint8_t *t = lut_lohi + (long)((j + l) / 4 + half) * 32;
                    __m256i tl = _mm256_broadcastsi128_si256(_mm_loadu_si128((const __m128i *)t));
                    __m256i th = _mm256_broadcastsi128_si256(_mm_loadu_si128((const __m128i *)(t + 16)));
                    __m256i idx = half ? hi : lo;
                    __m256i bl = _mm256_shuffle_epi8(tl, idx);      /* low bytes, ch 0..31 */
                    __m256i bh = _mm256_shuffle_epi8(th, idx);      /* high bytes */
                    __m256i v0 = _mm256_unpacklo_epi8(bl, bh);      /* ch 0-7 | 16-23 */
                    __m256i v1 = _mm256_unpackhi_epi8(bl, bh);      /* ch 8-15 | 24-31 */
                    a0 = _mm256_add_ps(a0, _mm256_cvtph_ps(_mm256_castsi256_si128(v0)));
                    a1 = _mm256_add_ps(a1, _mm256_cvtph_ps(_mm256_castsi256_si128(v1)));
                    a2 = _mm256_add_ps(a2, _mm256_cvtph_ps(_mm256_extracti128_si256(v0, 1)));
                    a3 = _mm256_add_ps(a3, _mm256_cvtph_ps(_mm256_extracti128_si256(v1, 1)));
                }
            }
            const h16 *s = w_scale + (long)i * in_channel / ActK + (long)32 * j / ActK;
            c0 = _mm256_fmadd_ps(a0, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(s + 0))), c0);
            c1 = _mm256_fmadd_ps(a1, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(s + 8))), c1);
            c2 = _mm256_fmadd_ps(a2, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(s + 16))), c2);
            c3 = _mm256_fmadd_ps(a3, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(s + 24))), c3);
        }
        _mm256_storeu_ps(out + i + 0, _mm256_add_ps(_mm256_loadu_ps(out + i + 0), c0));
        _mm256_storeu_ps(out + i + 8, _mm256_add_ps(_mm256_loadu_ps(out + i + 8), c1));
        _mm256_storeu_ps(out + i + 16, _mm256_add_ps(_mm256_loadu_ps(out + i + 16), c2));
        _mm256_storeu_ps(out + i + 24, _mm256_add_ps(_mm256_loadu_ps(out + i + 24), c3));
    }
}

int elutq_ref_gemv_fast(int k, int n, const h16 *input, h16 *output, const uint8_t *weight,
                        const h16 *w_scale, const h16 *w_zero, const h16 *bias, int Actk, int bit,
                        int threadnum)
{
    int chunk_size = (n + threadnum - 1) / threadnum;
    int fail = 0;
#pragma omp parallel for num_threads(threadnum) schedule(static, 1)
    for (int t = 0; t < threadnum; t++) {
        int start = chunk_size * t;
        int end = MINI(start + chunk_size, n);
        if (start >= end) continue;
        int nl = end - start;
        int ng = k / Actk;
        float *xs = (float *)malloc(sizeof(float) * (size_t)ng);
        float *acc = (float *)malloc(sizeof(float) * (size_t)nl);
        h16 *lut = (h16 *)malloc(sizeof(h16) * (size_t)k * 4);
        uint8_t *lohi = (uint8_t *)malloc((size_t)k * 8);
        if (!xs || !acc || !lut || !lohi) { fail = 1; free(xs); free(acc); free(lut); free(lohi); continue; }
        for (int g = 0; g < ng; g++) {
            float s = 0.f;
            for (int j = 0; j < Actk; j++) s += h2f(input[g * Actk + j]);
            xs[g] = s;
        }
        const h16 *z = w_zero + (long)start * k / Actk;
        for (int i = 0; i < nl; i += 32)
            for (int ch = 0; ch < 32; ch++) {
                float s = 0.f;
                for (int g = 0; g < ng; g++) s += xs[g] * h2f(z[(long)i * ng + 32 * g + ch]);
                acc[i + ch] = s;
            }
        elutq_ref_lut(k, input, lut);
        for (long c = 0; c < k / 4; c++)          /* split entries into byte planes (vld2q_u8) */
            for (int e = 0; e < 16; e++) {
                lohi[c * 32 + e] = (uint8_t)(lut[c * 16 + e] & 0xff);
                lohi[c * 32 + 16 + e] = (uint8_t)(lut[c * 16 + e] >> 8);
            }
        for (int b = 0; b < bit; b++)
            update_plane_avx2(acc, weight + (long)bit * start * k / 8 + (long)b * k * nl / 8, k, nl, lohi,
                              w_scale + (long)bit * start * k / Actk + (long)b * k * nl / Actk, Actk);
        for (int j = 0; j < nl; j++)
            output[start + j] = f2h(acc[j] + (bias ? h2f(bias[start + j]) : 0.f));
        free(xs); free(acc); free(lut); free(lohi);
    }
    return fail ? -1 : 0;
}

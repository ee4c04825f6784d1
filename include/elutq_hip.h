/*
 * elutq_hip.h -- C ABI of libelutq_hip.so: the HLQ bit-serial LUT GEMV / small-batch
 * GEMM for AMD MI355X (gfx950).
 *
 * HLQ stores a linear layer's weight W[N][K] as
 *     W[n][k] = sum_b  s[b][n][k/G] * B_b[n][k]  +  z[n][k/G]
 * with `bits` binary planes B_b, fp16 per-plane group scales s and an fp16 group
 * zero z, groups of G = 64 or 128 consecutive k.
 *
 * The entry points replace, one for one, the reference's CPU operator for this
 * path (file:line under the reference tree, Nkniexin/ELUTQ):
 *
 *   elutq_hlq_repack_*      load_Parameter(..LINEAR..)        C++/ops/src/arm/parameters.cpp:8-70
 *                           t_mac_g4_rearrange_weight_normal_impl
 *                                                            C++/ops/src/arm/arm_t_mac_kernal.cpp:472-552
 *   elutq_hlq_gemv_f16      arm_gemm(m == 1, bit <= 4)        C++/ops/include/arm/arm_gemm.h:4-14
 *                           MultiThread_arm_gemv_w_lowbit_activation_fp_impl
 *                                                            C++/ops/src/arm/arm_gemm.cpp:312-360
 *   elutq_hlq_gemm_f16      arm_gemm(m  > 1, bit <= 4)        C++/ops/src/arm/arm_gemm.cpp:362-387
 *   elutq_hlq_dequant_f16   dequantize_with_scales            GPTQ/quant.py:176-183
 *   elutq_hlq_sparse_*      arm_gemm(use_sparse)              C++/ops/src/arm/arm_gemm.cpp:683-868, 894-920
 *                           t_mac_g4_float_update_sparse_impl C++/ops/src/arm/arm_t_mac_kernal.cpp:678-788
 *
 * Conventions
 *   - plain C types only; every `d_` pointer is DEVICE memory owned by the caller,
 *     every `h_` pointer is HOST memory owned by the caller;
 *   - compute calls are asynchronous on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream), never synchronise, never allocate, and are
 *     capturable in a HIP graph;
 *   - every function returns ELUTQ_OK (0) or a negative elutq_status; nothing throws;
 *   - a workspace is private to one in-flight call: calls that share a workspace
 *     must be ordered on one stream.  It must be zero-filled once after allocation
 *     (elutq_hlq_workspace_init).  Its first 64 KiB are zero between calls -- arrival counters and the
 *     slots in which the K slices of a GEMV meet live there, and every kernel puts the zeros back --
 *     so nothing else may write into a workspace; what lies behind the 64 KiB may hold anything.
 */
#ifndef ELUTQ_HIP_H
#define ELUTQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum elutq_status {
    ELUTQ_OK = 0,
    ELUTQ_ERR_NULL = -1,       /* a required pointer is NULL */
    ELUTQ_ERR_SHAPE = -2,      /* K < 128, K % group != 0, K % 128 != 0 (at group 64: K % 128 == 64 is accepted), N or M < 1 */
    ELUTQ_ERR_BITS = -3,       /* bits outside 1..4 */
    ELUTQ_ERR_GROUP = -4,      /* group not 64 or 128 */
    ELUTQ_ERR_WORKSPACE = -5,  /* workspace smaller than elutq_hlq_workspace_bytes() */
    ELUTQ_ERR_HIP = -6,        /* a HIP runtime call failed (launch, attribute) */
    ELUTQ_ERR_TUNING = -7,     /* explicit ksplit / waves arguments out of range */
    ELUTQ_ERR_SPARSE = -8,     /* malformed block list of a sparse extra plane */
    ELUTQ_ERR_STATIC_LIMIT = -9 /* the shape needs more scratch than the static buffer of the _static entry point holds */
} elutq_status;

/* Library version (major*10000 + minor*100 + patch). */
int elutq_version(void);

/* Static description of a status code. */
const char *elutq_status_string(int status);

/* Sizes, in bytes, of the three device buffers holding a repacked layer. */
size_t elutq_hlq_planes_bytes(int K, int N, int bits);
size_t elutq_hlq_scales_bytes(int K, int N, int bits, int group);
size_t elutq_hlq_zeros_bytes(int K, int N, int group);

/*
 * Host-side repack: the reference's export files, byte for byte
 * (GPTQ/HLQ.py:207-251: w_quant.bin uint8 [bits][N][K/8] packed LSB-first along K,
 * w_scale.bin fp16 [bits][N][K/G], w_zero.bin fp16 [N][K/G]) -> the layout the
 * kernels read.  Output buffers are host memory of the sizes above; copy them to
 * the device unchanged.  Pure permutation, no arithmetic.
 */
int elutq_hlq_repack_host(const uint8_t *h_w_quant, const uint16_t *h_w_scale,
                          const uint16_t *h_w_zero, int K, int N, int bits, int group,
                          void *h_planes_out, void *h_scales_out, void *h_zeros_out);

/* Inverse of elutq_hlq_repack_host (kernel layout -> export layout). */
int elutq_hlq_unpack_host(const void *h_planes, const void *h_scales, const void *h_zeros,
                          int K, int N, int bits, int group,
                          uint8_t *h_w_quant_out, uint16_t *h_w_scale_out, uint16_t *h_w_zero_out);

/*
 * Which kernel the batch-1 GEMV entry points launch (process-wide; for tests, benchmarks and debugging):
 *   ELUTQ_GEMV_ENGINE_LUT   activation tables in LDS, 4-bit lookups (the T-MAC scheme of the reference's
 *                           t_mac_g4_float_update_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:364-469)
 *   ELUTQ_GEMV_ENGINE_MFMA  the plane bits go to the matrix cores as fp4 operands against balanced base-7 digits
 *                           of the activations (fp4 x fp4 MFMA); no lookups
 *   ELUTQ_GEMV_ENGINE_AUTO  the library's choice per launch (the default): the LUT kernels for a single GEMV of up to
 *                           256 column blocks of 64 (its launch is latency bound and the tables are built sooner than
 *                           the digits); the matrix-core kernel where a launch streams many column blocks per
 *                           workgroup -- grouped launches, and plain calls on layers with more than 256 column blocks
 *                           and K > 4096
 * Both compute the same sums (fp32 fold per group and plane); results agree to the final fp16 rounding and
 * are bit-identical where the arithmetic is exact.  Returns ELUTQ_ERR_TUNING for another value.
 */
#define ELUTQ_GEMV_ENGINE_AUTO 0
#define ELUTQ_GEMV_ENGINE_LUT 1
#define ELUTQ_GEMV_ENGINE_MFMA 2
int elutq_hlq_set_gemv_engine(int engine);
int elutq_hlq_get_gemv_engine(void);

/* Workspace size for a call with up to M activation rows. */
size_t elutq_hlq_workspace_bytes(int K, int N, int bits, int group, int M);

/* Zero-fills a freshly allocated workspace (asynchronous on `stream`). */
int elutq_hlq_workspace_init(void *d_workspace, size_t workspace_bytes, void *stream);

/*
 * y[N] = W x + bias, batch 1.  d_x fp16 [K], d_y fp16 [N], d_bias fp16 [N] or NULL.
 * Replaces arm_gemm(m = 1, ...) for bit <= 4, use_sparse = false (use_sparse:
 * elutq_hlq_sparse_gemv_f16).
 */
int elutq_hlq_gemv_f16(const void *d_planes, const void *d_scales, const void *d_zeros,
                       const void *d_bias, const void *d_x, void *d_y,
                       int K, int N, int bits, int group,
                       void *d_workspace, size_t workspace_bytes, void *stream);

/*
 * elutq_hlq_gemv_f16 for callers that cannot allocate and bring no workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference
 * (whose arm_gemm takes a caller-owned temp_workplace, as elutq_hlq_gemv_f16 takes a workspace).
 * Same inputs, outputs and results, bit for bit, as elutq_hlq_gemv_f16; the arrival counters and
 * partial sums of a K-sliced launch live in a device array inside the library instead
 * (elutq_hlq_static_scratch_bytes() = 64 KiB + ELUTQ_STATIC_PARTIAL_BYTES per GPU, held until the process
 * ends).  The call allocates nothing and frees nothing.  Shapes whose launch would need more partial-sum
 * space -- slices * ceil(N/64)*64 * 4 bytes with slices = elutq_hlq_gemv_slices(K, N, bits, group, 0, 0) --
 * return ELUTQ_ERR_STATIC_LIMIT (every LLaMA-3-8B / LLaMA-2-13B projection fits many times over).
 * All calls on one GPU share that GPU's array: calls that may overlap on one GPU (two streams, two
 * threads) race on it and must be ordered by the caller.  elutq_hlq_static_init() looks the array's
 * device address up for the current device; the first call on a device does it otherwise (call it
 * once per device before capturing a graph).
 */
#define ELUTQ_STATIC_PARTIAL_BYTES (2u << 20)
size_t elutq_hlq_static_scratch_bytes(void);
int elutq_hlq_static_init(void);
int elutq_hlq_gemv_f16_static(const void *d_planes, const void *d_scales, const void *d_zeros,
                              const void *d_bias, const void *d_x, void *d_y,
                              int K, int N, int bits, int group, void *stream);

/*
 * Same computation with the launch shape chosen by the caller: `ksplit` slices of K
 * per column block (1..K/128) and `waves` wavefronts per workgroup
 * (1..16); 0 = library default.  For tuning and for tests that must reach every
 * reduction path; results do not depend on these beyond fp32 summation order.
 * ksplit = ELUTQ_GEMV_NARROW16 / ELUTQ_GEMV_NARROW32 (with waves = 0) names the narrow-tile kernel:
 * a workgroup owns 16 / 32 columns over all of K, so a layer with few column blocks fills the chip
 * without K slices; K <= 8192, else ELUTQ_ERR_TUNING.  With ksplit = waves = 0 the library takes it
 * where the layer has at most 64 / 128 column blocks of 64; ksplit = ELUTQ_GEMV_WIDE keeps it on the
 * wide-tile kernel (64 columns per wavefront) with the library's own K slicing -- the kernel a call with
 * slices to hand over (elutq_gemv_fusion.d_slices_out) always runs on.
 */
#define ELUTQ_GEMV_NARROW16 (-16)
#define ELUTQ_GEMV_NARROW32 (-32)
#define ELUTQ_GEMV_WIDE (-64)
int elutq_hlq_gemv_f16_tuned(const void *d_planes, const void *d_scales, const void *d_zeros,
                             const void *d_bias, const void *d_x, void *d_y,
                             int K, int N, int bits, int group,
                             void *d_workspace, size_t workspace_bytes, void *stream,
                             int ksplit, int waves);

/*
 * The batch-1 GEMV with its lookup tables quantized to int8, the reference's int8-LUT variant
 * (arm_gemv, C++/ops/src/arm/arm_gemv.cpp:4-34, which nothing in the reference calls): per
 * quantization group of `group` activations the table entries -- fp16 subset sums of four activations --
 * share one scale = fp16(max|entry| / 127) and become saturate_int8(round-to-nearest-even(entry / scale))
 * (t_mac_g4_groupsize32_calculate_lut_impl, C++/ops/src/arm/arm_t_mac_kernal.cpp:15-93); the looked-up
 * entries of a group are summed as integers and the sum is multiplied by that scale and the weight's scale
 * (t_mac_g4_int8_update_impl, :258-362).  Here the weights stay HLQ layers -- a scale per plane and
 * a zero point, of which the reference's uniform format (one scale, planes weighted 2^order, no zero)
 * is the special case scale[b] = 2^b scale[0], zero = 0 -- the zero term uses the exact activation sums
 * and everything after the integer sums is fp32 with one rounding to fp16.  A lossy mode (the tables
 * keep seven bits): offered for parity with the reference's inventory, not used by any path here.
 * Arguments as elutq_hlq_gemv_f16; runs on the wide-tile LUT kernel.
 */
int elutq_hlq_gemv_int8lut_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                               const void *d_x, void *d_y, int K, int N, int bits, int group,
                               void *d_workspace, size_t workspace_bytes, void *stream);

/*
 * Batch-1 GEMV fused with the ops that surround a projection in a decoder layer, so a
 * decode step needs one launch where the reference runs two or three operators:
 *   prologue 1  x <- fp16(rmsnorm(x) * norm_weight)     launch_pre_rms_norm + arm_gemm
 *                                                       (C++/ops/src/arm/arm_rmsnorm.cpp:25-84)
 *   prologue 2  x <- fp16(silu(x[0:K]) * x[K:2K])        gated_silu + arm_gemm; d_x holds 2K values
 *                                                       (C++/ops/src/arm/arm_activation.cpp:22-53)
 *   d_residual  y <- y + residual (fp16 [N])            the residual add folded into the next
 *                                                       norm in the reference (arm_rmsnorm.cpp:43-85)
 * `fusion` is a HOST pointer (read before the call returns) or NULL for a plain GEMV.
 * ksplit / waves as in elutq_hlq_gemv_f16_tuned.
 *
 * A projection whose K is divided among workgroups can leave the sum of its K slices to the
 * projection that reads its output (in a decoder layer: o -> gate|up, down -> the next
 * layer's q|k|v), which saves the producing launch the meeting of its slices in device memory:
 *   producer  d_slices_out = fp32 [S][N], S = elutq_hlq_gemv_slices(K, N, bits, group, ksplit, waves) >= 2,
 *             N % 64 == 0: every slice's partial sums are stored there and d_y is NOT written;
 *             no bias and no d_residual (the consumer adds the residual)
 *   consumer  prologue 1 with n_slices_in = S (at most 4), d_slices_in = that buffer (row stride K),
 *             d_x = the residual: x <- fp16(((s0 + s1) + ...) + d_x) element by element, i.e. what
 *             the producer would have written with d_residual = d_x, bit for bit; the RMSNorm
 *             follows.  d_x_out (fp16 [K], or NULL; not d_x) receives that x for later readers.
 *             The consuming launch must have at most one tile per compute unit
 *             (ceil(N/64) * slices <= 256 on the wide-tile kernel; the narrow-tile kernel always has);
 *             wider projections return ELUTQ_ERR_TUNING.
 * No counterpart in the reference, whose operators run one after the other on whole vectors.
 */
typedef struct elutq_gemv_fusion {
    int prologue;               /* 0, 1 or 2 */
    float eps;                  /* RMSNorm epsilon (prologue 1) */
    const void *d_norm_weight;  /* fp16 [K] (prologue 1) */
    const void *d_residual;     /* fp16 [N] or NULL */
    void *d_slices_out;         /* producer of deferred K slices, or NULL */
    const void *d_slices_in;    /* consumer of deferred K slices (n_slices_in > 0) */
    int n_slices_in;            /* 0 = none */
    void *d_x_out;              /* fp16 [K] or NULL (consumer only) */
    size_t slices_out_bytes;    /* size of d_slices_out: at least S * N * 4 or the call returns ELUTQ_ERR_WORKSPACE */
    size_t slices_in_bytes;     /* size of d_slices_in: at least n_slices_in * K * 4 or ELUTQ_ERR_WORKSPACE */
} elutq_gemv_fusion;

/*
 * The K slices of a GEMV launch that meet through the zero-kept head of the workspace have one workgroup per column
 * block wait for the others' partial sums.  That wait is bounded (about a second); should it ever run out -- the
 * launch could not get its workgroups placed, say because many launches oversubscribe the GPU -- the block's 64
 * outputs are written as NaN and the event is counted in a word the library keeps on each GPU.  This call returns
 * that count for the current device (>= 0; it synchronizes with the device) and sets it back to zero if `clear`
 * is non-zero; negative: an elutq_status.  After a non-zero count the workspaces of the affected calls must be
 * zero-filled again (elutq_hlq_workspace_init) before they are reused.  No counterpart in the reference, whose
 * thread pool waits without a bound (C++/common/include/threadpool.h:107-113).
 */
int elutq_hlq_gemv_fault_count(int clear);

/* K slices the GEMV launch of this shape is divided into (ksplit / waves as in
 * elutq_hlq_gemv_f16_tuned, 0 = default); 0 for an unsupported shape or tuning.  With ksplit = 0 the
 * figure is that of the wide-tile kernel, on which a producer of handed-over slices runs (and an upper
 * bound otherwise: the narrow-tile kernel has no slices). */
int elutq_hlq_gemv_slices(int K, int N, int bits, int group, int ksplit, int waves);

/* 1 if a launch of this shape (ksplit / waves as the call would pass them) accepts `n_slices`
 * handed-over K slices (elutq_gemv_fusion.n_slices_in) in its RMSNorm prologue, else 0: the limits the
 * launch itself applies (1..4 slices, at most one tile per compute unit, tables plus the fp16 [K]
 * staging area within the LDS).  A caller decides with it, before it lets a producer leave its slices
 * unsummed, whether the consumer can take them. */
int elutq_hlq_gemv_accepts_slices(int K, int N, int bits, int group, int ksplit, int waves, int n_slices);

int elutq_hlq_gemv_fused_f16(const void *d_planes, const void *d_scales, const void *d_zeros,
                             const void *d_bias, const void *d_x, void *d_y,
                             int K, int N, int bits, int group,
                             void *d_workspace, size_t workspace_bytes, void *stream,
                             const elutq_gemv_fusion *fusion, int ksplit, int waves);

/*
 * Many independent batch-1 GEMVs in one launch (same bits and group size; any shapes).  The
 * reference issues arm_gemm once per projection (llama::forward, C++/examples/models/llama.cpp:
 * 244-739); projections that do not depend on each other -- q, k and v of a layer, gate and up,
 * the layers of a benchmark sweep -- can instead share one launch, which pays the launch, the
 * first memory round trips and the tail once and keeps HBM streaming across GEMV boundaries.
 * A plan holds the device-side problem list: create it once (allocates and copies; not
 * capturable), run it any number of times (one kernel launch, capturable), destroy it.
 * The workspace (elutq_hlq_gemv_group_workspace_bytes, zero-filled once) is bound at creation
 * and must not be shared with calls that may run concurrently.  On the LUT engine the results equal those of
 * elutq_hlq_gemv_f16_tuned with the same K slicing, which the group chooses itself.  On the matrix-core engine
 * (the default for a group whose layers all have K % 128 == 0) every workgroup streams one contiguous share of
 * all the layers' bytes and a tile covers all of K, so nothing meets in device memory and the workspace is not
 * used; a layer's sums are the same numbers added in an order that depends on where its tiles fall in the plan:
 * bit-identical from run to run of a plan, within the final fp16 rounding of any other launch of the layer,
 * exact where the arithmetic is exact.
 */
typedef struct elutq_gemv_problem {
    const void *d_planes, *d_scales, *d_zeros, *d_bias;  /* as for elutq_hlq_gemv_f16; bias may be NULL */
    const void *d_x;                                      /* fp16 [K] */
    void *d_y;                                            /* fp16 [N] */
    int K, N;
} elutq_gemv_problem;

size_t elutq_hlq_gemv_group_workspace_bytes(const elutq_gemv_problem *problems, int count, int bits, int group);
int elutq_hlq_gemv_group_create(const elutq_gemv_problem *problems, int count, int bits, int group,
                                void *d_workspace, size_t workspace_bytes, void **plan);
int elutq_hlq_gemv_group_run(void *plan, void *stream);
int elutq_hlq_gemv_group_destroy(void *plan);

/*
 * y[M][N] = x[M][K] W^T + bias, row-major fp16, 1 <= M.  Replaces arm_gemm(m > 1, ...),
 * which the reference defines as one GEMV per row.
 */
int elutq_hlq_gemm_f16(const void *d_planes, const void *d_scales, const void *d_zeros,
                       const void *d_bias, const void *d_x, void *d_y,
                       int M, int K, int N, int bits, int group,
                       void *d_workspace, size_t workspace_bytes, void *stream);

/*
 * Same computation with the launch shape chosen by the caller: `kparts` K parts inside a
 * workgroup (8 = its eight waves, or 0 for the default, which is the same; anything else
 * returns ELUTQ_ERR_TUNING) and `ksplit` K slices across workgroups (1..K/128); 0 = library
 * default.  The workspace must hold 64 KiB + ksplit * (M <= 32 ? 32 : 64) * ceil(N/64)*64 * 4
 * bytes when the shape ends up with more than one slice.  For tuning and for tests that must
 * reach every reduction path; results do not depend on these beyond fp32 summation order.
 */
int elutq_hlq_gemm_f16_tuned(const void *d_planes, const void *d_scales, const void *d_zeros,
                             const void *d_bias, const void *d_x, void *d_y,
                             int M, int K, int N, int bits, int group,
                             void *d_workspace, size_t workspace_bytes, void *stream,
                             int kparts, int ksplit);

/*
 * Decode-step glue between the q|k|v projection and the o projection, one launch per layer:
 * half-split RoPE on q and k at position *d_pos, append of k and v to the caches at that
 * position, single-token grouped-query attention over positions 0..*d_pos, fp16 output
 * [n_heads * head_dim].  Replaces launch_llama_qkv_apply_rotary + arm_cache + arm_attention
 * (C++/ops/src/arm/arm_rotary.cpp:4-89, arm_cache.cpp:17-22, arm_attention.cpp:162-316).
 * d_qkv fp16 [n_heads*d | n_kv_heads*d | n_kv_heads*d]; caches fp16 [max_seq][n_kv_heads][d];
 * d_pos a DEVICE int64 (so a captured graph can advance it); head_dim even, <= 128.
 * If *d_pos is outside [0, max_seq) the kernel reads and caches nothing and fills d_out with fp16 NaN, so that
 * a step beyond the cache shows in the logits instead of passing with the previous step's attention output.
 */
int elutq_decode_rope_attn_f16(const void *d_qkv, void *d_k_cache, void *d_v_cache, const void *d_pos,
                               void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                               float rope_base, void *stream);

/*
 * The same operator with the cached positions of every head divided among `splits`
 * workgroups (1..8; 0 = about one workgroup per CU), which meet in `d_workspace`
 * (elutq_decode_attn_workspace_bytes(n_heads, head_dim, splits) bytes, zero-filled once like the
 * GEMV workspace, which it may share: calls on one stream leave its counters at zero).  One
 * compute unit takes in a cache of a few hundred rows no faster than the whole chip takes in
 * all heads', so long contexts want the split.  The workgroups of a head read *d_pos and take
 * part only as far as the context warrants (up to 192 positions: one workgroup; up to 768: at most
 * four; beyond: all), so short contexts do not pay for the meeting.  head_dim other than 128
 * runs unsplit.
 * No counterpart in the reference beyond the operators elutq_decode_rope_attn_f16 replaces.
 */
size_t elutq_decode_attn_workspace_bytes(int n_heads, int head_dim, int splits);
int elutq_decode_rope_attn_split_f16(const void *d_qkv, void *d_k_cache, void *d_v_cache, const void *d_pos,
                                     void *d_out, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                     float rope_base, int splits, void *d_workspace, size_t workspace_bytes,
                                     void *stream);

/*
 * The same operator reading q|k|v as the unsummed K slices of the projection that produced it
 * (elutq_gemv_fusion.d_slices_out of that launch: fp32 rows of slice_stride floats, n_slices 1..4):
 * every element is fp16(((s0 + s1) + ...)), bit for bit what the projection would have stored.  A
 * workgroup reads only its own head's 3 x 128 elements, so the sum costs it next to nothing, while
 * the projection is spared the meeting of its slices in device memory.  head_dim 128 only.
 * No counterpart in the reference.
 */
int elutq_decode_rope_attn_sliced_f16(const void *d_qkv_slices, int n_slices, int slice_stride, void *d_k_cache,
                                      void *d_v_cache, const void *d_pos, void *d_out, int n_heads,
                                      int n_kv_heads, int head_dim, int max_seq, float rope_base, int splits,
                                      void *d_workspace, size_t workspace_bytes, void *stream);

/*
 * Tail of a decode step.  elutq_decode_rmsnorm_f16: out[i] = fp16(x[i] * rsqrt(mean(x^2) + eps)
 * * weight[i]), statistics in fp32 (launch_pre_rms_norm, C++/ops/src/arm/arm_rmsnorm.cpp:25-84).
 * elutq_decode_argmax_f16: *d_token (DEVICE int64) = first index of the strict maximum of the
 * fp16 logits (arm_argmax_last, C++/ops/src/arm/arm_argmax.cpp:3-30; NaNs never win), and, if
 * d_pos is not NULL, *d_pos (DEVICE int64) += 1 -- so a captured graph advances its own state.
 */
/*
 * Dense fp16 GEMV, y[n] = fp16(sum_k W[n][k] x[k] + bias[n]) with W fp16 [N][K] row-major: the bit == 16
 * branch of arm_gemm (C++/ops/src/arm/arm_gemm.cpp:883-886, MultiThreadGemvFP::Run :586-626), which a decode
 * step runs for an lm_head that was exported unquantized (lm_head.bin, C++/examples/models/llama.cpp:78).
 * Products and sums in fp32, one rounding (the reference accumulates in fp16).  d_norm_weight not NULL:
 * x <- fp16(x * rsqrt(mean(x^2) + eps) * norm_weight) first, i.e. the final launch_pre_rms_norm of the step
 * (C++/ops/src/arm/arm_rmsnorm.cpp:25-84) in the same launch.  d_bias may be NULL.  K % 8 == 0, 8 <= K <= 32768,
 * d_weight 16-byte aligned; no workspace.
 */
int elutq_fp16_gemv_f16(const void *d_weight, const void *d_bias, const void *d_x, void *d_y, int K, int N,
                        const void *d_norm_weight, float eps, void *stream);

/* Head of a decode step: out[0:hidden] = embed[*d_token][0:hidden], fp16 (arm_embedding,
 * C++/ops/src/arm/arm_embedding.cpp:4-20).  d_token is a DEVICE int64, so a captured graph follows the
 * token the previous step picked; a token outside [0, vocab) gives a zero row (the reference would read
 * outside the table).  hidden % 8 == 0, d_embed 16-byte aligned. */
int elutq_decode_embed_f16(const void *d_embed, const void *d_token, void *d_out, int hidden, int vocab, void *stream);
int elutq_decode_rmsnorm_f16(const void *d_x, const void *d_weight, void *d_out, int n, float eps, void *stream);
int elutq_decode_argmax_f16(const void *d_logits, int n, void *d_token, void *d_pos, void *stream);
/* The same pick by 64 workgroups that meet in `d_workspace` (64 KiB + 512 bytes, zero-filled once like
 * every workspace, which it may share: the call leaves its counter at zero): 128256 logits take one
 * workgroup 9 us and the 64 together 5.5 us.  Vectors under 65536 values (where the meeting costs more than
 * it saves) or not 16-byte aligned, and calls without a workspace, run the single-workgroup kernel. */
int elutq_decode_argmax_ws_f16(const void *d_logits, int n, void *d_token, void *d_pos, void *d_workspace,
                               size_t workspace_bytes, void *stream);

/* W[N][K] fp16 row-major from the repacked buffers (dequantize_with_scales). */
int elutq_hlq_dequant_f16(const void *d_planes, const void *d_scales, const void *d_zeros,
                          void *d_w_out, int K, int N, int bits, int group, void *stream);

/*
 * Block-sparse extra plane (weight_config.json "use_sparse": true).  Such a layer has
 * `base_bit` dense planes -- handled by the entry points above with bits = base_bit -- and
 * one more plane that exists only on listed blocks of 32 output channels x `group` inputs,
 * each block with 32 fp16 scales and no zero term.  As the reference's loader reads them
 * (C++/ops/src/arm/parameters.cpp:19-64):
 *   weight_mask.bin  uint32 pairs (channel start, k start), sparse_mask_len values, blocks of one
 *                    channel start adjacent and channel starts ascending;
 *   w_quant.bin      after the dense planes: block i as uint8 [32][group/8], LSB-first along K;
 *   w_scale.bin      after the dense scales: block i as fp16 [32].
 * The block bits and scales go to the device unchanged (no counterpart of
 * t_mac_g4_rearrange_weight_sparse_impl, arm_t_mac_kernal.cpp:554-647, is needed);
 * elutq_hlq_sparse_index_host turns the pair list into the index the kernels read
 * (elutq_hlq_sparse_index_bytes(N, nblk) bytes, nblk = mask_len / 2; copy it to the device
 * unchanged).  It rejects (ELUTQ_ERR_SPARSE) an odd mask_len, a channel start that is not a
 * multiple of 32 or not below N, a k start that is not a multiple of 4 or with k + group > K,
 * and descending channel starts.
 *
 * elutq_hlq_sparse_gemv_f16 / elutq_hlq_sparse_gemm_f16: the whole layer,
 *   y[m][n] = dense part + sum over the blocks on n's tile of scale * sum_{k in block, bit set} x[m][k],
 * as arm_gemm does for use_sparse (arm_gemm.cpp:894-920; the plane itself replaces
 * t_mac_g4_float_update_sparse_impl as called from arm_gemm.cpp:779-790).  Two launches on
 * `stream`: the plane's term in fp32 into the tail of the workspace, then the dense kernel, which
 * adds it before its one rounding to fp16.  `bits` counts the dense planes (base_bit).  The
 * workspace must hold elutq_hlq_sparse_workspace_bytes(K, N, bits, group, M) bytes, zero-filled
 * once like every workspace; d_blocks and d_x (and a norm weight) must be 4-byte aligned (ELUTQ_ERR_SHAPE).  elutq_hlq_sparse_dequant_add_f16: the plane added to a dense fp16
 * W [N][K] (after elutq_hlq_dequant_f16; W is then rounded twice).
 *
 * elutq_hlq_sparse_gemv_fused_f16: elutq_hlq_sparse_gemv_f16 in a decode step, i.e. with the prologue
 * and residual of elutq_hlq_gemv_fused_f16 (`fusion`, `ksplit`, `waves` as there; arm_gemm takes
 * use_sparse on any call, arm_gemm.cpp:894-920, so a layer held as blocks can stand anywhere in
 * llama.cpp:204-617).  The plane's launch forms the projection's input from the same stored vectors
 * with the same operations as the dense launch's prologue.  K slices handed over by, or left to,
 * another launch (d_slices_in / d_slices_out) are refused: ELUTQ_ERR_TUNING.
 *
 * The inline form -- one launch per layer.  Where every block lies on the grid of the quantization groups (k start a
 * multiple of `group`) and no two blocks share a cell, the batch-1 GEMV can look the blocks up in the activation tables
 * it builds for the dense planes anyway, as t_mac_g4_float_update_sparse_impl (arm_t_mac_kernal.cpp:678-788) looks
 * them up in the LUT of the dense update.  elutq_hlq_sparse_inline_host writes that form (per (column block, unit) a
 * record number, per record the 64 lanes' plane bits in the dense planes' layout and their fp16 scales) into h_out,
 * elutq_hlq_sparse_inline_bytes(K, N, group, nblk) bytes at most, *bytes_used of them used (may be NULL); copy it to
 * the device unchanged.  ELUTQ_ERR_SPARSE for a block list the form cannot hold (off the grid, repeated, malformed):
 * such a layer keeps the two-launch entry points above.  elutq_hlq_sparse_gemv_inline_f16 is elutq_hlq_gemv_fused_f16
 * (fusion may be NULL; prologues, residual, K slices handed over or left to the next launch as there) on such a layer,
 * `bits` = base_bit <= 3, on the table-lookup kernels (wide or narrow tiles as for a dense layer); the workspace is that of the dense layer;
 * `inline_bytes` = the bytes of the form on the device (*bytes_used): less than the layer's cell table is ELUTQ_ERR_WORKSPACE, and a
 * record number that points beyond it counts as "no block" instead of being followed.  The
 * result is the dense fp32 sum plus the blocks' terms, rounded once.
 */
size_t elutq_hlq_sparse_index_bytes(int N, int nblk);
int elutq_hlq_sparse_index_host(const uint32_t *h_mask, int mask_len, int K, int N, int group, void *h_index_out);
size_t elutq_hlq_sparse_workspace_bytes(int K, int N, int bits, int group, int M);
int elutq_hlq_sparse_gemv_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                              const void *d_x, void *d_y, int K, int N, int bits, int group,
                              void *d_workspace, size_t workspace_bytes, void *stream);
int elutq_hlq_sparse_gemm_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                              const void *d_x, void *d_y, int M, int K, int N, int bits, int group,
                              void *d_workspace, size_t workspace_bytes, void *stream);
int elutq_hlq_sparse_gemv_fused_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                    const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                                    const void *d_x, void *d_y, int K, int N, int bits, int group,
                                    void *d_workspace, size_t workspace_bytes, void *stream,
                                    const elutq_gemv_fusion *fusion, int ksplit, int waves);
int elutq_hlq_sparse_dequant_add_f16(const void *d_blocks, const void *d_blk_scales, const void *d_index, int nblk,
                                     void *d_w, int K, int N, int group, void *stream);
size_t elutq_hlq_sparse_inline_bytes(int K, int N, int group, int nblk);
int elutq_hlq_sparse_inline_host(const uint32_t *h_mask, int mask_len, const void *h_blocks, const void *h_blk_scales,
                                 int K, int N, int group, void *h_out, size_t *bytes_used);
int elutq_hlq_sparse_gemv_inline_f16(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                     const void *d_inline, size_t inline_bytes, const void *d_x, void *d_y, int K, int N,
                                     int bits, int group, void *d_workspace, size_t workspace_bytes, void *stream,
                                     const elutq_gemv_fusion *fusion, int ksplit, int waves);

#ifdef __cplusplus
}
#endif
#endif /* ELUTQ_HIP_H */

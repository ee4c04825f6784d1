// Calls between the library's own source files (not part of the C ABI).
#pragma once
#include <stddef.h>

#include "../../include/elutq_hip.h"

#define HLQ_INTERNAL __attribute__((visibility("hidden")))

// elutq_hlq_gemv_fused_f16 with an fp32 vector [N] (device) added to every output before it is
// rounded to fp16; d_extra may be null.  The matrix-core kernel has no instance that reads both the
// extra term and a prologue / residual (ELUTQ_ERR_TUNING where that engine is selected); no kernel
// leaves K slices to the next launch with an extra term due.
HLQ_INTERNAL int hlq_gemv_with_extra(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                     const void *d_x, void *d_y, int K, int N, int bits, int group, void *d_workspace,
                                     size_t workspace_bytes, void *stream, const elutq_gemv_fusion *fusion, int ksplit,
                                     int waves, const float *d_extra);

// elutq_hlq_gemv_fused_f16 on a layer whose block-sparse extra plane is held in its inline form (hlq_layout.h) on the
// device (`sp_inline_bytes` of it): one launch of a LUT kernel, which looks the blocks up in the tables it has built.
HLQ_INTERNAL int hlq_gemv_with_inline_sparse(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                                             const void *d_sp_inline, size_t sp_inline_bytes, const void *d_x, void *d_y, int K, int N, int bits,
                                             int group, void *d_workspace, size_t workspace_bytes, void *stream,
                                             const elutq_gemv_fusion *fusion, int ksplit, int waves);

// One launch of the MFMA GEMM kernel, 1 <= M <= HLQ_GEMM_MAX_M rows, with an fp32 [M][N] term
// (device) added to every output before it is rounded to fp16; d_extra may be null.
HLQ_INTERNAL int hlq_gemm_chunk_with_extra(const void *d_planes, const void *d_scales, const void *d_zeros,
                                           const void *d_bias, const void *d_x, void *d_y, int M, int K, int N, int bits,
                                           int group, void *d_workspace, size_t workspace_bytes, void *stream, int kparts,
                                           int ksplit, const float *d_extra);

// The matrix-core GEMV kernel (hlq_gemv_mfma.hip).  `gemv_args` is the launcher's argument block as
// hlq_gemv.hip fills it for the LUT kernel (hlq_gemv_dev.h: GemvArgs); ELUTQ_ERR_TUNING if a wave would
// have to hold more than two unit pairs.  hlq_gemv_mfma_lds_bytes: dynamic LDS of a launch without staged
// activations.
HLQ_INTERNAL int hlq_gemv_mfma_launch(const void *gemv_args, size_t args_bytes, int bits, int group, int waves,
                                      size_t stage_bytes, void *stream);
HLQ_INTERNAL size_t hlq_gemv_mfma_lds_bytes(int ups, int waves);
// Grouped launch of the matrix-core kernel.  hlq_gemv_mfma_group_plan cuts the column blocks of `count` layers
// (units[i] = K / 128, ncbs[i] = ceil(N / 64)) into `grid` contiguous shares of equal bytes and writes the tile list
// into h_blob (null: only the size is returned); the launch takes that blob on the device and a device array of the
// launcher's argument blocks (pointers, N, U, K, NT, ncb are read).  A tile covers all of K, so no workspace is used.
HLQ_INTERNAL size_t hlq_gemv_mfma_group_plan(const int *units, const int *ncbs, int count, int grid, void *h_blob);
HLQ_INTERNAL size_t hlq_gemv_mfma_group_lds_bytes(void);
HLQ_INTERNAL int hlq_gemv_mfma_group_launch(int bits, int group, const void *d_problems, const void *d_blob, int grid,
                                            void *stream);

// The same streaming kernel for one plain GEMV of a layer with many column blocks (no prologue, residual, extra term,
// handed-over slices; K a multiple of 128): every workgroup takes an equal share of the column blocks over all of K,
// so the launch uses no workspace.
HLQ_INTERNAL int hlq_gemv_mfma_wide_launch(const void *gemv_args, size_t args_bytes, int bits, int group, void *stream);

// The narrow-tile LUT GEMV kernel (hlq_gemv_narrow.hip): a workgroup owns `cw` = 16 or 32 columns over all of K,
// no K slices.  hlq_gemv_narrow_rounds: units per unit lane of a wave for a layer of U = K / 128 units, 0 where the
// kernel has no instance for it (its tables of all of K must fit the LDS of one workgroup);
// hlq_gemv_narrow_lds_bytes: dynamic LDS of a launch without staged activations (0: no instance).  The launch
// takes the launcher's argument block like hlq_gemv_mfma_launch; prologues, bias, residual and handed-over
// slices (n_slices_in, with `stage_bytes` = 2 K) and the extra term as the wide-tile kernel, no slices left
// to the next launch (ELUTQ_ERR_TUNING).
HLQ_INTERNAL int hlq_gemv_narrow_rounds(int U, int cw);
HLQ_INTERNAL size_t hlq_gemv_narrow_lds_bytes(int U, int cw);
HLQ_INTERNAL int hlq_gemv_narrow_launch(const void *gemv_args, size_t args_bytes, int bits, int group, int cw,
                                        size_t stage_bytes, void *stream);

// elutq_hlq_gemv_f16_static: the batch-1 GEMV for callers that cannot allocate or bring a workspace
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The arrival
// counters and partial sums that a K-sliced launch keeps in the caller's workspace live instead in a
// file-scope device array of fixed size, one copy per GPU, held until the process ends.
#include <hip/hip_runtime.h>
#include <mutex>
#include <stdint.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"
#include "hlq_internal.h"

namespace {

constexpr size_t STATIC_SCRATCH_BYTES = (size_t)HLQ_WS_COUNTER_BYTES + ELUTQ_STATIC_PARTIAL_BYTES;

// Workspace of the static entry point: [64 KiB arrival counters][partial sums of the K slices].
// Zero when the code object is loaded; the kernels return every counter they use to zero.
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_lock;
void *g_scratch_ptr[MAX_DEVICES] = {};      // device address of `scratch` on each GPU (its name is not one)

// The device address of this GPU's copy of `scratch`, looked up once per device with that device current.
int scratch_address(void **out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return ELUTQ_ERR_HIP;
    std::lock_guard<std::mutex> hold(g_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return ELUTQ_ERR_HIP;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return ELUTQ_OK;
}

// Arrival counters of the column blocks this call uses, set to zero in front of the launch that counts on
// them (a fill kernel, not a memset node: the call may be recorded into a graph).
__global__ void clear_counters_kernel(unsigned *counters, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counters[i] = 0u;
}

}  // namespace

extern "C" {

size_t elutq_hlq_static_scratch_bytes(void) { return STATIC_SCRATCH_BYTES; }

int elutq_hlq_static_init(void)
{
    void *p = nullptr;
    return scratch_address(&p);
}

int elutq_hlq_gemv_f16_static(const void *d_planes, const void *d_scales, const void *d_zeros, const void *d_bias,
                              const void *d_x, void *d_y, int K, int N, int bits, int group, void *stream)
{
    const int slices = elutq_hlq_gemv_slices(K, N, bits, group, 0, 0);      // 0: a shape no launch accepts
    void *ws = nullptr;
    size_t ws_bytes = 0;
    const bool bad_args = slices == 0 || !d_planes || !d_scales || !d_zeros || !d_x || !d_y;    // the launch reports which
    if (!bad_args) {
        const HlqGeo g = hlq_geo(K, N, bits, group);
        const size_t need = (size_t)HLQ_WS_COUNTER_BYTES + (size_t)slices * g.ncb * HLQ_CB * sizeof(float);
        if (slices > 1 && ((size_t)g.ncb * sizeof(unsigned) > (size_t)HLQ_WS_COUNTER_BYTES || need > STATIC_SCRATCH_BYTES))
            return ELUTQ_ERR_STATIC_LIMIT;
        // the launch always gets the array (an engine other than the one the figure above is for may slice where that
        // one does not; its counters are at zero then, as every kernel leaves them)
        const int rc = scratch_address(&ws);
        if (rc != ELUTQ_OK) return rc;
        ws_bytes = STATIC_SCRATCH_BYTES;
        if (slices > 1 && (size_t)g.ncb * sizeof(unsigned) <= (size_t)HLQ_WS_COUNTER_BYTES) {
            hipLaunchKernelGGL(clear_counters_kernel, dim3((g.ncb + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                               (unsigned *)ws, g.ncb);
            if (hipGetLastError() != hipSuccess) return ELUTQ_ERR_HIP;
        }
    }
    // shape, pointer and plane-count errors are reported by the launch itself, as for elutq_hlq_gemv_f16.  The launch
    // checks the array's size against the slices it actually makes (the figure above is the wide-tile kernel's, an
    // upper bound for the LUT kernels; another engine may slice differently): too small reads as the static limit.
    const int rc = hlq_gemv_with_extra(d_planes, d_scales, d_zeros, d_bias, d_x, d_y, K, N, bits, group, ws, ws_bytes, stream,
                                       nullptr, 0, 0, nullptr);
    return rc == ELUTQ_ERR_WORKSPACE && ws ? ELUTQ_ERR_STATIC_LIMIT : rc;
}

}  // extern "C"

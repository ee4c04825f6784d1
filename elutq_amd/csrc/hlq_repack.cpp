// Host-side repack between the reference's export layout and the kernel layout.
// Counterpart of load_Parameter + t_mac_g4_rearrange_weight_normal_impl
// (C++/ops/src/arm/parameters.cpp:8-70, C++/ops/src/arm/arm_t_mac_kernal.cpp:472-552):
// like the reference's loader it is a pure permutation of bytes; unlike it, the result
// does not depend on a thread count.
#include <string.h>

#include "../../include/elutq_hip.h"
#include "hlq_layout.h"

namespace {

inline uint32_t rotl32(uint32_t v, int r) { return (v << r) | (v >> (32 - r)); }
inline uint32_t rotr32(uint32_t v, int r) { return (v >> r) | (v << (32 - r)); }

int check_shape(int K, int N, int bits, int group)
{
    if (bits < 1 || bits > 4) return ELUTQ_ERR_BITS;
    if (group != 64 && group != 128) return ELUTQ_ERR_GROUP;
    if (N < 1 || !hlq_k_ok(K, group)) return ELUTQ_ERR_SHAPE;
    return ELUTQ_OK;
}

}  // namespace

extern "C" {

size_t elutq_hlq_planes_bytes(int K, int N, int bits)
{
    if (check_shape(K, N, bits, 64) != ELUTQ_OK) return 0;      // (the size does not depend on the group size)
    return hlq_planes_bytes(hlq_geo(K, N, bits, 64));
}

size_t elutq_hlq_scales_bytes(int K, int N, int bits, int group)
{
    if (check_shape(K, N, bits, group) != ELUTQ_OK) return 0;
    return hlq_scales_bytes(hlq_geo(K, N, bits, group));
}

size_t elutq_hlq_zeros_bytes(int K, int N, int group)
{
    if (check_shape(K, N, 1, group) != ELUTQ_OK) return 0;
    return hlq_zeros_bytes(hlq_geo(K, N, 1, group));
}

int elutq_hlq_repack_host(const uint8_t *w_quant, const uint16_t *w_scale, const uint16_t *w_zero,
                          int K, int N, int bits, int group,
                          void *planes_out, void *scales_out, void *zeros_out)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!w_quant || !w_scale || !w_zero || !planes_out || !scales_out || !zeros_out) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    uint32_t *planes = (uint32_t *)planes_out;
    uint32_t *scales = (uint32_t *)scales_out;
    uint32_t *zeros = (uint32_t *)zeros_out;
    const size_t row_bytes = (size_t)K / 8;

    for (int cb = 0; cb < g.ncb; cb++) {
        for (int u = 0; u < g.U; u++)
            for (int b = 0; b < bits; b++) {
                uint32_t *dst = planes + (((size_t)cb * g.U + u) * bits + b) * HLQ_CB * 4;
                for (int lane = 0; lane < HLQ_CB; lane++) {
                    const int n = cb * HLQ_CB + lane;
                    uint32_t d[4] = {0, 0, 0, 0};
                    if (n < N) {
                        const size_t have = row_bytes - (size_t)u * 16;          // 8 in a last unit that K ends half way through
                        memcpy(d, w_quant + ((size_t)b * N + n) * row_bytes + (size_t)u * 16, have < 16 ? have : 16);
                        for (int i = 0; i < 4; i++) d[i] = rotl32(d[i], HLQ_ROT);
                    }
                    memcpy(dst + lane * 4, d, 16);
                }
            }
        for (int t = 0; t < g.NT; t++) {
            for (int b = 0; b < bits; b++) {
                uint32_t *dst = scales + (((size_t)cb * g.NT + t) * bits + b) * HLQ_CB;
                for (int lane = 0; lane < HLQ_CB; lane++) {
                    const int n = cb * HLQ_CB + lane;
                    uint32_t lo = 0, hi = 0;
                    if (n < N) {
                        const uint16_t *s = w_scale + ((size_t)b * N + n) * g.NG;
                        lo = s[2 * t];
                        if (2 * t + 1 < g.NG) hi = s[2 * t + 1];
                    }
                    dst[lane] = lo | (hi << 16);
                }
            }
            uint32_t *dz = zeros + ((size_t)cb * g.NT + t) * HLQ_CB;
            for (int lane = 0; lane < HLQ_CB; lane++) {
                const int n = cb * HLQ_CB + lane;
                uint32_t lo = 0, hi = 0;
                if (n < N) {
                    const uint16_t *z = w_zero + (size_t)n * g.NG;
                    lo = z[2 * t];
                    if (2 * t + 1 < g.NG) hi = z[2 * t + 1];
                }
                dz[lane] = lo | (hi << 16);
            }
        }
    }
    return ELUTQ_OK;
}

int elutq_hlq_unpack_host(const void *planes_in, const void *scales_in, const void *zeros_in,
                          int K, int N, int bits, int group,
                          uint8_t *w_quant_out, uint16_t *w_scale_out, uint16_t *w_zero_out)
{
    int rc = check_shape(K, N, bits, group);
    if (rc != ELUTQ_OK) return rc;
    if (!planes_in || !scales_in || !zeros_in || !w_quant_out || !w_scale_out || !w_zero_out) return ELUTQ_ERR_NULL;
    const HlqGeo g = hlq_geo(K, N, bits, group);
    const uint32_t *planes = (const uint32_t *)planes_in;
    const uint32_t *scales = (const uint32_t *)scales_in;
    const uint32_t *zeros = (const uint32_t *)zeros_in;
    const size_t row_bytes = (size_t)K / 8;

    for (int n = 0; n < N; n++) {
        const int cb = n / HLQ_CB, lane = n % HLQ_CB;
        for (int b = 0; b < bits; b++) {
            for (int u = 0; u < g.U; u++) {
                uint32_t d[4];
                memcpy(d, planes + ((((size_t)cb * g.U + u) * bits + b) * HLQ_CB + lane) * 4, 16);
                for (int i = 0; i < 4; i++) d[i] = rotr32(d[i], HLQ_ROT);
                const size_t have = row_bytes - (size_t)u * 16;
                memcpy(w_quant_out + ((size_t)b * N + n) * row_bytes + (size_t)u * 16, d, have < 16 ? have : 16);
            }
            for (int gi = 0; gi < g.NG; gi++) {
                uint32_t v = scales[(((size_t)cb * g.NT + gi / 2) * bits + b) * HLQ_CB + lane];
                w_scale_out[((size_t)b * N + n) * g.NG + gi] = (uint16_t)(gi & 1 ? v >> 16 : v & 0xffff);
            }
        }
        for (int gi = 0; gi < g.NG; gi++) {
            uint32_t v = zeros[((size_t)cb * g.NT + gi / 2) * HLQ_CB + lane];
            w_zero_out[(size_t)n * g.NG + gi] = (uint16_t)(gi & 1 ? v >> 16 : v & 0xffff);
        }
    }
    return ELUTQ_OK;
}

}  // extern "C"

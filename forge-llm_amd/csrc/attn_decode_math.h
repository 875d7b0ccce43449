// The arithmetic a key slot of the split-sequence decode attention runs, shared by the kernel pair (attn_decode.hip) and
// the attention phase of the resident decode kernel (decode_persistent.hip) so that the two stay bit for bit the same.
#pragma once

#include "device_utils.h"

namespace fh {

struct __attribute__((aligned(16))) Half8 { uint32_t w[4]; };          // eight fp16 values as loaded (16 bytes)

__device__ __forceinline__ void unpack8(const Half8& h, float* f) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = f16_bits_to_f32((uint16_t)(h.w[i] & 0xFFFFu));
        f[2 * i + 1] = f16_bits_to_f32((uint16_t)(h.w[i] >> 16));
    }
}

// The lane's share of q . k for one key: eight products, then a fold over the LPK lanes that hold the key's row.
template <int LPK>
__device__ __forceinline__ float key_dot(const float (&qf)[8], const Half8& kr) {
    float kf[8];
    unpack8(kr, kf);
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) d = fmaf(qf[i], kf[i], d);
    static_assert(LPK == 8 || LPK == 16, "a key row over 8 or 16 lanes");
    d = lane_xor_add<1>(d); d = lane_xor_add<2>(d); d = lane_xor_add<4>(d);
    if (LPK == 16) d = lane_xor_add<8>(d);
    return d;
}

// Online softmax of one key slot advanced by U keys at once: the scores of the U keys first, ONE new maximum, one
// rescale of what was accumulated, then the U weighted value rows -- U + 1 exponentials where a key-by-key update needs
// 2 U.  (Both kernels call it with U = 2: wider steps keep more loaded rows alive than the resident kernel has registers for.)  s[u] = -inf for a key that does not exist (its weight is exp(-inf) = 0); a slot that has seen no key yet
// (m = -inf) and gets none here is left alone.  The value rows are unpacked one at a time (registers).
template <int U>
__device__ __forceinline__ void softmax_block_update(float& m, float& l, float (&acc)[8], const float (&s)[U], const Half8* vr) {
    float mn = m;
#pragma unroll
    for (int u = 0; u < U; u++) mn = fmaxf(mn, s[u]);
    if (mn == -INFINITY) return;
    const float alpha = __expf(m - mn);              // m = -inf before the first key: exp(-inf) = 0
    float p[U];
#pragma unroll
    for (int u = 0; u < U; u++) p[u] = __expf(s[u] - mn);
    float ps = p[0];
#pragma unroll
    for (int u = 1; u < U; u++) ps = ps + p[u];
    l = fmaf(l, alpha, ps);
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = acc[i] * alpha;
#pragma unroll
    for (int u = 0; u < U; u++) {
        float vf[8];
        unpack8(vr[u], vf);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = fmaf(p[u], vf[i], acc[i]);
    }
    m = mn;
}

}  // namespace fh

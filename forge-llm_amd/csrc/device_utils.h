// Device-side helpers shared by the kernels: fp16 bit conversions with the reference's
// rounding rules, the int8 block quantiser step and wave64 reductions.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fh {

constexpr int WAVE = 64;

__device__ __forceinline__ float f16_bits_to_f32(uint16_t bits) {
    return __half2float(__ushort_as_half(bits));
}

// Round-to-nearest-even like emit.rs:1460-1495, including its one deviation from IEEE:
// inputs below 2^-24 in magnitude (and f32 subnormals) become signed zero instead of
// possibly rounding up to the smallest fp16 subnormal.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float x) {
    if (fabsf(x) < 5.9604644775390625e-8f) return (uint16_t)((__float_as_uint(x) >> 16) & 0x8000u);
    return __half_as_ushort(__float2half_rn(x));
}

// `(v).round().clamp(-127, 127) as i8` (emit.rs:1433): round half away from zero.
__device__ __forceinline__ int quant_code(float v) {
    float r = roundf(v);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// Per-block activation scale of emit.rs:1421-1427: returns scale, sets inv.
__device__ __forceinline__ float act_scale(float absmax, float& inv) {
    if (absmax == 0.0f) { inv = 0.0f; return 1.0f; }
    float s = absmax / 127.0f;
    inv = 1.0f / s;
    return s;
}

// apply_repeat_penalty (project.rs:505-513) for one logit whose token occurs `count` times in the list: the reference
// applies the penalty once per occurrence, so this is `count` successive divisions (or multiplications), not a power.
__device__ __forceinline__ float repeat_penalised(float v, uint32_t count, float penalty) {
    for (uint32_t k = 0; k < count; k++) v = v > 0.0f ? v / penalty : v * penalty;
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Quantise 4 consecutive floats held by each of 8 consecutive lanes (one 32-element block).
// Returns the packed 4 int8 codes; lane%8==0 also gets the fp16 scale bits via `scale_bits`.
// `negate`: store -code instead of code (the scale stays positive): the fast prefill GEMM wants the odd blocks of a row
// that way (gemm.hip).
__device__ __forceinline__ uint32_t quantize_block_part(float4 v, uint16_t& scale_bits, bool negate = false) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1, WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 2, WAVE));
    amax = fmaxf(amax, __shfl_xor(amax, 4, WAVE));
    float inv;
    float s = act_scale(amax, inv);
    scale_bits = f32_to_f16_bits(s);
    if (negate) inv = -inv;          // rounding and clamping are symmetric: round(-x) = -round(x)
    uint32_t q0 = (uint32_t)quant_code(v.x * inv) & 0xFFu;
    uint32_t q1 = (uint32_t)quant_code(v.y * inv) & 0xFFu;
    uint32_t q2 = (uint32_t)quant_code(v.z * inv) & 0xFFu;
    uint32_t q3 = (uint32_t)quant_code(v.w * inv) & 0xFFu;
    return q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
}

}  // namespace fh

// Device-side helpers shared by the kernels: fp16 bit conversions with the reference's
// rounding rules, the int8 block quantiser step and wave64 reductions.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

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

// Lane exchange lane <-> lane ^ O without the LDS crossbar (`__shfl_xor` compiles to ds_bpermute_b32: an LDS
// instruction and its latency per step, which is what the short dependent chains of the decode kernels are made of).
// Inside a row of 16 lanes: DPP moves; across rows: the lane-swap instructions of gfx950.  Every lane of the pairs
// involved must be active.
template <int CTRL, typename T>
__device__ __forceinline__ T dpp_move(T v) { return __builtin_amdgcn_update_dpp((T)0, v, CTRL, 0xF, 0xF, false); }
template <int O>
__device__ __forceinline__ uint32_t lane_xor_bits(uint32_t v) {
    static_assert(O == 1 || O == 2 || O == 4 || O == 8 || O == 16 || O == 32, "one bit of the lane number");
    if constexpr (O == 1) return dpp_move<0xB1>(v);                      // quad_perm [1,0,3,2]
    else if constexpr (O == 2) return dpp_move<0x4E>(v);                 // quad_perm [2,3,0,1]
    else if constexpr (O == 4) {
        uint32_t r = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xF, 0x5, false);      // row_shl:4 into lanes 0-3, 8-11
        return __builtin_amdgcn_update_dpp(r, v, 0x114, 0xF, 0xA, false);            // row_shr:4 into lanes 4-7, 12-15
    } else if constexpr (O == 8) return dpp_move<0x128>(v);              // row_ror:8
    else if constexpr (O == 16) {
        // rows 1 and 3 of the first operand change places with rows 0 and 2 of the second
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        return (__lane_id() & 16u) ? r[0] : r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        return (__lane_id() & 32u) ? r[0] : r[1];
    }
}
template <int O> __device__ __forceinline__ float lane_xor(float v) { return __uint_as_float(lane_xor_bits<O>(__float_as_uint(v))); }
template <int O> __device__ __forceinline__ uint32_t lane_xor(uint32_t v) { return lane_xor_bits<O>(v); }
template <int O> __device__ __forceinline__ int lane_xor(int v) { return (int)lane_xor_bits<O>((uint32_t)v); }

// v + (lane ^ O's v) and the maximum likewise: across rows both halves of a swap are used as they come (the sum of a
// pair is the same number whichever of the two lanes computes it).
template <int O> __device__ __forceinline__ float lane_xor_add(float v) {
    if constexpr (O == 16) { const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false); return __uint_as_float(r[0]) + __uint_as_float(r[1]); }
    else if constexpr (O == 32) { const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false); return __uint_as_float(r[0]) + __uint_as_float(r[1]); }
    else return v + lane_xor<O>(v);
}
template <int O> __device__ __forceinline__ float lane_xor_max(float v) {
    if constexpr (O == 16) { const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false); return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])); }
    else if constexpr (O == 32) { const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false); return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])); }
    else return fmaxf(v, lane_xor<O>(v));
}
// The value of lane (lane & ~3) + I, for the four lanes of a quad.
template <int I> __device__ __forceinline__ uint32_t quad_broadcast(uint32_t v) { return dpp_move<I * 0x55>(v); }

// Sum over the wave in the pairing order 32, 16, ..., 1 (every lane ends with the same bits).
__device__ __forceinline__ float wave_sum(float v) {
    v = lane_xor_add<32>(v); v = lane_xor_add<16>(v); v = lane_xor_add<8>(v);
    v = lane_xor_add<4>(v); v = lane_xor_add<2>(v); v = lane_xor_add<1>(v);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = lane_xor_max<1>(v); v = lane_xor_max<2>(v); v = lane_xor_max<4>(v);
    v = lane_xor_max<8>(v); v = lane_xor_max<16>(v); v = lane_xor_max<32>(v);
    return v;
}
// Maximum over the aligned group of 32 lanes.
__device__ __forceinline__ float half_wave_max(float v) {
    v = lane_xor_max<1>(v); v = lane_xor_max<2>(v); v = lane_xor_max<4>(v);
    v = lane_xor_max<8>(v); v = lane_xor_max<16>(v);
    return v;
}

// Quantise 4 consecutive floats held by each of 8 consecutive lanes (one 32-element block).
// Returns the packed 4 int8 codes; lane%8==0 also gets the fp16 scale bits via `scale_bits`.
// `negate`: store -code instead of code (the scale stays positive): the fast prefill GEMM wants the odd blocks of a row
// that way (gemm.hip).
// `empty_zero`: an all-zero block gets the scale 0 instead of the reference's 1.0.  Its codes are zero either way; the fast
// prefill GEMM adds scale * (bias +- block sum) per block, and a scale of 1.0 next to neighbours of 0.01 would push the
// running sums to a magnitude where their low bits are lost.
__device__ __forceinline__ uint32_t quantize_block_part(float4 v, uint16_t& scale_bits, bool negate = false, bool empty_zero = false) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = lane_xor_max<1>(amax);
    amax = lane_xor_max<2>(amax);
    amax = lane_xor_max<4>(amax);
    float inv;
    float s = act_scale(amax, inv);
    scale_bits = (empty_zero && amax == 0.0f) ? (uint16_t)0 : f32_to_f16_bits(s);
    if (negate) inv = -inv;          // rounding and clamping are symmetric: round(-x) = -round(x)
    uint32_t q0 = (uint32_t)quant_code(v.x * inv) & 0xFFu;
    uint32_t q1 = (uint32_t)quant_code(v.y * inv) & 0xFFu;
    uint32_t q2 = (uint32_t)quant_code(v.z * inv) & 0xFFu;
    uint32_t q3 = (uint32_t)quant_code(v.w * inv) & 0xFFu;
    return q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
}

}  // namespace fh

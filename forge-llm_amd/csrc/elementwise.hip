// Small bandwidth-trivial kernels around the matmuls: activation quantiser, RMSNorm,
// SiLU-gate, RoPE + fp16 KV write, embedding gather, argmax.  Each fuses the int8 block
// quantisation of its output, because the consumer is always a quantised matmul
// (emit.rs:1410-1440 re-quantises the same vector once per matmul; the result is identical).
#include "common.h"
#include "device_utils.h"
#include "expf_ref.h"

namespace fh {

// ---- quantize_to_q8_0_blocks_into (emit.rs:1410-1440), planes instead of 34-byte blocks ----
__global__ __launch_bounds__(256) void quantize_act_kernel(const float* __restrict__ x, uint64_t n4,
                                                           uint32_t* __restrict__ q, uint16_t* __restrict__ sc,
                                                           uint32_t neg_odd_blocks_per_row) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < n4) v = reinterpret_cast<const float4*>(x)[i];
    uint16_t sb;
    const bool neg = neg_odd_blocks_per_row != 0 && (((i >> 3) % neg_odd_blocks_per_row) & 1) != 0;
    uint32_t packed = quantize_block_part(v, sb, neg, neg_odd_blocks_per_row != 0);
    if (i < n4) {
        q[i] = packed;
        if ((i & 7) == 0) sc[i >> 3] = sb;
    }
}

void launch_quantize_act(const float* x, uint32_t M, uint32_t K, int8_t* q, uint16_t* sc, hipStream_t s, bool neg_odd) {
    uint64_t n4 = (uint64_t)M * K / 4;
    if (n4 == 0) return;
    uint32_t grid = (uint32_t)((n4 + 255) / 256);
    fh::launch(quantize_act_kernel, grid, 256, 0, s, x, n4, reinterpret_cast<uint32_t*>(q), sc, neg_odd ? K / 32 : 0u);
}

// ---- rms_norm (emit.rs:327-334) + optional block quantisation -------------------------------
// One workgroup per row.  The sum of squares follows the reference's dot_f32 on its primary
// (aarch64) path bit for bit (emit.rs:272-295): sixteen fused-multiply-add accumulators over
// elements i mod 16, combined as (s[i]+s[i+4]) + (s[i+8]+s[i+12]) for i < 4, then pairwise,
// then the H mod 16 tail added in order.  inv = 1/sqrt(ss/n + eps), out = (x*inv)*w.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      float eps, uint32_t H, float* __restrict__ normed,
                                                      uint32_t* __restrict__ q, uint16_t* __restrict__ sc, uint32_t neg_odd) {
    extern __shared__ float xs[];          // the row, then 16 partial sums, then the result
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * H);
    const uint32_t n4 = H / 4;
    for (uint32_t i = tid; i < n4; i += 256) reinterpret_cast<float4*>(xs)[i] = xr[i];
    __syncthreads();
    float* part = xs + H;
    if (tid < 16) {
        float s = 0.f;
        const uint32_t chunks = H / 16;
        uint32_t c = 0;
        for (; c + 8 <= chunks; c += 8) {      // eight LDS reads in flight, then the dependent FMAs
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = xs[(c + i) * 16 + tid];
#pragma unroll
            for (int i = 0; i < 8; i++) s = fmaf(v[i], v[i], s);
        }
        for (; c < chunks; c++) { const float v = xs[c * 16 + tid]; s = fmaf(v, v, s); }
        part[tid] = s;
    }
    __syncthreads();
    if (tid == 0) {
        float t[4];
        for (int i = 0; i < 4; i++) t[i] = (part[i] + part[4 + i]) + (part[8 + i] + part[12 + i]);
        float r = (t[0] + t[1]) + (t[2] + t[3]);
        for (uint32_t i = H / 16 * 16; i < H; i++) r = r + xs[i] * xs[i];
        part[16] = r;
    }
    __syncthreads();
    const float ss = part[16];
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    const float4* wr = reinterpret_cast<const float4*>(w);
    const uint32_t n4_pad = (n4 + 255) / 256 * 256;
    for (uint32_t i = tid; i < n4_pad; i += 256) {
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < n4) {
            float4 v = xr[i], g = wr[i];
            o.x = v.x * inv * g.x; o.y = v.y * inv * g.y; o.z = v.z * inv * g.z; o.w = v.w * inv * g.w;
            if (normed) reinterpret_cast<float4*>(normed + (size_t)row * H)[i] = o;
        }
        if (q) {
            uint16_t sb;
            uint32_t packed = quantize_block_part(o, sb, neg_odd != 0 && ((i >> 3) & 1) != 0, neg_odd != 0);
            if (i < n4) {
                q[(size_t)row * n4 + i] = packed;
                if ((i & 7) == 0) sc[(size_t)row * (H / 32) + (i >> 3)] = sb;
            }
        }
    }
}

void launch_rmsnorm(const float* x, const float* w, float eps, uint32_t M, uint32_t H, float* normed, int8_t* q,
                    uint16_t* sc, hipStream_t s, bool neg_odd) {
    if (M == 0) return;
    fh::launch(rmsnorm_kernel, M, 256, (H + 32) * sizeof(float), s, x, w, eps, H, normed, reinterpret_cast<uint32_t*>(q), sc, neg_odd ? 1u : 0u);
}

// ---- silu_mul (emit.rs:380-386) + optional block quantisation --------------------------------
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       uint32_t I4, uint32_t row_stride, uint64_t total4,
                                                       float* __restrict__ out, uint32_t* __restrict__ q,
                                                       uint16_t* __restrict__ sc, uint32_t neg_odd) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    const bool neg = neg_odd != 0 && (((i % I4) >> 3) & 1) != 0;
    if (i < total4) {
        uint64_t r = i / I4, c = i % I4;
        float4 g = reinterpret_cast<const float4*>(gate + r * row_stride)[c];
        float4 u = reinterpret_cast<const float4*>(up + r * row_stride)[c];
        // exp as the CPU's C library computes it: the result is quantised to int8 next
        o.x = (g.x / (1.0f + expf_ref<true>(-g.x))) * u.x;
        o.y = (g.y / (1.0f + expf_ref<true>(-g.y))) * u.y;
        o.z = (g.z / (1.0f + expf_ref<true>(-g.z))) * u.z;
        o.w = (g.w / (1.0f + expf_ref<true>(-g.w))) * u.w;
        if (out) reinterpret_cast<float4*>(out)[i] = o;
    }
    if (q) {
        uint16_t sb;
        uint32_t packed = quantize_block_part(o, sb, neg, neg_odd != 0);
        if (i < total4) {
            q[i] = packed;
            if ((i & 7) == 0) sc[i >> 3] = sb;
        }
    }
}

void launch_silu_mul(const float* gate, const float* up, uint32_t M, uint32_t I, uint32_t row_stride, float* out,
                     int8_t* q, uint16_t* sc, hipStream_t s, bool neg_odd) {
    uint64_t total4 = (uint64_t)M * I / 4;
    if (total4 == 0) return;
    uint32_t grid = (uint32_t)((total4 + 255) / 256);
    fh::launch(silu_mul_kernel, grid, 256, 0, s, gate, up, I / 4, row_stride, total4, out, reinterpret_cast<uint32_t*>(q), sc, neg_odd ? 1u : 0u);
}

// ---- rope (emit.rs:508-528) + fp16 KV write ------------------------------------------------------
// One thread per (row, element pair).  Pair p of a head rotates (x[2p], x[2p+1]) by the
// angle pos*freq[p]; cos/sin come from a table built on the host with the C library, so
// they are the values the CPU path computes.
__global__ __launch_bounds__(256) void rope_kv_store_kernel(float* __restrict__ q, float* __restrict__ k,
                                                            const float* __restrict__ v, uint32_t q_stride,
                                                            uint32_t kv_stride, uint16_t* __restrict__ kc,
                                                            uint16_t* __restrict__ vc, uint32_t base_pos,
                                                            const uint32_t* __restrict__ pos_dev, uint32_t heads,
                                                            uint32_t kv_heads, uint32_t hd,
                                                            const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t,
                                                            const float* __restrict__ bias, PageTable pt) {
    // bias (optional): q | k | v bias vectors, added before the rotation (Qwen2, emit.rs:4105-4120)
    const uint32_t r = blockIdx.y;
    const uint32_t pos = (pos_dev ? *pos_dev : base_pos) + r;
    const size_t crow = paged_row(pt, pos);          // row of the cache (pool) that holds this position
    const uint32_t half = hd / 2;
    const uint32_t qp = heads * half, kp = kv_heads * half;
    const uint32_t p = blockIdx.x * 256 + threadIdx.x;
    if (p < qp) {
        const uint32_t i = p % half;
        const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
        float2* ptr = reinterpret_cast<float2*>(q + (size_t)r * q_stride) + p;
        float2 x = *ptr;
        if (bias) { x.x = x.x + bias[2 * p]; x.y = x.y + bias[2 * p + 1]; }
        float2 o;
        o.x = __fsub_rn(__fmul_rn(x.x, c), __fmul_rn(x.y, s));
        o.y = __fadd_rn(__fmul_rn(x.x, s), __fmul_rn(x.y, c));
        *ptr = o;
    } else if (p < qp + kp) {
        const uint32_t pk = p - qp, i = pk % half;
        const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
        float2* ptr = reinterpret_cast<float2*>(k + (size_t)r * kv_stride) + pk;
        float2 x = *ptr;
        if (bias) { x.x = x.x + bias[2 * qp + 2 * pk]; x.y = x.y + bias[2 * qp + 2 * pk + 1]; }
        float2 o;
        o.x = __fsub_rn(__fmul_rn(x.x, c), __fmul_rn(x.y, s));
        o.y = __fadd_rn(__fmul_rn(x.x, s), __fmul_rn(x.y, c));
        *ptr = o;
        uint32_t packed = (uint32_t)f32_to_f16_bits(o.x) | ((uint32_t)f32_to_f16_bits(o.y) << 16);
        reinterpret_cast<uint32_t*>(kc + crow * kv_heads * hd)[pk] = packed;
    } else if (p < qp + 2 * kp) {
        const uint32_t pv = p - qp - kp;
        float2 x = reinterpret_cast<const float2*>(v + (size_t)r * kv_stride)[pv];
        if (bias) { x.x = x.x + bias[2 * (qp + kp) + 2 * pv]; x.y = x.y + bias[2 * (qp + kp) + 2 * pv + 1]; }
        uint32_t packed = (uint32_t)f32_to_f16_bits(x.x) | ((uint32_t)f32_to_f16_bits(x.y) << 16);
        reinterpret_cast<uint32_t*>(vc + crow * kv_heads * hd)[pv] = packed;
    }
}

void launch_rope_kv_store(float* q, float* k, const float* v, uint32_t q_stride, uint32_t kv_stride, uint16_t* kc,
                          uint16_t* vc, uint32_t M, uint32_t base_pos, const uint32_t* pos_dev, uint32_t heads,
                          uint32_t kv_heads, uint32_t hd, const float* cos_t, const float* sin_t, const float* bias, hipStream_t s,
                          PageTable pt) {
    if (M == 0) return;
    uint32_t per_row = (heads + 2 * kv_heads) * hd / 2;
    dim3 grid((per_row + 255) / 256, M);
    fh::launch(rope_kv_store_kernel, grid, 256, 0, s, q, k, v, q_stride, kv_stride, kc, vc, base_pos, pos_dev, heads, kv_heads,
                                              hd, cos_t, sin_t, bias, pt);
}

// ---- embedding (emit.rs:585-589) -----------------------------------------------------------------
// `counts` (optional): how often each token id has been fed to the model; the row's first thread counts its token.
__global__ __launch_bounds__(256) void embedding_kernel(const float* __restrict__ table,
                                                        const uint32_t* __restrict__ tokens, uint32_t H4,
                                                        float* __restrict__ out, uint32_t* __restrict__ counts) {
    const uint32_t r = blockIdx.y;
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= H4) return;
    const uint32_t tok = tokens[r];
    if (counts && i == 0) atomicAdd(counts + tok, 1u);
    reinterpret_cast<float4*>(out)[(size_t)r * H4 + i] = reinterpret_cast<const float4*>(table)[(size_t)tok * H4 + i];
}

void launch_embedding(const float* table, const uint32_t* tokens_dev, uint32_t M, uint32_t H, float* out, uint32_t* counts,
                      hipStream_t s) {
    if (M == 0) return;
    dim3 grid((H / 4 + 255) / 256, M);
    fh::launch(embedding_kernel, grid, 256, 0, s, table, tokens_dev, H / 4, out, counts);
}

// ---- argmax (project.rs:501-503): the LAST index among equal maxima ------------------------------------
struct ArgPair { float v; uint32_t i; };
__device__ __forceinline__ ArgPair arg_better(ArgPair a, ArgPair b) {
    // keep the larger value; on equality the larger index
    bool take_b = (b.v > a.v) || (b.v == a.v && b.i > a.i);
    return take_b ? b : a;
}
__device__ __forceinline__ ArgPair arg_wave(ArgPair a) {
    auto fold = [&](auto O) { a = arg_better(a, ArgPair{lane_xor<O.value>(a.v), lane_xor<O.value>(a.i)}); };
    fold(std::integral_constant<int, 32>{}); fold(std::integral_constant<int, 16>{}); fold(std::integral_constant<int, 8>{});
    fold(std::integral_constant<int, 4>{}); fold(std::integral_constant<int, 2>{}); fold(std::integral_constant<int, 1>{});
    return a;
}
__device__ __forceinline__ ArgPair arg_block(ArgPair a, ArgPair* sh) {
    a = arg_wave(a);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = a;
    __syncthreads();
    ArgPair r = sh[0];
    for (int w = 1; w < 4; w++) r = arg_better(r, sh[w]);
    return r;
}

// `counts` (optional): apply_repeat_penalty (project.rs:505-513) on the fly, once per time the token was fed.
__global__ __launch_bounds__(256) void argmax_stage1(const float* __restrict__ x, uint32_t n, ArgPair* __restrict__ part,
                                                     const uint32_t* __restrict__ counts, float penalty) {
    __shared__ ArgPair sh[4];
    ArgPair a{-INFINITY, 0};
    bool any = false;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        ArgPair b{x[i], i};
        if (counts) b.v = repeat_penalised(b.v, counts[i], penalty);
        a = any ? arg_better(a, b) : b;
        any = true;
    }
    a = arg_block(a, sh);
    if (threadIdx.x == 0) part[blockIdx.x] = a;
}
// Final stage; optionally also advances the decode state (pos += 1, token = winner) so that the
// step needs no separate launch for it.
__global__ __launch_bounds__(256) void argmax_stage2(const ArgPair* __restrict__ part, uint32_t nparts,
                                                     uint32_t* __restrict__ out, uint32_t* pos, uint32_t* token) {
    __shared__ ArgPair sh[4];
    ArgPair a{-INFINITY, 0};
    if (threadIdx.x < nparts) a = part[threadIdx.x];
    a = arg_block(a, sh);
    if (threadIdx.x == 0) {
        *out = a.i;
        if (pos) *pos = *pos + 1;
        if (token) *token = a.i;
    }
}

void launch_argmax(const float* x, uint32_t n, uint32_t* out, void* scratch, uint32_t* pos_dev, uint32_t* token_dev,
                   const uint32_t* counts, float penalty, hipStream_t s) {
    uint32_t blocks = (n + 255) / 256;
    if (blocks > ARGMAX_BLOCKS) blocks = ARGMAX_BLOCKS;
    if (blocks == 0) blocks = 1;
    fh::launch(argmax_stage1, blocks, 256, 0, s, x, n, reinterpret_cast<ArgPair*>(scratch), counts, penalty);
    fh::launch(argmax_stage2, 1, 256, 0, s, reinterpret_cast<const ArgPair*>(scratch), blocks, out, pos_dev, token_dev);
}

}  // namespace fh

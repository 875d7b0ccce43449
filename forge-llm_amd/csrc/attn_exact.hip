// Order-faithful attention over the fp16 KV cache: attention_flash (emit.rs:656-715) and
// attention_flash_batch (emit.rs:754-883) with every f32 operation in the reference's own
// order — sequential q.k dots, 64-key blocks, block maximum, exp via the C library's
// algorithm, sequential block sums, and the two kernels' different P.V accumulation orders
// (flash: block-local sum then add; flash_batch: straight into the accumulator).
//
// This is the attention the model uses when it is created with FORGE_HIP_FLAG_EXACT: its
// output is bit-identical to the CPU path, which is what it takes for greedy tokens to be
// identical, because the output is quantised to int8 next and one flipped code cascades.
// It is a VALU kernel: one workgroup per (query row, head), keys across lanes for the
// scores, head dims across lanes for P.V.  The MFMA / split-sequence kernels are the fast
// path and agree with it to the float tolerance.
#include <algorithm>

#include "common.h"
#include "device_utils.h"
#include "expf_ref.h"

namespace fh {

constexpr int XB = 64;   // FLASH_ATTN_BLOCK_SIZE, emit.rs:201

template <int HD, bool BATCH>
__global__ void attn_exact_kernel(const float* __restrict__ q, uint32_t q_stride, const uint16_t* __restrict__ kc,
                                  const uint16_t* __restrict__ vc, float* __restrict__ out, uint32_t out_stride,
                                  int8_t* __restrict__ oq, uint16_t* __restrict__ osc, uint32_t base_pos,
                                  const uint32_t* __restrict__ pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t window) {
    __shared__ float qs[HD];
    __shared__ float e[XB];
    __shared__ float red[2];
    const uint32_t tid = threadIdx.x;
    const uint32_t h = blockIdx.x, r = blockIdx.y;
    const uint32_t kvh = h / (heads / kv_heads);
    const uint32_t qpos = (pos_dev ? *pos_dev : base_pos) + r;
    const uint32_t seq = qpos + 1;
    const uint32_t kv_stride = kv_heads * HD;
    const float scale = 1.0f / sqrtf((float)HD);

    if (tid < HD) qs[tid] = q[(size_t)r * q_stride + h * HD + tid];
    __syncthreads();

    float m_i = -INFINITY, l_i = 0.f, acc = 0.f;   // acc: head dim `tid`
    // attention_sliding_batch (emit.rs:907-1046, BATCH only): the same 64-key blocks, aligned at multiples of 64; blocks
    // that end before the query's window leave its state untouched, so the walk starts at the block that holds the
    // window's first key, and in that block the keys before it take no part (maximum, sums) or carry weight 0 (P.V:
    // adding 0 * v changes nothing).
    const uint32_t win_start = (window != 0 && seq > window) ? seq - window : 0;
    for (uint32_t bs = win_start / XB * XB; bs < seq; bs += XB) {
        const uint32_t bl = min((uint32_t)XB, seq - bs);
        const uint32_t lo = win_start > bs ? win_start - bs : 0;
        // ---- scores: thread bi owns key bs+bi; sum += q[i]*k[i] in order, then * scale
        float s = -INFINITY;
        if (tid >= lo && tid < bl) {
            const uint16_t* krow = kc + (size_t)(bs + tid) * kv_stride + kvh * HD;
            float sum = 0.f;
#pragma unroll
            for (int c = 0; c < HD / 8; c++) {
                const uint4 w = *reinterpret_cast<const uint4*>(krow + c * 8);
                const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    sum = sum + qs[c * 8 + 2 * j] * f16_bits_to_f32((uint16_t)(ww[j] & 0xFFFFu));
                    sum = sum + qs[c * 8 + 2 * j + 1] * f16_bits_to_f32((uint16_t)(ww[j] >> 16));
                }
            }
            s = sum * scale;
        }
        // ---- block maximum (order-free), running maximum, rescale
        if (tid < 64) {
            const float mb = wave_max(s);
            if (tid == 0) red[0] = mb;
        }
        __syncthreads();
        const float m_block = red[0];
        const float m_prev = m_i;
        if (m_block > m_i) m_i = m_block;
        const float exp_scale = expf_ref<true>(m_prev - m_i);
        l_i = l_i * exp_scale;
        acc = acc * exp_scale;
        if (tid >= lo && tid < bl) e[tid] = expf_ref<true>(s - m_i);
        __syncthreads();
        // ---- l_block: sequential over the block (every thread redundantly: same bits)
        float l_block = 0.f;
        for (uint32_t bi = lo; bi < bl; bi++) l_block = l_block + e[bi];
        l_i = l_i + l_block;
        // ---- P.V for head dim tid
        if (tid < HD) {
            const uint16_t* vcol = vc + (size_t)bs * kv_stride + kvh * HD + tid;
            if (BATCH) {
                for (uint32_t bi = lo; bi < bl; bi++) acc = acc + e[bi] * f16_bits_to_f32(vcol[(size_t)bi * kv_stride]);
            } else {
                float sum = 0.f;
                for (uint32_t bi = lo; bi < bl; bi++) sum = sum + e[bi] * f16_bits_to_f32(vcol[(size_t)bi * kv_stride]);
                acc = acc + sum;
            }
        }
        __syncthreads();   // e[] and red[] are rewritten by the next block
    }
    const float inv_l = 1.0f / l_i;
    const float o = acc * inv_l;
    if (tid < HD && out) out[(size_t)r * out_stride + h * HD + tid] = o;
    if (oq) {
        // int8 block quantisation of the output row (blocks of 32 head dims), for the O projection
        float amax = tid < HD ? fabsf(o) : 0.f;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
        float inv;
        const float sc = act_scale(amax, inv);
        if (tid < HD) {
            const size_t idx = (size_t)r * heads * HD + h * HD + tid;
            oq[idx] = (int8_t)quant_code(o * inv);
            if ((tid & 31) == 0) osc[idx / 32] = f32_to_f16_bits(sc);
        }
    }
}

// attention_flash_batch for many rows (batched prefill without a window), the same arithmetic as attn_exact_kernel<HD, true>
// value for value, arranged so that a key block is fetched once for 16 queries instead of once per query: a workgroup is
// ONE wave that carries up to 16 queries of one KV head (rows_per_wg consecutive rows x the heads that share the KV head)
// through the key blocks.  Per block: lane = key for the scores (the key's row in registers, the queries broadcast from
// LDS, 64-step sequential sums, four queries interleaved so that their chains overlap); lane = query for the running
// maximum, the rescale factor and the sequential block sum; lane = key again for the exponentials; lane = head dim for
// P.V (the block's V column in registers, the weights broadcast from LDS, added in key order straight into the
// accumulator).  Every query keeps the reference's own per-row block structure: blocks start at multiples of 64, a block
// past a row's last key leaves that row untouched, a row's last block is walked for its own number of keys only.
// BATCH = false: the rows in attention_flash's own order (emit.rs:656-715: a block's weighted values are summed first and the
// sum is added to the accumulator), for the rows of a prompt that the reference walks token by token through the decode
// attention (models with a format per projection).
template <int HD, bool BATCH = true>
__global__ __launch_bounds__(64) void attn_exact_batch_group_kernel(const float* __restrict__ q, uint32_t q_stride,
                                                                    const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
                                                                    float* __restrict__ out, uint32_t out_stride, uint32_t base_pos,
                                                                    uint32_t M, uint32_t heads, uint32_t kv_heads, uint32_t rows_per_wg) {
    constexpr int NQ = 16;                 // queries a wave carries
    constexpr int DPL = (HD + 63) / 64;    // head dims per lane in P.V: lane, lane + 64
    __shared__ __attribute__((aligned(16))) float qs[NQ][HD];
    __shared__ __attribute__((aligned(16))) float se[NQ][XB + 4];   // scores, then weights (rows 16-byte aligned)
    __shared__ float mi[NQ], es[NQ];
    const uint32_t lane = threadIdx.x;
    // the last rows walk the most key blocks: they are handed out first, the short ones fill the end
    const uint32_t kvh = blockIdx.x, r0 = (gridDim.y - 1 - blockIdx.y) * rows_per_wg;
    const uint32_t G = heads / kv_heads;
    const uint32_t rows = min(rows_per_wg, M - r0), nq = rows * G;
    const uint32_t kv_stride = kv_heads * HD;
    const float scale = 1.0f / sqrtf((float)HD);

    for (uint32_t i = lane; i < NQ * HD; i += 64) {
        const uint32_t qi = i / HD, d = i % HD;
        qs[qi][d] = qi < nq ? q[(size_t)(r0 + qi / G) * q_stride + (kvh * G + qi % G) * HD + d] : 0.f;
    }
    // lane j < nq keeps the softmax state of query j
    const uint32_t my_seq = lane < nq ? base_pos + r0 + lane / G + 1 : 0;
    float m_i = -INFINITY, l_i = 0.f;
    float acc[NQ][DPL];
#pragma unroll
    for (int qi = 0; qi < NQ; qi++)
#pragma unroll
        for (int t = 0; t < DPL; t++) acc[qi][t] = 0.f;
    const uint32_t seq_max = base_pos + r0 + rows;      // keys the last row sees
    // the key row of the NEXT block travels while this block is worked (zeros past the last key)
    uint4 kraw[HD / 8];
    auto fetch_k = [&](uint32_t bs) {
        const uint32_t key = bs + lane;
#pragma unroll
        for (int c = 0; c < HD / 8; c++)
            kraw[c] = key < seq_max ? *reinterpret_cast<const uint4*>(kc + (size_t)key * kv_stride + kvh * HD + c * 8) : make_uint4(0, 0, 0, 0);
    };
    fetch_k(0);
    __syncthreads();

    for (uint32_t bs = 0; bs < seq_max; bs += XB) {
        // ---- scores: lane = key bs + lane
        const uint32_t key = bs + lane;
        float sreg[NQ];
        float vf[XB][DPL];
        {
            float kf[HD];
#pragma unroll
            for (int c = 0; c < HD / 8; c++) {
                const uint32_t ww[4] = {kraw[c].x, kraw[c].y, kraw[c].z, kraw[c].w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    kf[c * 8 + 2 * j] = f16_bits_to_f32((uint16_t)(ww[j] & 0xFFFFu));
                    kf[c * 8 + 2 * j + 1] = f16_bits_to_f32((uint16_t)(ww[j] >> 16));
                }
            }
#pragma unroll
            for (int q0 = 0; q0 < NQ; q0 += 4) {
                float sum[4] = {0.f, 0.f, 0.f, 0.f};
                if ((uint32_t)q0 < nq) {
#pragma unroll
                for (int d = 0; d < HD; d++)
#pragma unroll
                    for (int u = 0; u < 4; u++) sum[u] = sum[u] + qs[q0 + u][d] * kf[d];
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const uint32_t seq_q = base_pos + r0 + (q0 + u) / G + 1;     // uniform
                    sreg[q0 + u] = ((uint32_t)(q0 + u) < nq && key < seq_q) ? sum[u] * scale : -INFINITY;
                    se[q0 + u][lane] = sreg[q0 + u];
                }
            }
        }
        // the block's V column (lane = head dim) is requested now and used after the softmax phases
#pragma unroll
        for (int bi = 0; bi < XB; bi++)
#pragma unroll
            for (int t = 0; t < DPL; t++) {
                const uint32_t d = lane + 64 * t;
                vf[bi][t] = (bs + bi < seq_max && d < HD) ? f16_bits_to_f32(vc[(size_t)(bs + bi) * kv_stride + kvh * HD + d]) : 0.f;
            }
        __syncthreads();
        // ---- lane = query: block maximum, running maximum, rescale factor
        const uint32_t my_bl = my_seq > bs ? min((uint32_t)XB, my_seq - bs) : 0;
        if (lane < nq) {
            float exp_scale = 1.0f;                 // a block past this row's keys: x * 1.0f is x
            if (my_bl) {
                float m_block = -INFINITY;
#pragma unroll 16
                for (int bi = 0; bi < XB; bi++) m_block = fmaxf(m_block, se[lane][bi]);   // keys past the row read -inf
                const float m_prev = m_i;
                if (m_block > m_i) m_i = m_block;
                exp_scale = expf_ref<true>(m_prev - m_i);
                l_i = l_i * exp_scale;
            }
            es[lane] = exp_scale;
            mi[lane] = m_i;
        }
        __syncthreads();
        // ---- lane = key: weights
#pragma unroll
        for (int qi = 0; qi < NQ; qi++) {
            if ((uint32_t)qi < nq) se[qi][lane] = sreg[qi] == -INFINITY ? 0.f : expf_ref<true>(sreg[qi] - mi[qi]);
        }
        __syncthreads();
        // ---- lane = query: sequential block sum over the row's own keys of the block
        if (lane < nq && my_bl) {
            float l_block = 0.f;
            if (my_bl == XB) {
#pragma unroll
                for (int bi = 0; bi < XB; bi++) l_block = l_block + se[lane][bi];
            } else {
#pragma unroll
                for (int bi = 0; bi < XB; bi++) l_block = (uint32_t)bi < my_bl ? l_block + se[lane][bi] : l_block;
            }
            l_i = l_i + l_block;
        }
        // ---- P.V: lane = head dim (and lane + 64)
        {
            fetch_k(bs + XB);
#pragma unroll
            for (int qi = 0; qi < NQ; qi++) {
                const uint32_t seq_q = base_pos + r0 + qi / G + 1;               // uniform
                // (a guard, not a break or continue: the loop must unroll completely, acc[] lives in registers)
                if ((uint32_t)qi < nq && seq_q > bs) {                           // else the block lies past this row's keys
                const uint32_t bl = min((uint32_t)XB, seq_q - bs);
                const float exp_scale = es[qi];
#pragma unroll
                for (int t = 0; t < DPL; t++) acc[qi][t] = acc[qi][t] * exp_scale;
                float part[DPL];                 // BATCH: the accumulator itself; else the block's own sum
#pragma unroll
                for (int t = 0; t < DPL; t++) part[t] = BATCH ? acc[qi][t] : 0.f;
                if (bl == XB) {
#pragma unroll
                    for (int bi = 0; bi < XB; bi++) {
                        const float e = se[qi][bi];
#pragma unroll
                        for (int t = 0; t < DPL; t++) part[t] = part[t] + e * vf[bi][t];
                    }
                } else {
#pragma unroll
                    for (int bi = 0; bi < XB; bi++) {
                        const float e = se[qi][bi];
#pragma unroll
                        for (int t = 0; t < DPL; t++) part[t] = (uint32_t)bi < bl ? part[t] + e * vf[bi][t] : part[t];
                    }
                }
#pragma unroll
                for (int t = 0; t < DPL; t++) acc[qi][t] = BATCH ? part[t] : acc[qi][t] + part[t];
                }
            }
        }
        __syncthreads();   // se, es and mi are rewritten by the next block
    }
    if (lane < nq) es[lane] = 1.0f / l_i;
    __syncthreads();
#pragma unroll
    for (int qi = 0; qi < NQ; qi++) {
        const float inv_l = es[qi];
#pragma unroll
        for (int t = 0; t < DPL; t++) {
            const uint32_t d = lane + 64 * t;
            if ((uint32_t)qi < nq && d < HD) out[(size_t)(r0 + qi / G) * out_stride + (kvh * G + qi % G) * HD + d] = acc[qi][t] * inv_l;
        }
    }
}

// attention_sliding (emit.rs:598-627), the decode attention of a model with a window: no blocks, a plain softmax over the
// last min(window, seq) rows — scores, their maximum, exp and a sequential sum, a multiplication by the reciprocal, then
// for every head dim a sequential sum of weight * v.  The scores live in dynamic LDS (wl floats).
template <int HD>
__global__ void attn_exact_sliding_kernel(const float* __restrict__ q, uint32_t q_stride, const uint16_t* __restrict__ kc,
                                          const uint16_t* __restrict__ vc, float* __restrict__ out, uint32_t out_stride,
                                          int8_t* __restrict__ oq, uint16_t* __restrict__ osc, uint32_t base_pos,
                                          const uint32_t* __restrict__ pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t window) {
    extern __shared__ float sc[];          // [wl] scores, then weights
    __shared__ float qs[HD];
    __shared__ float red[4];
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    const uint32_t h = blockIdx.x, r = blockIdx.y;
    const uint32_t kvh = h / (heads / kv_heads);
    const uint32_t seq = (pos_dev ? *pos_dev : base_pos) + r + 1;
    const uint32_t start = seq > window ? seq - window : 0, wl = seq - start;
    const uint32_t kv_stride = kv_heads * HD;
    const float scale = 1.0f / sqrtf((float)HD);
    if (tid < HD) qs[tid] = q[(size_t)r * q_stride + h * HD + tid];
    __syncthreads();
    float mx = -INFINITY;
    for (uint32_t si = tid; si < wl; si += nt) {
        const uint16_t* krow = kc + (size_t)(start + si) * kv_stride + kvh * HD;
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < HD / 8; c++) {
            const uint4 w = *reinterpret_cast<const uint4*>(krow + c * 8);
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                sum = sum + qs[c * 8 + 2 * j] * f16_bits_to_f32((uint16_t)(ww[j] & 0xFFFFu));
                sum = sum + qs[c * 8 + 2 * j + 1] * f16_bits_to_f32((uint16_t)(ww[j] >> 16));
            }
        }
        const float s = sum * scale;
        sc[si] = s;
        mx = fmaxf(mx, s);
    }
    mx = wave_max(mx);                      // the maximum does not depend on the order
    if ((tid & 63u) == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = red[0];
    for (uint32_t w = 1; w < nt / 64; w++) mx = fmaxf(mx, red[w]);
    for (uint32_t si = tid; si < wl; si += nt) sc[si] = expf_ref<true>(sc[si] - mx);
    __syncthreads();
    float sum = 0.f;                        // sequential, by every thread: same bits
    for (uint32_t si = 0; si < wl; si++) sum = sum + sc[si];
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    __syncthreads();
    for (uint32_t si = tid; si < wl; si += nt) sc[si] = sc[si] * inv;
    __syncthreads();
    float o = 0.f;
    if (tid < HD) {
        const uint16_t* vcol = vc + (size_t)start * kv_stride + kvh * HD + tid;
        for (uint32_t si = 0; si < wl; si++) o = o + sc[si] * f16_bits_to_f32(vcol[(size_t)si * kv_stride]);
        if (out) out[(size_t)r * out_stride + h * HD + tid] = o;
    }
    if (oq) {
        float amax = tid < HD ? fabsf(o) : 0.f;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
        float qinv;
        const float qsc = act_scale(amax, qinv);
        if (tid < HD) {
            const size_t idx = (size_t)r * heads * HD + h * HD + tid;
            oq[idx] = (int8_t)quant_code(o * qinv);
            if ((tid & 31) == 0) osc[idx / 32] = f32_to_f16_bits(qsc);
        }
    }
}

// ---- attention_flash for ONE query row (the decode step), spread over the chip.
// The reference's loop over 64-key blocks looks serial, but only a thin thread of it is: per block it needs the running
// maximum (a prefix maximum of the block maxima: order-free), then exp(s - m_i) per key, the block's sequential sums
// l_block and sum[d] -- all of which depend on nothing but this block's scores and m_i -- and only then the recurrence
//     l_i = l_i * exp_scale + l_block,   acc[d] = acc[d] * exp_scale + sum[d]        (two roundings each, in that order)
// that ties the blocks together.  So: (1) one workgroup per (block, head) computes the block's scores and maximum;
// (2) one workgroup per (block, head) computes m_i, the weights, l_block and sum[d], every sequential sum in the
// reference's order; (3) one workgroup per head runs the recurrence over the blocks' records.  Every f32 operation has
// the operands and the order it has in the one-workgroup kernel above, so the bits are the same; the work of steps 1
// and 2 (all the memory traffic and all but a few operations per block) runs on as many workgroups as there are blocks.
// Workspace per head: scores [rows_cap], then per block: maximum, m_i, l_block, sum[HD]  (nb_cap = rows_cap / 64 blocks).
constexpr uint32_t XD_MAX_BLOCKS = 4096;     // blocks whose exp_scale the last step keeps in LDS: caches up to 262144 rows

__host__ __device__ inline size_t xd_head_floats(uint32_t nb_cap, uint32_t hd) { return (size_t)nb_cap * (XB + 3 + hd); }

struct XdWs {
    float *scores, *bmax, *mi, *lblk, *sums;
};
__device__ __forceinline__ XdWs xd_ws(float* ws, uint32_t h, uint32_t nb_cap, uint32_t hd) {
    float* p = ws + (size_t)h * xd_head_floats(nb_cap, hd);
    return XdWs{p, p + (size_t)nb_cap * XB, p + (size_t)nb_cap * (XB + 1), p + (size_t)nb_cap * (XB + 2), p + (size_t)nb_cap * (XB + 3)};
}

template <int HD>
__global__ __launch_bounds__(64) void attn_exact_decode_scores_kernel(const float* __restrict__ q, const uint16_t* __restrict__ kc,
                                                                     float* __restrict__ ws, uint32_t base_pos,
                                                                     const uint32_t* __restrict__ pos_dev, uint32_t heads,
                                                                     uint32_t kv_heads, uint32_t nb_cap) {
    __shared__ float qs[HD];
    const uint32_t tid = threadIdx.x, b = blockIdx.x, h = blockIdx.y;
    const uint32_t seq = (pos_dev ? *pos_dev : base_pos) + 1, bs = b * XB;
    if (bs >= seq) return;
    const uint32_t kvh = h / (heads / kv_heads), kv_stride = kv_heads * HD, bl = min((uint32_t)XB, seq - bs);
    const float scale = 1.0f / sqrtf((float)HD);
    for (uint32_t i = tid; i < HD; i += 64) qs[i] = q[h * HD + i];
    __syncthreads();
    float sc = -INFINITY;
    if (tid < bl) {
        const uint16_t* krow = kc + (size_t)(bs + tid) * kv_stride + kvh * HD;
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < HD / 8; c++) {
            const uint4 w = *reinterpret_cast<const uint4*>(krow + c * 8);
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                sum = sum + qs[c * 8 + 2 * j] * f16_bits_to_f32((uint16_t)(ww[j] & 0xFFFFu));
                sum = sum + qs[c * 8 + 2 * j + 1] * f16_bits_to_f32((uint16_t)(ww[j] >> 16));
            }
        }
        sc = sum * scale;
    }
    const XdWs w = xd_ws(ws, h, nb_cap, HD);
    if (tid < bl) w.scores[bs + tid] = sc;
    const float mb = wave_max(sc);
    if (tid == 0) w.bmax[b] = mb;
}

template <int HD>
__global__ __launch_bounds__(HD <= 64 ? 64 : 128) void attn_exact_decode_block_kernel(const uint16_t* __restrict__ vc, float* __restrict__ ws,
                                                                                    uint32_t base_pos, const uint32_t* __restrict__ pos_dev,
                                                                                    uint32_t heads, uint32_t kv_heads, uint32_t nb_cap) {
    __shared__ float e[XB];
    __shared__ float red[1];
    const uint32_t tid = threadIdx.x, b = blockIdx.x, h = blockIdx.y;
    const uint32_t seq = (pos_dev ? *pos_dev : base_pos) + 1, bs = b * XB;
    if (bs >= seq) return;
    const uint32_t kvh = h / (heads / kv_heads), kv_stride = kv_heads * HD, bl = min((uint32_t)XB, seq - bs);
    const XdWs w = xd_ws(ws, h, nb_cap, HD);
    if (tid < 64) {
        // m_i after this block: the largest block maximum so far (`if m_block > m_i { m_i = m_block }` from -inf on)
        float m = -INFINITY;
        for (uint32_t i = tid; i <= b; i += 64) m = fmaxf(m, w.bmax[i]);
        m = wave_max(m);
        if (tid == 0) { red[0] = m; w.mi[b] = m; }
        if (tid < bl) e[tid] = expf_ref<true>(w.scores[bs + tid] - m);
    }
    __syncthreads();
    if (tid == 0) {
        float l_block = 0.f;
        for (uint32_t bi = 0; bi < bl; bi++) l_block = l_block + e[bi];
        w.lblk[b] = l_block;
    }
    if (tid < HD) {
        const uint16_t* vcol = vc + (size_t)bs * kv_stride + kvh * HD + tid;
        float sum = 0.f;
        if (bl == XB) {
#pragma unroll 16
            for (uint32_t bi = 0; bi < XB; bi++) sum = sum + e[bi] * f16_bits_to_f32(vcol[(size_t)bi * kv_stride]);
        } else {
            for (uint32_t bi = 0; bi < bl; bi++) sum = sum + e[bi] * f16_bits_to_f32(vcol[(size_t)bi * kv_stride]);
        }
        w.sums[(size_t)b * HD + tid] = sum;
    }
}

template <int HD>
__global__ __launch_bounds__(HD <= 64 ? 64 : 128) void attn_exact_decode_chain_kernel(float* __restrict__ ws, float* __restrict__ out,
                                                                                    int8_t* __restrict__ oq, uint16_t* __restrict__ osc,
                                                                                    uint32_t base_pos, const uint32_t* __restrict__ pos_dev,
                                                                                    uint32_t heads, uint32_t nb_cap) {
    __shared__ float es[XD_MAX_BLOCKS];
    const uint32_t tid = threadIdx.x, nt = blockDim.x, h = blockIdx.x;
    const uint32_t seq = (pos_dev ? *pos_dev : base_pos) + 1, nb = (seq + XB - 1) / XB;
    const XdWs w = xd_ws(ws, h, nb_cap, HD);
    // exp_scale of every block: exp(m_prev - m_i), m_prev = -inf before the first block
    for (uint32_t i = tid; i < nb; i += nt) es[i] = expf_ref<true>((i ? w.mi[i - 1] : -INFINITY) - w.mi[i]);
    __syncthreads();
    float l_i = 0.f, acc = 0.f;
    const uint32_t d = tid < HD ? tid : 0;
#pragma unroll 4
    for (uint32_t i = 0; i < nb; i++) {
        const float exp_scale = es[i];
        l_i = l_i * exp_scale;
        acc = acc * exp_scale;
        l_i = l_i + w.lblk[i];
        acc = acc + w.sums[(size_t)i * HD + d];
    }
    const float inv_l = 1.0f / l_i;
    const float o = acc * inv_l;
    if (tid < HD && out) out[h * HD + tid] = o;
    if (oq) {
        float amax = tid < HD ? fabsf(o) : 0.f;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
        float inv;
        const float sc = act_scale(amax, inv);
        if (tid < HD) {
            const size_t idx = (size_t)h * HD + tid;
            oq[idx] = (int8_t)quant_code(o * inv);
            if ((tid & 31) == 0) osc[idx / 32] = f32_to_f16_bits(sc);
        }
    }
}

// Workspace of the spread-out decode attention for a cache of up to max_rows rows; 0 if it does not apply (then the
// one-workgroup kernel runs).
size_t attn_exact_decode_workspace_bytes(uint32_t heads, uint32_t hd, uint32_t max_rows) {
    const uint32_t nb_cap = (max_rows + XB - 1) / XB;
    if (max_rows == 0 || nb_cap > XD_MAX_BLOCKS) return 0;
    return (size_t)heads * xd_head_floats(nb_cap, hd) * sizeof(float);
}

// Longest window (rows whose scores one workgroup keeps in LDS) the order-faithful decode attention takes.
uint32_t attn_exact_max_window() { return 12288; }

void launch_attn_exact(bool batch_order, const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc,
                       float* out, uint32_t out_stride, int8_t* oq, uint16_t* osc, uint32_t M, uint32_t base_pos,
                       const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd, uint32_t window, uint32_t max_rows,
                       void* ws, hipStream_t s) {
    if (M == 0) return;
    if (ws && !batch_order && window == 0 && M == 1 && attn_exact_decode_workspace_bytes(heads, hd, max_rows) != 0) {
        const uint32_t nb_cap = (max_rows + XB - 1) / XB;
        // blocks past the position (known to the device only when pos_dev is set) return at once
        const uint32_t nb = pos_dev ? nb_cap : (base_pos + XB) / XB;
        float* w = static_cast<float*>(ws);
        dim3 g2(nb, heads);
#define FH_XD(HD_)                                                                                                              \
    do {                                                                                                                        \
        fh::launch(attn_exact_decode_scores_kernel<HD_>, g2, 64, 0, s, q, kc, w, base_pos, pos_dev, heads, kv_heads, nb_cap);   \
        fh::launch(attn_exact_decode_block_kernel<HD_>, g2, HD_ <= 64 ? 64 : 128, 0, s, vc, w, base_pos, pos_dev, heads, kv_heads, nb_cap); \
        fh::launch(attn_exact_decode_chain_kernel<HD_>, dim3(heads), HD_ <= 64 ? 64 : 128, 0, s, w, out, oq, osc, base_pos, pos_dev, heads, nb_cap); \
    } while (0)
        if (hd == 64) FH_XD(64); else if (hd == 96) FH_XD(96); else FH_XD(128);
#undef FH_XD
        return;
    }
    // many rows without a window, in either order: a wave per 16 queries of one KV head (needs the f32 output form and at most
    // 16 heads per KV head; FORGE_HIP_EXACT_GROUP=0: the one-query kernel)
    static const bool group_ok = [] { const char* e = getenv("FORGE_HIP_EXACT_GROUP"); return !(e && e[0] == '0'); }();
    if (group_ok && window == 0 && M > 1 && out && !oq && !pos_dev && heads / kv_heads <= 16) {
        const uint32_t rows_per_wg = 16 / (heads / kv_heads);
        dim3 gg(kv_heads, (M + rows_per_wg - 1) / rows_per_wg);
#define FH_AXG(HD_, B_) \
    fh::launch(attn_exact_batch_group_kernel<HD_, B_>, gg, 64, 0, s, q, q_stride, kc, vc, out, out_stride, base_pos, M, heads, kv_heads, rows_per_wg)
        if (hd == 64) { if (batch_order) FH_AXG(64, true); else FH_AXG(64, false); }
        else if (hd == 96) { if (batch_order) FH_AXG(96, true); else FH_AXG(96, false); }
        else { if (batch_order) FH_AXG(128, true); else FH_AXG(128, false); }
#undef FH_AXG
        return;
    }
    dim3 grid(heads, M);
    const uint32_t threads = hd <= 64 ? 64 : 128;
    if (window != 0 && !batch_order) {
        // max_rows: the most rows the cache can hold (the position may be known to the device only)
        const size_t lds = (size_t)std::min(window, max_rows) * sizeof(float);
        if (hd == 64) fh::launch(attn_exact_sliding_kernel<64>, grid, 128, lds, s, q, q_stride, kc, vc, out, out_stride, oq, osc, base_pos, pos_dev, heads, kv_heads, window);
        else if (hd == 96) fh::launch(attn_exact_sliding_kernel<96>, grid, 128, lds, s, q, q_stride, kc, vc, out, out_stride, oq, osc, base_pos, pos_dev, heads, kv_heads, window);
        else fh::launch(attn_exact_sliding_kernel<128>, grid, 128, lds, s, q, q_stride, kc, vc, out, out_stride, oq, osc, base_pos, pos_dev, heads, kv_heads, window);
        return;
    }
#define FH_AX(HD_, B_) \
    fh::launch(attn_exact_kernel<HD_, B_>, grid, threads, 0, s, q, q_stride, kc, vc, out, out_stride, oq, osc, base_pos, pos_dev, heads, kv_heads, window)
    if (hd == 64) { if (batch_order) FH_AX(64, true); else FH_AX(64, false); }
    else if (hd == 96) { if (batch_order) FH_AX(96, true); else FH_AX(96, false); }
    else { if (batch_order) FH_AX(128, true); else FH_AX(128, false); }
#undef FH_AX
}

}  // namespace fh

// Decode GEMV for K-quant weights: matmul_vec_q4_k_KxN (emit.rs:3388-3490, dot_q4_k_q8_0 emit.rs:3035-3306) and
// matmul_vec_q6_k_KxN (emit.rs:3622-3655, dot_q6_k_q8_0 emit.rs:3553-3612).  Both multiply the SAME Q8_0-quantised
// activation blocks the Q8_0/Q4_0 kernels use against 256-element super-blocks, with exact int32 sub-block dots and an
// f32 combine that is one sequence of additions per row, the same on every host the reference runs on:
//   Q4_K   per 32-element sub-block j:  acc += x_s[j] * (d*sc_j * dot_j - dmin*m_j * sum_j),  dot_j = sum x q (q = 0..15)
//   Q6_K   per 32-element block b:      acc += d * x_s[b] * (sc_2b * dot_lo + sc_2b+1 * dot_hi),  q = 6-bit value - 32
// HBM-bound like the other GEMVs: a wave streams one row at a time with 16-byte loads that are contiguous across the wave,
// the products of a row are parked in LDS and one lane adds them in block order (unfused multiplies and adds).
//
// Device layout (split on upload so that every load is 16-byte aligned; the bytes themselves are the file's):
//   Q4_K   qs   uint8 [N][K/2]          the 128 nibble bytes of each super-block, in order
//          meta 16 B  [N][K/256]        d, dmin (fp16), then the 12 bytes of packed 6-bit scales and minima
//   Q6_K   qs   uint8 [N][K/256][192]   the 128 low-nibble bytes, then the 64 high-bit-pair bytes of each super-block
//          meta 32 B  [N][K/256]        the 16 int8 sub-block scales, d (fp16), padding
#include <string.h>

#include "common.h"
#include "device_utils.h"
#include "gemv_order.h"

namespace fh {

namespace {

__device__ __forceinline__ int kq_dot16(int4 w, int4 a, int acc) {
    acc = __builtin_amdgcn_sdot4(w.x, a.x, acc, false);
    acc = __builtin_amdgcn_sdot4(w.y, a.y, acc, false);
    acc = __builtin_amdgcn_sdot4(w.z, a.z, acc, false);
    acc = __builtin_amdgcn_sdot4(w.w, a.w, acc, false);
    return acc;
}
__device__ __forceinline__ uint32_t byte_of(const uint32_t* words, uint32_t i) { return (words[i >> 2] >> (8 * (i & 3))) & 0xFFu; }
__device__ __forceinline__ int pair_swap(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false); }          // quad_perm [1,0,3,2]
__device__ __forceinline__ float pair_swap(float v) { return __builtin_amdgcn_update_dpp(0.f, v, 0xB1, 0xF, 0xF, false); }
// (x - 32) for each of four 6-bit values held one per byte
__device__ __forceinline__ int sub32x4(uint32_t x) { return (int)(((x | 0x80808080u) - 0x20202020u) ^ 0x80808080u); }

constexpr int KQ_WAVES = 4;

// What a lane holds of RW rows for one pass of 64 pieces: its 16 bytes of quants and the super-block's scales.
template <bool Q6, int RW>
struct KqFrag;
template <int RW>
struct KqFrag<false, RW> {
    int4 wv[RW];
    uint4 mv[RW];
};
template <int RW>
struct KqFrag<true, RW> {
    uint4 ql[RW], qh[RW], sc[RW];
    uint32_t d[RW];
};

// A row is nsb * 8 pieces of 16 bytes of the first plane; piece p = 8 sb + t belongs to lane p % 64 of pass p / 64.
template <bool Q6, int RW>
__device__ __forceinline__ void kq_load(KqFrag<Q6, RW>& f, const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, uint32_t nsb,
                                        uint32_t N, uint32_t row0, uint32_t p) {
    if (p >= nsb * 8) return;
    const uint32_t sb = p >> 3, t = p & 7, e = t & 1;
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const size_t row = min(row0 + r, N - 1);                  // past the end: the last row again, never stored
        if constexpr (!Q6) {
            f.wv[r] = *reinterpret_cast<const int4*>(qs + (row * nsb + sb) * 128 + t * 16);
            f.mv[r] = *reinterpret_cast<const uint4*>(meta + (row * nsb + sb) * 16);
        } else {
            const uint32_t h = t >> 2, pp = (t >> 1) & 1;
            const uint8_t* sbp = qs + (row * nsb + sb) * 192;
            f.ql[r] = *reinterpret_cast<const uint4*>(sbp + 64 * h + 32 * pp + 16 * e);
            f.qh[r] = *reinterpret_cast<const uint4*>(sbp + 128 + 32 * h + 16 * e);
            const uint8_t* mp = meta + (row * nsb + sb) * 32;
            f.sc[r] = *reinterpret_cast<const uint4*>(mp);            // the 16 int8 sub-block scales
            f.d[r] = *reinterpret_cast<const uint32_t*>(mp + 16);     // d (fp16) in the low half
        }
    }
}

// The products of piece p of RW rows into the wave's LDS area.
template <bool Q6, int RW>
__device__ __forceinline__ void kq_products(const KqFrag<Q6, RW>& f, uint32_t nsb, uint32_t p, const int8_t* xa, const float* xs, const float* xsum,
                                            float* prod, uint32_t pstride) {
    if (p >= nsb * 8) return;
    const uint32_t sb = p >> 3, t = p & 7, e = t & 1;
    if constexpr (!Q6) {
        // piece t: bytes [16 t, +16) of the super-block's nibbles = elements [16 e, +16) of sub-blocks 2c (low
        // nibbles) and 2c + 1 (high nibbles), c = t / 2
        const uint32_t c = t >> 1;
        const uint32_t b_lo = sb * 8 + 2 * c;
        const int4 a_lo = *reinterpret_cast<const int4*>(xa + b_lo * 32 + e * 16);
        const int4 a_hi = *reinterpret_cast<const int4*>(xa + (b_lo + 1) * 32 + e * 16);
        // the even lane of the pair finishes sub-block 2c, the odd lane 2c + 1
        const uint32_t j = 2 * c + e, b = sb * 8 + j;
        const float x_s = xs[b], x_sum = xsum[b];
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const int4 w = f.wv[r];
            const uint4 mt = f.mv[r];
            const int m = 0x0F0F0F0F;
            const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
            const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
            int d_lo = kq_dot16(lo, a_lo, 0), d_hi = kq_dot16(hi, a_hi, 0);
            d_lo += pair_swap(d_lo);                     // the other 16 elements sit in the neighbouring lane
            d_hi += pair_swap(d_hi);
            const int dot = e ? d_hi : d_lo;
            const uint32_t sc12[3] = {mt.y, mt.z, mt.w};
            uint32_t sc, mn;                             // get_scale_min_k4, emit.rs:3013-3021
            if (j < 4) { sc = byte_of(sc12, j) & 63u; mn = byte_of(sc12, j + 4) & 63u; }
            else {
                sc = (byte_of(sc12, j + 4) & 0x0Fu) | ((byte_of(sc12, j - 4) >> 6) << 4);
                mn = (byte_of(sc12, j + 4) >> 4) | ((byte_of(sc12, j) >> 6) << 4);
            }
            const float d = f16_bits_to_f32((uint16_t)(mt.x & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(mt.x >> 16));
            const float d_w = d * (float)sc, m_w = dmin * (float)mn;
            prod[r * pstride + b] = x_s * (d_w * (float)dot - m_w * x_sum);
        }
    } else {
        // piece t = 4 h + 2 p + e: elements [16 e, +16) of blocks 4h + p (low nibbles of ql[64h + 32p ..], bit pair
        // 2p of qh[32h ..]) and 4h + 2 + p (high nibbles, bit pair 2 + p)
        const uint32_t h = t >> 2, pp = (t >> 1) & 1;
        const uint32_t bA = sb * 8 + 4 * h + pp, bB = bA + 2;
        const int4 xA = *reinterpret_cast<const int4*>(xa + bA * 32 + e * 16);
        const int4 xB = *reinterpret_cast<const int4*>(xa + bB * 32 + e * 16);
        const float xsA = xs[bA], xsB = xs[bB];
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t qlw[4] = {f.ql[r].x, f.ql[r].y, f.ql[r].z, f.ql[r].w}, qhw[4] = {f.qh[r].x, f.qh[r].y, f.qh[r].z, f.qh[r].w};
            const uint32_t scw[4] = {f.sc[r].x, f.sc[r].y, f.sc[r].z, f.sc[r].w};
            int4 qa, qb;
            int* qav = reinterpret_cast<int*>(&qa);
            int* qbv = reinterpret_cast<int*>(&qb);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                qav[i] = sub32x4((qlw[i] & 0x0F0F0F0Fu) | (((qhw[i] >> (2 * pp)) & 0x03030303u) << 4));
                qbv[i] = sub32x4(((qlw[i] >> 4) & 0x0F0F0F0Fu) | (((qhw[i] >> (4 + 2 * pp)) & 0x03030303u) << 4));
            }
            const int dA = kq_dot16(qa, xA, 0), dB = kq_dot16(qb, xB, 0);
            // this lane's 16 elements go under scale 2b + e; the even lane adds the pair: sc_lo*dot_lo + sc_hi*dot_hi
            const float sA = (float)(int)(int8_t)byte_of(scw, 2 * (4 * h + pp) + e), sB = (float)(int)(int8_t)byte_of(scw, 2 * (4 * h + 2 + pp) + e);
            const float tA = sA * (float)dA, tB = sB * (float)dB;
            const float uA = tA + pair_swap(tA), uB = tB + pair_swap(tB);      // even lane: lo + hi
            if (!e) {
                const float d = f16_bits_to_f32((uint16_t)(f.d[r] & 0xFFFFu));
                prod[r * pstride + bA] = (d * xsA) * uA;
                prod[r * pstride + bB] = (d * xsB) * uB;
            }
        }
    }
}

// The rows of one matrix that fall to workgroup `blk` of `nblks`.  A wave works RW rows at a time, a pass of 64 pieces after
// the other (one row of K = 2048 is a single kilobyte per pass, far too little in flight for HBM: hence RW rows, and the next
// pass is requested before this one is multiplied).  The weights do not depend on the activations: the first pass is on its
// way while `activations()` brings the codes, scales and (Q4_K) block sums into LDS.  Lane r adds row r's products in block
// order.
template <bool Q6, int RW, typename Activations>
__device__ __forceinline__ void kq_matrix(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, float* __restrict__ y, uint32_t K,
                                          uint32_t N, int accumulate, uint32_t blk, uint32_t nblks, const int8_t* xa, const float* xs,
                                          const float* xsum, float* prod, uint32_t lane, uint32_t wave, Activations&& activations) {
    const uint32_t nblk = K / 32, nsb = K / 256, pstride = prod_stride(nblk);
    const uint32_t pieces = nsb * 8;
    const uint32_t first = (blk * KQ_WAVES + wave) * RW, step = nblks * KQ_WAVES * RW;
    const uint32_t groups = first < N ? (N - first + step - 1) / step : 0u;
    const uint32_t total = groups * ((pieces + 63) / 64);
    KqFrag<Q6, RW> cur;
    if (total) kq_load<Q6, RW>(cur, qs, meta, nsb, N, first, lane);
    activations();
    uint32_t row0 = first, p0 = 0;
    for (uint32_t it = 0; it < total; it++) {
        uint32_t nrow0 = row0, np0 = p0 + 64;
        if (np0 >= pieces) { np0 = 0; nrow0 += step; }
        KqFrag<Q6, RW> nxt = cur;
        if (it + 1 < total) kq_load<Q6, RW>(nxt, qs, meta, nsb, N, nrow0, np0 + lane);
        kq_products<Q6, RW>(cur, nsb, p0 + lane, xa, xs, xsum, prod, pstride);
        // LDS operations of one wave execute in order: after a row's last pass its products are there.  Lane r adds row r's.
        if (np0 == 0 && lane < RW && row0 + lane < N) {
            float r = ordered_sum(prod + lane * pstride, nblk, false);
            if (accumulate) r = y[row0 + lane] + r;
            y[row0 + lane] = r;
        }
        cur = nxt;
        row0 = nrow0;
        p0 = np0;
    }
}

// Activations of one row into LDS: codes, scales as f32 and, for the Q4_K minimum term, the sum of every block's codes.
__device__ __forceinline__ void kq_load_activations(const int8_t* __restrict__ aq, const uint16_t* __restrict__ as, uint32_t K, int8_t* xa,
                                                    float* xs, float* xsum, uint32_t tid) {
    const uint32_t nblk = K / 32;
    for (uint32_t i = tid; i < K / 16; i += KQ_WAVES * 64) reinterpret_cast<int4*>(xa)[i] = reinterpret_cast<const int4*>(aq)[i];
    for (uint32_t b = tid; b < nblk; b += KQ_WAVES * 64) {
        xs[b] = f16_bits_to_f32(as[b]);
        const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
        const int4 a0 = reinterpret_cast<const int4*>(aq + (size_t)b * 32)[0], a1 = reinterpret_cast<const int4*>(aq + (size_t)b * 32)[1];
        xsum[b] = (float)kq_dot16(ones, a1, kq_dot16(ones, a0, 0));
    }
    __syncthreads();
}

// Where the quantised vector comes from.  Quantised: from memory.  RmsNorm: rms_norm(x) * norm_w, quantised by the workgroup
// itself (the arithmetic and the summation order of the stand-alone norm kernel: 16 strided partial sums, a fixed tree, then
// one block of 32 per 8 lanes).
enum class KqPro { Quantised, RmsNorm };
struct KqIn {
    const int8_t* aq;
    const uint16_t* as;
    const float* x;          // RmsNorm: the residual row
    const float* w;          // RmsNorm: the norm weights
    float eps;
};

__device__ __forceinline__ void kq_block_sums(uint32_t K, const int8_t* xa, float* xsum, uint32_t tid) {
    for (uint32_t b = tid; b < K / 32; b += KQ_WAVES * 64) {
        const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
        const int4 a0 = reinterpret_cast<const int4*>(xa + (size_t)b * 32)[0], a1 = reinterpret_cast<const int4*>(xa + (size_t)b * 32)[1];
        xsum[b] = (float)kq_dot16(ones, a1, kq_dot16(ones, a0, 0));
    }
}

// `tail`: K + 32 floats of LDS behind the products (RmsNorm only).
template <KqPro PRO>
__device__ __forceinline__ void kq_activations(const KqIn& in, uint32_t K, int8_t* xa, float* xs, float* xsum, float* tail, uint32_t tid) {
    constexpr uint32_t THREADS = KQ_WAVES * 64;
    if (PRO == KqPro::Quantised) {
        kq_load_activations(in.aq, in.as, K, xa, xs, xsum, tid);
        return;
    }
    uint32_t* codes = reinterpret_cast<uint32_t*>(xa);
    float* xf = tail;
    float* part = tail + K;
    for (uint32_t e4 = tid; e4 < K / 4; e4 += THREADS) reinterpret_cast<float4*>(xf)[e4] = reinterpret_cast<const float4*>(in.x)[e4];
    __syncthreads();
    if (tid < 16) {
        float sum = 0.f;
        const uint32_t chunks = K / 16;                   // K is a multiple of 256
        for (uint32_t c = 0; c < chunks; c += 8) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = xf[(c + i) * 16 + tid];
#pragma unroll
            for (int i = 0; i < 8; i++) sum = fmaf(v[i], v[i], sum);
        }
        part[tid] = sum;
    }
    __syncthreads();
    if (tid == 0) {
        float t[4];
        for (int i = 0; i < 4; i++) t[i] = (part[i] + part[4 + i]) + (part[8 + i] + part[12 + i]);
        part[16] = (t[0] + t[1]) + (t[2] + t[3]);
    }
    __syncthreads();
    const float inv_rms = 1.0f / sqrtf(part[16] / (float)K + in.eps);
    // (K / 4 is a multiple of 8 and so is THREADS: the 8 lanes of a block are in or out together)
    for (uint32_t e4 = tid; e4 < K / 4; e4 += THREADS) {
        const float4 xv = reinterpret_cast<const float4*>(xf)[e4], w4 = reinterpret_cast<const float4*>(in.w)[e4];
        const float4 v = make_float4(xv.x * inv_rms * w4.x, xv.y * inv_rms * w4.y, xv.z * inv_rms * w4.z, xv.w * inv_rms * w4.w);
        uint16_t sb;
        codes[e4] = quantize_block_part(v, sb);
        if ((e4 & 7u) == 0) xs[e4 >> 3] = f16_bits_to_f32(sb);
    }
    __syncthreads();
    kq_block_sums(K, xa, xsum, tid);
    __syncthreads();
}

// LDS: the activation codes [K], their scales as f32 [K/32], their sums as f32 [K/32], then per wave the products
// [RW][prod_stride(K/32)] (and the norm prologue's K + 32 floats).  A wave works RW rows at a time: all their loads are issued
// before the first is used (one row of K = 2048 is a single kilobyte, far too little in flight for HBM), and lane r adds row
// r's products in block order.
template <bool Q6, int RW, KqPro PRO>
__global__ __launch_bounds__(KQ_WAVES * 64) void gemv_kquant_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, KqIn in,
                                                                  float* __restrict__ y, uint32_t K, uint32_t N, int accumulate) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nblk = K / 32, pstride = prod_stride(nblk);
    int8_t* xa = reinterpret_cast<int8_t*>(lds);
    float* xs = reinterpret_cast<float*>(lds + K);
    float* xsum = xs + nblk;
    float* prod = xsum + nblk + (size_t)wave * RW * pstride;
    auto act = [&]() { kq_activations<PRO>(in, K, xa, xs, xsum, xsum + nblk + (size_t)KQ_WAVES * RW * pstride, tid); };
    kq_matrix<Q6, RW>(qs, meta, y, K, N, accumulate, blockIdx.x, gridDim.x, xa, xs, xsum, prod, lane, wave, act);
}

// Up to three matrices that multiply the SAME vector (q, k, v; gate, up) in one launch: a workgroup belongs to one of them.
struct KqMat {
    const uint8_t* qs;
    const uint8_t* meta;
    float* y;
    uint32_t N, q6, blk0, nblks;
};
struct KqMulti {
    KqMat m[3];
    uint32_t n;
};
template <int RW, KqPro PRO>
__global__ __launch_bounds__(KQ_WAVES * 64) void gemv_kquant_multi_kernel(KqMulti a, KqIn in, uint32_t K, int accumulate) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nblk = K / 32, pstride = prod_stride(nblk);
    int8_t* xa = reinterpret_cast<int8_t*>(lds);
    float* xs = reinterpret_cast<float*>(lds + K);
    float* xsum = xs + nblk;
    float* prod = xsum + nblk + (size_t)wave * RW * pstride;
    auto act = [&]() { kq_activations<PRO>(in, K, xa, xs, xsum, xsum + nblk + (size_t)KQ_WAVES * RW * pstride, tid); };
    uint32_t i = 0;
    while (i + 1 < a.n && blockIdx.x >= a.m[i + 1].blk0) i++;
    const KqMat mt = a.m[i];
    if (mt.q6) kq_matrix<true, RW>(mt.qs, mt.meta, mt.y, K, mt.N, accumulate, blockIdx.x - mt.blk0, mt.nblks, xa, xs, xsum, prod, lane, wave, act);
    else kq_matrix<false, RW>(mt.qs, mt.meta, mt.y, K, mt.N, accumulate, blockIdx.x - mt.blk0, mt.nblks, xa, xs, xsum, prod, lane, wave, act);
}

// The same matmul for MB rows of activations at once (a prompt through a model with K-quant projections): a workgroup holds
// the quantised activations of MB consecutive rows in LDS, every wave streams RW weight rows at a time and multiplies each
// weight piece with all MB activation rows before it moves on, so a matrix is read once per MB rows instead of once per row.
// Every (activation row, weight row) pair is computed exactly as the one-row kernel computes it -- the same sub-block dots, the
// same products, the same ordered sum -- so a row of the result has that kernel's bits whatever batch it is part of.
constexpr int KQR_WAVES = 8;
constexpr uint32_t KQR_PSTRIDE = 68;      // floats between two pairs' products of a pass: 64 + a pad that spreads the banks (16-byte units, odd)

template <bool Q6, int RW, int MB>
__global__ __launch_bounds__(KQR_WAVES * 64) void gemv_kquant_rows_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta,
                                                                        const int8_t* __restrict__ aq, const uint16_t* __restrict__ as,
                                                                        float* __restrict__ y, uint32_t K, uint32_t N, uint32_t M,
                                                                        uint32_t ldy, int accumulate) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nblk = K / 32, nsb = K / 256;
    constexpr uint32_t pstride = KQR_PSTRIDE;
    const uint32_t m0 = blockIdx.y * MB, mrows = min((uint32_t)MB, M - m0);
    // LDS: codes [MB][K] | scales f32 [MB][nblk] | (Q4_K) block sums f32 [MB][nblk] | per wave products [MB * RW][pstride].
    // A pass of the wave covers 64 pieces = the 64 blocks [p0, p0 + 64) of every (activation row, weight row) pair it carries;
    // lane (mb, r) adds that pair's 64 products to its running sum right after the pass, in block order: the sum is the same
    // chain of additions as one walk over all K / 32 products, and the product area holds one pass instead of a whole row.
    int8_t* xa = reinterpret_cast<int8_t*>(lds);
    float* xs = reinterpret_cast<float*>(lds + (size_t)MB * K);
    float* xsum = xs + (size_t)MB * nblk;
    float* prod = xsum + (size_t)MB * nblk + (size_t)wave * MB * RW * pstride;
    for (uint32_t i = tid; i < MB * (K / 16); i += KQR_WAVES * 64) {
        const uint32_t mb = i / (K / 16), c = i - mb * (K / 16);
        int4 v = make_int4(0, 0, 0, 0);
        if (mb < mrows) v = reinterpret_cast<const int4*>(aq + (size_t)(m0 + mb) * K)[c];
        reinterpret_cast<int4*>(xa)[i] = v;
    }
    for (uint32_t i = tid; i < MB * nblk; i += KQR_WAVES * 64) {
        const uint32_t mb = i / nblk, b = i - mb * nblk;
        float sc = 0.f, sm = 0.f;
        if (mb < mrows) {
            sc = f16_bits_to_f32(as[(size_t)(m0 + mb) * nblk + b]);
            if (!Q6) {
                const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
                const int4* ap = reinterpret_cast<const int4*>(aq + (size_t)(m0 + mb) * K + (size_t)b * 32);
                sm = (float)kq_dot16(ones, ap[1], kq_dot16(ones, ap[0], 0));
            }
        }
        xs[i] = sc;
        if (!Q6) xsum[i] = sm;
    }
    __syncthreads();

    const uint32_t pieces = nsb * 8;
    for (uint32_t row0 = (blockIdx.x * KQR_WAVES + wave) * RW; row0 < N; row0 += gridDim.x * KQR_WAVES * RW) {
        float run = 0.f;                               // lane (mb, r): the pair's sum so far
        for (uint32_t p0 = 0; p0 < pieces; p0 += 64) {
            const uint32_t p = p0 + lane;
            if (p < pieces) {
                const uint32_t sb = p >> 3, t = p & 7, e = t & 1;
                if (!Q6) {
                    const uint32_t c = t >> 1;
                    const uint32_t j = 2 * c + e, b = sb * 8 + j, b_lo = sb * 8 + 2 * c;
                    const uint32_t bl = b - p0;                       // the block's place in this pass
                    int4 lo[RW], hi[RW];
                    float d_w[RW], m_w[RW];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const size_t row = min(row0 + r, N - 1);
                        const int4 w = *reinterpret_cast<const int4*>(qs + (row * nsb + sb) * 128 + t * 16);
                        const uint4 mt = *reinterpret_cast<const uint4*>(meta + (row * nsb + sb) * 16);
                        const int m = 0x0F0F0F0F;
                        lo[r] = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                        hi[r] = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                        const uint32_t sc12[3] = {mt.y, mt.z, mt.w};
                        uint32_t sc, mn;                             // get_scale_min_k4, emit.rs:3013-3021
                        if (j < 4) { sc = byte_of(sc12, j) & 63u; mn = byte_of(sc12, j + 4) & 63u; }
                        else {
                            sc = (byte_of(sc12, j + 4) & 0x0Fu) | ((byte_of(sc12, j - 4) >> 6) << 4);
                            mn = (byte_of(sc12, j + 4) >> 4) | ((byte_of(sc12, j) >> 6) << 4);
                        }
                        const float d = f16_bits_to_f32((uint16_t)(mt.x & 0xFFFFu)), dmin = f16_bits_to_f32((uint16_t)(mt.x >> 16));
                        d_w[r] = d * (float)sc;
                        m_w[r] = dmin * (float)mn;
                    }
#pragma unroll 2
                    for (int mb = 0; mb < MB; mb++) {
                        const int8_t* xrow = xa + (size_t)mb * K;
                        const int4 a_lo = *reinterpret_cast<const int4*>(xrow + b_lo * 32 + e * 16);
                        const int4 a_hi = *reinterpret_cast<const int4*>(xrow + (b_lo + 1) * 32 + e * 16);
                        const float x_s = xs[mb * nblk + b], x_sum = xsum[mb * nblk + b];
#pragma unroll
                        for (int r = 0; r < RW; r++) {
                            int d_lo = kq_dot16(lo[r], a_lo, 0), d_hi = kq_dot16(hi[r], a_hi, 0);
                            d_lo += pair_swap(d_lo);
                            d_hi += pair_swap(d_hi);
                            const int dot = e ? d_hi : d_lo;
                            prod[(mb * RW + r) * pstride + bl] = x_s * (d_w[r] * (float)dot - m_w[r] * x_sum);
                        }
                    }
                } else {
                    const uint32_t h = t >> 2, pp = (t >> 1) & 1;
                    const uint32_t bA = sb * 8 + 4 * h + pp, bB = bA + 2;
                    int4 qa[RW], qb[RW];
                    float sA[RW], sB[RW], dd[RW];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const size_t row = min(row0 + r, N - 1);
                        const uint8_t* sbp = qs + (row * nsb + sb) * 192;
                        const uint4 qlv = *reinterpret_cast<const uint4*>(sbp + 64 * h + 32 * pp + 16 * e);
                        const uint4 qhv = *reinterpret_cast<const uint4*>(sbp + 128 + 32 * h + 16 * e);
                        const uint8_t* mp = meta + (row * nsb + sb) * 32;
                        const uint4 scv = *reinterpret_cast<const uint4*>(mp);
                        const uint32_t dv = *reinterpret_cast<const uint32_t*>(mp + 16);
                        const uint32_t qlw[4] = {qlv.x, qlv.y, qlv.z, qlv.w}, qhw[4] = {qhv.x, qhv.y, qhv.z, qhv.w};
                        const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
                        int* qav = reinterpret_cast<int*>(&qa[r]);
                        int* qbv = reinterpret_cast<int*>(&qb[r]);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            qav[i] = sub32x4((qlw[i] & 0x0F0F0F0Fu) | (((qhw[i] >> (2 * pp)) & 0x03030303u) << 4));
                            qbv[i] = sub32x4(((qlw[i] >> 4) & 0x0F0F0F0Fu) | (((qhw[i] >> (4 + 2 * pp)) & 0x03030303u) << 4));
                        }
                        sA[r] = (float)(int)(int8_t)byte_of(scw, 2 * (4 * h + pp) + e);
                        sB[r] = (float)(int)(int8_t)byte_of(scw, 2 * (4 * h + 2 + pp) + e);
                        dd[r] = f16_bits_to_f32((uint16_t)(dv & 0xFFFFu));
                    }
#pragma unroll 2
                    for (int mb = 0; mb < MB; mb++) {
                        const int8_t* xrow = xa + (size_t)mb * K;
                        const int4 xA = *reinterpret_cast<const int4*>(xrow + bA * 32 + e * 16);
                        const int4 xB = *reinterpret_cast<const int4*>(xrow + bB * 32 + e * 16);
                        const float xsA = xs[mb * nblk + bA], xsB = xs[mb * nblk + bB];
#pragma unroll
                        for (int r = 0; r < RW; r++) {
                            const int dA = kq_dot16(qa[r], xA, 0), dB = kq_dot16(qb[r], xB, 0);
                            const float tA = sA[r] * (float)dA, tB = sB[r] * (float)dB;
                            const float uA = tA + pair_swap(tA), uB = tB + pair_swap(tB);      // even lane: lo + hi
                            if (!e) {
                                prod[(mb * RW + r) * pstride + (bA - p0)] = (dd[r] * xsA) * uA;
                                prod[(mb * RW + r) * pstride + (bB - p0)] = (dd[r] * xsB) * uB;
                            }
                        }
                    }
                }
            }
            // LDS operations of one wave execute in order: the pass's products are there.  Lane (mb, r) adds that pair's, in
            // block order, to its running sum (the reads of a group of 16 are issued before its first add).
            if (lane < MB * RW) {
                const uint32_t cnt = min(64u, nblk - p0);            // a multiple of 8
                const float4* p4 = reinterpret_cast<const float4*>(prod + lane * pstride);
                for (uint32_t g = 0; g < cnt / 4; g += 4) {
                    float4 v[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) v[i] = g + i < cnt / 4 ? p4[g + i] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (g + i < cnt / 4) { run = run + v[i].x; run = run + v[i].y; run = run + v[i].z; run = run + v[i].w; }
                }
            }
        }
        if (lane < MB * RW) {
            const uint32_t mb = lane / RW, r = lane - mb * RW;
            if (mb < mrows && row0 + r < N) {
                float v = run;
                float* dst = y + (size_t)(m0 + mb) * ldy + row0 + r;
                if (accumulate) v = *dst + v;
                *dst = v;
            }
        }
    }
}

}  // namespace

size_t kquant_qs_row_bytes(uint32_t wdtype, uint32_t K) { return wdtype == FORGE_HIP_Q4_K ? K / 2 : (size_t)K / 256 * 192; }
size_t kquant_meta_row_bytes(uint32_t wdtype, uint32_t K) { return (size_t)K / 256 * (wdtype == FORGE_HIP_Q4_K ? 16 : 32); }

// Split raw GGUF super-blocks (144 / 210 bytes) into the two planes.
void repack_kquant_host(uint32_t wdtype, const uint8_t* raw, uint32_t K, uint64_t N, uint8_t* qs, uint8_t* meta) {
    const uint64_t nsb = K / 256;
    for (uint64_t r = 0; r < N; r++)
        for (uint64_t sb = 0; sb < nsb; sb++) {
            if (wdtype == FORGE_HIP_Q4_K) {
                const uint8_t* src = raw + (r * nsb + sb) * 144;
                memcpy(meta + (r * nsb + sb) * 16, src, 16);
                memcpy(qs + (r * nsb + sb) * 128, src + 16, 128);
            } else {
                const uint8_t* src = raw + (r * nsb + sb) * 210;
                memcpy(qs + (r * nsb + sb) * 192, src, 192);
                uint8_t* m = meta + (r * nsb + sb) * 32;
                memcpy(m, src + 192, 18);
                memset(m + 18, 0, 14);
            }
        }
}

bool kquant_k_supported(uint32_t K) { return K >= 256 && K % 256 == 0 && K <= 16384; }

namespace {
template <KqPro PRO>
void launch_kq_one(const QWeight& w, const KqIn& in, float* y, bool accumulate, hipStream_t s) {
    if (w.N == 0) return;
    const uint32_t nblk = w.K / 32;
    // rows a wave keeps in flight: four when that still leaves every CU several workgroups
    const int rw = w.N >= 16384 ? 4 : w.N >= 4096 ? 2 : 1;
    const size_t lds = (size_t)w.K + (size_t)nblk * 8 + (size_t)KQ_WAVES * rw * prod_stride(nblk) * 4;
    uint32_t grid = (w.N + KQ_WAVES * rw - 1) / (KQ_WAVES * rw);
    if (grid > 256 * 8) grid = 256 * 8;
    const uint8_t* meta = reinterpret_cast<const uint8_t*>(w.scales);
    const int acc = accumulate ? 1 : 0;
#define FH_KQ(Q6_, RW_) fh::launch(gemv_kquant_kernel<Q6_, RW_, PRO>, grid, KQ_WAVES * 64, lds, s, w.qs, meta, in, y, w.K, w.N, acc)
    if (w.wdtype == FORGE_HIP_Q6_K) { if (rw == 4) FH_KQ(true, 4); else if (rw == 2) FH_KQ(true, 2); else FH_KQ(true, 1); }
    else { if (rw == 4) FH_KQ(false, 4); else if (rw == 2) FH_KQ(false, 2); else FH_KQ(false, 1); }
#undef FH_KQ
}

template <KqPro PRO>
void launch_kq_multi(const QWeight* const* w, float* const* y, uint32_t n, const KqIn& in, bool accumulate, hipStream_t s) {
    if (n == 0) return;
    const uint32_t K = w[0]->K, nblk = K / 32;
    uint32_t ntot = 0;
    for (uint32_t i = 0; i < n; i++) ntot += w[i]->N;
    // rows a wave keeps in flight, by the rows of the whole launch
    const int rw = ntot >= 16384 ? 4 : ntot >= 4096 ? 2 : 1;
    KqMulti a{};
    a.n = n;
    uint32_t total = 0;
    for (uint32_t i = 0; i < n; i++) {
        uint32_t g = (w[i]->N + KQ_WAVES * rw - 1) / (KQ_WAVES * rw);
        if (g > 256 * 8) g = 256 * 8;
        a.m[i] = KqMat{w[i]->qs, reinterpret_cast<const uint8_t*>(w[i]->scales), y[i], w[i]->N, w[i]->wdtype == FORGE_HIP_Q6_K ? 1u : 0u, total, g};
        total += g;
    }
    const size_t lds = (size_t)K + (size_t)nblk * 8 + (size_t)KQ_WAVES * rw * prod_stride(nblk) * 4 + (PRO == KqPro::RmsNorm ? ((size_t)K + 32) * 4 : 0);
    const int acc = accumulate ? 1 : 0;
    if (rw == 4) fh::launch(gemv_kquant_multi_kernel<4, PRO>, total, KQ_WAVES * 64, lds, s, a, in, K, acc);
    else if (rw == 2) fh::launch(gemv_kquant_multi_kernel<2, PRO>, total, KQ_WAVES * 64, lds, s, a, in, K, acc);
    else fh::launch(gemv_kquant_multi_kernel<1, PRO>, total, KQ_WAVES * 64, lds, s, a, in, K, acc);
}
}  // namespace

void launch_gemv_kquant(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, hipStream_t s) {
    launch_kq_one<KqPro::Quantised>(w, KqIn{aq, as, nullptr, nullptr, 0.f}, y, accumulate, s);
}

// Up to three K-quant matrices over the same quantised vector in ONE launch (same K; each y[i] has N_i floats).  Every row has
// launch_gemv_kquant's bits.
void launch_gemv_kquant_multi(const QWeight* const* w, float* const* y, uint32_t n, const int8_t* aq, const uint16_t* as, bool accumulate,
                              hipStream_t s) {
    launch_kq_multi<KqPro::Quantised>(w, y, n, KqIn{aq, as, nullptr, nullptr, 0.f}, accumulate, s);
}

// The same over quantise(rms_norm(x) * norm_w), computed by every workgroup for itself in the stand-alone norm kernel's order:
// the norm launch in front of q/k/v or gate/up disappears.
void launch_gemv_kquant_multi_norm(const QWeight* const* w, float* const* y, uint32_t n, const float* x, const float* norm_w, float eps,
                                   hipStream_t s) {
    launch_kq_multi<KqPro::RmsNorm>(w, y, n, KqIn{nullptr, nullptr, x, norm_w, eps}, false, s);
}

// M rows at once: y[m][n] (=|+=) for m < M, rows of y `ldy` floats apart.  Each row has launch_gemv_kquant's bits.
void launch_gemv_kquant_rows(const QWeight& w, const int8_t* aq, const uint16_t* as, uint32_t M, float* y, uint32_t ldy, bool accumulate,
                             hipStream_t s) {
    if (w.N == 0 || M == 0) return;
    const uint32_t nblk = w.K / 32;
    const bool q6 = w.wdtype == FORGE_HIP_Q6_K;
    // (weight rows per wave, activation rows per workgroup): the first shape whose LDS lets two workgroups share a CU, else the
    // first that fits at all
    auto lds_for = [&](int rw, int mb) {
        return (size_t)mb * w.K + (size_t)mb * nblk * 8 + (size_t)KQR_WAVES * mb * rw * KQR_PSTRIDE * 4;
    };
    static const int shapes[4][2] = {{4, 8}, {2, 8}, {4, 4}, {2, 4}};
    int pick = -1;
    for (int i = 0; i < 4 && pick < 0; i++) if (lds_for(shapes[i][0], shapes[i][1]) <= 78 * 1024) pick = i;
    for (int i = 0; i < 4 && pick < 0; i++) if (lds_for(shapes[i][0], shapes[i][1]) <= 156 * 1024) pick = i;
    if (pick < 0) pick = 3;                      // K <= 16384: (2, 4) needs 98 KB at most
    const int rw = shapes[pick][0], mb = shapes[pick][1];
    const size_t lds = lds_for(rw, mb);
    uint32_t gx = (w.N + KQR_WAVES * rw - 1) / (KQR_WAVES * rw);
    if (gx > 1024) gx = 1024;
    const dim3 grid(gx, (M + mb - 1) / mb);
    const uint8_t* meta = reinterpret_cast<const uint8_t*>(w.scales);
    const int acc = accumulate ? 1 : 0;
#define FH_KQR(Q6_, RW_, MB_)                                                                                                    \
    do {                                                                                                                        \
        static const hipError_t ok = hipFuncSetAttribute((const void*)gemv_kquant_rows_kernel<Q6_, RW_, MB_>,                   \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);               \
        (void)ok;                                                                                                               \
        fh::launch(gemv_kquant_rows_kernel<Q6_, RW_, MB_>, grid, KQR_WAVES * 64, lds, s, w.qs, meta, aq, as, y, w.K, w.N, M, ldy, acc); \
    } while (0)
#define FH_KQR_SHAPE(Q6_)                                     \
    do {                                                      \
        if (pick == 0) FH_KQR(Q6_, 4, 8);                     \
        else if (pick == 1) FH_KQR(Q6_, 2, 8);                \
        else if (pick == 2) FH_KQR(Q6_, 4, 4);                \
        else FH_KQR(Q6_, 2, 4);                               \
    } while (0)
    if (q6) FH_KQR_SHAPE(true); else FH_KQR_SHAPE(false);
#undef FH_KQR_SHAPE
#undef FH_KQR
}

}  // namespace fh

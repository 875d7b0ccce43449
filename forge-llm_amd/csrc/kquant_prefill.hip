// Prompt matmuls for K-quant weights on the matrix unit (fast mode).
//
// The reference multiplies a Q4_K / Q6_K matrix one vector at a time (matmul_vec_q4_k_KxN, emit.rs:3388-3490; matmul_vec_q6_k_KxN,
// emit.rs:3622-3655) and walks a prompt through such a model token by token (emit.rs:4530-4534).  The order-faithful mode
// keeps that arithmetic (gemv_kquant.hip).  The fast mode re-expresses each matrix, once, as a matrix the int8 MFMA GEMM
// (gemm.hip) already multiplies -- int8 codes under one fp16 scale per block of 32, the Q8_0 layout -- its "twin":
//
//   Q4_K  w = d*sc_j * q - dmin*m_j, q = 0..15, per 32-element sub-block j, i.e.
//             sum_k x_k w_k  =  d*sc_j * sum x_k (q_k - 8)  +  (8 d*sc_j - dmin*m_j) * sum x_k
//         First term: codes (q - 8) * g under the scale fp16(d*sc_j / g), with the integer g = 9..15 that brings g * fp16(d*sc_j / g)
//         closest to d*sc_j (d*sc_j has up to 17 significant bits, fp16 has 11: among seven distinct roundings the best is
//         typically within 4e-5 of it, relative; that residue times the block's centred dot product is all that is dropped).
//         Second term: the block sums of the activations times a coefficient per (row, block), a small matmul of depth K/32
//         that the GEMM kernel runs on the f16 matrix unit in front of its epilogue (its mt_a / mt_w operands: hi | lo pairs).
//   Q6_K  w = d * sc_h * q, q = -32..31, sc_h an int8 per 16-element half.  sc_h * q = 64 hi + lo with lo in [-32, 31] and hi
//         in [-63, 64]: a block becomes two blocks of a matrix of depth 2K, the hi codes under the scale 64 d and the lo codes
//         under d.  Both scales are exact fp16 numbers (d is one), so nothing is dropped at all; the activations go in twice
//         (act_twice_kernel).  Blocks 2p, 2p + 1 of a row become hi(2p), hi(2p + 1), lo(2p), lo(2p + 1): neighbours of equal
//         scale, which is what the GEMM's alternating bias wants.
//
// Integer block sums stay exact; against the order-faithful result the difference is the order of the f32 additions and, for
// Q4_K, the residue above.
#include "common.h"
#include "device_utils.h"

namespace fh {

namespace {

// The operands of the minimum term travel as two fp16 numbers in the 4 bytes of an f32 slot: hi = fp16(x), lo = fp16(x - hi)
// (x to 2^-22 relative).  The GEMM multiplies them on the f16 matrix unit as hi*hi + hi*lo + lo*hi.  Powers of two keep both
// sides in fp16's range: activation block sums (up to 32 times the largest activation) arrive times 2^-8, coefficients times 2^8.
__device__ __forceinline__ float hi_lo_f16(float x) {
    const uint16_t h = f32_to_f16_bits(x);
    const uint16_t l = f32_to_f16_bits(x - f16_bits_to_f32(h));
    return __uint_as_float((uint32_t)h | ((uint32_t)l << 16));
}

// One thread per (row, 32-element block).  Planes of the source as gemv_kquant.hip lays them out.
__global__ __launch_bounds__(256) void twin_q4k_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, uint32_t K, uint64_t total,
                                                     int8_t* __restrict__ tq, uint16_t* __restrict__ ts, float* __restrict__ coef,
                                                     uint32_t* __restrict__ bad) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // n * nblk + b
    if (id >= total) return;
    const uint32_t nblk = K / 32;
    const uint64_t n = id / nblk;
    const uint32_t b = (uint32_t)(id % nblk), sb = b >> 3, j = b & 7, c = j >> 1;
    const uint8_t* mp = meta + (n * (K / 256) + sb) * 16;
    const float d = f16_bits_to_f32((uint16_t)(mp[0] | (mp[1] << 8))), dmin = f16_bits_to_f32((uint16_t)(mp[2] | (mp[3] << 8)));
    const uint8_t* s12 = mp + 4;
    uint32_t sc, mn;                                                       // get_scale_min_k4, emit.rs:3013-3021
    if (j < 4) { sc = s12[j] & 63u; mn = s12[j + 4] & 63u; }
    else {
        sc = (s12[j + 4] & 0x0Fu) | ((s12[j - 4] >> 6) << 4);
        mn = (s12[j + 4] >> 4) | ((s12[j] >> 6) << 4);
    }
    const float s = d * (float)sc;                                         // exact: 11 x 6 bits
    if (!(s >= 0.f) || !(s < 2.0f)) *bad = 1u;                             // outside what the GEMM's scale arithmetic covers
    // multipliers 9..15: seven different roundings (their odd parts differ), and codes that use the int8 range, which keeps
    // the GEMM's accumulation error small against the block sums
    int g = 15;
    uint16_t s16 = f32_to_f16_bits(s / 15.0f);
    float err = fabsf(f16_bits_to_f32(s16) * 15.0f - s);
    for (int cand = 14; cand >= 9; cand--) {
        const uint16_t h = f32_to_f16_bits(s / (float)cand);
        const float e = fabsf(f16_bits_to_f32(h) * (float)cand - s);
        if (e < err) { err = e; g = cand; s16 = h; }
    }
    ts[id] = s16;
    coef[id] = hi_lo_f16((8.0f * s - dmin * (float)mn) * 256.0f);
    // sub-block j = 2c + hi: element i is the low (hi = 0) or high nibble of byte 32 c + i
    const uint8_t* src = qs + (n * (K / 256) + sb) * 128 + 32 * c;
    const uint32_t sh = (j & 1) * 4;
    int8_t* dst = tq + id * 32;
    for (uint32_t i = 0; i < 32; i++) dst[i] = (int8_t)(((int)((src[i] >> sh) & 15u) - 8) * g);
}

__global__ __launch_bounds__(256) void twin_q6k_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, uint32_t K, uint64_t total,
                                                     int8_t* __restrict__ tq, uint16_t* __restrict__ ts, uint32_t* __restrict__ bad) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // n * nblk + b
    if (id >= total) return;
    const uint32_t nblk = K / 32;
    const uint64_t n = id / nblk;
    const uint32_t b = (uint32_t)(id % nblk), sb = b >> 3, jb = b & 7, h = jb >> 2, r = jb & 3;
    const uint8_t* sp = qs + (n * (K / 256) + sb) * 192;
    const uint8_t* mp = meta + (n * (K / 256) + sb) * 32;
    const float d = f16_bits_to_f32((uint16_t)(mp[16] | (mp[17] << 8)));
    const float mag = fabsf(d);
    if (!(mag * 64.0f < 2.0f)) *bad = 1u;
    const int sign = d < 0.f ? -1 : 1;
    // block 4h + r of the super-block: r = 0, 1 the low nibbles of ql[64h + 32r ..], r = 2, 3 the high nibbles of
    // ql[64h + 32(r - 2) ..]; bit pair r of qh[32h ..]
    const uint8_t* ql = sp + 64 * h + 32 * (r & 1);
    const uint8_t* qh = sp + 128 + 32 * h;
    const uint32_t nib_shift = (r >> 1) * 4, pair_shift = 2 * r;
    // blocks 2p + e of the row -> twin blocks 4p + e (hi) and 4p + 2 + e (lo)
    const uint64_t tb = n * 2 * nblk + 4 * (uint64_t)(b >> 1) + (b & 1);
    ts[tb] = f32_to_f16_bits(mag * 64.0f);                                 // exact: a power of two times an fp16 number
    ts[tb + 2] = f32_to_f16_bits(mag);
    int8_t* dst = tq + tb * 32;
    for (uint32_t i = 0; i < 32; i++) {
        const int q = (int)(((ql[i] >> nib_shift) & 15u) | (((qh[i] >> pair_shift) & 3u) << 4)) - 32;
        const int p = sign * (int)(int8_t)mp[2 * jb + (i >> 4)] * q;       // |p| <= 4096
        const int hi = (p + 32) >> 6;                                      // floor((p + 32) / 64): arithmetic shift
        dst[i] = (int8_t)hi;
        dst[64 + i] = (int8_t)(p - 64 * hi);
    }
}

// a_s[m][b] * sum of block b's codes * 2^-8 as a hi | lo pair of fp16 numbers, [M][K/32] slots of 4 bytes.  `neg_odd`: the codes of odd blocks arrive negated.
__global__ __launch_bounds__(256) void act_block_sums_kernel(const int8_t* __restrict__ aq, const uint16_t* __restrict__ as, uint64_t total,
                                                           uint32_t nblk, uint32_t neg_odd, float* __restrict__ out) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // m * nblk + b
    if (id >= total) return;
    const int4* p = reinterpret_cast<const int4*>(aq + id * 32);
    const int4 a0 = p[0], a1 = p[1];
    const int ones = 0x01010101;
    int sum = 0;
    sum = __builtin_amdgcn_sdot4(a0.x, ones, sum, false); sum = __builtin_amdgcn_sdot4(a0.y, ones, sum, false);
    sum = __builtin_amdgcn_sdot4(a0.z, ones, sum, false); sum = __builtin_amdgcn_sdot4(a0.w, ones, sum, false);
    sum = __builtin_amdgcn_sdot4(a1.x, ones, sum, false); sum = __builtin_amdgcn_sdot4(a1.y, ones, sum, false);
    sum = __builtin_amdgcn_sdot4(a1.z, ones, sum, false); sum = __builtin_amdgcn_sdot4(a1.w, ones, sum, false);
    if (neg_odd && ((id % nblk) & 1u)) sum = -sum;
    out[id] = hi_lo_f16(f16_bits_to_f32(as[id]) * (float)sum * 0.00390625f);
}

// Every pair of activation blocks twice, [M][2 K/32] blocks: blocks 2p, 2p + 1 of a row become 2p, 2p + 1, 2p, 2p + 1 (the hi
// and the lo blocks of a Q6_K twin meet the same activations).  Odd blocks stay odd, so codes that arrive with their odd
// blocks negated leave that way.
__global__ __launch_bounds__(256) void act_twice_kernel(const int8_t* __restrict__ aq, const uint16_t* __restrict__ as, uint64_t pairs,
                                                      int8_t* __restrict__ oq, uint16_t* __restrict__ os) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // pair * 4 + sixteen-byte quarter of the pair
    if (id >= pairs * 4) return;
    const uint64_t pair = id >> 2;
    const uint32_t part = (uint32_t)(id & 3);
    const int4 v = reinterpret_cast<const int4*>(aq)[id];
    int4* o = reinterpret_cast<int4*>(oq);
    o[pair * 8 + part] = v;
    o[pair * 8 + 4 + part] = v;
    if (part == 0) {
        const uint32_t s2 = reinterpret_cast<const uint32_t*>(as)[pair];
        reinterpret_cast<uint32_t*>(os)[pair * 2] = s2;
        reinterpret_cast<uint32_t*>(os)[pair * 2 + 1] = s2;
    }
}

}  // namespace

// One twin for `n` matrices of the same format and depth, their rows one after the other (q then k; gate then up): one GEMM
// launch for the group.  `*covered` = false (and no twin) when a block scale lies outside what the fast GEMM's scale
// arithmetic covers (a negative Q4_K scale, d * sc or 64 |d| not below 2): the caller keeps the multi-row GEMV.
int32_t kquant_twin_create(const QWeight* const* ws, uint32_t n, KqTwin* out, bool* covered, hipStream_t s) {
    *covered = false;
    const QWeight& w0 = *ws[0];
    uint64_t rows = 0;
    for (uint32_t i = 0; i < n; i++) {
        if (!ws[i]->kquant() || ws[i]->K % 256 != 0 || ws[i]->wdtype != w0.wdtype || ws[i]->K != w0.K) {
            set_error("kquant twin: K-quant matrices of one format and depth only");
            return FORGE_HIP_ERR_INVALID;
        }
        rows += ws[i]->N;
    }
    const uint32_t nblk = w0.K / 32;
    const bool q6 = w0.wdtype == FORGE_HIP_Q6_K;
    QWeight t;
    t.wdtype = FORGE_HIP_Q8_0;
    t.K = q6 ? 2 * w0.K : w0.K;
    t.N = (uint32_t)rows;
    t.owns = true;
    uint32_t* bad = nullptr;
    float* coef = nullptr;
    auto fail = [&](int32_t rc) {
        if (t.qs) (void)hipFree(t.qs);
        if (t.scales) (void)hipFree(t.scales);
        if (coef) (void)hipFree(coef);
        if (bad) (void)hipFree(bad);
        return rc;
    };
    if (hipMalloc(&t.qs, t.qs_bytes()) != hipSuccess || hipMalloc(&t.scales, t.scales_bytes()) != hipSuccess ||
        hipMalloc(&bad, 4) != hipSuccess || (!q6 && hipMalloc(&coef, rows * nblk * 4) != hipSuccess)) {
        (void)hipGetLastError();
        set_error("kquant twin: out of device memory");
        return fail(FORGE_HIP_ERR_HIP);
    }
    if (hipMemsetAsync(bad, 0, 4, s) != hipSuccess) return fail(FORGE_HIP_ERR_HIP);
    uint64_t row0 = 0;
    for (uint32_t i = 0; i < n; i++) {
        const QWeight& w = *ws[i];
        const uint64_t total = (uint64_t)w.N * nblk;
        const uint32_t grid = (uint32_t)((total + 255) / 256);
        const uint8_t* meta = reinterpret_cast<const uint8_t*>(w.scales);
        int8_t* tq = reinterpret_cast<int8_t*>(t.qs) + row0 * t.K;
        uint16_t* ts = t.scales + row0 * (t.K / 32);
        if (q6) fh::launch(twin_q6k_kernel, grid, 256, 0, s, w.qs, meta, w.K, total, tq, ts, bad);
        else fh::launch(twin_q4k_kernel, grid, 256, 0, s, w.qs, meta, w.K, total, tq, ts, coef + row0 * nblk, bad);
        row0 += w.N;
    }
    uint32_t flag = 0;
    if (hipMemcpyAsync(&flag, bad, 4, hipMemcpyDeviceToHost, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess) {
        set_error("kquant twin: conversion kernel failed");
        return fail(FORGE_HIP_ERR_HIP);
    }
    (void)hipFree(bad);
    bad = nullptr;
    if (flag) return fail(FORGE_HIP_OK);
    *covered = true;
    out->w = t;
    out->coef = coef;
    return FORGE_HIP_OK;
}

void kquant_twin_free(KqTwin* t) {
    if (!t) return;
    qweight_free(&t->w);
    if (t->coef) (void)hipFree(t->coef);
    t->coef = nullptr;
}

void launch_act_block_sums(const int8_t* aq, const uint16_t* as, uint32_t M, uint32_t K, bool neg_odd, float* out, hipStream_t s) {
    const uint64_t total = (uint64_t)M * (K / 32);
    if (total == 0) return;
    fh::launch(act_block_sums_kernel, (uint32_t)((total + 255) / 256), 256, 0, s, aq, as, total, K / 32, neg_odd ? 1u : 0u, out);
}

void launch_act_twice(const int8_t* aq, const uint16_t* as, uint32_t M, uint32_t K, int8_t* oq, uint16_t* os, hipStream_t s) {
    const uint64_t pairs = (uint64_t)M * (K / 64);
    if (pairs == 0) return;
    fh::launch(act_twice_kernel, (uint32_t)((pairs * 4 + 255) / 256), 256, 0, s, aq, as, pairs, oq, os);
}

}  // namespace fh

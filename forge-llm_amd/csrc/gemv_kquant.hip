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

// LDS: the activation codes [K], their scales as f32 [K/32], (Q4_K) their sums as f32 [K/32], then per wave the products
// [RW][prod_stride(K/32)].  A wave works RW rows at a time: all their loads are issued before the first is used (one row of
// K = 2048 is a single kilobyte, far too little in flight for HBM), and lane r adds row r's products in block order.
template <bool Q6, int RW>
__global__ __launch_bounds__(KQ_WAVES * 64) void gemv_kquant_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta,
                                                                  const int8_t* __restrict__ aq, const uint16_t* __restrict__ as,
                                                                  float* __restrict__ y, uint32_t K, uint32_t N, int accumulate) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nblk = K / 32, nsb = K / 256, pstride = prod_stride(nblk);
    int8_t* xa = reinterpret_cast<int8_t*>(lds);
    float* xs = reinterpret_cast<float*>(lds + K);
    float* xsum = xs + nblk;
    float* prod = xsum + nblk + (size_t)wave * RW * pstride;
    for (uint32_t i = tid; i < K / 16; i += KQ_WAVES * 64) reinterpret_cast<int4*>(xa)[i] = reinterpret_cast<const int4*>(aq)[i];
    for (uint32_t b = tid; b < nblk; b += KQ_WAVES * 64) {
        xs[b] = f16_bits_to_f32(as[b]);
        if (!Q6) {
            const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
            const int4 a0 = reinterpret_cast<const int4*>(aq + (size_t)b * 32)[0], a1 = reinterpret_cast<const int4*>(aq + (size_t)b * 32)[1];
            xsum[b] = (float)kq_dot16(ones, a1, kq_dot16(ones, a0, 0));
        }
    }
    __syncthreads();

    // a row is nsb * 8 pieces of 16 bytes of the first plane; piece p = 8 sb + t belongs to lane p % 64 of pass p / 64
    const uint32_t pieces = nsb * 8;
    for (uint32_t row0 = (blockIdx.x * KQ_WAVES + wave) * RW; row0 < N; row0 += gridDim.x * KQ_WAVES * RW) {
        for (uint32_t p0 = 0; p0 < pieces; p0 += 64) {
            const uint32_t p = p0 + lane;
            if (p < pieces) {
                const uint32_t sb = p >> 3, t = p & 7, e = t & 1;
                if (!Q6) {
                    // piece t: bytes [16 t, +16) of the super-block's nibbles = elements [16 e, +16) of sub-blocks 2c (low
                    // nibbles) and 2c + 1 (high nibbles), c = t / 2
                    const uint32_t c = t >> 1;
                    int4 wv[RW];
                    uint4 mv[RW];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const size_t row = min(row0 + r, N - 1);          // past the end: the last row again, never stored
                        wv[r] = *reinterpret_cast<const int4*>(qs + (row * nsb + sb) * 128 + t * 16);
                        mv[r] = *reinterpret_cast<const uint4*>(meta + (row * nsb + sb) * 16);
                    }
                    const uint32_t b_lo = sb * 8 + 2 * c;
                    const int4 a_lo = *reinterpret_cast<const int4*>(xa + b_lo * 32 + e * 16);
                    const int4 a_hi = *reinterpret_cast<const int4*>(xa + (b_lo + 1) * 32 + e * 16);
                    // the even lane of the pair finishes sub-block 2c, the odd lane 2c + 1
                    const uint32_t j = 2 * c + e, b = sb * 8 + j;
                    const float x_s = xs[b], x_sum = xsum[b];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const int4 w = wv[r];
                        const uint4 mt = mv[r];
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
                    uint4 qlv[RW], qhv[RW], scv[RW];
                    uint32_t dv[RW];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const size_t row = min(row0 + r, N - 1);
                        const uint8_t* sbp = qs + (row * nsb + sb) * 192;
                        qlv[r] = *reinterpret_cast<const uint4*>(sbp + 64 * h + 32 * pp + 16 * e);
                        qhv[r] = *reinterpret_cast<const uint4*>(sbp + 128 + 32 * h + 16 * e);
                        const uint8_t* mp = meta + (row * nsb + sb) * 32;
                        scv[r] = *reinterpret_cast<const uint4*>(mp);                 // the 16 int8 sub-block scales
                        dv[r] = *reinterpret_cast<const uint32_t*>(mp + 16);          // d (fp16) in the low half
                    }
                    const uint32_t bA = sb * 8 + 4 * h + pp, bB = bA + 2;
                    const int4 xA = *reinterpret_cast<const int4*>(xa + bA * 32 + e * 16);
                    const int4 xB = *reinterpret_cast<const int4*>(xa + bB * 32 + e * 16);
                    const float xsA = xs[bA], xsB = xs[bB];
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        const uint32_t qlw[4] = {qlv[r].x, qlv[r].y, qlv[r].z, qlv[r].w}, qhw[4] = {qhv[r].x, qhv[r].y, qhv[r].z, qhv[r].w};
                        const uint32_t scw[4] = {scv[r].x, scv[r].y, scv[r].z, scv[r].w};
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
                            const float d = f16_bits_to_f32((uint16_t)(dv[r] & 0xFFFFu));
                            prod[r * pstride + bA] = (d * xsA) * uA;
                            prod[r * pstride + bB] = (d * xsB) * uB;
                        }
                    }
                }
            }
        }
        // LDS operations of one wave execute in order: the products are there.  Lane r adds row r's.
        if (lane < RW && row0 + lane < N) {
            float r = ordered_sum(prod + lane * pstride, nblk, false);
            if (accumulate) r = y[row0 + lane] + r;
            y[row0 + lane] = r;
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

void launch_gemv_kquant(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, hipStream_t s) {
    if (w.N == 0) return;
    const uint32_t nblk = w.K / 32;
    // rows a wave keeps in flight: four when that still leaves every CU several workgroups
    const int rw = w.N >= 16384 ? 4 : w.N >= 4096 ? 2 : 1;
    const size_t lds = (size_t)w.K + (size_t)nblk * 8 + (size_t)KQ_WAVES * rw * prod_stride(nblk) * 4;
    uint32_t grid = (w.N + KQ_WAVES * rw - 1) / (KQ_WAVES * rw);
    if (grid > 256 * 8) grid = 256 * 8;
    const uint8_t* meta = reinterpret_cast<const uint8_t*>(w.scales);
    const int acc = accumulate ? 1 : 0;
#define FH_KQ(Q6_, RW_) fh::launch(gemv_kquant_kernel<Q6_, RW_>, grid, KQ_WAVES * 64, lds, s, w.qs, meta, aq, as, y, w.K, w.N, acc)
    if (w.wdtype == FORGE_HIP_Q6_K) { if (rw == 4) FH_KQ(true, 4); else if (rw == 2) FH_KQ(true, 2); else FH_KQ(true, 1); }
    else { if (rw == 4) FH_KQ(false, 4); else if (rw == 2) FH_KQ(false, 2); else FH_KQ(false, 1); }
#undef FH_KQ
}

}  // namespace fh

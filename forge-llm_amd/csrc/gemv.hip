// Decode-time quantised GEMV (matmul_vec_q8_0_KxN / matmul_vec_q4_0_KxN, emit.rs:1926-2092,
// 2797-2958): y[n] = sum_b (a_s[b]*w_s[n][b]) * f32(isum_b), isum_b the exact int32 dot of
// the 32 int8 activation codes of block b with the 32 weight codes.
//
// HBM-bound: every weight byte is read once, with 16-byte loads that are contiguous
// across the wave.  No LDS, no MFMA.  A wave owns RW consecutive rows at a time and keeps
// the quantised activation vector in registers for all of them.
//
// Q8_0: lane l of chunk j holds bytes [1024 j + 16 l, +16) of the row = half of block
//       32 j + l/2; the two halves are added as integers across the lane pair.
// Q4_0: lane l of chunk j holds the 16 packed bytes of block 64 j + l; nibbles are split
//       with masks and the -8 offset is applied as  sum((c-8) a) = sum(c a) - 8 sum(a).
#include "common.h"
#include "device_utils.h"

namespace fh {

__device__ __forceinline__ int dot16(int4 w, int4 a, int acc) {
    acc = __builtin_amdgcn_sdot4(w.x, a.x, acc, false);
    acc = __builtin_amdgcn_sdot4(w.y, a.y, acc, false);
    acc = __builtin_amdgcn_sdot4(w.z, a.z, acc, false);
    acc = __builtin_amdgcn_sdot4(w.w, a.w, acc, false);
    return acc;
}

// ISUMS: write the int32 block sums instead of y (debug/parity entry point).
template <int NCH, int RW, bool ISUMS>
__global__ __launch_bounds__(256) void gemv_q8_kernel(const uint8_t* __restrict__ qs, const uint16_t* __restrict__ ws,
                                                      const int8_t* __restrict__ aq, const uint16_t* __restrict__ as,
                                                      float* __restrict__ y, int32_t* __restrict__ isums, uint32_t K,
                                                      uint32_t N, int accumulate) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t nblk = K / 32;
    // activation fragment: NCH chunks of 16 codes, plus the block scale (zero on odd lanes so
    // that each block is counted once)
    int4 av[NCH];
    float asf[NCH];
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const uint32_t off = j * 1024 + lane * 16;
        if (off < K) {
            av[j] = *reinterpret_cast<const int4*>(aq + off);
            asf[j] = (ISUMS || (lane & 1)) ? 0.f : f16_bits_to_f32(as[off / 32]);
        } else {
            av[j] = make_int4(0, 0, 0, 0);
            asf[j] = 0.f;
        }
    }
    const uint32_t groups = (N + RW - 1) / RW;
    for (uint32_t g = blockIdx.x * 4 + wave; g < groups; g += gridDim.x * 4) {
        const uint32_t row0 = g * RW;
        int4 wv[RW][NCH];
        uint16_t wsb[RW][NCH];
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t row = min(row0 + r, N - 1);
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const uint32_t off = j * 1024 + lane * 16;
                if (off < K) {
                    wv[r][j] = *reinterpret_cast<const int4*>(qs + (size_t)row * K + off);
                    wsb[r][j] = ws[(size_t)row * nblk + off / 32];
                } else {
                    wv[r][j] = make_int4(0, 0, 0, 0);
                    wsb[r][j] = 0;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RW; r++) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                int half = dot16(wv[r][j], av[j], 0);
                int isum = half + __shfl_xor(half, 1, WAVE);
                if (ISUMS) {
                    const uint32_t off = j * 1024 + lane * 16;
                    if (!(lane & 1) && off < K && row0 + r < N) isums[(size_t)(row0 + r) * nblk + off / 32] = isum;
                } else {
                    acc += (asf[j] * f16_bits_to_f32(wsb[r][j])) * (float)isum;
                }
            }
            if (!ISUMS) {
                acc = wave_sum(acc);
                if (lane == 0 && row0 + r < N) {
                    if (accumulate) y[row0 + r] += acc;
                    else y[row0 + r] = acc;
                }
            }
        }
    }
}

template <int NCH, int RW, bool ISUMS>
__global__ __launch_bounds__(256) void gemv_q4_kernel(const uint8_t* __restrict__ qs, const uint16_t* __restrict__ ws,
                                                      const int8_t* __restrict__ aq, const uint16_t* __restrict__ as,
                                                      float* __restrict__ y, int32_t* __restrict__ isums, uint32_t K,
                                                      uint32_t N, int accumulate) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t nblk = K / 32;
    // activation fragment: chunk j covers blocks [64 j, 64 j + 64); lane l owns block 64 j + l
    int4 alo[NCH], ahi[NCH];
    int asum8[NCH];
    float asf[NCH];
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const uint32_t b = j * 64 + lane;
        if (b < nblk) {
            alo[j] = *reinterpret_cast<const int4*>(aq + (size_t)b * 32);
            ahi[j] = *reinterpret_cast<const int4*>(aq + (size_t)b * 32 + 16);
            asf[j] = ISUMS ? 0.f : f16_bits_to_f32(as[b]);
            const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
            asum8[j] = 8 * dot16(ones, ahi[j], dot16(ones, alo[j], 0));
        } else {
            alo[j] = ahi[j] = make_int4(0, 0, 0, 0);
            asf[j] = 0.f;
            asum8[j] = 0;
        }
    }
    const uint32_t groups = (N + RW - 1) / RW;
    const size_t row_bytes = (size_t)K / 2;
    for (uint32_t g = blockIdx.x * 4 + wave; g < groups; g += gridDim.x * 4) {
        const uint32_t row0 = g * RW;
        int4 wv[RW][NCH];
        uint16_t wsb[RW][NCH];
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t row = min(row0 + r, N - 1);
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const uint32_t b = j * 64 + lane;
                if (b < nblk) {
                    wv[r][j] = *reinterpret_cast<const int4*>(qs + (size_t)row * row_bytes + (size_t)b * 16);
                    wsb[r][j] = ws[(size_t)row * nblk + b];
                } else {
                    wv[r][j] = make_int4(0, 0, 0, 0);
                    wsb[r][j] = 0;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RW; r++) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const int4 w = wv[r][j];
                const int m = 0x0F0F0F0F;
                int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                int isum = dot16(hi, ahi[j], dot16(lo, alo[j], 0)) - asum8[j];
                if (ISUMS) {
                    const uint32_t b = j * 64 + lane;
                    if (b < nblk && row0 + r < N) isums[(size_t)(row0 + r) * nblk + b] = isum;
                } else {
                    acc += (asf[j] * f16_bits_to_f32(wsb[r][j])) * (float)isum;
                }
            }
            if (!ISUMS) {
                acc = wave_sum(acc);
                if (lane == 0 && row0 + r < N) {
                    if (accumulate) y[row0 + r] += acc;
                    else y[row0 + r] = acc;
                }
            }
        }
    }
}

namespace {

// Rows per wave: enough independent 16-byte loads in flight per lane (RW*NCH), without
// starving the grid on small matrices.
template <int NCH, bool ISUMS>
void launch_q8(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, int32_t* isums, bool acc,
               hipStream_t s) {
    constexpr int RW = NCH >= 8 ? 1 : (NCH >= 3 ? 2 : 4);
    uint32_t groups = (w.N + RW - 1) / RW;
    uint32_t grid = (groups + 3) / 4;
    if (grid > 256 * 8) grid = 256 * 8;
    gemv_q8_kernel<NCH, RW, ISUMS><<<grid, 256, 0, s>>>(w.qs, w.scales, aq, as, y, isums, w.K, w.N, acc ? 1 : 0);
}
template <int NCH, bool ISUMS>
void launch_q4(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, int32_t* isums, bool acc,
               hipStream_t s) {
    constexpr int RW = NCH >= 4 ? 2 : 4;
    uint32_t groups = (w.N + RW - 1) / RW;
    uint32_t grid = (groups + 3) / 4;
    if (grid > 256 * 8) grid = 256 * 8;
    gemv_q4_kernel<NCH, RW, ISUMS><<<grid, 256, 0, s>>>(w.qs, w.scales, aq, as, y, isums, w.K, w.N, acc ? 1 : 0);
}

template <bool ISUMS>
void dispatch(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, int32_t* isums, bool acc,
              hipStream_t s) {
    if (w.wdtype == FORGE_HIP_Q8_0) {
        uint32_t nch = (w.K + 1023) / 1024;
        switch (nch) {
            case 1: launch_q8<1, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 2: launch_q8<2, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 3: launch_q8<3, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 4: launch_q8<4, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 5: case 6: launch_q8<6, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 7: case 8: launch_q8<8, ISUMS>(w, aq, as, y, isums, acc, s); break;
            default: launch_q8<16, ISUMS>(w, aq, as, y, isums, acc, s); break;
        }
    } else {
        uint32_t nch = (w.K + 2047) / 2048;
        switch (nch) {
            case 1: launch_q4<1, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 2: launch_q4<2, ISUMS>(w, aq, as, y, isums, acc, s); break;
            case 3: case 4: launch_q4<4, ISUMS>(w, aq, as, y, isums, acc, s); break;
            default: launch_q4<8, ISUMS>(w, aq, as, y, isums, acc, s); break;
        }
    }
}

}  // namespace

// Largest K the register-resident activation fragment covers.
bool gemv_k_supported(uint32_t K) { return K % 32 == 0 && K >= 32 && K <= 16384; }

void launch_gemv(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, hipStream_t s) {
    dispatch<false>(w, aq, as, y, nullptr, accumulate, s);
}
void launch_gemv_isums(const QWeight& w, const int8_t* aq, int32_t* out, hipStream_t s) {
    dispatch<true>(w, aq, nullptr, nullptr, out, false, s);
}

}  // namespace fh

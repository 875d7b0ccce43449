// The reference's portable row dots (dot_q8_0 / dot_q4_0 on hosts other than aarch64, emit.rs:1359-1377 and
// 2337-2359) as a GEMV:  y[n] = sum over the row, element by element and in order, of  x[k] * (f32(q) * scale),
// f32 activations against weights dequantised on the fly -- the arithmetic an x86 build of the reference runs
// (matmul_vec calls the dot once per row, emit.rs:2046-2092; every row takes the same order).  It exists so that this
// arithmetic has a GPU counterpart that can be held to the CPU path bit for bit; the decode path proper uses the int8
// block-dot kernels (gemv.hip), which stream four times fewer activation bytes and use v_dot4.
//
// The sum of a row is one chain of K dependent f32 additions (the products are independent), so a lane owns a row
// and walks it; 64 rows share a wave.  Weight bytes reach the lanes through LDS: the wave loads a [64 rows x 128
// elements] tile with coalesced 16-byte loads (8 rows x 128 B per instruction for Q8_0, 16 rows x 64 B for Q4_0) into
// rows padded by 16 bytes, from where each lane reads its own row 16 bytes at a time without bank conflicts; the 128
// activations of the tile are read from LDS as broadcasts.  Multiplies and adds are not fused, as on the CPU.
#include "common.h"
#include "device_utils.h"

namespace fh {

constexpr int PV_ROWS = 64, PV_ELEMS = 128;

template <bool Q4>
__global__ __launch_bounds__(64) void gemv_f32_kernel(const uint8_t* __restrict__ qs, const uint16_t* __restrict__ ws,
                                                      const float* __restrict__ x, float* __restrict__ y, uint32_t K, uint32_t N) {
    constexpr int ROW_BYTES = Q4 ? PV_ELEMS / 2 : PV_ELEMS;      // bytes of one row's share of a tile
    constexpr int PITCH = ROW_BYTES + 16;
    __shared__ __attribute__((aligned(16))) uint8_t tile[PV_ROWS * PITCH];
    __shared__ __attribute__((aligned(16))) float xs[PV_ELEMS];
    const uint32_t lane = threadIdx.x;
    const uint32_t row0 = blockIdx.x * PV_ROWS, row = row0 + lane;
    const uint32_t nblk = K / 32, wrow = Q4 ? K / 2 : K;
    constexpr int LPR = ROW_BYTES / 16;                          // lanes that cover one row of the tile
    constexpr int RPI = 64 / LPR;                                // rows per load instruction
    float sum = 0.f;
    for (uint32_t k0 = 0; k0 < K; k0 += PV_ELEMS) {
        const uint32_t kb = Q4 ? k0 / 2 : k0;                    // byte offset of the tile in a row
        __syncthreads();                                         // the previous tile has been consumed
#pragma unroll
        for (int i = 0; i < PV_ROWS / RPI; i++) {
            const uint32_t r = i * RPI + lane / LPR, c = (lane % LPR) * 16;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (row0 + r < N && kb + c < wrow) v = *reinterpret_cast<const uint4*>(qs + (size_t)(row0 + r) * wrow + kb + c);
            *reinterpret_cast<uint4*>(tile + r * PITCH + c) = v;
        }
        if (lane < PV_ELEMS / 4) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (k0 + lane * 4 < K) v = *reinterpret_cast<const float4*>(x + k0 + lane * 4);
            *reinterpret_cast<float4*>(xs + lane * 4) = v;
        }
        __syncthreads();
        if (row < N) {
#pragma unroll
            for (int b = 0; b < PV_ELEMS / 32; b++) {
                if (k0 + b * 32 >= K) break;
                const float scale = f16_bits_to_f32(ws[(size_t)row * nblk + k0 / 32 + b]);
                if (Q4) {
                    // byte j of a block: element j in the low nibble, j + 16 in the high; the reference adds them in that order
                    const uint4 p = *reinterpret_cast<const uint4*>(tile + lane * PITCH + b * 16);
                    const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
                    for (int j = 0; j < 16; j++) {
                        const uint32_t byte = (w[j / 4] >> (8 * (j % 4))) & 0xFFu;
                        const int lo = (int)(byte & 0x0Fu) - 8, hi = (int)(byte >> 4) - 8;
                        sum = sum + xs[b * 32 + j] * ((float)lo * scale);
                        sum = sum + xs[b * 32 + j + 16] * ((float)hi * scale);
                    }
                } else {
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const uint4 p = *reinterpret_cast<const uint4*>(tile + lane * PITCH + b * 32 + h * 16);
                        const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
                        for (int j = 0; j < 16; j++) {
                            const int q = (int)(int8_t)((w[j / 4] >> (8 * (j % 4))) & 0xFFu);
                            sum = sum + xs[b * 32 + h * 16 + j] * ((float)q * scale);
                        }
                    }
                }
            }
        }
    }
    if (row < N) y[row] = sum;
}

void launch_gemv_f32(const QWeight& w, const float* x, float* y, hipStream_t s) {
    if (w.N == 0) return;
    const uint32_t grid = (w.N + PV_ROWS - 1) / PV_ROWS;
    if (w.wdtype == FORGE_HIP_Q4_0) fh::launch(gemv_f32_kernel<true>, grid, 64, 0, s, w.qs, w.scales, x, y, w.K, w.N);
    else fh::launch(gemv_f32_kernel<false>, grid, 64, 0, s, w.qs, w.scales, x, y, w.K, w.N);
}

}  // namespace fh

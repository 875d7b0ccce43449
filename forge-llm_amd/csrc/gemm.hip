// Batched-prefill quantised GEMM (matmul_mat_q8_0_KxN / matmul_mat_q4_0_KxN, emit.rs:2108-2302,
// 3667-3817):  y[m][n] = sum_b (a_s[m][b] * w_s[n][b]) * f32(isum[m][n][b]).
//
// Both products of the formula run on the matrix unit:
//   * v_mfma_i32_32x32x32_i8 has K = 32 = exactly one quant block, so each MFMA result is a 32x32 tile
//     of exact int32 block sums;
//   * the scale products a_s[m]*w_s[n] of that tile are a rank-1 outer product of fp16 values, exact in
//     f32 (11-bit x 11-bit significands): one v_mfma_f32_32x32x16_f16 with the scales in k = 0 and zeros
//     elsewhere (fp16 subnormal scales included; the unit does not flush them).
// The scaling itself is elementwise in (m, n, b) and has to be done on the VALU: int->float and one
// multiply-add per element (in exact mode multiply then add, which is bit for bit the reference's
// `r += (a_scale*w_scale) * f32(isum)` in block order).  That VALU work, not the matrix unit, bounds the
// kernel: 32 VALU instructions (128 cycles) per 64 cycles of MFMA.
//
// Tiling: 256 threads = 4 waves (2x2), workgroup tile 128 (m) x 128 (n), wave tile 64x64 = 2x2 MFMA
// tiles, K step 128 (4 blocks) staged through padded LDS.  Activations are the MFMA A operand (rows),
// weights the B operand (columns): a lane's 16 results share one weight row n, stores are contiguous in n.
// Two waves per SIMD (<= 256 VGPRs) so that MFMA results land in ordinary VGPRs, not AccVGPRs.
#include "common.h"
#include "device_utils.h"

namespace fh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int BM = 128, BN = 128, BK = 128;   // BK in elements (= bytes of int8)
constexpr int LDS_STRIDE = BK + 16;           // padded row stride: conflict-free 16-byte reads
constexpr int KB = BK / 32;                   // quant blocks per stage

// (c - 8) for each of four nibble codes c held in the low nibbles of the four bytes.
__device__ __forceinline__ uint32_t nib_minus8(uint32_t x) {
    return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// EXACT: multiply then add per block (bit-identical to the CPU path); otherwise one FMA per block.
template <bool Q4, bool DUMP, bool EXACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_q_kernel(const uint8_t* __restrict__ wq, const uint16_t* __restrict__ wsc, const int8_t* __restrict__ aq,
                   const uint16_t* __restrict__ asc, float* __restrict__ y, int32_t* __restrict__ isums, uint32_t M,
                   uint32_t N, uint32_t K, uint32_t ldy, int accumulate) {
    __shared__ __attribute__((aligned(16))) int8_t As[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) int8_t Bs[BN * LDS_STRIDE];
    __shared__ uint16_t Asc[KB][BM];     // fp16 scale bits
    __shared__ uint16_t Bsc[KB][BN];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t nblk = K / 32;
    const uint32_t lrow = lane & 31, lhalf = lane >> 5;

    float acc[2][2][16];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    // staging registers (global -> regs -> LDS)
    int4 ra[4];
    int4 rb[Q4 ? 2 : 4];
    uint16_t rs[KB];

    auto load_stage = [&](uint32_t k0) {
        // activations: 128 rows x 128 B; thread t takes 16-byte piece (t + 256 i): row = idx/8, c = idx%8
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t idx = tid + 256 * i, row = idx >> 3, c = idx & 7;
            const uint32_t m = m0 + row, k = k0 + c * 16;
            ra[i] = (m < M && k < K) ? *reinterpret_cast<const int4*>(aq + (size_t)m * K + k) : make_int4(0, 0, 0, 0);
        }
        if (Q4) {
            // weights: 128 rows x 4 blocks x 16 packed bytes; piece idx: row = idx/4, blk = idx%4
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t idx = tid + 256 * i, row = idx >> 2, bl = idx & 3;
                const uint32_t n = n0 + row, b = k0 / 32 + bl;
                rb[i] = (n < N && b < nblk) ? *reinterpret_cast<const int4*>(wq + ((size_t)n * nblk + b) * 16)
                                            : make_int4(0x88888888, 0x88888888, 0x88888888, 0x88888888);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t idx = tid + 256 * i, row = idx >> 3, c = idx & 7;
                const uint32_t n = n0 + row, k = k0 + c * 16;
                rb[i] = (n < N && k < K) ? *reinterpret_cast<const int4*>(wq + (size_t)n * K + k) : make_int4(0, 0, 0, 0);
            }
        }
        // scales: threads 0..127 take activation row t, threads 128..255 weight row t-128
        {
            const bool is_a = tid < 128;
            const uint32_t row = is_a ? tid : tid - 128;
            const uint32_t g = (is_a ? m0 : n0) + row;
            const bool ok = is_a ? (g < M) : (g < N);
            const uint16_t* src = (is_a ? asc : wsc) + (size_t)g * nblk + k0 / 32;
#pragma unroll
            for (int b = 0; b < KB; b++) rs[b] = (ok && k0 / 32 + b < nblk) ? src[b] : (uint16_t)0;
        }
    };

    auto store_stage = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t idx = tid + 256 * i, row = idx >> 3, c = idx & 7;
            *reinterpret_cast<int4*>(As + row * LDS_STRIDE + c * 16) = ra[i];
        }
        if (Q4) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t idx = tid + 256 * i, row = idx >> 2, bl = idx & 3;
                const int4 p = rb[i];
                const uint32_t m = 0x0F0F0F0Fu;
                int4 lo, hi;
                lo.x = nib_minus8((uint32_t)p.x & m); lo.y = nib_minus8((uint32_t)p.y & m);
                lo.z = nib_minus8((uint32_t)p.z & m); lo.w = nib_minus8((uint32_t)p.w & m);
                hi.x = nib_minus8(((uint32_t)p.x >> 4) & m); hi.y = nib_minus8(((uint32_t)p.y >> 4) & m);
                hi.z = nib_minus8(((uint32_t)p.z >> 4) & m); hi.w = nib_minus8(((uint32_t)p.w >> 4) & m);
                *reinterpret_cast<int4*>(Bs + row * LDS_STRIDE + bl * 32) = lo;       // elements 0..15
                *reinterpret_cast<int4*>(Bs + row * LDS_STRIDE + bl * 32 + 16) = hi;  // elements 16..31
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t idx = tid + 256 * i, row = idx >> 3, c = idx & 7;
                *reinterpret_cast<int4*>(Bs + row * LDS_STRIDE + c * 16) = rb[i];
            }
        }
        {
            const bool is_a = tid < 128;
            const uint32_t row = is_a ? tid : tid - 128;
#pragma unroll
            for (int b = 0; b < KB; b++) {
                if (is_a) Asc[b][row] = rs[b];
                else Bsc[b][row] = rs[b];
            }
        }
    };

    const v16i zero_i = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const v16f zero_f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    load_stage(0);
    for (uint32_t k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();   // previous stage fully consumed
        store_stage();
        __syncthreads();
        if (k0 + BK < K) load_stage(k0 + BK);   // prefetch next stage into registers
#pragma unroll 1
        for (int kb = 0; kb < KB; kb++) {
            v4i af[2], bf[2];
            v8h sa[2], sb[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                af[t] = *reinterpret_cast<const v4i*>(As + (wm * 64 + t * 32 + lrow) * LDS_STRIDE + kb * 32 + lhalf * 16);
                bf[t] = *reinterpret_cast<const v4i*>(Bs + (wn * 64 + t * 32 + lrow) * LDS_STRIDE + kb * 32 + lhalf * 16);
                // operands of the rank-1 scale product: the scale in k = 0 (lanes 0..31), zeros elsewhere
                const uint16_t sab = lhalf ? (uint16_t)0 : Asc[kb][wm * 64 + t * 32 + lrow];
                const uint16_t sbb = lhalf ? (uint16_t)0 : Bsc[kb][wn * 64 + t * 32 + lrow];
                const _Float16 z = (_Float16)0.0f;
                sa[t] = (v8h){__builtin_bit_cast(_Float16, sab), z, z, z, z, z, z, z};
                sb[t] = (v8h){__builtin_bit_cast(_Float16, sbb), z, z, z, z, z, z, z};
            }
            // four tiles, software-pipelined by one: the MFMAs of tile t+1 are issued before tile t is combined,
            // so the matrix unit works while the VALU scales, and only two tiles of temporaries are live
            v16i isum = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[0], bf[0], zero_i, 0, 0, 0);
            v16f S = __builtin_amdgcn_mfma_f32_32x32x16_f16(sa[0], sb[0], zero_f, 0, 0, 0);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int tm = t >> 1, tn = t & 1;
                v16i isum_n = zero_i;
                v16f S_n = zero_f;
                if (t < 3) {
                    const int tm2 = (t + 1) >> 1, tn2 = (t + 1) & 1;
                    isum_n = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tm2], bf[tn2], zero_i, 0, 0, 0);
                    S_n = __builtin_amdgcn_mfma_f32_32x32x16_f16(sa[tm2], sb[tn2], zero_f, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float f = (float)isum[r];
                    if (EXACT) acc[tm][tn][r] = acc[tm][tn][r] + S[r] * f;
                    else acc[tm][tn][r] = fmaf(S[r], f, acc[tm][tn][r]);
                }
                if (DUMP) {
                    const uint32_t b = k0 / 32 + kb;
                    const uint32_t n = n0 + wn * 64 + tn * 32 + lrow;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const uint32_t m = m0 + wm * 64 + tm * 32 + 8 * (r >> 2) + 4 * lhalf + (r & 3);
                        if (m < M && n < N && b < nblk) isums[((size_t)m * N + n) * nblk + b] = isum[r];
                    }
                }
                isum = isum_n;
                S = S_n;
            }
        }
    }

    // epilogue: lane holds column n = lrow, rows 8g + 4*lhalf + (r&3)
#pragma unroll
    for (int tm = 0; tm < 2; tm++)
#pragma unroll
        for (int tn = 0; tn < 2; tn++) {
            const uint32_t n = n0 + wn * 64 + tn * 32 + lrow;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t m = m0 + wm * 64 + tm * 32 + 8 * (r >> 2) + 4 * lhalf + (r & 3);
                if (m < M && n < N) {
                    float* p = y + (size_t)m * ldy + n;
                    if (accumulate) *p = *p + acc[tm][tn][r];
                    else *p = acc[tm][tn][r];
                }
            }
        }
}

void launch_gemm(const QWeight& w, const int8_t* aq, const uint16_t* as, uint32_t M, float* y, uint32_t ldy,
                 bool accumulate, bool exact, int32_t* isums, hipStream_t s) {
    if (M == 0) return;
    dim3 grid((w.N + BN - 1) / BN, (M + BM - 1) / BM);
    const int accf = accumulate ? 1 : 0;
    const bool q4 = w.wdtype == FORGE_HIP_Q4_0;
#define FH_GEMM_LAUNCH(Q4_, DUMP_, EXACT_) \
    fh::launch(gemm_q_kernel<Q4_, DUMP_, EXACT_>, grid, 256, 0, s, w.qs, w.scales, aq, as, y, isums, M, w.N, w.K, ldy, accf)
    if (q4) {
        if (isums) FH_GEMM_LAUNCH(true, true, true);
        else if (exact) FH_GEMM_LAUNCH(true, false, true);
        else FH_GEMM_LAUNCH(true, false, false);
    } else {
        if (isums) FH_GEMM_LAUNCH(false, true, true);
        else if (exact) FH_GEMM_LAUNCH(false, false, true);
        else FH_GEMM_LAUNCH(false, false, false);
    }
#undef FH_GEMM_LAUNCH
}

}  // namespace fh

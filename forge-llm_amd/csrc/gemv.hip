// Decode-time quantised GEMV (matmul_vec_q8_0_KxN / matmul_vec_q4_0_KxN, emit.rs:1926-2092,
// 2797-2958): y[n] = sum_b (a_s[b]*w_s[n][b]) * f32(isum_b), isum_b the exact int32 dot of
// the 32 int8 activation codes of block b with the 32 weight codes.
//
// HBM-bound: every weight byte is read once, with 16-byte loads that are contiguous
// across the wave; the int8 products run on v_dot4, no MFMA.  A wave owns RW consecutive
// rows at a time and keeps the quantised activation vector in registers for all of them.
//
// Q8_0: lane l of chunk j holds bytes [1024 j + 16 l, +16) of the row = half of block
//       32 j + l/2; the two halves are added as integers across the lane pair.
// Q4_0: lane l of chunk j holds the 16 packed bytes of block 64 j + l; nibbles are split
//       with masks and the -8 offset is applied as  sum((c-8) a) = sum(c a) - 8 sum(a).
//
// The f32 combine follows the reference's order exactly, because the result feeds an int8
// quantiser further down and a last-bit difference there changes tokens: every block's
// product (a_s*w_s)*f32(isum) is parked in LDS and one lane per row then adds them in block
// order (dot8/dot4: one accumulator, emit.rs:1770-1877; the N%4 tail rows of dot1: four
// interleaved accumulators, emit.rs:1558-1571).  Multiplies and adds are not fused (Rust
// never contracts).
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

struct GemvArgs {
    const uint8_t* qs;
    const uint16_t* ws;
    const int8_t* aq;
    const uint16_t* as;
    float* y;
    int32_t* isums;
    uint32_t K, N;
    uint32_t rc;          // rows per ordered-sum group (per wave)
    uint32_t chunk;       // 0, or 256: rows are grouped in chunks of this many for the tail rule
    uint32_t tail_mod;    // the last (len % tail_mod) rows of a chunk use the 4-accumulator order
    int accumulate;
};

// Ordered sum of one row's block products p[0..nblk): sequential, or the dot1 order.
__device__ __forceinline__ float ordered_sum(const float* p, uint32_t nblk, bool dot1) {
    if (!dot1) {
        float r = 0.f;
        uint32_t b = 0;
        for (; b + 8 <= nblk; b += 8) {          // eight LDS reads in flight, then the dependent adds
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = p[b + i];
#pragma unroll
            for (int i = 0; i < 8; i++) r = r + v[i];
        }
        for (; b < nblk; b++) r = r + p[b];
        return r;
    }
    float fa0 = 0.f, fa1 = 0.f, fa2 = 0.f, fa3 = 0.f;
    const uint32_t groups = nblk / 4;
    for (uint32_t g = 0; g < groups; g++) {
        fa0 = fa0 + p[4 * g]; fa1 = fa1 + p[4 * g + 1]; fa2 = fa2 + p[4 * g + 2]; fa3 = fa3 + p[4 * g + 3];
    }
    const uint32_t tail = groups * 4;
    if (tail < nblk) fa0 = fa0 + p[tail];
    if (tail + 1 < nblk) fa1 = fa1 + p[tail + 1];
    if (tail + 2 < nblk) fa2 = fa2 + p[tail + 2];
    return ((fa0 + fa1) + fa2) + fa3;
}

__device__ __forceinline__ bool row_is_dot1(uint32_t row, const GemvArgs& a) {
    const uint32_t base = a.chunk ? (row / a.chunk) * a.chunk : 0;
    const uint32_t len = a.chunk ? min(a.chunk, a.N - base) : a.N;
    return (row - base) >= len - (len % a.tail_mod);
}

// Q4 = false: Q8_0 planes; Q4 = true: Q4_0 planes.  ISUMS: write the int32 block sums instead of y.
template <bool Q4, int NCH, int RW, bool ISUMS>
__global__ __launch_bounds__(256) void gemv_kernel(GemvArgs a) {
    extern __shared__ float lds[];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t K = a.K, N = a.N, nblk = K / 32;
    const uint32_t pstride = nblk + 1;                       // +1: conflict-free column reads
    float* prod = lds + (size_t)wave * a.rc * pstride;

    // ---- activation fragment, resident for the whole kernel
    int4 av[NCH], av2[Q4 ? NCH : 1];
    int asum8[Q4 ? NCH : 1];
    float asf[NCH];
    uint32_t blk[NCH];
    bool own[NCH];                                           // this lane reports block blk[j]
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        if (Q4) {
            const uint32_t b = j * 64 + lane;
            blk[j] = b; own[j] = b < nblk;
            if (own[j]) {
                av[j] = *reinterpret_cast<const int4*>(a.aq + (size_t)b * 32);
                av2[j] = *reinterpret_cast<const int4*>(a.aq + (size_t)b * 32 + 16);
                const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
                asum8[j] = 8 * dot16(ones, av2[j], dot16(ones, av[j], 0));
            } else {
                av[j] = av2[j] = make_int4(0, 0, 0, 0); asum8[j] = 0;
            }
        } else {
            const uint32_t off = j * 1024 + lane * 16;
            blk[j] = off / 32; own[j] = off < K && !(lane & 1);
            av[j] = off < K ? *reinterpret_cast<const int4*>(a.aq + off) : make_int4(0, 0, 0, 0);
        }
        asf[j] = (!ISUMS && blk[j] < nblk) ? f16_bits_to_f32(a.as[blk[j]]) : 0.f;
    }

    const uint32_t ngroups = (N + a.rc - 1) / a.rc;
    for (uint32_t g0 = blockIdx.x * 4; g0 < ngroups; g0 += gridDim.x * 4) {
        const uint32_t g = g0 + wave;                         // may be >= ngroups: idle but keeps the barriers uniform
        const uint32_t row_base = g * a.rc;
        if (g < ngroups) {
            for (uint32_t sub = 0; sub < a.rc; sub += RW) {
                if (row_base + sub >= N) break;
                int4 wv[RW][NCH];
                uint16_t wsb[RW][NCH];
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    const uint32_t row = min(row_base + sub + r, N - 1);
#pragma unroll
                    for (int j = 0; j < NCH; j++) {
                        if (Q4) {
                            if (blk[j] < nblk) {
                                wv[r][j] = *reinterpret_cast<const int4*>(a.qs + ((size_t)row * nblk + blk[j]) * 16);
                                wsb[r][j] = a.ws[(size_t)row * nblk + blk[j]];
                            } else { wv[r][j] = make_int4(0, 0, 0, 0); wsb[r][j] = 0; }
                        } else {
                            const uint32_t off = j * 1024 + lane * 16;
                            if (off < K) {
                                wv[r][j] = *reinterpret_cast<const int4*>(a.qs + (size_t)row * K + off);
                                wsb[r][j] = a.ws[(size_t)row * nblk + blk[j]];
                            } else { wv[r][j] = make_int4(0, 0, 0, 0); wsb[r][j] = 0; }
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    const uint32_t row = row_base + sub + r;
#pragma unroll
                    for (int j = 0; j < NCH; j++) {
                        int isum;
                        if (Q4) {
                            const int4 w = wv[r][j];
                            const int m = 0x0F0F0F0F;
                            const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                            const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                            isum = dot16(hi, av2[j], dot16(lo, av[j], 0)) - asum8[j];
                        } else {
                            const int half = dot16(wv[r][j], av[j], 0);
                            isum = half + __shfl_xor(half, 1, WAVE);
                        }
                        if (own[j] && row < N) {
                            if (ISUMS) a.isums[(size_t)row * nblk + blk[j]] = isum;
                            else prod[(sub + r) * pstride + blk[j]] = (asf[j] * f16_bits_to_f32(wsb[r][j])) * (float)isum;
                        }
                    }
                }
            }
        }
        if (!ISUMS) {
            __syncthreads();
            const uint32_t row = row_base + lane;
            if (g < ngroups && lane < a.rc && row < N) {
                const float r = ordered_sum(prod + lane * pstride, nblk, row_is_dot1(row, a));
                a.y[row] = a.accumulate ? a.y[row] + r : r;
            }
            // no second barrier: the product area is private to the wave and LDS operations of
            // one wave execute in order
        }
    }
}

namespace {

// Rows per ordered-sum group.  One lane per row walks the block products in order, so a group costs
// about the same time whatever its size: large groups amortise it (lm_head), small groups keep every
// CU busy on the small matrices.  Bounded above by the LDS the products need.
uint32_t rows_per_group(uint32_t nblk, uint32_t N, uint32_t rw) {
    uint32_t cap = nblk <= 32 ? 64 : nblk <= 64 ? 32 : nblk <= 128 ? 16 : nblk <= 256 ? 8 : 4;
    uint32_t want = N / 4096 / rw * rw;          // aim for >= 4096 groups, i.e. >= 4 waves per SIMD
    if (want < rw) want = rw;
    return want < cap ? want : cap;
}

template <bool Q4, int NCH, int RW, bool ISUMS>
void launch_one(GemvArgs a, hipStream_t s) {
    const uint32_t nblk = a.K / 32;
    a.rc = rows_per_group(nblk, a.N, RW);
    const uint32_t ngroups = (a.N + a.rc - 1) / a.rc;
    uint32_t grid = (ngroups + 3) / 4;
    if (grid > 256 * 8) grid = 256 * 8;
    const size_t lds = ISUMS ? 0 : (size_t)4 * a.rc * (nblk + 1) * sizeof(float);
    gemv_kernel<Q4, NCH, RW, ISUMS><<<grid, 256, lds, s>>>(a);
}

template <bool ISUMS>
void dispatch(const QWeight& w, GemvArgs a, hipStream_t s) {
    if (w.wdtype == FORGE_HIP_Q8_0) {
        const uint32_t nch = (w.K + 1023) / 1024;
        switch (nch) {
            case 1: launch_one<false, 1, 4, ISUMS>(a, s); break;
            case 2: launch_one<false, 2, 4, ISUMS>(a, s); break;
            case 3: launch_one<false, 3, 2, ISUMS>(a, s); break;
            case 4: launch_one<false, 4, 2, ISUMS>(a, s); break;
            case 5: case 6: launch_one<false, 6, 2, ISUMS>(a, s); break;
            case 7: case 8: launch_one<false, 8, 1, ISUMS>(a, s); break;
            default: launch_one<false, 16, 1, ISUMS>(a, s); break;
        }
    } else {
        const uint32_t nch = (w.K + 2047) / 2048;
        switch (nch) {
            case 1: launch_one<true, 1, 4, ISUMS>(a, s); break;
            case 2: launch_one<true, 2, 4, ISUMS>(a, s); break;
            case 3: case 4: launch_one<true, 4, 2, ISUMS>(a, s); break;
            default: launch_one<true, 8, 1, ISUMS>(a, s); break;
        }
    }
}

}  // namespace

// Largest K the register-resident activation fragment covers.
bool gemv_k_supported(uint32_t K) { return K % 32 == 0 && K >= 32 && K <= 16384; }

void launch_gemv(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, GemvOrder order,
                 hipStream_t s) {
    GemvArgs a{};
    a.qs = w.qs; a.ws = w.scales; a.aq = aq; a.as = as; a.y = y; a.isums = nullptr; a.K = w.K; a.N = w.N;
    a.accumulate = accumulate ? 1 : 0;
    // matmul_vec: chunks of 256 rows once the matrix reaches 1 MB of GGUF bytes (emit.rs:1937,1971);
    // the lm_head GEMV always chunks, with an 8-row tail rule after batched prefill (emit.rs:5455-5470).
    const size_t raw_bytes = (size_t)w.N * (w.K / 32) * (w.wdtype == FORGE_HIP_Q8_0 ? 34 : 18);
    a.chunk = (order != GemvOrder::MatmulVec || raw_bytes >= 1000000) ? 256 : 0;
    a.tail_mod = order == GemvOrder::LmHeadAfterPrefill ? 8 : 4;
    dispatch<false>(w, a, s);
}

void launch_gemv_isums(const QWeight& w, const int8_t* aq, int32_t* out, hipStream_t s) {
    GemvArgs a{};
    a.qs = w.qs; a.ws = w.scales; a.aq = aq; a.as = nullptr; a.y = nullptr; a.isums = out; a.K = w.K; a.N = w.N;
    a.tail_mod = 4;
    dispatch<true>(w, a, s);
}

}  // namespace fh

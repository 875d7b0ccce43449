// Decode-time quantised GEMV (matmul_vec_q8_0_KxN / matmul_vec_q4_0_KxN, emit.rs:1926-2092,
// 2797-2958): y[n] = sum_b (a_s[b]*w_s[n][b]) * f32(isum_b), isum_b the exact int32 dot of
// the 32 int8 activation codes of block b with the 32 weight codes.
//
// HBM-bound: every weight byte is read once, with 16-byte loads that are contiguous
// across the wave; the int8 products run on v_dot4, no MFMA.  A wave owns RW consecutive
// rows at a time and keeps the quantised activation vector in registers for all of them
// (on matrices of few rows: its share of the vector, K being dealt to KS waves per row group).
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
//
// A kernel boundary costs several microseconds on this GPU, more than streaming a small
// matrix, so the decode step's neighbours are fused in:
//   prologue  RmsNorm: rms_norm (emit.rs:327-334, the 16-lane FMA order of emit.rs:272-295) and the
//             activation quantiser (emit.rs:1410-1440), recomputed by every workgroup from x, once per
//             workgroup: codes and scales go to LDS, every wave reads its fragment from there
//   epilogue  Add: residual_add (emit.rs:455-459);  RopeKv: rope (emit.rs:508-528) on the q and k
//             rows and the fp16 KV-cache write;  SiluQuant: silu_mul (emit.rs:380-386) of the gate
//             and up rows of a fused [gate;up] matrix and the quantisation of the result.
#include "common.h"
#include "device_utils.h"
#include "expf_ref.h"
#include "gemv_order.h"

namespace fh {

__device__ __forceinline__ int dot16(int4 w, int4 a, int acc) {
    acc = __builtin_amdgcn_sdot4(w.x, a.x, acc, false);
    acc = __builtin_amdgcn_sdot4(w.y, a.y, acc, false);
    acc = __builtin_amdgcn_sdot4(w.z, a.z, acc, false);
    acc = __builtin_amdgcn_sdot4(w.w, a.w, acc, false);
    return acc;
}

enum class Pro { Quant, RmsNorm };
enum class Epi { Store, Add, RopeKv, SiluQuant, Isums };


struct GemvArgs {
    const uint8_t* qs;
    const uint16_t* ws;
    uint32_t K, N;
    uint32_t rc;             // rows per ordered-sum group (per wave)
    Segment seg[3];          // row ranges of the reference matmuls (tail rule applies per matmul)
    uint32_t nseg, tail_mod;
    // Pro::Quant
    const int8_t* aq;
    const uint16_t* as;
    // Pro::RmsNorm
    const float* x;
    const float* norm_w;
    float eps;
    // Epi::Store / Add / Isums
    float* y;
    int32_t* isums;
    // Epi::RopeKv: rows [0,QKS) -> q_out f32 (rotated); [QKS,QKS+KV) -> kc (rotated, fp16); rest -> vc (fp16)
    float* q_out;
    uint16_t* kc;
    uint16_t* vc;
    const float* cos_t;
    const float* sin_t;
    const uint32_t* pos_dev;
    PageTable pt;            // where position *pos_dev lives in a paged cache
    const float* bias;       // optional: q | k | v bias, added before the rotation (Qwen2, emit.rs:4105-4120)
    uint32_t qks, kv, hd;
    // Epi::SiluQuant: rows [0,I) gate, [I,2I) up -> oq int8 [I], osc fp16 [I/32]
    int8_t* oq;
    uint16_t* osc;
    uint32_t inter;
};

__device__ __forceinline__ bool row_is_dot1(uint32_t row, const GemvArgs& a) {
    return segment_row_is_dot1(row, a.seg, a.nseg, a.tail_mod);
}

// KS > 1: a group's rows are worked by KS waves, each taking every KS-th chunk of K (its share of the activation
// fragment, of the loads to issue and of the products) — a wave that is alone on its SIMD issues an instruction only
// every few nanoseconds, so on the small matrices, where there is one workgroup per CU, what a wave has to issue is
// what the kernel takes.  The products meet in LDS as before and the first of the KS waves adds them in order.
template <bool Q4, int NCH, int RW, int WAVES, int KS, Pro PRO, Epi EPI>
__global__ __launch_bounds__(WAVES * 64) void gemv_kernel(GemvArgs a) {
    static_assert(NCH % KS == 0 && WAVES % KS == 0, "K split must divide the chunks and the waves");
    static_assert(KS == 1 || (EPI != Epi::SiluQuant && EPI != Epi::Isums), "no K split in these variants");
    extern __shared__ __align__(16) float lds[];
    constexpr uint32_t THREADS = WAVES * 64;
    constexpr int NL = NCH / KS;                             // chunks per wave
    constexpr uint32_t RWAVES = WAVES / KS;                  // row groups per workgroup
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t kpart = KS == 1 ? 0u : wave % KS, rwave = KS == 1 ? wave : wave / KS;
    const uint32_t K = a.K, N = a.N, nblk = K / 32;
    const uint32_t pstride = prod_stride(nblk);
    float* prod = lds + (size_t)rwave * a.rc * pstride;
    float* shared_tail = lds + (size_t)RWAVES * a.rc * pstride;   // prologue / epilogue scratch
    auto chunk = [&](int j) -> uint32_t { return (uint32_t)j * KS + kpart; };   // this wave's j-th chunk of K

    uint32_t blk[NL];
    bool own[NL];                                            // this lane reports block blk[j]
#pragma unroll
    for (int j = 0; j < NL; j++) {
        if (Q4) { blk[j] = chunk(j) * 64 + lane; own[j] = blk[j] < nblk; }
        else { const uint32_t off = chunk(j) * 1024 + lane * 16; blk[j] = off / 32; own[j] = off < K && !(lane & 1); }
    }

    // ---- row groups.  Standard: wave w of workgroup-group g0 owns rows [(g0+w) rc, +rc).
    //      SiluQuant (WAVES = 16, rc = 4): workgroup G owns inter indices [32 G, +32): waves 0..7 take the
    //      gate rows, waves 8..15 the up rows, four rows each.
    const uint32_t ngroups = EPI == Epi::SiluQuant ? (a.inter + 31) / 32 : (N + a.rc - 1) / a.rc;
    const uint32_t gstep = EPI == Epi::SiluQuant ? 1 : RWAVES;
    auto rows_of = [&](uint32_t g0, uint32_t& row_base, uint32_t& row_end) -> bool {
        if (EPI == Epi::SiluQuant) {
            const uint32_t i0 = g0 * 32 + (wave & 7) * 4;
            row_base = (wave >> 3) * a.inter + i0;
            row_end = (wave >> 3) * a.inter + min(a.inter, i0 + 4);
            return i0 < a.inter;
        }
        const uint32_t g = g0 + rwave;                       // may be >= ngroups: idle but keeps the barriers uniform
        row_base = g * a.rc;
        row_end = min(N, row_base + a.rc);
        return g < ngroups;
    };

    int4 wv[RW][NL];
    uint16_t wsb[RW][NL];
    auto load_rows = [&](uint32_t row0, uint32_t row_end) {
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t row = min(row0 + r, row_end - 1);
#pragma unroll
            for (int j = 0; j < NL; j++) {
                if (Q4) {
                    if (blk[j] < nblk) {
                        wv[r][j] = *reinterpret_cast<const int4*>(a.qs + ((size_t)row * nblk + blk[j]) * 16);
                        wsb[r][j] = a.ws[(size_t)row * nblk + blk[j]];
                    } else { wv[r][j] = make_int4(0, 0, 0, 0); wsb[r][j] = 0; }
                } else {
                    const uint32_t off = chunk(j) * 1024 + lane * 16;
                    if (off < K) {
                        wv[r][j] = *reinterpret_cast<const int4*>(a.qs + (size_t)row * K + off);
                        wsb[r][j] = a.ws[(size_t)row * nblk + blk[j]];
                    } else { wv[r][j] = make_int4(0, 0, 0, 0); wsb[r][j] = 0; }
                }
            }
        }
    };

    // Pro::RmsNorm: x and the norm weights are requested first (the first XE float4 per thread; what lies beyond is
    // fetched later, behind the weights): loads return in issue order, so behind the weights they would arrive only after them, and the
    // norm would wait for the weights instead of running while they travel.
    constexpr int XE = THREADS >= 1024 ? 1 : THREADS >= 512 ? 2 : 4;   // 4096 elements, at 16 waves within their 128 registers
    float4 xe[PRO == Pro::RmsNorm ? XE : 1], we[PRO == Pro::RmsNorm ? XE : 1];
    if (PRO == Pro::RmsNorm) {
#pragma unroll
        for (int i = 0; i < XE; i++) {
            const uint32_t e4 = i * THREADS + tid;
            xe[i] = we[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e4 < K / 4) { xe[i] = reinterpret_cast<const float4*>(a.x)[e4]; we[i] = reinterpret_cast<const float4*>(a.norm_w)[e4]; }
        }
    }

    // Weights do not depend on the activations: start streaming the first rows before the prologue.
    // The order in which this lane will add its row's products (lane i of a wave adds row i of the wave's group) is
    // worked out here as well, for the first group: a lone wave on a SIMD issues an instruction every few nanoseconds,
    // and these hundred-odd cost nothing while the loads are in flight.  Pinned, or the compiler moves them down in
    // front of their use behind the products barrier.
    bool prefetched = false;
    uint32_t d1_first = 0;
    {
        uint32_t rb, re;
        const uint32_t g0 = blockIdx.x * gstep;
        if (g0 < ngroups && rows_of(g0, rb, re) && rb < re) {
            load_rows(rb, re); prefetched = true;
            if (EPI != Epi::Isums && kpart == 0 && lane < a.rc && rb + lane < re) d1_first = row_is_dot1(rb + lane, a);
        }
        asm volatile("" : "+v"(d1_first));
    }
    bool first_group = true;

    // ---- activation fragment, resident for the whole kernel
    int4 av[NL], av2[Q4 ? NL : 1];
    int asum8[Q4 ? NL : 1];
    float asf[NL];
    if (PRO == Pro::RmsNorm) {
        // rms_norm of x[K] in the reference's summation order, then block quantisation, once per workgroup: 8 lanes
        // share a block of 32, codes and scales go to LDS and every wave picks its fragment up from there
        float* xs = shared_tail;                              // K floats
        float* part = xs + K;                                 // 17 (32 reserved)
        float* qsc = part + 32;                               // K/32 scales, as the f32 value of their fp16 rounding
        uint32_t* qcd = reinterpret_cast<uint32_t*>(qsc + ((nblk + 3u) & ~3u));   // K codes, 16-byte aligned
#pragma unroll
        for (int i = 0; i < XE; i++) { const uint32_t e4 = i * THREADS + tid; if (e4 < K / 4) reinterpret_cast<float4*>(xs)[e4] = xe[i]; }
        for (uint32_t e4 = XE * THREADS + tid; e4 < K / 4; e4 += THREADS) reinterpret_cast<float4*>(xs)[e4] = reinterpret_cast<const float4*>(a.x)[e4];
        __syncthreads();
        if (tid < 16) {
            float s = 0.f;
            const uint32_t chunks = K / 16;
            uint32_t c = 0;
            for (; c + 8 <= chunks; c += 8) {
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
            for (uint32_t i = K / 16 * 16; i < K; i++) r = r + xs[i] * xs[i];
            part[16] = r;
        }
        __syncthreads();
        const float inv_rms = 1.0f / sqrtf(part[16] / (float)K + a.eps);
        auto quantise4 = [&](uint32_t e4, float4 xv, float4 w4) {
            const float4 v = make_float4(xv.x * inv_rms * w4.x, xv.y * inv_rms * w4.y, xv.z * inv_rms * w4.z, xv.w * inv_rms * w4.w);
            uint16_t sb;
            qcd[e4] = quantize_block_part(v, sb);
            if ((e4 & 7u) == 0) qsc[e4 >> 3] = f16_bits_to_f32(sb);
        };
        // (K / 4 is a multiple of 8 and so is THREADS: the 8 lanes of a block are in or out together)
#pragma unroll
        for (int i = 0; i < XE; i++) { const uint32_t e4 = i * THREADS + tid; if (e4 < K / 4) quantise4(e4, reinterpret_cast<const float4*>(xs)[e4], we[i]); }
        for (uint32_t e4 = XE * THREADS + tid; e4 < K / 4; e4 += THREADS) quantise4(e4, reinterpret_cast<const float4*>(xs)[e4], reinterpret_cast<const float4*>(a.norm_w)[e4]);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NL; j++) {
            const uint8_t* codes = reinterpret_cast<const uint8_t*>(qcd);
            if (Q4) {
                av[j] = av2[j] = make_int4(0, 0, 0, 0);
                if (own[j]) { av[j] = *reinterpret_cast<const int4*>(codes + (size_t)blk[j] * 32); av2[j] = *reinterpret_cast<const int4*>(codes + (size_t)blk[j] * 32 + 16); }
            } else {
                const uint32_t off = chunk(j) * 1024 + lane * 16;
                av[j] = off < K ? *reinterpret_cast<const int4*>(codes + off) : make_int4(0, 0, 0, 0);
            }
            asf[j] = blk[j] < nblk ? qsc[blk[j]] : 0.f;
        }
        // (the SiluQuant epilogue reuses the first words of the tail: x, which nobody reads after the barrier above)
    } else {
#pragma unroll
        for (int j = 0; j < NL; j++) {
            if (Q4) {
                if (own[j]) {
                    av[j] = *reinterpret_cast<const int4*>(a.aq + (size_t)blk[j] * 32);
                    av2[j] = *reinterpret_cast<const int4*>(a.aq + (size_t)blk[j] * 32 + 16);
                } else { av[j] = av2[j] = make_int4(0, 0, 0, 0); }
            } else {
                const uint32_t off = chunk(j) * 1024 + lane * 16;
                av[j] = off < K ? *reinterpret_cast<const int4*>(a.aq + off) : make_int4(0, 0, 0, 0);
            }
            asf[j] = (EPI != Epi::Isums && blk[j] < nblk) ? f16_bits_to_f32(a.as[blk[j]]) : 0.f;
        }
    }
    if (Q4) {
        const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
#pragma unroll
        for (int j = 0; j < NL; j++) asum8[j] = 8 * dot16(ones, av2[j], dot16(ones, av[j], 0));
    }

    for (uint32_t g0 = blockIdx.x * gstep; g0 < ngroups; g0 += gridDim.x * gstep) {
        uint32_t row_base, row_end;   // this wave's rows [row_base, row_end)
        // the row distance is read afresh in every pass: otherwise the LDS address of every (row, chunk) product is
        // worked out ahead of the loop and kept, which at 16 waves per workgroup (128 registers) ends in spills that
        // are reloaded, one memory round trip each, between the products
        uint32_t ps = pstride;
        asm volatile("" : "+s"(ps));
        const bool wave_on = rows_of(g0, row_base, row_end);
        uint32_t d1 = d1_first;
        if (!first_group) {
            d1 = (EPI != Epi::Isums && wave_on && kpart == 0 && lane < a.rc && row_base + lane < row_end) ? row_is_dot1(row_base + lane, a) : 0u;
            asm volatile("" : "+v"(d1));
        }
        first_group = false;
        if (wave_on) {
            for (uint32_t sub = 0; sub < a.rc; sub += RW) {
                if (row_base + sub >= row_end) break;
                if (!prefetched) load_rows(row_base + sub, row_end);
                prefetched = false;
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    const uint32_t row = row_base + sub + r;
#pragma unroll
                    for (int j = 0; j < NL; j++) {
                        int isum;
                        if (Q4) {
                            const int4 w = wv[r][j];
                            const int m = 0x0F0F0F0F;
                            const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                            const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                            isum = dot16(hi, av2[j], dot16(lo, av[j], 0)) - asum8[j];
                        } else {
                            const int half = dot16(wv[r][j], av[j], 0);
                            isum = half + lane_xor<1>(half);
                        }
                        if (own[j] && row < row_end) {
                            if (EPI == Epi::Isums) a.isums[(size_t)row * nblk + blk[j]] = isum;
                            else prod[(sub + r) * ps + blk[j]] = (asf[j] * f16_bits_to_f32(wsb[r][j])) * (float)isum;
                        }
                    }
                }
            }
        }
        prefetched = false;
        if (EPI == Epi::Isums) continue;
        __syncthreads();
        // ---- ordered sums: lane i of the group's (first) wave owns row row_base + i
        const uint32_t row = row_base + lane;
        const bool active = wave_on && kpart == 0 && lane < a.rc && row < row_end;
        float r = 0.f;
        if (active) r = ordered_sum(prod + lane * ps, nblk, d1 != 0);
        if (EPI == Epi::Store) {
            if (active) a.y[row] = r;
        } else if (EPI == Epi::Add) {
            if (active) a.y[row] = a.y[row] + r;
        } else if (EPI == Epi::RopeKv) {
            // rows 2i, 2i+1 of a head sit in lanes 2i, 2i+1 (row_base and rc are even)
            if (a.bias && active) r = r + a.bias[row];
            const float other = lane_xor<1>(r);
            if (active) {
                const uint32_t pos = *a.pos_dev;
                if (row < a.qks + a.kv) {
                    const uint32_t d = row < a.qks ? row % a.hd : (row - a.qks) % a.hd;
                    const float c = a.cos_t[(size_t)pos * (a.hd / 2) + d / 2], s = a.sin_t[(size_t)pos * (a.hd / 2) + d / 2];
                    const float o = (row & 1) ? other * s + r * c : r * c - other * s;
                    if (row < a.qks) a.q_out[row] = o;
                    else a.kc[paged_row(a.pt, pos) * a.kv + (row - a.qks)] = f32_to_f16_bits(o);
                } else {
                    a.vc[paged_row(a.pt, pos) * a.kv + (row - a.qks - a.kv)] = f32_to_f16_bits(r);
                }
            }
        } else if (EPI == Epi::SiluQuant) {
            float* res = shared_tail;                         // [64]: gate 0..31, up 32..63
            if (active) res[(wave >> 3) * 32 + (wave & 7) * 4 + lane] = r;
            __syncthreads();
            if (tid < 32) {
                const uint32_t i = g0 * 32 + tid;
                const bool in = i < a.inter;
                const float gx = in ? res[tid] : 0.f, ux = in ? res[32 + tid] : 0.f;
                const float o = in ? (gx / (1.0f + expf_ref<true>(-gx))) * ux : 0.f;
                const float amax = half_wave_max(fabsf(o));
                float inv;
                const float sc = act_scale(amax, inv);
                if (in) {
                    a.oq[i] = (int8_t)quant_code(o * inv);
                    if (tid == 0) a.osc[i / 32] = f32_to_f16_bits(sc);
                }
            }
            // the next iteration's first barrier orders these reads before res[] is rewritten
        }
        // KS = 1: the product area is private to the wave and LDS operations of one wave execute in order, so no
        // barrier is needed before the next group overwrites it; shared between waves it is
        if (KS > 1) __syncthreads();
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
    want &= ~1u;                                 // rope pairs need both rows of a pair in one group
    if (want < 2) want = 2;
    return want < cap ? want : cap;
}

constexpr size_t LDS_LIMIT = 64 * 1024;
size_t lds_tail_bytes(bool norm, bool silu, uint32_t K) {
    // the norm prologue: x [K] f32, 32 words of partial sums, the scales [K/32] f32 (padded to 16 bytes), the codes [K]
    size_t tail = norm ? (size_t)(K + 32 + ((K / 32 + 3) & ~3u)) * sizeof(float) + K : 0;
    if (silu && tail < 64 * sizeof(float)) tail = 64 * sizeof(float);
    return tail;
}

template <bool Q4, int NCH, int RW, Pro PRO, Epi EPI, int KS = 1>
void launch_one(GemvArgs a, hipStream_t s) {
    constexpr int WAVES = EPI == Epi::SiluQuant ? 16 : 4;      // waves that own row groups; the kernel runs WAVES * KS
    const uint32_t nblk = a.K / 32;
    const size_t tail = lds_tail_bytes(PRO == Pro::RmsNorm, EPI == Epi::SiluQuant, a.K);
    a.rc = EPI == Epi::SiluQuant ? 4 : rows_per_group(nblk, a.N, RW);
    // shrink the group if the products and the prologue's copy of x do not fit LDS together
    constexpr uint32_t step = RW < 2 ? 2 : RW;
    while (EPI != Epi::SiluQuant && a.rc > step && (size_t)WAVES * a.rc * prod_stride(nblk) * sizeof(float) + tail > LDS_LIMIT) a.rc -= step;
    const uint32_t ngroups = EPI == Epi::SiluQuant ? (a.inter + 31) / 32 : ((a.N + a.rc - 1) / a.rc + WAVES - 1) / WAVES;
    uint32_t grid = ngroups;
    if (grid > 256 * 8) grid = 256 * 8;
    const size_t lds = EPI == Epi::Isums ? 0 : (size_t)WAVES * a.rc * prod_stride(nblk) * sizeof(float);
    fh::launch(gemv_kernel<Q4, NCH, (EPI == Epi::SiluQuant ? (RW > 4 ? 4 : RW) : RW), WAVES * KS, KS, PRO, EPI>, grid, WAVES * KS * 64, lds + tail, s, a);
}

template <Pro PRO, Epi EPI>
void dispatch(uint32_t wdtype, const GemvArgs& a, hipStream_t s) {
    // SiluQuant walks 16 rows per wave; RW must divide 16 (it always does).
    // Matrices of few rows (everything but an lm_head) leave a CU with a handful of waves: there K is dealt to KS waves
    // per row group, the largest KS on offer that keeps the launch within 16 waves per CU.
    constexpr bool CAN_SPLIT = EPI != Epi::SiluQuant && EPI != Epi::Isums;
    auto fits = [&](int rw, int ks) {
        const uint32_t rc = rows_per_group(a.K / 32, a.N, rw);
        return (uint64_t)((a.N + rc - 1) / rc) * ks <= 256u * 16u;
    };
#define FH_GEMV_ONE(Q4_, NCH_, RW_, KSA_, KSB_)                                                   \
    do {                                                                                          \
        if constexpr (CAN_SPLIT && KSA_ > 1) {                                                    \
            if (fits(RW_, KSA_)) { launch_one<Q4_, NCH_, RW_, PRO, EPI, KSA_>(a, s); break; }     \
        }                                                                                         \
        if constexpr (CAN_SPLIT && KSB_ > 1) {                                                    \
            if (fits(RW_, KSB_)) { launch_one<Q4_, NCH_, RW_, PRO, EPI, KSB_>(a, s); break; }     \
        }                                                                                         \
        launch_one<Q4_, NCH_, RW_, PRO, EPI>(a, s);                                               \
    } while (0)
    if (wdtype == FORGE_HIP_Q8_0) {
        const uint32_t nch = (a.K + 1023) / 1024;
        switch (nch) {
            case 1: FH_GEMV_ONE(false, 1, 4, 1, 1); break;
            case 2: FH_GEMV_ONE(false, 2, 4, 2, 1); break;
            case 3: FH_GEMV_ONE(false, 3, 2, 1, 1); break;
            case 4: FH_GEMV_ONE(false, 4, 2, 4, 2); break;
            case 5: case 6: FH_GEMV_ONE(false, 6, 2, 2, 1); break;
            case 7: case 8: FH_GEMV_ONE(false, 8, 2, 4, 2); break;
            default: FH_GEMV_ONE(false, 16, 1, 4, 2); break;
        }
    } else {
        const uint32_t nch = (a.K + 2047) / 2048;
        switch (nch) {
            case 1: FH_GEMV_ONE(true, 1, 4, 1, 1); break;
            case 2: FH_GEMV_ONE(true, 2, 4, 2, 1); break;
            case 3: case 4: FH_GEMV_ONE(true, 4, 2, 4, 2); break;
            default: FH_GEMV_ONE(true, 8, 1, 4, 2); break;
        }
    }
#undef FH_GEMV_ONE
}

GemvArgs base_args(const QWeight& w, GemvOrder order) {
    GemvArgs a{};
    a.qs = w.qs; a.ws = w.scales; a.K = w.K; a.N = w.N;
    a.nseg = 1; a.seg[0] = make_segment(w.wdtype, w.K, 0, w.N, order != GemvOrder::MatmulVec);
    a.tail_mod = order == GemvOrder::LmHeadAfterPrefill ? 8 : 4;
    return a;
}

}  // namespace

// Largest K the register-resident activation fragment covers.
bool gemv_k_supported(uint32_t K) { return K % 32 == 0 && K >= 32 && K <= 16384; }

// Whether the fused prologue / epilogue variants fit LDS for this K (else the caller launches the
// separate kernels).
bool gemv_norm_fusable(uint32_t K) {
    return gemv_k_supported(K) && (size_t)4 * 4 * prod_stride(K / 32) * sizeof(float) + lds_tail_bytes(true, false, K) <= LDS_LIMIT;
}
bool gemv_silu_fusable(uint32_t K) {
    return gemv_k_supported(K) && (size_t)16 * 4 * prod_stride(K / 32) * sizeof(float) + lds_tail_bytes(true, true, K) <= LDS_LIMIT;
}

void launch_gemv(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, GemvOrder order,
                 hipStream_t s) {
    GemvArgs a = base_args(w, order);
    a.aq = aq; a.as = as; a.y = y;
    if (accumulate) dispatch<Pro::Quant, Epi::Add>(w.wdtype, a, s);
    else dispatch<Pro::Quant, Epi::Store>(w.wdtype, a, s);
}

void launch_gemv_isums(const QWeight& w, const int8_t* aq, int32_t* out, hipStream_t s) {
    GemvArgs a = base_args(w, GemvOrder::MatmulVec);
    a.aq = aq; a.isums = out;
    dispatch<Pro::Quant, Epi::Isums>(w.wdtype, a, s);
}

void launch_gemv_norm(const QWeight& w, const float* x, const float* norm_w, float eps, float* y, GemvOrder order,
                      hipStream_t s) {
    GemvArgs a = base_args(w, order);
    a.x = x; a.norm_w = norm_w; a.eps = eps; a.y = y;
    dispatch<Pro::RmsNorm, Epi::Store>(w.wdtype, a, s);
}

void launch_gemv_norm_rope_kv(const QWeight& wqkv, const float* x, const float* norm_w, float eps, const float* bias, float* q_out,
                              uint16_t* kc, uint16_t* vc, const float* cos_t, const float* sin_t,
                              const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd, hipStream_t s,
                              PageTable pt) {
    GemvArgs a = base_args(wqkv, GemvOrder::MatmulVec);
    a.x = x; a.norm_w = norm_w; a.eps = eps;
    a.q_out = q_out; a.kc = kc; a.vc = vc; a.cos_t = cos_t; a.sin_t = sin_t; a.pos_dev = pos_dev;
    a.pt = pt;
    a.bias = bias;
    a.qks = heads * hd; a.kv = kv_heads * hd; a.hd = hd;
    a.nseg = 3;
    a.seg[0] = make_segment(wqkv.wdtype, wqkv.K, 0, a.qks, false);
    a.seg[1] = make_segment(wqkv.wdtype, wqkv.K, a.qks, a.kv, false);
    a.seg[2] = make_segment(wqkv.wdtype, wqkv.K, a.qks + a.kv, a.kv, false);
    dispatch<Pro::RmsNorm, Epi::RopeKv>(wqkv.wdtype, a, s);
}

void launch_gemv_norm_silu_quant(const QWeight& wgu, const float* x, const float* norm_w, float eps, int8_t* oq,
                                 uint16_t* osc, hipStream_t s) {
    GemvArgs a = base_args(wgu, GemvOrder::MatmulVec);
    a.x = x; a.norm_w = norm_w; a.eps = eps; a.oq = oq; a.osc = osc; a.inter = wgu.N / 2;
    a.nseg = 2;
    a.seg[0] = make_segment(wgu.wdtype, wgu.K, 0, a.inter, false);
    a.seg[1] = make_segment(wgu.wdtype, wgu.K, a.inter, a.inter, false);
    dispatch<Pro::RmsNorm, Epi::SiluQuant>(wgu.wdtype, a, s);
}

}  // namespace fh

// One decode token as ONE kernel: model::forward (emit.rs:4029-4227) for a single row, every CU busy
// from the embedding row to the argmax.
//
// Why: a decode step of a 1B model is ~100 small dependent operations, and a kernel boundary costs
// 4-5 us on this GPU -- more than streaming most of the matrices involved.  Here one workgroup per CU
// stays resident for the whole step and the operations become phases of the same kernel:
//
//   P1  rms_norm + quantise | [q;k;v] GEMV | rope, KV-cache write        (emit.rs:327, 1926, 508)
//   P2  attention over the fp16 cache, split along the sequence            (emit.rs:656)
//   P3  merge of the splits, quantise for the O projection
//   P4  O GEMV + residual                                                   (emit.rs:455)
//   P5  rms_norm + quantise | [gate;up] GEMV | silu(gate)*up, quantise     (emit.rs:380)
//   P6  down GEMV + residual
//   ... per layer, then final norm | lm_head GEMV | argmax (project.rs:501) and the position/token advance.
//
// Phases are not separated by grid barriers.  Every value one workgroup hands to another travels as an
// 8-byte element {payload32, tag32}, written with one write-through store and read with loads that
// bypass the per-XCD L2; the tag is the number of the phase instance that produced it (unique per token,
// layer and phase), so a consumer simply re-reads an element until its tag is the one it expects.  One
// memory round trip replaces the arrive/count/release/read chain of a barrier (measured on MI355X:
// ~2 us per all-to-all exchange of a 2048-element vector against 4-5 us through a tree barrier), and
// nothing ever has to invalidate or write back a cache.  A buffer is overwritten only by a phase whose
// inputs transitively depend on every reader of the previous version (each phase's consumers read
// before they produce, and every product is needed downstream), so a stale or too-new tag can only
// mean a stuck grid: polling is bounded, a workgroup that runs out of spins raises the abort flag and
// leaves, and the host reports an error instead of hanging.
//
// Weights do not depend on activations: each phase issues the loads of its first weight units before it
// starts waiting for its inputs, so HBM latency overlaps the hand-over.
//
// The arithmetic is that of the separate kernels (gemv.hip, attn_decode.hip, elementwise.hip), value for
// value: the same block products, the same ordered sums, the same split boundaries and merge order.
#include <algorithm>
#include <memory>
#include <vector>

#include "common.h"
#include "device_utils.h"
#include "expf_ref.h"
#include "gemv_order.h"

namespace fh {

namespace {

constexpr int PD_THREADS = 1024;
constexpr int PD_WAVES = PD_THREADS / 64;
constexpr int PD_D = 8;                       // weight units (1 KB) a wave holds in registers per round
constexpr uint32_t PD_MAX_TILE_ROWS = 128;
constexpr uint32_t PD_LDS_BYTES = 64 * 1024;
constexpr uint32_t PD_MISC_BYTES = 2048;

struct PdGemv {
    const uint8_t* qs;
    const uint16_t* ws;
    uint32_t K, N, nblk, U;       // U: weight units per row (Q8_0: 1024 elements, Q4_0: 2048)
    uint32_t T, ntiles;           // rows per tile, tiles (silu tiles: 32 gate rows + the matching 32 up rows)
    uint32_t inter;               // != 0: fused [gate;up] matrix, rows [0,inter) gate, [inter, 2 inter) up
    uint32_t nseg, tail_mod;
    Segment seg[3];
};

struct PdLayer {
    PdGemv qkv, o, gu, down;
    const float* attn_norm;
    const float* ffn_norm;
    uint16_t* kc;
    uint16_t* vc;
};

struct PdArgs {
    const PdLayer* layers;
    PdGemv lm;
    uint32_t n_layers, H, I, QKS, KV, heads, kv_heads, gt;
    float eps;
    const float* embed;
    const float* final_norm;
    const float* cos_t;
    const float* sin_t;
    // tagged exchange buffers
    uint64_t* tx;      // [H]            residual stream
    uint64_t* tq;      // [QKS]          rotated q
    uint64_t* tkv;     // [2 KV]         this position's K row (rotated) and V row, fp16 bits
    uint64_t* tws;     // [heads][DECODE_SPLITS][hd + 2]  split partials
    uint64_t* taq;     // [QKS/4 + QKS/32]  attention output, int8 codes (4 per element) then fp16 scales
    uint64_t* taq2;    // [I/4 + I/32]      silu(gate)*up, same format
    uint64_t* tpart;   // [2 G]          per-workgroup argmax candidates
    float* logits;
    uint32_t* state;   // [0] position  [1] token  [2] next token  [3] abort flag
    uint32_t tag_base, spin_limit;
    uint32_t off_act_s, off_misc, off_big;     // LDS byte offsets (activation codes sit at 0)
    unsigned long long* stamps;                // optional: wall clock at the start of every phase (workgroup 0)
};

// ---- coherent (agent-scope, L2-bypassing) accesses ----------------------------------------------------
__device__ __forceinline__ uint64_t ldc64(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc64(uint64_t* p, uint32_t tag, uint32_t payload) {
    __hip_atomic_store(p, ((uint64_t)tag << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PdCtx {
    uint32_t tid, lane, wave, wg, G;
    uint32_t spin_limit;
    uint32_t* sh_abort;      // LDS
    uint32_t* abort_flag;    // global
};

// Re-read one element until it carries `tag`; bounded.
__device__ __forceinline__ uint32_t poll(const uint64_t* p, uint32_t tag, const PdCtx& cx) {
    uint64_t w = ldc64(p);
    uint32_t spins = 0;
    while ((uint32_t)(w >> 32) != tag) {
        ++spins;
        if (spins > cx.spin_limit ||
            ((spins & 1023u) == 0 && __hip_atomic_load(cx.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
            *cx.sh_abort = 1;
            __hip_atomic_store(cx.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
        w = ldc64(p);
    }
    return (uint32_t)w;
}

// Up to N elements per thread: all loads are issued before any tag is looked at, so a hand-over costs one
// memory round trip however many elements a thread takes; only elements still carrying another tag are re-read.
template <int N, typename Addr>
__device__ __forceinline__ void poll_many(Addr addr, uint32_t n, uint32_t tag, uint32_t* out, const PdCtx& cx) {
    uint64_t w[N];
#pragma unroll
    for (int i = 0; i < N; i++) w[i] = (uint32_t)i < n ? ldc64(addr(i)) : ((uint64_t)tag << 32);
    uint32_t spins = 0;
    for (;;) {
        bool ok = true;
#pragma unroll
        for (int i = 0; i < N; i++) ok = ok && (uint32_t)(w[i] >> 32) == tag;
        if (ok) break;
        ++spins;
        if (spins > cx.spin_limit ||
            ((spins & 1023u) == 0 && __hip_atomic_load(cx.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
            *cx.sh_abort = 1;
            __hip_atomic_store(cx.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        __builtin_amdgcn_s_sleep(2);
#pragma unroll
        for (int i = 0; i < N; i++)
            if ((uint32_t)(w[i] >> 32) != tag) w[i] = ldc64(addr(i));
    }
#pragma unroll
    for (int i = 0; i < N; i++) out[i] = (uint32_t)w[i];
}

// A whole vector of `count` elements, four per thread and pass; `put(index, payload)` stores each.
template <typename Put>
__device__ __forceinline__ void poll_vec(const uint64_t* base, uint32_t count, uint32_t tag, const PdCtx& cx, Put put) {
    for (uint32_t i0 = cx.tid; i0 < count; i0 += 4 * PD_THREADS) {
        uint32_t v[4];
        const uint32_t n = (count - i0 + PD_THREADS - 1) / PD_THREADS;
        poll_many<4>([&](int i) { return base + i0 + (uint32_t)i * PD_THREADS; }, n < 4 ? n : 4, tag, v, cx);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i0 + (uint32_t)i * PD_THREADS < count) put(i0 + (uint32_t)i * PD_THREADS, v[i]);
    }
}

// Thousands of threads re-reading a buffer that is not ready yet would flood the memory fabric the weight
// stream needs.  One lane per workgroup watches a single element first; the full read starts when that
// element has arrived, which in a balanced phase is when the rest is about to.
__device__ __forceinline__ void wait_hint(const uint64_t* sentinel, uint32_t tag, const PdCtx& cx) {
    if (cx.tid == 0) (void)poll(sentinel, tag, cx);
    __syncthreads();
}

__device__ __forceinline__ int dot16(int4 w, int4 a, int acc) {
    acc = __builtin_amdgcn_sdot4(w.x, a.x, acc, false);
    acc = __builtin_amdgcn_sdot4(w.y, a.y, acc, false);
    acc = __builtin_amdgcn_sdot4(w.z, a.z, acc, false);
    acc = __builtin_amdgcn_sdot4(w.w, a.w, acc, false);
    return acc;
}

// ---- prologues: the activation vector of a GEMV phase, quantised, in LDS ------------------------------
// rms_norm (emit.rs:327-334, 16-lane FMA order of emit.rs:272-295) + activation quantiser (emit.rs:1410-1440).
// xs must already hold x[0..H); `part` is 32 floats of LDS.
__device__ __forceinline__ void pd_norm_quant(float* xs, const float* __restrict__ norm_w, float eps, uint32_t H,
                                              uint32_t* aq_lds, float* as_lds, float* part, const PdCtx& cx) {
    const uint32_t tid = cx.tid;
    __syncthreads();
    if (tid < 16) {
        float s = 0.f;
        const uint32_t chunks = H / 16;
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
        for (uint32_t i = H / 16 * 16; i < H; i++) r = r + xs[i] * xs[i];
        part[16] = r;
    }
    __syncthreads();
    const float inv_rms = 1.0f / sqrtf(part[16] / (float)H + eps);
    for (uint32_t e0 = tid * 4; e0 < H; e0 += PD_THREADS * 4) {
        const float4 xv = *reinterpret_cast<const float4*>(xs + e0);
        const float4 wv = *reinterpret_cast<const float4*>(norm_w + e0);
        const float4 v = make_float4(xv.x * inv_rms * wv.x, xv.y * inv_rms * wv.y, xv.z * inv_rms * wv.z, xv.w * inv_rms * wv.w);
        uint16_t sb;
        const uint32_t pk = quantize_block_part(v, sb);
        aq_lds[e0 / 4] = pk;
        if ((tid & 7u) == 0) as_lds[e0 / 32] = f16_bits_to_f32(sb);
    }
    __syncthreads();
}

// An already quantised vector (codes then scales, tagged) from another phase.
__device__ __forceinline__ void pd_load_aq(const uint64_t* t, uint32_t tag, uint32_t K, uint32_t* aq_lds, float* as_lds,
                                           const PdCtx& cx) {
    const uint32_t nq = K / 4, ns = K / 32;
    wait_hint(t + nq + ns - 1, tag, cx);
    poll_vec(t, nq + ns, tag, cx, [&](uint32_t i, uint32_t p) {
        if (i < nq) aq_lds[i] = p;
        else as_lds[i - nq] = f16_bits_to_f32((uint16_t)p);
    });
    __syncthreads();
}

// ---- the GEMV of a phase ------------------------------------------------------------------------------
struct WReg { int4 v[PD_D]; uint32_t s[PD_D]; };

__device__ __forceinline__ uint32_t pd_tile_rows(const PdGemv& g, uint32_t tile) {
    return g.inter ? 64u : min(g.T, g.N - tile * g.T);
}
__device__ __forceinline__ uint32_t pd_tile_row(const PdGemv& g, uint32_t tile, uint32_t lr) {
    if (g.inter) return lr < 32 ? tile * 32 + lr : g.inter + tile * 32 + (lr - 32);
    return tile * g.T + lr;
}

// Unit u of a tile = weight unit (u % U) of tile row (u / U); wave w takes units w, w + 16, ...; a round is
// PD_D units per wave, all loads issued before any is used.
template <bool Q4>
__device__ __forceinline__ void pd_load_round(const PdGemv& g, uint32_t tile, uint32_t round, const PdCtx& cx, WReg& W) {
    const uint32_t units = tile < g.ntiles ? pd_tile_rows(g, tile) * g.U : 0;
#pragma unroll
    for (int d = 0; d < PD_D; d++) {
        const uint32_t u = (round * PD_D + d) * PD_WAVES + cx.wave;
        W.v[d] = make_int4(0, 0, 0, 0);
        W.s[d] = 0;
        if (u < units) {
            const uint32_t lr = u / g.U, j = u - lr * g.U;
            const size_t row = pd_tile_row(g, tile, lr);
            if (Q4) {
                const uint32_t blk = j * 64 + cx.lane;
                if (blk < g.nblk) {
                    W.v[d] = *reinterpret_cast<const int4*>(g.qs + (row * g.nblk + blk) * 16);
                    W.s[d] = g.ws[row * g.nblk + blk];
                }
            } else {
                const uint32_t off = j * 1024 + cx.lane * 16;
                if (off < g.K) {
                    W.v[d] = *reinterpret_cast<const int4*>(g.qs + row * g.K + off);
                    W.s[d] = g.ws[row * g.nblk + off / 32];
                }
            }
        }
    }
}

// Exact int32 block dots on v_dot4, one f32 product (a_s*w_s)*f32(isum) per block parked in LDS.
template <bool Q4>
__device__ __forceinline__ void pd_compute_round(const PdGemv& g, uint32_t tile, uint32_t round, const PdCtx& cx, const WReg& W,
                                                 const uint32_t* aq_lds, const float* as_lds, float* prod, uint32_t pstride) {
    const uint32_t units = pd_tile_rows(g, tile) * g.U;
#pragma unroll
    for (int d = 0; d < PD_D; d++) {
        const uint32_t u = (round * PD_D + d) * PD_WAVES + cx.wave;
        if (u < units) {
            const uint32_t lr = u / g.U, j = u - lr * g.U;
            if (Q4) {
                const uint32_t blk = j * 64 + cx.lane;
                if (blk < g.nblk) {
                    const int4 a0 = *reinterpret_cast<const int4*>(aq_lds + blk * 8);
                    const int4 a1 = *reinterpret_cast<const int4*>(aq_lds + blk * 8 + 4);
                    const int4 w = W.v[d];
                    const int m = 0x0F0F0F0F;
                    const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                    const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                    const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
                    const int asum8 = 8 * dot16(ones, a1, dot16(ones, a0, 0));
                    const int isum = dot16(hi, a1, dot16(lo, a0, 0)) - asum8;
                    prod[lr * pstride + blk] = (as_lds[blk] * f16_bits_to_f32((uint16_t)W.s[d])) * (float)isum;
                }
            } else {
                const uint32_t off = j * 1024 + cx.lane * 16;
                const bool in = off < g.K;
                const int4 a = in ? *reinterpret_cast<const int4*>(aq_lds + off / 4) : make_int4(0, 0, 0, 0);
                const int half = dot16(W.v[d], a, 0);
                const int isum = half + __shfl_xor(half, 1, WAVE);
                if (in && !(cx.lane & 1u))
                    prod[lr * pstride + off / 32] = (as_lds[off / 32] * f16_bits_to_f32((uint16_t)W.s[d])) * (float)isum;
            }
        }
    }
}

// Runs the tiles of this workgroup.  `epi(tile, lr, row, value, active)` is called by whole waves (lanes past
// the tile's rows come with active = false) once the ordered sum of a row is known.
// `pre(tile, lr, row, active)` runs before the sums: the place to start loads the epilogue will need.
template <bool Q4, typename Pre, typename Epi>
__device__ __forceinline__ void pd_gemv(const PdGemv& g, bool prefetched, WReg& W, const uint32_t* aq_lds, const float* as_lds,
                                        float* prod, const PdCtx& cx, Pre pre, Epi epi) {
    const uint32_t pstride = g.nblk + 1;                    // +1: conflict-free column reads
    for (uint32_t tile = cx.wg; tile < g.ntiles; tile += cx.G) {
        const uint32_t rows = pd_tile_rows(g, tile);
        const uint32_t rounds = (rows * g.U + PD_D * PD_WAVES - 1) / (PD_D * PD_WAVES);
        for (uint32_t r = 0; r < rounds; r++) {
            if (!(prefetched && r == 0)) pd_load_round<Q4>(g, tile, r, cx, W);
            pd_compute_round<Q4>(g, tile, r, cx, W, aq_lds, as_lds, prod, pstride);
        }
        // the next tile's first loads fly while this tile's rows are summed
        prefetched = tile + cx.G < g.ntiles;
        if (prefetched) pd_load_round<Q4>(g, tile + cx.G, 0, cx, W);
        if (cx.tid < ((rows + 63u) & ~63u)) pre(tile, cx.tid, pd_tile_row(g, tile, cx.tid < rows ? cx.tid : 0), cx.tid < rows);
        __syncthreads();
        if (cx.tid < ((rows + 63u) & ~63u)) {
            const bool active = cx.tid < rows;
            const uint32_t row = pd_tile_row(g, tile, active ? cx.tid : 0);
            float v = 0.f;
            if (active) v = ordered_sum(prod + cx.tid * pstride, g.nblk, segment_row_is_dot1(row, g.seg, g.nseg, g.tail_mod));
            epi(tile, cx.tid, row, v, active);
        }
        __syncthreads();
    }
}

// ---- attention ------------------------------------------------------------------------------------------
struct __attribute__((aligned(16))) Half8 { uint32_t w[4]; };

__device__ __forceinline__ void unpack8(const Half8& h, float* f) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = f16_bits_to_f32((uint16_t)(h.w[i] & 0xFFFFu));
        f[2 * i + 1] = f16_bits_to_f32((uint16_t)(h.w[i] >> 16));
    }
}

template <int NV>
__device__ __forceinline__ void merge_state(float& m, float& l, float* a, float m2, float l2, const float* a2) {
    const float mn = fmaxf(m, m2);
    const float s1 = (m == -INFINITY) ? 0.f : __expf(m - mn);
    const float s2 = (m2 == -INFINITY) ? 0.f : __expf(m2 - mn);
    l = l * s1 + l2 * s2;
#pragma unroll
    for (int i = 0; i < NV; i++) a[i] = a[i] * s1 + a2[i] * s2;
    m = mn;
}

// P2: the work items of attn_decode_split_kernel (kv head group x split), one per workgroup at a time.  The
// separate kernel gives an item four waves that each carry all `gt` query heads of the group; here wave
// 4 g + w carries head g over the keys wave w would take (same keys, same order, same merges), which
// keeps the per-thread state small.  Keys before this position come from the cache, this position's K/V
// row and q from the tagged buffers P1 filled.
template <int HD>
__device__ __forceinline__ void pd_attn_split(const PdArgs& a, const PdLayer& L, uint32_t pos, uint32_t tag_in, uint32_t tag_out,
                                              float* big, const PdCtx& cx) {
    constexpr int LPK = HD <= 64 ? 8 : 16;
    constexpr int KPW = 64 / LPK;
    constexpr int REC = HD + 2;
    const uint32_t g = cx.wave >> 2, wave = cx.wave & 3u, lane = cx.lane;
    float* sh = big;                                                  // [4 waves][4][REC]
    float* q_lds = sh + 16 * REC;                                     // [gt][HD]
    uint32_t* kvn = reinterpret_cast<uint32_t*>(q_lds + 4 * HD);      // [2][HD] fp16 bits of this position's K and V
    const uint32_t gt = a.gt, gsize = a.heads / a.kv_heads, gpk = gsize / gt;
    const uint32_t nbx = a.kv_heads * gpk, n_items = nbx * DECODE_SPLITS;
    const uint32_t seq = pos + 1;
    const uint32_t c = lane % LPK, slot = lane / LPK;
    const bool dvalid = c * 8 < HD;
    const float scale = 1.0f / sqrtf((float)HD);
    const uint32_t kv_stride = a.KV;
    uint32_t chunk = (seq + DECODE_SPLITS - 1) / DECODE_SPLITS;
    chunk = (chunk + 4 * KPW - 1) / (4 * KPW) * (4 * KPW);

    for (uint32_t item = cx.wg; item < n_items; item += cx.G) {
        const uint32_t bx = item % nbx, split = item / nbx;
        const uint32_t kvh = bx / gpk, sub = bx % gpk;
        const uint32_t h0 = kvh * gsize + sub * gt;
        const uint32_t t0 = split * chunk;
        const uint32_t t1 = min(seq, t0 + chunk);
        const bool has_new = t0 <= pos && pos < t1;
        // q is awaited even when the split is empty: the wait orders this item's records after the previous layer's readers
        for (uint32_t e = cx.tid; e < gt * HD || (has_new && e < 2 * HD); e += PD_THREADS) {
            const bool need_q = e < gt * HD, need_kv = has_new && e < 2 * HD;
            const uint64_t* pq = a.tq + (size_t)h0 * HD + e;
            const uint64_t* pkv = a.tkv + (e < HD ? kvh * HD + e : a.KV + kvh * HD + (e - HD));
            uint32_t v[2];
            // one batch: an element that is not needed re-reads the needed one
            poll_many<2>([&](int i) { return (i == 0 ? need_q : !need_kv) ? pq : pkv; }, 2, tag_in, v, cx);
            if (need_q) q_lds[e] = __uint_as_float(v[0]);
            if (need_kv) kvn[e] = v[1];
        }
        __syncthreads();
        if (*cx.sh_abort) return;

        if (g < gt) {
            float qf[8], acc[8], m = -INFINITY, l = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) { acc[i] = 0.f; qf[i] = dvalid ? q_lds[g * HD + c * 8 + i] : 0.f; }
            constexpr int UNR = 4;        // key blocks whose K/V loads are issued together
            for (uint32_t tb0 = t0 + wave * KPW; tb0 < t1; tb0 += UNR * 4 * KPW) {
                Half8 kr[UNR], vr[UNR];
#pragma unroll
                for (int u = 0; u < UNR; u++) {
                    const uint32_t t = tb0 + u * 4 * KPW + slot;
                    kr[u] = Half8{{0, 0, 0, 0}};
                    vr[u] = Half8{{0, 0, 0, 0}};
                    if (t < t1 && dvalid) {
                        if (t == pos) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                kr[u].w[i] = (kvn[c * 8 + 2 * i] & 0xFFFFu) | (kvn[c * 8 + 2 * i + 1] << 16);
                                vr[u].w[i] = (kvn[HD + c * 8 + 2 * i] & 0xFFFFu) | (kvn[HD + c * 8 + 2 * i + 1] << 16);
                            }
                        } else {
                            const size_t off = (size_t)t * kv_stride + kvh * HD + c * 8;
                            kr[u] = *reinterpret_cast<const Half8*>(L.kc + off);
                            vr[u] = *reinterpret_cast<const Half8*>(L.vc + off);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < UNR; u++) {
                    const uint32_t tb = tb0 + u * 4 * KPW;
                    if (tb < t1) {
                        const bool valid = tb + slot < t1;
                        float kf[8], vf[8];
                        unpack8(kr[u], kf);
                        unpack8(vr[u], vf);
                        float d = 0.f;
#pragma unroll
                        for (int i = 0; i < 8; i++) d = fmaf(qf[i], kf[i], d);
#pragma unroll
                        for (int o = 1; o < LPK; o <<= 1) d += __shfl_xor(d, o, WAVE);
                        if (valid) {
                            const float sc = d * scale;
                            const float mn = fmaxf(m, sc);
                            const float alpha = __expf(m - mn);   // m = -inf on the first key: exp(-inf) = 0
                            const float p = __expf(sc - mn);
                            l = fmaf(l, alpha, p);
#pragma unroll
                            for (int i = 0; i < 8; i++) acc[i] = fmaf(acc[i], alpha, p * vf[i]);
                            m = mn;
                        }
                    }
                }
            }
            // merge the key slots of the wave
#pragma unroll
            for (int o = LPK; o < 64; o <<= 1) {
                float m2 = __shfl_xor(m, o, WAVE), l2 = __shfl_xor(l, o, WAVE);
                float a2[8];
#pragma unroll
                for (int i = 0; i < 8; i++) a2[i] = __shfl_xor(acc[i], o, WAVE);
                merge_state<8>(m, l, acc, m2, l2, a2);
            }
            if (slot == 0 && dvalid) {
                float* rec = sh + (wave * 4 + g) * REC;
#pragma unroll
                for (int i = 0; i < 8; i++) rec[c * 8 + i] = acc[i];
                if (c == 0) { rec[HD] = m; rec[HD + 1] = l; }
            }
        }
        __syncthreads();
        // merge the four key waves: one thread per output element
        for (uint32_t e = cx.tid; e < gt * HD; e += PD_THREADS) {
            const uint32_t gg = e / HD, d = e % HD;
            float mm = sh[gg * REC + HD], ll = sh[gg * REC + HD + 1], av = sh[gg * REC + d];
            for (int w = 1; w < 4; w++) {
                float a2 = sh[(w * 4 + gg) * REC + d];
                merge_state<1>(mm, ll, &av, sh[(w * 4 + gg) * REC + HD], sh[(w * 4 + gg) * REC + HD + 1], &a2);
            }
            uint64_t* rec = a.tws + ((size_t)(h0 + gg) * DECODE_SPLITS + split) * REC;
            stc64(rec + d, tag_out, __float_as_uint(av));
            if (d == 0) { stc64(rec + HD, tag_out, __float_as_uint(mm)); stc64(rec + HD + 1, tag_out, __float_as_uint(ll)); }
        }
        __syncthreads();
    }
}

// P3: attn_decode_combine_kernel, one head per workgroup at a time; output quantised for the O GEMV.  All
// threads fetch the head's split records into LDS in one round trip, then HD threads merge them.
template <int HD>
__device__ __forceinline__ void pd_attn_combine(const PdArgs& a, uint32_t tag_in, uint32_t tag_out, float* misc, float* big,
                                                const PdCtx& cx) {
    constexpr int REC = HD + 2;
    const uint32_t d = cx.tid;
    float* wgt_s = misc + 64;                    // [DECODE_SPLITS] + den
    float* recs = big;                           // [DECODE_SPLITS][REC]
    for (uint32_t h = cx.wg; h < a.heads; h += cx.G) {
        const uint64_t* base = a.tws + (size_t)h * DECODE_SPLITS * REC;
        poll_vec(base, DECODE_SPLITS * REC, tag_in, cx, [&](uint32_t i, uint32_t p) { recs[i] = __uint_as_float(p); });
        __syncthreads();
        if (*cx.sh_abort) return;
        if (d < 64) {
            const float ms = d < DECODE_SPLITS ? recs[d * REC + HD] : -INFINITY;
            const float ls = d < DECODE_SPLITS ? recs[d * REC + HD + 1] : 0.f;
            const float mm = wave_max(ms);
            const float wgt = (ms == -INFINITY) ? 0.f : __expf(ms - mm);
            const float den = wave_sum(wgt * ls);
            if (d < DECODE_SPLITS) wgt_s[d] = wgt;
            if (d == 0) wgt_s[DECODE_SPLITS] = den;
        }
        __syncthreads();
        if (d < HD) {
            float num = 0.f;
#pragma unroll
            for (uint32_t s = 0; s < DECODE_SPLITS; s++) num = fmaf(wgt_s[s], recs[s * REC + d], num);
            const float o = num * (1.0f / wgt_s[DECODE_SPLITS]);
            float amax = fabsf(o);
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
            float inv;
            const float sc = act_scale(amax, inv);
            const uint32_t code = (uint32_t)quant_code(o * inv) & 0xFFu;
            const uint32_t base_lane = cx.lane & ~3u;
            const uint32_t pk = __shfl(code, base_lane, WAVE) | (__shfl(code, base_lane + 1, WAVE) << 8) |
                                (__shfl(code, base_lane + 2, WAVE) << 16) | (__shfl(code, base_lane + 3, WAVE) << 24);
            const uint32_t e = h * HD + d;
            if ((d & 3u) == 0) stc64(a.taq + e / 4, tag_out, pk);
            if ((d & 31u) == 0) stc64(a.taq + a.QKS / 4 + e / 32, tag_out, f32_to_f16_bits(sc));
        }
        __syncthreads();
    }
}

// ---- argmax (project.rs:501-503): the LAST index among equal maxima --------------------------------------
struct ArgPair { float v; uint32_t i; };
__device__ __forceinline__ ArgPair arg_better(ArgPair a, ArgPair b) {
    const bool take_b = (b.v > a.v) || (b.v == a.v && b.i > a.i);
    return take_b ? b : a;
}
__device__ __forceinline__ ArgPair arg_wg(ArgPair a, float* misc, const PdCtx& cx) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgPair b;
        b.v = __shfl_xor(a.v, o, WAVE);
        b.i = __shfl_xor(a.i, o, WAVE);
        a = arg_better(a, b);
    }
    ArgPair* sh = reinterpret_cast<ArgPair*>(misc + 64);
    __syncthreads();
    if (cx.lane == 0) sh[cx.wave] = a;
    __syncthreads();
    ArgPair r = sh[0];
    for (int w = 1; w < PD_WAVES; w++) r = arg_better(r, sh[w]);
    return r;
}

#define PD_EXIT_IF_ABORTED() do { if (*cx.sh_abort) return; } while (0)
#define PD_STAMP(idx) do { if (a.stamps && cx.wg == 0 && cx.tid == 0) a.stamps[idx] = wall_clock64(); } while (0)

template <bool Q4, bool LMQ4, int HD>
__global__ __launch_bounds__(PD_THREADS) void decode_step_kernel(PdArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    __shared__ uint32_t sh_abort;
    uint32_t* aq_lds = reinterpret_cast<uint32_t*>(smem);
    float* as_lds = reinterpret_cast<float*>(smem + a.off_act_s);
    float* misc = reinterpret_cast<float*>(smem + a.off_misc);       // [0,32) norm partials, [64, ...) phase scratch
    float* big = reinterpret_cast<float*>(smem + a.off_big);         // x copy / block products / attention scratch

    PdCtx cx;
    cx.tid = threadIdx.x;
    cx.lane = threadIdx.x & 63u;
    cx.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    cx.wg = blockIdx.x;
    cx.G = gridDim.x;
    cx.spin_limit = a.spin_limit;
    cx.sh_abort = &sh_abort;
    cx.abort_flag = a.state + 3;
    if (cx.tid == 0) sh_abort = 0;
    __syncthreads();

    const uint32_t pos = a.state[0], token = a.state[1];
    const uint32_t H = a.H;
    const float* emb = a.embed + (size_t)token * H;
    uint32_t tag = a.tag_base;            // tag of phase instance k of this launch = tag_base + k
    uint32_t x_tag = 0;                   // tag of the current version of tx (0: x is still the embedding row)
    uint32_t stamp = 0;
    WReg W;

    {
        const PdGemv& g0 = a.layers[0].qkv;
        pd_load_round<Q4>(g0, cx.wg, 0, cx, W);
    }
    for (uint32_t l = 0; l < a.n_layers; l++) {
        const PdLayer& L = a.layers[l];
        // ---------------- P1: norm | qkv GEMV | rope + KV ----------------
        PD_STAMP(stamp++);
        const uint32_t t1 = ++tag;
        if (cx.wg < L.qkv.ntiles) {
            if (x_tag) {
                wait_hint(a.tx + H - 1, x_tag, cx);
                poll_vec(a.tx, H, x_tag, cx, [&](uint32_t i, uint32_t p) { big[i] = __uint_as_float(p); });
            } else {
                for (uint32_t i = cx.tid; i < H; i += PD_THREADS) big[i] = emb[i];
            }
            __syncthreads();
            PD_EXIT_IF_ABORTED();
            // the norm reads big[0..H); the products reuse the area afterwards
            pd_norm_quant(big, L.attn_norm, a.eps, H, aq_lds, as_lds, misc, cx);
            float rc = 0.f, rs = 0.f;
            pd_gemv<Q4>(L.qkv, true, W, aq_lds, as_lds, big, cx, [&](uint32_t, uint32_t, uint32_t row, bool active) {
                if (active && row < a.QKS + a.KV) {
                    const uint32_t d = row < a.QKS ? row % HD : (row - a.QKS) % HD;
                    rc = a.cos_t[(size_t)pos * (HD / 2) + d / 2];
                    rs = a.sin_t[(size_t)pos * (HD / 2) + d / 2];
                }
            }, [&](uint32_t, uint32_t, uint32_t row, float r, bool active) {
                // rope (emit.rs:508-528): rows 2i, 2i+1 of a head sit in neighbouring lanes
                const float other = __shfl_xor(r, 1, WAVE);
                if (!active) return;
                if (row < a.QKS + a.KV) {
                    const float c = rc, s = rs;
                    const float o = (row & 1u) ? other * s + r * c : r * c - other * s;
                    if (row < a.QKS) {
                        stc64(a.tq + row, t1, __float_as_uint(o));
                    } else {
                        const uint16_t hb = f32_to_f16_bits(o);
                        L.kc[(size_t)pos * a.KV + (row - a.QKS)] = hb;
                        stc64(a.tkv + (row - a.QKS), t1, hb);
                    }
                } else {
                    const uint16_t hb = f32_to_f16_bits(r);
                    L.vc[(size_t)pos * a.KV + (row - a.QKS - a.KV)] = hb;
                    stc64(a.tkv + a.KV + (row - a.QKS - a.KV), t1, hb);
                }
            });
        }
        // ---------------- P2: attention, split along the sequence ----------------
        PD_STAMP(stamp++);
        const uint32_t t2 = ++tag;
        pd_attn_split<HD>(a, L, pos, t1, t2, big, cx);
        PD_EXIT_IF_ABORTED();
        // ---------------- P3: merge the splits, quantise ----------------
        PD_STAMP(stamp++);
        const uint32_t t3 = ++tag;
        pd_attn_combine<HD>(a, t2, t3, misc, big, cx);
        PD_EXIT_IF_ABORTED();
        // ---------------- P4: O GEMV + residual ----------------
        PD_STAMP(stamp++);
        const uint32_t t4 = ++tag;
        if (cx.wg < L.o.ntiles) {
            pd_load_round<Q4>(L.o, cx.wg, 0, cx, W);
            pd_load_aq(a.taq, t3, a.QKS, aq_lds, as_lds, cx);
            PD_EXIT_IF_ABORTED();
            const uint32_t xin = x_tag;
            uint64_t res_w = 0;
            float res_e = 0.f;
            pd_gemv<Q4>(L.o, true, W, aq_lds, as_lds, big, cx, [&](uint32_t, uint32_t, uint32_t row, bool active) {
                if (!active) return;
                if (xin) res_w = ldc64(a.tx + row);       // in flight while the rows are summed; the tag is checked below
                else res_e = emb[row];
            }, [&](uint32_t, uint32_t, uint32_t row, float r, bool active) {
                if (!active) return;
                float res = res_e;
                if (xin) res = __uint_as_float((uint32_t)(res_w >> 32) == xin ? (uint32_t)res_w : poll(a.tx + row, xin, cx));
                stc64(a.tx + row, t4, __float_as_uint(res + r));       // residual_add, emit.rs:455-459
            });
            PD_EXIT_IF_ABORTED();
        }
        x_tag = t4;
        // ---------------- P5: norm | gate/up GEMV | silu*up, quantise ----------------
        PD_STAMP(stamp++);
        const uint32_t t5 = ++tag;
        if (cx.wg < L.gu.ntiles) {
            pd_load_round<Q4>(L.gu, cx.wg, 0, cx, W);
            wait_hint(a.tx + H - 1, x_tag, cx);
            poll_vec(a.tx, H, x_tag, cx, [&](uint32_t i, uint32_t p) { big[i] = __uint_as_float(p); });
            __syncthreads();
            PD_EXIT_IF_ABORTED();
            pd_norm_quant(big, L.ffn_norm, a.eps, H, aq_lds, as_lds, misc, cx);
            pd_gemv<Q4>(L.gu, true, W, aq_lds, as_lds, big, cx, [](uint32_t, uint32_t, uint32_t, bool) {},
                        [&](uint32_t tile, uint32_t lr, uint32_t, float r, bool) {
                // lanes 0..31 hold the gate rows of inter indices [32 tile, +32), lanes 32..63 the up rows
                const float ux = __shfl(r, (cx.lane & 31u) + 32, WAVE);
                if (lr >= 32) return;
                const float o = (r / (1.0f + expf_ref<true>(-r))) * ux;          // silu_mul, emit.rs:380-386
                float amax = fabsf(o);
#pragma unroll
                for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
                float inv;
                const float sc = act_scale(amax, inv);
                const uint32_t code = (uint32_t)quant_code(o * inv) & 0xFFu;
                const uint32_t bl = lr & ~3u;
                const uint32_t pk = __shfl(code, bl, WAVE) | (__shfl(code, bl + 1, WAVE) << 8) | (__shfl(code, bl + 2, WAVE) << 16) |
                                    (__shfl(code, bl + 3, WAVE) << 24);
                if ((lr & 3u) == 0) stc64(a.taq2 + tile * 8 + lr / 4, t5, pk);
                if (lr == 0) stc64(a.taq2 + a.I / 4 + tile, t5, f32_to_f16_bits(sc));
            });
        }
        // ---------------- P6: down GEMV + residual ----------------
        PD_STAMP(stamp++);
        const uint32_t t6 = ++tag;
        if (cx.wg < L.down.ntiles) {
            pd_load_round<Q4>(L.down, cx.wg, 0, cx, W);
            pd_load_aq(a.taq2, t5, a.I, aq_lds, as_lds, cx);
            PD_EXIT_IF_ABORTED();
            uint64_t res_w = 0;
            pd_gemv<Q4>(L.down, true, W, aq_lds, as_lds, big, cx, [&](uint32_t, uint32_t, uint32_t row, bool active) {
                if (active) res_w = ldc64(a.tx + row);
            }, [&](uint32_t, uint32_t, uint32_t row, float r, bool active) {
                if (!active) return;
                const float res = __uint_as_float((uint32_t)(res_w >> 32) == t4 ? (uint32_t)res_w : poll(a.tx + row, t4, cx));
                stc64(a.tx + row, t6, __float_as_uint(res + r));
            });
            PD_EXIT_IF_ABORTED();
        }
        x_tag = t6;
        if (l + 1 < a.n_layers) pd_load_round<Q4>(a.layers[l + 1].qkv, cx.wg, 0, cx, W);
    }

    // ---------------- head: final norm | lm_head GEMV | argmax ----------------
    PD_STAMP(stamp++);
    const uint32_t th = ++tag;
    ArgPair best{-INFINITY, 0};
    if (cx.wg < a.lm.ntiles) {
        WReg WL;
        pd_load_round<LMQ4>(a.lm, cx.wg, 0, cx, WL);
        wait_hint(a.tx + H - 1, x_tag, cx);
        poll_vec(a.tx, H, x_tag, cx, [&](uint32_t i, uint32_t p) { big[i] = __uint_as_float(p); });
        __syncthreads();
        PD_EXIT_IF_ABORTED();
        pd_norm_quant(big, a.final_norm, a.eps, H, aq_lds, as_lds, misc, cx);
        pd_gemv<LMQ4>(a.lm, true, WL, aq_lds, as_lds, big, cx, [](uint32_t, uint32_t, uint32_t, bool) {},
                      [&](uint32_t, uint32_t, uint32_t row, float r, bool active) {
            if (!active) return;
            a.logits[row] = r;
            best = arg_better(best, ArgPair{r, row});
        });
    }
    best = arg_wg(best, misc, cx);
    if (cx.tid == 0) {
        stc64(a.tpart + 2 * cx.wg, th, __float_as_uint(best.v));
        stc64(a.tpart + 2 * cx.wg + 1, th, best.i);
    }
    PD_STAMP(stamp++);
    if (cx.wg == 0) {
        ArgPair p{-INFINITY, 0};
        if (cx.tid < cx.G) {
            uint32_t v[2];
            poll_many<2>([&](int i) { return a.tpart + 2 * cx.tid + (uint32_t)i; }, 2, th, v, cx);
            p.v = __uint_as_float(v[0]);
            p.i = v[1];
        }
        p = arg_wg(p, misc, cx);
        PD_EXIT_IF_ABORTED();
        if (cx.tid == 0) {
            a.state[2] = p.i;
            a.state[1] = p.i;
            a.state[0] = pos + 1;
        }
        PD_STAMP(stamp++);
    }
}

template <typename T>
T* dev_alloc(size_t n, std::vector<void*>& owned) {
    void* p = nullptr;
    if (hipMalloc(&p, n < 16 ? 16 : n) != hipSuccess) return nullptr;
    owned.push_back(p);
    return reinterpret_cast<T*>(p);
}

uint32_t round_up(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

}  // namespace

struct PdState {
    PdArgs args{};
    std::vector<void*> owned;
    uint32_t grid = 0, lds = 0, hd = 0, tags_per_launch = 0, n_stamps = 0;
    bool q4 = false, lmq4 = false;
    size_t tagged_bytes = 0;
    void* tagged_base = nullptr;
    std::vector<unsigned long long> stamps_host;
    int wall_khz = 0;
    ~PdState() { for (void* p : owned) (void)hipFree(p); }
};

namespace {

// Tile plan of one matrix: rows per tile so that the tiles spread evenly over the grid and a tile's block
// products fit `big_bytes` of LDS.  Returns false if they cannot.
bool plan_gemv(const QWeight& w, uint32_t inter, uint32_t nseg, const Segment* seg, uint32_t tail_mod, uint32_t grid,
               uint32_t big_bytes, PdGemv* g) {
    g->qs = w.qs; g->ws = w.scales; g->K = w.K; g->N = w.N; g->nblk = w.K / 32;
    const uint32_t epu = w.wdtype == FORGE_HIP_Q8_0 ? 1024 : 2048;
    g->U = (w.K + epu - 1) / epu;
    g->inter = inter;
    g->nseg = nseg; g->tail_mod = tail_mod;
    for (uint32_t i = 0; i < nseg; i++) g->seg[i] = seg[i];
    const uint32_t row_bytes = (g->nblk + 1) * 4;
    uint32_t cap = big_bytes / row_bytes;
    if (cap > PD_MAX_TILE_ROWS) cap = PD_MAX_TILE_ROWS;
    cap &= ~1u;
    if (inter) {
        if (cap < 64 || inter % 32 != 0) return false;
        g->T = 64; g->ntiles = inter / 32;
        return true;
    }
    if (cap < 2) return false;
    const uint32_t rounds = (w.N + grid * cap - 1) / (grid * cap);
    uint32_t T = (w.N + grid * rounds - 1) / (grid * rounds);
    T = round_up(T, 2);
    if (T > cap) T = cap;
    g->T = T;
    g->ntiles = (w.N + T - 1) / T;
    return true;
}

template <bool Q4, bool LMQ4, int HD>
hipError_t launch_pd(const PdState* st, hipStream_t s) {
    void* kargs[] = {const_cast<PdArgs*>(&st->args)};
    return hipLaunchCooperativeKernel(reinterpret_cast<void*>(decode_step_kernel<Q4, LMQ4, HD>), dim3(st->grid), dim3(PD_THREADS), kargs,
                                      st->lds, s);
}

template <int HD>
hipError_t launch_pd_hd(const PdState* st, hipStream_t s) {
    if (!st->q4 && !st->lmq4) return launch_pd<false, false, HD>(st, s);
    if (st->q4 && st->lmq4) return launch_pd<true, true, HD>(st, s);
    if (st->q4) return launch_pd<true, false, HD>(st, s);
    return hipErrorInvalidValue;
}

}  // namespace

void pd_destroy(PdState* st) { delete st; }

// Plans the persistent decode step for a model.  Leaves *out null (and returns OK) when the shape or the
// device is outside what the kernel covers; the caller then keeps the multi-kernel step.
int32_t pd_create(const forge_hip_config& c, const std::vector<PdLayerIn>& layers, const QWeight& lm_head, const float* embed,
                  const float* final_norm, const float* cos_t, const float* sin_t, float* logits, uint32_t* state, PdState** out) {
    *out = nullptr;
    if (c.flags & FORGE_HIP_FLAG_EXACT) return FORGE_HIP_OK;
    if (c.head_dim != 64 && c.head_dim != 128) return FORGE_HIP_OK;
    if (c.wdtype == FORGE_HIP_Q8_0 && c.lm_head_dtype == FORGE_HIP_Q4_0) return FORGE_HIP_OK;
    int dev = 0, coop = 0, cus = 0, khz = 0;
    FH_HIP(hipGetDevice(&dev));
    FH_HIP(hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev));
    FH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    FH_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    if (!coop || cus < 1) return FORGE_HIP_OK;

    std::unique_ptr<PdState> st(new PdState());
    PdArgs& a = st->args;
    const uint32_t H = c.hidden, I = c.inter, hd = c.head_dim, QKS = c.heads * hd, KV = c.kv_heads * hd;
    const uint32_t kmax = std::max(std::max(H, I), QKS);
    const uint32_t gsize = c.heads / c.kv_heads;
    a.gt = gsize % 4 == 0 ? 4 : gsize % 3 == 0 ? 3 : gsize % 2 == 0 ? 2 : 1;
    st->grid = (uint32_t)cus;
    st->hd = hd;
    st->q4 = c.wdtype == FORGE_HIP_Q4_0;
    st->lmq4 = c.lm_head_dtype == FORGE_HIP_Q4_0;
    st->wall_khz = khz;

    // LDS: activation codes | activation scales | misc | big
    a.off_act_s = round_up(kmax, 16);
    a.off_misc = a.off_act_s + round_up(kmax / 32 * 4, 16);
    a.off_big = a.off_misc + PD_MISC_BYTES;
    if (a.off_big + 4096 > PD_LDS_BYTES) return FORGE_HIP_OK;
    const uint32_t big = PD_LDS_BYTES - 64 - a.off_big;
    const uint32_t attn_bytes = (16 * (hd + 2) + 6 * hd) * 4;
    if ((H + 32) * 4 > big || attn_bytes > big || DECODE_SPLITS * (hd + 2) * 4 > big) return FORGE_HIP_OK;
    st->lds = a.off_big + big;

    std::vector<PdLayer> hl(layers.size());
    for (size_t l = 0; l < layers.size(); l++) {
        const PdLayerIn& in = layers[l];
        PdLayer& L = hl[l];
        const uint32_t wt = c.wdtype;
        Segment sq[3] = {make_segment(wt, H, 0, QKS, false), make_segment(wt, H, QKS, KV, false), make_segment(wt, H, QKS + KV, KV, false)};
        Segment so[1] = {make_segment(wt, QKS, 0, H, false)};
        Segment sg[2] = {make_segment(wt, H, 0, I, false), make_segment(wt, H, I, I, false)};
        Segment sd[1] = {make_segment(wt, I, 0, H, false)};
        if (!plan_gemv(*in.qkv, 0, 3, sq, 4, st->grid, big, &L.qkv) || !plan_gemv(*in.o, 0, 1, so, 4, st->grid, big, &L.o) ||
            !plan_gemv(*in.gate_up, I, 2, sg, 4, st->grid, big, &L.gu) || !plan_gemv(*in.down, 0, 1, sd, 4, st->grid, big, &L.down))
            return FORGE_HIP_OK;
        L.attn_norm = in.attn_norm; L.ffn_norm = in.ffn_norm; L.kc = in.kc; L.vc = in.vc;
    }
    {
        Segment sl[1] = {make_segment(c.lm_head_dtype, H, 0, c.vocab, true)};
        if (!plan_gemv(lm_head, 0, 1, sl, 4, st->grid, big, &a.lm)) return FORGE_HIP_OK;
    }
    // cooperative residency: one workgroup per CU must fit
    {
        int per_cu = 0;
        hipError_t e = hipErrorInvalidValue;
        const bool q4 = st->q4, lq4 = st->lmq4;
#define PD_OCC(Q, LQ, HDV) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_step_kernel<Q, LQ, HDV>, PD_THREADS, st->lds)
        if (hd == 64) { if (!q4) PD_OCC(false, false, 64); else if (lq4) PD_OCC(true, true, 64); else PD_OCC(true, false, 64); }
        else { if (!q4) PD_OCC(false, false, 128); else if (lq4) PD_OCC(true, true, 128); else PD_OCC(true, false, 128); }
#undef PD_OCC
        if (e != hipSuccess || per_cu < 1) { (void)hipGetLastError(); return FORGE_HIP_OK; }
    }

    PdLayer* dl = dev_alloc<PdLayer>(hl.size() * sizeof(PdLayer), st->owned);
    if (!dl) return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory");
    FH_HIP(hipMemcpy(dl, hl.data(), hl.size() * sizeof(PdLayer), hipMemcpyHostToDevice));
    a.layers = dl;
    a.n_layers = (uint32_t)hl.size();
    a.H = H; a.I = I; a.QKS = QKS; a.KV = KV; a.heads = c.heads; a.kv_heads = c.kv_heads;
    a.eps = c.rms_eps;
    a.embed = embed; a.final_norm = final_norm; a.cos_t = cos_t; a.sin_t = sin_t;
    a.logits = logits; a.state = state;
    // one allocation for all tagged buffers (zeroed: tag 0 is never expected)
    const size_t n_tx = H, n_tq = QKS, n_tkv = 2 * (size_t)KV, n_tws = (size_t)c.heads * DECODE_SPLITS * (hd + 2),
                 n_taq = QKS / 4 + QKS / 32, n_taq2 = I / 4 + I / 32, n_tpart = 2 * (size_t)st->grid;
    const size_t total = n_tx + n_tq + n_tkv + n_tws + n_taq + n_taq2 + n_tpart;
    uint64_t* t = dev_alloc<uint64_t>(total * 8, st->owned);
    if (!t) return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory");
    FH_HIP(hipMemset(t, 0, total * 8));
    st->tagged_base = t; st->tagged_bytes = total * 8;
    a.tx = t; t += n_tx;
    a.tq = t; t += n_tq;
    a.tkv = t; t += n_tkv;
    a.tws = t; t += n_tws;
    a.taq = t; t += n_taq;
    a.taq2 = t; t += n_taq2;
    a.tpart = t;
    a.tag_base = 0;
    a.spin_limit = 400000;
    st->tags_per_launch = 6 * a.n_layers + 1;
    st->n_stamps = 6 * a.n_layers + 3;
    a.stamps = nullptr;
    *out = st.release();
    return FORGE_HIP_OK;
}

// Enqueue one decode step (token and position are in `state`).  With `profile` the kernel also records
// the wall clock at the start of every phase.
int32_t pd_enqueue(PdState* st, bool profile, hipStream_t s) {
    PdArgs& a = st->args;
    if (a.tag_base > 0xF0000000u) {      // tags are about to wrap: start again from zeroed buffers
        FH_HIP(hipMemsetAsync(st->tagged_base, 0, st->tagged_bytes, s));
        a.tag_base = 0;
    }
    if (profile && !a.stamps) {
        a.stamps = dev_alloc<unsigned long long>(st->n_stamps * 8, st->owned);
        if (!a.stamps) return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory");
    }
    unsigned long long* keep = a.stamps;
    if (!profile) a.stamps = nullptr;
    const hipError_t e = st->hd == 64 ? launch_pd_hd<64>(st, s) : launch_pd_hd<128>(st, s);
    a.stamps = keep;
    if (e != hipSuccess) return fail(FORGE_HIP_ERR_HIP, std::string("persistent decode launch: ") + hipGetErrorString(e));
    a.tag_base += st->tags_per_launch;
    return FORGE_HIP_OK;
}

// After the stream has drained: did every workgroup get through?  (state[3] is the abort flag.)
int32_t pd_after_sync(PdState* st, uint32_t abort_flag, hipStream_t s) {
    if (!abort_flag) return FORGE_HIP_OK;
    PdArgs& a = st->args;
    FH_HIP(hipMemsetAsync(st->tagged_base, 0, st->tagged_bytes, s));
    FH_HIP(hipMemsetAsync(a.state + 3, 0, 4, s));
    FH_HIP(hipStreamSynchronize(s));
    a.tag_base = 0;
    return fail(FORGE_HIP_ERR_HIP, "persistent decode step gave up waiting for another workgroup's data (grid not co-resident?)");
}

// Per-phase times of the last profiled step, in milliseconds: out[l][0..5] for the six phases of layer l, then
// [head, argmax].  Returns the number of entries written.
int32_t pd_phase_ms(PdState* st, std::vector<float>* out, hipStream_t s) {
    PdArgs& a = st->args;
    out->clear();
    if (!a.stamps) return FORGE_HIP_OK;
    st->stamps_host.resize(st->n_stamps);
    FH_HIP(hipMemcpyAsync(st->stamps_host.data(), a.stamps, st->n_stamps * 8, hipMemcpyDeviceToHost, s));
    FH_HIP(hipStreamSynchronize(s));
    for (uint32_t i = 0; i + 1 < st->n_stamps; i++)
        out->push_back((float)((double)(st->stamps_host[i + 1] - st->stamps_host[i]) / (double)st->wall_khz));
    return FORGE_HIP_OK;
}

}  // namespace fh

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
// starts waiting for its inputs, so HBM latency overlaps the hand-over.  Vector loads of a wave return in
// issue order on this architecture, so a wave that has weights in flight cannot see a polled element
// before those weights have landed.  The waves of a workgroup are therefore split: the first
// PD_POLL_WAVES ("pollers") fetch the phase's input first and issue their weight loads afterwards, the
// others ("streamers") issue weight loads at once and touch no other global memory until they consume
// them.  For the same reason the per-layer descriptors travel as kernel arguments (scalar loads, a
// counter of their own) and everything a wave needs besides weights (norm weights, rope factors, the
// residual) is requested before its weights are.
//
// The arithmetic is that of the separate kernels (gemv.hip, attn_decode.hip, elementwise.hip), value for
// value: the same block products, the same ordered sums, the same split boundaries and merge order.
#include <stddef.h>

#include <algorithm>
#include <memory>
#include <vector>

#include <chrono>

#include "attn_decode_math.h"
#include "common.h"
#include "device_utils.h"
#include "expf_ref.h"
#include "gemv_order.h"

namespace fh {

namespace {

constexpr int PD_THREADS = 512;
constexpr int PD_WAVES = PD_THREADS / 64;
constexpr int PD_D = 8;                       // weight units (1 KB) a wave holds in registers per round
constexpr uint32_t PD_MAX_TILE_ROWS = 128;      // = 64 PD_POLL_WAVES: the pollers own a tile's rows
constexpr uint32_t PD_LDS_BYTES = 64 * 1024;
constexpr uint32_t PD_MISC_BYTES = 2048 + 256;
constexpr int PD_POLL_WAVES = 2;              // waves that fetch a phase's input; the others stream weights
constexpr int PD_POLL_THREADS = PD_POLL_WAVES * 64;
constexpr int PD_STREAM_WAVES = PD_WAVES - PD_POLL_WAVES;
constexpr int PD_POLL_N = 20;                 // tagged elements a poller thread takes per round trip
// misc LDS (floats): [0,33) norm partial sums, [40] hint flag, [64,128) phase scratch
constexpr int PD_MISC_HINT = 40, PD_MISC_SCRATCH = 64;
// misc LDS words [PD_MISC_PT, 512): page-table entries of this workgroup's attention items, staged once per step (an item's
// key range is the same in every layer); slot (round, wave group) holds pt_cap entries
constexpr int PD_MISC_PT = 128, PD_MISC_PT_WORDS = 512 - PD_MISC_PT;
// misc LDS words [512, 576): the 32 table entries of expf_ref (ordered variants), so that an exp costs an LDS read, not a trip to memory
constexpr int PD_MISC_EXP = 512;
// `big` area: a GEMV phase's row sums sit at its start -- [rows][4] partial sums by default, [rows][nblk + 1] block products
// in the ordered variants -- and the residual row that a norm phase fetches (H floats) starts PD_X_WORDS further on.  The
// two poller waves leave a GEMV phase one after the other (the one without rows does not wait for the one that still adds
// its rows up) and the first thing a norm phase does is write that row: with the default sums (at most PD_MAX_TILE_ROWS
// rows of 4 words) the two ranges are disjoint by this offset; the ordered variants' products can reach anywhere, so they
// put a barrier in front of a norm phase's input instead.
constexpr uint32_t PD_X_WORDS = 512;
static_assert(PD_MAX_TILE_ROWS * 4 <= PD_X_WORDS, "default row sums must end before the residual row begins");
static_assert(PD_MISC_SCRATCH + 64 <= PD_MISC_PT, "phase scratch (64 floats: merge weights, argmax pairs, exp_scale chunk) ends before the page table words");

struct PdGemv {
    const uint8_t* qs;
    const uint16_t* ws;
    uint32_t K, N, nblk, U;       // U: weight units per row (Q8_0: 1024 elements, Q4_0: 2048)
    uint32_t T, ntiles;           // rows per tile, tiles (silu tiles: 32 gate rows + the matching 32 up rows)
    uint32_t inter;               // != 0: fused [gate;up] matrix, rows [0,inter) gate, [inter, 2 inter) up
    uint32_t nseg, tail_mod;
    Segment seg[3];
    uint32_t umagic;              // floor(2^32 / U) + 1: p / U = mulhi(p, umagic) for the few hundred positions of a tile (U >= 2)
};

// What differs from layer to layer: addresses only.  The shapes of the four matrices are shared.
struct PdLayer {
    const uint8_t* qs[4];      // qkv, o, gate_up, down
    const uint16_t* ws[4];
    const float* attn_norm;    // [2][H]: the layer's attention norm weights, then its feed-forward norm weights
    uint16_t* kc;
    uint16_t* vc;
};
constexpr uint32_t PD_MAX_LAYERS = 34;       // per launch: the descriptors travel as kernel arguments (4 KB in all)
constexpr uint32_t PD_MAX_SEGMENTS = 8;
enum { PD_QKV = 0, PD_O = 1, PD_GU = 2, PD_DOWN = 3, PD_LM = 4, PD_V = 5 };
// Weight formats of a phase's matrix.  Q8_0 and Q6_K units hold 32 blocks (two lanes per block), Q4_0 and Q4_K units 64 (a lane per
// block).  The K-quant matrices are re-laid out for this kernel when the model is created (pd_create):
//   Q4_K  codes: 16 bytes per 32-weight sub-block in Q4_0's byte order (byte i = weight i | weight i + 16 << 4), values 0..15;
//         one word per sub-block b: fp16 bits of d (b even) or dmin (b odd) | 6-bit scale << 16 | 6-bit minimum << 24 -- the two
//         sub-blocks of a pair belong to one super-block, so a lane gets the other half from its neighbour
//   Q6_K  codes: the 32 weights of a block as int8 (-32..31) in order (8 bits for 6: unpacking 6-bit codes cost a phase more
//         time than the bytes saved); one word per block: the int8 scales of its two halves | fp16 bits of d << 16
enum { WF_Q8 = 0, WF_Q4 = 1, WF_Q4K = 2, WF_Q6K = 3 };
__host__ __device__ constexpr bool wf_lane_per_block(int wf) { return wf == WF_Q4 || wf == WF_Q4K; }
// The (at most two) weight formats a kernel variant FMT carries code for: 0 Q8_0, 1 Q4_0, 2 both, 3 Q4_K + Q6_K,
// 4 Q4_0 + Q6_K, 5 Q8_0 + Q6_K (the last two: uniform projections under a Q6_K lm_head).
__host__ __device__ constexpr int fmt_first(int fmt) { return fmt == 0 || fmt == 2 || fmt == 5 ? WF_Q8 : fmt == 3 ? WF_Q4K : WF_Q4; }
__host__ __device__ constexpr int fmt_second(int fmt) { return fmt == 2 ? WF_Q4 : fmt >= 3 ? WF_Q6K : fmt_first(fmt); }

struct PdArgs {
    PdGemv shape[6];           // qkv, o, gate_up, down (addresses per layer, below), lm_head (addresses here) and, with split_v, v
    uint32_t n_layers, H, I, QKS, KV, heads, kv_heads, gt;   // n_layers: the layers of THIS launch, layers[0 .. n_layers)
    // A model of more layers than the descriptor array holds runs its step as several launches in a row: layers
    // [layer0, layer0 + n_layers) of total_layers; the first launch starts from the embedding row, the last one ends with
    // the lm_head and the argmax.  Tags and exchange buffers carry over from launch to launch unchanged.
    uint32_t layer0, total_layers, seg_last;
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
    uint64_t* tbm;     // [heads][nb_cap]          order-faithful attention: block maxima
    uint64_t* trec;    // [heads][nb_cap][hd + 2]  order-faithful attention: per block sum[d], then m_i, l_block
    uint32_t exact_attn, nb_cap;               // exact_attn: attention in the reference's own order (ordered kernel variants only)
    float* logits;
    uint32_t* state;   // [0] position  [1] token  [2] next token  [3] abort flag
    uint32_t tag_base, spin_limit;
    uint32_t token, token_from_arg;            // the step's input token when the host passes it with the launch
    uint32_t step_seq;                         // number of this step (never 0): left in state[4] by whoever counts the step's token
    unsigned long long* host_out;              // host-mapped {next token, launch number}: written last, or null
    uint32_t host_seq;
    // weight format of each matrix (WF_*): [PD_QKV .. PD_LM] and [PD_V].  split_v: the v rows are a matrix of their own
    // (shape[PD_V], another format than q and k: llama.cpp's K-quant recipes), its planes `v_qs_off` / `v_ws_off` bytes
    // behind the layer's q;k planes; shape[PD_QKV] then holds the q and k rows only.
    uint32_t wf[6];
    uint32_t split_v, v_qs_off, v_ws_off, v_wg0;
    uint32_t* counts;                          // u32 [vocab]: times each token id has been fed (this step's token is added here)
    const float* qkv_bias;                     // optional [layers][QKS + 2 KV]: added to q, k, v before the rotation (Qwen2)
    float penalty;                             // > 1: the argmax is taken over the penalised logits
    uint32_t window;                           // != 0: attention over the last `window` positions only (sliding window)
    PageTable pt;                              // paged KV cache (table == nullptr: flat); pt_cap: table entries an attention item may span
    uint32_t pt_cap;
    uint32_t use_hint;                         // pollers wait for one watched element before re-reading a whole buffer
    uint32_t off_act_s, off_misc, off_big;     // LDS byte offsets (activation codes sit at 0)
    unsigned long long* stamps;                // optional: wall clock at the start of every phase (workgroup 0)
    // Kernel arguments are read with scalar loads, which have their own completion counter: a wave can
    // fetch a descriptor while its weight loads are in flight without waiting for them.
    PdLayer layers[PD_MAX_LAYERS];
};
static_assert(sizeof(PdArgs) <= 4096, "kernel arguments exceed 4 KB");

// ---- plain global accesses -------------------------------------------------------------------------------
// Pointers that reach the kernel through descriptors in memory have lost their address space; a load through
// them would be a FLAT instruction, whose completion the compiler can only order with a full wait.  These
// say "global" explicitly.
typedef uint32_t pd_u32x4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ T ldg(const T* p) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (sizeof(T) == 16) {
        const pd_u32x4 v = *(const __attribute__((address_space(1))) pd_u32x4*)(uintptr_t)p;
        T r;
        __builtin_memcpy(&r, &v, 16);
        return r;
    } else {
        static_assert(sizeof(T) <= 8, "ldg: scalar or 16-byte types only");
        return *(const __attribute__((address_space(1))) T*)(uintptr_t)p;
    }
#else
    return *p;
#endif
}
template <typename T>
__device__ __forceinline__ void stg(T* p, T v) {
#if defined(__HIP_DEVICE_COMPILE__)
    *(__attribute__((address_space(1))) T*)(uintptr_t)p = v;
#else
    *p = v;
#endif
}

// ---- coherent (agent-scope, L2-bypassing) accesses ----------------------------------------------------
__device__ __forceinline__ uint64_t ldc64(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc64(uint64_t* p, uint32_t tag, uint32_t payload) {
    __hip_atomic_store(p, ((uint64_t)tag << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PdCtx {
    uint32_t tid, lane, wave, wg, G;
    uint32_t token;          // the token this step feeds
    uint32_t spin_limit;
    uint32_t* sh_abort;      // LDS
    uint32_t* abort_flag;    // global
    const uint64_t* exp_tab; // LDS: expf_ref's table (ordered variants)
};
struct LdsExpTab {
    const uint64_t* p;
    __device__ __forceinline__ uint64_t operator()(int i) const { return p[i]; }
};
template <bool kFma>
__device__ __forceinline__ float pd_expf(float x, const PdCtx& cx) { return expf_ref_with<kFma>(x, LdsExpTab{cx.exp_tab}); }

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

// Thousands of threads re-reading a buffer that is not ready yet would flood the memory fabric the weight
// stream needs.  After a first attempt that found something missing, the pollers of a workgroup therefore
// wait (on an LDS flag) until thread 0 has seen one watched element of the buffer arrive, which in a
// balanced phase is when the rest is about to.
struct Hint { const uint64_t* sentinel; volatile uint32_t* flag; };

// Up to N elements per thread: all loads are issued before any tag is looked at, so a hand-over costs one
// memory round trip however many elements a thread takes; only elements still carrying another tag are re-read.
template <int N, typename Addr>
__device__ __forceinline__ void poll_many(Addr addr, uint32_t n, uint32_t tag, uint32_t* out, const PdCtx& cx, Hint hint) {
    uint64_t w[N];
#pragma unroll
    for (int i = 0; i < N; i++) w[i] = (uint32_t)i < n ? ldc64(addr(i)) : ((uint64_t)tag << 32);
    if (hint.flag && cx.tid == 0) {
        (void)poll(hint.sentinel, tag, cx);
        *hint.flag = tag;
    }
    uint32_t spins = 0;
    bool waited = hint.flag == nullptr;
    for (;;) {
        bool ok = true;
#pragma unroll
        for (int i = 0; i < N; i++) ok = ok && (uint32_t)(w[i] >> 32) == tag;
        if (ok) break;
        if (!waited) {
            uint32_t s2 = 0;
            while (*hint.flag != tag && *cx.sh_abort == 0 && ++s2 < cx.spin_limit) __builtin_amdgcn_s_sleep(4);
            waited = true;
        } else {
            __builtin_amdgcn_s_sleep(2);
        }
        ++spins;
        if (spins > cx.spin_limit ||
            ((spins & 1023u) == 0 && __hip_atomic_load(cx.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
            *cx.sh_abort = 1;
            __hip_atomic_store(cx.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
#pragma unroll
        for (int i = 0; i < N; i++)
            if ((uint32_t)(w[i] >> 32) != tag) w[i] = ldc64(addr(i));
    }
#pragma unroll
    for (int i = 0; i < N; i++) out[i] = (uint32_t)w[i];
}

// A whole vector of `count` elements fetched by the first `nthreads` threads of the workgroup, N per thread and
// round trip; `put(index, payload)` stores each.  Threads past nthreads return at once.
template <int N, typename Put>
__device__ __forceinline__ void poll_vec(const uint64_t* base, uint32_t count, uint32_t tag, uint32_t nthreads, const PdCtx& cx,
                                         Hint hint, Put put) {
    if (cx.tid >= nthreads) return;
    for (uint32_t i0 = cx.tid; i0 < count; i0 += N * nthreads) {
        uint32_t v[N];
        const uint32_t n = (count - i0 + nthreads - 1) / nthreads;
        poll_many<N>([&](int i) { return base + i0 + (uint32_t)i * nthreads; }, n < (uint32_t)N ? n : (uint32_t)N, tag, v, cx, hint);
        hint.flag = nullptr;      // later passes: the buffer is known to be arriving
#pragma unroll
        for (int i = 0; i < N; i++)
            if (i0 + (uint32_t)i * nthreads < count) put(i0 + (uint32_t)i * nthreads, v[i]);
    }
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
// xs must already hold x[0..H); `part` is 32 floats of LDS; nw0 = norm_w[4 tid .. 4 tid + 4), requested by the
// caller before any weight load of this wave.
// ORDERED: the sum of squares in the reference's order (16 accumulators walked in sequence); otherwise every thread
// squares its own elements and the workgroup folds them (same terms, another order of addition).
template <bool ORDERED>
__device__ __forceinline__ void pd_norm_quant(float* xs, const float* __restrict__ norm_w, float4 nw0, float eps, uint32_t H,
                                              uint32_t* aq_lds, float* as_lds, float* part, const PdCtx& cx) {
    const uint32_t tid = cx.tid;
    float ss;                      // sum of squares of the row (the caller's barrier made xs visible)
    if (!ORDERED) {
        // the pollers left the squares of what they fetched as 8 partial sums (one per 16 lanes): every thread folds them
        static_assert(PD_POLL_THREADS / 16 == 8, "eight partial sums");
        float r = part[tid & 7u];
        r += __builtin_amdgcn_update_dpp(0.f, r, 0xB1, 0xF, 0xF, false);      // quad_perm [1,0,3,2]
        r += __builtin_amdgcn_update_dpp(0.f, r, 0x4E, 0xF, 0xF, false);      // quad_perm [2,3,0,1]
        r += __builtin_amdgcn_update_dpp(0.f, r, 0x141, 0xF, 0xF, false);     // row_half_mirror: lanes 0..7 <-> 7..0
        ss = r;
    } else {
      if (tid < 64) {
        // lane i < 16 owns accumulator i: x[i], x[16 + i], ... added in order with FMAs.  The reads of the next eight
        // values are issued before the current eight are consumed, so LDS latency stays off the dependent chain.
        float s = 0.f;
        const uint32_t chunks = H / 16, i16 = tid & 15u;
        uint32_t c = 0;
        if (chunks >= 8) {
            float v[8], w[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = xs[i * 16 + i16];
            for (c = 8; c + 8 <= chunks; c += 8) {
#pragma unroll
                for (int i = 0; i < 8; i++) w[i] = xs[(c + i) * 16 + i16];
#pragma unroll
                for (int i = 0; i < 8; i++) s = fmaf(v[i], v[i], s);
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = w[i];
            }
#pragma unroll
            for (int i = 0; i < 8; i++) s = fmaf(v[i], v[i], s);
        }
        for (; c < chunks; c++) { const float v = xs[c * 16 + i16]; s = fmaf(v, v, s); }
        // (p[i] + p[4+i]) + (p[8+i] + p[12+i]) for i = 0..3, then (t0 + t1) + (t2 + t3)
        const float t = (s + __shfl(s, (tid + 4) & 63, WAVE)) + (__shfl(s, (tid + 8) & 63, WAVE) + __shfl(s, (tid + 12) & 63, WAVE));
        float r = (t + __shfl(t, (tid + 1) & 63, WAVE)) + (__shfl(t, (tid + 2) & 63, WAVE) + __shfl(t, (tid + 3) & 63, WAVE));
        if (tid == 0) {
            for (uint32_t i = H / 16 * 16; i < H; i++) r = r + xs[i] * xs[i];
            part[PD_THREADS / 16] = r;
        }
      }
      __syncthreads();
      ss = part[PD_THREADS / 16];
    }
    const float inv_rms = 1.0f / sqrtf(ss / (float)H + eps);
    for (uint32_t e0 = tid * 4; e0 < H; e0 += PD_THREADS * 4) {
        const float4 xv = *reinterpret_cast<const float4*>(xs + e0);
        const float4 wv = e0 == tid * 4 ? nw0 : ldg(reinterpret_cast<const float4*>(norm_w + e0));
        const float4 v = make_float4(xv.x * inv_rms * wv.x, xv.y * inv_rms * wv.y, xv.z * inv_rms * wv.z, xv.w * inv_rms * wv.w);
        uint16_t sb;
        const uint32_t pk = quantize_block_part(v, sb);
        aq_lds[e0 / 4] = pk;
        if ((tid & 7u) == 0) as_lds[e0 / 32] = f16_bits_to_f32(sb);
    }
    __syncthreads();
}

// An already quantised vector (codes then scales, tagged) from another phase; fetched by the poller waves.
__device__ __forceinline__ void pd_load_aq(const uint64_t* t, uint32_t tag, uint32_t K, uint32_t* aq_lds, float* as_lds,
                                           float* misc, bool use_hint, const PdCtx& cx) {
    const uint32_t nq = K / 4, ns = K / 32;
    const Hint hint{t + nq + ns - 1, use_hint ? reinterpret_cast<volatile uint32_t*>(misc + PD_MISC_HINT) : nullptr};
    poll_vec<PD_POLL_N>(t, nq + ns, tag, PD_POLL_THREADS, cx, hint, [&](uint32_t i, uint32_t p) {
        if (i < nq) aq_lds[i] = p;
        else as_lds[i - nq] = f16_bits_to_f32((uint16_t)p);
    });
}

// The residual stream (tagged) into LDS as floats; fetched by the poller waves.
// `ssq` collects the squares of what this thread fetched.
__device__ __forceinline__ void pd_load_x(const uint64_t* tx, uint32_t tag, uint32_t H, float* xs, float* misc, bool use_hint,
                                          const PdCtx& cx, float& ssq) {
    const Hint hint{tx + H - 1, use_hint ? reinterpret_cast<volatile uint32_t*>(misc + PD_MISC_HINT) : nullptr};
    poll_vec<PD_POLL_N>(tx, H, tag, PD_POLL_THREADS, cx, hint, [&](uint32_t i, uint32_t p) {
        const float v = __uint_as_float(p);
        xs[i] = v;
        ssq += v * v;
    });
}

// ---- the GEMV of a phase ------------------------------------------------------------------------------
// One generic routine serves all five matrices (its code exists once: the kernel is a loop over steps, and an
// instruction cache that has to refill at every phase costs more than the branches).  What differs between
// the matrices is data: the shape, where the activation vector comes from and what happens to a finished row.
enum { PRO_NORM = 0, PRO_AQ = 1 };
enum { EPI_ROPE = 0, EPI_ADD = 1, EPI_SILU = 2, EPI_LOGITS = 3 };

struct GemvJob {
    uint32_t which;            // index of the shape in the kernel arguments (PD_QKV .. PD_LM)
    const uint8_t* qs;
    const uint16_t* ws;
    uint32_t wf;               // WF_*
    uint32_t row_off;          // EPI_ROPE: the matrix's first row is row `row_off` of q | k | v (the v matrix of a split phase)
    int pro, epi;
    const float* norm_w;       // PRO_NORM
    const uint64_t* tin;       // tagged input: residual stream (PRO_NORM) or quantised vector (PRO_AQ)
    uint32_t tin_tag;          // 0 with PRO_NORM: the input is the embedding row
    uint32_t in_len;           // elements of the input vector (= K)
    uint32_t tag_out;
    uint32_t res_tag;          // EPI_ADD: tag of the residual's current version (0: embedding row)
    uint16_t* kc;              // EPI_ROPE
    uint16_t* vc;
    const float* bias;         // EPI_ROPE, optional: this layer's q | k | v bias (emit.rs:4105-4120)
};

struct WReg { int4 v[PD_D]; uint32_t s[PD_D]; };

__device__ __forceinline__ uint32_t sgpr(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// Tells the register allocator that a weight register set holds nothing from here on (no instruction is emitted): whether a
// phase finds its first round already loaded is a run-time flag, so without this the set stays reserved through code that
// runs only when it is empty (the attention phases).
__device__ __forceinline__ void pd_forget(WReg& W) {
#pragma unroll
    for (int d = 0; d < PD_D; d++) asm volatile("" : "=v"(W.v[d].x), "=v"(W.v[d].y), "=v"(W.v[d].z), "=v"(W.v[d].w), "=v"(W.s[d]));
}

// The scalar fields of a shape, read once per phase into scalar registers.
struct Shape { uint32_t K, N, nblk, U, T, ntiles, inter, umagic; };
__device__ __forceinline__ Shape pd_shape(const PdGemv& g) {
    Shape h;
    h.K = sgpr(g.K); h.N = sgpr(g.N); h.nblk = sgpr(g.nblk); h.U = sgpr(g.U); h.T = sgpr(g.T); h.ntiles = sgpr(g.ntiles);
    h.inter = sgpr(g.inter); h.umagic = sgpr(g.umagic);
    return h;
}

// Rows of a tile: [row0, row0 + split) and, for the fused [gate;up] matrix, the matching rows `jump` further on.
// Everything here is wave-uniform and meant to live in scalar registers.
struct TilePos {
    uint32_t rows, row0, split, jump;
};
__device__ __forceinline__ TilePos pd_tile(const Shape& g, uint32_t tile) {
    TilePos t;
    if (g.inter) { t.rows = 64; t.row0 = tile * 32; t.split = 32; t.jump = g.inter - 32; }
    else { t.rows = min(g.T, g.N - tile * g.T); t.row0 = tile * g.T; t.split = 0xFFFFFFFFu; t.jump = 0; }
    return t;
}
__device__ __forceinline__ uint32_t pd_row(const TilePos& t, uint32_t lr) { return t.row0 + lr + (lr >= t.split ? t.jump : 0u); }
// position / U without a division: a scalar multiply (host: umagic = floor(2^32 / U) + 1, exact while position * U < 2^32)
__device__ __forceinline__ uint32_t pos_div_u(uint32_t p, const Shape& h) { return h.U == 1 ? p : sgpr(__umulhi(p, h.umagic)); }

// The weight streamers of a workgroup (waves PD_POLL_WAVES .. PD_WAVES-1, numbered sw = 0 .. PD_STREAM_WAVES-1) split a
// tile by rows: streamer sw takes tile rows sw, sw + PD_STREAM_WAVES, ... and walks each row's U weight units (1 KB:
// 32 Q8_0 blocks, two lanes per block, or 64 Q4_0 blocks) in order.  Position p of that walk is unit p % U of the
// wave's (p / U)-th row; a round is PD_D consecutive positions, all loaded before any is used.
// Every slot issues its two loads whatever the shape (slots past the wave's rows and lanes past a row's end re-read a
// valid address and their data is ignored): the number of loads in flight is then known at compile time and a round can
// be consumed while the next one is still arriving.
template <int WF>
__device__ __forceinline__ void pd_load_round(const GemvJob& job, const Shape& h, const TilePos& t, uint32_t round, uint32_t sw, uint32_t lane,
                                              WReg& W) {
    constexpr bool Q4 = wf_lane_per_block(WF);
    constexpr uint32_t BPU = Q4 ? 64 : 32, BPB = Q4 ? 16 : 32;
    const uint32_t U = h.U, nblk = h.nblk;
    const uint32_t lb = Q4 ? lane : lane >> 1;
    const uint32_t q = pos_div_u(round * PD_D, h);
    uint32_t j = round * PD_D - q * U, lr = sw + q * PD_STREAM_WAVES;
#pragma unroll
    for (int d = 0; d < PD_D; d++) {
        const uint32_t lrc = lr < t.rows ? lr : 0;                // a tile has at least one row
        const uint32_t b = j * BPU + lb;
        const uint32_t bc = b < nblk ? b : nblk - 1;
        const uint32_t bi = pd_row(t, lrc) * nblk + bc;             // block index in the matrix (fits 32 bits: N K / 32)
        W.v[d] = ldg(reinterpret_cast<const int4*>(job.qs + (size_t)bi * BPB + (Q4 ? 0u : (lane & 1u) * 16u)));
        if (WF == WF_Q4K || WF == WF_Q6K) W.s[d] = ldg(reinterpret_cast<const uint32_t*>(job.ws) + bi);
        else W.s[d] = ldg(job.ws + bi);
        j += 1;
        if (j == U) { j = 0; lr += PD_STREAM_WAVES; }
    }
}

// What a weight prefetch needs to know about a matrix.
struct Mat {
    uint32_t which;            // shape index; valid == false: nothing follows
    const uint8_t* qs;
    const uint16_t* ws;
    uint32_t wf;
    uint32_t wg_off;           // the matrix's tiles are spread over workgroups wg_off .. (a phase of two matrices side by side)
    bool valid;
};
template <int FMT>
__device__ __forceinline__ void pd_load_first(const PdArgs& a, const Mat& m, uint32_t wg, uint32_t sw, uint32_t lane, WReg& W) {
    const Shape h = pd_shape(a.shape[m.which]);
    if (wg >= h.ntiles) return;
    const TilePos t = pd_tile(h, wg);
    GemvJob j{};
    j.qs = m.qs; j.ws = m.ws;
    constexpr int WFA = fmt_first(FMT), WFB = fmt_second(FMT);
    if (WFB != WFA && m.wf == (uint32_t)WFB) pd_load_round<WFB>(j, h, t, 0, sw, lane, W);
    else pd_load_round<WFA>(j, h, t, 0, sw, lane, W);
}

// Exact int32 block dots on v_dot4 and one f32 product (a_s*w_s)*f32(isum) per block.
//   ORDERED   the products are parked in LDS (prod[row][block]) and summed later in the reference's order
//   otherwise each lane adds its products of a row as they come (`acc`, carried across rounds) and the wave folds
//             them when the row's last unit is done: rowsum[row].  Same terms, another order of addition.
template <int WF, bool ORDERED>
__device__ __forceinline__ void pd_compute_round(const Shape& h, const TilePos& t, uint32_t round, uint32_t sw, uint32_t lane, const WReg& W,
                                                 const uint32_t* aq_lds, const float* as_lds, const float* asum_w, float* prod, uint32_t pstride,
                                                 float& acc) {
    constexpr bool Q4 = wf_lane_per_block(WF);
    constexpr uint32_t BPU = Q4 ? 64 : 32;
    const uint32_t U = h.U, nblk = h.nblk;
    const uint32_t lb = Q4 ? lane : lane >> 1;
    const uint32_t q = pos_div_u(round * PD_D, h);
    uint32_t j = round * PD_D - q * U, lr = sw + q * PD_STREAM_WAVES;
#pragma unroll
    for (int d = 0; d < PD_D; d++) {
        if (lr < t.rows) {                                        // wave-uniform (scalar compare and branch)
            const uint32_t b = j * BPU + lb;
            const bool in = b < nblk;
            const uint32_t bs = in ? b : 0;
            if (WF == WF_Q4K || WF == WF_Q6K) {
                // K-quants: the block's term of dot_q4_k_q8_0 / dot_q6_k_q8_0 (emit.rs:3035-3306, 3553-3612) as gemv_kquant.hip forms it
                float term;
                bool mine;                                            // this lane reports the block
                if (WF == WF_Q4K) {
                    const int4 a0 = *reinterpret_cast<const int4*>(aq_lds + bs * 8);
                    const int4 a1 = *reinterpret_cast<const int4*>(aq_lds + bs * 8 + 4);
                    const int4 w = W.v[d];
                    const int m = 0x0F0F0F0F;
                    const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                    const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                    const int dot = dot16(hi, a1, dot16(lo, a0, 0));
                    const uint32_t sw_ = W.s[d];
                    const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sw_, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
                    const bool even = !(lane & 1u);
                    const float dd = f16_bits_to_f32((uint16_t)((even ? sw_ : other) & 0xFFFFu));
                    const float dmin = f16_bits_to_f32((uint16_t)((even ? other : sw_) & 0xFFFFu));
                    const float d_w = dd * (float)((sw_ >> 16) & 0xFFu), m_w = dmin * (float)(sw_ >> 24);
                    term = as_lds[bs] * (d_w * (float)dot - m_w * asum_w[bs]);      // the block's sum of codes: left there by this lane
                    mine = in;
                } else {
                    const int4 a = *reinterpret_cast<const int4*>(aq_lds + bs * 8 + (lane & 1u) * 4);
                    const int dh = in ? dot16(W.v[d], a, 0) : 0;      // this lane's 16 weights are one scale's
                    const uint32_t ww = W.s[d];
                    const float th = (float)((int)(ww << (24u - (lane & 1u) * 8u)) >> 24) * (float)dh;      // the int8 scale of this lane's half (two shifts: the signed bit-field builtin gave wrong values with a lane-dependent offset)
                    if (ORDERED) {
                        const float u = th + __builtin_amdgcn_update_dpp(0.f, th, 0xB1, 0xF, 0xF, false);       // lo + hi (even lane)
                        term = (f16_bits_to_f32((uint16_t)(ww >> 16)) * as_lds[bs]) * u;
                        mine = in && !(lane & 1u);
                    } else {
                        // each lane adds its own half (the sum of the two halves is formed with the row's other terms)
                        term = (f16_bits_to_f32((uint16_t)(ww >> 16)) * as_lds[bs]) * th;
                        mine = in;
                    }
                }
                if (ORDERED) {
                    if (mine) prod[lr * pstride + b] = term;
                } else {
                    if (mine) acc += term;
                    if (j == U - 1) {
                        float r = acc;
                        r += __builtin_amdgcn_update_dpp(0.f, r, 0xB1, 0xF, 0xF, false);     // quad_perm [1,0,3,2]
                        r += __builtin_amdgcn_update_dpp(0.f, r, 0x4E, 0xF, 0xF, false);     // quad_perm [2,3,0,1]
                        r += __builtin_amdgcn_update_dpp(0.f, r, 0x141, 0xF, 0xF, false);    // row_half_mirror
                        r += __builtin_amdgcn_update_dpp(0.f, r, 0x140, 0xF, 0xF, false);    // row_mirror
                        if ((lane & 15u) == 0) prod[lr * 4 + (lane >> 4)] = r;
                        acc = 0.f;
                    }
                }
                j += 1;
                if (j == U) { j = 0; lr += PD_STREAM_WAVES; }
                continue;
            }
            int isum;
            if (Q4) {
                const int4 a0 = *reinterpret_cast<const int4*>(aq_lds + bs * 8);
                const int4 a1 = *reinterpret_cast<const int4*>(aq_lds + bs * 8 + 4);
                const int4 w = W.v[d];
                const int m = 0x0F0F0F0F;
                const int4 lo = make_int4(w.x & m, w.y & m, w.z & m, w.w & m);
                const int4 hi = make_int4((w.x >> 4) & m, (w.y >> 4) & m, (w.z >> 4) & m, (w.w >> 4) & m);
                const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
                const int asum8 = 8 * dot16(ones, a1, dot16(ones, a0, 0));
                isum = dot16(hi, a1, dot16(lo, a0, 0)) - asum8;
            } else {
                const int4 a = *reinterpret_cast<const int4*>(aq_lds + bs * 8 + (lane & 1u) * 4);
                const int half = in ? dot16(W.v[d], a, 0) : 0;    // lanes past the row's end hold another block's data
                // the other half of the block sits in the neighbouring lane: quad_perm [1,0,3,2]
                isum = ORDERED ? half + __builtin_amdgcn_update_dpp(0, half, 0xB1, 0xF, 0xF, false) : half;
            }
            if (ORDERED) {
                if (in && (Q4 || !(lane & 1u))) prod[lr * pstride + b] = (as_lds[b] * f16_bits_to_f32((uint16_t)W.s[d])) * (float)isum;
            } else {
                if (in) acc += (as_lds[b] * f16_bits_to_f32((uint16_t)W.s[d])) * (float)isum;   // Q8_0: each lane its half block
                if (j == U - 1) {                                     // wave-uniform: the row is complete
                    // fold the 16 lanes of each DPP row (pairs, quads, halves, row); the epilogue adds the four row sums
                    float r = acc;
                    r += __builtin_amdgcn_update_dpp(0.f, r, 0xB1, 0xF, 0xF, false);     // quad_perm [1,0,3,2]
                    r += __builtin_amdgcn_update_dpp(0.f, r, 0x4E, 0xF, 0xF, false);     // quad_perm [2,3,0,1]
                    r += __builtin_amdgcn_update_dpp(0.f, r, 0x141, 0xF, 0xF, false);    // row_half_mirror
                    r += __builtin_amdgcn_update_dpp(0.f, r, 0x140, 0xF, 0xF, false);    // row_mirror
                    if ((lane & 15u) == 0) prod[lr * 4 + (lane >> 4)] = r;
                    acc = 0.f;
                }
            }
        }
        j += 1;
        if (j == U) { j = 0; lr += PD_STREAM_WAVES; }
    }
}

// ---- attention ------------------------------------------------------------------------------------------
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

// Key range [t0, t1) of attention work item number `round` of wave group `grp` of this workgroup (the items of
// attn_decode_split_kernel: kv head group x split), and which item it is.  The same in every layer of a step.
struct PdItem { uint32_t item, n_items, nbx, t0, t1, seq, start, chunk; bool on; };
template <int HD>
__device__ __forceinline__ PdItem pd_attn_item(const PdArgs& a, uint32_t pos, uint32_t round, uint32_t grp, const PdCtx& cx) {
    constexpr int LPK = HD <= 64 ? 8 : 16;
    constexpr int KPW = 64 / LPK;
    const bool dual = a.gt == 1;
    const uint32_t gsize = a.heads / a.kv_heads, gpk = gsize / a.gt;
    PdItem r;
    r.nbx = a.kv_heads * gpk; r.n_items = r.nbx * DECODE_SPLITS;
    r.seq = pos + 1;
    // attention_sliding (emit.rs:598-627): only the last `window` rows are keys (window 0: all of them)
    r.start = (a.window != 0 && r.seq > a.window) ? r.seq - a.window : 0;
    r.chunk = (r.seq - r.start + DECODE_SPLITS - 1) / DECODE_SPLITS;
    r.chunk = (r.chunk + 4 * KPW - 1) / (4 * KPW) * (4 * KPW);
    r.item = cx.wg + (dual ? 2 * round + grp : round) * cx.G;
    r.on = r.item < r.n_items;
    const uint32_t split = r.item / r.nbx;
    r.t0 = r.on ? min(r.seq, r.start + split * r.chunk) : r.seq;      // no item: an empty key range
    r.t1 = min(r.seq, r.t0 + r.chunk);
    return r;
}

// Paged cache: the table entries of every item of this workgroup, into LDS, once per step.
template <int HD>
__device__ __forceinline__ void pd_stage_pages(const PdArgs& a, uint32_t pos, uint32_t* pts, const PdCtx& cx) {
    if (!a.pt.table) return;
    const bool dual = a.gt == 1;
    const PdItem any = pd_attn_item<HD>(a, pos, 0, 0, cx);
    const uint32_t per_round = dual ? 2 * cx.G : cx.G, rounds = (any.n_items + per_round - 1) / per_round;
    for (uint32_t s = 0; s < rounds * (dual ? 2u : 1u); s++) {
        const PdItem it = pd_attn_item<HD>(a, pos, dual ? s >> 1 : s, dual ? s & 1u : 0u, cx);
        if (it.t1 <= it.t0) continue;
        const uint32_t first = it.t0 >> a.pt.shift, n = ((it.t1 - 1) >> a.pt.shift) - first + 1;
        for (uint32_t i = cx.tid; i < n && i < a.pt_cap; i += PD_THREADS) pts[s * a.pt_cap + i] = a.pt.table[first + i];
    }
}

// P2: the work items of attn_decode_split_kernel (kv head group x split), one per workgroup at a time.  The
// separate kernel gives an item four waves that each carry all `gt` query heads of the group; here wave
// 4 g + w carries head g over the keys wave w would take (same keys, same order, same merges), which
// keeps the per-thread state small.  Keys before this position come from the cache, this position's K/V
// row and q from the tagged buffers P1 filled.
template <int HD>
__device__ __forceinline__ void pd_attn_split(const PdArgs& a, const uint16_t* kc, const uint16_t* vc, uint32_t pos, uint32_t tag_in,
                                              uint32_t tag_out, float* big, const uint32_t* pts, const PdCtx& cx) {
    constexpr int LPK = HD <= 64 ? 8 : 16;
    constexpr int KPW = 64 / LPK;
    constexpr int REC = HD + 2;
    const uint32_t wave = cx.wave & 3u, lane = cx.lane;
    const uint32_t gt = a.gt, gsize = a.heads / a.kv_heads, gpk = gsize / gt;
    // With one query head per item only four of the eight waves have keys to walk: the other four then take an item of
    // their own at the same time (own LDS area, own 256 threads; the barriers are shared).
    const bool dual = gt == 1;
    const uint32_t grp = dual ? cx.wave >> 2 : 0u;
    const uint32_t ltid = dual ? (cx.tid & 255u) : cx.tid, lthreads = dual ? 256u : (uint32_t)PD_THREADS;
    constexpr int AREA = 16 * REC + 6 * HD;
    float* sh = big + grp * AREA;                                     // [4 waves][4][REC]
    float* q_lds = sh + 16 * REC;                                     // [gt][HD]
    uint32_t* kvn = reinterpret_cast<uint32_t*>(q_lds + 4 * HD);      // [2][HD] fp16 bits of this position's K and V
    const uint32_t nbx = a.kv_heads * gpk, n_items = nbx * DECODE_SPLITS;
    const uint32_t c = lane % LPK, slot = lane / LPK;
    const bool dvalid = c * 8 < HD;
    const float scale = 1.0f / sqrtf((float)HD);
    const uint32_t kv_stride = a.KV;
    const bool paged = a.pt.table != nullptr;

    // every workgroup walks the same number of rounds (the barriers inside are workgroup-wide); a wave group whose item
    // number is past the end only takes part in the barriers
    const uint32_t per_round = dual ? 2 * cx.G : cx.G;
    const uint32_t rounds = (n_items + per_round - 1) / per_round;
    for (uint32_t it = 0; it < rounds; it++) {
        const PdItem itm = pd_attn_item<HD>(a, pos, it, grp, cx);
        const uint32_t item = itm.item;
        const bool on = itm.on;
        const uint32_t bx = item % nbx, split = item / nbx;
        const uint32_t kvh = bx / gpk, sub = bx % gpk;
        const uint32_t h0 = kvh * gsize + sub * gt;
        const uint32_t t0 = itm.t0, t1 = itm.t1;
        const bool has_new = t0 <= pos && pos < t1;
        // row of the cache (pool) that holds position t of this item's range: the item's table entries sit in LDS
        const uint32_t* my_pts = pts + (dual ? 2 * it + grp : it) * a.pt_cap;
        const uint32_t pt_first = t0 >> a.pt.shift, pt_mask = (1u << a.pt.shift) - 1u;
        auto row_of = [&](uint32_t t) -> size_t {
            if (!paged) return t;
            return ((size_t)my_pts[(t >> a.pt.shift) - pt_first] << a.pt.shift) + (t & pt_mask);
        };
        // The cached K/V rows do not depend on q: the first key blocks of this wave are requested before q is awaited (loads
        // return in order, so the wait for q then costs the longer of the two latencies, not their sum).
        constexpr int UNR = 4;        // key blocks whose K/V loads are issued together
        const uint32_t tbw = t0 + wave * KPW;
        Half8 kr0[UNR], vr0[UNR];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const uint32_t t = tbw + u * 4 * KPW + slot;
            kr0[u] = Half8{{0, 0, 0, 0}};
            vr0[u] = Half8{{0, 0, 0, 0}};
            if (t < t1 && dvalid && t != pos) {
                const size_t off = row_of(t) * kv_stride + kvh * HD + c * 8;
                kr0[u] = ldg(reinterpret_cast<const Half8*>(kc + off));
                vr0[u] = ldg(reinterpret_cast<const Half8*>(vc + off));
            }
        }
        // The phase before this one is a GEMV whose rows the poller waves may still be summing out of the LDS area that q,
        // this position's K/V row and the wave records are about to be written to: in a GEMV phase only the pollers write
        // LDS inputs, here every wave does, and a streamer wave gets here as soon as it has issued its loads.  (The loads
        // above touch no LDS: they stay in front of the barrier.)
        if (it == 0) __syncthreads();
        // q is awaited even when the split is empty: the wait orders this item's records after the previous layer's readers
        for (uint32_t e = ltid; on && (e < gt * HD || (has_new && e < 2 * HD)); e += lthreads) {
            const bool need_q = e < gt * HD, need_kv = has_new && e < 2 * HD;
            const uint64_t* pq = a.tq + (size_t)h0 * HD + e;
            const uint64_t* pkv = a.tkv + (e < HD ? kvh * HD + e : a.KV + kvh * HD + (e - HD));
            uint32_t v[2];
            // one batch: an element that is not needed re-reads the needed one
            poll_many<2>([&](int i) { return (i == 0 ? need_q : !need_kv) ? pq : pkv; }, 2, tag_in, v, cx, Hint{nullptr, nullptr});
            if (need_q) q_lds[e] = __uint_as_float(v[0]);
            if (need_kv) kvn[e] = v[1];
        }
        __syncthreads();
        if (*cx.sh_abort) return;
#pragma unroll
        for (int u = 0; u < UNR; u++) {                      // this position's row arrived with q
            const uint32_t t = tbw + u * 4 * KPW + slot;
            if (t == pos && t < t1 && dvalid) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    kr0[u].w[i] = (kvn[c * 8 + 2 * i] & 0xFFFFu) | (kvn[c * 8 + 2 * i + 1] << 16);
                    vr0[u].w[i] = (kvn[HD + c * 8 + 2 * i] & 0xFFFFu) | (kvn[HD + c * 8 + 2 * i + 1] << 16);
                }
            }
        }

        // A wave carries the heads gA and gA + 2 of the group (those that exist) through ONE walk over its keys: each K/V
        // block is fetched once and used for both, every head's own sequence of operations is what a walk of its own gives.
        {
            const uint32_t gA = dual ? 0u : cx.wave >> 2;
            constexpr int NH = PD_WAVES / 4 == 2 ? 2 : 1;
            static_assert(PD_WAVES == 8, "two head slots per wave cover groups of up to four heads");
            bool has[NH];
            float qf[NH][8], acc[NH][8], m[NH], l[NH];
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
                const uint32_t g = gA + 2 * hh;
                has[hh] = g < gt;
                m[hh] = -INFINITY; l[hh] = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) { acc[hh][i] = 0.f; qf[hh][i] = (dvalid && has[hh]) ? q_lds[g * HD + c * 8 + i] : 0.f; }
            }
            for (uint32_t tb0 = tbw; tb0 < t1 && has[0]; tb0 += UNR * 4 * KPW) {
                Half8 kr[UNR], vr[UNR];
#pragma unroll
                for (int u = 0; u < UNR; u++) {
                    const uint32_t t = tb0 + u * 4 * KPW + slot;
                    kr[u] = kr0[u];
                    vr[u] = vr0[u];
                    if (tb0 != tbw && t < t1 && dvalid) {
                        if (t == pos) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                kr[u].w[i] = (kvn[c * 8 + 2 * i] & 0xFFFFu) | (kvn[c * 8 + 2 * i + 1] << 16);
                                vr[u].w[i] = (kvn[HD + c * 8 + 2 * i] & 0xFFFFu) | (kvn[HD + c * 8 + 2 * i + 1] << 16);
                            }
                        } else {
                            const size_t off = row_of(t) * kv_stride + kvh * HD + c * 8;
                            kr[u] = ldg(reinterpret_cast<const Half8*>(kc + off));
                            vr[u] = ldg(reinterpret_cast<const Half8*>(vc + off));
                        }
                    } else if (tb0 != tbw) {
                        kr[u] = Half8{{0, 0, 0, 0}};
                        vr[u] = Half8{{0, 0, 0, 0}};
                    }
                }
                // every key slot advances two keys at a time (attn_decode_math.h: the kernel pair's arithmetic)
#pragma unroll
                for (int u0 = 0; u0 < UNR; u0 += 2)
#pragma unroll
                    for (int hh = 0; hh < NH; hh++) {
                        if (!has[hh]) continue;
                        float sc[2];
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            const float d = key_dot<LPK>(qf[hh], kr[u0 + u]);
                            sc[u] = tb0 + (u0 + u) * 4 * KPW + slot < t1 ? d * scale : -INFINITY;
                        }
                        softmax_block_update<2>(m[hh], l[hh], acc[hh], sc, vr + u0);
                    }
            }
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
                if (!has[hh]) continue;
                // merge the key slots of the wave
                auto merge_with = [&](auto O) {
                    const float m2 = lane_xor<O.value>(m[hh]), l2 = lane_xor<O.value>(l[hh]);
                    float a2[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) a2[i] = lane_xor<O.value>(acc[hh][i]);
                    merge_state<8>(m[hh], l[hh], acc[hh], m2, l2, a2);
                };
                if (LPK == 8) merge_with(std::integral_constant<int, 8>{});
                merge_with(std::integral_constant<int, 16>{});
                merge_with(std::integral_constant<int, 32>{});
                if (slot == 0 && dvalid) {
                    float* rec = sh + (wave * 4 + gA + 2 * hh) * REC;
#pragma unroll
                    for (int i = 0; i < 8; i++) rec[c * 8 + i] = acc[hh][i];
                    if (c == 0) { rec[HD] = m[hh]; rec[HD + 1] = l[hh]; }
                }
            }
        }
        __syncthreads();
        // merge the four key waves: one thread per output element
        for (uint32_t e = ltid; on && e < gt * HD; e += lthreads) {
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
    float* wgt_s = misc + PD_MISC_SCRATCH;                    // [DECODE_SPLITS] + den
    float* recs = big;                           // [DECODE_SPLITS][REC]
    for (uint32_t h = cx.wg; h < a.heads; h += cx.G) {
        const uint64_t* base = a.tws + (size_t)h * DECODE_SPLITS * REC;
        poll_vec<(DECODE_SPLITS * REC + PD_THREADS - 1) / PD_THREADS>(base, DECODE_SPLITS * REC, tag_in, PD_THREADS, cx, Hint{nullptr, nullptr},
                    [&](uint32_t i, uint32_t p) { recs[i] = __uint_as_float(p); });
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
            const float amax = half_wave_max(fabsf(o));
            float inv;
            const float sc = act_scale(amax, inv);
            const uint32_t code = (uint32_t)quant_code(o * inv) & 0xFFu;
            const uint32_t pk = quad_broadcast<0>(code) | (quad_broadcast<1>(code) << 8) | (quad_broadcast<2>(code) << 16) |
                                (quad_broadcast<3>(code) << 24);
            const uint32_t e = h * HD + d;
            if ((d & 3u) == 0) stc64(a.taq + e / 4, tag_out, pk);
            if ((d & 31u) == 0) stc64(a.taq + a.QKS / 4 + e / 32, tag_out, f32_to_f16_bits(sc));
        }
        __syncthreads();
    }
}

// ---- attention in the reference's order (attention_flash, emit.rs:656-715) ---------------------------------
// The reference walks the keys in blocks of 64; per block: scores (sequential q.k sums), the block maximum, the running
// maximum m_i, exp(s - m_i), the sequential sums l_block and sum[d], and the recurrence
//     l_i = l_i * exp_scale + l_block,   acc[d] = acc[d] * exp_scale + sum[d],   exp_scale = exp(m_prev - m_i)
// which is the only part that ties the blocks together; m_i is a prefix maximum of the block maxima (order-free).  So a
// (block, head) pair is a work item of ONE WAVE here: lane = key for the scores, lane = head dim for sum[d], the weights
// and q broadcast from registers (v_readlane), no LDS.  A wave first computes the scores of all its items and publishes
// their maxima, then, per item, reads the maxima of the blocks before it, forms the weights and publishes the block's
// record; one workgroup per head then runs the recurrence over the records and quantises the row for the O projection.
// Every f32 operation has the operands and the order it has in attn_exact.hip's kernels (and in the reference).
constexpr uint32_t PX_B = 64;        // FLASH_ATTN_BLOCK_SIZE, emit.rs:201
constexpr uint32_t PX_CHUNK = 64;    // block records the recurrence takes into LDS at a time
constexpr uint32_t PX_MAX_BLOCKS = 4096;
static_assert(PX_CHUNK <= 64 && DECODE_SPLITS + 1 <= 64 && PD_WAVES * 2 <= 64, "users of the 64 floats of phase scratch in the misc area");

// What the two stages need of the kernel arguments.
struct PxArgs {
    const uint64_t* tq;
    const uint64_t* tkv;
    uint64_t* tbm;
    uint64_t* trec;
    uint64_t* taq;
    uint32_t nb_cap, heads, kv_heads, KV, QKS;
};
__device__ __forceinline__ PxArgs px_args(const PdArgs& a) {
    return PxArgs{a.tq, a.tkv, a.tbm, a.trec, a.taq, a.nb_cap, a.heads, a.kv_heads, a.KV, a.QKS};
}

template <int HD>
__device__ __forceinline__ void pd_attn_exact_blocks(const PxArgs& a, const uint16_t* kc, const uint16_t* vc, uint32_t pos, uint32_t tag_in,
                                                     uint32_t tag_out, const PdCtx& cx) {
    constexpr int REC = HD + 2;
    constexpr int NQ = (HD + 63) / 64;            // registers per lane of a head-sized vector spread over the wave
    constexpr int VB = 64 / NQ;                   // keys whose V elements a lane requests together (64 registers)
    const uint32_t lane = cx.lane;
    const uint32_t seq = pos + 1, nb = (seq + PX_B - 1) / PX_B, n_items = nb * a.heads;
    const uint32_t gsize = a.heads / a.kv_heads, kv_stride = a.KV;
    const float scale = 1.0f / sqrtf((float)HD);
    const uint32_t slots = cx.G * PD_WAVES;
    // Items in block-major order, item = block * heads + head, one per wave and pass.  What an item waits for (the maxima
    // of the earlier blocks of its head) belongs to items of a lower number, which their waves reach in the same or an
    // earlier pass; the score stage of a pass waits for nothing but q, so every pass completes.
#pragma nounroll
    for (uint32_t item = sgpr(cx.wg + cx.G * cx.wave); item < n_items; item += slots) {
        const uint32_t b = item / a.heads, h = item - b * a.heads, kvh = h / gsize;
        const uint32_t bs = b * PX_B, bl = min(PX_B, seq - bs), t = bs + lane;
        const bool has_new = b == nb - 1;                    // the block that holds this position
        // the key's row and the first V elements do not depend on q: requested first (loads return in order)
        uint4 kr[HD / 8];
#pragma unroll
        for (int c = 0; c < HD / 8; c++) kr[c] = make_uint4(0, 0, 0, 0);
        if (lane < bl && t != pos) {
            const uint16_t* krow = kc + (size_t)t * kv_stride + kvh * HD;
#pragma unroll
            for (int c = 0; c < HD / 8; c++) kr[c] = ldg(reinterpret_cast<const uint4*>(krow + c * 8));
        }
        const uint16_t* vcol = vc + (size_t)bs * kv_stride + kvh * HD + lane;
        uint16_t vv[VB][NQ];
        auto load_v = [&](uint32_t k0) {
#pragma unroll
            for (int u = 0; u < VB; u++)
#pragma unroll
                for (int j = 0; j < NQ; j++) {
                    const uint32_t bi = k0 + (uint32_t)u;
                    vv[u][j] = 0;
                    if (bi < bl && bs + bi != pos && lane + 64u * (uint32_t)j < (uint32_t)HD) vv[u][j] = ldg(vcol + (size_t)bi * kv_stride + 64 * j);
                }
        };
        // (heads of more than 64 dims: the key row alone takes 48-64 registers, the V elements are requested after the scores)
        if (NQ == 1) load_v(0);
        // q of this head, and with the last block this position's K and V rows: one round trip; a lane without an
        // element of its own re-reads its first one
        uint32_t got[3 * NQ];
        {
            const uint64_t* pq = a.tq + (size_t)h * HD;
            const uint64_t* pk = a.tkv + kvh * HD;
            const uint64_t* pv = a.tkv + a.KV + kvh * HD;
            auto addr = [&](int i) -> const uint64_t* {
                const int j = i % NQ;
                const uint32_t e = lane + 64u * (uint32_t)j < (uint32_t)HD ? lane + 64u * (uint32_t)j : lane % 32u;
                return (i < NQ || !has_new) ? pq + e : (i < 2 * NQ ? pk + e : pv + e);
            };
            poll_many<3 * NQ>(addr, 3 * NQ, tag_in, got, cx, Hint{nullptr, nullptr});
        }
        // ---- scores (sequential q.k sums, lane = key) and the block maximum
        float sum = 0.f;
        const bool mine_new = has_new && t == pos;
#pragma unroll
        for (int i = 0; i < HD; i++) {
            const float qi = __int_as_float(__builtin_amdgcn_readlane((int)got[i / 64], i % 64));
            const uint4 w4 = kr[i / 8];
            const uint32_t w = (i % 8) / 2 == 0 ? w4.x : (i % 8) / 2 == 1 ? w4.y : (i % 8) / 2 == 2 ? w4.z : w4.w;
            uint32_t kb = (i & 1) ? w >> 16 : w & 0xFFFFu;
            if (has_new) {
                const uint32_t kn = (uint32_t)__builtin_amdgcn_readlane((int)got[NQ + i / 64], i % 64);
                kb = mine_new ? kn & 0xFFFFu : kb;
            }
            sum = sum + qi * f16_bits_to_f32((uint16_t)kb);
        }
        if (NQ != 1) load_v(0);
        const float sc = lane < bl ? sum * scale : -INFINITY;
        const float mb = wave_max(sc);
        if (lane == 0) stc64(a.tbm + (size_t)h * a.nb_cap + b, tag_out, __float_as_uint(mb));
        // ---- m_i after this block: the largest block maximum so far (`if m_block > m_i { m_i = m_block }` from -inf on)
        float m = mb;
        for (uint32_t j0 = 0; j0 < b; j0 += 128) {
            uint32_t v[2];
            poll_many<2>([&](int i) { return a.tbm + (size_t)h * a.nb_cap + min(j0 + lane + 64u * (uint32_t)i, b - 1); }, 2, tag_out, v, cx,
                         Hint{nullptr, nullptr});
            m = fmaxf(m, fmaxf(__uint_as_float(v[0]), __uint_as_float(v[1])));
        }
        m = wave_max(m);
        // ---- weights, l_block and sum[d] (sequential over the block's keys; lane = head dim)
        const float e = lane < bl ? pd_expf<true>(sc - m, cx) : 0.f;
        float l_block = 0.f, acc[NQ];
#pragma unroll
        for (int j = 0; j < NQ; j++) acc[j] = 0.f;
#pragma nounroll
        for (uint32_t k0 = 0; k0 < bl; k0 += VB) {
            if (k0) load_v(k0);
#pragma unroll
            for (int u = 0; u < VB; u++) {
                const uint32_t bi = k0 + (uint32_t)u;
                if (bi < bl) {                                  // wave-uniform
                    const float eb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(e), (int)bi));
                    l_block = l_block + eb;
#pragma unroll
                    for (int j = 0; j < NQ; j++) {
                        const uint16_t hb = bs + bi == pos ? (uint16_t)got[2 * NQ + j] : vv[u][j];
                        acc[j] = acc[j] + eb * f16_bits_to_f32(hb);
                    }
                }
            }
        }
        uint64_t* rec = a.trec + ((size_t)h * a.nb_cap + b) * REC;
#pragma unroll
        for (int j = 0; j < NQ; j++)
            if (lane + 64u * (uint32_t)j < (uint32_t)HD) stc64(rec + lane + 64 * j, tag_out, __float_as_uint(acc[j]));
        if (lane == 0) { stc64(rec + HD, tag_out, __float_as_uint(m)); stc64(rec + HD + 1, tag_out, __float_as_uint(l_block)); }
    }
}

// The recurrence over a head's block records (one head per workgroup at a time), the division by l_i and the quantised row
// for the O projection (attn_exact_decode_chain_kernel's arithmetic).
template <int HD>
__device__ __forceinline__ void pd_attn_exact_chain(const PxArgs& a, uint32_t pos, uint32_t tag_in, uint32_t tag_out, float* misc, float* big,
                                                    const PdCtx& cx) {
    constexpr int REC = HD + 2;
    const uint32_t tid = cx.tid;
    const uint32_t nb = (pos + PX_B) / PX_B;
    float* es = misc + PD_MISC_SCRATCH;          // [PX_CHUNK] exp_scale of the chunk's blocks
    float* recs = big;                           // [PX_CHUNK][REC]
    __syncthreads();                             // the GEMV phase before may still be summing rows out of `big`
    for (uint32_t h = cx.wg; h < a.heads; h += cx.G) {
        float l_i = 0.f, acc = 0.f, m_prev = -INFINITY;
        for (uint32_t c0 = 0; c0 < nb; c0 += PX_CHUNK) {
            const uint32_t n = min(PX_CHUNK, nb - c0);
            const uint64_t* base = a.trec + ((size_t)h * a.nb_cap + c0) * REC;
            poll_vec<(PX_CHUNK * REC + PD_THREADS - 1) / PD_THREADS>(base, n * REC, tag_in, PD_THREADS, cx, Hint{nullptr, nullptr},
                        [&](uint32_t i, uint32_t p) { recs[i] = __uint_as_float(p); });
            __syncthreads();
            if (*cx.sh_abort) return;
            // exp_scale = exp(m_prev - m_i), m_prev = -inf before the first block
            if (tid < n) es[tid] = pd_expf<true>((tid ? recs[(tid - 1) * REC + HD] : m_prev) - recs[tid * REC + HD], cx);
            m_prev = recs[(n - 1) * REC + HD];
            __syncthreads();
            if (tid < HD) {
                // the four operations of a block form two dependent chains; the operands of the next eight blocks are read
                // from LDS while the current eight are worked through
                auto step = [&](float exp_scale, float lb, float sd) {
                    l_i = l_i * exp_scale;
                    acc = acc * exp_scale;
                    l_i = l_i + lb;
                    acc = acc + sd;
                };
                uint32_t i = 0;
                if (n >= 8) {
                    float e0[8], b0[8], s0[8], e1[8], b1[8], s1[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) { e0[k] = es[k]; b0[k] = recs[k * REC + HD + 1]; s0[k] = recs[k * REC + tid]; }
                    for (i = 8; i + 8 <= n; i += 8) {
#pragma unroll
                        for (int k = 0; k < 8; k++) { e1[k] = es[i + k]; b1[k] = recs[(i + k) * REC + HD + 1]; s1[k] = recs[(i + k) * REC + tid]; }
#pragma unroll
                        for (int k = 0; k < 8; k++) step(e0[k], b0[k], s0[k]);
#pragma unroll
                        for (int k = 0; k < 8; k++) { e0[k] = e1[k]; b0[k] = b1[k]; s0[k] = s1[k]; }
                    }
#pragma unroll
                    for (int k = 0; k < 8; k++) step(e0[k], b0[k], s0[k]);
                }
                for (; i < n; i++) step(es[i], recs[i * REC + HD + 1], recs[i * REC + tid]);
            }
            __syncthreads();
        }
        if (tid < HD) {
            const float inv_l = 1.0f / l_i;
            const float o = acc * inv_l;
            const float amax = half_wave_max(fabsf(o));
            float inv;
            const float scq = act_scale(amax, inv);
            const uint32_t code = (uint32_t)quant_code(o * inv) & 0xFFu;
            const uint32_t pk = quad_broadcast<0>(code) | (quad_broadcast<1>(code) << 8) | (quad_broadcast<2>(code) << 16) |
                                (quad_broadcast<3>(code) << 24);
            const uint32_t e = h * HD + tid;
            if ((tid & 3u) == 0) stc64(a.taq + e / 4, tag_out, pk);
            if ((tid & 31u) == 0) stc64(a.taq + a.QKS / 4 + e / 32, tag_out, f32_to_f16_bits(scq));
        }
    }
}

// ---- argmax (project.rs:501-503): the LAST index among equal maxima --------------------------------------
struct ArgPair { float v; uint32_t i; };
__device__ __forceinline__ ArgPair arg_better(ArgPair a, ArgPair b) {
    const bool take_b = (b.v > a.v) || (b.v == a.v && b.i > a.i);
    return take_b ? b : a;
}
__device__ __forceinline__ ArgPair arg_wg(ArgPair a, float* misc, const PdCtx& cx) {
    auto fold = [&](auto O) { a = arg_better(a, ArgPair{lane_xor<O.value>(a.v), lane_xor<O.value>(a.i)}); };
    fold(std::integral_constant<int, 32>{}); fold(std::integral_constant<int, 16>{}); fold(std::integral_constant<int, 8>{});
    fold(std::integral_constant<int, 4>{}); fold(std::integral_constant<int, 2>{}); fold(std::integral_constant<int, 1>{});
    ArgPair* sh = reinterpret_cast<ArgPair*>(misc + PD_MISC_SCRATCH);
    __syncthreads();
    if (cx.lane == 0) sh[cx.wave] = a;
    __syncthreads();
    ArgPair r = sh[0];
    for (int w = 1; w < PD_WAVES; w++) r = arg_better(r, sh[w]);
    return r;
}


// One GEMV phase of this workgroup: inputs, tiles, epilogues.
//   inputs    the streamers issue the first weight loads of their rows at once; the poller wave fetches the activation
//             vector (it never has weights in flight, so nothing delays what it polls)
//   tiles     compute a round from registers, issue the next round (or the next tile's first), sum, finish the rows
// One instance per kernel: the prologues and epilogues are most of the code and do not depend on the weight format, so a
// kernel that carries two formats chooses between them (a scalar branch on job.wf) only where the streamers load and
// multiply.  The step runs every phase's code once per layer: what does not fit the instruction cache is fetched again
// each time.
template <int HD, int FMT, bool ORDERED, bool PEN>
__device__ __forceinline__ void pd_gemv_phase(const PdArgs& a, const GemvJob& job, const Mat& next, bool early, WReg& W, WReg& W1, const float* emb,
                                              uint32_t pos, size_t crow, uint32_t* aq_lds, float* as_lds, float* misc, float* big, ArgPair& best,
                                              const PdCtx& cx) {
    const PdGemv& g = a.shape[job.which];
    const Shape h = pd_shape(g);
    const bool streamer = cx.wave >= (uint32_t)PD_POLL_WAVES;
    const uint32_t sw = cx.wave - PD_POLL_WAVES;
    constexpr int WFA = fmt_first(FMT), WFB = fmt_second(FMT);      // the format(s) this kernel carries
    const bool second = WFB != WFA && job.wf == (uint32_t)WFB;
    auto load_round = [&](const TilePos& tt, uint32_t r, WReg& w) {
        if (second) pd_load_round<WFB>(job, h, tt, r, sw, cx.lane, w);
        else pd_load_round<WFA>(job, h, tt, r, sw, cx.lane, w);
    };
    if (cx.wg >= h.ntiles) {
        // nothing to do here; the streamers still start on the matrix that follows
        if (streamer && next.valid) pd_load_first<FMT>(a, next, cx.wg - next.wg_off, sw, cx.lane, W);
        return;
    }
    const uint32_t pstride = h.nblk + 1;                    // +1: conflict-free column reads
    const uint32_t K = job.in_len, U = h.U;
    TilePos t = pd_tile(h, cx.wg);

    float* xs = big + PD_X_WORDS;                           // the residual row of a norm phase
    // ordered variants: the other poller wave may still be adding up the previous phase's block products, which can lie
    // where this phase's input is about to be written (see PD_X_WORDS)
    if (ORDERED && job.pro == PRO_NORM) __syncthreads();
    // ---- inputs (norm weights are requested before this wave's weights: loads return in order)
    float4 nw = make_float4(0.f, 0.f, 0.f, 0.f);
    if (job.pro == PRO_NORM && cx.tid * 4 < K) nw = ldg(reinterpret_cast<const float4*>(job.norm_w + cx.tid * 4));
    if (streamer) {
        if (!early) load_round(t, 0, W);                                  // otherwise the previous phase's tail issued them
    } else {
        float ssq = 0.f;
        if (job.pro == PRO_AQ) pd_load_aq(job.tin, job.tin_tag, K, aq_lds, as_lds, misc, a.use_hint != 0, cx);
        else if (job.tin_tag) pd_load_x(job.tin, job.tin_tag, K, xs, misc, a.use_hint != 0, cx, ssq);
        else for (uint32_t i = cx.tid; i < K; i += PD_POLL_THREADS) { const float v = emb[i]; xs[i] = v; ssq += v * v; }
        if (!ORDERED && job.pro == PRO_NORM) {
            // the pollers square what they fetched: the sum of squares needs no pass (and no barrier) of its own
            ssq += __builtin_amdgcn_update_dpp(0.f, ssq, 0xB1, 0xF, 0xF, false);      // quad_perm [1,0,3,2]
            ssq += __builtin_amdgcn_update_dpp(0.f, ssq, 0x4E, 0xF, 0xF, false);      // quad_perm [2,3,0,1]
            ssq += __builtin_amdgcn_update_dpp(0.f, ssq, 0x141, 0xF, 0xF, false);     // row_half_mirror
            ssq += __builtin_amdgcn_update_dpp(0.f, ssq, 0x140, 0xF, 0xF, false);     // row_mirror
            if ((cx.tid & 15u) == 0) misc[cx.tid >> 4] = ssq;                         // PD_POLL_THREADS / 16 = 8 partial sums
        }
    }
    __syncthreads();
    if (*cx.sh_abort) return;
    // the norm reads the row; the products use the area from its start afterwards
    if (job.pro == PRO_NORM) pd_norm_quant<ORDERED>(xs, job.norm_w, nw, a.eps, K, aq_lds, as_lds, misc, cx);
    // Q4_K: the sum of a block's activation codes (the minimum's factor) is the same for every row; a lane only ever multiplies
    // blocks lane, lane + 64, ..., so it leaves their sums in its wave's own strip of LDS once per phase (no barrier: lanes read
    // what they wrote themselves)
    const float* asum_w = nullptr;
    if (FMT == 3) {
        const uint32_t strip = (a.off_misc - a.off_act_s) / (4u * (PD_STREAM_WAVES + 1));     // floats per strip; strip 0 holds the scales
        float* mine_w = as_lds + ((streamer ? sw : 0u) + 1) * strip;
        asum_w = mine_w;
        if (streamer && !second) {
            const int4 ones = make_int4(0x01010101, 0x01010101, 0x01010101, 0x01010101);
            for (uint32_t b = cx.lane; b < h.nblk; b += 64) {
                const int4 a0 = *reinterpret_cast<const int4*>(aq_lds + b * 8);
                const int4 a1 = *reinterpret_cast<const int4*>(aq_lds + b * 8 + 4);
                mine_w[b] = (float)dot16(ones, a1, dot16(ones, a0, 0));
            }
        }
    }

    // ---- tiles
    float acc = 0.f;
#pragma nounroll
    for (uint32_t tile = cx.wg; tile < h.ntiles; tile += cx.G) {
        const uint32_t rounds = ((t.rows + PD_STREAM_WAVES - 1) / PD_STREAM_WAVES * U + PD_D - 1) / PD_D;
        const bool more = tile + cx.G < h.ntiles;
        const TilePos tn = more ? pd_tile(h, tile + cx.G) : t;
        // what the epilogue needs from global memory is requested early (by wave 0, which streams nothing, for tiles of
        // up to 64 rows)
        const bool mine = cx.tid < t.rows;
        const uint32_t row = pd_row(t, mine ? cx.tid : 0);
        const uint32_t erow = row + (job.epi == EPI_ROPE ? job.row_off : 0u);      // row of q | k | v
        float rc = 0.f, rs = 0.f;
        uint64_t res_w = 0;
        float res_e = 0.f;
        if (mine) {
            if (job.epi == EPI_ROPE && erow < a.QKS + a.KV) {
                const uint32_t d = erow < a.QKS ? erow % HD : (erow - a.QKS) % HD;
                rc = a.cos_t[(size_t)pos * (HD / 2) + d / 2];
                rs = a.sin_t[(size_t)pos * (HD / 2) + d / 2];
            } else if (job.epi == EPI_ADD) {
                if (job.res_tag) res_w = ldc64(a.tx + row);   // in flight while the tile is computed; the tag is checked below
                else res_e = emb[row];
            }
        }
        if (streamer) {
            // two register sets alternate: a round is computed while the next one is arriving; round 0 of a tile is
            // always in W
#pragma nounroll
            for (uint32_t r = 0; r < rounds; r += 2) {
                if (r + 1 < rounds) load_round(t, r + 1, W1);
                if (second) pd_compute_round<WFB, ORDERED>(h, t, r, sw, cx.lane, W, aq_lds, as_lds, asum_w, big, pstride, acc);
                else pd_compute_round<WFA, ORDERED>(h, t, r, sw, cx.lane, W, aq_lds, as_lds, asum_w, big, pstride, acc);
                if (r + 1 < rounds) {
                    if (r + 2 < rounds) load_round(t, r + 2, W);
                    if (second) pd_compute_round<WFB, ORDERED>(h, t, r + 1, sw, cx.lane, W1, aq_lds, as_lds, asum_w, big, pstride, acc);
                    else pd_compute_round<WFA, ORDERED>(h, t, r + 1, sw, cx.lane, W1, aq_lds, as_lds, asum_w, big, pstride, acc);
                }
            }
        }
        __syncthreads();
        // While the pollers (which own every row of a tile: at most 64 PD_POLL_WAVES rows) sum and finish the rows, the
        // streamers start on what comes next: the next tile, or the next matrix.  Issuing a wave's loads takes about as
        // long as the data takes to arrive (the memory pipeline holds only so many misses), so it must not sit between
        // the products and the sums.
        if (streamer) {
            if (more) load_round(tn, 0, W);
            else if (next.valid) pd_load_first<FMT>(a, next, cx.wg - next.wg_off, sw, cx.lane, W);
        }
        if (cx.tid < ((t.rows + 63u) & ~63u)) {
            float v = 0.f;
            if (mine) v = ORDERED ? ordered_sum_words(big + cx.tid * pstride, h.nblk, segment_row_is_dot1(row, g.seg, g.nseg, g.tail_mod)) : (big[cx.tid * 4] + big[cx.tid * 4 + 1]) + (big[cx.tid * 4 + 2] + big[cx.tid * 4 + 3]);
            if (job.epi == EPI_ROPE) {
                if (PEN && job.bias && mine) v = v + job.bias[erow];     // the kernel variant with the optional extras carries it
                // rope (emit.rs:508-528): rows 2i, 2i+1 of a head sit in neighbouring lanes
                const float other = lane_xor<1>(v);
                if (mine) {
                    if (erow < a.QKS + a.KV) {
                        const float o = (erow & 1u) ? other * rs + v * rc : v * rc - other * rs;
                        if (erow < a.QKS) {
                            stc64(a.tq + erow, job.tag_out, __float_as_uint(o));
                        } else {
                            const uint16_t hb = f32_to_f16_bits(o);
                            stg(job.kc + crow * a.KV + (erow - a.QKS), hb);
                            stc64(a.tkv + (erow - a.QKS), job.tag_out, hb);
                        }
                    } else {
                        const uint16_t hb = f32_to_f16_bits(v);
                        stg(job.vc + crow * a.KV + (erow - a.QKS - a.KV), hb);
                        stc64(a.tkv + a.KV + (erow - a.QKS - a.KV), job.tag_out, hb);
                    }
                }
            } else if (job.epi == EPI_ADD) {
                if (mine) {
                    float res = res_e;
                    if (job.res_tag)
                        res = __uint_as_float((uint32_t)(res_w >> 32) == job.res_tag ? (uint32_t)res_w : poll(a.tx + row, job.res_tag, cx));
                    stc64(a.tx + row, job.tag_out, __float_as_uint(res + v));       // residual_add, emit.rs:455-459
                }
            } else if (job.epi == EPI_SILU) {
                // lanes 0..31 hold the gate rows of inter indices [32 tile, +32), lanes 32..63 the up rows
                const uint32_t lr = cx.tid;
                const float ux = lane_xor<32>(v);         // lanes 0..31: the up row of the same inter index
                if (lr < 32) {
                    // silu_mul, emit.rs:380-386; the C library's expf bit for bit where the reference order is asked for
                    const float o = (v / (1.0f + (ORDERED ? pd_expf<true>(-v, cx) : __expf(-v)))) * ux;
                    const float amax = half_wave_max(fabsf(o));
                    float inv;
                    const float sc = act_scale(amax, inv);
                    const uint32_t code = (uint32_t)quant_code(o * inv) & 0xFFu;
                    const uint32_t pk = quad_broadcast<0>(code) | (quad_broadcast<1>(code) << 8) | (quad_broadcast<2>(code) << 16) |
                                        (quad_broadcast<3>(code) << 24);
                    if ((lr & 3u) == 0) stc64(a.taq2 + tile * 8 + lr / 4, job.tag_out, pk);
                    if (lr == 0) stc64(a.taq2 + a.I / 4 + tile, job.tag_out, f32_to_f16_bits(sc));
                }
            } else {
                if (mine) {
                    a.logits[row] = v;
                    // apply_repeat_penalty (project.rs:505-513) before the argmax.  The thread that owns the row of the
                    // token being fed is the only one in the grid to touch that counter: it adds this step's occurrence.
                    // (A kernel built without PEN counts the token in its last stage and never reads the counters.)
                    if (PEN) {
                        const bool fed = row == cx.token;
                        const uint32_t c = a.counts[row] + (fed ? 1u : 0u);
                        if (fed) { a.counts[row] = c; a.state[4] = a.step_seq; }      // so that a step that gives up later can be undone
                        if (a.penalty > 1.0f) v = repeat_penalised(v, c, a.penalty);
                    }
                    best = arg_better(best, ArgPair{v, row});
                }
            }
        }
        // before the next tile's products overwrite this tile's; after the last tile nothing touches LDS until the
        // next phase's inputs are in (the streamers only issue loads, the pollers write what they poll), so the pollers
        // need not wait for the streamers' loads to be issued
        if (more) __syncthreads();
        t = tn;
    }
}

// FMT: which weight formats the kernel carries code for (fmt_first / fmt_second) -- a kernel that fits the instruction
// cache matters more than one binary for all models.
// ORD: the GEMV rows are summed in the reference's block order (bit-identical to the kernel sequence) instead of as the
// products come.
// XA (ordered variants only): the attention walks the keys in the reference's own order instead of in splits; each kernel
// carries one of the two.
template <int HD, int FMT, bool ORD, bool PEN, bool XA>
__global__ __launch_bounds__(PD_THREADS) void decode_step_kernel(PdArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    __shared__ uint32_t sh_abort;
    uint32_t* aq_lds = reinterpret_cast<uint32_t*>(smem);
    float* as_lds = reinterpret_cast<float*>(smem + a.off_act_s);
    float* misc = reinterpret_cast<float*>(smem + a.off_misc);
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
    if (cx.tid == 0) { sh_abort = 0; reinterpret_cast<uint32_t*>(misc)[PD_MISC_HINT] = 0; }
    cx.exp_tab = reinterpret_cast<const uint64_t*>(misc + PD_MISC_EXP);
    if (ORD && cx.tid < 32) reinterpret_cast<uint64_t*>(misc + PD_MISC_EXP)[cx.tid] = expf_detail::tab((int)cx.tid);
    __syncthreads();

    const uint32_t pos = a.state[0], token = a.token_from_arg ? a.token : a.state[1];
    const size_t crow = paged_row(a.pt, pos);        // row of the cache (pool) that this position's K and V go to
    uint32_t* pts = reinterpret_cast<uint32_t*>(misc) + PD_MISC_PT;
    pd_stage_pages<HD>(a, pos, pts, cx);             // published by the first barrier of the first phase
    const float* emb = a.embed + (size_t)token * a.H;
    cx.token = token;
    const uint32_t L = a.n_layers;
    ArgPair best{-INFINITY, 0};
    WReg W, W1;
    bool early = false;

    // steps 4 l + {0: qkv, 1: attention then o, 2: gate/up, 3: down}; step 4 L: lm_head.  Phase instance k of this
    // launch carries tag tag_base + k: per layer 1 qkv, 2 attention split, 3 attention merge, 4 o, 5 gate/up, 6 down.
    const uint32_t n_steps = 4 * L + (a.seg_last ? 1u : 0u);
#pragma nounroll
    for (uint32_t step = 0; step < n_steps; step++) {
        // The thread's number is read afresh in every step: otherwise LDS addresses derived from it are worked out
        // ahead of the loop, where they do not all fit the 256 registers, and the ones that were parked in scratch
        // memory came back through a load and a wait for every outstanding load in front of the norm's LDS writes.
        asm volatile("" : "+v"(cx.tid), "+v"(cx.lane));
        const bool is_lm = step == 4 * L;
        const uint32_t l = is_lm ? L - 1 : step >> 2, ph = is_lm ? 4u : (step & 3u);     // l: index into a.layers
        const uint32_t lg = a.layer0 + l;                     // the layer's number in the model
        const uint32_t base = a.tag_base + 6 * lg;
        const uint32_t x_in = lg ? base : 0;                 // tag of x entering the layer (0: still the embedding row)
        if (ph == 1) {
            if (a.stamps && cx.wg == 0 && cx.tid == 0) a.stamps[6 * lg + 1] = wall_clock64();
            if (XA) {
                pd_attn_exact_blocks<HD>(px_args(a), a.layers[l].kc, a.layers[l].vc, pos, base + 1, base + 2, cx);
                if (a.stamps && cx.wg == 0 && cx.tid == 0) a.stamps[6 * lg + 2] = wall_clock64();
                pd_attn_exact_chain<HD>(px_args(a), pos, base + 2, base + 3, misc, big, cx);
                __syncthreads();
                if (sh_abort) return;
            } else {
                pd_attn_split<HD>(a, a.layers[l].kc, a.layers[l].vc, pos, base + 1, base + 2, big, pts, cx);
                if (sh_abort) return;
                if (a.stamps && cx.wg == 0 && cx.tid == 0) a.stamps[6 * lg + 2] = wall_clock64();
                pd_attn_combine<HD>(a, base + 2, base + 3, misc, big, cx);
                if (sh_abort) return;
            }
            pd_forget(W);          // the O projection loads its first round itself (`early` is false here)
            pd_forget(W1);
        }
        if (a.stamps && cx.wg == 0 && cx.tid == 0) {
            static const int slot[5] = {0, 3, 4, 5, 6};
            a.stamps[6 * lg + slot[ph]] = wall_clock64();
        }
        const bool vside = FMT == 3 && a.split_v && cx.wg >= a.v_wg0;
        GemvJob job;
        job.which = ph;
        job.qs = is_lm ? a.shape[PD_LM].qs : a.layers[l].qs[ph];
        job.ws = is_lm ? a.shape[PD_LM].ws : a.layers[l].ws[ph];
        job.wf = a.wf[is_lm ? (uint32_t)PD_LM : ph];
        job.row_off = 0;
        Mat next;
        {
            const uint32_t ns = step + 1;
            const bool n_lm = ns == 4 * L;
            const uint32_t nl = n_lm ? L - 1 : ns >> 2, nph = n_lm ? 4u : (ns & 3u);
            // the O projection follows attention, which needs every wave at once: its (few) weights are loaded when it starts
            next.valid = ns < n_steps && nph != 1;
            next.which = nph;
            next.qs = n_lm ? a.shape[PD_LM].qs : a.layers[next.valid ? nl : 0].qs[nph & 3u];
            next.ws = n_lm ? a.shape[PD_LM].ws : a.layers[next.valid ? nl : 0].ws[nph & 3u];
            next.wf = a.wf[n_lm ? (uint32_t)PD_LM : nph];
            next.wg_off = 0;
            if (FMT == 3 && a.split_v && nph == 0 && !n_lm && vside) {      // this workgroup's share of the q;k;v phase is the v matrix
                next.which = PD_V;
                next.qs += a.v_qs_off;
                next.ws = reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(next.ws) + a.v_ws_off);
                next.wf = a.wf[PD_V];
                next.wg_off = a.v_wg0;
            }
        }
        job.pro = (ph == 1 || ph == 3) ? PRO_AQ : PRO_NORM;
        job.epi = ph == 0 ? EPI_ROPE : ph == 2 ? EPI_SILU : ph == 4 ? EPI_LOGITS : EPI_ADD;
        job.norm_w = ph == 0 ? a.layers[l].attn_norm : ph == 2 ? a.layers[l].attn_norm + a.H : a.final_norm;
        job.tin = ph == 1 ? a.taq : ph == 3 ? a.taq2 : a.tx;
        job.tin_tag = ph == 0 ? x_in : ph == 1 ? base + 3 : ph == 2 ? base + 4 : ph == 3 ? base + 5 : base + 6;
        job.in_len = ph == 1 ? a.QKS : ph == 3 ? a.I : a.H;
        job.tag_out = is_lm ? 0 : base + (ph == 0 ? 1u : ph == 1 ? 4u : ph == 2 ? 5u : 6u);
        job.res_tag = ph == 1 ? x_in : base + 4;
        job.kc = a.layers[l].kc;
        job.bias = (PEN && a.qkv_bias && ph == 0) ? a.qkv_bias + (size_t)lg * (a.QKS + 2 * a.KV) : nullptr;
        job.vc = a.layers[l].vc;
        // v in another format than q and k (K-quant recipes): two matrices side by side in the q;k;v phase.  The first v_wg0
        // workgroups take the q;k rows, the others the v rows, each side tiling its matrix over its own share of the grid;
        // both read the same normed row and write q | k | v rows under the same tag, so nothing changes for the phases
        // around them.  (One call for every case: the phase's code is in the kernel once.)
        PdCtx side = cx;
        if (FMT == 3 && a.split_v && ph == 0) {
            if (vside) {
                side.wg = cx.wg - a.v_wg0; side.G = cx.G - a.v_wg0;
                job.which = PD_V;
                job.qs += a.v_qs_off;
                job.ws = reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(job.ws) + a.v_ws_off);
                job.wf = a.wf[PD_V];
                job.row_off = a.QKS + a.KV;
            } else {
                side.G = a.v_wg0;
            }
        }
        pd_gemv_phase<HD, FMT, ORD, PEN>(a, job, next, early, W, W1, emb, pos, crow, aq_lds, as_lds, misc, big, best, side);
        early = next.valid;
        if (sh_abort) return;
    }

    if (!a.seg_last) return;          // the next launch goes on from the exchange buffers
    // ---------------- argmax (and the position / token advance) ----------------
    const uint32_t th = a.tag_base + 6 * a.total_layers + 1;
    best = arg_wg(best, misc, cx);
    if (cx.tid == 0) {
        stc64(a.tpart + 2 * cx.wg, th, __float_as_uint(best.v));
        stc64(a.tpart + 2 * cx.wg + 1, th, best.i);
    }
    if (a.stamps && cx.wg == 0 && cx.tid == 0) a.stamps[6 * a.total_layers + 1] = wall_clock64();
    if (cx.wg == 0) {
        ArgPair p{-INFINITY, 0};
        for (uint32_t w = cx.tid; w < cx.G; w += PD_THREADS) {
            uint32_t v[2];
            poll_many<2>([&](int i) { return a.tpart + 2 * w + (uint32_t)i; }, 2, th, v, cx, Hint{nullptr, nullptr});
            p = arg_better(p, ArgPair{__uint_as_float(v[0]), v[1]});
        }
        p = arg_wg(p, misc, cx);
        if (sh_abort) return;
        if (cx.tid == 0) {
            a.state[2] = p.i;
            a.state[1] = p.i;
            a.state[0] = pos + 1;
            if (!PEN) a.counts[token] += 1;          // nobody read the counters in this launch
            if (a.stamps) a.stamps[6 * a.total_layers + 2] = wall_clock64();
            // the host may be spinning on this word instead of waiting for the stream
            if (a.host_out)
                __hip_atomic_store(a.host_out, ((unsigned long long)a.host_seq << 32) | p.i, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
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
    bool q4 = false, lmq4 = false, kquant = false, ordered = false, cooperative = true;
    bool lmk = false;              // a K-quant (Q6_K) lm_head over Q8_0 / Q4_0 projections
    size_t tagged_bytes = 0;
    void* tagged_base = nullptr;
    std::vector<unsigned long long> stamps_host;
    std::vector<PdLayer> all_layers;           // every layer's descriptors; a launch takes a slice of at most PD_MAX_LAYERS
    int wall_khz = 0;
    unsigned long long* host_out = nullptr;    // pinned, mapped into the device's address space
    unsigned long long* host_out_dev = nullptr;
    uint32_t seq = 0;
    ~PdState() {
        for (void* p : owned) (void)hipFree(p);
        if (host_out) (void)hipHostFree(host_out);
    }
};

namespace {

// K-quant matrices as this kernel's weight units (layouts at WF_*), from the planes gemv_kquant.hip keeps.  One thread per
// (row, 32-weight block).
__global__ __launch_bounds__(256) void pd_repack_q4k_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, uint32_t K, uint64_t total,
                                                          uint8_t* __restrict__ codes, uint32_t* __restrict__ words) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // n * nblk + b
    if (id >= total) return;
    const uint32_t nblk = K / 32;
    const uint64_t n = id / nblk;
    const uint32_t b = (uint32_t)(id % nblk), sb = b >> 3, j = b & 7, c = j >> 1;
    const uint8_t* mp = meta + (n * (K / 256) + sb) * 16;
    const uint8_t* s12 = mp + 4;
    uint32_t sc, mn;                                                       // get_scale_min_k4, emit.rs:3013-3021
    if (j < 4) { sc = s12[j] & 63u; mn = s12[j + 4] & 63u; }
    else {
        sc = (s12[j + 4] & 0x0Fu) | ((s12[j - 4] >> 6) << 4);
        mn = (s12[j + 4] >> 4) | ((s12[j] >> 6) << 4);
    }
    const uint32_t h16 = (b & 1u) ? (uint32_t)(mp[2] | (mp[3] << 8)) : (uint32_t)(mp[0] | (mp[1] << 8));     // odd: dmin, even: d
    words[id] = h16 | (sc << 16) | (mn << 24);
    // sub-block j = 2c + hi: weight i is the low (hi = 0) or high nibble of byte 32 c + i of the super-block
    const uint8_t* src = qs + (n * (K / 256) + sb) * 128 + 32 * c;
    const uint32_t sh = (j & 1) * 4;
    uint8_t* dst = codes + id * 16;
    for (uint32_t i = 0; i < 16; i++) dst[i] = (uint8_t)(((src[i] >> sh) & 15u) | (((src[i + 16] >> sh) & 15u) << 4));
}

__global__ __launch_bounds__(256) void pd_repack_q6k_kernel(const uint8_t* __restrict__ qs, const uint8_t* __restrict__ meta, uint32_t K, uint64_t total,
                                                          uint8_t* __restrict__ codes, uint32_t* __restrict__ words) {
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;       // n * nblk + b
    if (id >= total) return;
    const uint32_t nblk = K / 32;
    const uint64_t n = id / nblk;
    const uint32_t b = (uint32_t)(id % nblk), sb = b >> 3, jb = b & 7, h = jb >> 2, r = jb & 3;
    const uint8_t* sp = qs + (n * (K / 256) + sb) * 192;
    const uint8_t* mp = meta + (n * (K / 256) + sb) * 32;
    // block 4h + r of the super-block: r = 0, 1 the low nibbles of ql[64h + 32r ..], r = 2, 3 the high nibbles of
    // ql[64h + 32(r - 2) ..]; bit pair r of qh[32h ..]
    const uint8_t* ql = sp + 64 * h + 32 * (r & 1);
    const uint8_t* qh = sp + 128 + 32 * h;
    const uint32_t nib_shift = (r >> 1) * 4, pair_shift = 2 * r;
    uint8_t* dst = codes + id * 32;
    for (uint32_t e = 0; e < 32; e++) {
        const int c = (int)(((ql[e] >> nib_shift) & 15u) | (((qh[e] >> pair_shift) & 3u) << 4)) - 32;       // the weight: -32..31
        dst[e] = (uint8_t)(int8_t)c;
    }
    // the int8 scales of the block's two halves, then d (fp16)
    words[id] = (uint32_t)mp[2 * jb] | ((uint32_t)mp[2 * jb + 1] << 8) | ((uint32_t)mp[16] << 16) | ((uint32_t)mp[17] << 24);
}

// Bytes of the two planes of an [N][K] K-quant matrix in the kernel's layout.
size_t pd_kq_code_bytes(uint32_t wdtype, uint64_t N, uint32_t K) { return wdtype == FORGE_HIP_Q4_K ? N * (K / 32) * 16 : N * (K / 32) * 32; }
size_t pd_kq_word_bytes(uint32_t, uint64_t N, uint32_t K) { return N * (K / 32) * 4; }

void pd_repack_kquant(const QWeight& w, uint8_t* codes, uint8_t* words, hipStream_t s) {
    const uint64_t total = (uint64_t)w.N * (w.K / 32);
    const uint32_t grid = (uint32_t)((total + 255) / 256);
    const uint8_t* meta = reinterpret_cast<const uint8_t*>(w.scales);
    if (w.wdtype == FORGE_HIP_Q4_K) fh::launch(pd_repack_q4k_kernel, grid, 256, 0, s, w.qs, meta, w.K, total, codes, reinterpret_cast<uint32_t*>(words));
    else fh::launch(pd_repack_q6k_kernel, grid, 256, 0, s, w.qs, meta, w.K, total, codes, reinterpret_cast<uint32_t*>(words));
}

uint32_t wf_of(uint32_t wdtype) {
    return wdtype == FORGE_HIP_Q8_0 ? WF_Q8 : wdtype == FORGE_HIP_Q4_0 ? WF_Q4 : wdtype == FORGE_HIP_Q4_K ? WF_Q4K : WF_Q6K;
}

// Tile plan of one matrix: rows per tile so that the tiles spread evenly over the grid and a tile's block
// products fit `big_bytes` of LDS.  Returns false if they cannot.
bool plan_gemv(const QWeight& w, uint32_t inter, uint32_t nseg, const Segment* seg, uint32_t tail_mod, uint32_t grid,
               uint32_t big_bytes, PdGemv* g) {
    g->qs = w.qs; g->ws = w.scales; g->K = w.K; g->N = w.N; g->nblk = w.K / 32;
    const uint32_t epu = (w.wdtype == FORGE_HIP_Q8_0 || w.wdtype == FORGE_HIP_Q6_K) ? 1024 : 2048;
    g->U = (w.K + epu - 1) / epu;
    g->umagic = g->U >= 2 ? (uint32_t)(0x100000000ull / g->U) + 1u : 0u;
    g->inter = inter;
    g->nseg = nseg; g->tail_mod = tail_mod;
    for (uint32_t i = 0; i < nseg; i++) g->seg[i] = seg[i];
    // rows in the four-accumulator order are the last len % tail_mod of each chunk: a matrix without any (the usual case:
    // every chunk a multiple of tail_mod rows) tells the kernel so by carrying no segments, and no row asks
    bool any_dot1 = false;
    for (uint32_t i = 0; i < nseg && tail_mod; i++) {
        const Segment& sg = seg[i];
        if (!sg.chunk) any_dot1 = any_dot1 || sg.len % tail_mod != 0;
        else any_dot1 = any_dot1 || sg.chunk % tail_mod != 0 || (sg.len % sg.chunk) % tail_mod != 0;
    }
    if (!any_dot1) g->nseg = 0;
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

template <int HD, bool ORD, bool PEN, bool XA>
const void* pd_kernel_ord(const PdState* st) {
    // (K-quant models always run the variant with the optional extras)
    if (st->kquant) return reinterpret_cast<const void*>(decode_step_kernel<HD, 3, ORD, true, XA>);
    if (st->lmk) return st->q4 ? reinterpret_cast<const void*>(decode_step_kernel<HD, 4, ORD, true, false>)
                               : reinterpret_cast<const void*>(decode_step_kernel<HD, 5, ORD, true, false>);
    if (st->q4 != st->lmq4) return reinterpret_cast<const void*>(decode_step_kernel<HD, 2, ORD, PEN, XA>);
    return st->q4 ? reinterpret_cast<const void*>(decode_step_kernel<HD, 1, ORD, PEN, XA>)
                  : reinterpret_cast<const void*>(decode_step_kernel<HD, 0, ORD, PEN, XA>);
}
// The repeat penalty (lm_head epilogue) and the QKV bias (qkv epilogue) are code of their own: the default kernel is
// built without them (the ordered variants always carry them).
template <int HD>
const void* pd_kernel(const PdState* st) {
    if (st->ordered) return st->args.exact_attn ? pd_kernel_ord<HD, true, true, true>(st) : pd_kernel_ord<HD, true, true, false>(st);
    return (st->args.penalty > 1.0f || st->args.qkv_bias) ? pd_kernel_ord<HD, false, true, false>(st) : pd_kernel_ord<HD, false, false, false>(st);
}
template <int HD>
hipError_t launch_pd_hd(const PdState* st, hipStream_t s) {
    void* kargs[] = {const_cast<PdArgs*>(&st->args)};
    if (!st->cooperative) return hipLaunchKernel(pd_kernel<HD>(st), dim3(st->grid), dim3(PD_THREADS), kargs, st->lds, s);
    return hipLaunchCooperativeKernel(pd_kernel<HD>(st), dim3(st->grid), dim3(PD_THREADS), kargs, st->lds, s);
}

const void* pd_kernel_for(const PdState* st) {
    return st->hd == 64 ? pd_kernel<64>(st) : st->hd == 96 ? pd_kernel<96>(st) : pd_kernel<128>(st);
}

}  // namespace

void pd_destroy(PdState* st) { delete st; }

// Kernel launches of one decode step: 1, or one per slice of PD_MAX_LAYERS layers for a deeper model.
uint32_t pd_launches_per_step(const PdState* st) { return (st->args.total_layers + PD_MAX_LAYERS - 1) / PD_MAX_LAYERS; }

// Plans the persistent decode step for a model.  Leaves *out null (and returns OK) when the shape or the
// device is outside what the kernel covers; the caller then keeps the multi-kernel step.
int32_t pd_create(const forge_hip_config& c, const std::vector<PdLayerIn>& layers, const QWeight& lm_head, const float* embed,
                  const float* final_norm, const float* cos_t, const float* sin_t, float* logits, uint32_t* state, uint32_t* counts,
                  const float* qkv_bias, PdState** out) {
    *out = nullptr;
    // The order-faithful mode can run as this kernel too: the ordered variant with the attention phases in the reference's
    // order.  It is bit-identical to the kernel sequence but not faster across shapes (Llama-3.2-1B shape at 2.5k context:
    // 925 against 935 us per token; 3B: 2125 against 2118; SmolLM2-135M: 1204 against 1041 -- the ordered norm and row sums
    // cost every GEMV phase 1-2 us that the separate kernels hide behind their launches), so for Q8_0 / Q4_0 models the sequence
    // stays the default and FORGE_HIP_PD_EXACT=1 asks for the kernel.  Models of K-quant matrices, whose sequence has a launch
    // per projection group (117 per token at 16 layers), take the kernel by default (Q4_K_M recipe, 1B shape: 928 against 989
    // us per token); FORGE_HIP_PD_EXACT=0 keeps their sequence.  A window (attention_sliding: another algorithm) and caches of
    // more than 4096 blocks always keep the sequence.
    const bool exact = (c.flags & FORGE_HIP_FLAG_EXACT) != 0;
    const uint32_t nb_cap = (c.max_seq + PX_B - 1) / PX_B;
    if (exact && (c.sliding_window != 0 || nb_cap > PX_MAX_BLOCKS)) return FORGE_HIP_OK;
    if (exact) {
        const char* e = getenv("FORGE_HIP_PD_EXACT");
        const bool kquant_model = !layers.empty() && layers[0].q != nullptr;
        if (!(e ? e[0] == '1' : kquant_model)) return FORGE_HIP_OK;
    }
    if (c.head_dim != 64 && c.head_dim != 96 && c.head_dim != 128) return FORGE_HIP_OK;
    int dev = 0, coop = 0, cus = 0, khz = 0;
    FH_HIP(hipGetDevice(&dev));
    FH_HIP(hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev));
    FH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    FH_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    if (!coop || cus < 1) return FORGE_HIP_OK;

    std::unique_ptr<PdState> st(new PdState());
    PdArgs& a = st->args;
    a.qkv_bias = qkv_bias;                 // selects the kernel variant: before the residency check below
    const uint32_t H = c.hidden, I = c.inter, hd = c.head_dim, QKS = c.heads * hd, KV = c.kv_heads * hd;
    const uint32_t kmax = std::max(std::max(H, I), QKS);
    const uint32_t gsize = c.heads / c.kv_heads;
    a.gt = gsize % 4 == 0 ? 4 : gsize % 3 == 0 ? 3 : gsize % 2 == 0 ? 2 : 1;
    st->grid = (uint32_t)cus;
    st->hd = hd;
    st->q4 = c.wdtype == FORGE_HIP_Q4_0;
    st->lmq4 = c.lm_head_dtype == FORGE_HIP_Q4_0;
    // a model of K-quant matrices: every projection and the lm_head Q4_K or Q6_K, q and k of one format, gate and up too
    if (layers.empty()) return FORGE_HIP_OK;
    st->kquant = layers[0].q != nullptr;
    // Q8_0 / Q4_0 projections under a Q6_K lm_head (fast mode only, like the all-K-quant models)
    st->lmk = !st->kquant && lm_head.kquant();
    if (st->lmk && (lm_head.wdtype != FORGE_HIP_Q6_K || exact)) return FORGE_HIP_OK;
    if (st->kquant) {
        const PdLayerIn& in = layers[0];
        const QWeight* all[7] = {in.q, in.k, in.v, in.o, in.gate, in.up, in.down};
        for (const QWeight* w : all)
            if (!w || !w->kquant()) return FORGE_HIP_OK;
        if (!lm_head.kquant() || in.q->wdtype != in.k->wdtype || in.gate->wdtype != in.up->wdtype) return FORGE_HIP_OK;
    }
    st->wall_khz = khz;
    // FORGE_HIP_PD_ORDERED=1: GEMV rows summed in the reference's block order, bit-identical to the kernel sequence
    { const char* e = getenv("FORGE_HIP_PD_ORDERED"); st->ordered = exact || (e && e[0] == '1'); }
    a.exact_attn = exact ? 1u : 0u;
    a.nb_cap = nb_cap;

    // LDS: activation codes | activation scales | misc | big
    a.off_act_s = round_up(kmax, 16);
    // K-quant models: one more strip of kmax / 32 floats per streaming wave behind the scales (each wave's sums of activation codes)
    a.off_misc = a.off_act_s + round_up(kmax / 32 * 4, 16) * (st->kquant ? PD_STREAM_WAVES + 1 : 1);
    a.off_big = a.off_misc + PD_MISC_BYTES;
    if (a.off_big + 4096 > PD_LDS_BYTES) return FORGE_HIP_OK;
    const uint32_t big = PD_LDS_BYTES - 64 - a.off_big;
    const uint32_t attn_bytes = (a.gt == 1 ? 2 : 1) * (16 * (hd + 2) + 6 * hd) * 4;      // two items at a time when a group has one head
    if ((H + 32 + PD_X_WORDS) * 4 > big || attn_bytes > big || DECODE_SPLITS * (hd + 2) * 4 > big) return FORGE_HIP_OK;
    if (exact && (PX_CHUNK * (hd + 2) * 4 > big || c.heads > st->grid * PD_WAVES)) return FORGE_HIP_OK;
    st->lds = a.off_big + big;

    if (layers.empty() || layers.size() > PD_MAX_LAYERS * PD_MAX_SEGMENTS) return FORGE_HIP_OK;
    QWeight lm_res = lm_head;                     // K-quant models: the lm_head in the kernel's layout
    if (st->kquant) {
        const PdLayerIn& in0 = layers[0];
        // descriptors of the matrices as the kernel sees them: q;k (with v behind it when v shares their format), o, gate;up, down
        const bool split_v = in0.v->wdtype != in0.q->wdtype;
        auto desc = [](uint32_t wdtype, uint32_t K, uint32_t N) { QWeight d; d.wdtype = wdtype; d.K = K; d.N = N; return d; };
        const QWeight dqk = desc(in0.q->wdtype, H, split_v ? QKS + KV : QKS + 2 * KV), dv = desc(in0.v->wdtype, H, KV),
                      dgu = desc(in0.gate->wdtype, H, 2 * I);
        // a v matrix of its own shares the grid with q;k in proportion to the bytes each side streams
        uint32_t g_qk = st->grid;
        if (split_v) {
            if (st->grid < 2) return FORGE_HIP_OK;
            const double bq = (double)(pd_kq_code_bytes(dqk.wdtype, dqk.N, H) + pd_kq_word_bytes(dqk.wdtype, dqk.N, H)),
                         bv = (double)(pd_kq_code_bytes(dv.wdtype, dv.N, H) + pd_kq_word_bytes(dv.wdtype, dv.N, H));
            g_qk = (uint32_t)((double)st->grid * bq / (bq + bv) + 0.5);
            g_qk = std::min(std::max(g_qk, 1u), st->grid - 1);
        }
        a.v_wg0 = g_qk;
        if (!plan_gemv(dqk, 0, 0, nullptr, 4, g_qk, big, &a.shape[PD_QKV]) || !plan_gemv(*in0.o, 0, 0, nullptr, 4, st->grid, big, &a.shape[PD_O]) ||
            !plan_gemv(dgu, I, 0, nullptr, 4, st->grid, big, &a.shape[PD_GU]) || !plan_gemv(*in0.down, 0, 0, nullptr, 4, st->grid, big, &a.shape[PD_DOWN]) ||
            (split_v && !plan_gemv(dv, 0, 0, nullptr, 4, st->grid - g_qk, big, &a.shape[PD_V])) ||
            !plan_gemv(lm_head, 0, 0, nullptr, 4, st->grid, big, &a.shape[PD_LM]))
            return FORGE_HIP_OK;
        for (int k = 0; k < 6; k++) { a.shape[k].qs = nullptr; a.shape[k].ws = nullptr; }
        a.wf[PD_QKV] = wf_of(dqk.wdtype); a.wf[PD_O] = wf_of(in0.o->wdtype); a.wf[PD_GU] = wf_of(dgu.wdtype);
        a.wf[PD_DOWN] = wf_of(in0.down->wdtype); a.wf[PD_LM] = wf_of(lm_head.wdtype); a.wf[PD_V] = wf_of(dv.wdtype);
        a.split_v = split_v ? 1u : 0u;
        // the layout per layer: codes [q | k | v], words [q | k | v], then o, gate;up, down each
        const size_t cq = pd_kq_code_bytes(in0.q->wdtype, QKS, H), ck = pd_kq_code_bytes(in0.k->wdtype, KV, H), cv = pd_kq_code_bytes(in0.v->wdtype, KV, H);
        const size_t wq = pd_kq_word_bytes(in0.q->wdtype, QKS, H), wk = pd_kq_word_bytes(in0.k->wdtype, KV, H), wv = pd_kq_word_bytes(in0.v->wdtype, KV, H);
        a.v_qs_off = (uint32_t)(cq + ck);
        a.v_ws_off = (uint32_t)(wq + wk);
        if (cq + ck + cv > 0xFFFFFFFFull) return FORGE_HIP_OK;
        for (size_t l = 0; l < layers.size(); l++) {
            const PdLayerIn& in = layers[l];
            const QWeight* all[7] = {in.q, in.k, in.v, in.o, in.gate, in.up, in.down};
            for (int i = 0; i < 7; i++)
                if (!all[i] || all[i]->wdtype != (i == 0 || i == 1 ? in0.q->wdtype : i == 2 ? in0.v->wdtype : i == 3 ? in0.o->wdtype : i < 6 ? in0.gate->wdtype : in0.down->wdtype))
                    return FORGE_HIP_OK;
            st->all_layers.emplace_back();
            PdLayer& L = st->all_layers.back();
            auto plane = [&](size_t n) -> uint8_t* { return n ? dev_alloc<uint8_t>(n, st->owned) : nullptr; };
            uint8_t* c_qkv = plane(cq + ck + cv);
            uint8_t* w_qkv = plane(wq + wk + wv);
            const size_t co = pd_kq_code_bytes(in.o->wdtype, H, QKS), wo = pd_kq_word_bytes(in.o->wdtype, H, QKS);
            const size_t cg = pd_kq_code_bytes(in.gate->wdtype, I, H), wg = pd_kq_word_bytes(in.gate->wdtype, I, H);
            const size_t cd = pd_kq_code_bytes(in.down->wdtype, H, I), wd = pd_kq_word_bytes(in.down->wdtype, H, I);
            uint8_t *c_o = plane(co), *w_o = plane(wo), *c_gu = plane(2 * cg), *w_gu = plane(2 * wg), *c_d = plane(cd), *w_d = plane(wd);
            if (!c_qkv || !c_o || !c_gu || !c_d || (wq + wk + wv && !w_qkv) || (wo && !w_o) || (wg && !w_gu) || (wd && !w_d))
                return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory for the K-quant weight units");
            pd_repack_kquant(*in.q, c_qkv, w_qkv, nullptr);
            pd_repack_kquant(*in.k, c_qkv + cq, w_qkv ? w_qkv + wq : nullptr, nullptr);
            pd_repack_kquant(*in.v, c_qkv + cq + ck, w_qkv ? w_qkv + wq + wk : nullptr, nullptr);
            pd_repack_kquant(*in.o, c_o, w_o, nullptr);
            pd_repack_kquant(*in.gate, c_gu, w_gu, nullptr);
            pd_repack_kquant(*in.up, c_gu + cg, w_gu ? w_gu + wg : nullptr, nullptr);
            pd_repack_kquant(*in.down, c_d, w_d, nullptr);
            L.qs[0] = c_qkv; L.ws[0] = reinterpret_cast<const uint16_t*>(w_qkv);
            L.qs[1] = c_o; L.ws[1] = reinterpret_cast<const uint16_t*>(w_o);
            L.qs[2] = c_gu; L.ws[2] = reinterpret_cast<const uint16_t*>(w_gu);
            L.qs[3] = c_d; L.ws[3] = reinterpret_cast<const uint16_t*>(w_d);
            if (in.ffn_norm != in.attn_norm + H) return FORGE_HIP_OK;          // the kernel finds the second norm H floats behind the first
            L.attn_norm = in.attn_norm; L.kc = in.kc; L.vc = in.vc;
        }
        {
            const size_t cl = pd_kq_code_bytes(lm_head.wdtype, c.vocab, H), wl = pd_kq_word_bytes(lm_head.wdtype, c.vocab, H);
            uint8_t* c_l = dev_alloc<uint8_t>(cl, st->owned);
            uint8_t* w_l = wl ? dev_alloc<uint8_t>(wl, st->owned) : nullptr;
            if (!c_l || (wl && !w_l)) return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory for the K-quant weight units");
            pd_repack_kquant(lm_head, c_l, w_l, nullptr);
            lm_res.qs = c_l;
            lm_res.scales = reinterpret_cast<uint16_t*>(w_l);
            a.shape[PD_LM].qs = c_l;
            a.shape[PD_LM].ws = reinterpret_cast<const uint16_t*>(w_l);
        }
        FH_HIP(hipDeviceSynchronize());
        FH_HIP(hipGetLastError());
    } else {
        const PdLayerIn& in = layers[0];
        const uint32_t wt = c.wdtype;
        Segment sq[3] = {make_segment(wt, H, 0, QKS, false), make_segment(wt, H, QKS, KV, false), make_segment(wt, H, QKS + KV, KV, false)};
        Segment so[1] = {make_segment(wt, QKS, 0, H, false)};
        Segment sg[2] = {make_segment(wt, H, 0, I, false), make_segment(wt, H, I, I, false)};
        Segment sd[1] = {make_segment(wt, I, 0, H, false)};
        if (!plan_gemv(*in.qkv, 0, 3, sq, 4, st->grid, big, &a.shape[PD_QKV]) || !plan_gemv(*in.o, 0, 1, so, 4, st->grid, big, &a.shape[PD_O]) ||
            !plan_gemv(*in.gate_up, I, 2, sg, 4, st->grid, big, &a.shape[PD_GU]) ||
            !plan_gemv(*in.down, 0, 1, sd, 4, st->grid, big, &a.shape[PD_DOWN]))
            return FORGE_HIP_OK;
        for (int k = 0; k < 4; k++) { a.shape[k].qs = nullptr; a.shape[k].ws = nullptr; }
    }
    for (size_t l = 0; l < layers.size() && !st->kquant; l++) {
        const PdLayerIn& in = layers[l];
        st->all_layers.emplace_back();
        PdLayer& L = st->all_layers.back();
        const QWeight* w[4] = {in.qkv, in.o, in.gate_up, in.down};
        for (int k = 0; k < 4; k++) { L.qs[k] = w[k]->qs; L.ws[k] = w[k]->scales; }
        if (in.ffn_norm != in.attn_norm + H) return FORGE_HIP_OK;          // the kernel finds the second norm H floats behind the first
            L.attn_norm = in.attn_norm; L.kc = in.kc; L.vc = in.vc;
    }
    if (!st->kquant) {
        a.wf[PD_QKV] = a.wf[PD_O] = a.wf[PD_GU] = a.wf[PD_DOWN] = a.wf[PD_V] = st->q4 ? WF_Q4 : WF_Q8;
        a.split_v = 0; a.v_qs_off = 0; a.v_ws_off = 0; a.v_wg0 = 0;
        if (st->lmk) {
            // a Q6_K lm_head over Q8_0 / Q4_0 projections: the matrix in the kernel's layout, its rows summed in block order
            if (!plan_gemv(lm_head, 0, 0, nullptr, 4, st->grid, big, &a.shape[PD_LM])) return FORGE_HIP_OK;
            const size_t cl = pd_kq_code_bytes(lm_head.wdtype, c.vocab, H), wl = pd_kq_word_bytes(lm_head.wdtype, c.vocab, H);
            uint8_t* c_l = dev_alloc<uint8_t>(cl, st->owned);
            uint8_t* w_l = dev_alloc<uint8_t>(wl, st->owned);
            if (!c_l || !w_l) return fail(FORGE_HIP_ERR_HIP, "persistent decode: out of device memory for the K-quant weight units");
            pd_repack_kquant(lm_head, c_l, w_l, nullptr);
            FH_HIP(hipDeviceSynchronize());
            FH_HIP(hipGetLastError());
            a.shape[PD_LM].qs = c_l;
            a.shape[PD_LM].ws = reinterpret_cast<const uint16_t*>(w_l);
            a.wf[PD_LM] = WF_Q6K;
        } else {
            Segment sl[1] = {make_segment(c.lm_head_dtype, H, 0, c.vocab, true)};
            if (!plan_gemv(lm_head, 0, 1, sl, 4, st->grid, big, &a.shape[PD_LM])) return FORGE_HIP_OK;
            a.wf[PD_LM] = st->lmq4 ? WF_Q4 : WF_Q8;
        }
    }
    (void)lm_res;
    // cooperative residency: one workgroup per CU must fit
    {
        int per_cu = 0;
        hipError_t e = hipErrorInvalidValue;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, pd_kernel_for(st.get()), PD_THREADS, st->lds);
        if (e != hipSuccess || per_cu < 1) { (void)hipGetLastError(); return FORGE_HIP_OK; }
    }

    a.total_layers = (uint32_t)layers.size();
    a.layer0 = 0;
    a.n_layers = std::min<uint32_t>(a.total_layers, PD_MAX_LAYERS);
    a.seg_last = a.n_layers == a.total_layers;
    for (uint32_t l = 0; l < a.n_layers; l++) a.layers[l] = st->all_layers[l];
    a.H = H; a.I = I; a.QKS = QKS; a.KV = KV; a.heads = c.heads; a.kv_heads = c.kv_heads;
    a.eps = c.rms_eps;
    a.window = c.sliding_window;
    a.pt = PageTable{}; a.pt_cap = 0;
    a.embed = embed; a.final_norm = final_norm; a.cos_t = cos_t; a.sin_t = sin_t;
    a.logits = logits; a.state = state;
    a.counts = counts; a.penalty = 1.0f;
    // one allocation for all tagged buffers (zeroed: tag 0 is never expected)
    const size_t n_tx = H, n_tq = QKS, n_tkv = 2 * (size_t)KV, n_tws = (size_t)c.heads * DECODE_SPLITS * (hd + 2),
                 n_taq = QKS / 4 + QKS / 32, n_taq2 = I / 4 + I / 32, n_tpart = 2 * (size_t)st->grid;
    const size_t n_tbm = exact ? (size_t)c.heads * nb_cap : 0, n_trec = n_tbm * (hd + 2);
    const size_t total = n_tx + n_tq + n_tkv + n_tws + n_taq + n_taq2 + n_tpart + n_tbm + n_trec;
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
    a.tpart = t; t += n_tpart;
    a.tbm = t; t += n_tbm;
    a.trec = t;
    a.tag_base = 0;
    // FORGE_HIP_PD_TAG_START: start the tag sequence elsewhere (a test starts it just below the point where it is rewound)
    { const char* e = getenv("FORGE_HIP_PD_TAG_START"); if (e) a.tag_base = (uint32_t)strtoul(e, nullptr, 0); }
    a.spin_limit = 400000;
    // FORGE_HIP_PD_SPIN_LIMIT: how often a wait re-reads before the workgroup gives up (a test sets it to 1 to walk the
    // give-up path: every wait in the kernel is bounded by it, so the kernel still ends normally)
    { const char* e = getenv("FORGE_HIP_PD_SPIN_LIMIT"); if (e && atoi(e) > 0) a.spin_limit = (uint32_t)atoi(e); }
    // The watcher (one thread polls one element of a buffer, the other pollers wait for its word in LDS before they re-read
    // what they missed) pays on narrow models, where a phase is nothing but its hand-over (hidden 576: +2 %); from a hidden
    // size of 1024 up the pollers re-read on their own (1B +1.0 %, 3B +1.7 %, 8B +0.9 % over the watcher).
    // FORGE_HIP_PD_HINT=0 / 1 forces either.
    { const char* e = getenv("FORGE_HIP_PD_HINT"); a.use_hint = e ? (e[0] == '0' ? 0 : 1) : (a.H < 1024 ? 1 : 0); }
    a.token = 0; a.token_from_arg = 0; a.host_out = nullptr; a.host_seq = 0;
    // All workgroups are co-resident by construction (one per CU, checked above), and every wait in the kernel is
    // bounded, so an ordinary launch is enough; it costs ~7 us less per step than a cooperative one.
    // FORGE_HIP_PD_COOP=1 asks for the cooperative launch (which re-checks residency on every launch).
    { const char* e = getenv("FORGE_HIP_PD_COOP"); st->cooperative = e && e[0] == '1'; }
    if (!(getenv("FORGE_HIP_PD_HOSTWORD") && getenv("FORGE_HIP_PD_HOSTWORD")[0] == '0')) {
        void* hp = nullptr;
        if (hipHostMalloc(&hp, 64, hipHostMallocMapped) == hipSuccess) {
            void* dp = nullptr;
            if (hipHostGetDevicePointer(&dp, hp, 0) == hipSuccess) {
                st->host_out = reinterpret_cast<unsigned long long*>(hp);
                st->host_out_dev = reinterpret_cast<unsigned long long*>(dp);
                st->host_out[0] = 0;
            } else {
                (void)hipGetLastError();
                (void)hipHostFree(hp);
            }
        } else {
            (void)hipGetLastError();
        }
    }
    st->tags_per_launch = 6 * a.total_layers + 1;
    st->n_stamps = 6 * a.total_layers + 3;
    a.stamps = nullptr;
    *out = st.release();
    return FORGE_HIP_OK;
}

// Paged KV cache (pt.table == nullptr: back to the flat cache).  The kernel keeps the table entries of a workgroup's
// attention items in a fixed LDS area: fails if `max_seq` rows in pages this small would need more.
int32_t pd_set_kv_pages(PdState* st, PageTable pt, uint32_t max_seq) {
    PdArgs& a = st->args;
    if (!pt.table) { a.pt = PageTable{}; a.pt_cap = 0; return FORGE_HIP_OK; }
    const bool dual = a.gt == 1;
    const uint32_t n_items = a.kv_heads * ((a.heads / a.kv_heads) / a.gt) * DECODE_SPLITS;
    const uint32_t per_round = (dual ? 2u : 1u) * st->grid, slots = (n_items + per_round - 1) / per_round * (dual ? 2u : 1u);
    const uint32_t max_chunk = round_up((max_seq + DECODE_SPLITS - 1) / DECODE_SPLITS, 32);       // 4 KPW <= 32 keys
    const uint32_t cap = (max_chunk >> pt.shift) + 2;
    if (slots * cap > (uint32_t)PD_MISC_PT_WORDS)
        return fail(FORGE_HIP_ERR_INVALID, "kv pages: pages this small need more page-table entries per attention item than the decode kernel keeps (" +
                                               std::to_string(slots * cap) + " > " + std::to_string(PD_MISC_PT_WORDS) + "): use larger pages");
    a.pt = pt; a.pt_cap = cap;
    return FORGE_HIP_OK;
}

// Polls before a workgroup gives up (0: the default).  A test knob: 1 makes every wait fail that is not satisfied at once.
void pd_set_poll_limit(PdState* st, uint32_t n) { st->args.spin_limit = n ? n : 400000u; }

// A penalty > 1 selects the kernel variant that carries the penalty code: check that it, too, fits one workgroup per CU.
int32_t pd_set_repeat_penalty(PdState* st, float penalty) {
    const float old = st->args.penalty;
    st->args.penalty = penalty;
    int per_cu = 0;
    const hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, pd_kernel_for(st), PD_THREADS, st->lds);
    if (e != hipSuccess || per_cu < 1) {
        (void)hipGetLastError();
        st->args.penalty = old;
        return fail(FORGE_HIP_ERR_HIP, "persistent decode: the kernel variant with the repeat penalty does not fit the device");
    }
    return FORGE_HIP_OK;
}

// Enqueue one decode step at the position in `state` for `token` (travels as a kernel argument).  With `profile`
// the kernel also records the wall clock at the start of every phase.
int32_t pd_enqueue(PdState* st, bool profile, uint32_t token, hipStream_t s) {
    PdArgs& a = st->args;
    a.token = token;
    a.token_from_arg = 1;
    a.step_seq = a.step_seq + 1 ? a.step_seq + 1 : 1;
    a.host_out = st->host_out_dev;
    if (a.host_out) a.host_seq = ++st->seq;
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
    hipError_t e = hipSuccess;
    for (uint32_t l0 = 0; l0 < a.total_layers && e == hipSuccess; l0 += PD_MAX_LAYERS) {
        if (a.total_layers > PD_MAX_LAYERS) {       // one launch per slice of layers (the arguments are copied at launch)
            a.layer0 = l0;
            a.n_layers = std::min<uint32_t>(PD_MAX_LAYERS, a.total_layers - l0);
            a.seg_last = l0 + a.n_layers == a.total_layers;
            for (uint32_t l = 0; l < a.n_layers; l++) a.layers[l] = st->all_layers[l0 + l];
        }
        e = st->hd == 64 ? launch_pd_hd<64>(st, s) : st->hd == 96 ? launch_pd_hd<96>(st, s) : launch_pd_hd<128>(st, s);
    }
    a.stamps = keep;
    if (e != hipSuccess) return fail(FORGE_HIP_ERR_HIP, std::string("persistent decode launch: ") + hipGetErrorString(e));
    a.tag_base += st->tags_per_launch;
    return FORGE_HIP_OK;
}

// Waits for the next token of the step enqueued last by watching the word the kernel writes into host memory
// when its result is final (a few microseconds earlier than the stream reports completion, and without a
// device-to-host copy).  Returns false if the word is not in use or did not arrive in time: the caller then
// waits for the stream and reads the state from the device.
bool pd_wait_token(PdState* st, uint32_t* next) {
    if (!st->host_out || !st->args.host_out) return false;
    const volatile unsigned long long* w = st->host_out;
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spin = 0;; spin++) {
        const unsigned long long v = *w;
        if ((uint32_t)(v >> 32) == st->seq) { *next = (uint32_t)v; return true; }
        if ((spin & 1023u) == 1023u &&
            std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(200)) return false;
    }
}

// After the stream has drained: did every workgroup get through?  (state[3] is the abort flag.)
int32_t pd_after_sync(PdState* st, uint32_t abort_flag, hipStream_t s) {
    if (!abort_flag) return FORGE_HIP_OK;
    PdArgs& a = st->args;
    // The step did not happen: the position was not advanced (the kernel does that last), the cache row of this position
    // will be written again; what may have happened is the count of the step's token (the kernel variant with the repeat
    // penalty counts it in its lm_head phase).  It says so in state[4]: take the count back.
    {
        uint32_t seq = 0;
        FH_HIP(hipMemcpyAsync(&seq, a.state + 4, 4, hipMemcpyDeviceToHost, s));
        FH_HIP(hipStreamSynchronize(s));
        if (seq == a.step_seq && a.counts) {
            uint32_t c = 0;
            FH_HIP(hipMemcpyAsync(&c, a.counts + a.token, 4, hipMemcpyDeviceToHost, s));
            FH_HIP(hipStreamSynchronize(s));
            if (c) c -= 1;
            FH_HIP(hipMemcpyAsync(a.counts + a.token, &c, 4, hipMemcpyHostToDevice, s));
            FH_HIP(hipStreamSynchronize(s));
        }
    }
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

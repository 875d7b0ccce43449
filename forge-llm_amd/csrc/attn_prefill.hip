// Batched-prefill causal attention (attention_flash_batch, emit.rs:754-883) over an fp16 KV
// cache, with both matrix products on fp16 MFMA (v_mfma_f32_32x32x16_f16) and the online
// softmax in f32.
//
// Workgroup = 8 waves = 128 consecutive queries of one head: four groups of 32 queries, each shared by two
// waves that take one half (32 keys) of every key tile and merge their (max, sum, output) once at the end, so
// that the longest chain of dependent tile steps (the last query tile's) is worked on by twice the waves.
// K/V are streamed in tiles of 64 keys through two LDS buffers (K row-major, V transposed so that
// the contraction index of P.V is contiguous per lane; a thread fetches 4 head dims of two
// consecutive keys and writes the pairs as dwords).  Scores stay in the base-2 domain
// (s * scale * log2 e) so that the exponential is one v_exp_f32 after one FMA; keys are masked only in
// tiles that reach past the wave's first query, and the accumulators are rescaled only when some
// query of the wave saw a new maximum.
//
// Both products are computed transposed, S^T = K Q^T and O^T = V^T P^T.  In the 32x32 MFMA
// result layout a lane then owns ONE query (column = lane%32) and 16 keys (or 16 head dims),
// so the softmax row statistics are per-lane scalars (plus one exchange with lane^32), and
// the exponentiated scores are already in the register layout the second MFMA wants for
// its B operand.
#include "common.h"
#include "device_utils.h"

namespace fh {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int QW = 32;        // queries per wave pair
constexpr int QB = 128;       // queries per workgroup
constexpr int KT = 64;        // keys per tile
constexpr int AP_THREADS = 512;   // the 8-wave form; the 4-wave form runs 256

// QUANT: instead of f32 rows the kernel writes what the o projection's GEMM reads, the activation quantiser's int8
// codes oq[M][heads*HD] and fp16 scales osc[M][heads*HD/32] of the same values (a 32-element block is one 32-wide
// head_dim tile of one query: 16 values in this lane, 16 in lane ^ 32).
// WIN: sliding-window attention (attention_sliding_batch, emit.rs:907-1046): the query at position p sees the keys
// [max(0, p - window + 1), p]; key tiles that lie before the window of the workgroup's first query are never loaded.
// KH: 32-key halves of a tile that one wave works.  1 = the 8-wave form described above (two waves share a query group and
// merge at the end: twice the waves on the longest chain, for short sequences); 2 = 4 waves, each takes its 32 queries
// through all 64 keys of a tile: two independent score tiles per step to overlap, one maximum / rescale / lane exchange
// per 64 keys, no merge.
template <int HD, bool QUANT, bool WIN, int KH>
__global__ __launch_bounds__(AP_THREADS / KH) __attribute__((amdgpu_waves_per_eu(2)))
void attn_prefill_kernel(const float* __restrict__ q, const uint16_t* __restrict__ kc_flat, const uint16_t* __restrict__ vc_flat,
                         float* __restrict__ out, uint32_t q_stride, uint32_t out_stride, uint32_t M, uint32_t base_pos,
                         uint32_t heads, uint32_t kv_heads, int8_t* __restrict__ oq, uint16_t* __restrict__ osc, uint32_t window,
                         PageTable pt) {
    constexpr int KS = HD + 8;    // K tile row stride (halfs): 16-byte pad
    constexpr int VS = KT + 4;    // V^T tile row stride (halfs): 8-byte pad
    constexpr int KTOTAL = KT * HD / 8;          // 16-byte pieces of K per tile
    constexpr int VTOTAL = KT * HD / 8;          // (key pair, 4 dims) items of V per tile
    constexpr int NT = AP_THREADS / KH;           // threads of the workgroup
    constexpr int KPIECES = (KTOTAL + NT - 1) / NT, VITEMS = (VTOTAL + NT - 1) / NT;
    constexpr int DG = HD / 4;    // groups of 4 head dims
    constexpr int NS = HD / 16;   // MFMA k-steps over head_dim
    constexpr int ND = HD / 32;   // 32-wide head_dim tiles of the output
    constexpr int KBYTES = KT * KS * 2, VBYTES = HD * VS * 2;
    constexpr int MERGE_FLOATS = 2 + ND * 16;    // per lane: m, l and the output accumulators
    static_assert(KH == 2 || 2 * (KBYTES + VBYTES) >= 4 * 64 * MERGE_FLOATS * 4, "the merge reuses the tile buffers");
    // two tiles each: the loads of tile t+1 are written while tile t is read, one barrier per tile
    __shared__ __attribute__((aligned(16))) uint8_t smem[2 * (KBYTES + VBYTES)];
    auto Ks = [&](uint32_t buf) { return reinterpret_cast<_Float16*>(smem + buf * KBYTES); };
    auto Vt = [&](uint32_t buf) { return reinterpret_cast<_Float16*>(smem + 2 * KBYTES + buf * VBYTES); };

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t qg = KH == 1 ? wave >> 1 : wave, kh = KH == 1 ? (wave & 1) : 0;   // query group of 32, (first) half of every key tile
    const uint32_t lq = lane & 31, lh = lane >> 5;
    // tile-major order, heaviest (latest) query tiles first: they stream the most keys, and whatever does not fit the
    // machine at once is the light end, handed out as the first workgroups finish
    const uint32_t head = blockIdx.x % heads, kvh = head / (heads / kv_heads);
    const uint32_t ntq = gridDim.x / heads;
    const uint32_t qtile = ntq - 1 - blockIdx.x / heads;
    const uint32_t q0 = qtile * QB;
    const uint32_t kv_stride = kv_heads * HD;
    const uint32_t seq_total = base_pos + M;
    // scores are kept in the base-2 domain: s * (scale * log2 e), so that exp is the bare v_exp_f32
    const float c2 = (1.0f / sqrtf((float)HD)) * 1.4426950408889634f;

    // ---- Q fragment (B operand of S^T = K Q^T): lane (lq, lh) holds q[row][16 s + 8 lh + 0..7]
    const uint32_t qrow = q0 + qg * QW + lq;
    const uint32_t qpos = base_pos + qrow;
    v8h qf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        if (qrow < M) {
            const float4* p = reinterpret_cast<const float4*>(q + (size_t)qrow * q_stride + head * HD + 16 * s + 8 * lh);
            float4 a = p[0], b = p[1];
            qf[s] = (v8h){(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w,
                          (_Float16)b.x, (_Float16)b.y, (_Float16)b.z, (_Float16)b.w};
        } else {
            qf[s] = (v8h){0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    v16f oacc[ND];
#pragma unroll
    for (int d = 0; d < ND; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[d][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const uint32_t wg_max_pos = base_pos + min(q0 + QB, M) - 1;
    const uint32_t ntiles = wg_max_pos / KT + 1;
    const uint32_t wave_max_pos = base_pos + min(q0 + qg * QW + QW, M) - 1;   // may underflow if the group is empty
    const uint32_t wave_min_pos = base_pos + q0 + qg * QW;                    // position of the group's first query
    const bool wave_active = q0 + qg * QW < M;
    // first key any query of the workgroup / of this wave's group may see
    const uint32_t wg_lo = (WIN && base_pos + q0 + 1 > window) ? base_pos + q0 + 1 - window : 0;
    const uint32_t wave_lo = (WIN && wave_min_pos + 1 > window) ? wave_min_pos + 1 - window : 0;
    const uint32_t tile0 = wg_lo / KT;

    int4 kreg[KPIECES];
    uint2 va[VITEMS], vb[VITEMS];
    auto load_tile = [&](uint32_t kt) {
        // a paged cache: a tile of 64 keys lies within one page (pages are multiples of 64 rows), `shift` rows further on
        const ptrdiff_t shift = pt.table ? (ptrdiff_t)paged_row(pt, kt * KT) - (ptrdiff_t)(kt * KT) : 0;
        const uint16_t* kc = kc_flat + shift * (ptrdiff_t)kv_stride;
        const uint16_t* vc = vc_flat + shift * (ptrdiff_t)kv_stride;
#pragma unroll
        for (int i = 0; i < KPIECES; i++) {
            const uint32_t idx = tid + NT * i, key = idx / (HD / 8), dc = idx % (HD / 8);
            const uint32_t t = kt * KT + key;
            kreg[i] = (idx < KTOTAL && t < seq_total) ? *reinterpret_cast<const int4*>(kc + (size_t)t * kv_stride + kvh * HD + dc * 8)
                                                     : make_int4(0, 0, 0, 0);
        }
        // V: an item is 4 head dims of two consecutive keys (seq rows t, t+1)
#pragma unroll
        for (int i = 0; i < VITEMS; i++) {
            const uint32_t idx = tid + NT * i, kp = idx / DG, dg = idx % DG;
            const uint32_t t = kt * KT + 2 * kp;
            const uint16_t* src = vc + (size_t)t * kv_stride + kvh * HD + dg * 4;
            va[i] = (idx < VTOTAL && t < seq_total) ? *reinterpret_cast<const uint2*>(src) : make_uint2(0, 0);
            vb[i] = (idx < VTOTAL && t + 1 < seq_total) ? *reinterpret_cast<const uint2*>(src + kv_stride) : make_uint2(0, 0);
        }
    };
    auto store_tile = [&](uint32_t buf) {
#pragma unroll
        for (int i = 0; i < KPIECES; i++) {
            const uint32_t idx = tid + NT * i, key = idx / (HD / 8), dc = idx % (HD / 8);
            if (idx < KTOTAL) *reinterpret_cast<int4*>(Ks(buf) + key * KS + dc * 8) = kreg[i];
        }
        // V^T[d][key]: the two keys' values of one head dim side by side in a dword
#pragma unroll
        for (int i = 0; i < VITEMS; i++) {
            const uint32_t idx = tid + NT * i, kp = idx / DG, dg = idx % DG;
            if (idx < VTOTAL) {
                uint32_t* vt = reinterpret_cast<uint32_t*>(Vt(buf) + (dg * 4) * VS + 2 * kp);
                vt[0 * (VS / 2)] = __builtin_amdgcn_perm(vb[i].x, va[i].x, 0x05040100u);
                vt[1 * (VS / 2)] = __builtin_amdgcn_perm(vb[i].x, va[i].x, 0x07060302u);
                vt[2 * (VS / 2)] = __builtin_amdgcn_perm(vb[i].y, va[i].y, 0x05040100u);
                vt[3 * (VS / 2)] = __builtin_amdgcn_perm(vb[i].y, va[i].y, 0x07060302u);
            }
        }
    };

    load_tile(tile0);
    store_tile(tile0 & 1);
    __syncthreads();
    for (uint32_t kt = tile0; kt < ntiles; kt++) {
        const uint32_t buf = kt & 1;
        if (kt + 1 < ntiles) load_tile(kt + 1);          // in flight while this tile is computed
        const uint32_t k0 = kt * KT + kh * 32;            // this wave's first 32 keys of the tile
        constexpr uint32_t KW = 32 * KH;                  // keys of the tile this wave works
        if (wave_active && k0 <= wave_max_pos && k0 + KW > wave_lo) {   // else they lie entirely in the group's future, or before every window
            const _Float16* Kb = Ks(buf);
            const _Float16* Vb = Vt(buf);
            // ---- S^T tiles: sacc[h][r] = q . k for key k0 + 32 h + 8(r/4) + 4 lh + r%4, query lq
            v16f sacc[KH];
#pragma unroll
            for (int h = 0; h < KH; h++)
#pragma unroll
                for (int r = 0; r < 16; r++) sacc[h][r] = 0.f;
#pragma unroll
            for (int s = 0; s < NS; s++)
#pragma unroll
                for (int h = 0; h < KH; h++) {
                    v8h kf = *reinterpret_cast<const v8h*>(Kb + ((kh + h) * 32 + lq) * KS + 16 * s + 8 * lh);
                    sacc[h] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s], sacc[h], 0, 0, 0);
                }
            // ---- causal mask: only keys past the group's first query can be masked for some query
            // with a window, also keys that the group's last query no longer sees
#pragma unroll
            for (int h = 0; h < KH; h++) {
                const uint32_t kb = k0 + 32 * h;
                if (WIN && (kb + 31 > wave_min_pos || kb + window <= wave_max_pos)) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const uint32_t t = kb + 8 * (r >> 2) + 4 * lh + (r & 3);
                        sacc[h][r] = (t <= qpos && t + window > qpos) ? sacc[h][r] : -INFINITY;
                    }
                } else if (!WIN && kb + 31 > wave_min_pos) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const uint32_t t = kb + 8 * (r >> 2) + 4 * lh + (r & 3);
                        sacc[h][r] = (t <= qpos) ? sacc[h][r] : -INFINITY;
                    }
                }
            }
            // ---- online softmax in base 2 (per-lane scalars: a lane owns one query)
            float m_tile = -INFINITY;
#pragma unroll
            for (int h = 0; h < KH; h++)
#pragma unroll
                for (int r = 0; r < 16; r++) m_tile = fmaxf(m_tile, sacc[h][r]);
            m_tile = lane_xor_max<32>(m_tile) * c2;      // c2 > 0: max commutes with the scaling
            const float m_new = fmaxf(m_run, m_tile);
            // a query that has seen no key yet (all of these keys masked for it) keeps m = -inf: exponentiate
            // against 0 instead, every p is then 2^-inf = 0
            const float m_exp = m_new == -INFINITY ? 0.f : m_new;
            float l_tile = 0.f;
            v8h pb[KH][2];
#pragma unroll
            for (int h = 0; h < KH; h++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const float p = __builtin_amdgcn_exp2f(fmaf(sacc[h][8 * j + e], c2, -m_exp));   // 2^-inf = 0 for masked keys
                        l_tile += p;
                        pb[h][j][e] = (_Float16)p;
                    }
            // rescale what has been accumulated, unless no query of the wave saw a new maximum
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
                const float alpha = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int d = 0; d < ND; d++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[d][r] *= alpha;
            }
            l_run += l_tile;
            m_run = m_new;
            // ---- O^T += V^T P^T over this wave's keys
#pragma unroll
            for (int h = 0; h < KH; h++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int d = 0; d < ND; d++) {
                        const _Float16* vrow = Vb + (d * 32 + lq) * VS + (kh + h) * 32 + 16 * j + 4 * lh;
                        v4h v0 = *reinterpret_cast<const v4h*>(vrow);
                        v4h v1 = *reinterpret_cast<const v4h*>(vrow + 8);
                        v8h vf = (v8h){v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                        oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pb[h][j], oacc[d], 0, 0, 0);
                    }
        }
        if (kt + 1 < ntiles) store_tile(buf ^ 1);   // nobody reads that buffer: its tile was finished before the last barrier
        __syncthreads();
    }

    // ---- the two waves of a query group merge their halves: the odd one hands (m, l, O) over through LDS
    float* mg = reinterpret_cast<float*>(smem) + (qg * 64 + lane) * MERGE_FLOATS;
    if (KH == 1) {
    if (kh == 1) {
        mg[0] = m_run;
        mg[1] = l_run;
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) mg[2 + d * 16 + r] = oacc[d][r];
    }
    __syncthreads();
    if (kh == 1) return;
    {
        const float m1 = mg[0], l1 = mg[1];
        const float m = fmaxf(m_run, m1);            // finite: every query sees itself (without a window, key 0 in the even half too)
        const float a0 = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m), a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - m);
        l_run = l_run * a0 + l1 * a1;
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[d][r] = oacc[d][r] * a0 + mg[2 + d * 16 + r] * a1;
    }
    }

    // ---- normalise and store: lane (lq, lh) holds out[qrow][32 d + 8 g + 4 lh + 0..3]
    const float l_tot = lane_xor_add<32>(l_run);
    if (QUANT) {
        const float inv_l = 1.0f / l_tot;
        const uint32_t width = heads * HD;
#pragma unroll
        for (int d = 0; d < ND; d++) {
            float o[16], amax = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) { o[r] = oacc[d][r] * inv_l; amax = fmaxf(amax, fabsf(o[r])); }
            amax = lane_xor_max<32>(amax);
            float inv;
            const float sc = act_scale(amax, inv);
            // QUANT has no f32 output, so out_stride carries a flag instead: store the odd blocks of a row negated
            if (out_stride != 0 && ((head * (HD / 32) + d) & 1u) != 0) inv = -inv;
            if (qrow < M) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const uint32_t pk = ((uint32_t)quant_code(o[4 * g] * inv) & 0xFFu) | (((uint32_t)quant_code(o[4 * g + 1] * inv) & 0xFFu) << 8) |
                                        (((uint32_t)quant_code(o[4 * g + 2] * inv) & 0xFFu) << 16) | (((uint32_t)quant_code(o[4 * g + 3] * inv) & 0xFFu) << 24);
                    *reinterpret_cast<uint32_t*>(oq + (size_t)qrow * width + head * HD + 32 * d + 8 * g + 4 * lh) = pk;
                }
                // (for the fast GEMM an all-zero block carries the scale 0, see quantize_block_part)
                if (lh == 0) osc[(size_t)qrow * (width / 32) + head * (HD / 32) + d] = (out_stride != 0 && amax == 0.f) ? (uint16_t)0 : f32_to_f16_bits(sc);
            }
        }
        return;
    }
    if (qrow < M) {
        const float inv_l = 1.0f / l_tot;
        float* orow = out + (size_t)qrow * out_stride + head * HD;
#pragma unroll
        for (int d = 0; d < ND; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float4 o = make_float4(oacc[d][4 * g] * inv_l, oacc[d][4 * g + 1] * inv_l, oacc[d][4 * g + 2] * inv_l,
                                       oacc[d][4 * g + 3] * inv_l);
                *reinterpret_cast<float4*>(orow + 32 * d + 8 * g + 4 * lh) = o;
            }
    }
}

namespace {
template <int HD, bool QUANT>
void launch_win(dim3 grid, hipStream_t s, const float* q, const uint16_t* kc, const uint16_t* vc, float* out, uint32_t q_stride,
                uint32_t out_stride, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads, int8_t* oq, uint16_t* osc,
                uint32_t window, PageTable pt) {
    // The 4-wave form when there are clearly more workgroups than the machine holds at once (three per CU at head_dim 64,
    // two above: then throughput decides, and a wave with two score tiles per step does 15-30 % more of it); the 8-wave form
    // when they all fit (then the longest workgroup's chain of tile steps decides, and twice the waves halve its steps).
    // Measured, 32 heads: 3001 tokens of head_dim 96 143 -> 108 us, 8192 tokens of head_dim 128 978 -> 842 us; 2502 tokens of
    // head_dim 64 59 -> 67 us, which is why the count decides.  FORGE_HIP_ATTN_WAVES=8 / 4 forces one.
    static const int forced = [] { const char* e = getenv("FORGE_HIP_ATTN_WAVES"); return e ? atoi(e) : 0; }();
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 256;
        return n > 0 ? n : 256;
    }();
    const uint32_t slots = (uint32_t)cus * (HD == 64 ? 3 : 2);
    const bool four = forced == 4 || (forced != 8 && grid.x * 4 >= slots * 5);
    // a window that covers every key of the call is plain causal attention
    const bool win = window != 0 && window < base_pos + M;
#define FH_AP(WIN_, KH_) \
    fh::launch(attn_prefill_kernel<HD, QUANT, WIN_, KH_>, grid, AP_THREADS / KH_, 0, s, q, kc, vc, out, q_stride, out_stride, M, base_pos, heads, kv_heads, oq, osc, WIN_ ? window : 0u, pt)
    if (win) { if (four) FH_AP(true, 2); else FH_AP(true, 1); }
    else { if (four) FH_AP(false, 2); else FH_AP(false, 1); }
#undef FH_AP
}
template <bool QUANT>
void launch_hd(uint32_t hd, dim3 grid, hipStream_t s, const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
               uint32_t q_stride, uint32_t out_stride, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads, int8_t* oq,
               uint16_t* osc, uint32_t window, PageTable pt) {
    if (hd == 64) launch_win<64, QUANT>(grid, s, q, kc, vc, out, q_stride, out_stride, M, base_pos, heads, kv_heads, oq, osc, window, pt);
    else if (hd == 96) launch_win<96, QUANT>(grid, s, q, kc, vc, out, q_stride, out_stride, M, base_pos, heads, kv_heads, oq, osc, window, pt);
    else launch_win<128, QUANT>(grid, s, q, kc, vc, out, q_stride, out_stride, M, base_pos, heads, kv_heads, oq, osc, window, pt);
}
}  // namespace

void launch_attn_prefill(const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc, float* out,
                         uint32_t out_stride, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                         uint32_t hd, uint32_t window, hipStream_t s, PageTable pt) {
    if (M == 0) return;
    dim3 grid(((M + QB - 1) / QB) * heads);
    launch_hd<false>(hd, grid, s, q, kc, vc, out, q_stride, out_stride, M, base_pos, heads, kv_heads, nullptr, nullptr, window, pt);
}

void launch_attn_prefill_quant(const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc, int8_t* oq, uint16_t* osc,
                               uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads, uint32_t hd, uint32_t window,
                               hipStream_t s, bool neg_odd, PageTable pt) {
    if (M == 0) return;
    dim3 grid(((M + QB - 1) / QB) * heads);
    launch_hd<true>(hd, grid, s, q, kc, vc, nullptr, q_stride, neg_odd ? 1u : 0u, M, base_pos, heads, kv_heads, oq, osc, window, pt);
}

}  // namespace fh

// Decode attention (attention_flash, emit.rs:656-715) over an fp16 KV cache, split along the
// sequence so that one query fills the GPU ("flash decoding"): grid = (kv head groups,
// DECODE_SPLITS).  HBM-bound: each K/V row is read once per group of query heads that share
// it.  A key row of head_dim fp16 values is spread over LPK lanes (16 bytes each); the
// lanes of a wave cover 64/LPK keys per load, a wave keeps four such loads of K and of V in flight
// (and the next four requested before it computes), and every key slot keeps its own online-softmax
// state, advanced two keys at a time (one new maximum and one rescale per pair), so the loop
// needs no cross-slot traffic; slots, waves and splits are merged at the end with the usual
// (max, sum, acc) rescaling.
#include <mutex>

#include "attn_decode_math.h"
#include "common.h"
#include "device_utils.h"

namespace fh {

// merge (m2,l2,a2) into (m,l,a)
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

// A paged cache (PAGED): kc / vc are pools of pages of 2^page_shift rows, and row t of the sequence is row t % page of
// pool page page_table[t / page].  A split's table entries are copied into LDS first (they are few), so the address of
// a key costs one LDS read more than in the flat cache; nothing else changes, the bits included.
constexpr uint32_t PAGE_ENTRIES_MAX = 2048;   // table entries one split may span (else: contiguous-only)

// workspace record per (kv group, split, head-in-group): [HD acc][m][l]
template <int HD, int GT, bool PAGED = false>
__global__ __launch_bounds__(256) void attn_decode_split_kernel(const float* __restrict__ q,
                                                                const uint16_t* __restrict__ kc,
                                                                const uint16_t* __restrict__ vc,
                                                                float* __restrict__ ws, uint32_t seq_len_arg,
                                                                const uint32_t* __restrict__ pos_dev, uint32_t heads,
                                                                uint32_t kv_heads, uint32_t gsize, uint32_t window, PageTable pt) {
    constexpr int LPK = HD <= 64 ? 8 : 16;   // lanes per key row
    constexpr int KPW = 64 / LPK;            // keys per wave load
    constexpr int REC = HD + 2;
    __shared__ float sh[4][GT][REC];

    const uint32_t seq = pos_dev ? (*pos_dev + 1) : seq_len_arg;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t c = lane % LPK, slot = lane / LPK;
    const bool dvalid = c * 8 < HD;
    const uint32_t gpk = gsize / GT;   // head sub-groups per kv head
    const uint32_t kvh = blockIdx.x / gpk, sub = blockIdx.x % gpk;
    const uint32_t h0 = kvh * gsize + sub * GT;
    const uint32_t split = blockIdx.y, nsplit = gridDim.y;
    const float scale = 1.0f / sqrtf((float)HD);
    const uint32_t kv_stride = kv_heads * HD;

    // attention_sliding (emit.rs:598-627): only the last `window` rows are keys (window 0: all of them)
    const uint32_t start = (window != 0 && seq > window) ? seq - window : 0;
    uint32_t chunk = (seq - start + nsplit - 1) / nsplit;
    chunk = (chunk + 4 * KPW - 1) / (4 * KPW) * (4 * KPW);
    const uint32_t t0 = min(seq, start + split * chunk);
    const uint32_t t1 = min(seq, t0 + chunk);

    __shared__ uint32_t pt_s[PAGED ? PAGE_ENTRIES_MAX : 1];
    const uint32_t pt_first = PAGED ? t0 >> pt.shift : 0;
    if (PAGED) {
        const uint32_t n_entries = t1 > t0 ? ((t1 - 1) >> pt.shift) - pt_first + 1 : 0;
        for (uint32_t i = threadIdx.x; i < n_entries; i += 256) pt_s[i] = pt.table[pt_first + i];
        __syncthreads();
    }
    // row of the cache (pool) that holds position t
    auto row_of = [&](uint32_t t) -> size_t {
        if (!PAGED) return t;
        return ((size_t)pt_s[(t >> pt.shift) - pt_first] << pt.shift) + (t & ((1u << pt.shift) - 1));
    };

    float qf[GT][8];
#pragma unroll
    for (int g = 0; g < GT; g++)
#pragma unroll
        for (int i = 0; i < 8; i++) qf[g][i] = dvalid ? q[(size_t)(h0 + g) * HD + c * 8 + i] : 0.f;

    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int g = 0; g < GT; g++) {
        m[g] = -INFINITY; l[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[g][i] = 0.f;
    }

    // A wave takes UNR key blocks (UNR * KPW keys) per step, all their K and V loads in flight together and the next step's
    // issued before this step's arithmetic; every key slot advances its online softmax by UNR keys at once.
    constexpr int UNR = 4;
    const uint32_t tbw = t0 + wave * KPW, tstep = UNR * 4 * KPW;
    auto load_step = [&](uint32_t tb0, Half8 (&kr)[UNR], Half8 (&vr)[UNR]) {
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const uint32_t t = tb0 + u * 4 * KPW + slot;
            kr[u] = Half8{{0, 0, 0, 0}};
            vr[u] = Half8{{0, 0, 0, 0}};
            if (t < t1 && dvalid) {
                const size_t off = row_of(t) * kv_stride + kvh * HD + c * 8;
                kr[u] = *reinterpret_cast<const Half8*>(kc + off);
                vr[u] = *reinterpret_cast<const Half8*>(vc + off);
            }
        }
    };
    Half8 kr[UNR], vr[UNR], kn[UNR], vn[UNR];
    if (tbw < t1) load_step(tbw, kr, vr);
    for (uint32_t tb0 = tbw; tb0 < t1; tb0 += tstep) {
        const bool more = tb0 + tstep < t1;
        if (more) load_step(tb0 + tstep, kn, vn);
#pragma unroll
        for (int u0 = 0; u0 < UNR; u0 += 2)
#pragma unroll
            for (int g = 0; g < GT; g++) {
                float sc[2];
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const float d = key_dot<LPK>(qf[g], kr[u0 + u]);
                    sc[u] = tb0 + (u0 + u) * 4 * KPW + slot < t1 ? d * scale : -INFINITY;
                }
                softmax_block_update<2>(m[g], l[g], acc[g], sc, vr + u0);
            }
        if (more) {
#pragma unroll
            for (int u = 0; u < UNR; u++) { kr[u] = kn[u]; vr[u] = vn[u]; }
        }
    }

    // merge the key slots of the wave
#pragma unroll
    for (int g = 0; g < GT; g++) {
        auto merge_with = [&](auto O) {
            const float m2 = lane_xor<O.value>(m[g]), l2 = lane_xor<O.value>(l[g]);
            float a2[8];
#pragma unroll
            for (int i = 0; i < 8; i++) a2[i] = lane_xor<O.value>(acc[g][i]);
            merge_state<8>(m[g], l[g], acc[g], m2, l2, a2);
        };
        if (LPK == 8) merge_with(std::integral_constant<int, 8>{});
        merge_with(std::integral_constant<int, 16>{});
        merge_with(std::integral_constant<int, 32>{});
        if (slot == 0 && dvalid) {
#pragma unroll
            for (int i = 0; i < 8; i++) sh[wave][g][c * 8 + i] = acc[g][i];
            if (c == 0) { sh[wave][g][HD] = m[g]; sh[wave][g][HD + 1] = l[g]; }
        }
    }
    __syncthreads();
    // merge the four waves: thread d of the first GT*HD threads owns one output element
    for (uint32_t e = threadIdx.x; e < GT * HD; e += 256) {
        const uint32_t g = e / HD, d = e % HD;
        float mm = sh[0][g][HD], ll = sh[0][g][HD + 1], a = sh[0][g][d];
        for (int w = 1; w < 4; w++) {
            float a2 = sh[w][g][d];
            merge_state<1>(mm, ll, &a, sh[w][g][HD], sh[w][g][HD + 1], &a2);
        }
        float* rec = ws + ((size_t)(h0 + g) * nsplit + split) * REC;
        rec[d] = a;
        if (d == 0) { rec[HD] = mm; rec[HD + 1] = ll; }
    }
}

// One workgroup of HD threads per head: merge the splits, normalise, optionally quantise
// the 32-element blocks of the output for the O projection.
template <int HD>
__global__ void attn_decode_combine_kernel(const float* __restrict__ ws, uint32_t nsplit, float* __restrict__ out,
                                           int8_t* __restrict__ oq, uint16_t* __restrict__ osc) {
    constexpr int REC = HD + 2;
    __shared__ float wgt_s[DECODE_SPLITS];
    __shared__ float den_s;
    const uint32_t h = blockIdx.x, d = threadIdx.x;
    const float* base = ws + (size_t)h * nsplit * REC;
    // lanes 0..nsplit-1 of the first wave fetch the split maxima and sums in parallel
    if (d < 64) {
        const float ms = d < nsplit ? base[d * REC + HD] : -INFINITY;
        const float ls = d < nsplit ? base[d * REC + HD + 1] : 0.f;
        const float mm = wave_max(ms);
        const float wgt = (ms == -INFINITY) ? 0.f : __expf(ms - mm);
        const float den = wave_sum(wgt * ls);
        if (d < nsplit) wgt_s[d] = wgt;
        if (d == 0) den_s = den;
    }
    __syncthreads();
    float part[DECODE_SPLITS];
#pragma unroll
    for (uint32_t s = 0; s < DECODE_SPLITS; s++) part[s] = s < nsplit ? base[s * REC + d] : 0.f;   // all loads in flight
    float num = 0.f;
#pragma unroll
    for (uint32_t s = 0; s < DECODE_SPLITS; s++) num = fmaf(wgt_s[s < nsplit ? s : 0], part[s], num);
    const float o = num * (1.0f / den_s);
    if (out) out[(size_t)h * HD + d] = o;
    if (oq) {
        const float amax = half_wave_max(fabsf(o));
        float inv;
        const float sc = act_scale(amax, inv);
        oq[(size_t)h * HD + d] = (int8_t)quant_code(o * inv);
        if ((d & 31) == 0) osc[((size_t)h * HD + d) / 32] = f32_to_f16_bits(sc);
    }
}

size_t attn_decode_workspace_bytes(uint32_t heads, uint32_t hd) {
    return (size_t)heads * DECODE_SPLITS * (hd + 2) * sizeof(float);
}

bool attn_head_dim_supported(uint32_t hd) { return hd == 64 || hd == 96 || hd == 128; }

namespace {
template <int HD, int GT>
void launch_split(const float* q, const uint16_t* kc, const uint16_t* vc, float* ws, uint32_t seq,
                  const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t window, PageTable pt, hipStream_t s) {
    const uint32_t gsize = heads / kv_heads;
    dim3 grid(kv_heads * (gsize / GT), DECODE_SPLITS);
    if (pt.table) fh::launch(attn_decode_split_kernel<HD, GT, true>, grid, 256, 0, s, q, kc, vc, ws, seq, pos_dev, heads, kv_heads, gsize, window, pt);
    else fh::launch(attn_decode_split_kernel<HD, GT, false>, grid, 256, 0, s, q, kc, vc, ws, seq, pos_dev, heads, kv_heads, gsize, window, pt);
}
template <int HD>
void launch_hd(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int8_t* oq, uint16_t* osc,
               uint32_t seq, const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t window, float* ws, PageTable pt,
               hipStream_t s) {
    const uint32_t gsize = heads / kv_heads;
    if (gsize % 4 == 0) launch_split<HD, 4>(q, kc, vc, ws, seq, pos_dev, heads, kv_heads, window, pt, s);
    else if (gsize % 3 == 0) launch_split<HD, 3>(q, kc, vc, ws, seq, pos_dev, heads, kv_heads, window, pt, s);
    else if (gsize % 2 == 0) launch_split<HD, 2>(q, kc, vc, ws, seq, pos_dev, heads, kv_heads, window, pt, s);
    else launch_split<HD, 1>(q, kc, vc, ws, seq, pos_dev, heads, kv_heads, window, pt, s);
    fh::launch(attn_decode_combine_kernel<HD>, heads, HD, 0, s, ws, DECODE_SPLITS, out, oq, osc);
}
}  // namespace

// Whether a paged call with these sizes is covered: pages of a power of two of rows, and no split spanning more table
// entries than the kernel keeps in LDS.
bool attn_decode_paged_supported(uint32_t seq_len, uint32_t page_rows) {
    if (page_rows == 0 || (page_rows & (page_rows - 1)) != 0) return false;
    const uint32_t per_split = (seq_len + DECODE_SPLITS - 1) / DECODE_SPLITS + 64;
    return per_split / page_rows + 2 <= PAGE_ENTRIES_MAX;
}

void launch_attn_decode_paged(const float* q, const uint16_t* k_pool, const uint16_t* v_pool, const uint32_t* page_table,
                              uint32_t page_rows, float* out, uint32_t seq_len, uint32_t heads, uint32_t kv_heads, uint32_t hd,
                              void* workspace, hipStream_t s) {
    float* ws = reinterpret_cast<float*>(workspace);
    PageTable pt{page_table, (uint32_t)__builtin_ctz(page_rows)};
    if (hd == 64) launch_hd<64>(q, k_pool, v_pool, out, nullptr, nullptr, seq_len, nullptr, heads, kv_heads, 0u, ws, pt, s);
    else if (hd == 96) launch_hd<96>(q, k_pool, v_pool, out, nullptr, nullptr, seq_len, nullptr, heads, kv_heads, 0u, ws, pt, s);
    else launch_hd<128>(q, k_pool, v_pool, out, nullptr, nullptr, seq_len, nullptr, heads, kv_heads, 0u, ws, pt, s);
}

void launch_attn_decode(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int8_t* oq, uint16_t* osc,
                        uint32_t seq_len, const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd,
                        uint32_t window, void* workspace, hipStream_t s, PageTable pt) {
    float* ws = reinterpret_cast<float*>(workspace);
    if (hd == 64) launch_hd<64>(q, kc, vc, out, oq, osc, seq_len, pos_dev, heads, kv_heads, window, ws, pt, s);
    else if (hd == 96) launch_hd<96>(q, kc, vc, out, oq, osc, seq_len, pos_dev, heads, kv_heads, window, ws, pt, s);
    else launch_hd<128>(q, kc, vc, out, oq, osc, seq_len, pos_dev, heads, kv_heads, window, ws, pt, s);
}

}  // namespace fh

// ---- decode attention for callers that cannot allocate ----------------------------------------------------------
// The split records of the two kernels above normally live in a lazily grown allocation of the op-level API.  Code
// under HIP graph capture, tight serving loops and harnesses that forbid allocation get the same kernels over a
// fixed array in the library's own device image instead.  Each GPU holds its own copy of the array (until the
// process ends) at its own address, which the host learns once per device with hipGetSymbolAddress: the array's
// name in host code is only a handle for that query, never a device address.
namespace {
constexpr uint32_t NOALLOC_MAX_HEADS = 128, NOALLOC_MAX_HEAD_DIM = 128;
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)NOALLOC_MAX_HEADS * fh::DECODE_SPLITS * (NOALLOC_MAX_HEAD_DIM + 2) * sizeof(float);
constexpr int NOALLOC_MAX_DEVICES = 64;

static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

std::mutex g_scratch_mutex;
void* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device (looked up on the first call per device).
int32_t scratch_on_current_device(void** out) {
    int dev = -1;
    FH_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return fh::fail(FORGE_HIP_ERR_INVALID, "attn_decode_noalloc: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        FH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fh::fail(FORGE_HIP_ERR_HIP, "attn_decode_noalloc: hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FORGE_HIP_OK;
}
}  // namespace

// Set-up calls (forge_hip_model_create, forge_hip_qweight_create) look the address up for their device, so that a caller
// who has made one of them never pays the lookup (which may load the code object) inside forge_hip_attn_decode_f16kv_noalloc,
// for instance under a stream capture.  A failure is left for the entry point itself to report.
void fh::attn_decode_noalloc_prepare() {
    void* p = nullptr;
    if (scratch_on_current_device(&p) != FORGE_HIP_OK) (void)hipGetLastError();
}

extern "C" int32_t forge_hip_attn_decode_f16kv_noalloc(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                                       float* out_dev, uint32_t seq_len, uint32_t heads, uint32_t kv_heads,
                                                       uint32_t head_dim, void* stream) {
    FH_CHECK(q_dev && k_cache_dev && v_cache_dev && out_dev, "attn_decode_noalloc: null pointer");
    FH_CHECK(seq_len >= 1, "attn_decode_noalloc: seq_len must be at least 1");
    FH_CHECK(fh::attn_head_dim_supported(head_dim), "attn_decode_noalloc: head_dim must be 64, 96 or 128");
    FH_CHECK(kv_heads != 0 && heads != 0 && heads % kv_heads == 0, "attn_decode_noalloc: heads must be a positive multiple of kv_heads");
    FH_CHECK(heads <= NOALLOC_MAX_HEADS && fh::attn_decode_workspace_bytes(heads, head_dim) <= NOALLOC_SCRATCH_BYTES,
             "attn_decode_noalloc: more than 128 query heads do not fit the fixed scratch array");
    void* ws = nullptr;
    int32_t rc = scratch_on_current_device(&ws);
    if (rc) return rc;
    // every (head, split) record is written by the split kernel before the merge kernel reads it, empty splits
    // included, so nothing of the previous call's contents has to be cleared
    fh::launch_attn_decode(q_dev, k_cache_dev, v_cache_dev, out_dev, nullptr, nullptr, seq_len, nullptr, heads, kv_heads, head_dim, 0u,
                           ws, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

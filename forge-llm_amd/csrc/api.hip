// extern "C" surface, part 1: error string, host format helpers and the op-level entry points.
// The op-level calls own one lazily grown device scratch area per process (activation
// codes, split-attention partials, rope tables); they are for one caller thread at a time.
#include <math.h>

#include <vector>

#include <algorithm>

#include "common.h"
#include "expf_ref.h"

namespace fh {

int32_t qweight_upload(uint32_t wdtype, const uint8_t* raw_host, uint32_t K, uint32_t N, QWeight* out) {
    QWeight w;
    w.wdtype = wdtype; w.K = K; w.N = N; w.owns = true;
    std::vector<uint8_t> qs(w.qs_bytes());
    std::vector<uint16_t> sc((w.scales_bytes() + 1) / 2);
    if (w.kquant()) repack_kquant_host(wdtype, raw_host, K, N, qs.data(), reinterpret_cast<uint8_t*>(sc.data()));
    else repack_host(wdtype, raw_host, K, N, qs.data(), sc.data());
    FH_HIP(hipMalloc((void**)&w.qs, std::max<size_t>(qs.size(), 16)));
    hipError_t e = hipMalloc((void**)&w.scales, std::max<size_t>(w.scales_bytes(), 16));
    if (e != hipSuccess) { (void)hipFree(w.qs); return fail(FORGE_HIP_ERR_HIP, "hipMalloc(scales) failed"); }
    e = hipMemcpy(w.qs, qs.data(), qs.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(w.scales, sc.data(), w.scales_bytes(), hipMemcpyHostToDevice);
    if (e != hipSuccess) { qweight_free(&w); return fail(FORGE_HIP_ERR_HIP, std::string("weight upload: ") + hipGetErrorString(e)); }
    *out = w;
    return FORGE_HIP_OK;
}

void qweight_free(QWeight* w) {
    if (w->owns) {
        if (w->qs) (void)hipFree(w->qs);
        if (w->scales) (void)hipFree(w->scales);
    }
    w->qs = nullptr; w->scales = nullptr; w->owns = false;
}

namespace {

// One area per device (the process may drive several): it grows when a call needs more than any earlier call on that device,
// in steps of at least half its size again, so that a run of growing shapes re-allocates a few times and not at every call.
struct Scratch {
    static constexpr int MAX_DEVICES = 16;
    void* area[MAX_DEVICES] = {};
    size_t cap[MAX_DEVICES] = {};
    static int device() {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) dev = 0;
        return dev;
    }
    void* ptr() const { return area[device()]; }
    size_t capacity() const { return cap[device()]; }
    int32_t reserve(size_t n) {
        const int d = device();
        if (n <= cap[d]) return FORGE_HIP_OK;
        const size_t want = std::max(n, cap[d] + cap[d] / 2);
        if (area[d]) { FH_HIP(hipFree(area[d])); area[d] = nullptr; cap[d] = 0; }      // waits for the device
        FH_HIP(hipMalloc(&area[d], want));
        cap[d] = want;
        return FORGE_HIP_OK;
    }
};
Scratch g_act;    // quantised activations: codes then scales
Scratch g_attn;   // decode-attention partials / argmax partials
Scratch g_rope;   // cos | sin tables
Scratch g_gemm;   // partial tiles and counters of the GEMM's K-range variant
Scratch g_twin;   // K-quant twins: block sums of the activations, or the activations with every block twice

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

bool valid_wdtype(uint32_t t) { return t == FORGE_HIP_Q8_0 || t == FORGE_HIP_Q4_0; }

// Quantise x[M][K] into the shared scratch; returns pointers.
int32_t quantise_into_scratch(const float* x, uint32_t M, uint32_t K, int8_t** q, uint16_t** sc, hipStream_t s, bool neg_odd = false) {
    const size_t qbytes = align256((size_t)M * K);
    const size_t sbytes = (size_t)M * (K / 32) * 2;
    int32_t rc = g_act.reserve(qbytes + sbytes);
    if (rc) return rc;
    *q = reinterpret_cast<int8_t*>(g_act.ptr());
    *sc = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(g_act.ptr()) + qbytes);
    launch_quantize_act(x, M, K, *q, *sc, s, neg_odd);
    return FORGE_HIP_OK;
}

}  // namespace
}  // namespace fh

using namespace fh;

struct forge_hip_qweight {
    QWeight w;
    // K-quant matrices: the matrix as the int8 MFMA GEMM takes it, built by the first forge_hip_gemm_q without FLAG_EXACT
    KqTwin twin;
    bool twin_tried = false, twin_covered = false;
};

extern "C" {

const char* forge_hip_last_error(void) { return last_error_cstr(); }

int32_t forge_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

float forge_hip_f16_to_f32(uint16_t bits) { return f16_to_f32_host(bits); }
uint16_t forge_hip_f32_to_f16(float x) { return f32_to_f16_host(x); }

int32_t forge_hip_quantize_f32(uint32_t wdtype, const float* data_host, uint64_t n, uint8_t* out_host) {
    FH_CHECK(valid_wdtype(wdtype), "quantize_f32: wdtype must be Q8_0 (8) or Q4_0 (2)");
    FH_CHECK(data_host && out_host, "quantize_f32: null pointer");
    quantize_host(wdtype, data_host, n, out_host);
    return FORGE_HIP_OK;
}

int32_t forge_hip_dequant(uint32_t wdtype, const uint8_t* data_host, uint64_t n, float* out_host) {
    FH_CHECK(valid_wdtype(wdtype), "dequant: wdtype must be Q8_0 (8) or Q4_0 (2)");
    FH_CHECK(data_host && out_host, "dequant: null pointer");
    dequant_host(wdtype, data_host, n, out_host);
    return FORGE_HIP_OK;
}

int32_t forge_hip_qweight_create(uint32_t wdtype, const uint8_t* raw_host, uint32_t K, uint32_t N,
                                 forge_hip_qweight** out) {
    FH_CHECK(out, "qweight_create: null out");
    *out = nullptr;
    const bool kq = wdtype == FORGE_HIP_Q4_K || wdtype == FORGE_HIP_Q6_K;
    FH_CHECK(valid_wdtype(wdtype) || kq, "qweight_create: wdtype must be Q8_0 (8), Q4_0 (2), Q4_K (12) or Q6_K (14)");
    FH_CHECK(raw_host, "qweight_create: null weights");
    FH_CHECK(K >= 32 && K % 32 == 0 && N >= 1, "qweight_create: K must be a positive multiple of 32 and N >= 1");
    FH_CHECK(!kq || kquant_k_supported(K), "qweight_create: a K-quant matrix needs K to be a multiple of 256, at most 16384");
    if (forge_hip_device_count() < 1) return fail(FORGE_HIP_ERR_NO_DEVICE, "no HIP device");
    attn_decode_noalloc_prepare();
    forge_hip_qweight* h = new forge_hip_qweight();
    int32_t rc = qweight_upload(wdtype, raw_host, K, N, &h->w);
    if (rc) { delete h; return rc; }
    *out = h;
    return FORGE_HIP_OK;
}

void forge_hip_qweight_destroy(forge_hip_qweight* w) {
    if (!w) return;
    qweight_free(&w->w);
    kquant_twin_free(&w->twin);
    delete w;
}

int32_t forge_hip_quantize_act(const float* x_dev, uint32_t M, uint32_t K, int8_t* q_dev, uint16_t* scales_dev,
                               void* stream) {
    FH_CHECK(x_dev && q_dev && scales_dev, "quantize_act: null pointer");
    FH_CHECK(K % 32 == 0, "quantize_act: K must be a multiple of 32");
    launch_quantize_act(x_dev, M, K, q_dev, scales_dev, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_gemv_q(const forge_hip_qweight* w, const float* x_dev, float* y_dev, void* stream) {
    FH_CHECK(w && x_dev && y_dev, "gemv_q: null pointer");
    FH_CHECK(gemv_k_supported(w->w.K), "gemv_q: K must be a multiple of 32, at most 16384");
    int8_t* q; uint16_t* sc;
    int32_t rc = quantise_into_scratch(x_dev, 1, w->w.K, &q, &sc, (hipStream_t)stream);
    if (rc) return rc;
    if (w->w.kquant()) launch_gemv_kquant(w->w, q, sc, y_dev, false, (hipStream_t)stream);
    else launch_gemv(w->w, q, sc, y_dev, false, GemvOrder::MatmulVec, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_gemm_q(const forge_hip_qweight* w, const float* x_dev, uint32_t M, float* y_dev, uint32_t flags,
                         void* stream) {
    FH_CHECK(w && x_dev && y_dev, "gemm_q: null pointer");
    FH_CHECK((flags & ~FORGE_HIP_FLAG_EXACT) == 0, "gemm_q: unknown flag bits");
    if (M == 0) return FORGE_HIP_OK;
    int8_t* q; uint16_t* sc;
    const bool exact = (flags & FORGE_HIP_FLAG_EXACT) != 0;
    if (w->w.kquant()) {
        FH_CHECK(kquant_k_supported(w->w.K), "gemm_q: K must be a multiple of 256, at most 16384");
        hipStream_t s = (hipStream_t)stream;
        forge_hip_qweight* h = const_cast<forge_hip_qweight*>(w);
        if (!exact && !h->twin_tried) {
            const QWeight* one[1] = {&h->w};
            int32_t rct = kquant_twin_create(one, 1, &h->twin, &h->twin_covered, s);
            if (rct) return rct;
            h->twin_tried = true;
        }
        if (exact || !h->twin_covered) {
            // the reference has no batched matmul for these formats: M rows of matmul_vec, the matrix read once per 8 rows
            int32_t rck = quantise_into_scratch(x_dev, M, w->w.K, &q, &sc, s, false);
            if (rck) return rck;
            launch_gemv_kquant_rows(w->w, q, sc, M, y_dev, w->w.N, false, s);
            FH_HIP(hipGetLastError());
            return FORGE_HIP_OK;
        }
        // fast mode: the matrix's twin on the int8 MFMA GEMM (kquant_prefill.hip)
        const uint32_t K = w->w.K;
        int32_t rck = quantise_into_scratch(x_dev, M, K, &q, &sc, s, true);
        if (rck) return rck;
        void* split_ws = nullptr;
        if (M > 64) {
            const bool fresh = g_gemm.capacity() < gemm_split_workspace_bytes();
            if ((rck = g_gemm.reserve(gemm_split_workspace_bytes()))) return rck;
            if (fresh) FH_HIP(hipMemsetAsync(g_gemm.ptr(), 0, gemm_split_workspace_bytes(), s));
            split_ws = g_gemm.ptr();
        }
        if (h->twin.coef) {
            if ((rck = g_twin.reserve((size_t)M * (K / 32) * 4))) return rck;
            launch_act_block_sums(q, sc, M, K, true, reinterpret_cast<float*>(g_twin.ptr()), s);
            launch_gemm(h->twin.w, q, sc, M, y_dev, w->w.N, false, false, nullptr, s, split_ws, nullptr, nullptr,
                        reinterpret_cast<const float*>(g_twin.ptr()), h->twin.coef);
        } else {
            const size_t qbytes = align256((size_t)M * K * 2);
            if ((rck = g_twin.reserve(qbytes + (size_t)M * (K / 32) * 4))) return rck;
            int8_t* q2 = reinterpret_cast<int8_t*>(g_twin.ptr());
            uint16_t* sc2 = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(g_twin.ptr()) + qbytes);
            launch_act_twice(q, sc, M, K, q2, sc2, s);
            launch_gemm(h->twin.w, q2, sc2, M, y_dev, w->w.N, false, false, nullptr, s, split_ws);
        }
        FH_HIP(hipGetLastError());
        return FORGE_HIP_OK;
    }
    int32_t rc = quantise_into_scratch(x_dev, M, w->w.K, &q, &sc, (hipStream_t)stream, !exact);   // the fast kernel takes odd blocks negated
    if (rc) return rc;
    // fast mode may cut tiles along K to fill the CUs: that kernel parks partial tiles in a workspace
    void* split_ws = nullptr;
    if (!exact && M > 64) {
        const bool fresh = g_gemm.capacity() < gemm_split_workspace_bytes();
        if ((rc = g_gemm.reserve(gemm_split_workspace_bytes()))) return rc;
        // its counters start at zero and are left at zero; cleared on the caller's stream, so that the clear is ordered
        // before the kernel whatever kind of stream that is (a null-stream memset does not wait for, and is not waited
        // for by, a non-blocking stream)
        if (fresh) FH_HIP(hipMemsetAsync(g_gemm.ptr(), 0, gemm_split_workspace_bytes(), (hipStream_t)stream));
        split_ws = g_gemm.ptr();
    }
    launch_gemm(w->w, q, sc, M, y_dev, w->w.N, false, exact, nullptr, (hipStream_t)stream, split_ws);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_gemm_silu_q(const forge_hip_qweight* w, const float* x_dev, uint32_t M, int8_t* out_q_dev, uint16_t* out_scales_dev,
                              void* stream) {
    FH_CHECK(w && x_dev && out_q_dev && out_scales_dev, "gemm_silu_q: null pointer");
    FH_CHECK(!w->w.kquant(), "gemm_silu_q: Q8_0 and Q4_0 matrices only");
    if (M == 0) return FORGE_HIP_OK;
    FH_CHECK(w->w.N % 128 == 0 && gemm_silu_supported(w->w, w->w.N / 2, M),
             "gemm_silu_q: the matrix must hold gate rows then up rows, a multiple of 64 each, and M * max(K, N / 2) must stay below 2^31");
    int8_t* q; uint16_t* sc;
    int32_t rc = quantise_into_scratch(x_dev, M, w->w.K, &q, &sc, (hipStream_t)stream, true);
    if (rc) return rc;
    void* split_ws = nullptr;
    if (M > 64) {
        const bool fresh = g_gemm.capacity() < gemm_split_workspace_bytes();
        if ((rc = g_gemm.reserve(gemm_split_workspace_bytes()))) return rc;
        if (fresh) FH_HIP(hipMemsetAsync(g_gemm.ptr(), 0, gemm_split_workspace_bytes(), (hipStream_t)stream));
        split_ws = g_gemm.ptr();
    }
    launch_gemm(w->w, q, sc, M, nullptr, w->w.N, false, false, nullptr, (hipStream_t)stream, split_ws, out_q_dev, out_scales_dev);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_gemv_q_f32act(const forge_hip_qweight* w, const float* x_dev, float* y_dev, void* stream) {
    FH_CHECK(w && x_dev && y_dev, "gemv_q_f32act: null pointer");
    FH_CHECK(!w->w.kquant(), "gemv_q_f32act: Q8_0 and Q4_0 matrices only");
    launch_gemv_f32(w->w, x_dev, y_dev, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_block_isums(const forge_hip_qweight* w, const float* x_dev, uint32_t M, int32_t* out_dev,
                              uint32_t path, void* stream) {
    FH_CHECK(w && x_dev && out_dev, "block_isums: null pointer");
    FH_CHECK(!w->w.kquant(), "block_isums: Q8_0 and Q4_0 matrices only");
    FH_CHECK(path <= 2, "block_isums: path must be 0 (GEMV kernel), 1 (MFMA GEMM kernel, exact mode) or 2 (MFMA GEMM kernel, fast mode)");
    if (M == 0) return FORGE_HIP_OK;
    int8_t* q; uint16_t* sc;
    int32_t rc = quantise_into_scratch(x_dev, M, w->w.K, &q, &sc, (hipStream_t)stream, path == 2);
    if (rc) return rc;
    const size_t nblk = w->w.K / 32;
    if (path == 0) {
        FH_CHECK(gemv_k_supported(w->w.K), "block_isums: K too large for the GEMV path");
        for (uint32_t r = 0; r < M; r++)
            launch_gemv_isums(w->w, q + (size_t)r * w->w.K, out_dev + (size_t)r * w->w.N * nblk, (hipStream_t)stream);
    } else {
        FH_CHECK((uint64_t)M * w->w.N * nblk * 4 < 0x7FFFFFFFull, "block_isums: more than 2 GiB of block sums in one call");
        // The GEMM kernel also writes y; give it the tail of the scratch as a sink.
        Scratch& sink = g_attn;
        rc = sink.reserve((size_t)M * w->w.N * sizeof(float));
        if (rc) return rc;
        launch_gemm(w->w, q, sc, M, reinterpret_cast<float*>(sink.ptr()), w->w.N, false, path == 1, out_dev, (hipStream_t)stream);
    }
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_rms_norm(const float* x_dev, const float* w_dev, float eps, uint32_t M, uint32_t H, float* out_dev,
                           void* stream) {
    FH_CHECK(x_dev && w_dev && out_dev, "rms_norm: null pointer");
    FH_CHECK(H % 4 == 0 && H >= 4 && H <= 16352, "rms_norm: H must be a multiple of 4, at most 16352");
    launch_rmsnorm(x_dev, w_dev, eps, M, H, out_dev, nullptr, nullptr, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_silu_mul(const float* gate_dev, const float* up_dev, uint64_t n, float* out_dev, void* stream) {
    FH_CHECK(gate_dev && up_dev && out_dev, "silu_mul: null pointer");
    FH_CHECK(n % 4 == 0 && n <= 0xFFFFFFFFull, "silu_mul: n must be a multiple of 4");
    launch_silu_mul(gate_dev, up_dev, 1, (uint32_t)n, (uint32_t)n, out_dev, nullptr, nullptr, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_rope_kv_store(float* q_dev, float* k_dev, const float* v_dev, uint16_t* k_cache_dev,
                                uint16_t* v_cache_dev, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                                uint32_t head_dim, float theta, void* stream) {
    FH_CHECK(q_dev && k_dev && v_dev && k_cache_dev && v_cache_dev, "rope_kv_store: null pointer");
    FH_CHECK(head_dim % 2 == 0 && head_dim >= 2 && heads >= 1 && kv_heads >= 1, "rope_kv_store: bad head shape");
    if (M == 0) return FORGE_HIP_OK;
    const uint32_t half = head_dim / 2, n_pos = base_pos + M;
    // rope_freqs + per-position sin_cos, emit.rs:501-517, evaluated with the host C library.
    std::vector<float> tab((size_t)2 * n_pos * half);
    for (uint32_t i = 0; i < half; i++) {
        const float f = 1.0f / powf(theta, 2.0f * (float)i / (float)head_dim);
        for (uint32_t p = 0; p < n_pos; p++) {
            const float a = (float)p * f;
            tab[(size_t)p * half + i] = cosf(a);
            tab[(size_t)n_pos * half + (size_t)p * half + i] = sinf(a);
        }
    }
    int32_t rc = g_rope.reserve(tab.size() * sizeof(float));
    if (rc) return rc;
    FH_HIP(hipMemcpyAsync(g_rope.ptr(), tab.data(), tab.size() * sizeof(float), hipMemcpyHostToDevice, (hipStream_t)stream));
    FH_HIP(hipStreamSynchronize((hipStream_t)stream));   // `tab` is pageable and about to go out of scope
    const float* cos_t = reinterpret_cast<const float*>(g_rope.ptr());
    const float* sin_t = cos_t + (size_t)n_pos * half;
    launch_rope_kv_store(q_dev, k_dev, v_dev, heads * head_dim, kv_heads * head_dim, k_cache_dev, v_cache_dev, M,
                         base_pos, nullptr, heads, kv_heads, head_dim, cos_t, sin_t, nullptr, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

static int32_t check_attn_shape(const char* who, uint32_t heads, uint32_t kv_heads, uint32_t head_dim) {
    if (!attn_head_dim_supported(head_dim)) return fail(FORGE_HIP_ERR_INVALID, std::string(who) + ": head_dim must be 64, 96 or 128");
    if (kv_heads == 0 || heads == 0 || heads % kv_heads != 0)
        return fail(FORGE_HIP_ERR_INVALID, std::string(who) + ": heads must be a positive multiple of kv_heads");
    return FORGE_HIP_OK;
}

int32_t forge_hip_attn_prefill_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                     float* out_dev, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                                     uint32_t head_dim, uint32_t flags, void* stream) {
    FH_CHECK(q_dev && k_cache_dev && v_cache_dev && out_dev, "attn_prefill: null pointer");
    FH_CHECK((flags & ~FORGE_HIP_FLAG_EXACT) == 0, "attn_prefill: unknown flag bits");
    int32_t rc = check_attn_shape("attn_prefill", heads, kv_heads, head_dim);
    if (rc) return rc;
    if (flags & FORGE_HIP_FLAG_EXACT)
        launch_attn_exact(true, q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, nullptr,
                          nullptr, M, base_pos, nullptr, heads, kv_heads, head_dim, 0u, 0u, nullptr, (hipStream_t)stream);
    else
        launch_attn_prefill(q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, M, base_pos,
                            heads, kv_heads, head_dim, 0u, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_attn_prefill_sliding_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                             float* out_dev, uint32_t M, uint32_t base_pos, uint32_t window, uint32_t heads,
                                             uint32_t kv_heads, uint32_t head_dim, uint32_t flags, void* stream) {
    FH_CHECK(q_dev && k_cache_dev && v_cache_dev && out_dev, "attn_prefill_sliding: null pointer");
    FH_CHECK(window >= 1, "attn_prefill_sliding: window must be at least 1");
    FH_CHECK((flags & ~FORGE_HIP_FLAG_EXACT) == 0, "attn_prefill_sliding: unknown flag bits");
    int32_t rc = check_attn_shape("attn_prefill_sliding", heads, kv_heads, head_dim);
    if (rc) return rc;
    if (flags & FORGE_HIP_FLAG_EXACT)
        launch_attn_exact(true, q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, nullptr, nullptr, M,
                          base_pos, nullptr, heads, kv_heads, head_dim, window, base_pos + M, nullptr, (hipStream_t)stream);
    else
        launch_attn_prefill(q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, M, base_pos, heads,
                            kv_heads, head_dim, window, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_attn_decode_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                    float* out_dev, uint32_t seq_len, uint32_t heads, uint32_t kv_heads,
                                    uint32_t head_dim, uint32_t flags, void* stream) {
    FH_CHECK(q_dev && k_cache_dev && v_cache_dev && out_dev, "attn_decode: null pointer");
    FH_CHECK(seq_len >= 1, "attn_decode: seq_len must be at least 1");
    FH_CHECK((flags & ~FORGE_HIP_FLAG_EXACT) == 0, "attn_decode: unknown flag bits");
    int32_t rc = check_attn_shape("attn_decode", heads, kv_heads, head_dim);
    if (rc) return rc;
    if (flags & FORGE_HIP_FLAG_EXACT) {
        // spread over (key block, head) workgroups when the cache is short enough for that kernel's tables
        const size_t xb = attn_exact_decode_workspace_bytes(heads, head_dim, seq_len);
        if (xb) {
            rc = g_attn.reserve(xb);
            if (rc) return rc;
        }
        launch_attn_exact(false, q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, nullptr,
                          nullptr, 1, seq_len - 1, nullptr, heads, kv_heads, head_dim, 0u, seq_len, xb ? g_attn.ptr() : nullptr,
                          (hipStream_t)stream);
    } else {
        rc = g_attn.reserve(attn_decode_workspace_bytes(heads, head_dim));
        if (rc) return rc;
        launch_attn_decode(q_dev, k_cache_dev, v_cache_dev, out_dev, nullptr, nullptr, seq_len, nullptr, heads, kv_heads,
                           head_dim, 0u, g_attn.ptr(), (hipStream_t)stream);
    }
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_attn_decode_f16kv_paged(const float* q_dev, const uint16_t* k_pool_dev, const uint16_t* v_pool_dev,
                                          const uint32_t* page_table_dev, uint32_t page_rows, float* out_dev, uint32_t seq_len,
                                          uint32_t heads, uint32_t kv_heads, uint32_t head_dim, void* stream) {
    FH_CHECK(q_dev && k_pool_dev && v_pool_dev && page_table_dev && out_dev, "attn_decode_paged: null pointer");
    FH_CHECK(seq_len >= 1, "attn_decode_paged: seq_len must be at least 1");
    int32_t rc = check_attn_shape("attn_decode_paged", heads, kv_heads, head_dim);
    if (rc) return rc;
    FH_CHECK(page_rows >= 1 && (page_rows & (page_rows - 1)) == 0, "attn_decode_paged: page_rows must be a power of two");
    FH_CHECK(attn_decode_paged_supported(seq_len, page_rows), "attn_decode_paged: pages too small for a sequence this long (more than 2048 table entries per split)");
    rc = g_attn.reserve(attn_decode_workspace_bytes(heads, head_dim));
    if (rc) return rc;
    launch_attn_decode_paged(q_dev, k_pool_dev, v_pool_dev, page_table_dev, page_rows, out_dev, seq_len, heads, kv_heads, head_dim,
                             g_attn.ptr(), (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_attn_decode_sliding_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                            float* out_dev, uint32_t seq_len, uint32_t window, uint32_t heads,
                                            uint32_t kv_heads, uint32_t head_dim, uint32_t flags, void* stream) {
    FH_CHECK(q_dev && k_cache_dev && v_cache_dev && out_dev, "attn_decode_sliding: null pointer");
    FH_CHECK(seq_len >= 1, "attn_decode_sliding: seq_len must be at least 1");
    FH_CHECK(window >= 1, "attn_decode_sliding: window must be at least 1");
    FH_CHECK((flags & ~FORGE_HIP_FLAG_EXACT) == 0, "attn_decode_sliding: unknown flag bits");
    int32_t rc = check_attn_shape("attn_decode_sliding", heads, kv_heads, head_dim);
    if (rc) return rc;
    if (flags & FORGE_HIP_FLAG_EXACT) {
        FH_CHECK(std::min(window, seq_len) <= attn_exact_max_window(), "attn_decode_sliding: the exact kernel keeps at most 12288 scores");
        launch_attn_exact(false, q_dev, heads * head_dim, k_cache_dev, v_cache_dev, out_dev, heads * head_dim, nullptr, nullptr, 1,
                          seq_len - 1, nullptr, heads, kv_heads, head_dim, window, seq_len, nullptr, (hipStream_t)stream);
    } else {
        rc = g_attn.reserve(attn_decode_workspace_bytes(heads, head_dim));
        if (rc) return rc;
        launch_attn_decode(q_dev, k_cache_dev, v_cache_dev, out_dev, nullptr, nullptr, seq_len, nullptr, heads, kv_heads, head_dim,
                           window, g_attn.ptr(), (hipStream_t)stream);
    }
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

int32_t forge_hip_expf_host(const float* x_host, uint64_t n, float* out_host) {
    FH_CHECK(x_host && out_host, "expf_host: null pointer");
    for (uint64_t i = 0; i < n; i++) out_host[i] = expf_ref<true>(x_host[i]);
    return FORGE_HIP_OK;
}

int32_t forge_hip_argmax(const float* x_dev, uint32_t n, uint32_t* out_dev, void* stream) {
    FH_CHECK(x_dev && out_dev && n >= 1, "argmax: null pointer or empty input");
    int32_t rc = g_attn.reserve(ARGMAX_BLOCKS * 8);
    if (rc) return rc;
    launch_argmax(x_dev, n, out_dev, g_attn.ptr(), nullptr, nullptr, nullptr, 1.0f, (hipStream_t)stream);
    FH_HIP(hipGetLastError());
    return FORGE_HIP_OK;
}

}  // extern "C"

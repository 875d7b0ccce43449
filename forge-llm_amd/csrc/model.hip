// extern "C" surface, part 2: the model object (MetalModel::{new, forward,
// forward_prefill_batch, reset}, metal:4209-5981; model::{forward, forward_prefill_batched},
// emit.rs:4029-5486) on one GPU.
//
// HBM layout: f32 embedding table; per layer two norm vectors and four quantised matrices
// as planes (q|k|v rows fused into one matrix, gate|up rows fused into one — the blob stores
// them back to back for exactly this, crates/forgellm-cli/src/main.rs:2722-2736); fp16 KV cache
// [layer][max_seq][kv_heads*head_dim] for K and V; cos/sin tables [max_seq][head_dim/2];
// f32 scratch for one decode step and for one prefill chunk.
//
// The decode step is captured once into a HIP graph (position and token live in device
// memory so the graph never changes) and replayed per token.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <memory>
#include <vector>

#include "common.h"

namespace fh {

constexpr uint32_t PREFILL_CHUNK = 4096;   // rows of scratch for batched prefill

struct Layer {
    float* attn_norm = nullptr;
    float* ffn_norm = nullptr;
    QWeight qkv, o, gate_up, down;
    QWeight q, k, v, gate, up;           // a model with a storage format per projection keeps these five apart (qkv, gate_up unused)
    // fast mode: the K-quant ones among q, k, v, o, gate, up, down as matrices of the int8 MFMA GEMM.  Neighbours of one format
    // that read the same rows (q, k, v; gate, up) share a twin: twin[i] then covers twin_span[i] projections from i on
    KqTwin twin[7];
    uint8_t twin_span[7] = {0, 0, 0, 0, 0, 0, 0};
    float* qkv_bias = nullptr;           // [QKS + 2 KV]: q | k | v bias, in the row order of the fused qkv matrix (FLAG_QKV_BIAS)
};

struct DevBuf {
    void* p = nullptr;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int32_t alloc(size_t n) {
        FH_HIP(hipMalloc(&p, n < 16 ? 16 : n));
        return FORGE_HIP_OK;
    }
    template <typename T> T* as() const { return reinterpret_cast<T*>(p); }
};

}  // namespace fh

using namespace fh;

struct forge_hip_model {
    forge_hip_config cfg{};
    uint32_t H = 0, I = 0, QKS = 0, KV = 0, QKV = 0, KMAX = 0;
    hipStream_t stream = nullptr;
    DevBuf embed, final_norm, norms;     // norms: [layers][2][H]
    DevBuf biases;                       // [layers][QKS + 2 KV] f32 (FLAG_QKV_BIAS)
    std::vector<Layer> layers;
    QWeight lm_head;
    DevBuf kcache, vcache;               // fp16 [layers][max_seq][KV]
    DevBuf cos_t, sin_t;
    // decode scratch
    DevBuf x, qkv, gu, logits, aq, asc, attn_ws, gemm_ws, state, argmax_ws;
    DevBuf counts;                       // u32 [vocab]: how often each token id has been fed since the last reset
    DevBuf page_table;                   // u32 [max_seq / page_rows]: pool page of each page of the sequence (paged KV cache)
    PageTable pt;                        // table == nullptr: the flat cache
    std::vector<uint32_t> page_table_host;
    float repeat_penalty = 1.0f;         // > 1: forward_greedy picks the maximum of the penalised logits
    // prefill scratch (chunk_rows rows)
    DevBuf px, pqkv, pattn, pgu, paq, pasc, paq2, pasc2, ptok;
    DevBuf pbsum, paq3, pasc3;           // K-quant twins: block sums of the activations (f32), the activations with every block twice
    bool mixed_twins = false;            // fast mode: K-quant projections of a prompt run on the MFMA GEMM (kquant_prefill.hip)
    bool prefill_fuse_quant = true;              // fast mode: attention writes int8 codes + scales (FORGE_HIP_FUSE=0: separate quantiser)
    bool mixed_fuse = true;          // K-quant projections over a normed row norm and quantise it themselves: a launch less, the same bits
    bool mixed_plain_layers = false;     // per-projection formats, but all seven are one of Q8_0 / Q4_0 (only the lm_head differs): decode layers run the uniform model's launches
    bool mixed_batched = false;                  // per-projection formats: the prompt runs in batches of rows (see enqueue_mixed_prefill_layer)
    bool prefill_fuse_silu = false;              // fast mode: the gate/up GEMM writes silu(gate) * up quantised (FORGE_HIP_FUSE=0: separate kernel)
    uint32_t chunk_rows = 0;
    // pinned host staging: [0] token, [1] next token, [2] position
    uint32_t* h_stage = nullptr;
    float* h_logits = nullptr;          // pinned: logits come home at PCIe speed and are copied to the caller's (pageable) buffer from here
    int64_t pos = 0;
    bool use_graph = true;
    bool fuse_norm = false, fuse_silu = false;   // fused GEMV prologue/epilogue variants fit LDS for this model
    hipGraphExec_t decode_graph = nullptr;
    PdState* pd = nullptr;               // the decode step as one resident kernel, when the shape is covered
    // ProjectionDTypes (ir.rs:410-421): q, k, v, o, gate, up, down each in its own storage format (GGML ids 8, 2, 12, 14).
    // `mixed`: they are not all cfg.wdtype, or the lm_head is a K-quant: every projection is then a GEMV launch of its own
    // and a prompt is walked token by token, as the reference does for such models (emit.rs:4530-4534, 4621-5040).
    bool mixed = false;
    uint32_t pd_types[7] = {0, 0, 0, 0, 0, 0, 0};
    // forward_profile / prefill_profile: one event pair per kernel launch, tagged with the stage of the
    // enclosing StageMark (ST_COUNT = outside any stage, not measured)
    int prof_cur = 0;
    std::vector<hipEvent_t> prof_ev;
    std::vector<int> prof_stage;
    size_t prof_used = 0;

    uint32_t* d_pos() const { return state.as<uint32_t>(); }
    uint32_t* d_token() const { return state.as<uint32_t>() + 1; }
    uint32_t* d_next() const { return state.as<uint32_t>() + 2; }
    uint16_t* kc(uint32_t l) const { return kcache.as<uint16_t>() + (size_t)l * cfg.max_seq * KV; }
    uint16_t* vc(uint32_t l) const { return vcache.as<uint16_t>() + (size_t)l * cfg.max_seq * KV; }

    ~forge_hip_model() {
        if (decode_graph) (void)hipGraphExecDestroy(decode_graph);
        pd_destroy(pd);
        for (hipEvent_t e : prof_ev) (void)hipEventDestroy(e);
        for (auto& L : layers) {
            qweight_free(&L.qkv); qweight_free(&L.o); qweight_free(&L.gate_up); qweight_free(&L.down);
            qweight_free(&L.q); qweight_free(&L.k); qweight_free(&L.v); qweight_free(&L.gate); qweight_free(&L.up);
            for (KqTwin& t : L.twin) kquant_twin_free(&t);
        }
        qweight_free(&lm_head);
        if (h_stage) (void)hipHostFree(h_stage);
        if (h_logits) (void)hipHostFree(h_logits);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

namespace {

// Stage ids of forward_profile / prefill_profile (the order of FORGE_HIP_STAGE_* in forge_hip.h).
enum Stage { ST_EMBED = 0, ST_RMSNORM, ST_QKV, ST_ROPE, ST_ATTN, ST_QUANT, ST_O, ST_GATE_UP, ST_SILU, ST_DOWN, ST_LM_HEAD,
             ST_ARGMAX, ST_COUNT };
static_assert(ST_COUNT == FORGE_HIP_NUM_STAGES, "stage table out of step with forge_hip.h");

// While the model is profiling, names the stage that the launches of one scope are counted under.
struct StageMark {
    forge_hip_model* m;
    int saved;
    StageMark(forge_hip_model* model, int stage) : m(model), saved(model->prof_cur) { m->prof_cur = stage; }
    ~StageMark() { m->prof_cur = saved; }
};

// Hands every kernel launch of a profiled pass its own pair of events (fh::launch attaches them to the
// dispatch) and remembers the stage it belongs to.
struct ModelProbe : LaunchProbe {
    forge_hip_model* m;
    explicit ModelProbe(forge_hip_model* model) : m(model) {
        m->prof_used = 0; m->prof_stage.clear(); m->prof_cur = ST_COUNT;
        launch_probe() = this;
    }
    ~ModelProbe() override { launch_probe() = nullptr; }
    bool next(hipEvent_t* start, hipEvent_t* stop) override {
        if (m->prof_cur == ST_COUNT) return false;
        if (m->prof_used + 2 > m->prof_ev.size()) {
            for (int i = 0; i < 2; i++) {
                hipEvent_t e = nullptr;
                if (hipEventCreate(&e) != hipSuccess) return false;
                m->prof_ev.push_back(e);
            }
        }
        *start = m->prof_ev[m->prof_used];
        *stop = m->prof_ev[m->prof_used + 1];
        m->prof_stage.push_back(m->prof_cur);
        m->prof_used += 2;
        return true;
    }
};

// Sum the kernels' device times per stage (milliseconds) after the stream has drained.
int32_t collect_profile(forge_hip_model* m, float* stage_ms, uint32_t* stage_launches) {
    for (int i = 0; i < ST_COUNT; i++) { stage_ms[i] = 0.f; if (stage_launches) stage_launches[i] = 0; }
    for (size_t i = 0; i * 2 < m->prof_used; i++) {
        float ms = 0.f;
        FH_HIP(hipEventElapsedTime(&ms, m->prof_ev[2 * i], m->prof_ev[2 * i + 1]));
        stage_ms[m->prof_stage[i]] += ms;
        if (stage_launches) stage_launches[m->prof_stage[i]] += 1;
    }
    return FORGE_HIP_OK;
}

bool is_kquant(uint32_t d) { return d == FORGE_HIP_Q4_K || d == FORGE_HIP_Q6_K; }
// bytes of an [n][k] matrix in a storage format (project.rs:195-213)
size_t wsize(uint32_t dtype, uint64_t n, uint64_t k) {
    if (is_kquant(dtype)) return (size_t)(n * (k / 256) * (dtype == FORGE_HIP_Q4_K ? 144 : 210));
    return (size_t)(n * (k / 32) * (dtype == FORGE_HIP_Q8_0 ? 34 : 18));
}

// The numbers sizes are computed from: formats, dimensions the kernels cover.
int32_t validate_shape(const forge_hip_config* c, bool lm_head_kquant_ok = false) {
    FH_CHECK(c, "config is null");
    FH_CHECK(c->wdtype == FORGE_HIP_Q8_0 || c->wdtype == FORGE_HIP_Q4_0, "wdtype must be Q8_0 (8) or Q4_0 (2)");
    FH_CHECK(c->lm_head_dtype == FORGE_HIP_Q8_0 || c->lm_head_dtype == FORGE_HIP_Q4_0 || (lm_head_kquant_ok && is_kquant(c->lm_head_dtype)),
             "lm_head_dtype must be Q8_0 (8) or Q4_0 (2) (Q4_K (12) / Q6_K (14): forge_hip_model_create_mixed)");
    FH_CHECK(c->hidden >= 32 && c->hidden % 32 == 0 && c->hidden <= 16352, "hidden must be a multiple of 32 in [32, 16352]");
    FH_CHECK(c->inter >= 32 && c->inter % 32 == 0, "inter must be a positive multiple of 32");
    FH_CHECK(c->layers >= 1 && c->vocab >= 1 && c->max_seq >= 1, "layers, vocab and max_seq must be positive");
    FH_CHECK(c->heads >= 1 && c->kv_heads >= 1 && c->heads % c->kv_heads == 0, "heads must be a positive multiple of kv_heads");
    FH_CHECK(attn_head_dim_supported(c->head_dim), "head_dim must be 64, 96 or 128");
    FH_CHECK(c->heads <= 16384 / 64 && gemv_k_supported(c->hidden) && gemv_k_supported(c->inter) && gemv_k_supported(c->heads * c->head_dim),
             "hidden, inter and heads*head_dim must be at most 16384");
    return FORGE_HIP_OK;
}

int32_t validate_cfg(const forge_hip_config* c, bool lm_head_kquant_ok = false) {
    const int32_t rc = validate_shape(c, lm_head_kquant_ok);
    if (rc) return rc;
    FH_CHECK((c->flags & ~(FORGE_HIP_FLAG_EXACT | FORGE_HIP_FLAG_QKV_BIAS)) == 0, "unknown bits in flags");
    // The reference switches to its non-flash attention (a different summation order) when
    // max_seq_len <= 512 (emit.rs:126-128); the order-faithful kernels follow the flash variants only.
    FH_CHECK(!(c->flags & FORGE_HIP_FLAG_EXACT) || c->max_seq > 512, "FORGE_HIP_FLAG_EXACT needs max_seq > 512");
    // a model with a window runs attention_sliding in the reference (emit.rs:598-627, 4156-4170), whose order-faithful
    // restatement keeps one row of scores in LDS
    FH_CHECK(!(c->flags & FORGE_HIP_FLAG_EXACT) || c->sliding_window == 0 || std::min(c->sliding_window, c->max_seq) <= attn_exact_max_window(),
             "FORGE_HIP_FLAG_EXACT with a sliding window needs min(sliding_window, max_seq) <= 12288");
    return FORGE_HIP_OK;
}

// Attention + O projection of one decode row; q is in qkv[0, QKS), attention output goes out quantised.
void enqueue_decode_attention(forge_hip_model* m, uint32_t l, const float* q, uint32_t q_stride) {
    const forge_hip_config& c = m->cfg;
    hipStream_t s = m->stream;
    const bool exact = (c.flags & FORGE_HIP_FLAG_EXACT) != 0;
    int8_t* aq = m->aq.as<int8_t>();
    uint16_t* asc = m->asc.as<uint16_t>();
    {
        StageMark t(m, ST_ATTN);
        if (exact)
            launch_attn_exact(false, q, q_stride, m->kc(l), m->vc(l), nullptr, m->QKS, aq, asc, 1, 0, m->d_pos(), c.heads,
                              c.kv_heads, c.head_dim, c.sliding_window, c.max_seq, m->attn_ws.p, s);
        else
            launch_attn_decode(q, m->kc(l), m->vc(l), nullptr, aq, asc, 0, m->d_pos(), c.heads, c.kv_heads, c.head_dim,
                               c.sliding_window, m->attn_ws.p, s, m->pt);
    }
    { StageMark t(m, ST_O); launch_gemv(m->layers[l].o, aq, asc, m->x.as<float>(), true, GemvOrder::MatmulVec, s); }
}

// One projection in its own storage format (matmul_call, emit.rs:3316-3334): y (=|+=) W * the quantised vector.
void gemv_any(const QWeight& w, const int8_t* aq, const uint16_t* asc, float* y, bool accumulate, GemvOrder order, hipStream_t s) {
    if (w.kquant()) launch_gemv_kquant(w, aq, asc, y, accumulate, s);
    else launch_gemv(w, aq, asc, y, accumulate, order, s);
}

// Projections that multiply quantise(rms_norm(x) * norm_w).  All K-quant: one launch that norms, quantises and multiplies.
// Otherwise the norm kernel first, then the K-quant ones among them in one launch and the others one each.
static void norm_gemv_group(forge_hip_model* m, const float* norm_w, const QWeight* const* w, float* const* y, uint32_t n, int stage) {
    hipStream_t s = m->stream;
    int8_t* aq = m->aq.as<int8_t>();
    uint16_t* asc = m->asc.as<uint16_t>();
    const QWeight* kw[3];
    float* ky[3];
    uint32_t nk = 0;
    for (uint32_t i = 0; i < n; i++)
        if (w[i]->kquant()) { kw[nk] = w[i]; ky[nk++] = y[i]; }
    if (nk == n && m->mixed_fuse) {
        StageMark t(m, stage);
        launch_gemv_kquant_multi_norm(kw, ky, nk, m->x.as<float>(), norm_w, m->cfg.rms_eps, s);
        return;
    }
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(m->x.as<float>(), norm_w, m->cfg.rms_eps, 1, m->H, nullptr, aq, asc, s); }
    StageMark t(m, stage);
    for (uint32_t i = 0; i < n; i++)
        if (!w[i]->kquant()) launch_gemv(*w[i], aq, asc, y[i], false, GemvOrder::MatmulVec, s);
    if (nk == 1) launch_gemv_kquant(*kw[0], aq, asc, ky[0], false, s);
    else if (nk > 1) launch_gemv_kquant_multi(kw, ky, nk, aq, asc, false, s);
}

// One decoder layer for ONE row of a model with a storage format per projection (model::forward, emit.rs:4029-4500, with
// the projection calls of emit.rs:4085-4100, 4200-4260): every projection a launch of its own kernel family.  The row sits
// at `pos` (pos_dev == nullptr: a token of a prompt) or at *pos_dev (a decode step).
void enqueue_mixed_layer(forge_hip_model* m, uint32_t l, uint32_t pos, const uint32_t* pos_dev) {
    const forge_hip_config& c = m->cfg;
    Layer& L = m->layers[l];
    hipStream_t s = m->stream;
    const uint32_t I = m->I, QKS = m->QKS, KV = m->KV, QKV = m->QKV;
    float* x = m->x.as<float>();
    float* qkv = m->qkv.as<float>();
    float* gu = m->gu.as<float>();
    int8_t* aq = m->aq.as<int8_t>();
    uint16_t* asc = m->asc.as<uint16_t>();
    const GemvOrder mv = GemvOrder::MatmulVec;
    const bool exact = (c.flags & FORGE_HIP_FLAG_EXACT) != 0;
    {
        const QWeight* w[3] = {&L.q, &L.k, &L.v};
        float* y[3] = {qkv, qkv + QKS, qkv + QKS + KV};
        norm_gemv_group(m, L.attn_norm, w, y, 3, ST_QKV);
    }
    {
        StageMark t(m, ST_ROPE);
        launch_rope_kv_store(qkv, qkv + QKS, qkv + QKS + KV, QKV, QKV, m->kc(l), m->vc(l), 1, pos, pos_dev, c.heads, c.kv_heads,
                             c.head_dim, m->cos_t.as<float>(), m->sin_t.as<float>(), L.qkv_bias, s, m->pt);
    }
    {
        StageMark t(m, ST_ATTN);
        // a model with a window: decode steps attend to the last `sliding_window` rows (attention_sliding, emit.rs:4156-4170); a
        // token of a prompt to every row so far through `attention` (emit.rs:4717-4720), which is attention_sliding's
        // arithmetic with a window that covers everything
        const uint32_t win = c.sliding_window == 0 ? 0u : pos_dev ? c.sliding_window : c.max_seq;
        if (exact)
            launch_attn_exact(false, qkv, QKS, m->kc(l), m->vc(l), nullptr, QKS, aq, asc, 1, pos, pos_dev, c.heads, c.kv_heads,
                              c.head_dim, win, c.max_seq, m->attn_ws.p, s);
        else
            launch_attn_decode(qkv, m->kc(l), m->vc(l), nullptr, aq, asc, pos + 1, pos_dev, c.heads, c.kv_heads, c.head_dim,
                               pos_dev ? c.sliding_window : 0u, m->attn_ws.p, s, m->pt);
    }
    { StageMark t(m, ST_O); gemv_any(L.o, aq, asc, x, true, mv, s); }
    {
        const QWeight* w[2] = {&L.gate, &L.up};
        float* y[2] = {gu, gu + I};
        norm_gemv_group(m, L.ffn_norm, w, y, 2, ST_GATE_UP);
    }
    { StageMark t(m, ST_SILU); launch_silu_mul(gu, gu + I, 1, I, 2 * I, nullptr, aq, asc, s); }
    { StageMark t(m, ST_DOWN); gemv_any(L.down, aq, asc, x, true, mv, s); }
}

// One decoder layer of the decode step (one row, position read from device memory).  Six launches
// when the fused GEMV variants fit LDS: [norm+quant | qkv GEMV | rope + KV write], attention split,
// attention merge + quant, [o GEMV | residual], [norm+quant | gate/up GEMV | silu*up + quant],
// [down GEMV | residual].
void enqueue_decode_layer(forge_hip_model* m, uint32_t l) {
    if (m->mixed && !m->mixed_plain_layers) { enqueue_mixed_layer(m, l, 0, m->d_pos()); return; }
    const forge_hip_config& c = m->cfg;
    Layer& L = m->layers[l];
    hipStream_t s = m->stream;
    const uint32_t H = m->H, I = m->I, QKS = m->QKS, KV = m->KV, QKV = m->QKV;
    float* x = m->x.as<float>();
    float* qkv = m->qkv.as<float>();
    float* gu = m->gu.as<float>();
    int8_t* aq = m->aq.as<int8_t>();
    uint16_t* asc = m->asc.as<uint16_t>();
    const GemvOrder mv = GemvOrder::MatmulVec;
    if (m->fuse_norm) {
        StageMark t(m, ST_QKV);
        launch_gemv_norm_rope_kv(L.qkv, x, L.attn_norm, c.rms_eps, L.qkv_bias, qkv, m->kc(l), m->vc(l), m->cos_t.as<float>(),
                                 m->sin_t.as<float>(), m->d_pos(), c.heads, c.kv_heads, c.head_dim, s, m->pt);
        // q now sits compact in qkv[0, QKS)
    } else {
        { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.attn_norm, c.rms_eps, 1, H, nullptr, aq, asc, s); }
        { StageMark t(m, ST_QKV); launch_gemv(L.qkv, aq, asc, qkv, false, mv, s); }
        {
            StageMark t(m, ST_ROPE);
            launch_rope_kv_store(qkv, qkv + QKS, qkv + QKS + KV, QKV, QKV, m->kc(l), m->vc(l), 1, 0, m->d_pos(), c.heads,
                                 c.kv_heads, c.head_dim, m->cos_t.as<float>(), m->sin_t.as<float>(), L.qkv_bias, s, m->pt);
        }
    }
    enqueue_decode_attention(m, l, qkv, QKS);
    if (m->fuse_silu) {
        StageMark t(m, ST_GATE_UP);
        launch_gemv_norm_silu_quant(L.gate_up, x, L.ffn_norm, c.rms_eps, aq, asc, s);
    } else {
        { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.ffn_norm, c.rms_eps, 1, H, nullptr, aq, asc, s); }
        { StageMark t(m, ST_GATE_UP); launch_gemv(L.gate_up, aq, asc, gu, false, mv, s); }
        { StageMark t(m, ST_SILU); launch_silu_mul(gu, gu + I, 1, I, 2 * I, nullptr, aq, asc, s); }
    }
    { StageMark t(m, ST_DOWN); launch_gemv(L.down, aq, asc, x, true, mv, s); }
}

// M rows through one projection of a model with a format per projection: K-quant matrices with the multi-row GEMV (each row
// has the one-row kernel's bits), Q8_0 / Q4_0 matrices with the order-faithful GEMM (plain activation codes, as the K-quant
// kernel takes them).
void matmul_rows_any(forge_hip_model* m, const QWeight& w, const int8_t* aq, const uint16_t* asc, uint32_t M, float* y, uint32_t ldy,
                     bool accumulate) {
    if (w.kquant()) launch_gemv_kquant_rows(w, aq, asc, M, y, ldy, accumulate, m->stream);
    else launch_gemm(w, aq, asc, M, y, ldy, accumulate, true, nullptr, m->stream, nullptr);
}

// One decoder layer for M rows of a model with a format per projection.  The reference walks such a prompt token by token
// (emit.rs:4530-4534, 4621-5040); the operations of a token depend on earlier tokens only through the K/V cache, so a layer can
// take all rows of a chunk at once: every projection row is the row the one-token kernel computes (K-quant matrices: bit for
// bit), the cache rows of the chunk are written before attention reads them.  Fast mode: MFMA attention.  Order-faithful mode
// (only when all seven projections are K-quants, so that no row's bits depend on the batch): attention_flash's own order per row.
void enqueue_mixed_prefill_layer(forge_hip_model* m, uint32_t l, uint32_t M, uint32_t base_pos) {
    const forge_hip_config& c = m->cfg;
    Layer& L = m->layers[l];
    hipStream_t s = m->stream;
    const uint32_t H = m->H, I = m->I, QKS = m->QKS, KV = m->KV, QKV = m->QKV;
    float* x = m->px.as<float>();
    float* qkv = m->pqkv.as<float>();
    float* gu = m->pgu.as<float>();
    float* attn = m->pattn.as<float>();
    int8_t* aq = m->paq.as<int8_t>();
    uint16_t* asc = m->pasc.as<uint16_t>();
    const bool exact = (c.flags & FORGE_HIP_FLAG_EXACT) != 0;
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.attn_norm, c.rms_eps, M, H, nullptr, aq, asc, s); }
    {
        StageMark t(m, ST_QKV);
        matmul_rows_any(m, L.q, aq, asc, M, qkv, QKV, false);
        matmul_rows_any(m, L.k, aq, asc, M, qkv + QKS, QKV, false);
        matmul_rows_any(m, L.v, aq, asc, M, qkv + QKS + KV, QKV, false);
    }
    {
        StageMark t(m, ST_ROPE);
        launch_rope_kv_store(qkv, qkv + QKS, qkv + QKS + KV, QKV, QKV, m->kc(l), m->vc(l), M, base_pos, nullptr, c.heads, c.kv_heads,
                             c.head_dim, m->cos_t.as<float>(), m->sin_t.as<float>(), L.qkv_bias, s, m->pt);
    }
    if (exact) {
        // (a model with a window: `attention` over all rows so far, see enqueue_mixed_layer)
        { StageMark t(m, ST_ATTN); launch_attn_exact(false, qkv, QKV, m->kc(l), m->vc(l), attn, QKS, nullptr, nullptr, M, base_pos, nullptr, c.heads, c.kv_heads, c.head_dim, c.sliding_window ? c.max_seq : 0u, c.max_seq, nullptr, s); }
        { StageMark t(m, ST_QUANT); launch_quantize_act(attn, M, QKS, aq, asc, s); }
    } else {
        StageMark t(m, ST_ATTN);
        launch_attn_prefill_quant(qkv, QKV, m->kc(l), m->vc(l), aq, asc, M, base_pos, c.heads, c.kv_heads, c.head_dim, 0u, s, false, m->pt);
    }
    { StageMark t(m, ST_O); matmul_rows_any(m, L.o, aq, asc, M, x, H, true); }
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.ffn_norm, c.rms_eps, M, H, nullptr, aq, asc, s); }
    {
        StageMark t(m, ST_GATE_UP);
        matmul_rows_any(m, L.gate, aq, asc, M, gu, 2 * I, false);
        matmul_rows_any(m, L.up, aq, asc, M, gu + I, 2 * I, false);
    }
    { StageMark t(m, ST_SILU); launch_silu_mul(gu, gu + I, M, I, 2 * I, nullptr, aq, asc, s); }
    { StageMark t(m, ST_DOWN); matmul_rows_any(m, L.down, aq, asc, M, x, H, true); }
}

// The projections ids[0..n) of a layer multiply the same quantised rows (aq, asc: depth K, odd blocks negated) and write
// neighbouring columns of y, all on the int8 MFMA GEMM (fast mode): Q8_0 / Q4_0 matrices as they are, K-quant matrices
// through their twins, which first get what they need of the rows (Q4_K: the scaled block sums; Q6_K: every block twice).
// silu_q: the group is gate, up under ONE twin and the launch writes quantize(silu(gate) * up) instead of y.
static void matmul_group_mfma(forge_hip_model* m, Layer& L, const int* ids, int n, const int8_t* aq, const uint16_t* asc, uint32_t M,
                              uint32_t K, float* y, uint32_t ldy, bool accumulate, int8_t* silu_q = nullptr, uint16_t* silu_sc = nullptr) {
    hipStream_t s = m->stream;
    const QWeight* w[7] = {&L.q, &L.k, &L.v, &L.o, &L.gate, &L.up, &L.down};
    bool sums = false, twice = false;
    for (int j = 0; j < n; j++)
        if (L.twin_span[ids[j]]) (L.twin[ids[j]].coef ? sums : twice) = true;
    if (sums) launch_act_block_sums(aq, asc, M, K, true, m->pbsum.as<float>(), s);
    if (twice) launch_act_twice(aq, asc, M, K, m->paq3.as<int8_t>(), m->pasc3.as<uint16_t>(), s);
    float* col = y;
    for (int j = 0; j < n;) {
        const int id = ids[j];
        if (!w[id]->kquant()) {
            launch_gemm(*w[id], aq, asc, M, col, ldy, accumulate, false, nullptr, s, m->gemm_ws.p);
            col += w[id]->N;
            j++;
            continue;
        }
        const KqTwin& t = L.twin[id];
        if (t.coef) launch_gemm(t.w, aq, asc, M, col, ldy, accumulate, false, nullptr, s, m->gemm_ws.p, silu_q, silu_sc, m->pbsum.as<float>(), t.coef);
        else launch_gemm(t.w, m->paq3.as<int8_t>(), m->pasc3.as<uint16_t>(), M, col, ldy, accumulate, false, nullptr, s, m->gemm_ws.p, silu_q, silu_sc);
        col += t.w.N;
        j += L.twin_span[id];
    }
}

// The same layer in fast mode with every projection on the int8 MFMA GEMM.  Block sums are exact integers as in the one-row
// kernels; the f32 accumulation order is the GEMM's, and the scale of a Q4_K block is rounded as kquant_prefill.hip says.
void enqueue_mixed_prefill_layer_mfma(forge_hip_model* m, uint32_t l, uint32_t M, uint32_t base_pos) {
    const forge_hip_config& c = m->cfg;
    Layer& L = m->layers[l];
    hipStream_t s = m->stream;
    const uint32_t H = m->H, I = m->I, QKS = m->QKS, KV = m->KV, QKV = m->QKV;
    float* x = m->px.as<float>();
    float* qkv = m->pqkv.as<float>();
    float* gu = m->pgu.as<float>();
    int8_t* aq = m->paq.as<int8_t>();
    uint16_t* asc = m->pasc.as<uint16_t>();
    static const int qkv_ids[3] = {0, 1, 2}, o_ids[1] = {3}, gu_ids[2] = {4, 5}, down_ids[1] = {6};
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.attn_norm, c.rms_eps, M, H, nullptr, aq, asc, s, true); }
    { StageMark t(m, ST_QKV); matmul_group_mfma(m, L, qkv_ids, 3, aq, asc, M, H, qkv, QKV, false); }
    {
        StageMark t(m, ST_ROPE);
        launch_rope_kv_store(qkv, qkv + QKS, qkv + QKS + KV, QKV, QKV, m->kc(l), m->vc(l), M, base_pos, nullptr, c.heads, c.kv_heads,
                             c.head_dim, m->cos_t.as<float>(), m->sin_t.as<float>(), L.qkv_bias, s, m->pt);
    }
    {
        StageMark t(m, ST_ATTN);
        launch_attn_prefill_quant(qkv, QKV, m->kc(l), m->vc(l), aq, asc, M, base_pos, c.heads, c.kv_heads, c.head_dim, 0u, s, true, m->pt);
    }
    { StageMark t(m, ST_O); matmul_group_mfma(m, L, o_ids, 1, aq, asc, M, QKS, x, H, true); }
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.ffn_norm, c.rms_eps, M, H, nullptr, aq, asc, s, true); }
    if (m->prefill_fuse_silu && L.twin_span[4] == 2 && gemm_silu_supported(L.twin[4].w, I, M)) {
        // gate and up under one twin: the GEMM's epilogue writes silu(gate) * up quantised, the [M][2 inter] floats never exist
        { StageMark t(m, ST_GATE_UP); matmul_group_mfma(m, L, gu_ids, 2, aq, asc, M, H, nullptr, 2 * I, false, m->paq2.as<int8_t>(), m->pasc2.as<uint16_t>()); }
        aq = m->paq2.as<int8_t>();
        asc = m->pasc2.as<uint16_t>();
    } else {
        { StageMark t(m, ST_GATE_UP); matmul_group_mfma(m, L, gu_ids, 2, aq, asc, M, H, gu, 2 * I, false); }
        { StageMark t(m, ST_SILU); launch_silu_mul(gu, gu + I, M, I, 2 * I, nullptr, aq, asc, s, true); }
    }
    { StageMark t(m, ST_DOWN); matmul_group_mfma(m, L, down_ids, 1, aq, asc, M, I, x, H, true); }
}

// One decoder layer of a batched prefill: M rows at positions base_pos.. .
void enqueue_prefill_layer(forge_hip_model* m, uint32_t l, uint32_t M, uint32_t base_pos) {
    const forge_hip_config& c = m->cfg;
    Layer& L = m->layers[l];
    hipStream_t s = m->stream;
    const uint32_t H = m->H, I = m->I, QKS = m->QKS, KV = m->KV, QKV = m->QKV;
    float* x = m->px.as<float>();
    float* qkv = m->pqkv.as<float>();
    float* gu = m->pgu.as<float>();
    float* attn = m->pattn.as<float>();
    int8_t* aq = m->paq.as<int8_t>();
    uint16_t* asc = m->pasc.as<uint16_t>();
    const bool exact = (c.flags & FORGE_HIP_FLAG_EXACT) != 0;      // the fast GEMM takes the odd blocks of its activations negated
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.attn_norm, c.rms_eps, M, H, nullptr, aq, asc, s, !exact); }
    { StageMark t(m, ST_QKV); launch_gemm(L.qkv, aq, asc, M, qkv, QKV, false, exact, nullptr, s, m->gemm_ws.p); }
    {
        StageMark t(m, ST_ROPE);
        launch_rope_kv_store(qkv, qkv + QKS, qkv + QKS + KV, QKV, QKV, m->kc(l), m->vc(l), M, base_pos, nullptr, c.heads,
                             c.kv_heads, c.head_dim, m->cos_t.as<float>(), m->sin_t.as<float>(), L.qkv_bias, s, m->pt);
    }
    if (exact) {
        { StageMark t(m, ST_ATTN); launch_attn_exact(true, qkv, QKV, m->kc(l), m->vc(l), attn, QKS, nullptr, nullptr, M, base_pos, nullptr, c.heads, c.kv_heads, c.head_dim, c.sliding_window, c.max_seq, nullptr, s); }
        { StageMark t(m, ST_QUANT); launch_quantize_act(attn, M, QKS, aq, asc, s); }
    } else if (m->prefill_fuse_quant) {
        // the attention kernel writes the o projection's quantised input itself
        StageMark t(m, ST_ATTN);
        launch_attn_prefill_quant(qkv, QKV, m->kc(l), m->vc(l), aq, asc, M, base_pos, c.heads, c.kv_heads, c.head_dim, c.sliding_window, s, true, m->pt);
    } else {
        { StageMark t(m, ST_ATTN); launch_attn_prefill(qkv, QKV, m->kc(l), m->vc(l), attn, QKS, M, base_pos, c.heads, c.kv_heads, c.head_dim, c.sliding_window, s, m->pt); }
        { StageMark t(m, ST_QUANT); launch_quantize_act(attn, M, QKS, aq, asc, s, true); }
    }
    { StageMark t(m, ST_O); launch_gemm(L.o, aq, asc, M, x, H, true, exact, nullptr, s, m->gemm_ws.p); }
    { StageMark t(m, ST_RMSNORM); launch_rmsnorm(x, L.ffn_norm, c.rms_eps, M, H, nullptr, aq, asc, s, !exact); }
    if (m->prefill_fuse_silu && gemm_silu_supported(L.gate_up, I, M)) {
        // the GEMM's epilogue writes silu(gate) * up quantised: the [M][2 I] floats never exist.  The kernel reads `aq` while
        // it runs, so its output goes to the second code buffer and the down projection reads that.
        StageMark t(m, ST_GATE_UP);
        launch_gemm(L.gate_up, aq, asc, M, nullptr, 2 * I, false, false, nullptr, s, m->gemm_ws.p, m->paq2.as<int8_t>(), m->pasc2.as<uint16_t>());
        aq = m->paq2.as<int8_t>();
        asc = m->pasc2.as<uint16_t>();
    } else {
        { StageMark t(m, ST_GATE_UP); launch_gemm(L.gate_up, aq, asc, M, gu, 2 * I, false, exact, nullptr, s, m->gemm_ws.p); }
        { StageMark t(m, ST_SILU); launch_silu_mul(gu, gu + I, M, I, 2 * I, nullptr, aq, asc, s, !exact); }
    }
    { StageMark t(m, ST_DOWN); launch_gemm(L.down, aq, asc, M, x, H, true, exact, nullptr, s, m->gemm_ws.p); }
}

// Final norm of one row + lm_head GEMV + argmax (+ pos/token advance when `advance`).
void enqueue_head(forge_hip_model* m, const float* xrow, bool after_prefill, bool advance) {
    hipStream_t s = m->stream;
    const GemvOrder order = after_prefill ? GemvOrder::LmHeadAfterPrefill : GemvOrder::LmHead;
    // The lm_head runs thousands of workgroups; repeating the norm prologue in each costs more than the
    // one extra launch, so the fused form is used only for small vocabularies.
    if (m->mixed) {
        // the per-token forward_prefill ends with the lm_head loop of forward (emit.rs:4880-5040), not with the batched one's
        {
            StageMark t(m, ST_RMSNORM);
            launch_rmsnorm(xrow, m->final_norm.as<float>(), m->cfg.rms_eps, 1, m->H, nullptr, m->aq.as<int8_t>(), m->asc.as<uint16_t>(), s);
        }
        {
            StageMark t(m, ST_LM_HEAD);
            gemv_any(m->lm_head, m->aq.as<int8_t>(), m->asc.as<uint16_t>(), m->logits.as<float>(), false, GemvOrder::LmHead, s);
        }
    } else if (m->fuse_norm && m->cfg.vocab <= 16384) {
        StageMark t(m, ST_LM_HEAD);
        launch_gemv_norm(m->lm_head, xrow, m->final_norm.as<float>(), m->cfg.rms_eps, m->logits.as<float>(), order, s);
    } else {
        {
            StageMark t(m, ST_RMSNORM);
            launch_rmsnorm(xrow, m->final_norm.as<float>(), m->cfg.rms_eps, 1, m->H, nullptr, m->aq.as<int8_t>(),
                           m->asc.as<uint16_t>(), s);
        }
        {
            StageMark t(m, ST_LM_HEAD);
            launch_gemv(m->lm_head, m->aq.as<int8_t>(), m->asc.as<uint16_t>(), m->logits.as<float>(), false, order, s);
        }
    }
    {
        StageMark t(m, ST_ARGMAX);
        // the token sampled right after a prefill is not penalised (project.rs:719-720), those inside the loop are (:742-744)
        const bool pen = !after_prefill && m->repeat_penalty > 1.0f;
        launch_argmax(m->logits.as<float>(), m->cfg.vocab, m->d_next(), m->argmax_ws.p, advance ? m->d_pos() : nullptr,
                      advance ? m->d_token() : nullptr, pen ? m->counts.as<uint32_t>() : nullptr, m->repeat_penalty, s);
    }
}

void enqueue_decode_step(forge_hip_model* m) {
    { StageMark t(m, ST_EMBED); launch_embedding(m->embed.as<float>(), m->d_token(), 1, m->H, m->x.as<float>(), m->counts.as<uint32_t>(), m->stream); }
    for (uint32_t l = 0; l < m->cfg.layers; l++) enqueue_decode_layer(m, l);
    enqueue_head(m, m->x.as<float>(), false, true);
}

int32_t run_decode_step(forge_hip_model* m, uint32_t token) {
    if (m->pd) return pd_enqueue(m->pd, false, token, m->stream);   // the token rides with the launch
    m->h_stage[0] = token;
    FH_HIP(hipMemcpyAsync(m->d_token(), &m->h_stage[0], 4, hipMemcpyHostToDevice, m->stream));
    if (m->use_graph && !m->decode_graph) {
        hipGraph_t g = nullptr;
        FH_HIP(hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal));
        enqueue_decode_step(m);
        hipError_t e = hipStreamEndCapture(m->stream, &g);
        if (e != hipSuccess || !g) return fail(FORGE_HIP_ERR_HIP, std::string("graph capture failed: ") + hipGetErrorString(e));
        e = hipGraphInstantiate(&m->decode_graph, g, nullptr, nullptr, 0);
        (void)hipGraphDestroy(g);
        if (e != hipSuccess) { m->decode_graph = nullptr; return fail(FORGE_HIP_ERR_HIP, std::string("graph instantiate failed: ") + hipGetErrorString(e)); }
    }
    if (m->decode_graph) FH_HIP(hipGraphLaunch(m->decode_graph, m->stream));
    else { enqueue_decode_step(m); FH_HIP(hipGetLastError()); }
    return FORGE_HIP_OK;
}

// Reads back {next token, abort flag} after a decode step and waits for the stream.
int32_t finish_decode_step(forge_hip_model* m) {
    FH_HIP(hipMemcpyAsync(&m->h_stage[4], m->d_next(), 8, hipMemcpyDeviceToHost, m->stream));
    FH_HIP(hipStreamSynchronize(m->stream));
    if (m->pd) return pd_after_sync(m->pd, m->h_stage[5], m->stream);
    return FORGE_HIP_OK;
}

// Enqueues a decode step.  The position is counted as advanced here; a step that turns out not to have happened (the
// resident kernel gave up) is taken back by step_failed().
int32_t forward_common(forge_hip_model* m, uint32_t token) {
    FH_CHECK(m, "model is null");
    if (m->pos >= (int64_t)m->cfg.max_seq) return fail(FORGE_HIP_ERR_POSITION, "KV cache is full (pos == max_seq)");
    if (token >= m->cfg.vocab) return fail(FORGE_HIP_ERR_POSITION, "token id out of range");
    int32_t rc = run_decode_step(m, token);
    if (rc) return rc;
    m->pos += 1;
    return FORGE_HIP_OK;
}

// finish_decode_step() with the host's view put back in line with the device's when the step failed: the device position
// was not advanced, so neither is the host's, and the same token can be fed again.
int32_t finish_or_undo(forge_hip_model* m) {
    const int32_t rc = finish_decode_step(m);
    if (rc && m->pos > 0) m->pos -= 1;
    return rc;
}

}  // namespace

namespace fh {
int32_t validate_config_shape(const forge_hip_config* c) { return validate_shape(c); }
}  // namespace fh

extern "C" {

uint64_t forge_hip_weights_nbytes(const forge_hip_config* c) {
    if (!c) return 0;
    // every field is a caller's (or a file's) 32-bit number: the sum is formed with checked arithmetic and is 0 when
    // it does not fit 64 bits -- no blob has that length, so forge_hip_model_create refuses such a configuration
    bool over = false;
    auto mul = [&](uint64_t a, uint64_t b) { uint64_t r = 0; over = over || __builtin_mul_overflow(a, b, &r); return r; };
    auto add = [&](uint64_t a, uint64_t b) { uint64_t r = 0; over = over || __builtin_add_overflow(a, b, &r); return r; };
    auto w = [&](uint32_t t, uint64_t n, uint64_t k) { return mul(mul(n, k / 32), t == FORGE_HIP_Q8_0 ? 34 : 18); };
    const uint64_t H = c->hidden, I = c->inter, QKS = mul(c->heads, c->head_dim), KV = mul(c->kv_heads, c->head_dim);
    uint64_t per_layer = add(mul(H, 8), add(add(w(c->wdtype, QKS, H), mul(2, w(c->wdtype, KV, H))), w(c->wdtype, H, QKS)));
    per_layer = add(per_layer, add(mul(2, w(c->wdtype, I, H)), w(c->wdtype, H, I)));
    if (c->flags & FORGE_HIP_FLAG_QKV_BIAS) per_layer = add(per_layer, mul(add(QKS, mul(2, KV)), 4));
    const uint64_t total = add(add(mul(mul(c->vocab, H), 4), mul(c->layers, per_layer)), add(mul(H, 4), w(c->lm_head_dtype, c->vocab, H)));
    return over ? 0 : total;
}

uint64_t forge_hip_weights_nbytes_mixed(const forge_hip_config* c, const uint32_t* pd) {
    if (!c || !pd) return 0;
    bool over = false;
    auto mul = [&](uint64_t a, uint64_t b) { uint64_t r = 0; over = over || __builtin_mul_overflow(a, b, &r); return r; };
    auto add = [&](uint64_t a, uint64_t b) { uint64_t r = 0; over = over || __builtin_add_overflow(a, b, &r); return r; };
    auto w = [&](uint32_t t, uint64_t n, uint64_t k) {
        if (is_kquant(t)) return mul(mul(n, k / 256), t == FORGE_HIP_Q4_K ? 144 : 210);
        return mul(mul(n, k / 32), t == FORGE_HIP_Q8_0 ? 34 : 18);
    };
    const uint64_t H = c->hidden, I = c->inter, QKS = mul(c->heads, c->head_dim), KV = mul(c->kv_heads, c->head_dim);
    uint64_t per_layer = add(mul(H, 8), add(add(w(pd[0], QKS, H), add(w(pd[1], KV, H), w(pd[2], KV, H))), w(pd[3], H, QKS)));
    per_layer = add(per_layer, add(add(w(pd[4], I, H), w(pd[5], I, H)), w(pd[6], H, I)));
    if (c->flags & FORGE_HIP_FLAG_QKV_BIAS) per_layer = add(per_layer, mul(add(QKS, mul(KV, 2)), 4));       // q | k | v bias, project.rs:286-292
    const uint64_t total = add(add(mul(mul(c->vocab, H), 4), mul(c->layers, per_layer)), add(mul(H, 4), w(c->lm_head_dtype, c->vocab, H)));
    return over ? 0 : total;
}

static int32_t model_create_impl(const forge_hip_config* cfg, const uint32_t* pd, const uint8_t* blob, uint64_t nbytes, forge_hip_model** out);

int32_t forge_hip_model_create(const forge_hip_config* cfg, const uint8_t* blob, uint64_t nbytes, forge_hip_model** out) {
    return model_create_impl(cfg, nullptr, blob, nbytes, out);
}

int32_t forge_hip_model_create_mixed(const forge_hip_config* cfg, const uint32_t* proj_dtypes, const uint8_t* blob, uint64_t nbytes,
                                     forge_hip_model** out) {
    FH_CHECK(out, "model_create_mixed: null out");
    *out = nullptr;
    FH_CHECK(cfg && proj_dtypes, "model_create_mixed: null pointer");
    bool mixed = is_kquant(cfg->lm_head_dtype);
    for (int i = 0; i < 7; i++) {
        const uint32_t d = proj_dtypes[i];
        FH_CHECK(d == FORGE_HIP_Q8_0 || d == FORGE_HIP_Q4_0 || is_kquant(d), "model_create_mixed: a projection's format must be Q8_0 (8), Q4_0 (2), Q4_K (12) or Q6_K (14)");
        mixed = mixed || d != cfg->wdtype;
    }
    return model_create_impl(cfg, mixed ? proj_dtypes : nullptr, blob, nbytes, out);
}

static int32_t model_create_impl(const forge_hip_config* cfg, const uint32_t* pd, const uint8_t* blob, uint64_t nbytes, forge_hip_model** out) {
    FH_CHECK(out, "model_create: null out");
    *out = nullptr;
    int32_t rc = validate_cfg(cfg, pd != nullptr);
    if (rc) return rc;
    FH_CHECK(blob, "model_create: null weights");
    if (pd) {
        // what the per-projection path covers: K-quant matrices over K % 256 == 0.  (A model with a sliding window: its prompt
        // rows see ALL earlier positions -- the reference's token-by-token prompt calls `attention`, not `attention_sliding`,
        // emit.rs:4717-4720 with use_flash_attention false for such a model, emit.rs:126-128 -- and only decode steps the window.)
        FH_CHECK(!(cfg->flags & FORGE_HIP_FLAG_EXACT) || cfg->sliding_window == 0 || cfg->max_seq <= attn_exact_max_window(),
                 "model_create_mixed: FORGE_HIP_FLAG_EXACT with a sliding window needs max_seq <= 12288 (a prompt row's scores sit in LDS)");
        const uint32_t kin[7] = {cfg->hidden, cfg->hidden, cfg->hidden, cfg->heads * cfg->head_dim, cfg->hidden, cfg->hidden, cfg->inter};
        for (int i = 0; i < 7; i++)
            FH_CHECK(!is_kquant(pd[i]) || kquant_k_supported(kin[i]), "model_create_mixed: a K-quant projection needs an input width that is a multiple of 256, at most 16384");
        FH_CHECK(!is_kquant(cfg->lm_head_dtype) || kquant_k_supported(cfg->hidden), "model_create_mixed: a K-quant lm_head needs hidden to be a multiple of 256");
    }
    const uint64_t want = pd ? forge_hip_weights_nbytes_mixed(cfg, pd) : forge_hip_weights_nbytes(cfg);
    if (nbytes != want)
        return fail(FORGE_HIP_ERR_BLOB_SIZE, "weights blob is " + std::to_string(nbytes) + " bytes, config needs " + std::to_string(want));
    if (forge_hip_device_count() < 1) return fail(FORGE_HIP_ERR_NO_DEVICE, "no HIP device");
    attn_decode_noalloc_prepare();

    std::unique_ptr<forge_hip_model> m(new forge_hip_model());
    m->cfg = *cfg;
    m->mixed = pd != nullptr;
    if (pd) {
        memcpy(m->pd_types, pd, sizeof(m->pd_types));
        // The prompt runs in batches of rows when no row's bits can depend on the batch in the mode asked for: always in the fast
        // mode; in the order-faithful mode when all seven projections are K-quants (their multi-row kernel gives every row the
        // one-row kernel's bits).  FORGE_HIP_MIXED_BATCH=0: token by token, as the reference walks such a prompt.
        bool all_k = true;
        for (int i = 0; i < 7; i++) all_k = all_k && is_kquant(pd[i]);
        const char* benv = getenv("FORGE_HIP_MIXED_BATCH");
        const char* fenv = getenv("FORGE_HIP_MIXED_FUSE");
        m->mixed_fuse = !(fenv && fenv[0] == '0');
        m->mixed_batched = !(benv && benv[0] == '0') && (all_k || !(cfg->flags & FORGE_HIP_FLAG_EXACT));
    }
    const uint32_t H = m->H = cfg->hidden, I = m->I = cfg->inter;
    const uint32_t QKS = m->QKS = cfg->heads * cfg->head_dim, KV = m->KV = cfg->kv_heads * cfg->head_dim;
    m->QKV = QKS + 2 * KV;
    m->KMAX = std::max(std::max(H, I), QKS);
    const char* genv = getenv("FORGE_HIP_GRAPH");
    m->use_graph = !(genv && genv[0] == '0');
    const char* fenv = getenv("FORGE_HIP_FUSE");
    const bool fuse_ok = !(fenv && fenv[0] == '0');
    // seven projections of one plain format (the lm_head is what differs): the layers of a decode step are the uniform model's
    bool plain_layers = pd != nullptr && !is_kquant(pd[0]);
    for (int i = 1; i < 7 && plain_layers; i++) plain_layers = pd[i] == pd[0];
    m->mixed_plain_layers = plain_layers;
    m->fuse_norm = fuse_ok && (!pd || plain_layers) && gemv_norm_fusable(H);
    m->fuse_silu = fuse_ok && (!pd || plain_layers) && gemv_silu_fusable(H);
    m->prefill_fuse_quant = fuse_ok;
    // FORGE_HIP_FUSE_SILU_GEMM=0: the gate/up GEMM writes floats and silu_mul + the quantiser run as a kernel of their own
    // (the fused epilogue uses the hardware exponential and reciprocals: same values to the fast mode's tolerance, not the same bits)
    const char* senv2 = getenv("FORGE_HIP_FUSE_SILU_GEMM");
    m->prefill_fuse_silu = fuse_ok && !(senv2 && senv2[0] == '0') && !(cfg->flags & FORGE_HIP_FLAG_EXACT) && !pd && I % 64 == 0;
    FH_HIP(hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking));
    FH_HIP(hipHostMalloc((void**)&m->h_stage, 64, hipHostMallocDefault));
    FH_HIP(hipHostMalloc((void**)&m->h_logits, (size_t)cfg->vocab * 4, hipHostMallocDefault));

    // ---- weights (blob order: project.rs:342-407) ----
    const uint8_t* p = blob;
    rc = m->embed.alloc((size_t)cfg->vocab * H * 4);
    if (rc) return rc;
    FH_HIP(hipMemcpy(m->embed.p, p, (size_t)cfg->vocab * H * 4, hipMemcpyHostToDevice));
    p += (size_t)cfg->vocab * H * 4;
    rc = m->norms.alloc((size_t)cfg->layers * 2 * H * 4);
    if (rc) return rc;
    m->layers.resize(cfg->layers);
    const bool has_bias = (cfg->flags & FORGE_HIP_FLAG_QKV_BIAS) != 0;
    if (has_bias) {
        rc = m->biases.alloc((size_t)cfg->layers * m->QKV * 4);
        if (rc) return rc;
    }
    const uint32_t wt = cfg->wdtype;
    for (uint32_t l = 0; l < cfg->layers; l++) {
        Layer& L = m->layers[l];
        L.attn_norm = m->norms.as<float>() + (size_t)(2 * l) * H;
        L.ffn_norm = L.attn_norm + H;
        FH_HIP(hipMemcpy(L.attn_norm, p, H * 4, hipMemcpyHostToDevice));
        p += H * 4;
        if (pd) {
            // Q8_0 / Q4_0 neighbours of one format (q, k, v; gate, up) go up as one matrix, as in the uniform model (the
            // resident decode kernel multiplies them in one phase); the per-projection launches see its row ranges
            auto rows_of = [](const QWeight& whole, uint32_t row0, uint32_t rows) {
                QWeight v;
                v.wdtype = whole.wdtype; v.K = whole.K; v.N = rows;
                v.qs = whole.qs + (size_t)row0 * whole.qs_row_bytes();
                v.scales = whole.scales + (size_t)row0 * (whole.K / 32);
                return v;                                     // owns stays false
            };
            if (!is_kquant(pd[0]) && pd[0] == pd[1] && pd[1] == pd[2]) {
                if ((rc = qweight_upload(pd[0], p, H, m->QKV, &L.qkv))) return rc;
                p += wsize(pd[0], m->QKV, H);
                L.q = rows_of(L.qkv, 0, QKS); L.k = rows_of(L.qkv, QKS, KV); L.v = rows_of(L.qkv, QKS + KV, KV);
            } else {
                if ((rc = qweight_upload(pd[0], p, H, QKS, &L.q))) return rc;
                p += wsize(pd[0], QKS, H);
                if ((rc = qweight_upload(pd[1], p, H, KV, &L.k))) return rc;
                p += wsize(pd[1], KV, H);
                if ((rc = qweight_upload(pd[2], p, H, KV, &L.v))) return rc;
                p += wsize(pd[2], KV, H);
            }
            if (has_bias) {                                   // q_bias | k_bias | v_bias, project.rs:286-292
                L.qkv_bias = m->biases.as<float>() + (size_t)l * m->QKV;
                FH_HIP(hipMemcpy(L.qkv_bias, p, (size_t)m->QKV * 4, hipMemcpyHostToDevice));
                p += (size_t)m->QKV * 4;
            }
            if ((rc = qweight_upload(pd[3], p, QKS, H, &L.o))) return rc;
            p += wsize(pd[3], H, QKS);
            FH_HIP(hipMemcpy(L.ffn_norm, p, H * 4, hipMemcpyHostToDevice));
            p += H * 4;
            if (!is_kquant(pd[4]) && pd[4] == pd[5]) {
                if ((rc = qweight_upload(pd[4], p, H, 2 * I, &L.gate_up))) return rc;
                p += wsize(pd[4], 2 * (uint64_t)I, H);
                L.gate = rows_of(L.gate_up, 0, I); L.up = rows_of(L.gate_up, I, I);
            } else {
                if ((rc = qweight_upload(pd[4], p, H, I, &L.gate))) return rc;
                p += wsize(pd[4], I, H);
                if ((rc = qweight_upload(pd[5], p, H, I, &L.up))) return rc;
                p += wsize(pd[5], I, H);
            }
            if ((rc = qweight_upload(pd[6], p, I, H, &L.down))) return rc;
            p += wsize(pd[6], H, I);
            continue;
        }
        // q, k, v are adjacent in the blob and all have K = hidden: upload as one matrix.
        rc = qweight_upload(wt, p, H, m->QKV, &L.qkv);
        if (rc) return rc;
        p += wsize(wt, m->QKV, H);
        if (has_bias) {                                       // q_bias | k_bias | v_bias, project.rs:286-292
            L.qkv_bias = m->biases.as<float>() + (size_t)l * m->QKV;
            FH_HIP(hipMemcpy(L.qkv_bias, p, (size_t)m->QKV * 4, hipMemcpyHostToDevice));
            p += (size_t)m->QKV * 4;
        }
        rc = qweight_upload(wt, p, QKS, H, &L.o);
        if (rc) return rc;
        p += wsize(wt, H, QKS);
        FH_HIP(hipMemcpy(L.ffn_norm, p, H * 4, hipMemcpyHostToDevice));
        p += H * 4;
        rc = qweight_upload(wt, p, H, 2 * I, &L.gate_up);   // gate rows then up rows, adjacent in the blob
        if (rc) return rc;
        p += wsize(wt, 2 * (uint64_t)I, H);
        rc = qweight_upload(wt, p, I, H, &L.down);
        if (rc) return rc;
        p += wsize(wt, H, I);
    }
    rc = m->final_norm.alloc(H * 4);
    if (rc) return rc;
    FH_HIP(hipMemcpy(m->final_norm.p, p, H * 4, hipMemcpyHostToDevice));
    p += H * 4;
    rc = qweight_upload(cfg->lm_head_dtype, p, H, cfg->vocab, &m->lm_head);
    if (rc) return rc;

    // ---- KV cache, rope tables ----
    const size_t cache_bytes = (size_t)cfg->layers * cfg->max_seq * KV * 2;
    if ((rc = m->kcache.alloc(cache_bytes)) || (rc = m->vcache.alloc(cache_bytes))) return rc;
    {
        const uint32_t half = cfg->head_dim / 2;
        std::vector<float> ct((size_t)cfg->max_seq * half), st((size_t)cfg->max_seq * half);
        for (uint32_t i = 0; i < half; i++) {
            // rope_freqs, emit.rs:501-504; angle and sin_cos, emit.rs:514-516 — host C library
            const float f = 1.0f / powf(cfg->rope_theta, 2.0f * (float)i / (float)cfg->head_dim);
            for (uint32_t t = 0; t < cfg->max_seq; t++) {
                const float a = (float)t * f;
                ct[(size_t)t * half + i] = cosf(a);
                st[(size_t)t * half + i] = sinf(a);
            }
        }
        if ((rc = m->cos_t.alloc(ct.size() * 4)) || (rc = m->sin_t.alloc(st.size() * 4))) return rc;
        FH_HIP(hipMemcpy(m->cos_t.p, ct.data(), ct.size() * 4, hipMemcpyHostToDevice));
        FH_HIP(hipMemcpy(m->sin_t.p, st.data(), st.size() * 4, hipMemcpyHostToDevice));
    }

    // ---- scratch ----
    if ((rc = m->x.alloc(H * 4)) || (rc = m->qkv.alloc(m->QKV * 4)) || (rc = m->gu.alloc(2 * (size_t)I * 4)) ||
        (rc = m->logits.alloc((size_t)cfg->vocab * 4)) || (rc = m->aq.alloc(m->KMAX)) ||
        (rc = m->asc.alloc(m->KMAX / 32 * 2)) || (rc = m->attn_ws.alloc(std::max(attn_decode_workspace_bytes(cfg->heads, cfg->head_dim), (cfg->flags & FORGE_HIP_FLAG_EXACT) ? attn_exact_decode_workspace_bytes(cfg->heads, cfg->head_dim, cfg->max_seq) : (size_t)0))) ||
        (rc = m->state.alloc(64)) || (rc = m->argmax_ws.alloc(ARGMAX_BLOCKS * 8)) || (rc = m->counts.alloc((size_t)cfg->vocab * 4)))
        return rc;
    FH_HIP(hipMemset(m->state.p, 0, 64));
    FH_HIP(hipMemset(m->counts.p, 0, (size_t)cfg->vocab * 4));
    const uint32_t R = m->chunk_rows = std::min(PREFILL_CHUNK, cfg->max_seq);
    if ((rc = m->px.alloc((size_t)R * H * 4)) || (rc = m->pqkv.alloc((size_t)R * m->QKV * 4)) ||
        (rc = m->pattn.alloc((size_t)R * QKS * 4)) || (rc = m->pgu.alloc((size_t)R * 2 * I * 4)) ||
        (rc = m->paq.alloc((size_t)R * m->KMAX)) || (rc = m->pasc.alloc((size_t)R * (m->KMAX / 32) * 2)) ||
        (rc = m->ptok.alloc((size_t)R * 4)))
        return rc;
    if (m->prefill_fuse_silu && ((rc = m->paq2.alloc((size_t)R * I)) || (rc = m->pasc2.alloc((size_t)R * (I / 32) * 2)))) return rc;
    const bool fuse_silu_twins = fuse_ok && !(senv2 && senv2[0] == '0') && I % 64 == 0;
    // fast mode: the prefill GEMMs may cut left-over tiles along K (FORGE_HIP_GEMM_SPLIT=0: never)
    const char* senv = getenv("FORGE_HIP_GEMM_SPLIT");
    if (!(cfg->flags & FORGE_HIP_FLAG_EXACT) && !(senv && senv[0] == '0')) {
        if ((rc = m->gemm_ws.alloc(gemm_split_workspace_bytes()))) return rc;
        FH_HIP(hipMemset(m->gemm_ws.p, 0, gemm_split_workspace_bytes()));
    }
    // fast mode, prompt in batches: the K-quant projections get twins for the MFMA GEMM (FORGE_HIP_KQ_MFMA=0: the multi-row
    // GEMV, whose rows are the one-row kernel's bit for bit).  A matrix with a block scale outside the GEMM's scale
    // arithmetic keeps the whole model on the GEMV.
    const char* tenv = getenv("FORGE_HIP_KQ_MFMA");
    if (pd && m->mixed_batched && !(cfg->flags & FORGE_HIP_FLAG_EXACT) && !(tenv && tenv[0] == '0')) {
        bool all = true, any_k = false;
        static const int groups[4][4] = {{0, 1, 2, -1}, {3, -1, -1, -1}, {4, 5, -1, -1}, {6, -1, -1, -1}};
        for (uint32_t l = 0; l < cfg->layers && all; l++) {
            Layer& L = m->layers[l];
            const QWeight* w[7] = {&L.q, &L.k, &L.v, &L.o, &L.gate, &L.up, &L.down};
            for (int g = 0; g < 4 && all; g++)
                for (int j = 0; groups[g][j] >= 0 && all;) {
                    const int id = groups[g][j];
                    if (!w[id]->kquant()) { j++; continue; }
                    // this projection and the neighbours of its format that follow it in the group
                    const QWeight* part[3];
                    uint32_t span = 0;
                    while (groups[g][j] >= 0 && w[groups[g][j]]->wdtype == w[id]->wdtype) part[span++] = w[groups[g][j++]];
                    any_k = true;
                    bool covered = false;
                    if ((rc = kquant_twin_create(part, span, &L.twin[id], &covered, m->stream))) return rc;
                    L.twin_span[id] = (uint8_t)span;
                    all = covered;
                }
        }
        if (!all)
            for (auto& L : m->layers)
                for (int i = 0; i < 7; i++) { kquant_twin_free(&L.twin[i]); L.twin_span[i] = 0; }
        m->mixed_twins = all;
        if (all && any_k &&
            ((rc = m->pbsum.alloc((size_t)R * (m->KMAX / 32) * 4)) || (rc = m->paq3.alloc((size_t)R * m->KMAX * 2)) ||
             (rc = m->pasc3.alloc((size_t)R * (m->KMAX / 32) * 2 * 2))))
            return rc;
        if (all && fuse_silu_twins) {
            m->prefill_fuse_silu = true;
            if ((rc = m->paq2.alloc((size_t)R * I)) || (rc = m->pasc2.alloc((size_t)R * (I / 32) * 2))) return rc;
        }
    }
    const char* penv = getenv("FORGE_HIP_PERSIST");
    const char* kenv = getenv("FORGE_HIP_PD_KQUANT");
    if (pd && !(penv && penv[0] == '0') && !(kenv && kenv[0] == '0')) {
        // a model whose matrices are all Q4_K / Q6_K (q and k of one format, gate and up too) runs its decode step as the
        // resident kernel with K-quant weight units (a second copy of the matrices in the kernel's layout): bit-identical to
        // the kernel sequence in the ordered variant.  FORGE_HIP_PD_KQUANT=0 keeps the kernel sequence for such models;
        // pd_create leaves m->pd null for any other mix.
        bool all_k = is_kquant(cfg->lm_head_dtype);
        for (int i = 0; i < 7; i++) all_k = all_k && is_kquant(pd[i]);
        if (all_k && pd[0] == pd[1] && pd[4] == pd[5]) {
            std::vector<PdLayerIn> pl(cfg->layers);
            for (uint32_t l = 0; l < cfg->layers; l++) {
                Layer& L = m->layers[l];
                pl[l] = PdLayerIn{nullptr, &L.o, nullptr, &L.down, L.attn_norm, L.ffn_norm, m->kc(l), m->vc(l), &L.q, &L.k, &L.v, &L.gate, &L.up};
            }
            rc = pd_create(*cfg, pl, m->lm_head, m->embed.as<float>(), m->final_norm.as<float>(), m->cos_t.as<float>(),
                           m->sin_t.as<float>(), m->logits.as<float>(), m->state.as<uint32_t>(), m->counts.as<uint32_t>(),
                           has_bias ? m->biases.as<float>() : nullptr, &m->pd);
            if (rc) return rc;
        }
    }
    if (pd && !m->pd && !(penv && penv[0] == '0') && !(kenv && kenv[0] == '0') && cfg->lm_head_dtype == FORGE_HIP_Q6_K && !is_kquant(pd[0])) {
        // seven Q8_0 or seven Q4_0 projections under a Q6_K lm_head (what llama.cpp writes for its Q4_0 / Q8_0 recipes with
        // a K-quant output matrix): the uniform model's resident kernel with the lm_head as K-quant weight units
        bool same = true;
        for (int i = 1; i < 7; i++) same = same && pd[i] == pd[0];
        if (same) {
            forge_hip_config c2 = *cfg;
            c2.wdtype = pd[0];
            std::vector<PdLayerIn> pl(cfg->layers);
            for (uint32_t l = 0; l < cfg->layers; l++) {
                Layer& L = m->layers[l];
                pl[l] = PdLayerIn{&L.qkv, &L.o, &L.gate_up, &L.down, L.attn_norm, L.ffn_norm, m->kc(l), m->vc(l)};
            }
            rc = pd_create(c2, pl, m->lm_head, m->embed.as<float>(), m->final_norm.as<float>(), m->cos_t.as<float>(),
                           m->sin_t.as<float>(), m->logits.as<float>(), m->state.as<uint32_t>(), m->counts.as<uint32_t>(),
                           has_bias ? m->biases.as<float>() : nullptr, &m->pd);
            if (rc) return rc;
        }
    }
    if (!pd && !(penv && penv[0] == '0')) {       // uniform Q8_0 / Q4_0 models
        std::vector<PdLayerIn> pl(cfg->layers);
        for (uint32_t l = 0; l < cfg->layers; l++) {
            Layer& L = m->layers[l];
            pl[l] = PdLayerIn{&L.qkv, &L.o, &L.gate_up, &L.down, L.attn_norm, L.ffn_norm, m->kc(l), m->vc(l)};
        }
        rc = pd_create(*cfg, pl, m->lm_head, m->embed.as<float>(), m->final_norm.as<float>(), m->cos_t.as<float>(),
                       m->sin_t.as<float>(), m->logits.as<float>(), m->state.as<uint32_t>(), m->counts.as<uint32_t>(),
                       has_bias ? m->biases.as<float>() : nullptr, &m->pd);
        if (rc) return rc;
    }
    FH_HIP(hipDeviceSynchronize());
    *out = m.release();
    return FORGE_HIP_OK;
}

void forge_hip_model_destroy(forge_hip_model* m) {
    if (!m) return;
    if (m->stream) (void)hipStreamSynchronize(m->stream);
    delete m;
}

int32_t forge_hip_forward(forge_hip_model* m, uint32_t token, float* logits_host) {
    FH_CHECK(logits_host, "forward: null logits");
    int32_t rc = forward_common(m, token);
    if (rc) return rc;
    FH_HIP(hipMemcpyAsync(m->h_logits, m->logits.p, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost, m->stream));
    rc = finish_or_undo(m);
    if (rc) return rc;
    memcpy(logits_host, m->h_logits, (size_t)m->cfg.vocab * 4);
    return FORGE_HIP_OK;
}

int32_t forge_hip_forward_greedy(forge_hip_model* m, uint32_t token, uint32_t* next_token_host) {
    FH_CHECK(next_token_host, "forward_greedy: null out");
    int32_t rc = forward_common(m, token);
    if (rc) return rc;
    // the resident kernel hands the token over through host memory as soon as it is final
    if (m->pd && pd_wait_token(m->pd, next_token_host)) return FORGE_HIP_OK;
    rc = finish_or_undo(m);
    if (rc) return rc;
    *next_token_host = m->h_stage[4];
    return FORGE_HIP_OK;
}

int32_t forge_hip_prefill_batch(forge_hip_model* m, const uint32_t* tokens, uint64_t n, float* logits_host) {
    FH_CHECK(m && tokens, "prefill_batch: null pointer");
    FH_CHECK(n >= 1, "prefill_batch: empty token list");
    if ((uint64_t)m->pos + n > m->cfg.max_seq)
        return fail(FORGE_HIP_ERR_POSITION, "prompt does not fit the KV cache (pos + n > max_seq)");
    for (uint64_t i = 0; i < n; i++)
        if (tokens[i] >= m->cfg.vocab) return fail(FORGE_HIP_ERR_POSITION, "token id out of range");
    hipStream_t s = m->stream;
    if (m->mixed && m->mixed_batched) {
        uint64_t fed = 0;
        uint32_t last_rows = 0;
        while (fed < n) {
            const uint32_t rows = (uint32_t)std::min<uint64_t>(m->chunk_rows, n - fed);
            FH_HIP(hipMemcpyAsync(m->ptok.p, tokens + fed, (size_t)rows * 4, hipMemcpyHostToDevice, s));
            launch_embedding(m->embed.as<float>(), m->ptok.as<uint32_t>(), rows, m->H, m->px.as<float>(), m->counts.as<uint32_t>(), s);
            // seven projections of one plain format, fast mode, no window (whose rule differs for these models): the uniform
            // model's layer, with q;k;v and gate;up as one GEMM each and the fused epilogues
            const bool uniform_rows = m->mixed_plain_layers && m->mixed_twins && m->cfg.sliding_window == 0;
            for (uint32_t l = 0; l < m->cfg.layers; l++) {
                if (uniform_rows) enqueue_prefill_layer(m, l, rows, (uint32_t)(m->pos + fed));
                else if (m->mixed_twins) enqueue_mixed_prefill_layer_mfma(m, l, rows, (uint32_t)(m->pos + fed));
                else enqueue_mixed_prefill_layer(m, l, rows, (uint32_t)(m->pos + fed));
            }
            FH_HIP(hipGetLastError());
            fed += rows;
            last_rows = rows;
        }
        m->pos += (int64_t)n;
        m->h_stage[2] = (uint32_t)m->pos;
        FH_HIP(hipMemcpyAsync(m->d_pos(), &m->h_stage[2], 4, hipMemcpyHostToDevice, s));
        if (logits_host) {
            enqueue_head(m, m->px.as<float>() + (size_t)(last_rows - 1) * m->H, true, false);
            FH_HIP(hipGetLastError());
            FH_HIP(hipMemcpyAsync(m->h_logits, m->logits.p, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost, s));
        }
        FH_HIP(hipStreamSynchronize(s));
        if (logits_host) memcpy(logits_host, m->h_logits, (size_t)m->cfg.vocab * 4);
        return FORGE_HIP_OK;
    }
    if (m->mixed) {
        // forward_prefill of a model that is not uniformly Q8_0 or Q4_0 (emit.rs:4530-4534, 4621-5040): one token at a time
        // through forward's own operations, the lm_head once after the last token
        uint64_t fed = 0;
        while (fed < n) {
            const uint32_t rows = (uint32_t)std::min<uint64_t>(m->chunk_rows, n - fed);
            FH_HIP(hipMemcpyAsync(m->ptok.p, tokens + fed, (size_t)rows * 4, hipMemcpyHostToDevice, s));
            for (uint32_t r = 0; r < rows; r++) {
                launch_embedding(m->embed.as<float>(), m->ptok.as<uint32_t>() + r, 1, m->H, m->x.as<float>(), m->counts.as<uint32_t>(), s);
                for (uint32_t l = 0; l < m->cfg.layers; l++) enqueue_mixed_layer(m, l, (uint32_t)(m->pos + fed + r), nullptr);
            }
            FH_HIP(hipGetLastError());
            FH_HIP(hipStreamSynchronize(s));          // the token staging area is reused by the next chunk
            fed += rows;
        }
        m->pos += (int64_t)n;
        m->h_stage[2] = (uint32_t)m->pos;
        FH_HIP(hipMemcpyAsync(m->d_pos(), &m->h_stage[2], 4, hipMemcpyHostToDevice, s));
        if (logits_host) {
            enqueue_head(m, m->x.as<float>(), true, false);
            FH_HIP(hipGetLastError());
            FH_HIP(hipMemcpyAsync(m->h_logits, m->logits.p, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost, s));
        }
        FH_HIP(hipStreamSynchronize(s));
        if (logits_host) memcpy(logits_host, m->h_logits, (size_t)m->cfg.vocab * 4);
        return FORGE_HIP_OK;
    }
    uint64_t done = 0;
    uint32_t last_rows = 0;
    while (done < n) {
        const uint32_t rows = (uint32_t)std::min<uint64_t>(m->chunk_rows, n - done);
        // pageable source: the copy is complete (staged) when the call returns
        FH_HIP(hipMemcpyAsync(m->ptok.p, tokens + done, (size_t)rows * 4, hipMemcpyHostToDevice, s));
        launch_embedding(m->embed.as<float>(), m->ptok.as<uint32_t>(), rows, m->H, m->px.as<float>(), m->counts.as<uint32_t>(), s);
        for (uint32_t l = 0; l < m->cfg.layers; l++) enqueue_prefill_layer(m, l, rows, (uint32_t)(m->pos + done));
        FH_HIP(hipGetLastError());
        done += rows;
        last_rows = rows;
    }
    m->pos += (int64_t)n;
    m->h_stage[2] = (uint32_t)m->pos;
    FH_HIP(hipMemcpyAsync(m->d_pos(), &m->h_stage[2], 4, hipMemcpyHostToDevice, s));
    if (logits_host) {
        enqueue_head(m, m->px.as<float>() + (size_t)(last_rows - 1) * m->H, true, false);
        FH_HIP(hipGetLastError());
        FH_HIP(hipMemcpyAsync(m->h_logits, m->logits.p, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost, s));
    }
    FH_HIP(hipStreamSynchronize(s));
    if (logits_host) memcpy(logits_host, m->h_logits, (size_t)m->cfg.vocab * 4);
    return FORGE_HIP_OK;
}

int32_t forge_hip_forward_profile(forge_hip_model* m, uint32_t token, float* stage_ms, uint32_t* stage_launches) {
    FH_CHECK(m && stage_ms, "forward_profile: null pointer");
    if (m->pos >= (int64_t)m->cfg.max_seq) return fail(FORGE_HIP_ERR_POSITION, "KV cache is full (pos == max_seq)");
    if (token >= m->cfg.vocab) return fail(FORGE_HIP_ERR_POSITION, "token id out of range");
    if (m->pd) {
        // one kernel: the stages are its phases, timed by the kernel's own clock stamps
        int32_t rc = pd_enqueue(m->pd, true, token, m->stream);
        if (rc) return rc;
        rc = finish_decode_step(m);
        if (rc) return rc;
        m->pos += 1;
        std::vector<float> ph;
        rc = pd_phase_ms(m->pd, &ph, m->stream);
        if (rc) return rc;
        for (int i = 0; i < ST_COUNT; i++) { stage_ms[i] = 0.f; if (stage_launches) stage_launches[i] = 0; }
        // the second attention phase (merge of the splits, or the recurrence over the blocks, and the quantised row for the O
        // projection) is reported as the quantise stage
        static const int phase_stage[6] = {ST_QKV, ST_ATTN, ST_QUANT, ST_O, ST_GATE_UP, ST_DOWN};
        for (size_t i = 0; i < ph.size(); i++) {
            const size_t nl = 6 * (size_t)m->cfg.layers;
            const int st = i < nl ? phase_stage[i % 6] : (i == nl ? ST_LM_HEAD : ST_ARGMAX);
            stage_ms[st] += ph[i];
            if (stage_launches) stage_launches[st] += 1;
        }
        return FORGE_HIP_OK;
    }
    m->h_stage[0] = token;
    FH_HIP(hipMemcpyAsync(m->d_token(), &m->h_stage[0], 4, hipMemcpyHostToDevice, m->stream));
    {
        ModelProbe probe(m);
        enqueue_decode_step(m);        // eager launches, each carrying its own pair of events
    }
    FH_HIP(hipGetLastError());
    FH_HIP(hipStreamSynchronize(m->stream));
    m->pos += 1;
    return collect_profile(m, stage_ms, stage_launches);
}

int32_t forge_hip_prefill_profile(forge_hip_model* m, const uint32_t* tokens, uint64_t n, float* stage_ms,
                                  uint32_t* stage_launches) {
    FH_CHECK(m && stage_ms, "prefill_profile: null pointer");
    int32_t rc;
    {
        ModelProbe probe(m);
        rc = forge_hip_prefill_batch(m, tokens, n, nullptr);
    }
    if (rc) return rc;
    FH_HIP(hipStreamSynchronize(m->stream));
    return collect_profile(m, stage_ms, stage_launches);
}

int32_t forge_hip_model_decode_launches(const forge_hip_model* m) {
    if (!m) return -1;
    if (m->pd) return (int32_t)pd_launches_per_step(m->pd);
    const bool exact = (m->cfg.flags & FORGE_HIP_FLAG_EXACT) != 0;
    const int attn = exact ? 1 : 2;
    if (m->mixed && m->mixed_plain_layers)
        return 1 + (int)m->cfg.layers * ((m->fuse_norm ? 1 : 3) + attn + 1 + (m->fuse_silu ? 1 : 3) + 1) + 4;
    if (m->mixed) {
        // a group of projections over the same normed vector: all K-quant -> one launch that norms as well; else the norm, one
        // launch for the K-quant ones and one for each of the others
        auto kq = [&](int cat) { return m->pd_types[cat] == FORGE_HIP_Q4_K || m->pd_types[cat] == FORGE_HIP_Q6_K; };
        auto group = [&](std::initializer_list<int> cats) {
            int plain = 0, k = 0;
            for (int cat : cats) (kq(cat) ? k : plain)++;
            return (plain == 0 && m->mixed_fuse) ? 1 : 1 + plain + (k ? 1 : 0);
        };
        return 1 + (int)m->cfg.layers * (group({0, 1, 2}) + 1 + attn + 1 + group({4, 5}) + 2) + 4;
    }
    const int layer = (m->fuse_norm ? 1 : 3) + attn + 1 + (m->fuse_silu ? 1 : 3) + 1;
    const int head = ((m->fuse_norm && m->cfg.vocab <= 16384) ? 1 : 2) + 2;
    return 1 + (int)m->cfg.layers * layer + head;
}

int32_t forge_hip_reset(forge_hip_model* m) {
    FH_CHECK(m, "reset: model is null");
    m->pos = 0;
    m->h_stage[2] = 0;
    FH_HIP(hipMemcpyAsync(m->d_pos(), &m->h_stage[2], 4, hipMemcpyHostToDevice, m->stream));
    FH_HIP(hipMemsetAsync(m->counts.p, 0, (size_t)m->cfg.vocab * 4, m->stream));      // recent_tokens starts empty again
    FH_HIP(hipStreamSynchronize(m->stream));
    return FORGE_HIP_OK;
}

int32_t forge_hip_model_set_repeat_penalty(forge_hip_model* m, float penalty) {
    FH_CHECK(m, "set_repeat_penalty: model is null");
    FH_CHECK(penalty == penalty && penalty > 0.0f, "set_repeat_penalty: the penalty must be a positive number");
    if (penalty == m->repeat_penalty) return FORGE_HIP_OK;
    FH_HIP(hipStreamSynchronize(m->stream));
    if (m->pd) {
        const int32_t rc = pd_set_repeat_penalty(m->pd, penalty);
        if (rc) return rc;
    }
    m->repeat_penalty = penalty;
    // the captured kernel sequence carries the old value in its launch arguments: capture again at the next step
    if (m->decode_graph) { (void)hipGraphExecDestroy(m->decode_graph); m->decode_graph = nullptr; }
    return FORGE_HIP_OK;
}

int32_t forge_hip_model_set_poll_limit(forge_hip_model* m, uint32_t polls) {
    FH_CHECK(m, "set_poll_limit: model is null");
    FH_HIP(hipStreamSynchronize(m->stream));
    if (m->pd) pd_set_poll_limit(m->pd, polls);
    return FORGE_HIP_OK;
}

int64_t forge_hip_model_pos(const forge_hip_model* m) { return m ? m->pos : -1; }

int32_t forge_hip_model_set_kv_pages(forge_hip_model* m, uint32_t page_rows, const uint32_t* page_table_host, uint32_t n_pages) {
    FH_CHECK(m, "set_kv_pages: model is null");
    FH_CHECK(m->pos == 0, "set_kv_pages: the cache layout can only change while the cache is empty (after create or reset)");
    FH_HIP(hipStreamSynchronize(m->stream));
    PageTable pt{};
    std::vector<uint32_t> table;
    if (page_rows != 0) {
        FH_CHECK(!(m->cfg.flags & FORGE_HIP_FLAG_EXACT), "set_kv_pages: the order-faithful kernels (FORGE_HIP_FLAG_EXACT) read a flat cache only");
        FH_CHECK((page_rows & (page_rows - 1)) == 0 && page_rows >= 64, "set_kv_pages: page_rows must be a power of two, at least 64");
        FH_CHECK(m->cfg.max_seq % page_rows == 0 && n_pages == m->cfg.max_seq / page_rows,
                 "set_kv_pages: n_pages must be max_seq / page_rows (max_seq a multiple of page_rows)");
        FH_CHECK(page_table_host, "set_kv_pages: null page table");
        // every pool page at most once: two pages of the sequence must not share memory
        std::vector<uint8_t> seen(n_pages, 0);
        for (uint32_t i = 0; i < n_pages; i++) {
            FH_CHECK(page_table_host[i] < n_pages && !seen[page_table_host[i]], "set_kv_pages: the table must name every pool page below n_pages at most once");
            seen[page_table_host[i]] = 1;
        }
        table.assign(page_table_host, page_table_host + n_pages);
        if (!m->page_table.p) {
            const int32_t rc = m->page_table.alloc((size_t)m->cfg.max_seq / 64 * 4);      // room for the smallest page size
            if (rc) return rc;
        }
        FH_HIP(hipMemcpy(m->page_table.p, table.data(), (size_t)n_pages * 4, hipMemcpyHostToDevice));
        pt.table = m->page_table.as<uint32_t>();
        pt.shift = (uint32_t)__builtin_ctz(page_rows);
    }
    if (m->pd) {
        const int32_t rc = pd_set_kv_pages(m->pd, pt, m->cfg.max_seq);
        if (rc) return rc;
    }
    m->pt = pt;
    m->page_table_host.swap(table);
    // the captured kernel sequence carries the old layout in its launch arguments: capture again at the next step
    if (m->decode_graph) { (void)hipGraphExecDestroy(m->decode_graph); m->decode_graph = nullptr; }
    return FORGE_HIP_OK;
}

int32_t forge_hip_model_read_kv(forge_hip_model* m, uint32_t layer, uint32_t which, uint16_t* out_host) {
    FH_CHECK(m && out_host, "read_kv: null pointer");
    FH_CHECK(layer < m->cfg.layers && which <= 1, "read_kv: layer or selector out of range");
    FH_HIP(hipStreamSynchronize(m->stream));
    const uint16_t* src = which == 0 ? m->kc(layer) : m->vc(layer);
    if (m->pos > 0 && !m->pt.table) FH_HIP(hipMemcpy(out_host, src, (size_t)m->pos * m->KV * 2, hipMemcpyDeviceToHost));
    if (m->pos > 0 && m->pt.table) {
        // paged cache: the sequence's rows page by page, in sequence order
        const uint64_t page_rows = 1ull << m->pt.shift;
        for (uint64_t t0 = 0; t0 < (uint64_t)m->pos; t0 += page_rows) {
            const uint64_t rows = std::min<uint64_t>(page_rows, (uint64_t)m->pos - t0);
            const uint64_t pool_row = (uint64_t)m->page_table_host[t0 >> m->pt.shift] << m->pt.shift;
            FH_HIP(hipMemcpy(out_host + t0 * m->KV, src + pool_row * m->KV, rows * m->KV * 2, hipMemcpyDeviceToHost));
        }
    }
    return FORGE_HIP_OK;
}

}  // extern "C"

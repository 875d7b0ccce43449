// Shared declarations for libforge_hip: error plumbing, the device-side weight layout and
// the launch functions each translation unit exports to the others.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "forge_hip.h"

namespace fh {

// ---- error plumbing -------------------------------------------------------------------
void set_error(const std::string& msg);
int32_t fail(int32_t code, const std::string& msg);

#define FH_HIP(expr)                                                                                   \
    do {                                                                                               \
        hipError_t _e = (expr);                                                                        \
        if (_e != hipSuccess)                                                                          \
            return ::fh::fail(FORGE_HIP_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(_e)); \
    } while (0)

#define FH_CHECK(cond, msg)                                           \
    do {                                                              \
        if (!(cond)) return ::fh::fail(FORGE_HIP_ERR_INVALID, (msg)); \
    } while (0)

// ---- kernel launch -------------------------------------------------------------------------
// Every kernel of the library is launched through fh::launch.  While a LaunchProbe is installed on
// the calling thread (forward_profile / prefill_profile), each launch asks it for a pair of events
// and attaches them to the dispatch itself, so that their elapsed time is the kernel's own begin-to-end
// device time (the dispatch timestamps a kernel trace reports), free of the cost of recording events
// around it on the stream.
struct LaunchProbe {
    virtual bool next(hipEvent_t* start, hipEvent_t* stop) = 0;
    virtual ~LaunchProbe() = default;
};
LaunchProbe*& launch_probe();      // thread-local slot, null when not profiling

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t s, Args... args) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    LaunchProbe* p = launch_probe();
    if (p && p->next(&e0, &e1))
        hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds_bytes, s, e0, e1, 0, static_cast<KArgs>(args)...);
    else
        hipLaunchKernelGGL(kernel, grid, block, (uint32_t)lds_bytes, s, static_cast<KArgs>(args)...);
}

// ---- device weight layout ----------------------------------------------------------------
// GGUF interleaves a 2-byte scale with every 32 quants (34- or 18-byte blocks, 2-byte
// aligned).  On upload each matrix is split into two planes so that every lane can issue
// aligned 16-byte loads:
//   qs     Q8_0: int8  [N][K]      (row n = its K quants in order)
//          Q4_0: uint8 [N][K/2]    (row n = its K/32 blocks of 16 packed bytes, byte j of a
//                                   block = element j in the low nibble, j+16 in the high)
//   scales fp16 bits [N][K/32]
// The planes hold exactly the bytes of the GGUF blocks, regrouped; nothing is dequantised.
struct QWeight {
    uint32_t wdtype = 0, K = 0, N = 0;
    uint8_t* qs = nullptr;
    uint16_t* scales = nullptr;
    bool owns = false;
    bool kquant() const { return wdtype == FORGE_HIP_Q4_K || wdtype == FORGE_HIP_Q6_K; }
    // K-quants (gemv_kquant.hip): qs = nibble bytes (Q4_K, K/2 per row) or low nibbles + high bit pairs (Q6_K, 192 per
    // super-block); `scales` then points at the second plane (16 / 32 bytes per super-block)
    size_t qs_row_bytes() const { return wdtype == FORGE_HIP_Q6_K ? (size_t)K / 256 * 192 : wdtype == FORGE_HIP_Q8_0 ? K : K / 2; }
    size_t qs_bytes() const { return (size_t)N * qs_row_bytes(); }
    size_t scales_bytes() const { return kquant() ? (size_t)N * (K / 256) * (wdtype == FORGE_HIP_Q4_K ? 16 : 32) : (size_t)N * (K / 32) * 2; }
};

// Split raw GGUF rows into the two planes (host side).
void repack_host(uint32_t wdtype, const uint8_t* raw, uint32_t K, uint64_t N, uint8_t* qs, uint16_t* scales);

// ---- host format helpers (format.hip) ------------------------------------------------------
float f16_to_f32_host(uint16_t bits);
uint16_t f32_to_f16_host(float x);
void quantize_host(uint32_t wdtype, const float* d, uint64_t n, uint8_t* out);
void dequant_host(uint32_t wdtype, const uint8_t* data, uint64_t n, float* out);
const char* last_error_cstr();
// Upload raw GGUF rows as planes into freshly allocated device memory.
int32_t qweight_upload(uint32_t wdtype, const uint8_t* raw_host, uint32_t K, uint32_t N, QWeight* out);
void qweight_free(QWeight* w);

// ---- paged KV cache --------------------------------------------------------------------------
// A cache may be a pool of pages of 2^shift rows: row t of the sequence is then row t % page of pool page
// table[t / page] (table: uint32 in device memory).  table == nullptr: the flat cache, row t is row t.
struct PageTable {
    const uint32_t* table = nullptr;
    uint32_t shift = 0;          // log2(rows per page)
};
__device__ __forceinline__ size_t paged_row(const PageTable& pt, uint32_t t) {
    if (!pt.table) return t;
    return ((size_t)pt.table[t >> pt.shift] << pt.shift) + (t & ((1u << pt.shift) - 1u));
}

// ---- kernel launchers ------------------------------------------------------------------------
// All are asynchronous on `s` and validate nothing: callers check shapes first.

// elementwise.hip
// neg_odd (here and below): the codes of a row's odd blocks are stored negated and an all-zero block gets the scale 0
// (the reference's quantiser gives it 1.0), as the fast prefill GEMM takes them.
void launch_quantize_act(const float* x, uint32_t M, uint32_t K, int8_t* q, uint16_t* sc, hipStream_t s, bool neg_odd = false);
// rms_norm of M rows; writes f32 `normed` if non-null and the quantised row (q, sc) if q non-null.
void launch_rmsnorm(const float* x, const float* w, float eps, uint32_t M, uint32_t H, float* normed, int8_t* q,
                    uint16_t* sc, hipStream_t s, bool neg_odd = false);
// out = silu(gate)*up over M rows where gate = gu[r][0..I), up = gu[r][I..2I) when fused, else two
// pointers; writes f32 out if non-null and quantised (q, sc) if q non-null.
void launch_silu_mul(const float* gate, const float* up, uint32_t M, uint32_t I, uint32_t row_stride, float* out,
                     int8_t* q, uint16_t* sc, hipStream_t s, bool neg_odd = false);
// Interleaved-pair RoPE on q,k and fp16 cache write of k,v.  Position of row r is
// (pos_dev ? *pos_dev : base_pos) + r.  q/k/v rows have strides q_stride/kv_stride floats.
void launch_rope_kv_store(float* q, float* k, const float* v, uint32_t q_stride, uint32_t kv_stride, uint16_t* kc,
                          uint16_t* vc, uint32_t M, uint32_t base_pos, const uint32_t* pos_dev, uint32_t heads,
                          uint32_t kv_heads, uint32_t hd, const float* cos_t, const float* sin_t, const float* bias, hipStream_t s,
                          PageTable pt = PageTable{});
void launch_embedding(const float* table, const uint32_t* tokens_dev, uint32_t M, uint32_t H, float* out, uint32_t* counts,
                      hipStream_t s);
// Index of the LAST maximum.  `scratch` needs 2*ARGMAX_BLOCKS uint32/float pairs.
constexpr uint32_t ARGMAX_BLOCKS = 256;
// If pos_dev is given, the final stage also advances the decode state: *pos_dev += 1, *token_dev = *out.
void launch_argmax(const float* x, uint32_t n, uint32_t* out, void* scratch, uint32_t* pos_dev, uint32_t* token_dev,
                   const uint32_t* counts, float penalty, hipStream_t s);

// gemv.hip — y[n] (=|+=) sum_b f32(isum_b) * (a_s[b]*w_s[n][b]); activations already quantised.
// `order` selects which rows take the reference's 4-accumulator (dot1) order instead of the sequential one.
enum class GemvOrder { MatmulVec, LmHead, LmHeadAfterPrefill };
void launch_gemv(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, GemvOrder order,
                 hipStream_t s);
void launch_gemv_isums(const QWeight& w, const int8_t* aq, int32_t* out, hipStream_t s);
bool gemv_k_supported(uint32_t K);
// Fused decode variants (one launch instead of three): rms_norm + activation quantiser in the prologue.
bool gemv_norm_fusable(uint32_t K);
bool gemv_silu_fusable(uint32_t K);
// y = W * quant(rms_norm(x))
void launch_gemv_norm(const QWeight& w, const float* x, const float* norm_w, float eps, float* y, GemvOrder order,
                      hipStream_t s);
// fused [q;k;v] matrix: q rows -> q_out (rotated), k rows -> K cache (rotated, fp16), v rows -> V cache, at *pos_dev
void launch_gemv_norm_rope_kv(const QWeight& wqkv, const float* x, const float* norm_w, float eps, const float* bias, float* q_out,
                              uint16_t* kc, uint16_t* vc, const float* cos_t, const float* sin_t,
                              const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd, hipStream_t s,
                              PageTable pt = PageTable{});
// fused [gate;up] matrix: quant(silu(gate)*up) -> (oq, osc)
void launch_gemv_norm_silu_quant(const QWeight& wgu, const float* x, const float* norm_w, float eps, int8_t* oq,
                                 uint16_t* osc, hipStream_t s);

// gemv_f32.hip — the reference's portable row dot (f32 activations x weights dequantised on the fly, one sequential sum
// per row): y[n] = sum_k x[k] * (f32(q[n][k]) * w_s[n][k/32]).
void launch_gemv_f32(const QWeight& w, const float* x, float* y, hipStream_t s);

// gemv_kquant.hip — matmul_vec_q4_k / matmul_vec_q6_k: Q8_0-quantised activations against 256-element super-blocks.
void repack_kquant_host(uint32_t wdtype, const uint8_t* raw, uint32_t K, uint64_t N, uint8_t* qs, uint8_t* meta);
bool kquant_k_supported(uint32_t K);
void launch_gemv_kquant(const QWeight& w, const int8_t* aq, const uint16_t* as, float* y, bool accumulate, hipStream_t s);
// Up to three Q4_K / Q6_K matrices of the same K over one quantised vector in a single launch (q, k, v; gate, up).
void launch_gemv_kquant_multi(const QWeight* const* w, float* const* y, uint32_t n, const int8_t* aq, const uint16_t* as, bool accumulate,
                              hipStream_t s);
// ... over quantise(rms_norm(x) * norm_w), normed and quantised inside the kernel (the norm kernel's bits).
void launch_gemv_kquant_multi_norm(const QWeight* const* w, float* const* y, uint32_t n, const float* x, const float* norm_w, float eps,
                                   hipStream_t s);
// kquant_prefill.hip -- K-quant matrices on the int8 MFMA GEMM (fast mode).  The twin of a matrix is the same weights in
// the Q8_0 layout: Q4_K as codes (q - 8) * g of depth K plus one f32 coefficient per (row, block) for the minimum term,
// Q6_K as the hi and lo parts of sc * q, two blocks per block (depth 2K), under the exact scales 64 d and d.
struct KqTwin {
    QWeight w;                 // Q8_0 layout, [N][K] (Q4_K) or [N][2K] (Q6_K)
    float* coef = nullptr;     // Q4_K: [N][K/32] slots, (8 * d * sc - dmin * min) * 2^8 as a hi | lo pair of fp16 numbers
    bool present() const { return w.qs != nullptr; }
};
int32_t kquant_twin_create(const QWeight* const* ws, uint32_t n, KqTwin* out, bool* covered, hipStream_t s);
void kquant_twin_free(KqTwin* t);
// out[m][b] = a_s[m][b] * (sum of block b's codes), f32 [M][K/32]
void launch_act_block_sums(const int8_t* aq, const uint16_t* as, uint32_t M, uint32_t K, bool neg_odd, float* out, hipStream_t s);
// every pair of blocks twice: codes [M][2K], scales [M][2K/32]; blocks 2p, 2p + 1 -> 2p, 2p + 1, 2p, 2p + 1
void launch_act_twice(const int8_t* aq, const uint16_t* as, uint32_t M, uint32_t K, int8_t* oq, uint16_t* os, hipStream_t s);
// The same for M rows of quantised activations (codes [M][K], scales [M][K/32]); rows of y are ldy floats apart.  Every row has the
// bits launch_gemv_kquant gives it alone.
void launch_gemv_kquant_rows(const QWeight& w, const int8_t* aq, const uint16_t* as, uint32_t M, float* y, uint32_t ldy, bool accumulate,
                             hipStream_t s);

// gemm.hip — y[m][n] (=|+=) ...; aq int8 [M][K], as fp16 [M][K/32].  isums (optional) int32 [M][N][K/32].
// exact: unfused multiply/add per block (bit-identical to the CPU path); otherwise one FMA per block, and then the
// activation codes of every row's odd blocks must come negated (the neg_odd flag of the quantising launchers).
// split_ws (optional, gemm_split_workspace_bytes() bytes, its last KB zero before the first use and left zero by every
// launch): lets the fast mode cut the tiles that do not fill a whole round of CUs along K; launches that share a
// workspace must be ordered (one stream).  With it a row's low bits may depend on where in the batch the row sits.
size_t gemm_split_workspace_bytes();
// silu_q / silu_sc (fast mode, no isums, gemm_silu_supported(w, w.N / 2, M)): w is a fused [gate; up] matrix; instead of y
// the launch writes quantize(silu(gate) * up) for the down projection: codes [M][N / 2] with odd blocks negated and fp16
// scales [M][N / 64] (silu_mul emit.rs:380-386 with the hardware exponential, quantiser emit.rs:1410-1440).
bool gemm_silu_supported(const QWeight& w, uint32_t inter, uint32_t M);
// mt_a / mt_w (fast mode, Q8_0-layout matrices, no isums): [M][K/32] and [N][K/32] slots of 4 bytes, each a hi | lo pair of
// fp16 numbers (launch_act_block_sums, kquant_twin_create write them); every element of the result additionally receives
// sum_b mt_a[m][b] * mt_w[n][b] (before the SiLU epilogue, if any).
void launch_gemm(const QWeight& w, const int8_t* aq, const uint16_t* as, uint32_t M, float* y, uint32_t ldy,
                 bool accumulate, bool exact, int32_t* isums, hipStream_t s, void* split_ws = nullptr, int8_t* silu_q = nullptr,
                 uint16_t* silu_sc = nullptr, const float* mt_a = nullptr, const float* mt_w = nullptr);

// model.hip — the part of forge_hip_model_create's checks that sizes depend on (formats, dimensions the kernels cover);
// sets the error message.
int32_t validate_config_shape(const forge_hip_config* c);

// attn_decode.hip
constexpr uint32_t DECODE_SPLITS = 32;
size_t attn_decode_workspace_bytes(uint32_t heads, uint32_t hd);
// seq_len = pos_dev ? *pos_dev + 1 : seq_len.  Writes f32 out if non-null and quantised (q, sc) if q non-null.
// window != 0: only the last `window` rows are keys (attention_sliding, emit.rs:598-627).
void launch_attn_decode(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int8_t* oq, uint16_t* osc,
                        uint32_t seq_len, const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd,
                        uint32_t window, void* workspace, hipStream_t s, PageTable pt = PageTable{});
// The same over a paged cache: k_pool / v_pool fp16 [pages][page_rows][kv_heads*hd], row t of the sequence is row
// t % page_rows of pool page page_table[t / page_rows].  f32 output, no window.
bool attn_decode_paged_supported(uint32_t seq_len, uint32_t page_rows);
void launch_attn_decode_paged(const float* q, const uint16_t* k_pool, const uint16_t* v_pool, const uint32_t* page_table,
                              uint32_t page_rows, float* out, uint32_t seq_len, uint32_t heads, uint32_t kv_heads, uint32_t hd,
                              void* workspace, hipStream_t s);

// Looks up, once per device, the address of the fixed scratch array of forge_hip_attn_decode_f16kv_noalloc on the current
// device; called from the library's set-up entry points.
void attn_decode_noalloc_prepare();

// attn_prefill.hip
// q rows / out rows have strides q_stride / out_stride floats (q may live inside a fused qkv buffer).
// window != 0: the query at position p sees keys [max(0, p - window + 1), p] (attention_sliding_batch, emit.rs:907-1046).
// pt: a paged cache needs pages of a multiple of 64 rows (a key tile then lies within one page).
void launch_attn_prefill(const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc, float* out,
                         uint32_t out_stride, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                         uint32_t hd, uint32_t window, hipStream_t s, PageTable pt = PageTable{});

// The same attention, written as the activation quantiser's output of its rows: int8 codes oq[M][heads*hd] and fp16 scales
// osc[M][heads*hd/32] (bit-identical to launch_attn_prefill followed by launch_quantize_act).
void launch_attn_prefill_quant(const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc, int8_t* oq, uint16_t* osc,
                               uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads, uint32_t hd, uint32_t window,
                               hipStream_t s, bool neg_odd = false, PageTable pt = PageTable{});

bool attn_head_dim_supported(uint32_t hd);

// attn_exact.hip — order-faithful attention (one workgroup per row and head).  batch_order selects
// attention_flash_batch's accumulation order, otherwise attention_flash's.  Row r sits at position
// (pos_dev ? *pos_dev : base_pos) + r and sees keys [0, that position].  window != 0: attention_sliding_batch's order
// (batch_order) or attention_sliding's plain softmax over the last `window` rows, whose scores take min(window, max_rows)
// floats of LDS (max_rows = the rows the cache can hold; window <= attn_exact_max_window() or max_rows <= it).
void launch_attn_exact(bool batch_order, const float* q, uint32_t q_stride, const uint16_t* kc, const uint16_t* vc,
                       float* out, uint32_t out_stride, int8_t* oq, uint16_t* osc, uint32_t M, uint32_t base_pos,
                       const uint32_t* pos_dev, uint32_t heads, uint32_t kv_heads, uint32_t hd, uint32_t window, uint32_t max_rows,
                       void* ws, hipStream_t s);
// One decode row without a window runs spread over (key block, head) workgroups when `ws` holds
// attn_exact_decode_workspace_bytes(heads, hd, max_rows) bytes (0: caches that long keep the one-workgroup kernel): same bits.
size_t attn_exact_decode_workspace_bytes(uint32_t heads, uint32_t hd, uint32_t max_rows);
uint32_t attn_exact_max_window();

// decode_persistent.hip — the whole decode step as one resident kernel (fast mode only)
struct PdLayerIn {
    const QWeight* qkv;        // uniform models: the fused matrices
    const QWeight* o;
    const QWeight* gate_up;
    const QWeight* down;

    const float* attn_norm;
    const float* ffn_norm;
    uint16_t* kc;
    uint16_t* vc;
    // K-quant models (every matrix Q4_K or Q6_K; qkv and gate_up are then null): the projections one by one, re-laid out for
    // the kernel by pd_create.  q and k must share a format, gate and up too; v may have its own.
    const QWeight *q = nullptr, *k = nullptr, *v = nullptr, *gate = nullptr, *up = nullptr;
};
struct PdState;
// Leaves *out null (returning OK) when the shape or device is not covered; `state` = {position, token, next token, abort flag}.
uint32_t pd_launches_per_step(const PdState* st);
int32_t pd_create(const forge_hip_config& c, const std::vector<PdLayerIn>& layers, const QWeight& lm_head, const float* embed,
                  const float* final_norm, const float* cos_t, const float* sin_t, float* logits, uint32_t* state, uint32_t* counts,
                  const float* qkv_bias, PdState** out);
int32_t pd_set_repeat_penalty(PdState* st, float penalty);
void pd_set_poll_limit(PdState* st, uint32_t n);
int32_t pd_set_kv_pages(PdState* st, PageTable pt, uint32_t max_seq);
void pd_destroy(PdState* st);
int32_t pd_enqueue(PdState* st, bool profile, uint32_t token, hipStream_t s);
// Spins on the host word the kernel writes last; false = not available, wait for the stream instead.
bool pd_wait_token(PdState* st, uint32_t* next);
// Call with the abort flag read back after the stream drained; resets the exchange buffers and fails if it is set.
int32_t pd_after_sync(PdState* st, uint32_t abort_flag, hipStream_t s);
// Milliseconds between the phase starts of the last profiled step: six per layer, then head and argmax.
int32_t pd_phase_ms(PdState* st, std::vector<float>* out, hipStream_t s);

}  // namespace fh

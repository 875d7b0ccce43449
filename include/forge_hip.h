/* libforge_hip — C ABI of the MI355X (gfx950) backend for ForgeLLM's quantized-Llama hot path.
 *
 * This is what a `forgellm-codegen-hip` crate's generated `model.rs` binds (extern "C"),
 * in place of the Rust kernels that crates/forgellm-codegen-cpu/src/emit.rs ("emit.rs")
 * generates and of the MSL kernels of crates/forgellm-codegen-metal/src/lib.rs ("metal").
 * Every entry point names the reference interface it replaces.
 *
 * Conventions
 *  - Every function returns a status: 0 = OK, negative = error class below.  The reference
 *    panics on these conditions (metal:4212, project.rs:342-406); here they are codes plus a
 *    thread-local message from forge_hip_last_error().
 *  - "dev" pointers are device (HBM) addresses; "host" pointers are ordinary memory.
 *  - `stream` is a hipStream_t passed as void*; NULL = the null stream.  Op-level calls are
 *    asynchronous on that stream.  Model calls run on the model's own stream and return
 *    after the results they hand back are complete.
 *  - A model handle is NOT thread-safe (the reference API is `&mut self`, metal:5070).
 *  - Arithmetic: activations are quantised per 32-element block to int8 exactly as
 *    emit.rs:1410-1440, block dot products are exact int32 (emit.rs:1543-1553,
 *    2522-2552), the per-block combine and everything else is f32.  KV cache is fp16.
 *
 * Supported envelope (anything outside it is refused with FORGE_HIP_ERR_INVALID and a message, never
 * computed wrongly):
 *  - model API: projection and lm_head weights Q8_0 or Q4_0 (forge_hip_model_create_mixed: also Q4_K and Q6_K, a
 *    format per projection); hidden a multiple of 32 in [32, 16352];
 *    inter and heads*head_dim multiples of 32, at most 16384; head_dim 64, 96 or 128; heads a multiple
 *    of kv_heads, at most 256; FORGE_HIP_FLAG_EXACT needs max_seq > 512 (below that the reference runs
 *    its non-flash attention, which has no order-faithful kernel here) and, with a sliding window,
 *    min(sliding_window, max_seq) <= 12288.  forge_hip_prefill_batch takes any n up to the free cache;
 *    it works through the prompt in chunks of at most 4096 rows, so its scratch does not grow with n.
 *  - op-level API: K a multiple of 32, at most 16384 (K-quants: a multiple of 256); M and S bounded
 *    only by memory; head_dim as above.
 *
 * Device memory and threads
 *  - A model allocates all its device buffers in forge_hip_model_create (weights, KV cache for max_seq,
 *    activations for one prefill chunk); later calls allocate no device memory (the kernel-sequence
 *    decode path instantiates its HIP graph at the first decode step).
 *  - The op-level calls keep a few scratch areas per device (quantised activations, attention / argmax
 *    partial results, RoPE tables, 16 MB of partial GEMM tiles, K-quant operands) that GROW ON DEMAND: a call that needs more
 *    than any earlier call on that device did frees the old area, which waits for the device, and allocates one at least half
 *    as large again (hipFree + hipMalloc on the call path, a few times over a run of growing shapes).  They are shared by
 *    all streams of a device and not locked: use the op-level API from one thread and one stream per device at a time, and call
 *    the largest shape once at start-up if the allocation must not happen later.  forge_hip_attn_decode_f16kv_noalloc is the one op-level
 *    call that never allocates.
 *  - The one-kernel decode step (forge_hip_model_decode_launches() == 1) runs one workgroup per compute
 *    unit and its workgroups wait on each other's results, so all of them must be resident at once:
 *    the library assumes that the process has the GPU to itself.  If another process or another
 *    stream of this process holds compute units for long enough, the kernel's bounded wait expires,
 *    the call returns FORGE_HIP_ERR_HIP with the model's position and repeat counts unchanged, and the
 *    caller may repeat it or set FORGE_HIP_PERSIST=0 before model_create to use the kernel sequence,
 *    which has no such requirement.
 */
#ifndef FORGE_HIP_H
#define FORGE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FORGE_HIP_OK 0
#define FORGE_HIP_ERR_INVALID (-1)   /* bad argument / unsupported shape */
#define FORGE_HIP_ERR_BLOB_SIZE (-2) /* weights blob length does not match the config */
#define FORGE_HIP_ERR_POSITION (-3)  /* cache full, or token id out of range */
#define FORGE_HIP_ERR_NO_DEVICE (-4)
#define FORGE_HIP_ERR_HIP (-5)       /* a HIP runtime call failed */

/* Bit for config.flags and for the `flags` argument of the op-level calls.
 * EXACT: every f32 operation follows the CPU path's own order (sequential block combine without
 * fused multiply-add, 64-key attention blocks with sequential sums, the C library's expf), so
 * results are bit-identical to the CPU path and greedy tokens are identical.  Without it the
 * prefill GEMM fuses its per-block multiply-add and attention runs on the MFMA / split-sequence
 * kernels: same integer block sums, f32 results within rel 1e-3 / abs 1e-3, much faster.  Only EXACT
 * results are independent of how rows are batched: without the flag the GEMM may add a row's blocks in
 * K ranges chosen from the batch size, so the same row can differ in its last bits between two batch
 * sizes (a repeated call with the same sizes reproduces its bits). */
#define FORGE_HIP_FLAG_EXACT 1u
/* Bit for config.flags only.  QKV_BIAS: the q, k and v projections add a bias vector before RoPE (Qwen2,
 * emit.rs:3906-3915, 4105-4120) and the weights blob carries, per layer after the v weights, q_bias [heads*head_dim],
 * k_bias and v_bias [kv_heads*head_dim] as f32 (project.rs:286-292). */
#define FORGE_HIP_FLAG_QKV_BIAS 2u

#define FORGE_HIP_Q4_0 2u /* GGML type ids, crates/forgellm-frontend/src/gguf.rs:207-258 */
#define FORGE_HIP_Q8_0 8u
#define FORGE_HIP_Q4_K 12u /* op level only: forge_hip_qweight_create + forge_hip_gemv_q */
#define FORGE_HIP_Q6_K 14u

/* Mirrors the fields of ModelConfig (crates/forgellm-frontend/src/ir.rs:484-519) that the
 * code generators read. */
typedef struct forge_hip_config {
    uint32_t hidden, inter, layers, heads, kv_heads, head_dim, vocab, max_seq;
    float rms_eps, rope_theta;
    uint32_t wdtype;        /* projection weights: FORGE_HIP_Q8_0 or FORGE_HIP_Q4_0 */
    uint32_t lm_head_dtype; /* same coding */
    uint32_t flags;         /* FORGE_HIP_FLAG_EXACT, FORGE_HIP_FLAG_QKV_BIAS, both or neither */
    uint32_t sliding_window; /* ModelConfig::sliding_window_size (ir.rs:512), 0 = None: a position attends to itself and the
                              * sliding_window - 1 positions before it (attention_sliding, emit.rs:598-627; attention_sliding_batch,
                              * emit.rs:907-1046; Mistral).  With FORGE_HIP_FLAG_EXACT min(sliding_window, max_seq) must be <= 12288. */
} forge_hip_config;

typedef struct forge_hip_model forge_hip_model;
typedef struct forge_hip_qweight forge_hip_qweight;

const char* forge_hip_last_error(void);
/* Number of visible GPUs; 0 when there is none. */
int32_t forge_hip_device_count(void);

/* ---------------- model API (replaces MetalModel, metal:4209-5981, and
 * model::{forward, forward_prefill_batched, KVCache}, emit.rs:3954-5486) ---------------- */

/* Exact byte length of the headerless weights.bin for this config (writer:
 * crates/forgellm-cli/src/main.rs:2714-2757; reader: project.rs:342-407). */
uint64_t forge_hip_weights_nbytes(const forge_hip_config* cfg);

/* MetalModel::new(weights: &[u8]) (metal:4209).  Copies/repacks the blob into HBM; the caller
 * keeps ownership of `weights_bin` and may free it on return. */
int32_t forge_hip_model_create(const forge_hip_config* cfg, const uint8_t* weights_bin_host, uint64_t nbytes,
                               forge_hip_model** out);

/* A model whose projections do not share one storage format (ProjectionDTypes, crates/forgellm-frontend/src/ir.rs:410-421;
 * chosen per GGUF tensor category by detect_gguf_proj_dtypes, crates/forgellm-cli/src/main.rs:608-680; each projection then
 * calls the kernel of its own format, matmul_call, emit.rs:3316-3334).  proj_dtypes = the GGML type ids of
 * {q, k, v, o, gate, up, down}, each Q8_0 (8), Q4_0 (2), Q4_K (12) or Q6_K (14); the lm_head's format is
 * cfg->lm_head_dtype and may be a K-quant too; cfg->wdtype is not read unless all seven agree with it.  The blob has
 * forge_hip_model_create's layout with every matrix in its own format, K-quant matrices as the GGUF file's own
 * super-blocks (144 bytes per 256 weights for Q4_K, 210 for Q6_K).  In the reference such a model has no batched
 * prefill (model_is_q8/q4 gate, emit.rs:4530-4534): the prompt goes one token at a time through the decode operations
 * (forward_prefill, emit.rs:4621-5040) and the lm_head runs once, in forward's order.  forge_hip_prefill_batch takes the
 * prompt in batches of rows where that changes no bit the mode promises: with FORGE_HIP_FLAG_EXACT when all seven
 * projections are K-quants (multi-row K-quant GEMV: every row has the one-row kernel's bits, so logits, cache and tokens are
 * the token-by-token walk's), otherwise token by token; without the flag always, on the int8 MFMA GEMM (K-quant matrices
 * through re-expressions built at create time, see forge_hip_gemm_q: the device then holds both forms of those matrices).
 * Decode: a model whose seven projections and lm_head are all Q4_K / Q6_K (q and k of one format, gate and up too) runs the
 * step as one resident kernel over a third form of the matrices built at create time (K-quant weight units: 5 bits per weight
 * for Q4_K, 9 for Q6_K; FORGE_HIP_PD_KQUANT=0 in the environment keeps the kernel sequence) -- with FORGE_HIP_FLAG_EXACT in the
 * kernel's order-faithful variant, bit for bit the sequence (FORGE_HIP_PD_EXACT=0 keeps the sequence; a sliding window always
 * does) -- and so does, without the flag, a model of seven Q8_0 or seven Q4_0 projections under a Q6_K lm_head (the uniform
 * model's kernel with the lm_head as weight units); any other mix runs the kernel sequence (K-quant projections over the same normed row share a launch), captured
 * in a graph.  K-quant matrices need an input width that is a multiple of 256.
 * FORGE_HIP_FLAG_QKV_BIAS works as in forge_hip_model_create (the bias vectors follow the v weights of every layer,
 * project.rs:286-292).  A sliding window follows the reference's rule for such models: the rows of a prompt see ALL earlier
 * positions (its token-by-token prompt calls `attention`, never attention_sliding, emit.rs:4717-4720 with
 * use_flash_attention false, emit.rs:126-128) and only decode steps apply the window (emit.rs:4156-4170); with
 * FORGE_HIP_FLAG_EXACT such a model needs max_seq <= 12288.  When all seven formats equal cfg->wdtype and the lm_head is Q8_0 or Q4_0 this is forge_hip_model_create. */
uint64_t forge_hip_weights_nbytes_mixed(const forge_hip_config* cfg, const uint32_t* proj_dtypes);
int32_t forge_hip_model_create_mixed(const forge_hip_config* cfg, const uint32_t* proj_dtypes, const uint8_t* weights_bin_host,
                                     uint64_t nbytes, forge_hip_model** out);
void forge_hip_model_destroy(forge_hip_model* m);

/* MetalModel::forward(token_id) -> Vec<f32> (metal:5070) / model::forward (emit.rs:4029):
 * one decode step at the current position; writes vocab logits to host memory; advances pos. */
int32_t forge_hip_forward(forge_hip_model* m, uint32_t token, float* logits_host);

/* forward() followed by argmax (project.rs:501-503: LAST index among equal maxima), with the
 * argmax done on the device so that only 4 bytes cross PCIe. */
int32_t forge_hip_forward_greedy(forge_hip_model* m, uint32_t token, uint32_t* next_token_host);

/* MetalModel::forward_prefill_batch(tokens) (metal:5568) / model::forward_prefill_batched
 * (emit.rs:5118): fills the KV cache for n tokens from the current position.  If
 * `logits_host` is non-NULL it receives the logits of the LAST token (the CPU signature);
 * NULL skips the lm_head (the Metal signature). */
int32_t forge_hip_prefill_batch(forge_hip_model* m, const uint32_t* tokens_host, uint64_t n, float* logits_host);

/* MetalModel::forward_profile (metal:5307-5330: one decode step with a wait per stage, timings
 * printed).  Here: one decode step launched eagerly with a pair of events attached to every kernel
 * dispatch (begin and end of the kernel itself, the times a kernel trace reports);
 * stage_ms_host[FORGE_HIP_NUM_STAGES] receives the summed kernel time per stage in milliseconds,
 * stage_launches_host (may be NULL) the number of kernel launches.  The position advances
 * like forward(); no logits are returned.  prefill_profile does the same for a batched prefill.
 * When the decode step is one resident kernel (forge_hip_model_decode_launches() == 1) its phases are the
 * stages: the kernel stamps the device wall clock at the start of each phase and the differences are
 * reported ("attention" = split + merge phases; "launches" then counts phases). */
#define FORGE_HIP_NUM_STAGES 12
#define FORGE_HIP_STAGE_NAMES                                                                                  \
    "embedding", "rms_norm", "qkv_matmul", "rope_kv_store", "attention", "quantize_act", "o_matmul", "gate_up_matmul", \
        "silu_mul", "down_matmul", "lm_head_matmul", "argmax"
int32_t forge_hip_forward_profile(forge_hip_model* m, uint32_t token, float* stage_ms_host,
                                  uint32_t* stage_launches_host);
int32_t forge_hip_prefill_profile(forge_hip_model* m, const uint32_t* tokens_host, uint64_t n, float* stage_ms_host,
                                  uint32_t* stage_launches_host);

/* Kernel launches one decode step costs on this model: 1 when the whole step runs as one resident kernel
 * (fast mode, covered shapes; one launch per 34 layers for a deeper model), otherwise the length of the kernel sequence.  The Metal backend's counterpart
 * is the fixed encoder sequence of MetalModel::forward (metal:5070-5300). */
int32_t forge_hip_model_decode_launches(const forge_hip_model* m);

/* MetalModel::reset() (metal:5981): position back to 0. */
int32_t forge_hip_reset(forge_hip_model* m);
/* Current position (KVCache.len, emit.rs:3960). */
int64_t forge_hip_model_pos(const forge_hip_model* m);
/* How often a workgroup of the resident decode kernel polls for another workgroup's data before the step gives up
 * (0: the default, 400000 polls, far beyond any wait of a healthy step).  A step that gives up returns
 * FORGE_HIP_ERR_HIP from forge_hip_forward / forge_hip_forward_greedy and has not happened: the position, the token
 * counts of the repeat penalty and the context in the cache are what they were before the call, and the same token can
 * be fed again.  No counterpart in the reference (its CPU loop has nothing to wait for); a no-op for a model that runs
 * the kernel sequence. */
int32_t forge_hip_model_set_poll_limit(forge_hip_model* m, uint32_t polls);
/* A PAGED KV cache for the model: the cache memory of every layer is taken as a pool of n_pages = max_seq / page_rows pages
 * of page_rows rows, and position t of the sequence lives in row t % page_rows of pool page page_table[t / page_rows].  For
 * hosts that hand a sequence its cache pages from a shared allocator; it has no counterpart in the reference, whose
 * model object owns one flat array per layer (emit.rs:3954-4019, metal:3525-3553).  Every kernel of the fast mode follows
 * the table (prefill: RoPE + cache write, MFMA attention; decode: the resident kernel and the kernel sequence), and the
 * results are, bit for bit, those of the flat cache.  page_rows: a power of two, at least 64 (a 64-key attention tile
 * then lies within one page), dividing max_seq; page_table_host: n_pages pool page numbers, each below n_pages, none
 * twice.  page_rows = 0 switches back to the flat cache.  Only while the cache is empty (after create or reset); not with
 * FORGE_HIP_FLAG_EXACT (the order-faithful kernels read a flat cache).  forge_hip_model_read_kv returns rows in sequence
 * order under either layout. */
int32_t forge_hip_model_set_kv_pages(forge_hip_model* m, uint32_t page_rows, const uint32_t* page_table_host, uint32_t n_pages);
/* Debug/parity: copy layer `layer`'s cached K (which=0) or V (which=1) rows [0,pos) to host as
 * fp16 bit patterns, row-major [pos][kv_heads*head_dim]. */
int32_t forge_hip_model_read_kv(forge_hip_model* m, uint32_t layer, uint32_t which, uint16_t* out_host);

/* ---------------- host-side format helpers (no GPU needed) ---------------- */
/* f16_bits_to_f32 / f32_to_f16_bits (emit.rs:1245-1264, 1460-1495). */
float forge_hip_f16_to_f32(uint16_t bits);
uint16_t forge_hip_f32_to_f16(float x);
/* quantize_f32_to_q8_0 / _q4_0 (weight_loader.rs:1454-1544): n floats -> ceil(n/32) blocks. */
int32_t forge_hip_quantize_f32(uint32_t wdtype, const float* data_host, uint64_t n, uint8_t* out_host);
/* f32::exp as the GPU kernels evaluate it (silu_mul emit.rs:384, softmax emit.rs:688-699): the
 * table-driven binary64 algorithm of the C library's expf, so that CPU and GPU agree bit for bit.
 * This is its host twin, exported so that it can be checked against the C library. */
int32_t forge_hip_expf_host(const float* x_host, uint64_t n, float* out_host);
/* dequant_q8_0 / dequant_q4_0 (weight_loader.rs:860-926). */
int32_t forge_hip_dequant(uint32_t wdtype, const uint8_t* data_host, uint64_t n, float* out_host);

/* ---------------- op-level API ---------------- */

/* Upload one weight matrix given as raw GGUF blocks, row-major [N][K/32] (the `weight: &[u8]`
 * argument of matmul_vec_q8_0_KxN, emit.rs:1958).  K must be a multiple of 32.
 * wdtype FORGE_HIP_Q4_K / FORGE_HIP_Q6_K: raw 144- / 210-byte super-blocks, row-major [N][K/256] (the `weight` argument of
 * matmul_vec_q4_k_KxN / matmul_vec_q6_k_KxN, emit.rs:3411, 3636); K a multiple of 256, at most 16384.  Such a handle is
 * taken by forge_hip_gemv_q only: the reference has no batched matmul for these formats. */
int32_t forge_hip_qweight_create(uint32_t wdtype, const uint8_t* raw_host, uint32_t K, uint32_t N,
                                 forge_hip_qweight** out);
void forge_hip_qweight_destroy(forge_hip_qweight* w);

/* quantize_to_q8_0_blocks_into (emit.rs:1410-1440) for M rows of K floats.
 * q_dev: int8 [M][K]; scales_dev: fp16 bit patterns [M][K/32]. */
int32_t forge_hip_quantize_act(const float* x_dev, uint32_t M, uint32_t K, int8_t* q_dev, uint16_t* scales_dev,
                               void* stream);

/* matmul_vec_q8_0_KxN / matmul_vec_q4_0_KxN (emit.rs:1926-2092, 2797-2958): y[N] = W x.
 * x_dev f32 [K], y_dev f32 [N].  For a Q4_K / Q6_K handle: matmul_vec_q4_k_KxN / matmul_vec_q6_k_KxN (emit.rs:3388-3490,
 * 3622-3655; dots emit.rs:3035-3306, 3553-3612), bit-identical f32. */
int32_t forge_hip_gemv_q(const forge_hip_qweight* w, const float* x_dev, float* y_dev, void* stream);

/* The same matmul in the arithmetic the reference runs on hosts other than aarch64: its portable dot_q8_0 / dot_q4_0
 * (emit.rs:1359-1377, 2337-2359) called once per row by matmul_vec (emit.rs:2046-2092) -- f32 activations against
 * weights dequantised on the fly, y[n] = sum_k x[k] * (f32(q) * scale) added element by element in order (Q4_0: low
 * nibble j, then high nibble j + 16, per byte).  Bit-identical to that code; no activation quantiser is involved. */
int32_t forge_hip_gemv_q_f32act(const forge_hip_qweight* w, const float* x_dev, float* y_dev, void* stream);

/* matmul_mat_q8_0_KxN / matmul_mat_q4_0_KxN (emit.rs:2108-2302, 3667-3817):
 * y[M][N] = x[M][K] W^T, row-major.  With FORGE_HIP_FLAG_EXACT every row has the CPU path's bits.  Without it the block sums
 * are still exact and the f32 combine is within 1e-3, for data whose per-block activation scale is below 256 (largest
 * activation of a block below 32 512) and whose weight scales are below 2: the kernel removes a bias from its block sums with
 * an fp16 matrix instruction on scales multiplied by powers of two, which is exact inside that range only.
 * A Q4_K / Q6_K handle: the reference has no batched matmul for these formats.  With FORGE_HIP_FLAG_EXACT the call computes M
 * rows of matmul_vec_q4_k / _q6_k, each row with forge_hip_gemv_q's bits, reading the matrix once per 8 rows.  Without the
 * flag it runs the int8 MFMA kernel on a re-expression of the matrix in int8 codes and fp16 block scales (Q4_K: codes
 * (q - 8) * g with the multiplier g that makes fp16(d * sc / g) * g closest to d * sc, the minimum term as an f32 product over
 * the activations' block sums; Q6_K: sc * q split into hi and lo codes under the exact scales 64 d and d): block sums stay
 * exact, results lie within 1e-3 of |value| + the row's root mean square.  The first such call builds the re-expression in
 * device memory (Q4_K: 9.5 bits per weight, Q6_K: 17) and the handle keeps it, so the handle must not be used from two
 * threads at once; a matrix with a negative Q4_K d or a block scale of 2 or more falls back to the order-faithful rows.
 * An all-zero block of activations goes into the fast kernel with the scale 0 (the reference's quantiser says 1.0; the codes
 * are zero either way). */
int32_t forge_hip_gemm_q(const forge_hip_qweight* w, const float* x_dev, uint32_t M, float* y_dev, uint32_t flags,
                         void* stream);

/* The gate / up half of the batched feed-forward block in one launch (fast mode): for a handle whose N rows are the gate
 * projection's rows followed by the up projection's (N / 2 each, a multiple of 64), gate = x Wg^T and up = x Wu^T as
 * forge_hip_gemm_q computes them, then silu_mul (emit.rs:380-386, hardware exponential) and the activation quantiser
 * (quantize_to_q8_0_blocks_into, emit.rs:1410-1440) in the kernel's epilogue: out_q_dev int8 [M][N / 2] with the codes of
 * every row's odd blocks negated (the form forge_hip_gemm_q's fast kernel takes its activations in), out_scales_dev
 * fp16 bits [M][N / 64].  What forward_prefill_batched does between the gate / up matmuls and the down matmul
 * (emit.rs:5390-5420) without the [M][N] floats in memory. */
int32_t forge_hip_gemm_silu_q(const forge_hip_qweight* w, const float* x_dev, uint32_t M, int8_t* out_q_dev, uint16_t* out_scales_dev,
                              void* stream);

/* The int32 block sums the two calls above combine: out_dev int32 [M][N][K/32]
 * (dot_q8_0_q8_0 / dot_q4_0_q8_0 `vaddvq_s32(acc)`, emit.rs:1543-1553, 2522-2552).
 * path 0 = the GEMV kernel's dot, path 1 = the MFMA GEMM kernel's tiles in exact mode, path 2 = the same kernel in the
 * fast mode (which accumulates the sums on top of a floating-point bias, negates odd blocks and feeds 4-bit codes times
 * 16: the sums written out are recovered from those accumulators, so they show what the fast arithmetic really summed). */
int32_t forge_hip_block_isums(const forge_hip_qweight* w, const float* x_dev, uint32_t M, int32_t* out_dev,
                              uint32_t path, void* stream);

/* rms_norm (emit.rs:327-334) on M rows of H floats. */
int32_t forge_hip_rms_norm(const float* x_dev, const float* w_dev, float eps, uint32_t M, uint32_t H, float* out_dev,
                           void* stream);
/* silu_mul (emit.rs:380-386). */
int32_t forge_hip_silu_mul(const float* gate_dev, const float* up_dev, uint64_t n, float* out_dev, void* stream);

/* rope (emit.rs:508-528) on q and k for M tokens at positions base_pos.., then the KV-cache
 * write of k and v as fp16 (the reference's GPU backend: metal:3475-3553).
 * q_dev f32 [M][heads*hd] (rotated in place); k_dev, v_dev f32 [M][kv_heads*hd] (k rotated in
 * place); k_cache_dev, v_cache_dev: fp16 [max_seq][kv_heads*hd]. */
int32_t forge_hip_rope_kv_store(float* q_dev, float* k_dev, const float* v_dev, uint16_t* k_cache_dev,
                                uint16_t* v_cache_dev, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                                uint32_t head_dim, float theta, void* stream);

/* attention_flash_batch (emit.rs:754-883) over an fp16 cache: causal, GQA.
 * q_dev f32 [M][heads*hd] (already rotated); caches hold rows [0, base_pos+M);
 * out_dev f32 [M][heads*hd]. */
int32_t forge_hip_attn_prefill_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                     float* out_dev, uint32_t M, uint32_t base_pos, uint32_t heads, uint32_t kv_heads,
                                     uint32_t head_dim, uint32_t flags, void* stream);

/* attention_flash (emit.rs:656-715) over an fp16 cache: one query against seq_len rows.
 * q_dev f32 [heads*hd], out_dev f32 [heads*hd]. */
int32_t forge_hip_attn_decode_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                    float* out_dev, uint32_t seq_len, uint32_t heads, uint32_t kv_heads,
                                    uint32_t head_dim, uint32_t flags, void* stream);

/* forge_hip_attn_decode_f16kv without FORGE_HIP_FLAG_EXACT for callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same kernels, same
 * results bit for bit; the split records (heads * 32 * (head_dim + 2) floats) go to a fixed 2 129 920-byte array in the
 * library's device image (one copy per GPU, held until the process ends) instead of the op-level API's lazily grown
 * allocation, and the call makes no hipMalloc / hipFree.  heads <= 128, else FORGE_HIP_ERR_INVALID.  Every call on a GPU
 * uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 * The array's device address is looked up once per device when a model or a weight handle is created there
 * (forge_hip_model_create*, forge_hip_qweight_create), else at the first call on the device: a caller that holds neither
 * makes one call outside a graph capture first. */
int32_t forge_hip_attn_decode_f16kv_noalloc(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                            float* out_dev, uint32_t seq_len, uint32_t heads, uint32_t kv_heads,
                                            uint32_t head_dim, void* stream);

/* forge_hip_attn_decode_f16kv (fast arithmetic) over a PAGED fp16 cache, for hosts whose KV memory is a pool of pages
 * shared by several sequences.  The reference's own cache is one flat array per model (emit.rs:532-545, metal:3525-3553), so
 * this has no reference call to replace; its result is, bit for bit, that of forge_hip_attn_decode_f16kv on the same rows
 * laid out flat.  k_pool_dev / v_pool_dev: fp16 [pages][page_rows][kv_heads*head_dim]; row t of the sequence is row
 * t % page_rows of pool page page_table_dev[t / page_rows] (uint32 indices, ceil(seq_len / page_rows) entries);
 * page_rows a power of two (a 262 144-row sequence needs pages of at least 8 rows). */
int32_t forge_hip_attn_decode_f16kv_paged(const float* q_dev, const uint16_t* k_pool_dev, const uint16_t* v_pool_dev,
                                          const uint32_t* page_table_dev, uint32_t page_rows, float* out_dev, uint32_t seq_len,
                                          uint32_t heads, uint32_t kv_heads, uint32_t head_dim, void* stream);

/* attention_sliding_batch (emit.rs:907-1046) over an fp16 cache: as forge_hip_attn_prefill_f16kv, but the query at
 * position p = base_pos + row sees only the keys [max(0, p - window + 1), p]; window >= 1. */
int32_t forge_hip_attn_prefill_sliding_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                             float* out_dev, uint32_t M, uint32_t base_pos, uint32_t window, uint32_t heads,
                                             uint32_t kv_heads, uint32_t head_dim, uint32_t flags, void* stream);

/* attention_sliding (emit.rs:598-627) over an fp16 cache: one query against the last min(window, seq_len) of seq_len
 * cached rows; window >= 1.  With FORGE_HIP_FLAG_EXACT at most 12288 rows (their scores stay in LDS). */
int32_t forge_hip_attn_decode_sliding_f16kv(const float* q_dev, const uint16_t* k_cache_dev, const uint16_t* v_cache_dev,
                                            float* out_dev, uint32_t seq_len, uint32_t window, uint32_t heads,
                                            uint32_t kv_heads, uint32_t head_dim, uint32_t flags, void* stream);

/* argmax (project.rs:501-503): index of the LAST maximum of n floats -> *out_dev (uint32). */
int32_t forge_hip_argmax(const float* x_dev, uint32_t n, uint32_t* out_dev, void* stream);

/* ---------------- GGUF input (host code; no GPU needed except for the last call) ----------------
 * The reference reads a model from a GGUF file in three steps: gguf::parse (crates/forgellm-frontend/src/gguf.rs:484-551),
 * load_config (crates/forgellm-cli/src/main.rs:700-830) and `forge export-weights` (main.rs:2585-2757, tensor names
 * mapped by weight_loader.rs:400-447), whose output file is the blob forge_hip_model_create takes.  These entry points are
 * those three steps.  Supported: architectures "llama", "qwen2" (sets FORGE_HIP_FLAG_QKV_BIAS) , "mistral"
 * (`<arch>.attention.sliding_window` becomes config.sliding_window, main.rs:764-767) and "phi3" / "phi" (main.rs:759; the fused
 * attn_qkv.weight and ffn_up.weight tensors are cut apart like split_fused_tensors, weight_loader.rs:543-583);
 * tensors of GGML type F32, F16, BF16, Q8_0, Q4_0 and -- turned into Q8_0 blocks when they are read, as the reference's loader
 * does (weight_loader.rs:219-229) -- Q4_1, Q4_K, Q5_K, Q6_K, Q8_K; projections mostly Q8_0 or mostly Q4_0 by the reference's
 * majority vote, which counts those other types as Q8_0 (a file whose projections are mostly Q4_K is refused: the reference
 * runs it on Q4_K kernels of its own). */
typedef struct forge_hip_gguf forge_hip_gguf;

/* gguf::parse over a file (memory-mapped until close) or over bytes the caller keeps alive until close.  Failures are
 * FORGE_HIP_ERR_INVALID with the reference's GGUFError text (invalid magic, unsupported version, unsupported GGML
 * type / metadata value type, invalid UTF-8, more than 4 dimensions) or a message saying where the file ends early. */
int32_t forge_hip_gguf_open(const char* path, forge_hip_gguf** out);
int32_t forge_hip_gguf_parse(const uint8_t* data_host, uint64_t nbytes, forge_hip_gguf** out);
void forge_hip_gguf_close(forge_hip_gguf* g);

/* Fields of GGUFFile (gguf.rs:287-297). */
uint32_t forge_hip_gguf_version(const forge_hip_gguf* g);
uint64_t forge_hip_gguf_alignment(const forge_hip_gguf* g);
uint64_t forge_hip_gguf_tensor_data_offset(const forge_hip_gguf* g);
uint64_t forge_hip_gguf_tensor_count(const forge_hip_gguf* g);
uint64_t forge_hip_gguf_metadata_count(const forge_hip_gguf* g);
/* GGUFTensorInfo (gguf.rs:262-285) of tensor `index`; any output pointer may be NULL.  `name` stays valid until close;
 * dims4 receives 4 values (unused ones 0); data_size = ceil(numel / block) * bytes per block. */
int32_t forge_hip_gguf_tensor(const forge_hip_gguf* g, uint64_t index, const char** name, uint32_t* n_dims, uint64_t* dims4,
                              uint32_t* ggml_type, uint64_t* offset, uint64_t* data_size);
/* GGUFFile::tensor (gguf.rs:338-340): index of the tensor of that name, or -1. */
int64_t forge_hip_gguf_find_tensor(const forge_hip_gguf* g, const char* name);
/* One metadata value: its GGUF type id (0..12); `bits` = the bytes of a scalar, little endian, zero-extended (a bool is 0 or
 * 1); `str` for type 8 (else NULL); element type and element count for type 9 (array elements are not kept).
 * Unknown key: FORGE_HIP_ERR_INVALID. */
int32_t forge_hip_gguf_meta(const forge_hip_gguf* g, const char* key, uint32_t* type, uint64_t* bits, const char** str,
                            uint32_t* elem_type, uint64_t* count);

/* load_config (main.rs:700-830): `<arch>.embedding_length`, `.block_count`, `.attention.head_count`, `.attention.head_count_kv`
 * (default: head_count), `.feed_forward_length` (4 x hidden), vocabulary = length of `tokenizer.ggml.tokens`, else
 * `<arch>.vocab_size`, else 32000; `.context_length` (2048), `.attention.layer_norm_rms_epsilon` (1e-5), `.rope.freq_base`
 * (10000); head_dim = hidden / heads; weight format by majority vote over the projection tensors; lm_head format from
 * `output.weight` (absent: tied to the embedding, stored in the projections' format).  max_seq = 0 takes the file's context
 * length. */
int32_t forge_hip_gguf_config(const forge_hip_gguf* g, uint32_t max_seq, uint32_t flags, forge_hip_config* out);
/* `forge export-weights` (main.rs:2585-2757) into the caller's buffer of exactly forge_hip_weights_nbytes(cfg) bytes:
 * f32 embedding table, per layer attn_norm | q | k | v | o | ffn_norm | gate | up | down, final norm, lm_head.  A tensor
 * stored in another format than the blob needs is converted with the reference's own routines (dequant
 * weight_loader.rs:809-926, quantisers :1454-1544). */
int32_t forge_hip_gguf_export_weights(const forge_hip_gguf* g, const forge_hip_config* cfg, uint8_t* out_host, uint64_t nbytes);
/* `dequantize` (weight_loader.rs:809-825) for one tensor's bytes: GGML types F32 (0), F16 (1), BF16 (30), Q8_0 (8), Q4_0 (2),
 * Q4_1 (3), Q4_K (12), Q5_K (13), Q6_K (14), Q8_K (15); n = number of elements. */
int32_t forge_hip_dequant_ggml(uint32_t ggml_type, const uint8_t* data_host, uint64_t n, float* out_host);
/* A GGUF file whose tensor categories are not all stored alike (llama.cpp's Q4_K_M: Q4_K for most projections, Q6_K for
 * half of attn_v / ffn_down and for the output matrix).  detect_gguf_proj_dtypes (main.rs:608-680): per category (q, k, v, o,
 * gate, up, down, the embedding table, the output matrix) the format most of its tensors have among Q8_0, Q4_0, Q4_K, Q6_K
 * and "dense" (F32 / F16 / BF16), equal counts going to the more precise one; a category none of whose tensors votes takes
 * the file's majority format (forge_hip_gguf_config's vote, which here may also come out as Q4_K); without an output tensor
 * the lm_head takes the embedding's format.  proj_dtypes receives the seven projection formats, *embed_dtype (may be NULL)
 * the embedding's (1 = dense), out->lm_head_dtype the lm_head's; out->wdtype is the majority format when that is Q8_0 or
 * Q4_0, else Q8_0 (forge_hip_model_create_mixed does not read it).  A dense projection or lm_head category is reported as
 * the majority format (Q8_0 under a Q4_K majority): the reference would keep such weights as f32, which this library does
 * not carry. */
int32_t forge_hip_gguf_config_mixed(const forge_hip_gguf* g, uint32_t max_seq, uint32_t flags, forge_hip_config* out,
                                    uint32_t* proj_dtypes, uint32_t* embed_dtype);
/* The blob of forge_hip_model_create_mixed (exactly forge_hip_weights_nbytes_mixed(cfg, proj_dtypes) bytes) from the file's
 * tensors, as load_from_file_mixed_per_tensor + export-weights produce it (weight_loader.rs:152-238, main.rs:2556-2757): a
 * tensor that already has its category's format is copied; for a Q4_K / Q6_K category any other tensor is dequantised and
 * quantised again with quantize_f32_to_q4_k / _q6_k; for a Q8_0 / Q4_0 category the conversion is that of
 * forge_hip_gguf_export_weights; a Q4_K / Q6_K embedding table is dequantised directly into the f32 table.  Fused Phi-3
 * tensors and QKV bias are refused here. */
int32_t forge_hip_gguf_export_weights_mixed(const forge_hip_gguf* g, const forge_hip_config* cfg, const uint32_t* proj_dtypes,
                                            uint8_t* out_host, uint64_t nbytes);
/* quantize_f32_to_q4_k (weight_loader.rs:1773-1882, sub-block fit make_qkx2_quants :1666-1768) and quantize_f32_to_q6_k
 * (:2025-2140): n floats -> ceil(n / 256) super-blocks of 144 (ggml_type 12) or 210 (14) bytes; a tail is padded with zeros. */
int32_t forge_hip_quantize_kquant(uint32_t ggml_type, const float* data_host, uint64_t n, uint8_t* out_host);
/* open + config + export_weights + forge_hip_model_create; a file that forge_hip_gguf_config_mixed finds to hold several
 * formats (or a K-quant lm_head) goes through the _mixed functions and forge_hip_model_create_mixed instead. */
int32_t forge_hip_model_create_from_gguf(const char* path, uint32_t max_seq, uint32_t flags, forge_hip_model** out);

/* ---------------- sampling (the loop of the generated main.rs, project.rs:714-751) ----------------
 * The reference's default generation is greedy WITH a repeat penalty of 1.1 (project.rs:607-611): after every
 * `forward` it runs apply_repeat_penalty over all tokens fed so far (prompt and generated, once per occurrence) and then
 * takes the argmax.  The model keeps that occurrence count per token id on the device (prefill and decode steps add to
 * it, reset clears it); with a penalty > 1 set here, forge_hip_forward_greedy returns the last maximum of the penalised
 * logits, bit for bit what apply_repeat_penalty + argmax give on the logits of forge_hip_forward.  The logits handed
 * back by forge_hip_forward / forge_hip_prefill_batch stay unpenalised, as the reference's `forward` returns them, and
 * the token after a prefill is the caller's argmax of those (the reference does not penalise it, project.rs:719-720).
 * penalty <= 1 switches the penalty off (the reference's `if penalty <= 1.0 { return; }`). */
int32_t forge_hip_model_set_repeat_penalty(forge_hip_model* m, float penalty);

/* apply_repeat_penalty (project.rs:505-513) on host logits: for each entry of `recent`, in order,
 * `l > 0 ? l /= penalty : l *= penalty`. */
int32_t forge_hip_apply_repeat_penalty(float* logits_host, uint64_t n, const uint32_t* recent_host, uint64_t n_recent,
                                       float penalty);
/* sample (project.rs:515-555) on host logits, which it overwrites like the reference's `&mut [f32]`: temperature,
 * softmax with sequential f32 sums, top-k, top-p (the entry that crosses the threshold is dropped too, as in the
 * reference), renormalisation, one xorshift64 step of *rng_state, `r = state as f32 / u64::MAX as f32`, first index whose
 * running sum reaches r (else the last index).  temperature <= 0: the last maximum, state untouched.  A NaN logit is
 * FORGE_HIP_ERR_INVALID (the reference panics).  Among equal probabilities the lower index sorts first (the
 * reference's unstable sort leaves that order open). */
int32_t forge_hip_sample(float* logits_host, uint64_t n, float temperature, uint64_t top_k, float top_p, uint64_t* rng_state,
                         uint32_t* out);

#ifdef __cplusplus
}
#endif
#endif /* FORGE_HIP_H */

// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// CPU restatement (oracle) of the ForgeLLM reference's generated CPU kernels for the
// quantized-Llama hot path.  Only tests, the smoke check and the benchmark's
// cpu_baseline leg may load this library; the HIP product never calls into it.
//
// The reference emits these kernels as Rust source text from
// crates/forgellm-codegen-cpu/src/emit.rs ("emit.rs" below) and
// crates/forgellm-frontend/src/weight_loader.rs ("wl" below); each function here cites
// the lines it follows.  Two arithmetic variants exist in the reference, selected by
// target_arch, and both are restated:
//   variant A (aarch64): activations quantised per 32-block to int8, exact int32 block
//                        dots, f32 combine                     (emit.rs:1410-1440,1511-1911)
//   variant B (other):   f32 activations x on-the-fly dequantised weights, one sequential
//                        f32 accumulator per row               (emit.rs:1359-1377,2337-2359)
// KV cache modes: 0 = int8 + per-token f32 scale (the reference CPU path, emit.rs:532-545),
//                 1 = fp16 (what the reference's GPU backend and the HIP product store).
//
// Build with -ffp-contract=off: Rust never contracts a*b+c, so neither may this file
// (fused multiply-adds appear only where the reference itself uses vfmaq_f32).
//
// Pinning status (what a test checks each function against, other than itself):
//   f16<->f32, dequant, weight quantisers, kv quantiser, rms_norm, silu, softmax, rope,
//   argmax, attention vs attention_flash vs attention_flash_batch: pinned by the
//   reference's own unit-test vectors and closed forms (tests/test_oracle_*.py).
//   attention_sliding / attention_sliding_batch: no reference test executes them; pinned by
//   an fp64 softmax over the window written from the definition, by window >= seq being
//   attention_std, and by batch == per-token.
//   block isums: pinned by brute-force int64.  f32 combines / matmuls: pinned against an
//   fp64 evaluation of the same quantised operands.
//   forward / forward_prefill_batched for Q8_0/Q4_0: PARITY UNPINNED by any reference
//   test (the reference never executes them in a test); pinned only by self-consistency
//   (per-token loop == batched prefill) and by the fp64 checks of the pieces.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#if defined(_OPENMP)
#include <omp.h>
#endif

namespace {

constexpr int QK = 32;          // elements per quant block (gguf.rs:236-240)
constexpr int Q8_BYTES = 34;    // f16 scale + 32 x i8
constexpr int Q4_BYTES = 18;    // f16 scale + 16 packed bytes
constexpr int FLASH_BLOCK = 64; // FLASH_ATTN_BLOCK_SIZE (emit.rs:201)

inline float bits_f32(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }
inline uint32_t f32_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }

// emit.rs:1245-1264 (same as wl:1327-1358)
float f16_to_f32(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u;
    uint32_t exponent = (bits >> 10) & 0x1Fu;
    uint32_t mantissa = bits & 0x3FFu;
    if (exponent == 0) {
        if (mantissa == 0) return bits_f32(sign << 31);
        uint32_t m = mantissa;
        int e = -14;
        while ((m & 0x400u) == 0) { m <<= 1; e -= 1; }
        m &= 0x3FFu;
        uint32_t fe = (uint32_t)(e + 127) & 0xFFu;
        return bits_f32((sign << 31) | (fe << 23) | (m << 13));
    }
    if (exponent == 31) return bits_f32((sign << 31) | (0xFFu << 23) | (mantissa << 13));
    uint32_t fe = (uint32_t)((int)exponent - 15 + 127);
    return bits_f32((sign << 31) | (fe << 23) | (mantissa << 13));
}

// emit.rs:1460-1495 (same as wl:1361-1442): round-to-nearest-even, except that f32
// subnormals and anything with unbiased exponent < -24 become signed zero.
uint16_t f32_to_f16(float x) {
    uint32_t bits = f32_bits(x);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int exp_f32 = (int)((bits >> 23) & 0xFFu);
    uint32_t mant = bits & 0x7FFFFFu;
    if (exp_f32 == 0xFF) {
        uint16_t h_mant = (uint16_t)((mant >> 13) & 0x3FFu);
        if (mant != 0 && h_mant == 0) h_mant = 1;
        return (uint16_t)(sign | 0x7C00u | h_mant);
    }
    if (exp_f32 == 0) return sign;
    int unbiased = exp_f32 - 127;
    if (unbiased > 15) return (uint16_t)(sign | 0x7C00u);
    if (unbiased < -24) return sign;
    uint32_t implicit = mant | 0x00800000u;
    uint32_t shift = unbiased < -14 ? (uint32_t)(-1 - unbiased) : 13u;
    uint32_t mask = (1u << shift) - 1u;
    uint32_t dropped = implicit & mask;
    uint32_t half = 1u << (shift - 1);
    uint32_t truncated = implicit >> shift;
    if (dropped > half || (dropped == half && (truncated & 1u) == 1u)) truncated += 1;
    if (unbiased < -14) {
        if (truncated >= 0x400u) return (uint16_t)(sign | (1u << 10));
        return (uint16_t)(sign | truncated);
    }
    uint32_t h_exp = (uint32_t)(unbiased + 15);
    if (truncated >= 0x800u) {
        h_exp += 1;
        if (h_exp >= 0x1Fu) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | (h_exp << 10));
    }
    return (uint16_t)(sign | (h_exp << 10) | (truncated & 0x3FFu));
}

inline uint16_t rd16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

// Rust `(x).round().clamp(-127.0, 127.0) as i8`: round half away from zero.
inline int8_t round_clamp_i8(float v) {
    float r = roundf(v);
    if (r < -127.0f) r = -127.0f;
    if (r > 127.0f) r = 127.0f;
    if (r != r) return 0; // NaN as i8 == 0 in Rust
    return (int8_t)r;
}

// wl:860-888
void dequant_q8_0(const uint8_t* data, int64_t n, float* out) {
    int64_t nb = (n + QK - 1) / QK;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = data + b * Q8_BYTES;
        float scale = f16_to_f32(rd16(blk));
        for (int j = 0; j < QK && b * QK + j < n; j++) out[b * QK + j] = (float)(int8_t)blk[2 + j] * scale;
    }
}

// wl:893-926
void dequant_q4_0(const uint8_t* data, int64_t n, float* out) {
    int64_t nb = (n + QK - 1) / QK;
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t* blk = data + b * Q4_BYTES;
        float scale = f16_to_f32(rd16(blk));
        for (int j = 0; j < 16; j++) {
            uint8_t byte = blk[2 + j];
            int lo = (int)(byte & 0x0F) - 8;
            int hi = (int)((byte >> 4) & 0x0F) - 8;
            int64_t ilo = b * QK + j, ihi = b * QK + j + 16;
            if (ilo < n) out[ilo] = (float)lo * scale;
            if (ihi < n) out[ihi] = (float)hi * scale;
        }
    }
}

// wl:1454-1486
void quantize_f32_to_q8_0(const float* data, int64_t n, uint8_t* out) {
    int64_t nb = (n + QK - 1) / QK;
    std::memset(out, 0, (size_t)nb * Q8_BYTES);
    for (int64_t blk = 0; blk < nb; blk++) {
        int64_t base = blk * QK, end = std::min<int64_t>(base + QK, n);
        float amax = 0.0f;
        for (int64_t i = base; i < end; i++) { float a = fabsf(data[i]); if (a > amax) amax = a; }
        float scale = amax == 0.0f ? 0.0f : amax / 127.0f;
        float inv = scale != 0.0f ? 1.0f / scale : 0.0f;
        uint8_t* ob = out + blk * Q8_BYTES;
        uint16_t sb = f32_to_f16(scale);
        ob[0] = (uint8_t)sb; ob[1] = (uint8_t)(sb >> 8);
        for (int64_t i = base; i < end; i++) ob[2 + (i - base)] = (uint8_t)round_clamp_i8(data[i] * inv);
    }
}

// wl:1494-1544 (scale = unsigned amax / 8; code = clamp(round(v*inv)+8, 0, 15))
void quantize_f32_to_q4_0(const float* data, int64_t n, uint8_t* out) {
    int64_t nb = (n + QK - 1) / QK;
    for (int64_t blk = 0; blk < nb; blk++) {
        int64_t base = blk * QK, end = std::min<int64_t>(base + QK, n);
        float amax = 0.0f;
        for (int64_t i = base; i < end; i++) { float a = fabsf(data[i]); if (a > amax) amax = a; }
        float scale = amax / 8.0f;
        float inv = scale != 0.0f ? 1.0f / scale : 0.0f;
        uint8_t* ob = out + blk * Q4_BYTES;
        uint16_t sb = f32_to_f16(scale);
        ob[0] = (uint8_t)sb; ob[1] = (uint8_t)(sb >> 8);
        for (int j = 0; j < 16; j++) {
            float lo_v = base + j < n ? data[base + j] : 0.0f;
            float hi_v = base + j + 16 < n ? data[base + j + 16] : 0.0f;
            // Rust: ((v*inv).round() as i32 + 8).clamp(0,15); `as i32` saturates.
            auto code = [](float v) -> uint8_t {
                float r = roundf(v);
                int64_t q = (r != r) ? 0 : (int64_t)std::max(-2147483648.0f, std::min(r, 2147483520.0f));
                q += 8;
                if (q < 0) q = 0;
                if (q > 15) q = 15;
                return (uint8_t)q;
            };
            ob[2 + j] = (uint8_t)(code(lo_v * inv) | (code(hi_v * inv) << 4));
        }
    }
}

// emit.rs:1410-1440 — activation quantiser of variant A.
void quantize_act_q8_0(const float* in, int64_t k, uint8_t* out) {
    int64_t nb = (k + QK - 1) / QK;
    for (int64_t b = 0; b < nb; b++) {
        int64_t s = b * QK, e = std::min<int64_t>(s + QK, k);
        float absmax = 0.0f;
        for (int64_t i = s; i < e; i++) absmax = fmaxf(absmax, fabsf(in[i]));
        float scale, inv;
        if (absmax == 0.0f) { scale = 1.0f; inv = 0.0f; }
        else { scale = absmax / 127.0f; inv = 1.0f / scale; }
        uint16_t sb = f32_to_f16(scale);
        uint8_t* ob = out + b * Q8_BYTES;
        ob[0] = (uint8_t)(sb & 0xFF); ob[1] = (uint8_t)(sb >> 8);
        for (int64_t i = s; i < e; i++) ob[2 + (i - s)] = (uint8_t)round_clamp_i8(in[i] * inv);
        for (int64_t j = e - s; j < QK; j++) ob[2 + j] = 0;
    }
}

// Exact int32 block dot of one Q8_0 activation block with one weight block
// (emit.rs:1543-1553 for Q8_0 weights; emit.rs:2522-2552 for Q4_0 weights: low nibbles
// pair with activation elements 0..15, high nibbles with 16..31, both minus 8).
inline int32_t block_isum(int wdtype, const uint8_t* a_blk, const uint8_t* w_blk) {
    const int8_t* a = (const int8_t*)(a_blk + 2);
    int32_t s = 0;
    if (wdtype == 8) {
        const int8_t* w = (const int8_t*)(w_blk + 2);
        for (int j = 0; j < QK; j++) s += (int32_t)a[j] * (int32_t)w[j];
    } else {
        const uint8_t* w = w_blk + 2;
        for (int j = 0; j < 16; j++) {
            int lo = (int)(w[j] & 0x0F) - 8, hi = (int)(w[j] >> 4) - 8;
            s += lo * (int32_t)a[j] + hi * (int32_t)a[j + 16];
        }
    }
    return s;
}
inline int wbytes(int wdtype) { return wdtype == 8 ? Q8_BYTES : Q4_BYTES; }

// Row dot, variant A.  seq=true: dot8/dot4 order, r += s_b * f32(isum_b) for b ascending
// (emit.rs:1770-1877, 1630-1696, 2666-2782).  seq=false: dot1 order with four interleaved
// accumulators and the fa0,fa1,fa2 tail rule (emit.rs:1558-1571, 2555-2563).
float dot_a(int wdtype, const uint8_t* a_q8, const uint8_t* w, int64_t k, bool seq) {
    int64_t nb = k / QK;
    int wb = wbytes(wdtype);
    auto block = [&](int64_t b) -> float {
        float a_s = f16_to_f32(rd16(a_q8 + b * Q8_BYTES));
        float w_s = f16_to_f32(rd16(w + b * wb));
        float combined = a_s * w_s;
        return combined * (float)block_isum(wdtype, a_q8 + b * Q8_BYTES, w + b * wb);
    };
    if (seq) {
        float r = 0.0f;
        for (int64_t b = 0; b < nb; b++) r += block(b);
        return r;
    }
    float fa0 = 0, fa1 = 0, fa2 = 0, fa3 = 0;
    int64_t groups = nb / 4;
    for (int64_t g = 0; g < groups; g++) {
        fa0 += block(g * 4); fa1 += block(g * 4 + 1); fa2 += block(g * 4 + 2); fa3 += block(g * 4 + 3);
    }
    int64_t tail = groups * 4;
    if (tail < nb) fa0 += block(tail);
    if (tail + 1 < nb) fa1 += block(tail + 1);
    if (tail + 2 < nb) fa2 += block(tail + 2);
    return fa0 + fa1 + fa2 + fa3;
}

// Row dot, variant B (emit.rs:1359-1377 Q8_0; emit.rs:2337-2359 Q4_0).
float dot_b(int wdtype, const float* x, const uint8_t* w, int64_t k) {
    int64_t nb = (k + QK - 1) / QK;
    float sum = 0.0f;
    if (wdtype == 8) {
        for (int64_t b = 0; b < nb; b++) {
            const uint8_t* blk = w + b * Q8_BYTES;
            float scale = f16_to_f32(rd16(blk));
            int64_t s = b * QK, e = std::min<int64_t>(s + QK, k);
            for (int64_t j = 0; j < e - s; j++) sum += x[s + j] * ((float)(int8_t)blk[2 + j] * scale);
        }
    } else {
        for (int64_t b = 0; b < nb; b++) {
            const uint8_t* blk = w + b * Q4_BYTES;
            float scale = f16_to_f32(rd16(blk));
            for (int j = 0; j < 16; j++) {
                uint8_t byte = blk[2 + j];
                int lo = (int)(byte & 0x0F) - 8, hi = (int)((byte >> 4) & 0x0F) - 8;
                int64_t ilo = b * QK + j, ihi = b * QK + j + 16;
                if (ilo < k) sum += x[ilo] * ((float)lo * scale);
                if (ihi < k) sum += x[ihi] * ((float)hi * scale);
            }
        }
    }
    return sum;
}

// Which rows of a variant-A matmul take the dot1 (4-accumulator) order instead of the
// sequential dot8/dot4 order.  matmul_vec (emit.rs:1971-2046): when N*row_bytes >= 1e6 the
// rows are split in chunks of 256 and within a chunk of length L the last L%4 rows use
// dot1; otherwise L = N.  matmul_mat (emit.rs:2150-2268): L = N.  lm_head inside
// forward_prefill_batched (emit.rs:5455-5470): chunks of 256, last L%8 rows use dot1.
inline bool row_is_dot1(int64_t row, int64_t n, int64_t chunk, int tail_mod) {
    int64_t base = chunk > 0 ? (row / chunk) * chunk : 0;
    int64_t len = chunk > 0 ? std::min<int64_t>(chunk, n - base) : n;
    int64_t i = row - base;
    return i >= len - (len % tail_mod);
}

// The switch to 256-row chunks compares N * ceil(K/32) * 34 with one megabyte for Q8_0 (emit.rs:1971) and, with the
// same 34-byte figure, for Q4_0 (emit.rs:2837); the lm_head loops are always chunked (emit.rs:4304, 5452).
inline bool matmul_vec_is_chunked(int64_t k, int64_t n, int lm_head_mode) {
    return lm_head_mode != 0 || n * ((k + QK - 1) / QK * Q8_BYTES) >= 1000000;
}

void matmul_vec(int wdtype, int variant, float* out, const float* in, const uint8_t* w,
                int64_t k, int64_t n, int lm_head_mode /*0 vec,1 forward lm,2 prefill lm*/) {
    int64_t row_bytes = (k + QK - 1) / QK * wbytes(wdtype);
    bool par = matmul_vec_is_chunked(k, n, lm_head_mode);
    int64_t chunk = par ? 256 : 0;
    int tail_mod = lm_head_mode == 2 ? 8 : 4;
    if (variant == 0) {
        std::vector<uint8_t> a_q8((size_t)((k + QK - 1) / QK * Q8_BYTES));
        quantize_act_q8_0(in, k, a_q8.data());
#pragma omp parallel for schedule(static) if (par)
        for (int64_t r = 0; r < n; r++)
            out[r] = dot_a(wdtype, a_q8.data(), w + r * row_bytes, k, !row_is_dot1(r, n, chunk, tail_mod));
    } else {
#pragma omp parallel for schedule(static) if (par)
        for (int64_t r = 0; r < n; r++) out[r] = dot_b(wdtype, in, w + r * row_bytes, k);
    }
}

// emit.rs:2108-2302 (Q8_0), emit.rs:3667-3817 (Q4_0).
void matmul_mat(int wdtype, int variant, float* out, int64_t m, const float* in, const uint8_t* w,
                int64_t k, int64_t n) {
    int64_t row_bytes = (k + QK - 1) / QK * wbytes(wdtype);
    if (variant == 0) {
        int64_t a_row = (k + QK - 1) / QK * Q8_BYTES;
        std::vector<uint8_t> a_q8((size_t)(m * a_row));
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < m; r++) quantize_act_q8_0(in + r * k, k, a_q8.data() + r * a_row);
        int64_t nblk = (n + 7) / 8;
#pragma omp parallel for schedule(dynamic, 4)
        for (int64_t nb = 0; nb < nblk; nb++) {
            int64_t j0 = nb * 8, j1 = std::min<int64_t>(j0 + 8, n);
            for (int64_t r = 0; r < m; r++)
                for (int64_t j = j0; j < j1; j++)
                    out[r * n + j] = dot_a(wdtype, a_q8.data() + r * a_row, w + j * row_bytes, k,
                                           !row_is_dot1(j, n, 0, 4));
        }
    } else {
        // emit.rs:2276-2299: a loop of matmul_vec over the m rows.
        for (int64_t r = 0; r < m; r++) matmul_vec(wdtype, 1, out + r * n, in + r * k, w, k, n, 0);
    }
}

// dot_f32: variant B / generic = sequential (emit.rs:298-304); variant A = the NEON
// 16-lane fused order (emit.rs:272-295).
float dot_f32(const float* a, const float* b, int64_t len, int variant) {
    if (variant != 0) {
        float s = 0.0f;
        for (int64_t i = 0; i < len; i++) s += a[i] * b[i];
        return s;
    }
    float s[16];
    for (int i = 0; i < 16; i++) s[i] = 0.0f;
    int64_t chunks = len / 16;
    for (int64_t c = 0; c < chunks; c++)
        for (int i = 0; i < 16; i++) s[i] = fmaf(a[c * 16 + i], b[c * 16 + i], s[i]);
    float t[4];
    for (int i = 0; i < 4; i++) { float s01 = s[i] + s[4 + i]; float s23 = s[8 + i] + s[12 + i]; t[i] = s01 + s23; }
    float r = (t[0] + t[1]) + (t[2] + t[3]); // vaddvq_f32 = pairwise adds
    for (int64_t i = chunks * 16; i < len; i++) r += a[i] * b[i];
    return r;
}

// emit.rs:306-334
void rms_norm(float* out, const float* in, const float* w, int64_t n, float eps, int variant) {
    float ss = dot_f32(in, in, n, variant);
    float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int64_t i = 0; i < n; i++) out[i] = in[i] * inv * w[i];
}

// emit.rs:380-386
void silu_mul(float* out, const float* g, const float* u, int64_t n) {
    for (int64_t i = 0; i < n; i++) { float x = g[i]; out[i] = (x / (1.0f + expf(-x))) * u[i]; }
}

// emit.rs:490-497
void softmax(float* v, int64_t n) {
    float mx = -INFINITY;
    for (int64_t i = 0; i < n; i++) mx = fmaxf(mx, v[i]);
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) { v[i] = expf(v[i] - mx); sum += v[i]; }
    float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    for (int64_t i = 0; i < n; i++) v[i] *= inv;
}

// emit.rs:501-504
void rope_freqs(float* f, int head_dim, float theta) {
    for (int i = 0; i < head_dim / 2; i++) f[i] = 1.0f / powf(theta, 2.0f * (float)i / (float)head_dim);
}

// emit.rs:508-528 — interleaved pairs (2i, 2i+1), one table for all heads.
void rope(float* data, int64_t pos, int head_dim, int num_heads, const float* freqs) {
    int half = head_dim / 2;
    std::vector<float> c(half), s(half);
    for (int i = 0; i < half; i++) {
        float angle = (float)pos * freqs[i];
        s[i] = sinf(angle); c[i] = cosf(angle);
    }
    for (int h = 0; h < num_heads; h++) {
        float* d = data + (int64_t)h * head_dim;
        for (int i = 0; i < half; i++) {
            float x0 = d[2 * i], x1 = d[2 * i + 1];
            d[2 * i] = x0 * c[i] - x1 * s[i];
            d[2 * i + 1] = x0 * s[i] + x1 * c[i];
        }
    }
}

// emit.rs:532-545
float quantize_kv(const float* v, int64_t n, int8_t* out) {
    float max_abs = 0.0f;
    for (int64_t i = 0; i < n; i++) { float a = fabsf(v[i]); if (a > max_abs) max_abs = a; }
    float scale = max_abs / 127.0f;
    float inv = max_abs > 0.0f ? 127.0f / max_abs : 0.0f;
    for (int64_t i = 0; i < n; i++) out[i] = round_clamp_i8(v[i] * inv);
    return scale;
}

// KV cache view for one layer.  mode 0: int8 rows + per-token scales (emit.rs:3954-4019);
// mode 1: fp16 bit patterns, no scales (scale taken as exactly 1).
struct KVView {
    int mode;
    const int8_t* k8; const int8_t* v8; const float* ks; const float* vs;
    const uint16_t* k16; const uint16_t* v16;
};

// emit.rs:549-556 (int8) — and its fp16 counterpart: sequential f32 sum of q[i]*f32(k[i]).
inline float kdot(const KVView& c, const float* q, int64_t t, int64_t off, int hd) {
    float sum = 0.0f;
    if (c.mode == 0) {
        const int8_t* k = c.k8 + off;
        for (int i = 0; i < hd; i++) sum += q[i] * (float)k[i];
        return sum * c.ks[t];
    }
    const uint16_t* k = c.k16 + off;
    for (int i = 0; i < hd; i++) sum += q[i] * f16_to_f32(k[i]);
    return sum;
}
inline float vval(const KVView& c, int64_t t, int64_t idx) {
    if (c.mode == 0) return (float)c.v8[idx] * c.vs[t];
    return f16_to_f32(c.v16[idx]);
}

// emit.rs:558-583
void attention_std(float* out, const float* q, const KVView& c, int64_t seq, int nh, int nkv, int hd) {
    int gsize = nh / nkv;
    float scale = 1.0f / sqrtf((float)hd);
    int64_t stride = (int64_t)nkv * hd;
    std::vector<float> scores((size_t)seq);
    for (int h = 0; h < nh; h++) {
        int kvh = h / gsize;
        const float* qh = q + (int64_t)h * hd;
        for (int64_t t = 0; t < seq; t++) scores[t] = kdot(c, qh, t, t * stride + (int64_t)kvh * hd, hd) * scale;
        softmax(scores.data(), seq);
        for (int d = 0; d < hd; d++) {
            float sum = 0.0f;
            for (int64_t t = 0; t < seq; t++) sum += scores[t] * vval(c, t, t * stride + (int64_t)kvh * hd + d);
            out[(int64_t)h * hd + d] = sum;
        }
    }
}

// emit.rs:656-715
void attention_flash(float* out, const float* q, const KVView& c, int64_t seq, int nh, int nkv, int hd) {
    int gsize = nh / nkv;
    float scale = 1.0f / sqrtf((float)hd);
    int64_t stride = (int64_t)nkv * hd;
    float scores[FLASH_BLOCK];
    std::vector<float> acc(hd);
    for (int h = 0; h < nh; h++) {
        int kvh = h / gsize;
        const float* qh = q + (int64_t)h * hd;
        float m_i = -INFINITY, l_i = 0.0f;
        std::fill(acc.begin(), acc.end(), 0.0f);
        for (int64_t bs = 0; bs < seq;) {
            int64_t be = std::min<int64_t>(bs + FLASH_BLOCK, seq);
            int64_t bl = be - bs;
            float m_block = -INFINITY;
            for (int64_t bi = 0; bi < bl; bi++) {
                int64_t t = bs + bi;
                float s = kdot(c, qh, t, t * stride + (int64_t)kvh * hd, hd) * scale;
                scores[bi] = s;
                if (s > m_block) m_block = s;
            }
            float m_prev = m_i;
            if (m_block > m_i) m_i = m_block;
            float exp_scale = expf(m_prev - m_i);
            l_i *= exp_scale;
            for (int d = 0; d < hd; d++) acc[d] *= exp_scale;
            float l_block = 0.0f;
            for (int64_t bi = 0; bi < bl; bi++) { float e = expf(scores[bi] - m_i); scores[bi] = e; l_block += e; }
            l_i += l_block;
            for (int d = 0; d < hd; d++) {
                float sum = 0.0f;
                for (int64_t bi = 0; bi < bl; bi++) {
                    int64_t t = bs + bi;
                    sum += scores[bi] * vval(c, t, t * stride + (int64_t)kvh * hd + d);
                }
                acc[d] += sum;
            }
            bs = be;
        }
        float inv_l = 1.0f / l_i;
        for (int d = 0; d < hd; d++) out[(int64_t)h * hd + d] = acc[d] * inv_l;
    }
}

// emit.rs:754-883
void attention_flash_batch(float* out, const float* qb, const KVView& c, int64_t m, int64_t base_pos,
                           int nh, int nkv, int hd) {
    constexpr int Q_TILE = 16;
    int gsize = nh / nkv;
    float scale = 1.0f / sqrtf((float)hd);
    int64_t stride = (int64_t)nkv * hd;
    int64_t ostride = (int64_t)nh * hd;
#pragma omp parallel for schedule(dynamic, 1)
    for (int h = 0; h < nh; h++) {
        int kvh = h / gsize;
        int64_t qo = (int64_t)h * hd;
        std::vector<float> acc((size_t)Q_TILE * hd);
        std::vector<float> scores((size_t)Q_TILE * FLASH_BLOCK);
        for (int64_t qs = 0; qs < m;) {
            int64_t ql = std::min<int64_t>(Q_TILE, m - qs);
            int64_t max_q_pos = base_pos + qs + ql - 1;
            float m_state[Q_TILE], l_state[Q_TILE];
            for (int i = 0; i < Q_TILE; i++) { m_state[i] = -INFINITY; l_state[i] = 0.0f; }
            std::fill(acc.begin(), acc.end(), 0.0f);
            for (int64_t bs = 0; bs <= max_q_pos;) {
                int64_t be = std::min<int64_t>(bs + FLASH_BLOCK, max_q_pos + 1);
                int64_t bl = be - bs;
                std::fill(scores.begin(), scores.end(), 0.0f);
                for (int64_t bi = 0; bi < bl; bi++) {
                    int64_t t = bs + bi;
                    for (int64_t qi = 0; qi < ql; qi++) {
                        const float* qrow = qb + (qs + qi) * ostride + qo;
                        scores[qi * FLASH_BLOCK + bi] = kdot(c, qrow, t, t * stride + (int64_t)kvh * hd, hd) * scale;
                    }
                }
                for (int64_t qi = 0; qi < ql; qi++) {
                    int64_t q_pos = base_pos + qs + qi;
                    int64_t ve = q_pos + 1 > bs ? q_pos + 1 - bs : 0;
                    if (ve > bl) ve = bl;
                    float* sc = &scores[qi * FLASH_BLOCK];
                    if (ve == 0) { for (int64_t bi = 0; bi < bl; bi++) sc[bi] = 0.0f; continue; }
                    float m_block = -INFINITY;
                    for (int64_t bi = 0; bi < ve; bi++) if (sc[bi] > m_block) m_block = sc[bi];
                    float m_prev = m_state[qi];
                    float m_new = fmaxf(m_prev, m_block);
                    m_state[qi] = m_new;
                    float exp_scale = expf(m_prev - m_new);
                    l_state[qi] *= exp_scale;
                    for (int d = 0; d < hd; d++) acc[qi * hd + d] *= exp_scale;
                    float l_block = 0.0f;
                    for (int64_t bi = 0; bi < ve; bi++) { float e = expf(sc[bi] - m_new); sc[bi] = e; l_block += e; }
                    for (int64_t bi = ve; bi < bl; bi++) sc[bi] = 0.0f;
                    l_state[qi] += l_block;
                }
                for (int64_t bi = 0; bi < bl; bi++) {
                    int64_t t = bs + bi;
                    int64_t vo = t * stride + (int64_t)kvh * hd;
                    for (int d = 0; d < hd; d++) {
                        float v = vval(c, t, vo + d);
                        for (int64_t qi = 0; qi < ql; qi++) acc[qi * hd + d] += scores[qi * FLASH_BLOCK + bi] * v;
                    }
                }
                bs = be;
            }
            for (int64_t qi = 0; qi < ql; qi++) {
                float inv_l = 1.0f / l_state[qi];
                float* p = out + (qs + qi) * ostride + qo;
                for (int d = 0; d < hd; d++) p[d] = acc[qi * hd + d] * inv_l;
            }
            qs += ql;
        }
    }
}

// emit.rs:598-627 — plain softmax over the last `window` cached rows.
void attention_sliding(float* out, const float* q, const KVView& c, int64_t seq, int64_t window, int nh, int nkv, int hd) {
    int64_t start = seq > window ? seq - window : 0;
    int64_t wl = seq - start;
    int gsize = nh / nkv;
    float scale = 1.0f / sqrtf((float)hd);
    int64_t stride = (int64_t)nkv * hd;
    std::vector<float> scores((size_t)wl);
    for (int h = 0; h < nh; h++) {
        int kvh = h / gsize;
        const float* qh = q + (int64_t)h * hd;
        for (int64_t si = 0; si < wl; si++) {
            int64_t t = start + si;
            scores[si] = kdot(c, qh, t, t * stride + (int64_t)kvh * hd, hd) * scale;
        }
        softmax(scores.data(), wl);
        for (int d = 0; d < hd; d++) {
            float sum = 0.0f;
            for (int64_t si = 0; si < wl; si++) {
                int64_t t = start + si;
                sum += scores[si] * vval(c, t, t * stride + (int64_t)kvh * hd + d);
            }
            out[(int64_t)h * hd + d] = sum;
        }
    }
}

// emit.rs:907-1046 — 16-query tiles, 64-key blocks from the block that holds the tile's first visible key; per query
// the keys [max(0, q_pos - window + 1), q_pos] take part, the others carry weight 0.
void attention_sliding_batch(float* out, const float* qb, const KVView& c, int64_t m, int64_t base_pos, int64_t window,
                             int nh, int nkv, int hd) {
    constexpr int Q_TILE = 16;
    int gsize = nh / nkv;
    float scale = 1.0f / sqrtf((float)hd);
    int64_t stride = (int64_t)nkv * hd;
    int64_t ostride = (int64_t)nh * hd;
#pragma omp parallel for schedule(dynamic, 1)
    for (int h = 0; h < nh; h++) {
        int kvh = h / gsize;
        int64_t qo = (int64_t)h * hd;
        std::vector<float> acc((size_t)Q_TILE * hd);
        std::vector<float> scores((size_t)Q_TILE * FLASH_BLOCK);
        for (int64_t qs = 0; qs < m;) {
            int64_t ql = std::min<int64_t>(Q_TILE, m - qs);
            int64_t first_pos = base_pos + qs, last_pos = base_pos + qs + ql - 1;
            int64_t tile_min_k = first_pos > window - 1 ? first_pos - (window - 1) : 0;
            float m_state[Q_TILE], l_state[Q_TILE];
            for (int i = 0; i < Q_TILE; i++) { m_state[i] = -INFINITY; l_state[i] = 0.0f; }
            std::fill(acc.begin(), acc.end(), 0.0f);
            for (int64_t bs = tile_min_k / FLASH_BLOCK * FLASH_BLOCK; bs <= last_pos;) {
                int64_t be = std::min<int64_t>(bs + FLASH_BLOCK, last_pos + 1);
                int64_t bl = be - bs;
                std::fill(scores.begin(), scores.end(), 0.0f);
                for (int64_t bi = 0; bi < bl; bi++) {
                    int64_t t = bs + bi;
                    for (int64_t qi = 0; qi < ql; qi++) {
                        const float* qrow = qb + (qs + qi) * ostride + qo;
                        scores[qi * FLASH_BLOCK + bi] = kdot(c, qrow, t, t * stride + (int64_t)kvh * hd, hd) * scale;
                    }
                }
                for (int64_t qi = 0; qi < ql; qi++) {
                    int64_t q_pos = base_pos + qs + qi;
                    int64_t win_start = q_pos > window - 1 ? q_pos - (window - 1) : 0;
                    int64_t lo = std::max(win_start, bs) - bs;
                    int64_t hi = q_pos + 1 > bs ? q_pos + 1 - bs : 0;
                    if (hi > bl) hi = bl;
                    float* sc = &scores[qi * FLASH_BLOCK];
                    if (lo >= hi) { for (int64_t bi = 0; bi < bl; bi++) sc[bi] = 0.0f; continue; }
                    float m_block = -INFINITY;
                    for (int64_t bi = lo; bi < hi; bi++) if (sc[bi] > m_block) m_block = sc[bi];
                    float m_prev = m_state[qi];
                    float m_new = fmaxf(m_prev, m_block);
                    m_state[qi] = m_new;
                    float exp_scale = expf(m_prev - m_new);
                    l_state[qi] *= exp_scale;
                    for (int d = 0; d < hd; d++) acc[qi * hd + d] *= exp_scale;
                    float l_block = 0.0f;
                    for (int64_t bi = lo; bi < hi; bi++) { float e = expf(sc[bi] - m_new); sc[bi] = e; l_block += e; }
                    for (int64_t bi = 0; bi < lo; bi++) sc[bi] = 0.0f;
                    for (int64_t bi = hi; bi < bl; bi++) sc[bi] = 0.0f;
                    l_state[qi] += l_block;
                }
                for (int64_t bi = 0; bi < bl; bi++) {
                    int64_t t = bs + bi;
                    int64_t vo = t * stride + (int64_t)kvh * hd;
                    for (int d = 0; d < hd; d++) {
                        float v = vval(c, t, vo + d);
                        for (int64_t qi = 0; qi < ql; qi++) acc[qi * hd + d] += scores[qi * FLASH_BLOCK + bi] * v;
                    }
                }
                bs = be;
            }
            for (int64_t qi = 0; qi < ql; qi++) {
                float inv_l = l_state[qi] > 0.0f ? 1.0f / l_state[qi] : 0.0f;
                float* p = out + (qs + qi) * ostride + qo;
                for (int d = 0; d < hd; d++) p[d] = acc[qi * hd + d] * inv_l;
            }
            qs += ql;
        }
    }
}

// crates/forgellm-codegen-cpu/src/project.rs:501-503 — Iterator::max_by returns the LAST
// maximal element.
uint32_t argmax_last(const float* v, int64_t n) {
    if (n <= 0) return 0;
    int64_t best = 0;
    for (int64_t i = 1; i < n; i++) if (!(v[i] < v[best])) best = i;
    return (uint32_t)best;
}

} // namespace

// ---------------------------------------------------------------------------------------
// Model (emit.rs:3875-4019 Weights/LayerWeights/KVCache; blob layout project.rs:342-407,
// writer order crates/forgellm-cli/src/main.rs:2714-2757).
// ---------------------------------------------------------------------------------------
// ---- K-quant row dots (emit.rs:2978-3310 Q4_K, emit.rs:3508-3615 Q6_K) ---------------------------------------------------
// Both take the SAME Q8_0-quantised activation blocks as the Q8_0/Q4_0 dots (one 32-element block per 32 weights) and
// are one arithmetic on every host: the aarch64 forms (sdot, one row or four rows at a time, emit.rs:3035-3243) compute
// the same integers and combine them with the same f32 operations in the same order as the scalar forms restated here.

// get_scale_min_k4, emit.rs:3013-3021.
static inline void scale_min_k4(int j, const uint8_t* sc, int* scale, int* mn) {
    if (j < 4) { *scale = sc[j] & 63; *mn = sc[j + 4] & 63; }
    else { *scale = (sc[j + 4] & 0x0F) | ((sc[j - 4] >> 6) << 4); *mn = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4); }
}

// dot_q4_k_q8_0, emit.rs:3246-3306: per 256-element super-block (144 bytes: d, dmin, 12 bytes of 6-bit scales and
// minima, 128 bytes of nibbles), four chunks of 32 bytes; a chunk's low nibbles are sub-block 2c, its high nibbles
// sub-block 2c+1;  acc += x_scale * (d*sc * dot - dmin*m * sum)  for the one, then for the other.
float dot_q4_k(const uint8_t* a_q8, const uint8_t* w, int64_t k) {
    const int64_t num_sb = k / 256;
    float acc = 0.0f;
    for (int64_t sb = 0; sb < num_sb; sb++) {
        const uint8_t* blk = w + sb * 144;
        const float d = f16_to_f32(rd16(blk)), dmin = f16_to_f32(rd16(blk + 2));
        const uint8_t* scales = blk + 4;
        const uint8_t* qs = blk + 16;
        for (int chunk = 0; chunk < 4; chunk++) {
            const int is = chunk * 2;
            int sc1, m1, sc2, m2;
            scale_min_k4(is, scales, &sc1, &m1);
            scale_min_k4(is + 1, scales, &sc2, &m2);
            const float d1_w = d * (float)sc1, m1_w = dmin * (float)m1, d2_w = d * (float)sc2, m2_w = dmin * (float)m2;
            const uint8_t* qc = qs + chunk * 32;
            const uint8_t* x1 = a_q8 + (sb * 8 + is) * Q8_BYTES;
            const uint8_t* x2 = a_q8 + (sb * 8 + is + 1) * Q8_BYTES;
            const float x1_scale = f16_to_f32(rd16(x1)), x2_scale = f16_to_f32(rd16(x2));
            int32_t dot1 = 0, sum1 = 0, dot2 = 0, sum2 = 0;
            for (int i = 0; i < 32; i++) {
                const int xi = (int8_t)x1[2 + i];
                dot1 += xi * (qc[i] & 0x0F);
                sum1 += xi;
            }
            acc += x1_scale * (d1_w * (float)dot1 - m1_w * (float)sum1);
            for (int i = 0; i < 32; i++) {
                const int xi = (int8_t)x2[2 + i];
                dot2 += xi * (qc[i] >> 4);
                sum2 += xi;
            }
            acc += x2_scale * (d2_w * (float)dot2 - m2_w * (float)sum2);
        }
    }
    return acc;
}

// dot_q6_k_q8_0, emit.rs:3553-3612: per super-block (210 bytes: 128 of low nibbles, 64 of high bit pairs, 16 int8 scales,
// d) eight activation blocks; block b takes its 32 six-bit values (minus 32) from the table's nibble and bit-pair fields,
// 16 under scale 2b and 16 under scale 2b+1;  acc += d * x_scale * (sc_lo * dot_lo + sc_hi * dot_hi).
float dot_q6_k(const uint8_t* a_q8, const uint8_t* w, int64_t k) {
    static const int T[8][5] = {{0, 0, 0, 0, 0}, {32, 0, 0, 2, 2}, {0, 0, 4, 4, 4}, {32, 0, 4, 6, 6},
                                {64, 32, 0, 0, 8}, {96, 32, 0, 2, 10}, {64, 32, 4, 4, 12}, {96, 32, 4, 6, 14}};
    const int64_t num_sb = k / 256;
    float acc = 0.0f;
    for (int64_t sb = 0; sb < num_sb; sb++) {
        const uint8_t* blk = w + sb * 210;
        const uint8_t* ql = blk;
        const uint8_t* qh = blk + 128;
        const int8_t* scales = reinterpret_cast<const int8_t*>(blk + 192);
        const float d = f16_to_f32(rd16(blk + 208));
        for (int b = 0; b < 8; b++) {
            const uint8_t* x = a_q8 + (sb * 8 + b) * Q8_BYTES;
            const float x_scale = f16_to_f32(rd16(x));
            const int sc_lo = scales[T[b][4]], sc_hi = scales[T[b][4] + 1];
            int32_t dot_lo = 0, dot_hi = 0;
            for (int l = 0; l < 32; l++) {
                const int q6 = (((ql[T[b][0] + l] >> T[b][2]) & 0x0F) | (((qh[T[b][1] + l] >> T[b][3]) & 0x03) << 4)) - 32;
                const int xi = (int8_t)x[2 + l];
                if (l < 16) dot_lo += q6 * xi; else dot_hi += q6 * xi;
            }
            acc += d * x_scale * ((float)sc_lo * (float)dot_lo + (float)sc_hi * (float)dot_hi);
        }
    }
    return acc;
}

// matmul_vec_q4_k_KxN / matmul_vec_q6_k_KxN (emit.rs:3388-3490, 3622-3655): quantise the input once, one dot per row.
void matmul_vec_kquant(int ggml_type, float* out, const float* in, const uint8_t* w, int64_t k, int64_t n) {
    std::vector<uint8_t> a_q8((size_t)(k / QK * Q8_BYTES));
    quantize_act_q8_0(in, k, a_q8.data());
    const int64_t row_bytes = k / 256 * (ggml_type == 12 ? 144 : 210);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; r++)
        out[r] = ggml_type == 12 ? dot_q4_k(a_q8.data(), w + r * row_bytes, k) : dot_q6_k(a_q8.data(), w + r * row_bytes, k);
}

extern "C" {
float fo_dot_kquant(int ggml_type, const uint8_t* a_q8, const uint8_t* w, int64_t k) {
    return ggml_type == 12 ? dot_q4_k(a_q8, w, k) : dot_q6_k(a_q8, w, k);
}
void fo_matmul_vec_kquant(int ggml_type, float* out, const float* in, const uint8_t* w, int64_t k, int64_t n) {
    matmul_vec_kquant(ggml_type, out, in, w, k, n);
}

struct fo_config {
    uint32_t hidden, inter, layers, heads, kv_heads, head_dim, vocab, max_seq;
    float rms_eps, rope_theta;
    uint32_t wdtype;        // 8 = Q8_0, 2 = Q4_0 (GGML type ids)
    uint32_t lm_head_dtype; // same coding
    uint32_t flags;         // bit 1 (value 2): the blob carries QKV bias vectors (Qwen2, emit.rs:3906-3915)
    uint32_t sliding_window; // ModelConfig::sliding_window_size, 0 = None (emit.rs:97-99, 4156-4170, 5312-5340)
};

struct fo_layer {
    const float* attn_norm; const uint8_t *q, *k, *v, *o; const float* ffn_norm; const uint8_t *gate, *up, *down;
    const float *q_bias = nullptr, *k_bias = nullptr, *v_bias = nullptr;      // project.rs:286-292: after the v weights
};

struct fo_model {
    fo_config cfg;
    int variant, kvmode;
    // storage format of q, k, v, o, gate, up, down (ProjectionDTypes, ir.rs:410-421): 8 = Q8_0, 2 = Q4_0, 12 = Q4_K, 14 = Q6_K
    // (GGML ids); `mixed`: not all equal to cfg.wdtype, or the lm_head a K-quant
    uint32_t pd[7];
    bool mixed = false;
    std::vector<uint8_t> blob;
    const float* embed; std::vector<fo_layer> layers; const float* final_norm; const uint8_t* lm_head;
    std::vector<std::vector<int8_t>> k8, v8; std::vector<std::vector<float>> ks, vs;
    std::vector<std::vector<uint16_t>> k16, v16;
    std::vector<float> freqs;
    int64_t len;
};

// bytes of an [n][k] matrix in a storage format (project.rs:195-213: 34 / 18 bytes per 32, 144 / 210 bytes per 256 elements)
static int64_t wsize(uint32_t dtype, int64_t n, int64_t k) {
    if (dtype == 12 || dtype == 14) return n * ((k + 255) / 256) * (dtype == 12 ? 144 : 210);
    return n * ((k + QK - 1) / QK) * (dtype == 8 ? Q8_BYTES : Q4_BYTES);
}
static bool is_kquant(uint32_t d) { return d == 12 || d == 14; }
// One projection in its own storage format (matmul_call, emit.rs:3316-3334).  The K-quant kernels quantise their input to
// Q8_0 blocks on every target architecture (emit.rs:3388-3490, 3622-3655), so `variant` does not reach them.
static void matmul_vec_any(uint32_t dtype, int variant, float* out, const float* in, const uint8_t* w, int64_t k, int64_t n, int lm_mode) {
    if (is_kquant(dtype)) matmul_vec_kquant((int)dtype, out, in, w, k, n);
    else matmul_vec((int)dtype, variant, out, in, w, k, n, lm_mode);
}

uint64_t fo_weights_nbytes(const fo_config* c) {
    int64_t H = c->hidden, I = c->inter, QKS = (int64_t)c->heads * c->head_dim, KV = (int64_t)c->kv_heads * c->head_dim;
    int64_t per_layer = H * 4 + wsize(c->wdtype, QKS, H) + 2 * wsize(c->wdtype, KV, H) + wsize(c->wdtype, H, QKS) + H * 4 +
                        2 * wsize(c->wdtype, I, H) + wsize(c->wdtype, H, I) + ((c->flags & 2u) ? (QKS + 2 * KV) * 4 : 0);
    return (uint64_t)((int64_t)c->vocab * H * 4 + c->layers * per_layer + H * 4 + wsize(c->lm_head_dtype, c->vocab, H));
}

// The same with a storage format per projection: pd = {q, k, v, o, gate, up, down}; the lm_head's is c->lm_head_dtype.
uint64_t fo_weights_nbytes_mixed(const fo_config* c, const uint32_t* pd) {
    int64_t H = c->hidden, I = c->inter, QKS = (int64_t)c->heads * c->head_dim, KV = (int64_t)c->kv_heads * c->head_dim;
    int64_t per_layer = H * 4 + wsize(pd[0], QKS, H) + wsize(pd[1], KV, H) + wsize(pd[2], KV, H) + wsize(pd[3], H, QKS) + H * 4 +
                        wsize(pd[4], I, H) + wsize(pd[5], I, H) + wsize(pd[6], H, I) + ((c->flags & 2u) ? (QKS + 2 * KV) * 4 : 0);
    return (uint64_t)((int64_t)c->vocab * H * 4 + c->layers * per_layer + H * 4 + wsize(c->lm_head_dtype, c->vocab, H));
}

fo_model* fo_model_create_mixed(const fo_config* c, const uint32_t* pd, const uint8_t* blob, uint64_t nbytes, int variant, int kvmode);
fo_model* fo_model_create(const fo_config* c, const uint8_t* blob, uint64_t nbytes, int variant, int kvmode) {
    const uint32_t pd[7] = {c->wdtype, c->wdtype, c->wdtype, c->wdtype, c->wdtype, c->wdtype, c->wdtype};
    return fo_model_create_mixed(c, pd, blob, nbytes, variant, kvmode);
}

fo_model* fo_model_create_mixed(const fo_config* c, const uint32_t* pd, const uint8_t* blob, uint64_t nbytes, int variant, int kvmode) {
    if (nbytes != fo_weights_nbytes_mixed(c, pd)) return nullptr;
    fo_model* m = new fo_model();
    m->cfg = *c; m->variant = variant; m->kvmode = kvmode; m->len = 0;
    for (int i = 0; i < 7; i++) { m->pd[i] = pd[i]; m->mixed = m->mixed || pd[i] != c->wdtype; }
    m->mixed = m->mixed || is_kquant(c->lm_head_dtype);
    m->blob.assign(blob, blob + nbytes);
    const uint8_t* p = m->blob.data();
    int64_t H = c->hidden, I = c->inter, QKS = (int64_t)c->heads * c->head_dim, KV = (int64_t)c->kv_heads * c->head_dim;
    m->embed = (const float*)p; p += (int64_t)c->vocab * H * 4;
    for (uint32_t l = 0; l < c->layers; l++) {
        fo_layer L;
        L.attn_norm = (const float*)p; p += H * 4;
        L.q = p; p += wsize(pd[0], QKS, H);
        L.k = p; p += wsize(pd[1], KV, H);
        L.v = p; p += wsize(pd[2], KV, H);
        if (c->flags & 2u) {
            L.q_bias = (const float*)p; p += QKS * 4;
            L.k_bias = (const float*)p; p += KV * 4;
            L.v_bias = (const float*)p; p += KV * 4;
        }
        L.o = p; p += wsize(pd[3], H, QKS);
        L.ffn_norm = (const float*)p; p += H * 4;
        L.gate = p; p += wsize(pd[4], I, H);
        L.up = p; p += wsize(pd[5], I, H);
        L.down = p; p += wsize(pd[6], H, I);
        m->layers.push_back(L);
    }
    m->final_norm = (const float*)p; p += H * 4;
    m->lm_head = p;
    size_t cache_elems = (size_t)c->max_seq * KV;
    if (kvmode == 0) {
        m->k8.assign(c->layers, std::vector<int8_t>(cache_elems)); m->v8 = m->k8;
        m->ks.assign(c->layers, std::vector<float>(c->max_seq)); m->vs = m->ks;
    } else {
        m->k16.assign(c->layers, std::vector<uint16_t>(cache_elems)); m->v16 = m->k16;
    }
    m->freqs.resize(c->head_dim / 2);
    rope_freqs(m->freqs.data(), c->head_dim, c->rope_theta);
    return m;
}
void fo_model_destroy(fo_model* m) { delete m; }
void fo_model_reset(fo_model* m) { m->len = 0; }
int64_t fo_model_pos(fo_model* m) { return m->len; }

static KVView kv_view(fo_model* m, int l) {
    KVView c{};
    c.mode = m->kvmode;
    if (m->kvmode == 0) { c.k8 = m->k8[l].data(); c.v8 = m->v8[l].data(); c.ks = m->ks[l].data(); c.vs = m->vs[l].data(); }
    else { c.k16 = m->k16[l].data(); c.v16 = m->v16[l].data(); }
    return c;
}

static void store_kv(fo_model* m, int l, int64_t pos, const float* k, const float* v) {
    int64_t KV = (int64_t)m->cfg.kv_heads * m->cfg.head_dim;
    if (m->kvmode == 0) {
        m->ks[l][pos] = quantize_kv(k, KV, m->k8[l].data() + pos * KV);
        m->vs[l][pos] = quantize_kv(v, KV, m->v8[l].data() + pos * KV);
    } else {
        for (int64_t i = 0; i < KV; i++) { m->k16[l][pos * KV + i] = f32_to_f16(k[i]); m->v16[l][pos * KV + i] = f32_to_f16(v[i]); }
    }
}

// model::forward (emit.rs:4029-4500) and one token of the per-token forward_prefill (emit.rs:4553-5048; logits == NULL: not
// the prompt's last token, the lm_head is skipped).
// prompt_walk: the token belongs to a prompt that forward_prefill walks one token at a time (models with a format per
// projection).  The walk's attention is `attention_flash` when use_flash_attention(config) and plain `attention` otherwise
// (emit.rs:4717-4720) -- it never calls attention_sliding, so a model with a window (for which use_flash_attention is false,
// emit.rs:126-128) lets every prompt row see ALL earlier positions; only decode steps apply the window (emit.rs:4156-4170).
static int forward_impl(fo_model* m, uint32_t token, float* logits, bool prompt_walk) {
    const fo_config& c = m->cfg;
    int64_t H = c.hidden, I = c.inter, QKS = (int64_t)c.heads * c.head_dim, KV = (int64_t)c.kv_heads * c.head_dim;
    int64_t pos = m->len;
    if (pos >= c.max_seq || token >= c.vocab) return -3;
    std::vector<float> hs(m->embed + (int64_t)token * H, m->embed + (int64_t)(token + 1) * H);
    std::vector<float> normed(H), q(QKS), k(KV), v(KV), attn(QKS), proj(H), gate(I), up(I), ffn(I), ffo(H);
    bool flash = c.max_seq > 512; // emit.rs:126-128
    for (uint32_t l = 0; l < c.layers; l++) {
        const fo_layer& L = m->layers[l];
        rms_norm(normed.data(), hs.data(), L.attn_norm, H, c.rms_eps, m->variant);
        matmul_vec_any(m->pd[0], m->variant, q.data(), normed.data(), L.q, H, QKS, 0);
        matmul_vec_any(m->pd[1], m->variant, k.data(), normed.data(), L.k, H, KV, 0);
        matmul_vec_any(m->pd[2], m->variant, v.data(), normed.data(), L.v, H, KV, 0);
        if (L.q_bias) {                                       // emit.rs:4105-4120
            for (int64_t i = 0; i < QKS; i++) q[i] += L.q_bias[i];
            for (int64_t i = 0; i < KV; i++) k[i] += L.k_bias[i];
            for (int64_t i = 0; i < KV; i++) v[i] += L.v_bias[i];
        }
        rope(q.data(), pos, c.head_dim, c.heads, m->freqs.data());
        rope(k.data(), pos, c.head_dim, c.kv_heads, m->freqs.data());
        store_kv(m, l, pos, k.data(), v.data());
        KVView cv = kv_view(m, l);
        if (c.sliding_window && !prompt_walk) attention_sliding(attn.data(), q.data(), cv, pos + 1, c.sliding_window, c.heads, c.kv_heads, c.head_dim);
        else if (flash && !c.sliding_window) attention_flash(attn.data(), q.data(), cv, pos + 1, c.heads, c.kv_heads, c.head_dim);
        else attention_std(attn.data(), q.data(), cv, pos + 1, c.heads, c.kv_heads, c.head_dim);
        matmul_vec_any(m->pd[3], m->variant, proj.data(), attn.data(), L.o, QKS, H, 0);
        for (int64_t i = 0; i < H; i++) hs[i] += proj[i];
        rms_norm(normed.data(), hs.data(), L.ffn_norm, H, c.rms_eps, m->variant);
        matmul_vec_any(m->pd[4], m->variant, gate.data(), normed.data(), L.gate, H, I, 0);
        matmul_vec_any(m->pd[5], m->variant, up.data(), normed.data(), L.up, H, I, 0);
        silu_mul(ffn.data(), gate.data(), up.data(), I);
        matmul_vec_any(m->pd[6], m->variant, ffo.data(), ffn.data(), L.down, I, H, 0);
        for (int64_t i = 0; i < H; i++) hs[i] += ffo[i];
    }
    if (logits) {
        rms_norm(normed.data(), hs.data(), m->final_norm, H, c.rms_eps, m->variant);
        matmul_vec_any(c.lm_head_dtype, m->variant, logits, normed.data(), m->lm_head, H, c.vocab, 1);
    }
    m->len += 1;
    return 0;
}

// emit.rs:4029-4500.  Returns 0, or -3 when the cache is full.
// logits == NULL: the lm_head is skipped.
int fo_forward(fo_model* m, uint32_t token, float* logits) { return forward_impl(m, token, logits, false); }

// emit.rs:5118-5486.  logits may be NULL (then the lm_head is skipped).
int fo_prefill_batched(fo_model* m, const uint32_t* tokens, int64_t n, float* logits) {
    const fo_config& c = m->cfg;
    int64_t H = c.hidden, I = c.inter, QKS = (int64_t)c.heads * c.head_dim, KV = (int64_t)c.kv_heads * c.head_dim;
    int64_t base = m->len;
    if (n <= 0 || base + n > c.max_seq) return -3;
    for (int64_t r = 0; r < n; r++) if (tokens[r] >= c.vocab) return -3;
    if (m->mixed) {
        // forward_prefill hands the prompt to the batched function only when every projection is Q8_0 or every one Q4_0
        // (emit.rs:4530-4534); otherwise it walks the tokens one at a time with forward's own operations and runs the
        // lm_head once, after the last (emit.rs:4621-5040: chunks of 256 rows, dot8 / dot4 groups and a dot1 tail like
        // forward's)
        for (int64_t r = 0; r < n; r++) {
            const int rc = forward_impl(m, tokens[r], r == n - 1 ? logits : nullptr, true);
            if (rc) return rc;
        }
        return 0;
    }
    std::vector<float> hs((size_t)n * H), normed((size_t)n * H), q((size_t)n * QKS), k((size_t)n * KV), v((size_t)n * KV),
        attn((size_t)n * QKS), proj((size_t)n * H), gate((size_t)n * I), up((size_t)n * I), ffn((size_t)n * I), ffo((size_t)n * H);
    for (int64_t r = 0; r < n; r++) std::memcpy(&hs[r * H], m->embed + (int64_t)tokens[r] * H, H * 4);
    bool flash = c.max_seq > 512;
    for (uint32_t l = 0; l < c.layers; l++) {
        const fo_layer& L = m->layers[l];
        for (int64_t r = 0; r < n; r++) rms_norm(&normed[r * H], &hs[r * H], L.attn_norm, H, c.rms_eps, m->variant);
        matmul_mat(c.wdtype, m->variant, q.data(), n, normed.data(), L.q, H, QKS);
        matmul_mat(c.wdtype, m->variant, k.data(), n, normed.data(), L.k, H, KV);
        matmul_mat(c.wdtype, m->variant, v.data(), n, normed.data(), L.v, H, KV);
        for (int64_t r = 0; r < n; r++) {
            if (L.q_bias) {                                   // emit.rs:5246-5260
                for (int64_t i = 0; i < QKS; i++) q[r * QKS + i] += L.q_bias[i];
                for (int64_t i = 0; i < KV; i++) k[r * KV + i] += L.k_bias[i];
                for (int64_t i = 0; i < KV; i++) v[r * KV + i] += L.v_bias[i];
            }
            rope(&q[r * QKS], base + r, c.head_dim, c.heads, m->freqs.data());
            rope(&k[r * KV], base + r, c.head_dim, c.kv_heads, m->freqs.data());
            store_kv(m, l, base + r, &k[r * KV], &v[r * KV]);
        }
        KVView cv = kv_view(m, l);
        if (c.sliding_window) attention_sliding_batch(attn.data(), q.data(), cv, n, base, c.sliding_window, c.heads, c.kv_heads, c.head_dim);
        else if (flash) attention_flash_batch(attn.data(), q.data(), cv, n, base, c.heads, c.kv_heads, c.head_dim);
        else for (int64_t r = 0; r < n; r++)
            attention_std(&attn[r * QKS], &q[r * QKS], cv, base + r + 1, c.heads, c.kv_heads, c.head_dim);
        matmul_mat(c.wdtype, m->variant, proj.data(), n, attn.data(), L.o, QKS, H);
        for (int64_t i = 0; i < n * H; i++) hs[i] += proj[i];
        for (int64_t r = 0; r < n; r++) rms_norm(&normed[r * H], &hs[r * H], L.ffn_norm, H, c.rms_eps, m->variant);
        matmul_mat(c.wdtype, m->variant, gate.data(), n, normed.data(), L.gate, H, I);
        matmul_mat(c.wdtype, m->variant, up.data(), n, normed.data(), L.up, H, I);
        for (int64_t r = 0; r < n; r++) silu_mul(&ffn[r * I], &gate[r * I], &up[r * I], I);
        matmul_mat(c.wdtype, m->variant, ffo.data(), n, ffn.data(), L.down, I, H);
        for (int64_t i = 0; i < n * H; i++) hs[i] += ffo[i];
    }
    if (logits) {
        std::vector<float> nrm(H);
        rms_norm(nrm.data(), &hs[(n - 1) * H], m->final_norm, H, c.rms_eps, m->variant);
        matmul_vec(c.lm_head_dtype, m->variant, logits, nrm.data(), m->lm_head, H, c.vocab, 2);
    }
    m->len += n;
    return 0;
}

// Copy one layer's cached K or V rows [0, len) out as f32 (dequantised), for tests.
void fo_model_read_kv(fo_model* m, int layer, int which, float* out) {
    int64_t KV = (int64_t)m->cfg.kv_heads * m->cfg.head_dim;
    for (int64_t t = 0; t < m->len; t++)
        for (int64_t i = 0; i < KV; i++) {
            int64_t idx = t * KV + i;
            if (m->kvmode == 0) out[idx] = which == 0 ? (float)m->k8[layer][idx] * m->ks[layer][t] : (float)m->v8[layer][idx] * m->vs[layer][t];
            else out[idx] = f16_to_f32(which == 0 ? m->k16[layer][idx] : m->v16[layer][idx]);
        }
}

// The inverse of fo_model_read_kv: rows [0, n) of one layer's K and V cache are stored from f32 rows through the model's own
// cache write (int8 + per-token scale, or fp16), and the cache length is set to n.  Lets a model take over the context
// another one has computed (a timing aid: a decode step at a long context without this model's own prefill of it).
int fo_model_write_kv(fo_model* m, int layer, int64_t n, const float* k, const float* v) {
    int64_t KV = (int64_t)m->cfg.kv_heads * m->cfg.head_dim;
    if (layer < 0 || layer >= (int)m->cfg.layers || n < 0 || n > (int64_t)m->cfg.max_seq) return -3;
    for (int64_t t = 0; t < n; t++) store_kv(m, layer, t, k + t * KV, v + t * KV);
    m->len = n;
    return 0;
}

// ---- op-level entry points ----
float fo_f16_to_f32(uint16_t b) { return f16_to_f32(b); }
uint16_t fo_f32_to_f16(float x) { return f32_to_f16(x); }
void fo_f32_to_f16_array(const float* x, int64_t n, uint16_t* out) { for (int64_t i = 0; i < n; i++) out[i] = f32_to_f16(x[i]); }
void fo_f16_to_f32_array(const uint16_t* x, int64_t n, float* out) { for (int64_t i = 0; i < n; i++) out[i] = f16_to_f32(x[i]); }
void fo_dequant(int wdtype, const uint8_t* d, int64_t n, float* out) { wdtype == 8 ? dequant_q8_0(d, n, out) : dequant_q4_0(d, n, out); }
void fo_quantize_weights(int wdtype, const float* d, int64_t n, uint8_t* out) { wdtype == 8 ? quantize_f32_to_q8_0(d, n, out) : quantize_f32_to_q4_0(d, n, out); }
void fo_quantize_act(const float* in, int64_t k, uint8_t* out) { quantize_act_q8_0(in, k, out); }
// int32 block sums of one quantised activation row against n weight rows: out[n][k/32].
void fo_block_isums(int wdtype, const uint8_t* a_q8, const uint8_t* w, int64_t k, int64_t n, int32_t* out) {
    int64_t nb = k / QK, rb = nb * wbytes(wdtype);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; r++)
        for (int64_t b = 0; b < nb; b++) out[r * nb + b] = block_isum(wdtype, a_q8 + b * Q8_BYTES, w + r * rb + b * wbytes(wdtype));
}
float fo_dot_a(int wdtype, const uint8_t* a_q8, const uint8_t* w, int64_t k, int seq) { return dot_a(wdtype, a_q8, w, k, seq != 0); }
float fo_dot_b(int wdtype, const float* x, const uint8_t* w, int64_t k) { return dot_b(wdtype, x, w, k); }
void fo_matmul_vec(int wdtype, int variant, float* out, const float* in, const uint8_t* w, int64_t k, int64_t n) { matmul_vec(wdtype, variant, out, in, w, k, n, 0); }
void fo_matmul_mat(int wdtype, int variant, float* out, int64_t m, const float* in, const uint8_t* w, int64_t k, int64_t n) { matmul_mat(wdtype, variant, out, m, in, w, k, n); }
void fo_rms_norm(float* out, const float* in, const float* w, int64_t n, float eps, int variant) { rms_norm(out, in, w, n, eps, variant); }
void fo_silu_mul(float* out, const float* g, const float* u, int64_t n) { silu_mul(out, g, u, n); }
void fo_softmax(float* v, int64_t n) { softmax(v, n); }
void fo_rope(float* data, int64_t pos, int head_dim, int num_heads, float theta) {
    std::vector<float> f(head_dim / 2);
    rope_freqs(f.data(), head_dim, theta);
    rope(data, pos, head_dim, num_heads, f.data());
}
// cos/sin table exactly as rope() derives it: [n_pos][head_dim/2] each.
void fo_rope_table(int64_t n_pos, int head_dim, float theta, float* cos_out, float* sin_out) {
    std::vector<float> f(head_dim / 2);
    rope_freqs(f.data(), head_dim, theta);
    for (int64_t p = 0; p < n_pos; p++)
        for (int i = 0; i < head_dim / 2; i++) {
            float a = (float)p * f[i];
            sin_out[p * (head_dim / 2) + i] = sinf(a);
            cos_out[p * (head_dim / 2) + i] = cosf(a);
        }
}
float fo_quantize_kv(const float* v, int64_t n, int8_t* out) { return quantize_kv(v, n, out); }
uint32_t fo_argmax(const float* v, int64_t n) { return argmax_last(v, n); }
// Which output rows add their block products in the 4-accumulator (dot1) order: out[r] = 1 for those rows.
// mode: 0 matmul_vec, 1 lm_head of forward, 2 lm_head of forward_prefill_batched, 3 matmul_mat.  wdtype does not enter
// the rule (both formats compare 34-byte blocks with the threshold); it is an argument so that callers state the format.
void fo_row_order(int wdtype, int64_t k, int64_t n, int mode, uint8_t* out) {
    (void)wdtype;
    for (int64_t r = 0; r < n; r++) {
        if (mode == 3) out[r] = row_is_dot1(r, n, 0, 4);
        else out[r] = row_is_dot1(r, n, matmul_vec_is_chunked(k, n, mode) ? 256 : 0, mode == 2 ? 8 : 4);
    }
}
// The C library's expf (what Rust's f32::exp calls on Linux), element-wise.
void fo_expf_array(const float* x, int64_t n, float* out) { for (int64_t i = 0; i < n; i++) out[i] = expf(x[i]); }

// Attention over an externally supplied cache.  kvmode 0: k,v are int8 with ks/vs scales;
// kvmode 1: k,v are fp16 bit patterns.  kind 0 standard, 1 flash, 2 flash_batch (then q is
// [m][nh*hd], out likewise, and the cache holds base_pos+m rows), 3 sliding, 4 sliding_batch (both with `window`).
void fo_attention(int kind, int kvmode, float* out, const float* q, const void* k, const void* v, const float* ks,
                  const float* vs, int64_t seq_or_m, int64_t base_pos, int nh, int nkv, int hd, int64_t window) {
    KVView c{};
    c.mode = kvmode;
    if (kvmode == 0) { c.k8 = (const int8_t*)k; c.v8 = (const int8_t*)v; c.ks = ks; c.vs = vs; }
    else { c.k16 = (const uint16_t*)k; c.v16 = (const uint16_t*)v; }
    if (kind == 0) attention_std(out, q, c, seq_or_m, nh, nkv, hd);
    else if (kind == 1) attention_flash(out, q, c, seq_or_m, nh, nkv, hd);
    else if (kind == 2) attention_flash_batch(out, q, c, seq_or_m, base_pos, nh, nkv, hd);
    else if (kind == 3) attention_sliding(out, q, c, seq_or_m, window, nh, nkv, hd);
    else attention_sliding_batch(out, q, c, seq_or_m, base_pos, window, nh, nkv, hd);
}

int fo_num_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void fo_set_num_threads(int n) {
#if defined(_OPENMP)
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

} // extern "C"

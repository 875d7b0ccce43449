// The order in which the reference's decode GEMV adds a row's per-block products, shared by the
// GEMV kernels: which rows take the four-accumulator (dot1) order and the ordered sum itself.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "forge_hip.h"

namespace fh {

// One reference matmul inside a (possibly fused) matrix: rows [start, start+len), processed by the
// reference in chunks of `chunk` rows (0 = unchunked).
struct Segment { uint32_t start, len, chunk; };

// matmul_vec chunks rows by 256 once the matrix reaches 1 MB of GGUF bytes (emit.rs:1937,1971); the
// lm_head GEMV always chunks (emit.rs:5455-5470).
inline Segment make_segment(uint32_t wdtype, uint32_t K, uint32_t start, uint32_t len, bool always_chunk) {
    const size_t raw_bytes = (size_t)len * (K / 32) * (wdtype == FORGE_HIP_Q8_0 ? 34 : 18);
    Segment sg;
    sg.start = start; sg.len = len;
    sg.chunk = (always_chunk || raw_bytes >= 1000000) ? 256 : 0;
    return sg;
}

// Rows of a chunk are taken 8 (then 4) at a time by dot8/dot4; the last len % tail_mod rows of each chunk go
// through dot1, whose block products are added by four interleaved accumulators (emit.rs:1558-1571).
__device__ __forceinline__ bool segment_row_is_dot1(uint32_t row, const Segment* seg, uint32_t nseg, uint32_t tail_mod) {
    for (uint32_t s = 0; s < nseg; s++) {
        const Segment sg = seg[s];
        if (row >= sg.start && row < sg.start + sg.len) {
            const uint32_t i = row - sg.start;
            const uint32_t base = sg.chunk ? (i / sg.chunk) * sg.chunk : 0;
            const uint32_t len = sg.chunk ? min(sg.chunk, sg.len - base) : sg.len;
            return (i - base) >= len - (len % tail_mod);
        }
    }
    return false;
}

// Distance in floats between two rows of block products in LDS: rows start on 16-byte boundaries (the sum below
// reads four products per instruction) and the distance is an odd number of 16-byte units, so that lanes that
// walk neighbouring rows at the same time spread over the banks.
__host__ __device__ inline uint32_t prod_stride(uint32_t nblk) {
    uint32_t s = ((nblk + 3u) & ~3u) + 4u;
    if (((s >> 2) & 1u) == 0) s += 4u;
    return s;
}

// Ordered sum of one row's block products p[0..nblk), p 16-byte aligned: sequential (dot8/dot4,
// emit.rs:1770-1877), or the dot1 order.  Adds are never fused with the multiplies that made the products.
// The adds of the sequential order form one dependent chain, and the lane that walks it is usually alone on its
// SIMD: what the chain costs is its instruction count.  Products are read four at a time, 64 per step, all reads
// of a step issued before its first add.
__device__ __forceinline__ float ordered_sum(const float* p, uint32_t nblk, bool dot1) {
    const float4* p4 = reinterpret_cast<const float4*>(p);
    const uint32_t n4 = nblk / 4;
    uint32_t g = 0;
    if (!dot1) {
        float r = 0.f;
        for (; g + 16 <= n4; g += 16) {
            float4 v[16];
#pragma unroll
            for (int i = 0; i < 16; i++) v[i] = p4[g + i];
#pragma unroll
            for (int i = 0; i < 16; i++) { r = r + v[i].x; r = r + v[i].y; r = r + v[i].z; r = r + v[i].w; }
        }
        for (; g + 4 <= n4; g += 4) {
            float4 v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = p4[g + i];
#pragma unroll
            for (int i = 0; i < 4; i++) { r = r + v[i].x; r = r + v[i].y; r = r + v[i].z; r = r + v[i].w; }
        }
        for (; g < n4; g++) { const float4 v = p4[g]; r = r + v.x; r = r + v.y; r = r + v.z; r = r + v.w; }
        for (uint32_t b = n4 * 4; b < nblk; b++) r = r + p[b];
        return r;
    }
    float fa0 = 0.f, fa1 = 0.f, fa2 = 0.f, fa3 = 0.f;
    for (; g + 8 <= n4; g += 8) {
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = p4[g + i];
#pragma unroll
        for (int i = 0; i < 8; i++) { fa0 = fa0 + v[i].x; fa1 = fa1 + v[i].y; fa2 = fa2 + v[i].z; fa3 = fa3 + v[i].w; }
    }
    for (; g < n4; g++) { const float4 v = p4[g]; fa0 = fa0 + v.x; fa1 = fa1 + v.y; fa2 = fa2 + v.z; fa3 = fa3 + v.w; }
    const uint32_t tail = n4 * 4;
    if (tail < nblk) fa0 = fa0 + p[tail];
    if (tail + 1 < nblk) fa1 = fa1 + p[tail + 1];
    if (tail + 2 < nblk) fa2 = fa2 + p[tail + 2];
    return ((fa0 + fa1) + fa2) + fa3;
}

// The same sum for rows of products at any 4-byte distance (the resident decode kernel's ordered variant, whose
// tiling is tied to rows of nblk + 1 words), one product per read: p[0..nblk): sequential (dot8/dot4, emit.rs:1770-1877), or the
// dot1 order.  Adds are never fused with the multiplies that made the products.
__device__ __forceinline__ float ordered_sum_words(const float* p, uint32_t nblk, bool dot1) {
    if (!dot1) {
        // the adds form one dependent chain; two register sets alternate so that the reads of the next eight products
        // are in flight while the current eight are added
        float r = 0.f;
        uint32_t b = 0;
        if (nblk >= 8) {
            float v[8], w[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = p[i];
            b = 8;                                   // v holds products [b - 8, b)
            while (b + 16 <= nblk) {
#pragma unroll
                for (int i = 0; i < 8; i++) w[i] = p[b + i];
#pragma unroll
                for (int i = 0; i < 8; i++) r = r + v[i];
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = p[b + 8 + i];
#pragma unroll
                for (int i = 0; i < 8; i++) r = r + w[i];
                b += 16;
            }
            if (b + 8 <= nblk) {
#pragma unroll
                for (int i = 0; i < 8; i++) w[i] = p[b + i];
#pragma unroll
                for (int i = 0; i < 8; i++) r = r + v[i];
#pragma unroll
                for (int i = 0; i < 8; i++) r = r + w[i];
                b += 8;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) r = r + v[i];
            }
        }
        for (; b < nblk; b++) r = r + p[b];
        return r;
    }
    float fa0 = 0.f, fa1 = 0.f, fa2 = 0.f, fa3 = 0.f;
    const uint32_t groups = nblk / 4;
    for (uint32_t g = 0; g < groups; g++) {
        fa0 = fa0 + p[4 * g]; fa1 = fa1 + p[4 * g + 1]; fa2 = fa2 + p[4 * g + 2]; fa3 = fa3 + p[4 * g + 3];
    }
    const uint32_t tail = groups * 4;
    if (tail < nblk) fa0 = fa0 + p[tail];
    if (tail + 1 < nblk) fa1 = fa1 + p[tail + 1];
    if (tail + 2 < nblk) fa2 = fa2 + p[tail + 2];
    return ((fa0 + fa1) + fa2) + fa3;
}

}  // namespace fh

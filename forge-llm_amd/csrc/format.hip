// Host-side format code: fp16 bit conversions, the GGUF Q8_0/Q4_0 (de)quantisers and the
// split of raw GGUF rows into the device planes.  No GPU involved.
#include <math.h>
#include <string.h>

#include <algorithm>
#include <thread>
#include <vector>

#include "common.h"

namespace fh {

namespace {
thread_local std::string g_error;
inline float bits_to_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
inline uint32_t f32_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
}  // namespace

void set_error(const std::string& msg) { g_error = msg; }
int32_t fail(int32_t code, const std::string& msg) { g_error = msg; return code; }
const char* last_error_cstr() { return g_error.c_str(); }

LaunchProbe*& launch_probe() {
    static thread_local LaunchProbe* probe = nullptr;
    return probe;
}

// f16_bits_to_f32, emit.rs:1245-1264
float f16_to_f32_host(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return bits_to_f32(sign);
        int shift = 0;
        while (!(m & 0x400u)) { m <<= 1; shift++; }
        return bits_to_f32(sign | ((uint32_t)(113 - shift) << 23) | ((m & 0x3FFu) << 13));
    }
    if (e == 31) return bits_to_f32(sign | 0x7F800000u | (m << 13));
    return bits_to_f32(sign | ((e + 112) << 23) | (m << 13));
}

// f32_to_f16_bits, emit.rs:1460-1495: nearest-even, but anything below 2^-24 in magnitude
// (f32 subnormals included) becomes signed zero.
uint16_t f32_to_f16_host(float x) {
    const uint32_t b = f32_to_bits(x);
    const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    const int e = (int)((b >> 23) & 0xFFu);
    const uint32_t man = b & 0x7FFFFFu;
    if (e == 0xFF) {
        uint16_t hm = (uint16_t)(man >> 13);
        if (man && !hm) hm = 1;
        return (uint16_t)(sign | 0x7C00u | hm);
    }
    const int ue = e - 127;
    if (e == 0 || ue < -24) return sign;
    if (ue > 15) return (uint16_t)(sign | 0x7C00u);
    const uint32_t full = man | 0x800000u;
    const int sh = ue < -14 ? -1 - ue : 13;
    uint32_t t = full >> sh;
    const uint32_t rem = full & ((1u << sh) - 1u), halfway = 1u << (sh - 1);
    if (rem > halfway || (rem == halfway && (t & 1u))) t++;
    if (ue < -14) return (uint16_t)(sign | (t >= 0x400u ? 0x400u : t));
    uint32_t he = (uint32_t)(ue + 15);
    if (t >= 0x800u) {
        he++;
        return (uint16_t)(he >= 31 ? (sign | 0x7C00u) : (sign | (he << 10)));
    }
    return (uint16_t)(sign | (he << 10) | (t & 0x3FFu));
}

namespace {

inline float absmax32(const float* p, uint64_t cnt) {
    float a = 0.f;
    for (uint64_t i = 0; i < cnt; i++) { float v = fabsf(p[i]); if (v > a) a = v; }
    return a;
}
inline float round_half_away(float v) { return roundf(v); }

// quantize_f32_to_q8_0, weight_loader.rs:1454-1486
void q8_blocks(const float* d, uint64_t n, uint64_t b0, uint64_t b1, uint8_t* out) {
    for (uint64_t b = b0; b < b1; b++) {
        const uint64_t base = b * 32, cnt = std::min<uint64_t>(32, n - base);
        const float amax = absmax32(d + base, cnt);
        const float sc = amax == 0.f ? 0.f : amax / 127.0f;
        const float inv = sc != 0.f ? 1.0f / sc : 0.f;
        uint8_t* o = out + b * 34;
        const uint16_t sb = f32_to_f16_host(sc);
        o[0] = (uint8_t)sb; o[1] = (uint8_t)(sb >> 8);
        for (uint64_t j = 0; j < 32; j++) {
            int8_t code = 0;
            if (j < cnt) {
                float r = round_half_away(d[base + j] * inv);
                r = std::max(-127.0f, std::min(127.0f, r));
                code = (int8_t)r;
            }
            o[2 + j] = (uint8_t)code;
        }
    }
}

// quantize_f32_to_q4_0, weight_loader.rs:1494-1544 (scale = amax/8, unsigned amax)
void q4_blocks(const float* d, uint64_t n, uint64_t b0, uint64_t b1, uint8_t* out) {
    for (uint64_t b = b0; b < b1; b++) {
        const uint64_t base = b * 32, cnt = std::min<uint64_t>(32, n - base);
        const float amax = absmax32(d + base, cnt);
        const float sc = amax / 8.0f;
        const float inv = sc != 0.f ? 1.0f / sc : 0.f;
        uint8_t* o = out + b * 18;
        const uint16_t sb = f32_to_f16_host(sc);
        o[0] = (uint8_t)sb; o[1] = (uint8_t)(sb >> 8);
        auto code = [&](uint64_t idx) -> uint32_t {
            const float v = idx < cnt ? d[base + idx] : 0.f;
            int c = (int)round_half_away(v * inv) + 8;
            return (uint32_t)std::max(0, std::min(15, c));
        };
        for (uint64_t j = 0; j < 16; j++) o[2 + j] = (uint8_t)(code(j) | (code(j + 16) << 4));
    }
}

template <typename F>
void parallel_blocks(uint64_t nblocks, F&& fn) {
    unsigned nt = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    if (nblocks < 4096) nt = 1;
    if (nt == 1) { fn(0, nblocks); return; }
    std::vector<std::thread> th;
    const uint64_t per = (nblocks + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const uint64_t a = t * per, b = std::min(nblocks, a + per);
        if (a < b) th.emplace_back([=, &fn] { fn(a, b); });
    }
    for (auto& t : th) t.join();
}

}  // namespace

void quantize_host(uint32_t wdtype, const float* d, uint64_t n, uint8_t* out) {
    const uint64_t nb = (n + 31) / 32;
    if (wdtype == FORGE_HIP_Q8_0) parallel_blocks(nb, [&](uint64_t a, uint64_t b) { q8_blocks(d, n, a, b, out); });
    else parallel_blocks(nb, [&](uint64_t a, uint64_t b) { q4_blocks(d, n, a, b, out); });
}

// dequant_q8_0 / dequant_q4_0, weight_loader.rs:860-926
void dequant_host(uint32_t wdtype, const uint8_t* data, uint64_t n, float* out) {
    const uint64_t nb = (n + 31) / 32;
    parallel_blocks(nb, [&](uint64_t b0, uint64_t b1) {
    for (uint64_t b = b0; b < b1; b++) {
        if (wdtype == FORGE_HIP_Q8_0) {
            const uint8_t* blk = data + b * 34;
            const float sc = f16_to_f32_host((uint16_t)(blk[0] | (blk[1] << 8)));
            for (uint64_t j = 0; j < 32 && b * 32 + j < n; j++) out[b * 32 + j] = (float)(int8_t)blk[2 + j] * sc;
        } else {
            const uint8_t* blk = data + b * 18;
            const float sc = f16_to_f32_host((uint16_t)(blk[0] | (blk[1] << 8)));
            for (uint64_t j = 0; j < 16; j++) {
                const int lo = (blk[2 + j] & 0x0F) - 8, hi = (blk[2 + j] >> 4) - 8;
                if (b * 32 + j < n) out[b * 32 + j] = (float)lo * sc;
                if (b * 32 + j + 16 < n) out[b * 32 + j + 16] = (float)hi * sc;
            }
        }
    }
    });
}

void repack_host(uint32_t wdtype, const uint8_t* raw, uint32_t K, uint64_t N, uint8_t* qs, uint16_t* scales) {
    const uint64_t nblk = K / 32;
    const uint64_t qb = wdtype == FORGE_HIP_Q8_0 ? 32 : 16, bb = qb + 2;
    parallel_blocks(N, [&](uint64_t r0, uint64_t r1) {
        for (uint64_t r = r0; r < r1; r++) {
            const uint8_t* src = raw + r * nblk * bb;
            uint8_t* dq = qs + r * nblk * qb;
            uint16_t* ds = scales + r * nblk;
            for (uint64_t b = 0; b < nblk; b++) {
                ds[b] = (uint16_t)(src[b * bb] | (src[b * bb + 1] << 8));
                memcpy(dq + b * qb, src + b * bb + 2, qb);
            }
        }
    });
}

}  // namespace fh

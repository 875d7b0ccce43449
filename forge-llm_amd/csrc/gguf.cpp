// GGUF on the input side of the hot path (host code only): the file parser, the model configuration read from
// its metadata, and the conversion of its tensors into the headerless weights blob that forge_hip_model_create takes.
//
//   parse            crates/forgellm-frontend/src/gguf.rs:484-551 (header, metadata, tensor descriptors, alignment)
//   config           crates/forgellm-cli/src/main.rs:700-830 (metadata keys, defaults, majority vote on the dtype)
//   tensor names     crates/forgellm-frontend/src/weight_loader.rs:400-447 (gguf_name_to_hf)
//   blob order       crates/forgellm-cli/src/main.rs:2714-2757 (export-weights)
//
// A file is memory-mapped and tensors are converted straight from the mapping into the caller's buffer.
#include <errno.h>
#include <fcntl.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <memory>
#include <new>
#include <stdexcept>

#include "common.h"

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;      // "GGUF", gguf.rs:18
constexpr uint64_t DEFAULT_ALIGNMENT = 32;         // gguf.rs:21

enum : uint32_t { T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q8_0 = 8, T_BF16 = 30 };

// Elements per block and bytes per block of every GGML type id the reference knows (gguf.rs:207-258);
// other ids are refused (GGUFError::UnsupportedGGMLType).
bool ggml_type_layout(uint32_t id, uint32_t* block, uint32_t* bytes) {
    static const struct { uint32_t id, block, bytes; } t[] = {
        {0, 1, 4},     {1, 1, 2},     {2, 32, 18},   {3, 32, 20},   {6, 32, 22},   {7, 32, 24},   {8, 32, 34},  {9, 32, 40},
        {10, 256, 84}, {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292}, {16, 256, 66}, {17, 256, 74},
        {18, 256, 98}, {19, 256, 50},  {20, 32, 18},  {21, 256, 110}, {22, 256, 82},  {23, 32, 36},   {24, 1, 1},   {25, 1, 2},
        {26, 1, 4},    {27, 1, 8},    {28, 1, 8},    {29, 256, 56},  {30, 1, 2}};
    for (const auto& e : t)
        if (e.id == id) { *block = e.block; *bytes = e.bytes; return true; }
    return false;
}

struct MetaValue {
    uint32_t type = 0;           // GGUF value type id 0..12
    uint64_t bits = 0;           // scalars: the value's bytes, little endian, zero-extended
    std::string str;             // type 8
    uint32_t elem_type = 0;      // type 9
    uint64_t count = 0;          // type 9: number of elements (elements themselves are skipped, only counted)
};

// No tensor of a real file comes near this; below it, element counts times bytes per block cannot wrap 64 bits.
constexpr uint64_t MAX_TENSOR_ELEMENTS = 1ull << 48;

struct TensorInfo {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[4] = {0, 0, 0, 0};
    uint32_t type = 0;
    uint64_t offset = 0;         // from the start of the tensor data section
    uint64_t numel() const { uint64_t n = 1; for (uint32_t i = 0; i < n_dims; i++) n *= dims[i]; return n; }
    uint64_t data_size() const {                              // gguf.rs:278-284
        uint32_t block = 1, bytes = 0;
        ggml_type_layout(type, &block, &bytes);
        return (numel() + block - 1) / block * bytes;
    }
};

struct Reader {
    const uint8_t* p;
    uint64_t n, pos = 0;
    bool ok = true;
    bool take(void* dst, uint64_t k) {
        if (!ok || k > n - pos) { ok = false; memset(dst, 0, k); return false; }
        memcpy(dst, p + pos, k);
        pos += k;
        return true;
    }
    template <typename T> T get() { T v{}; take(&v, sizeof(T)); return v; }
    bool str(std::string* s) {
        const uint64_t len = get<uint64_t>();
        if (!ok || len > n - pos) { ok = false; return false; }
        s->assign(reinterpret_cast<const char*>(p + pos), len);
        pos += len;
        return true;
    }
};

bool valid_utf8(const std::string& s) {
    size_t i = 0;
    while (i < s.size()) {
        const uint8_t c = (uint8_t)s[i];
        int extra = c < 0x80 ? 0 : (c >> 5) == 6 ? 1 : (c >> 4) == 14 ? 2 : (c >> 3) == 30 ? 3 : -1;
        if (extra < 0 || i + extra >= s.size() + (extra == 0)) return false;
        for (int k = 1; k <= extra; k++)
            if (((uint8_t)s[i + k] >> 6) != 2) return false;
        i += extra + 1;
    }
    return true;
}

}  // namespace

struct forge_hip_gguf {
    const uint8_t* data = nullptr;
    uint64_t nbytes = 0;
    void* map = nullptr;          // set when the library mapped the file itself
    uint64_t map_len = 0;
    uint32_t version = 0;
    uint64_t alignment = DEFAULT_ALIGNMENT, tensor_data_offset = 0;
    std::map<std::string, MetaValue> meta;
    std::vector<TensorInfo> tensors;
    ~forge_hip_gguf() { if (map) munmap(map, map_len); }
    const MetaValue* find(const std::string& k) const { auto it = meta.find(k); return it == meta.end() ? nullptr : &it->second; }
    const TensorInfo* tensor(const std::string& name) const {
        for (const auto& t : tensors) if (t.name == name) return &t;
        return nullptr;
    }
    bool get_u32(const std::string& k, uint32_t* out) const {         // gguf.rs:306-308: a Uint32 value only
        const MetaValue* v = find(k);
        if (!v || v->type != 4) return false;
        *out = (uint32_t)v->bits;
        return true;
    }
    bool get_u64(const std::string& k, uint64_t* out) const {         // gguf.rs:311-317: Uint64, or Uint32 widened
        const MetaValue* v = find(k);
        if (!v || (v->type != 10 && v->type != 4)) return false;
        *out = v->bits;
        return true;
    }
    bool get_f32(const std::string& k, float* out) const {
        const MetaValue* v = find(k);
        if (!v || v->type != 6) return false;
        const uint32_t b = (uint32_t)v->bits;
        memcpy(out, &b, 4);
        return true;
    }
};

namespace {

using fh::fail;

// One metadata value (gguf.rs:447-476).  Array elements are parsed (they may be strings or nested arrays) but not kept.
int32_t read_value(Reader& r, uint32_t type, MetaValue* v, int depth) {
    static const int width[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
    if (type > 12) return fail(FORGE_HIP_ERR_INVALID, "gguf: unsupported metadata value type: " + std::to_string(type));
    if (v) v->type = type;
    if (type == 8) {
        std::string s;
        if (!r.str(&s)) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside a metadata string");
        if (!valid_utf8(s)) return fail(FORGE_HIP_ERR_INVALID, "gguf: invalid UTF-8 in string");
        if (v) v->str = std::move(s);
        return FORGE_HIP_OK;
    }
    if (type == 9) {
        const uint32_t et = r.get<uint32_t>();
        const uint64_t count = r.get<uint64_t>();
        if (!r.ok) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside a metadata array");
        if (depth > 8) return fail(FORGE_HIP_ERR_INVALID, "gguf: metadata arrays nested too deeply");
        if (v) { v->elem_type = et; v->count = count; }
        if (et <= 12 && width[et]) {                        // fixed-width elements: skip them in one step
            if (count > (r.n - r.pos) / width[et]) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside a metadata array");
            r.pos += count * width[et];
            return FORGE_HIP_OK;
        }
        for (uint64_t i = 0; i < count; i++) {
            const int32_t rc = read_value(r, et, nullptr, depth + 1);
            if (rc) return rc;
        }
        return FORGE_HIP_OK;
    }
    uint64_t bits = 0;
    if (!r.take(&bits, width[type])) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside a metadata value");
    if (type == 7) bits = bits != 0;                        // read_bool, gguf.rs:436-438
    if (v) v->bits = bits;
    return FORGE_HIP_OK;
}

int32_t parse_into(forge_hip_gguf* g) {
    Reader r{g->data, g->nbytes};
    const uint32_t magic = r.get<uint32_t>();
    if (!r.ok) return fail(FORGE_HIP_ERR_INVALID, "gguf: file shorter than its header");
    if (magic != GGUF_MAGIC) {
        char buf[64];
        snprintf(buf, sizeof buf, "gguf: invalid GGUF magic number: got 0x%08X", magic);
        return fail(FORGE_HIP_ERR_INVALID, buf);
    }
    g->version = r.get<uint32_t>();
    if (r.ok && g->version != 2 && g->version != 3)
        return fail(FORGE_HIP_ERR_INVALID, "gguf: unsupported GGUF version: " + std::to_string(g->version) + " (supported: 2, 3)");
    const uint64_t n_tensors = r.get<uint64_t>(), n_meta = r.get<uint64_t>();
    if (!r.ok) return fail(FORGE_HIP_ERR_INVALID, "gguf: file shorter than its header");
    for (uint64_t i = 0; i < n_meta; i++) {
        std::string key;
        if (!r.str(&key)) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside the metadata");
        if (!valid_utf8(key)) return fail(FORGE_HIP_ERR_INVALID, "gguf: invalid UTF-8 in string");
        const uint32_t type = r.get<uint32_t>();
        if (!r.ok) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside the metadata");
        MetaValue v;
        const int32_t rc = read_value(r, type, &v, 0);
        if (rc) return rc;
        g->meta[key] = std::move(v);                        // a repeated key keeps the last value (HashMap::insert)
    }
    for (uint64_t i = 0; i < n_tensors; i++) {
        TensorInfo t;
        if (!r.str(&t.name)) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside the tensor descriptors");
        if (!valid_utf8(t.name)) return fail(FORGE_HIP_ERR_INVALID, "gguf: invalid UTF-8 in string");
        t.n_dims = r.get<uint32_t>();
        if (r.ok && t.n_dims > 4)
            return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor dimension count " + std::to_string(t.n_dims) + " exceeds maximum (4)");
        for (uint32_t d = 0; d < t.n_dims; d++) t.dims[d] = r.get<uint64_t>();
        {
            // the sizes below are products of these: refuse what no file can hold before anything multiplies them
            uint64_t n = 1;
            bool over = false;
            for (uint32_t d = 0; d < t.n_dims; d++) over = over || __builtin_mul_overflow(n, t.dims[d], &n);
            if (r.ok && (over || n > MAX_TENSOR_ELEMENTS))
                return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + t.name + " has more than 2^48 elements");
        }
        t.type = r.get<uint32_t>();
        t.offset = r.get<uint64_t>();
        if (!r.ok) return fail(FORGE_HIP_ERR_INVALID, "gguf: file ends inside the tensor descriptors");
        uint32_t block, bytes;
        if (!ggml_type_layout(t.type, &block, &bytes))
            return fail(FORGE_HIP_ERR_INVALID, "gguf: unsupported GGML type ID: " + std::to_string(t.type));
        g->tensors.push_back(std::move(t));
    }
    uint32_t al = 0;
    g->alignment = g->get_u32("general.alignment", &al) ? al : DEFAULT_ALIGNMENT;
    if (g->alignment == 0) return fail(FORGE_HIP_ERR_INVALID, "gguf: general.alignment is 0");
    g->tensor_data_offset = (r.pos + g->alignment - 1) / g->alignment * g->alignment;
    return FORGE_HIP_OK;
}

// ---- tensors -> blob --------------------------------------------------------------------------------------

// GGUF name of a tensor the blob needs (inverse of gguf_name_to_hf, weight_loader.rs:400-447).
std::string blk(uint32_t l, const char* suffix) { return "blk." + std::to_string(l) + "." + suffix; }

struct Source {
    const TensorInfo* t;
    const uint8_t* bytes;
};

int32_t locate(const forge_hip_gguf* g, const std::string& name, uint64_t numel, Source* out) {
    const TensorInfo* t = g->tensor(name);
    if (!t) return fail(FORGE_HIP_ERR_INVALID, "gguf: weight not found: " + name);
    if (t->numel() != numel)
        return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + name + " has " + std::to_string(t->numel()) + " elements, the configuration needs " +
                                               std::to_string(numel));
    const uint64_t start = g->tensor_data_offset + t->offset, size = t->data_size();
    if (t->offset > g->nbytes || start > g->nbytes || size > g->nbytes - start)
        return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + name + " extends past end of file");      // weight_loader.rs:172-177
    out->t = t;
    out->bytes = g->data + start;
    return FORGE_HIP_OK;
}

// ---- the other block formats the reference's loader reads (weight_loader.rs:809-825) --------------------------------
// Values in the reference's order of f32 operations (no fused multiply-add: this file is built with -ffp-contract=off).

// get_scale_min_k4, weight_loader.rs:977-987: 6-bit scale and minimum j of the 12 packed bytes of a K-quant super-block.
void scale_min_k4(int j, const uint8_t* sc, uint8_t* scale, uint8_t* mn) {
    if (j < 4) { *scale = sc[j] & 63; *mn = sc[j + 4] & 63; }
    else { *scale = (uint8_t)((sc[j + 4] & 0x0F) | ((sc[j - 4] >> 6) << 4)); *mn = (uint8_t)((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)); }
}
float half_at(const uint8_t* p) { return fh::f16_to_f32_host((uint16_t)(p[0] | (p[1] << 8))); }

// dequant_q4_1, weight_loader.rs:931-965: 20 bytes = f16 scale, f16 minimum, 16 bytes of nibbles; q * scale + min.
void dequant_q4_1(const uint8_t* d, uint64_t n, float* out) {
    for (uint64_t b = 0; b * 32 < n; b++) {
        const uint8_t* blk = d + b * 20;
        const float scale = half_at(blk), mn = half_at(blk + 2);
        for (uint64_t j = 0; j < 16; j++) {
            const float lo = (float)(blk[4 + j] & 0x0F), hi = (float)(blk[4 + j] >> 4);
            if (b * 32 + j < n) out[b * 32 + j] = lo * scale + mn;
            if (b * 32 + j + 16 < n) out[b * 32 + j + 16] = hi * scale + mn;
        }
    }
}
// dequant_q4_k (weight_loader.rs:1146-1201) and dequant_q5_k (:1071-1135): 256 elements in four chunks of 64, each with
// two (scale, minimum) pairs; value = (d * sc) * q - (dmin * m).  Q5_K adds one high bit per element from `qh`.
void dequant_q45_k(bool five, const uint8_t* d, uint64_t n, float* out) {
    const uint64_t bytes = five ? 176 : 144;
    for (uint64_t b = 0; b * 256 < n; b++) {
        const uint8_t* blk = d + b * bytes;
        const float dd = half_at(blk), dmin = half_at(blk + 2);
        const uint8_t* scales = blk + 4;
        const uint8_t* qh = blk + 16;                       // Q5_K only
        const uint8_t* qs = blk + (five ? 48 : 16);
        for (int chunk = 0; chunk < 4; chunk++) {
            uint8_t sc1, m1, sc2, m2;
            scale_min_k4(2 * chunk, scales, &sc1, &m1);
            scale_min_k4(2 * chunk + 1, scales, &sc2, &m2);
            const float d1 = dd * (float)sc1, mm1 = dmin * (float)m1, d2 = dd * (float)sc2, mm2 = dmin * (float)m2;
            const uint8_t u1 = (uint8_t)(1u << (2 * chunk)), u2 = (uint8_t)(2u << (2 * chunk));
            for (uint64_t l = 0; l < 32; l++) {
                const uint64_t o = b * 256 + chunk * 64 + l;
                const uint8_t q = qs[chunk * 32 + l];
                const uint32_t lo = (q & 0x0F) + ((five && (qh[l] & u1)) ? 16u : 0u);
                const uint32_t hi = (q >> 4) + ((five && (qh[l] & u2)) ? 16u : 0u);
                if (o < n) out[o] = d1 * (float)lo - mm1;
                if (o + 32 < n) out[o + 32] = d2 * (float)hi - mm2;
            }
        }
    }
}
// dequant_q6_k, weight_loader.rs:997-1057: 210 bytes = 128 low nibbles, 64 bytes of high bit pairs, 16 int8 scales, f16 d;
// two halves of 128 elements, four interleaved values per step; value = (d * sc) * (q - 32).
void dequant_q6_k(const uint8_t* d, uint64_t n, float* out) {
    for (uint64_t b = 0; b * 256 < n; b++) {
        const uint8_t* blk = d + b * 210;
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t* sc = reinterpret_cast<const int8_t*>(blk + 192);
        const float dd = half_at(blk + 208);
        for (uint64_t half = 0; half < 2; half++) {
            const uint8_t *l4 = ql + 64 * half, *h2 = qh + 32 * half;
            const int8_t* s = sc + 8 * half;
            for (uint64_t l = 0; l < 32; l++) {
                const int is = (int)(l / 16);
                const int q1 = (int)((l4[l] & 0x0F) | ((h2[l] & 3) << 4)) - 32;
                const int q2 = (int)((l4[l + 32] & 0x0F) | (((h2[l] >> 2) & 3) << 4)) - 32;
                const int q3 = (int)((l4[l] >> 4) | (((h2[l] >> 4) & 3) << 4)) - 32;
                const int q4 = (int)((l4[l + 32] >> 4) | (((h2[l] >> 6) & 3) << 4)) - 32;
                const uint64_t o = b * 256 + 128 * half + l;
                if (o < n) out[o] = dd * (float)s[is] * (float)q1;
                if (o + 32 < n) out[o + 32] = dd * (float)s[is + 2] * (float)q2;
                if (o + 64 < n) out[o + 64] = dd * (float)s[is + 4] * (float)q3;
                if (o + 96 < n) out[o + 96] = dd * (float)s[is + 6] * (float)q4;
            }
        }
    }
}
// dequant_q8_k, weight_loader.rs:1206-1229: f32 scale + 256 int8 (+ 32 bytes of block sums that are not used).
void dequant_q8_k(const uint8_t* d, uint64_t n, float* out) {
    for (uint64_t b = 0; b * 256 < n; b++) {
        const uint8_t* blk = d + b * 292;
        float scale;
        memcpy(&scale, blk, 4);
        for (uint64_t j = 0; j < 256 && b * 256 + j < n; j++) out[b * 256 + j] = scale * (float)(int8_t)blk[4 + j];
    }
}

// Types whose tensors the reference's loader turns into Q8_0 when it reads them (weight_loader.rs:219-229).
bool requantised_on_load(uint32_t type) { return type == 3 || type == 12 || type == 13 || type == 14 || type == 15; }

// `dequantize` of weight_loader.rs:809-825 for the types this library reads.
bool dequant_ggml(uint32_t type, const uint8_t* d, uint64_t n, float* out) {
    switch (type) {
        case T_F32: memcpy(out, d, n * 4); return true;
        case T_F16: for (uint64_t i = 0; i < n; i++) out[i] = half_at(d + 2 * i); return true;
        case T_BF16:
            for (uint64_t i = 0; i < n; i++) { const uint32_t b = ((uint32_t)(d[2 * i] | (d[2 * i + 1] << 8))) << 16; memcpy(out + i, &b, 4); }
            return true;
        case T_Q8_0: fh::dequant_host(FORGE_HIP_Q8_0, d, n, out); return true;
        case T_Q4_0: fh::dequant_host(FORGE_HIP_Q4_0, d, n, out); return true;
        case 3: dequant_q4_1(d, n, out); return true;
        case 12: dequant_q45_k(false, d, n, out); return true;
        case 13: dequant_q45_k(true, d, n, out); return true;
        case 14: dequant_q6_k(d, n, out); return true;
        case 15: dequant_q8_k(d, n, out); return true;
        default: return false;
    }
}

// ---- the K-quant weight quantisers (weight_loader.rs:1646-2140): used when a tensor's format differs from the format its
// projection category is stored in (load_from_file_mixed_per_tensor, weight_loader.rs:193-218) -----------------------------

inline float round_away(float v) { return roundf(v); }          // f32::round: halves away from zero
inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

// make_qkx2_quants (weight_loader.rs:1666-1768) for one sub-block of 32: returns scale and the_min (>= 0) with
// dequant(L) = scale * L - the_min, L in [0, nmax]; a search over nstep + 1 slightly shifted inverse scales, each refitted by
// two-parameter least squares, keeping the candidate with the least squared error.
void make_qkx2_quants(const float* x, float nmax, float rmin, float rdelta, int nstep, float* scale_out, float* min_out, uint8_t* L) {
    const int n = 32;
    float mn = x[0], mx = x[0];
    for (int i = 1; i < n; i++) { if (x[i] < mn) mn = x[i]; if (x[i] > mx) mx = x[i]; }
    if (mx == mn) { *scale_out = 0.0f; *min_out = -mn; memset(L, 0, n); return; }
    if (mn > 0.0f) mn = 0.0f;
    const float iscale = nmax / (mx - mn);
    const float scale = 1.0f / iscale;
    float best_mad = 0.0f;
    for (int i = 0; i < n; i++) {
        const float li = clampf(round_away((x[i] - mn) * iscale), 0.0f, nmax);
        L[i] = (uint8_t)li;
        const float diff = scale * (float)L[i] + mn - x[i];
        best_mad += diff * diff;
    }
    float best_min = mn, best_scale = scale;
    uint8_t laux[32];
    for (int is = 0; is <= nstep && nstep > 0; is++) {
        const float iscale_try = (rmin + rdelta * (float)is + nmax) / (mx - mn);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_x = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; i++) {
            laux[i] = (uint8_t)clampf(round_away((x[i] - mn) * iscale_try), 0.0f, nmax);
            const float lif = (float)laux[i];
            sum_l += lif;
            sum_l2 += lif * lif;
            sum_x += x[i];
            sum_xl += lif * x[i];
        }
        const float nf = (float)n;
        const float det = nf * sum_l2 - sum_l * sum_l;
        if (!(det > 0.0f)) continue;
        float this_scale = (nf * sum_xl - sum_x * sum_l) / det;
        float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / det;
        if (this_min > 0.0f) {
            this_min = 0.0f;
            if (sum_l2 > 0.0f) this_scale = sum_xl / sum_l2;
        }
        if (!(this_scale > 0.0f)) continue;
        float mad = 0.0f;
        for (int i = 0; i < n; i++) {
            const float diff = this_scale * (float)laux[i] + this_min - x[i];
            mad += diff * diff;
        }
        if (mad < best_mad) { memcpy(L, laux, n); best_mad = mad; best_scale = this_scale; best_min = this_min; }
    }
    *scale_out = best_scale;
    *min_out = -best_min;
}

// quantize_f32_to_q4_k, weight_loader.rs:1773-1882: n floats -> ceil(n / 256) super-blocks of 144 bytes (a tail is padded with zeros).
void quantize_q4_k(const float* data, uint64_t n, uint8_t* out) {
    const uint64_t nsb = (n + 255) / 256;
    for (uint64_t sb = 0; sb < nsb; sb++) {
        float padded[256] = {0};
        const uint64_t have = std::min<uint64_t>(256, n - sb * 256);
        memcpy(padded, data + sb * 256, have * 4);
        float sub_scale[8], sub_min[8];
        uint8_t q[8][32];
        for (int j = 0; j < 8; j++) make_qkx2_quants(padded + j * 32, 15.0f, -1.0f, 0.1f, 20, &sub_scale[j], &sub_min[j], q[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) { if (sub_scale[j] > max_scale) max_scale = sub_scale[j]; if (sub_min[j] > max_min) max_min = sub_min[j]; }
        const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        const float d = max_scale > 0.0f ? max_scale / 63.0f : 0.0f;
        const float dmin = max_min > 0.0f ? max_min / 63.0f : 0.0f;
        uint8_t sq[8], mq[8];
        for (int j = 0; j < 8; j++) {
            sq[j] = (uint8_t)clampf(round_away(sub_scale[j] * inv_scale), 0.0f, 63.0f);
            mq[j] = (uint8_t)clampf(round_away(sub_min[j] * inv_min), 0.0f, 63.0f);
        }
        // the codes are fitted again to the scales as stored (6 bits under an fp16 super-block scale), :1826-1850
        const uint16_t d_bits = fh::f32_to_f16_host(d), dmin_bits = fh::f32_to_f16_host(dmin);
        const float d_stored = fh::f16_to_f32_host(d_bits), dmin_stored = fh::f16_to_f32_host(dmin_bits);
        for (int j = 0; j < 8; j++) {
            const float s_eff = d_stored * (float)sq[j];
            if (s_eff == 0.0f) { memset(q[j], 0, 32); continue; }
            const float inv_s_eff = 1.0f / s_eff;
            const float dm_eff = dmin_stored * (float)mq[j];
            for (int i = 0; i < 32; i++) q[j][i] = (uint8_t)clampf(round_away((padded[j * 32 + i] + dm_eff) * inv_s_eff), 0.0f, 15.0f);
        }
        uint8_t* o = out + sb * 144;
        o[0] = (uint8_t)d_bits; o[1] = (uint8_t)(d_bits >> 8); o[2] = (uint8_t)dmin_bits; o[3] = (uint8_t)(dmin_bits >> 8);
        for (int i = 0; i < 4; i++) {                 // inverse of get_scale_min_k4
            o[4 + i] = (uint8_t)((sq[i] & 63) | (((sq[i + 4] >> 4) & 3) << 6));
            o[8 + i] = (uint8_t)((mq[i] & 63) | (((mq[i + 4] >> 4) & 3) << 6));
            o[12 + i] = (uint8_t)((sq[i + 4] & 0x0F) | ((mq[i + 4] & 0x0F) << 4));
        }
        for (int c = 0; c < 4; c++)
            for (int i = 0; i < 32; i++) o[16 + c * 32 + i] = (uint8_t)((q[2 * c][i] & 0x0F) | (q[2 * c + 1][i] << 4));
    }
}

// make_q6k_quants' scale (weight_loader.rs:1987-2010): -max/32 for the signed value of largest magnitude (the FIRST of equals), 0 for a
// sub-block of zeros.  The codes it also fits are not used by the caller.
float q6k_sub_scale(const float* x) {
    float mx = 0.0f, amax = 0.0f;
    for (int i = 0; i < 16; i++) { const float av = fabsf(x[i]); if (av > amax) { amax = av; mx = x[i]; } }
    if (amax < 1e-30f) return 0.0f;
    const float iscale = -32.0f / mx;
    return 1.0f / iscale;
}

// quantize_f32_to_q6_k, weight_loader.rs:2025-2140: n floats -> ceil(n / 256) super-blocks of 210 bytes.
void quantize_q6_k(const float* data, uint64_t n, uint8_t* out) {
    const uint64_t nsb = (n + 255) / 256;
    for (uint64_t sb = 0; sb < nsb; sb++) {
        float padded[256] = {0};
        const uint64_t have = std::min<uint64_t>(256, n - sb * 256);
        memcpy(padded, data + sb * 256, have * 4);
        float sub[16];
        float max_scale = 0.0f, max_abs = 0.0f;
        for (int j = 0; j < 16; j++) {
            sub[j] = q6k_sub_scale(padded + j * 16);
            if (fabsf(sub[j]) > max_abs) { max_abs = fabsf(sub[j]); max_scale = sub[j]; }
        }
        uint8_t* o = out + sb * 210;
        memset(o, 0, 210);
        if (max_abs < 1e-30f) continue;
        const float super_iscale = -128.0f / max_scale;
        const float super_d = 1.0f / super_iscale;
        const uint16_t d_bits = fh::f32_to_f16_host(super_d);
        o[208] = (uint8_t)d_bits; o[209] = (uint8_t)(d_bits >> 8);
        int8_t sq[16];
        for (int j = 0; j < 16; j++) {
            int v = (int)round_away(super_iscale * sub[j]);
            v = v < -128 ? -128 : (v > 127 ? 127 : v);
            sq[j] = (int8_t)v;
            o[192 + j] = (uint8_t)sq[j];
        }
        const float d_stored = fh::f16_to_f32_host(d_bits);
        int8_t L[256] = {0};
        for (int j = 0; j < 16; j++) {
            const float s_eff = d_stored * (float)sq[j];
            if (s_eff == 0.0f) continue;
            const float inv = 1.0f / s_eff;
            for (int i = 0; i < 16; i++) {
                int v = (int)round_away(inv * padded[j * 16 + i]);
                L[j * 16 + i] = (int8_t)(v < -32 ? -32 : (v > 31 ? 31 : v));
            }
        }
        for (int half = 0; half < 2; half++) {
            uint8_t* ql = o + half * 64;
            uint8_t* qh = o + 128 + half * 32;
            const int8_t* l = L + half * 128;
            for (int i = 0; i < 32; i++) {
                const uint8_t q1 = (uint8_t)(l[i] + 32), q2 = (uint8_t)(l[i + 32] + 32), q3 = (uint8_t)(l[i + 64] + 32), q4 = (uint8_t)(l[i + 96] + 32);
                ql[i] = (uint8_t)((q1 & 0x0F) | ((q3 & 0x0F) << 4));
                ql[i + 32] = (uint8_t)((q2 & 0x0F) | ((q4 & 0x0F) << 4));
                qh[i] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
            }
        }
    }
}

const char* const SUPPORTED_TYPES = "F32, F16, BF16, Q8_0, Q4_0, Q4_1, Q4_K, Q5_K, Q6_K and Q8_K";

// f32 values of a tensor as the reference holds it after loading: dense types and Q8_0 / Q4_0 decode directly
// (weight_loader.rs:809-926); any other quantised type is first turned into Q8_0 blocks by the loader
// (dequantise, quantize_f32_to_q8_0: weight_loader.rs:219-229), so its values are those of the Q8_0 blocks.
int32_t to_f32(const Source& s, uint64_t numel, float* out) {
    if (!dequant_ggml(s.t->type, s.bytes, numel, out))
        return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + s.t->name + " has GGML type " + std::to_string(s.t->type) +
                                               "; this library reads " + SUPPORTED_TYPES + " tensors");
    if (requantised_on_load(s.t->type)) {
        std::vector<uint8_t> q8((numel + 31) / 32 * 34);
        fh::quantize_host(FORGE_HIP_Q8_0, out, numel, q8.data());
        fh::dequant_host(FORGE_HIP_Q8_0, q8.data(), numel, out);
    }
    return FORGE_HIP_OK;
}

uint64_t qbytes(uint32_t wdtype, uint64_t numel) { return numel / 32 * (wdtype == FORGE_HIP_Q8_0 ? 34 : 18); }

// A projection matrix in the blob's format: the file's bytes when it already has that format, otherwise its values
// quantised again with the reference's weight quantiser (weight_loader.rs:1454-1544).
int32_t write_quantised(const forge_hip_gguf* g, const std::string& name, uint32_t wdtype, uint64_t numel, uint8_t* out) {
    Source s;
    int32_t rc = locate(g, name, numel, &s);
    if (rc) return rc;
    if (s.t->type == wdtype) { memcpy(out, s.bytes, qbytes(wdtype, numel)); return FORGE_HIP_OK; }
    std::vector<float> v(numel);
    rc = to_f32(s, numel, v.data());
    if (rc) return rc;
    fh::quantize_host(wdtype, v.data(), numel, out);
    return FORGE_HIP_OK;
}

// Elements [first, first + numel) of a tensor of `total` elements, in the blob's format: one part of a fused Phi-3 tensor
// (split_weight_three / split_weight_two, weight_loader.rs:543-583, 641-700).  The reference splits what its loader made of the
// whole tensor, so a tensor in another format is converted whole and then cut; parts start on 32-element block boundaries
// because every row has a multiple of 32 elements.
int32_t write_quantised_part(const forge_hip_gguf* g, const std::string& name, uint32_t wdtype, uint64_t total, uint64_t first,
                             uint64_t numel, uint8_t* out) {
    Source s;
    int32_t rc = locate(g, name, total, &s);
    if (rc) return rc;
    if (first % 32 || numel % 32 || first + numel > total)
        return fail(FORGE_HIP_ERR_INVALID, "gguf: fused tensor " + name + " cannot be split on block boundaries");
    if (s.t->type == wdtype) { memcpy(out, s.bytes + qbytes(wdtype, first), qbytes(wdtype, numel)); return FORGE_HIP_OK; }
    std::vector<float> v(total);
    rc = to_f32(s, total, v.data());
    if (rc) return rc;
    fh::quantize_host(wdtype, v.data() + first, numel, out);
    return FORGE_HIP_OK;
}

int32_t write_f32(const forge_hip_gguf* g, const std::string& name, uint64_t numel, uint8_t* out) {
    Source s;
    const int32_t rc = locate(g, name, numel, &s);
    if (rc) return rc;
    return to_f32(s, numel, reinterpret_cast<float*>(out));
}

}  // namespace

// An allocation that fails (a vector sized from a damaged or hostile file) must not leave through the C boundary.
template <typename F>
int32_t no_throw(const char* name, F&& body) {
    try {
        return body();
    } catch (const std::bad_alloc&) {
        return fh::fail(FORGE_HIP_ERR_INVALID, std::string(name) + ": out of host memory");
    } catch (const std::length_error&) {
        return fh::fail(FORGE_HIP_ERR_INVALID, std::string(name) + ": a size in the file is too large");
    }
}

extern "C" {

int32_t forge_hip_gguf_parse(const uint8_t* data_host, uint64_t nbytes, forge_hip_gguf** out) {
    return no_throw("gguf_parse", [&]() -> int32_t {
        FH_CHECK(out, "gguf_parse: null out");
        *out = nullptr;
        FH_CHECK(data_host || nbytes == 0, "gguf_parse: null data");
        std::unique_ptr<forge_hip_gguf> g(new forge_hip_gguf());
        g->data = data_host;
        g->nbytes = nbytes;
        const int32_t rc = parse_into(g.get());
        if (rc) return rc;
        *out = g.release();
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_gguf_open(const char* path, forge_hip_gguf** out) {
    return no_throw("gguf_open", [&]() -> int32_t {
        FH_CHECK(out, "gguf_open: null out");
        *out = nullptr;
        FH_CHECK(path, "gguf_open: null path");
        const int fd = open(path, O_RDONLY);
        if (fd < 0) return fh::fail(FORGE_HIP_ERR_INVALID, std::string("gguf_open: cannot open ") + path + ": " + strerror(errno));
        struct stat st;
        if (fstat(fd, &st) != 0 || st.st_size <= 0) {
            close(fd);
            return fh::fail(FORGE_HIP_ERR_INVALID, std::string("gguf_open: cannot read ") + path);
        }
        void* map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
        close(fd);
        if (map == MAP_FAILED) return fh::fail(FORGE_HIP_ERR_INVALID, std::string("gguf_open: cannot map ") + path + ": " + strerror(errno));
        std::unique_ptr<forge_hip_gguf> g(new forge_hip_gguf());
        g->map = map;
        g->map_len = (uint64_t)st.st_size;
        g->data = reinterpret_cast<const uint8_t*>(map);
        g->nbytes = g->map_len;
        const int32_t rc = parse_into(g.get());
        if (rc) return rc;
        *out = g.release();
        return FORGE_HIP_OK;
    });
}

void forge_hip_gguf_close(forge_hip_gguf* g) { delete g; }

uint32_t forge_hip_gguf_version(const forge_hip_gguf* g) { return g ? g->version : 0; }
uint64_t forge_hip_gguf_alignment(const forge_hip_gguf* g) { return g ? g->alignment : 0; }
uint64_t forge_hip_gguf_tensor_data_offset(const forge_hip_gguf* g) { return g ? g->tensor_data_offset : 0; }
uint64_t forge_hip_gguf_tensor_count(const forge_hip_gguf* g) { return g ? g->tensors.size() : 0; }
uint64_t forge_hip_gguf_metadata_count(const forge_hip_gguf* g) { return g ? g->meta.size() : 0; }

int32_t forge_hip_gguf_tensor(const forge_hip_gguf* g, uint64_t index, const char** name, uint32_t* n_dims, uint64_t* dims4,
                              uint32_t* ggml_type, uint64_t* offset, uint64_t* data_size) {
    FH_CHECK(g, "gguf_tensor: null handle");
    FH_CHECK(index < g->tensors.size(), "gguf_tensor: index out of range");
    const TensorInfo& t = g->tensors[index];
    if (name) *name = t.name.c_str();
    if (n_dims) *n_dims = t.n_dims;
    if (dims4) for (int i = 0; i < 4; i++) dims4[i] = t.dims[i];
    if (ggml_type) *ggml_type = t.type;
    if (offset) *offset = t.offset;
    if (data_size) *data_size = t.data_size();
    return FORGE_HIP_OK;
}

int64_t forge_hip_gguf_find_tensor(const forge_hip_gguf* g, const char* name) {
    if (!g || !name) return -1;
    for (size_t i = 0; i < g->tensors.size(); i++)
        if (g->tensors[i].name == name) return (int64_t)i;
    return -1;
}

int32_t forge_hip_gguf_meta(const forge_hip_gguf* g, const char* key, uint32_t* type, uint64_t* bits, const char** str,
                            uint32_t* elem_type, uint64_t* count) {
    FH_CHECK(g && key, "gguf_meta: null argument");
    const MetaValue* v = g->find(key);
    if (!v) return fh::fail(FORGE_HIP_ERR_INVALID, std::string("gguf_meta: no such key: ") + key);
    if (type) *type = v->type;
    if (bits) *bits = v->bits;
    if (str) *str = v->type == 8 ? v->str.c_str() : nullptr;
    if (elem_type) *elem_type = v->elem_type;
    if (count) *count = v->count;
    return FORGE_HIP_OK;
}

int32_t forge_hip_dequant_ggml(uint32_t ggml_type, const uint8_t* data_host, uint64_t n, float* out_host) {
    return no_throw("dequant_ggml", [&]() -> int32_t {
        FH_CHECK(data_host && out_host, "dequant_ggml: null pointer");
        if (!dequant_ggml(ggml_type, data_host, n, out_host))
            return fh::fail(FORGE_HIP_ERR_INVALID, "dequant_ggml: GGML type " + std::to_string(ggml_type) + " is not one of " + SUPPORTED_TYPES);
        return FORGE_HIP_OK;
    });
}

}  // extern "C"

namespace {

// Everything of load_config (main.rs:700-830) but the weight formats: shape, context, RoPE, window, bias flag; `majority` =
// detect_gguf_dtype's vote over the projection tensors (main.rs:479-555): Q8_0 (8), Q4_0 (2), Q4_K (12), or 0 for a dense majority.
int32_t config_base(const forge_hip_gguf* g, uint32_t max_seq, uint32_t flags, forge_hip_config* out, uint32_t* majority) {
    {
        const MetaValue* arch_v = g->find("general.architecture");
        const std::string arch = arch_v && arch_v->type == 8 ? arch_v->str : "unknown";
        // The kernels here cover the Llama layer, with the QKV bias of Qwen2 (main.rs:770: the bias goes with the
        // architecture): no GeLU or embedding scale (gemma).  Mistral is the Llama layer plus an optional sliding window;
        // Phi-3 is the Llama layer with fused tensors in the file, which export_weights splits (main.rs:759).
        if (arch != "llama" && arch != "mistral" && arch != "qwen2" && arch != "phi3" && arch != "phi")
            return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: unsupported GGUF architecture: " + arch);
        const std::string p = arch + ".";
        uint32_t hidden = 0, layers = 0, heads = 0, kv_heads = 0, inter = 0;
        g->get_u32(p + "embedding_length", &hidden);
        g->get_u32(p + "block_count", &layers);
        g->get_u32(p + "attention.head_count", &heads);
        if (!g->get_u32(p + "attention.head_count_kv", &kv_heads)) kv_heads = heads;
        if (hidden == 0 || layers == 0 || heads == 0) return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: could not extract model config from GGUF metadata");
    if (!g->get_u32(p + "feed_forward_length", &inter)) {
            FH_CHECK(hidden <= 0x3FFFFFFFu, "gguf: embedding_length out of range");
            inter = hidden * 4;
        }
        uint64_t vocab = 32000, ctx = 2048;
        const MetaValue* tokens = g->find("tokenizer.ggml.tokens");
        if (tokens && tokens->type == 9) vocab = tokens->count;
        else g->get_u64(p + "vocab_size", &vocab);
        g->get_u64(p + "context_length", &ctx);
        float eps = 1e-5f, theta = 10000.0f;
        g->get_f32(p + "attention.layer_norm_rms_epsilon", &eps);
        g->get_f32(p + "rope.freq_base", &theta);
        uint32_t window = 0;
        const bool has_window = g->get_u32(p + "attention.sliding_window", &window);

        // majority vote over the projection tensors (main.rs:479-555)
        uint64_t q8 = 0, q4 = 0, q4k = 0, f16 = 0, f32 = 0;
        for (const auto& t : g->tensors) {
            const std::string& n = t.name;
            const bool proj = n.find(".weight") != std::string::npos && n.find("token_embd") == std::string::npos &&
                              n.find("output.weight") == std::string::npos && n.find("_norm") == std::string::npos;
            if (!proj) continue;
            switch (t.type) {
                case T_Q8_0: q8++; break;
                case T_Q4_0: q4++; break;
                case 12: q4k++; break;
                case T_F16: case T_BF16: f16++; break;
                case T_F32: f32++; break;
                case 3: case 20: case 23: case 6: case 7: case 9: case 10: case 11: case 13: case 14: case 15: case 16: case 17: case 22:
                case 18: case 21: case 19: case 29: q8++; break;
                default: break;
            }
        }
        const uint64_t total = q8 + q4 + q4k + f16 + f32;
        *majority = 0;
        if (total) {
            if (q4k > total / 2) *majority = FORGE_HIP_Q4_K;
            else if (q8 > total / 2) *majority = FORGE_HIP_Q8_0;
            else if (q4 > total / 2) *majority = FORGE_HIP_Q4_0;
        }
        const uint64_t seq = max_seq ? max_seq : ctx;
        // Some(0) would make the reference attend to nothing (emit.rs:604-605)
        if (has_window && window == 0) return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: a sliding window of 0 positions");
        FH_CHECK(vocab <= 0xFFFFFFFFull && seq <= 0xFFFFFFFFull, "gguf: vocabulary or context length out of range");
        forge_hip_config c{};
        c.hidden = hidden; c.inter = inter; c.layers = layers; c.heads = heads; c.kv_heads = kv_heads;
        c.head_dim = hidden / heads;                     // main.rs:731
        c.vocab = (uint32_t)vocab; c.max_seq = (uint32_t)seq;
        c.rms_eps = eps; c.rope_theta = theta;
        c.flags = flags | (arch == "qwen2" ? FORGE_HIP_FLAG_QKV_BIAS : 0u);
        c.sliding_window = has_window ? window : 0u;     // main.rs:764-767
        *out = c;
        return FORGE_HIP_OK;
    }
}

// ---- a storage format per projection category (detect_gguf_proj_dtypes, main.rs:608-680) ------------------------------------

enum Cat { C_EMBED, C_Q, C_K, C_V, C_O, C_GATE, C_UP, C_DOWN, C_LM, C_COUNT, C_NONE };
constexpr uint32_t DENSE = 1;      // the reference's DType::F16, which stands for every dense tensor type here

// ProjCategory::from_gguf_name, ir.rs:382-401
Cat category_of(const std::string& name) {
    if (name == "token_embd.weight") return C_EMBED;
    if (name == "output.weight" || name == "lm_head.weight") return C_LM;
    if (name.compare(0, 4, "blk.") != 0) return C_NONE;
    const size_t dot = name.find('.', 4);
    if (dot == std::string::npos) return C_NONE;
    const std::string suffix = name.substr(dot + 1);
    if (suffix == "attn_q.weight") return C_Q;
    if (suffix == "attn_k.weight") return C_K;
    if (suffix == "attn_v.weight") return C_V;
    if (suffix == "attn_output.weight") return C_O;
    if (suffix == "ffn_gate.weight") return C_GATE;
    if (suffix == "ffn_up.weight") return C_UP;
    if (suffix == "ffn_down.weight") return C_DOWN;
    return C_NONE;
}

// ggml_type_storage_dtype, main.rs:586-599: the format a tensor of this type can be kept in; 0 = none (the tensor does not vote)
uint32_t storage_dtype(uint32_t type) {
    switch (type) {
        case T_Q8_0: return FORGE_HIP_Q8_0;
        case T_Q4_0: return FORGE_HIP_Q4_0;
        case 12: return FORGE_HIP_Q4_K;
        case 14: return FORGE_HIP_Q6_K;
        case T_F32: case T_F16: case T_BF16: return DENSE;
        default: return 0;
    }
}

// precision_rank, main.rs:630-640: decides a tie of counts in favour of the more precise format
int precision_rank(uint32_t d) {
    switch (d) {
        case DENSE: return 5;
        case FORGE_HIP_Q8_0: return 4;
        case FORGE_HIP_Q6_K: return 3;
        case FORGE_HIP_Q4_K: return 2;
        case FORGE_HIP_Q4_0: return 1;
        default: return 0;
    }
}

// The nine category formats: the majority among the category's tensors, `fallback` for a category without a tensor that votes;
// a file without an output tensor takes the embedding's format for the lm_head (main.rs:668-678).
void detect_categories(const forge_hip_gguf* g, uint32_t fallback, uint32_t out[C_COUNT]) {
    static const uint32_t kinds[5] = {FORGE_HIP_Q8_0, FORGE_HIP_Q4_0, FORGE_HIP_Q4_K, FORGE_HIP_Q6_K, DENSE};
    uint64_t counts[C_COUNT][5] = {};
    bool has_lm = false;
    for (const auto& t : g->tensors) {
        const Cat c = category_of(t.name);
        if (c == C_NONE) continue;
        if (c == C_LM) has_lm = true;
        const uint32_t d = storage_dtype(t.type);
        for (int k = 0; k < 5; k++) if (kinds[k] == d) counts[c][k]++;
    }
    for (int c = 0; c < C_COUNT; c++) {
        uint32_t best = fallback;
        uint64_t best_n = 0;
        for (int k = 0; k < 5; k++)
            if (counts[c][k] > best_n || (counts[c][k] == best_n && best_n > 0 && precision_rank(kinds[k]) > precision_rank(best))) {
                best = kinds[k];
                best_n = counts[c][k];
            }
        out[c] = best;
    }
    if (!has_lm) out[C_LM] = out[C_EMBED];
}

uint64_t qbytes_any(uint32_t dtype, uint64_t numel) {
    if (dtype == FORGE_HIP_Q4_K) return numel / 256 * 144;
    if (dtype == FORGE_HIP_Q6_K) return numel / 256 * 210;
    return qbytes(dtype, numel);
}

// One tensor in the format of its category (load_from_file_mixed_per_tensor, weight_loader.rs:190-230): the file's bytes when the
// tensor already has that format; for a K-quant target its values (dequantised directly) quantised with that format's
// quantiser; for a Q8_0 / Q4_0 target the conversion of the uniform export.
int32_t write_in_format(const forge_hip_gguf* g, const std::string& name, uint32_t dtype, uint64_t numel, uint8_t* out) {
    if (dtype == FORGE_HIP_Q8_0 || dtype == FORGE_HIP_Q4_0) return write_quantised(g, name, dtype, numel, out);
    Source s;
    int32_t rc = locate(g, name, numel, &s);
    if (rc) return rc;
    if (numel % 256) return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + name + " is no whole number of 256-weight super-blocks");
    if (s.t->type == dtype) { memcpy(out, s.bytes, qbytes_any(dtype, numel)); return FORGE_HIP_OK; }
    std::vector<float> v(numel);
    if (!dequant_ggml(s.t->type, s.bytes, numel, v.data()))
        return fail(FORGE_HIP_ERR_INVALID, "gguf: tensor " + name + " has GGML type " + std::to_string(s.t->type) + "; this library reads " +
                                               SUPPORTED_TYPES + " tensors");
    if (dtype == FORGE_HIP_Q4_K) quantize_q4_k(v.data(), numel, out);
    else quantize_q6_k(v.data(), numel, out);
    return FORGE_HIP_OK;
}

}  // namespace

extern "C" {

int32_t forge_hip_gguf_config(const forge_hip_gguf* g, uint32_t max_seq, uint32_t flags, forge_hip_config* out) {
    return no_throw("gguf_config", [&]() -> int32_t {
        FH_CHECK(g && out, "gguf_config: null argument");
        forge_hip_config c{};
        uint32_t wdtype = 0;
        const int32_t brc = config_base(g, max_seq, flags, &c, &wdtype);
        if (brc) return brc;
        if (wdtype != FORGE_HIP_Q8_0 && wdtype != FORGE_HIP_Q4_0)
            return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: the projection weights are neither mostly Q8_0 nor mostly Q4_0");
        // lm_head: the type of output.weight after loading (main.rs:567-581, gguf.rs:168-205); without that tensor the
        // embedding table serves, converted to the projections' format
        uint32_t lm = wdtype;
        const TensorInfo* ot = g->tensor("output.weight");
        if (!ot) ot = g->tensor("lm_head.weight");
        if (ot) {
            if (ot->type == T_Q4_0) lm = FORGE_HIP_Q4_0;
            else if (ot->type == T_Q8_0) lm = FORGE_HIP_Q8_0;
            else if (ot->type == T_F32 || ot->type == T_F16 || ot->type == T_BF16) lm = wdtype;   // dense: quantised like the projections
            else if (requantised_on_load(ot->type)) lm = FORGE_HIP_Q8_0;                          // GGMLType::to_dtype, gguf.rs:168-205
            else return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: output.weight has GGML type " + std::to_string(ot->type) +
                                                           "; this library reads " + SUPPORTED_TYPES + " tensors");
        }
        c.wdtype = wdtype; c.lm_head_dtype = lm;
        // what the kernels cannot run is refused here, before any size is computed from these numbers
        const int32_t vrc = fh::validate_config_shape(&c);
        if (vrc) return vrc;
        *out = c;
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_gguf_export_weights(const forge_hip_gguf* g, const forge_hip_config* c, uint8_t* out_host, uint64_t nbytes) {
    return no_throw("gguf_export_weights", [&]() -> int32_t {
        FH_CHECK(g && c && out_host, "gguf_export_weights: null argument");
        FH_CHECK(c->wdtype == FORGE_HIP_Q8_0 || c->wdtype == FORGE_HIP_Q4_0, "gguf_export_weights: wdtype must be Q8_0 or Q4_0");
        FH_CHECK(c->lm_head_dtype == FORGE_HIP_Q8_0 || c->lm_head_dtype == FORGE_HIP_Q4_0, "gguf_export_weights: lm_head_dtype must be Q8_0 or Q4_0");
        FH_CHECK(c->hidden % 32 == 0 && c->inter % 32 == 0 && (c->heads * c->head_dim) % 32 == 0, "gguf_export_weights: row lengths must be multiples of 32");
        const int32_t vrc = fh::validate_config_shape(c);
        if (vrc) return vrc;
        const uint64_t need = forge_hip_weights_nbytes(c);
        if (need == 0 || nbytes != need)
            return fh::fail(FORGE_HIP_ERR_BLOB_SIZE, "gguf_export_weights: buffer is " + std::to_string(nbytes) + " bytes, config needs " + std::to_string(need));
        const uint64_t H = c->hidden, I = c->inter, QKS = (uint64_t)c->heads * c->head_dim, KV = (uint64_t)c->kv_heads * c->head_dim, V = c->vocab;
        const uint32_t wt = c->wdtype;
        uint8_t* p = out_host;
        int32_t rc;
    #define FH_STEP(call, bytes) do { rc = (call); if (rc) return rc; p += (bytes); } while (0)
        // the embedding table is always f32 in the blob (main.rs:2690-2722)
        FH_STEP(write_f32(g, "token_embd.weight", V * H, p), V * H * 4);
        for (uint32_t l = 0; l < c->layers; l++) {
            FH_STEP(write_f32(g, blk(l, "attn_norm.weight"), H, p), H * 4);
            if (!g->tensor(blk(l, "attn_q.weight")) && g->tensor(blk(l, "attn_qkv.weight"))) {
                // Phi-3: Q|K|V rows in one tensor (weight_loader.rs:425-427, 552-567)
                const uint64_t all = (QKS + 2 * KV) * H;
                FH_STEP(write_quantised_part(g, blk(l, "attn_qkv.weight"), wt, all, 0, QKS * H, p), qbytes(wt, QKS * H));
                FH_STEP(write_quantised_part(g, blk(l, "attn_qkv.weight"), wt, all, QKS * H, KV * H, p), qbytes(wt, KV * H));
                FH_STEP(write_quantised_part(g, blk(l, "attn_qkv.weight"), wt, all, (QKS + KV) * H, KV * H, p), qbytes(wt, KV * H));
            } else {
                FH_STEP(write_quantised(g, blk(l, "attn_q.weight"), wt, QKS * H, p), qbytes(wt, QKS * H));
                FH_STEP(write_quantised(g, blk(l, "attn_k.weight"), wt, KV * H, p), qbytes(wt, KV * H));
                FH_STEP(write_quantised(g, blk(l, "attn_v.weight"), wt, KV * H, p), qbytes(wt, KV * H));
            }
            if (c->flags & FORGE_HIP_FLAG_QKV_BIAS) {             // main.rs:2737-2742
                FH_STEP(write_f32(g, blk(l, "attn_q.bias"), QKS, p), QKS * 4);
                FH_STEP(write_f32(g, blk(l, "attn_k.bias"), KV, p), KV * 4);
                FH_STEP(write_f32(g, blk(l, "attn_v.bias"), KV, p), KV * 4);
            }
            FH_STEP(write_quantised(g, blk(l, "attn_output.weight"), wt, H * QKS, p), qbytes(wt, H * QKS));
            FH_STEP(write_f32(g, blk(l, "ffn_norm.weight"), H, p), H * 4);
            const TensorInfo* up = g->tensor(blk(l, "ffn_up.weight"));
            if (!g->tensor(blk(l, "ffn_gate.weight")) && up && up->numel() == 2 * I * H) {
                // Phi-3: gate|up rows in one tensor (weight_loader.rs:569-580)
                FH_STEP(write_quantised_part(g, blk(l, "ffn_up.weight"), wt, 2 * I * H, 0, I * H, p), qbytes(wt, I * H));
                FH_STEP(write_quantised_part(g, blk(l, "ffn_up.weight"), wt, 2 * I * H, I * H, I * H, p), qbytes(wt, I * H));
            } else {
                FH_STEP(write_quantised(g, blk(l, "ffn_gate.weight"), wt, I * H, p), qbytes(wt, I * H));
                FH_STEP(write_quantised(g, blk(l, "ffn_up.weight"), wt, I * H, p), qbytes(wt, I * H));
            }
            FH_STEP(write_quantised(g, blk(l, "ffn_down.weight"), wt, H * I, p), qbytes(wt, H * I));
        }
        FH_STEP(write_f32(g, "output_norm.weight", H, p), H * 4);
        // lm_head: output.weight, or the embedding table of a model with tied weights (main.rs:2632-2676)
        const char* lm_name = g->tensor("output.weight") ? "output.weight" : g->tensor("lm_head.weight") ? "lm_head.weight" : "token_embd.weight";
        FH_STEP(write_quantised(g, lm_name, c->lm_head_dtype, V * H, p), qbytes(c->lm_head_dtype, V * H));
    #undef FH_STEP
        if ((uint64_t)(p - out_host) != need) return fh::fail(FORGE_HIP_ERR_INVALID, "gguf_export_weights: internal size mismatch");
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_quantize_kquant(uint32_t ggml_type, const float* data_host, uint64_t n, uint8_t* out_host) {
    return no_throw("quantize_kquant", [&]() -> int32_t {
        FH_CHECK(ggml_type == FORGE_HIP_Q4_K || ggml_type == FORGE_HIP_Q6_K, "quantize_kquant: the type must be Q4_K (12) or Q6_K (14)");
        FH_CHECK(out_host && (data_host || n == 0), "quantize_kquant: null pointer");
        if (ggml_type == FORGE_HIP_Q4_K) quantize_q4_k(data_host, n, out_host);
        else quantize_q6_k(data_host, n, out_host);
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_gguf_config_mixed(const forge_hip_gguf* g, uint32_t max_seq, uint32_t flags, forge_hip_config* out, uint32_t* proj_dtypes,
                                    uint32_t* embed_dtype) {
    return no_throw("gguf_config_mixed", [&]() -> int32_t {
        FH_CHECK(g && out && proj_dtypes, "gguf_config_mixed: null argument");
        forge_hip_config c{};
        uint32_t majority = 0;
        const int32_t brc = config_base(g, max_seq, flags, &c, &majority);
        if (brc) return brc;
        if (!majority) return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: the projection weights are neither mostly Q8_0, Q4_0 nor Q4_K");
        uint32_t cat[C_COUNT];
        detect_categories(g, majority, cat);
        if (embed_dtype) *embed_dtype = cat[C_EMBED];
        // The blob keeps the embedding table as f32 whatever the file holds (main.rs:2690-2722).  A dense projection category or a
        // dense lm_head is stored in the majority format here, as the uniform export does (the reference would keep f32 weights
        // and run its f32 dot product, which this library does not carry).
        const uint32_t dense_as = majority == FORGE_HIP_Q4_K ? (uint32_t)FORGE_HIP_Q8_0 : majority;
        for (int i = C_Q; i <= C_LM; i++) if (cat[i] == DENSE) cat[i] = dense_as;
        for (int i = 0; i < 7; i++) proj_dtypes[i] = cat[C_Q + i];
        c.wdtype = (majority == FORGE_HIP_Q8_0 || majority == FORGE_HIP_Q4_0) ? majority : (uint32_t)FORGE_HIP_Q8_0;
        c.lm_head_dtype = cat[C_LM];
        *out = c;
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_gguf_export_weights_mixed(const forge_hip_gguf* g, const forge_hip_config* c, const uint32_t* pd, uint8_t* out_host,
                                            uint64_t nbytes) {
    return no_throw("gguf_export_weights_mixed", [&]() -> int32_t {
        FH_CHECK(g && c && pd && out_host, "gguf_export_weights_mixed: null argument");
        const uint64_t need = forge_hip_weights_nbytes_mixed(c, pd);
        if (need == 0 || nbytes != need)
            return fh::fail(FORGE_HIP_ERR_BLOB_SIZE, "gguf_export_weights_mixed: buffer is " + std::to_string(nbytes) + " bytes, config needs " + std::to_string(need));
        const uint64_t H = c->hidden, I = c->inter, QKS = (uint64_t)c->heads * c->head_dim, KV = (uint64_t)c->kv_heads * c->head_dim, V = c->vocab;
        auto known = [](uint32_t d) { return d == FORGE_HIP_Q8_0 || d == FORGE_HIP_Q4_0 || d == FORGE_HIP_Q4_K || d == FORGE_HIP_Q6_K; };
        for (int i = 0; i < 7; i++) FH_CHECK(known(pd[i]), "gguf_export_weights_mixed: a projection's format must be Q8_0, Q4_0, Q4_K or Q6_K");
        FH_CHECK(known(c->lm_head_dtype), "gguf_export_weights_mixed: lm_head_dtype must be Q8_0, Q4_0, Q4_K or Q6_K");
        FH_CHECK(H % 32 == 0 && I % 32 == 0 && QKS % 32 == 0, "gguf_export_weights_mixed: row lengths must be multiples of 32");
        uint8_t* p = out_host;
        int32_t rc;
    #define FH_STEP(call, bytes) do { rc = (call); if (rc) return rc; p += (bytes); } while (0)
        {
            // the per-tensor loader keeps a Q4_K / Q6_K embedding table in its own format, and the exporter dequantises that
            // directly (main.rs:2697-2712); every other type goes the way of the uniform export
            Source e;
            rc = locate(g, "token_embd.weight", V * H, &e);
            if (rc) return rc;
            if (e.t->type == 12 || e.t->type == 14) dequant_ggml(e.t->type, e.bytes, V * H, reinterpret_cast<float*>(p));
            else if ((rc = write_f32(g, "token_embd.weight", V * H, p))) return rc;
            p += V * H * 4;
        }
        for (uint32_t l = 0; l < c->layers; l++) {
            if (!g->tensor(blk(l, "attn_q.weight")) || !g->tensor(blk(l, "ffn_gate.weight")))
                return fh::fail(FORGE_HIP_ERR_INVALID, "gguf: fused attn_qkv / gate-up tensors are split for uniformly Q8_0 / Q4_0 files only");
            FH_STEP(write_f32(g, blk(l, "attn_norm.weight"), H, p), H * 4);
            FH_STEP(write_in_format(g, blk(l, "attn_q.weight"), pd[0], QKS * H, p), qbytes_any(pd[0], QKS * H));
            FH_STEP(write_in_format(g, blk(l, "attn_k.weight"), pd[1], KV * H, p), qbytes_any(pd[1], KV * H));
            FH_STEP(write_in_format(g, blk(l, "attn_v.weight"), pd[2], KV * H, p), qbytes_any(pd[2], KV * H));
            if (c->flags & FORGE_HIP_FLAG_QKV_BIAS) {      // main.rs:2737-2742
                FH_STEP(write_f32(g, blk(l, "attn_q.bias"), QKS, p), QKS * 4);
                FH_STEP(write_f32(g, blk(l, "attn_k.bias"), KV, p), KV * 4);
                FH_STEP(write_f32(g, blk(l, "attn_v.bias"), KV, p), KV * 4);
            }
            FH_STEP(write_in_format(g, blk(l, "attn_output.weight"), pd[3], H * QKS, p), qbytes_any(pd[3], H * QKS));
            FH_STEP(write_f32(g, blk(l, "ffn_norm.weight"), H, p), H * 4);
            FH_STEP(write_in_format(g, blk(l, "ffn_gate.weight"), pd[4], I * H, p), qbytes_any(pd[4], I * H));
            FH_STEP(write_in_format(g, blk(l, "ffn_up.weight"), pd[5], I * H, p), qbytes_any(pd[5], I * H));
            FH_STEP(write_in_format(g, blk(l, "ffn_down.weight"), pd[6], H * I, p), qbytes_any(pd[6], H * I));
        }
        FH_STEP(write_f32(g, "output_norm.weight", H, p), H * 4);
        const char* lm_name = g->tensor("output.weight") ? "output.weight" : g->tensor("lm_head.weight") ? "lm_head.weight" : "token_embd.weight";
        FH_STEP(write_in_format(g, lm_name, c->lm_head_dtype, V * H, p), qbytes_any(c->lm_head_dtype, V * H));
    #undef FH_STEP
        if ((uint64_t)(p - out_host) != need) return fh::fail(FORGE_HIP_ERR_INVALID, "gguf_export_weights_mixed: internal size mismatch");
        return FORGE_HIP_OK;
    });
}

int32_t forge_hip_model_create_from_gguf(const char* path, uint32_t max_seq, uint32_t flags, forge_hip_model** out) {
    return no_throw("model_create_from_gguf", [&]() -> int32_t {
        FH_CHECK(out, "model_create_from_gguf: null out");
        *out = nullptr;
        forge_hip_gguf* g = nullptr;
        int32_t rc = forge_hip_gguf_open(path, &g);
        if (rc) return rc;
        std::unique_ptr<forge_hip_gguf> hold(g);
        forge_hip_config c;
        uint32_t pd[7];
        rc = forge_hip_gguf_config_mixed(g, max_seq, flags, &c, pd, nullptr);
        if (rc) return rc;
        bool uniform = c.lm_head_dtype == FORGE_HIP_Q8_0 || c.lm_head_dtype == FORGE_HIP_Q4_0;
        for (int i = 0; i < 7; i++) uniform = uniform && pd[i] == c.wdtype;
        if (uniform) {
            // every projection in the majority format, Q8_0 or Q4_0: the export and the model of the uniform case
            rc = forge_hip_gguf_config(g, max_seq, flags, &c);
            if (rc) return rc;
        }
        const uint64_t n = uniform ? forge_hip_weights_nbytes(&c) : forge_hip_weights_nbytes_mixed(&c, pd);
        if (n == 0) return fh::fail(FORGE_HIP_ERR_INVALID, "model_create_from_gguf: the configuration's weight size does not fit 64 bits");
        std::unique_ptr<uint8_t[]> blob(new (std::nothrow) uint8_t[n]);
        if (!blob) return fh::fail(FORGE_HIP_ERR_INVALID, "model_create_from_gguf: out of host memory for " + std::to_string(n) + " bytes");
        rc = uniform ? forge_hip_gguf_export_weights(g, &c, blob.get(), n) : forge_hip_gguf_export_weights_mixed(g, &c, pd, blob.get(), n);
        if (rc) return rc;
        return uniform ? forge_hip_model_create(&c, blob.get(), n, out) : forge_hip_model_create_mixed(&c, pd, blob.get(), n, out);
    });
}

}  // extern "C"

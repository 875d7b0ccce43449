// The sampler of the generated main.rs (crates/forgellm-codegen-cpu/src/project.rs:505-555), host code: what a caller
// that samples with a temperature runs on the logits `forge_hip_forward` hands back.  Every f32 operation is done in the
// reference's order (sequential sums, one division per element), `exp` is the C library's expf.
#include <math.h>

#include <algorithm>
#include <numeric>

#include "common.h"

extern "C" {

// apply_repeat_penalty, project.rs:505-513: once per entry of `recent`, in order.
int32_t forge_hip_apply_repeat_penalty(float* logits_host, uint64_t n, const uint32_t* recent_host, uint64_t n_recent, float penalty) {
    FH_CHECK(logits_host && (recent_host || n_recent == 0), "apply_repeat_penalty: null pointer");
    if (penalty <= 1.0f) return FORGE_HIP_OK;
    for (uint64_t k = 0; k < n_recent; k++) {
        const uint64_t idx = recent_host[k];
        if (idx < n) {
            if (logits_host[idx] > 0.0f) logits_host[idx] /= penalty;
            else logits_host[idx] *= penalty;
        }
    }
    return FORGE_HIP_OK;
}

// sample, project.rs:515-555.  `logits_host` is overwritten like the reference's `&mut [f32]` (it ends up holding the
// final probabilities).  temperature <= 0 returns the last maximum (argmax, project.rs:501-503) and leaves the
// state alone.  A NaN makes the reference panic (`partial_cmp().unwrap()`): FORGE_HIP_ERR_INVALID here.
// Equal probabilities: the reference sorts with `sort_unstable_by`, whose order among equal keys is unspecified;
// here the lower index comes first.
int32_t forge_hip_sample(float* logits_host, uint64_t n, float temperature, uint64_t top_k, float top_p, uint64_t* rng_state,
                         uint32_t* out) {
    FH_CHECK(logits_host && rng_state && out, "sample: null pointer");
    FH_CHECK(n >= 1 && n <= 0xFFFFFFFFull, "sample: the number of logits must be in 1 .. 2^32-1");
    float* l = logits_host;
    for (uint64_t i = 0; i < n; i++) FH_CHECK(l[i] == l[i], "sample: a logit is NaN");
    if (temperature <= 0.0f) {
        uint64_t best = 0;
        for (uint64_t i = 1; i < n; i++) if (l[i] >= l[best]) best = i;        // max_by keeps the last maximum
        *out = (uint32_t)best;
        return FORGE_HIP_OK;
    }
    for (uint64_t i = 0; i < n; i++) l[i] /= temperature;
    float max_val = -INFINITY;
    for (uint64_t i = 0; i < n; i++) max_val = fmaxf(max_val, l[i]);
    float sum = 0.0f;
    for (uint64_t i = 0; i < n; i++) l[i] = l[i] - max_val;
    (void)forge_hip_expf_host(l, n, l);                     // f32::exp = the C library's expf
    for (uint64_t i = 0; i < n; i++) sum += l[i];
    for (uint64_t i = 0; i < n; i++) l[i] /= sum;
    for (uint64_t i = 0; i < n; i++) FH_CHECK(l[i] == l[i], "sample: a probability is NaN");
    const bool need_order = (top_k > 0 && top_k < n) || (top_p > 0.0f && top_p < 1.0f);
    if (need_order) {
        std::vector<uint32_t> idx(n);
        std::iota(idx.begin(), idx.end(), 0u);
        std::stable_sort(idx.begin(), idx.end(), [l](uint32_t a, uint32_t b) { return l[a] > l[b]; });
        if (top_k > 0 && top_k < n)
            for (uint64_t k = top_k; k < n; k++) l[idx[k]] = 0.0f;
        if (top_p > 0.0f && top_p < 1.0f) {
            float cumsum = 0.0f;
            for (uint64_t k = 0; k < n; k++) {
                cumsum += l[idx[k]];
                if (cumsum > top_p) l[idx[k]] = 0.0f;       // the entry that crosses the threshold goes too (project.rs:535-540)
            }
        }
    }
    sum = 0.0f;
    for (uint64_t i = 0; i < n; i++) sum += l[i];
    if (sum > 0.0f)
        for (uint64_t i = 0; i < n; i++) l[i] /= sum;
    uint64_t s = *rng_state;                                  // xorshift64, project.rs:545-547
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    *rng_state = s;
    const float r = (float)s / (float)UINT64_MAX;
    float cumsum = 0.0f;
    for (uint64_t i = 0; i < n; i++) {
        cumsum += l[i];
        if (cumsum >= r) { *out = (uint32_t)i; return FORGE_HIP_OK; }
    }
    *out = (uint32_t)(n - 1);
    return FORGE_HIP_OK;
}

}  // extern "C"

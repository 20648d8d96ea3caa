// Host-side logit sampling for the non-greedy branch of forward_token: soft
// cap, temperature, min-p filter, one multinomial draw.
//
// Mirrors sample_softcap_min_p (crates/ksearch_gemma/src/sample.rs:9-77)
// operation for operation on f32 logits (the reference reads them as f16): the
// same pass structure, the same f32 accumulators, the same splitmix32 draw, so
// that a seed picks the same id.
#include <cmath>
#include <vector>

#include "ksh_internal.hpp"

namespace {

// sample.rs:79-85
uint32_t splitmix32(uint32_t &state)
{
    state += 0x9E3779B9u;
    uint32_t z = state;
    z = (z ^ (z >> 16)) * 0x7feb352du;
    z = (z ^ (z >> 15)) * 0x846ca68bu;
    return z ^ (z >> 16);
}

}  // namespace

extern "C" int ksh_sample_softcap_min_p(const float *logits, size_t n, float cap, float temperature, float min_p, uint32_t seed,
                                        uint32_t *out)
{
    using namespace ksh;
    if (!logits || !n || !out) return set_error("ksh_sample_softcap_min_p: bad arguments");
    uint32_t best_i = 0;
    float best_v = -INFINITY;
    std::vector<float> xs(n);
    for (size_t i = 0; i < n; i++) {
        const float x = logits[i];
        const float y = cap > 0.0f ? cap * std::tanh(x / cap) : x;
        xs[i] = y;
        if (y > best_v) { best_v = y; best_i = (uint32_t)i; }
    }
    *out = best_i;
    if (temperature < 1e-6f) return 0;   // greedy: argmax after the soft cap, lowest index on ties
    float sum = 0.0f;
    for (float &x : xs) {
        x = std::exp((x - best_v) / temperature);
        sum += x;
    }
    const float inv = 1.0f / std::fmax(sum, 1e-30f);
    float p_max = 0.0f;
    for (float &x : xs) {
        x *= inv;
        if (x > p_max) p_max = x;
    }
    const float threshold = p_max * std::fmax(min_p, 0.0f);
    float filtered = 0.0f;
    for (float &x : xs) {
        if (x < threshold) x = 0.0f;
        else filtered += x;
    }
    if (filtered <= 1e-9f) return 0;
    uint32_t rng = seed | 1u;
    const float r = ((float)splitmix32(rng) / 4294967296.0f) * filtered;
    float cdf = 0.0f;
    for (size_t i = 0; i < n; i++) {
        cdf += xs[i];
        if (r < cdf) { *out = (uint32_t)i; return 0; }
    }
    *out = (uint32_t)(n - 1);
    return 0;
}

// CPU-side sampler of the reference (models/sampler.rs:14-130): greedy for
// temperature 0, else temperature scaling, softmax, and multinomial or top-p
// (nucleus) sampling.  The random number is an argument (`coin` in [0, 1)), so a
// caller with a seeded generator gets reproducible text.  Host only.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <vector>

#include "common.h"

using namespace wgml;

namespace {

// Sampler::sample_mult (models/sampler.rs:58-76)
uint32_t sample_mult(const float *p, uint32_t n, float coin) {
    float cdf = 0.0f;
    for (uint32_t i = 0; i < n; ++i) {
        cdf += p[i];
        if (coin < cdf) return i;
    }
    return n - 1;
}

// Sampler::sample_topp (models/sampler.rs:78-130)
uint32_t sample_topp(const float *p, uint32_t n, float topp, float coin) {
    // values below (1 - topp) / (n - 1) cannot be part of the nucleus
    const float cutoff = (1.0f - topp) / ((float)n - 1.0f);
    std::vector<uint32_t> idx;
    idx.reserve(256);
    for (uint32_t i = 0; i < n; ++i)
        if (p[i] >= cutoff) idx.push_back(i);
    if (idx.empty()) return n - 1;
    // decreasing probability; ties keep their index order (the reference's sort is stable)
    std::stable_sort(idx.begin(), idx.end(), [p](uint32_t a, uint32_t b) { return p[a] > p[b]; });
    float cumulative = 0.0f;
    size_t last = idx.size() - 1;  // in case of rounding errors consider all elements
    for (size_t i = 0; i < idx.size(); ++i) {
        cumulative += p[idx[i]];
        if (cumulative > topp) {
            last = i;
            break;
        }
    }
    const float r = coin * cumulative;
    float cdf = 0.0f;
    for (size_t i = 0; i <= last; ++i) {
        cdf += p[idx[i]];
        if (r < cdf) return idx[i];
    }
    return idx[last];
}

}  // namespace

extern "C" {

int wgml_sample(float *logits, uint32_t n, float temperature, float topp, float coin,
                uint32_t *out_token) {
    WGML_REQUIRE(logits && out_token && n > 0, "wgml_sample: bad argument");
    WGML_REQUIRE(temperature >= 0.0f, "wgml_sample: negative temperature %g", (double)temperature);
    WGML_REQUIRE(coin >= 0.0f && coin < 1.0f, "wgml_sample: coin %g outside [0, 1)", (double)coin);
    if (temperature == 0.0f) {  // Sampler::sample_argmax: first index of the maximum
        uint32_t best = 0;
        for (uint32_t i = 1; i < n; ++i)
            if (logits[i] > logits[best]) best = i;
        *out_token = best;
        return WGML_OK;
    }
    for (uint32_t i = 0; i < n; ++i) logits[i] /= temperature;
    // SoftMax::run_cpu (ops/softmax.rs:36-49)
    float max_val = logits[0];
    for (uint32_t i = 1; i < n; ++i) max_val = std::max(max_val, logits[i]);
    float sum = 0.0f;
    for (uint32_t i = 0; i < n; ++i) {
        logits[i] = std::exp(logits[i] - max_val);
        sum += logits[i];
    }
    for (uint32_t i = 0; i < n; ++i) logits[i] /= sum;
    *out_token = (topp <= 0.0f || topp >= 1.0f) ? sample_mult(logits, n, coin)
                                                : sample_topp(logits, n, topp, coin);
    return WGML_OK;
}

}  // extern "C"

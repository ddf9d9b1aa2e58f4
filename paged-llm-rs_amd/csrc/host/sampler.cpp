#include "sampler.hpp"

#include <algorithm>
#include <cmath>
#include <vector>

namespace pl {

uint64_t Rng::next_u64() {
    state += 0x9E3779B97F4A7C15ULL;
    uint64_t z = state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

float Rng::next_f32() { return static_cast<float>(next_u64() >> 40) / 16777216.0f; }

const char* sampling_problem(float temperature, int has_top_k, long top_k, int has_top_p, float top_p) {
    if (!std::isfinite(temperature) || temperature < 0.f) return "temperature has to be zero or above";
    if (has_top_k && top_k <= 0) return "top_k 0 would leave no token to choose from";
    if (has_top_p && (!std::isfinite(top_p) || top_p <= 0.f || top_p > 1.f)) return "top_p has to sit in (0, 1]";
    return "";
}

uint32_t argmax(const float* logits, size_t count) {
    size_t best = 0;
    for (size_t i = 1; i < count; ++i)
        if (logits[i] > logits[best]) best = i;
    return static_cast<uint32_t>(best);
}

uint32_t sample(const Sampling& how, const float* logits, size_t count, Rng& rng) {
    if (how.greedy()) return argmax(logits, count);
    const float inverse = 1.0f / how.temperature;
    std::vector<std::pair<float, uint32_t>> candidates(count);
    for (size_t i = 0; i < count; ++i) candidates[i] = {logits[i] * inverse, static_cast<uint32_t>(i)};
    auto before = [](const std::pair<float, uint32_t>& a, const std::pair<float, uint32_t>& b) {
        return a.first > b.first || (a.first == b.first && a.second < b.second);
    };
    size_t keep = count;
    if (how.top_k > 0 && static_cast<size_t>(how.top_k) < count) {
        keep = static_cast<size_t>(how.top_k);
        std::partial_sort(candidates.begin(), candidates.begin() + keep, candidates.end(), before);
        candidates.resize(keep);
    } else {
        std::sort(candidates.begin(), candidates.end(), before);
    }
    const float largest = candidates[0].first;
    float total = 0.f;
    for (auto& c : candidates) {
        c.first = std::exp(c.first - largest);
        total += c.first;
    }
    if (how.top_p < 1.f) {
        const float target = how.top_p * total;
        float running = 0.f;
        size_t kept = 1;
        for (size_t i = 0; i < candidates.size(); ++i) {
            running += candidates[i].first;
            kept = i + 1;
            if (running >= target) break;  // the token that crosses the threshold is kept
        }
        candidates.resize(kept);
        total = 0.f;
        for (auto& c : candidates) total += c.first;
    }
    float point = rng.next_f32() * total;
    for (auto& c : candidates) {
        point -= c.first;
        if (point <= 0.f) return c.second;
    }
    return candidates.back().second;
}

}  // namespace pl

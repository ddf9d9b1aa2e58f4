// Picking the next token from a row of logits on the host
// (reference: crates/pagedllm/src/sampler.rs).
#pragma once

#include <cstddef>
#include <cstdint>

namespace pl {

// splitmix64 (sampler.rs:17-44): the same seed gives the same tokens anywhere.
struct Rng {
    uint64_t state;
    explicit Rng(uint64_t seed = 0) : state(seed) {}
    uint64_t next_u64();
    // A number in [0, 1) from the top 24 bits.
    float next_f32();
};

struct Sampling {
    float temperature = 0.f;  // 0: the largest logit, no draw
    int top_k = 0;            // 0: all
    float top_p = 1.f;        // 1: all
    bool greedy() const { return temperature <= 0.f; }
};

// Empty when the parameters are in range, else what is wrong (sampler.rs:72-95).
const char* sampling_problem(float temperature, int has_top_k, long top_k, int has_top_p, float top_p);

// The first maximum wins (sampler.rs:186-194).
uint32_t argmax(const float* logits, size_t count);

// Temperature, then top-k, then top-p, then one draw walked through the weights
// in descending order (sampler.rs:113-183).  Equal logits are ordered by id
// ascending, which the reference leaves open.  Greedy never moves the generator.
uint32_t sample(const Sampling& how, const float* logits, size_t count, Rng& rng);

}  // namespace pl

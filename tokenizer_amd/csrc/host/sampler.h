// Greedy and temperature / nucleus sampling on the host, with the reference's rules
// (qwen-infer/src/sample.rs:43-137) in float32, and the counter-based generator of uniform numbers:
// draw k of seed s is a function of (s, k) alone, so a sequence's draws do not depend on the batch.
#pragma once
#include <cstdint>

namespace ta {

uint64_t splitmix(uint64_t z);
// Uniform in [0, 1) with 24 bits: draw `counter` of the generator seeded with `seed`.
float uniform_f32(uint64_t seed, uint64_t counter);
// Lowest index among the maxima; NaN never wins; 0 if nothing is above -inf.  -1 for no logits.
int greedy_token(const float* logits, int64_t count);
// The draw for a given uniform number in [0, 1).  -1 no logits, -2 bad temperature, -3 bad top_p.
int sample_with_uniform(const float* logits, int64_t count, float temperature, float top_p, float uniform);

}  // namespace ta

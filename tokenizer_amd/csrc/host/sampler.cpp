#include "sampler.h"

#include <algorithm>
#include <cmath>
#include <limits>
#include <numeric>
#include <vector>

namespace ta {

uint64_t splitmix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

float uniform_f32(uint64_t seed, uint64_t counter) {
  const uint64_t key = splitmix(seed);
  const uint64_t bits = splitmix(key ^ splitmix(counter));
  return (float)((double)(bits >> 40) * (1.0 / (double)(1 << 24)));
}

int greedy_token(const float* logits, int64_t count) {
  if (count <= 0) return -1;
  const float neg_inf = -std::numeric_limits<float>::infinity();
  float best = neg_inf;
  int64_t at = 0;
  for (int64_t i = 0; i < count; ++i) {
    if (logits[i] > best) {                                 // false for NaN: a scan with `>` from -inf
      best = logits[i];
      at = i;
    }
  }
  return (int)at;
}

int sample_with_uniform(const float* logits, int64_t count, float temperature, float top_p, float uniform) {
  if (count <= 0) return -1;
  if (!std::isfinite(temperature) || temperature < 0) return -2;
  if (!std::isfinite(top_p) || top_p < 0) return -3;
  if (temperature == 0) return greedy_token(logits, count);
  float highest = -std::numeric_limits<float>::infinity();
  bool any_nan = false;
  for (int64_t i = 0; i < count; ++i) {
    if (std::isnan(logits[i])) any_nan = true;
    else highest = std::max(highest, logits[i]);
  }
  if (any_nan) return greedy_token(logits, count);        // a NaN weight makes every sum non-finite
  std::vector<float> weight(count);
  for (int64_t i = 0; i < count; ++i) {
    const float scaled = (logits[i] - highest) / temperature;
    weight[i] = (float)std::exp((double)scaled);
  }
  // Falling logit, the lower index first among equals (sample.rs:100-101).
  std::vector<int64_t> order(count);
  std::iota(order.begin(), order.end(), (int64_t)0);
  std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) { return logits[a] > logits[b]; });
  auto sequential_sum = [](const float* values, int64_t n, const int64_t* index) {
    float sum = 0.f;
    for (int64_t i = 0; i < n; ++i) sum += values[index ? index[i] : i];
    return sum;
  };
  int64_t cutoff = count;
  if (top_p < 1.0f) {
    const float total = sequential_sum(weight.data(), count, nullptr);
    if (total == 0 || !std::isfinite(total)) return greedy_token(logits, count);
    float cumulative = 0.f;
    for (int64_t i = 0; i < count; ++i) {
      cumulative += weight[order[i]] / total;
      if (cumulative >= top_p) {
        cutoff = i + 1;
        break;
      }
    }
  }
  const float kept_sum = sequential_sum(weight.data(), cutoff, order.data());
  if (kept_sum == 0 || !std::isfinite(kept_sum)) return greedy_token(logits, count);
  float threshold = uniform * kept_sum;
  for (int64_t i = 0; i < cutoff; ++i) {
    const float mass = weight[order[i]];
    if (threshold < mass) return (int)order[i];
    threshold -= mass;
  }
  return (int)order[cutoff - 1];
}

}  // namespace ta

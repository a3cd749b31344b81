#include "bpe_core.h"

#include <climits>
#include <cstring>

namespace ta {

int BpeCore::add_token(int32_t id, const uint8_t* bytes, int len, bool findable) {
  if (id < 0 || len < 0) return -1;
  if ((size_t)id < known_.size() && known_[id]) return -1;
  kept_.emplace_back(reinterpret_cast<const char*>(bytes), (size_t)len);
  const std::string_view view(kept_.back());
  if (findable && !id_of_.emplace(view, id).second) { kept_.pop_back(); return -1; }
  if ((size_t)id >= by_id_.size()) { by_id_.resize((size_t)id + 1); known_.resize((size_t)id + 1, 0); }
  by_id_[id] = view;
  known_[id] = 1;
  return 0;
}

int BpeCore::add_merge(const uint8_t* merged, int len, int rank) {
  if (len <= 0) return -1;
  kept_.emplace_back(reinterpret_cast<const char*>(merged), (size_t)len);
  if (!rank_of_.emplace(std::string_view(kept_.back()), rank).second) { kept_.pop_back(); return -1; }
  return 0;
}

int BpeCore::encode_piece(const uint8_t* piece, int len, int32_t* out, int capacity) const {
  if (len <= 0) return 0;
  const char* text = reinterpret_cast<const char*>(piece);
  // Parts as offsets into the piece: part i is [start[i], start[i + 1]).  rank[i]: the rank of joining part i with
  // part i + 1, or INT_MAX.  A join changes the ranks of the two pairs the new part belongs to, nothing else.
  std::vector<int> start(len + 1), rank(len, INT_MAX);
  for (int i = 0; i <= len; ++i) start[i] = i;
  int parts = len;
  auto pair_rank = [&](int i) {                      // of parts i and i + 1
    if (i < 0 || i + 1 >= parts) return INT_MAX;
    const auto found = rank_of_.find(std::string_view(text + start[i], (size_t)(start[i + 2] - start[i])));
    return found == rank_of_.end() ? INT_MAX : found->second;
  };
  for (int i = 0; i + 1 < parts; ++i) rank[i] = pair_rank(i);
  while (parts > 1) {
    int best = INT_MAX, at = -1;
    for (int i = 0; i + 1 < parts; ++i)
      if (rank[i] < best) { best = rank[i]; at = i; }                  // strictly lower: the leftmost of equals stays
    if (at < 0) break;
    start.erase(start.begin() + at + 1);                               // parts at and at + 1 become one
    rank.erase(rank.begin() + at);
    --parts;
    if (at < parts) rank[at] = pair_rank(at);
    if (at > 0) rank[at - 1] = pair_rank(at - 1);
  }
  if (parts > capacity) return -parts;
  for (int i = 0; i < parts; ++i) {
    const auto found = id_of_.find(std::string_view(text + start[i], (size_t)(start[i + 1] - start[i])));
    if (found == id_of_.end()) return INT32_MIN;
    out[i] = found->second;
  }
  return parts;
}

int64_t BpeCore::decode(const int32_t* ids, int count, uint8_t* out, int64_t capacity, int* bad_at) const {
  int64_t total = 0;
  for (int i = 0; i < count; ++i) {
    const int32_t id = ids[i];
    if (id < 0 || (size_t)id >= by_id_.size() || !known_[id]) {
      if (bad_at) *bad_at = i;
      return INT32_MIN;
    }
    total += (int64_t)by_id_[id].size();
  }
  if (total > capacity) return -total;
  for (int i = 0; i < count; ++i) {
    const std::string_view bytes = by_id_[ids[i]];
    std::memcpy(out, bytes.data(), bytes.size());
    out += bytes.size();
  }
  return total;
}

}  // namespace ta

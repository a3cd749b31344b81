// The inner loops of the byte-level BPE tokenizer: the merges inside one piece of text and the way back from ids
// to bytes (rules of src/rank.rs:485-514,536-586 and 192-204 of the reference).  What surrounds them (the
// tokenizer file, normalisation, the regex that cuts text into pieces, added tokens) stays with the caller.
#pragma once
#include <cstdint>
#include <deque>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

namespace ta {

class BpeCore {
 public:
  // A token's bytes under its id.  -1: the id is negative or taken, or the bytes are (an ordinary token's bytes
  // are unique; `findable` false for an added token, which is matched in the text before pieces are cut and
  // never comes out of a merge).
  int add_token(int32_t id, const uint8_t* bytes, int len, bool findable);
  // The rank of the merge that produces these bytes (a lower rank merges first).  -1 if they have one already.
  int add_merge(const uint8_t* merged, int len, int rank);
  int vocab_size() const { return (int)by_id_.size(); }

  // The ids of one piece: neighbouring parts are joined, lowest rank first and the leftmost of equal ranks, until
  // no neighbouring pair has a rank.  Returns how many ids were written, -(needed) if `capacity` is too small, or
  // INT32_MIN if some part is no token (a vocabulary without all single bytes).
  int encode_piece(const uint8_t* piece, int len, int32_t* out, int capacity) const;
  // The bytes of a run of ids.  Returns their number, -(needed) if `capacity` is too small; with an unknown id,
  // INT32_MIN and the index of the first one in *bad_at.
  int64_t decode(const int32_t* ids, int count, uint8_t* out, int64_t capacity, int* bad_at) const;

 private:
  std::deque<std::string> kept_;                                   // backs the views below
  std::unordered_map<std::string_view, int32_t> id_of_;
  std::unordered_map<std::string_view, int> rank_of_;
  std::vector<std::string_view> by_id_;
  std::vector<char> known_;
};

}  // namespace ta

// Host-side cross-tokenizer tables: a byte trie over the student vocabulary, the longest-prefix
// map teacher token -> student token, and its CSR form (student id -> teacher ids).
// Plain C++ on host memory; no GPU involved.  No reference counterpart.
#include "distill_hip.h"

#include <cstdint>
#include <cstring>
#include <unordered_map>
#include <vector>

namespace {

// Node 0 is the root.  Edges live in one hash map keyed by (node << 8 | byte); `owner[n]` is the
// smallest student id whose byte string ends at node n, or -1.
struct ByteTrie {
  std::unordered_map<uint64_t, int32_t> edge;
  std::vector<int32_t> owner{-1};

  void insert(const uint8_t* s, int64_t len, int32_t id) {
    int32_t node = 0;
    for (int64_t i = 0; i < len; ++i) {
      const uint64_t key = ((uint64_t)node << 8) | s[i];
      auto it = edge.find(key);
      if (it == edge.end()) {
        const int32_t fresh = (int32_t)owner.size();
        owner.push_back(-1);
        edge.emplace(key, fresh);
        node = fresh;
      } else {
        node = it->second;
      }
    }
    if (owner[node] < 0) owner[node] = id;      // ids arrive ascending: the smallest keeps the string
  }

  // Student id of the longest stored string that is a prefix of s[0..len), or -1.
  int32_t longest_prefix(const uint8_t* s, int64_t len) const {
    int32_t node = 0, best = -1;
    for (int64_t i = 0; i < len; ++i) {
      auto it = edge.find(((uint64_t)node << 8) | s[i]);
      if (it == edge.end()) break;
      node = it->second;
      if (owner[node] >= 0) best = owner[node];
    }
    return best;
  }
};

}  // namespace

extern "C" int dl_trie_longest_prefix_map(const uint8_t* student_bytes, const int64_t* student_offsets,
                                          int64_t n_student, const uint8_t* teacher_bytes,
                                          const int64_t* teacher_offsets, int64_t n_teacher,
                                          const int32_t* byte_fallback, int32_t* out_t2s) {
  if (!student_offsets || !teacher_offsets || !out_t2s) return DL_ERR_NULL;
  if (n_student < 0 || n_teacher < 0) return DL_ERR_SHAPE;
  if (n_student > 0x7fffffffLL || n_teacher > 0x7fffffffLL) return DL_ERR_LIMIT;
  for (int64_t i = 0; i < n_student; ++i)
    if (student_offsets[i + 1] < student_offsets[i]) return DL_ERR_SHAPE;
  for (int64_t i = 0; i < n_teacher; ++i)
    if (teacher_offsets[i + 1] < teacher_offsets[i]) return DL_ERR_SHAPE;
  if ((n_student > 0 && student_offsets[n_student] > 0 && !student_bytes) ||
      (n_teacher > 0 && teacher_offsets[n_teacher] > 0 && !teacher_bytes))
    return DL_ERR_NULL;
  ByteTrie trie;
  trie.edge.reserve((size_t)(n_student > 0 ? student_offsets[n_student] : 0) + 16);
  for (int64_t i = 0; i < n_student; ++i) {
    const int64_t len = student_offsets[i + 1] - student_offsets[i];
    if (len > 0) trie.insert(student_bytes + student_offsets[i], len, (int32_t)i);
  }
  for (int64_t t = 0; t < n_teacher; ++t) {
    const int64_t len = teacher_offsets[t + 1] - teacher_offsets[t];
    int32_t hit = -1;
    if (len > 0) {
      const uint8_t* s = teacher_bytes + teacher_offsets[t];
      hit = trie.longest_prefix(s, len);
      if (hit < 0 && byte_fallback && byte_fallback[s[0]] >= 0 && byte_fallback[s[0]] < n_student)
        hit = byte_fallback[s[0]];
    }
    out_t2s[t] = hit;
  }
  return DL_OK;
}

extern "C" int dl_csr_from_map(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int32_t* offsets,
                               int32_t* indices, int64_t* n_mapped) {
  if (!t2s || !offsets || !indices) return DL_ERR_NULL;
  if (n_teacher < 0 || n_student < 0) return DL_ERR_SHAPE;
  if (n_teacher > 0x7fffffffLL || n_student > 0x7ffffffeLL) return DL_ERR_LIMIT;
  std::memset(offsets, 0, (size_t)(n_student + 1) * sizeof(int32_t));
  for (int64_t t = 0; t < n_teacher; ++t) {
    const int32_t s = t2s[t];
    if (s >= n_student) return DL_ERR_SHAPE;
    if (s >= 0) ++offsets[s + 1];
  }
  for (int64_t s = 0; s < n_student; ++s) offsets[s + 1] += offsets[s];
  std::vector<int32_t> cursor(offsets, offsets + n_student);
  for (int64_t t = 0; t < n_teacher; ++t) {          // ascending t keeps every segment sorted
    const int32_t s = t2s[t];
    if (s >= 0) indices[cursor[s]++] = (int32_t)t;
  }
  if (n_mapped) *n_mapped = offsets[n_student];
  return DL_OK;
}

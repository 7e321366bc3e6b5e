// Host-side cross-tokenizer tables: a byte trie over the student vocabulary, the longest-prefix
// map teacher token -> student token, and its CSR form (student id -> teacher ids).
// Plain C++ on host memory; no GPU involved.  No reference counterpart.
#include "distill_hip.h"

#include <cstdint>
#include <algorithm>
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

// ---- marginalisation plan --------------------------------------------------------------------
// Layout consumed by the planned marginalisation kernels (1024 threads = 16 waves per workgroup):
// the teacher vocabulary is cut into tiles of `tile` ids; student id s is owned by thread s % 1024;
// for tile k and wave w, rows row_off[k*16 + w] .. row_off[k*16 + w + 1] of `ent` hold, 64 entries
// per row (one per lane, 0xffffffff = padding), the entries (s << log2(tile) | t - k*tile) of the
// wave's threads, each thread's entries sorted by (s, t).
extern "C" int dl_marginal_plan_build(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int* tile_out,
                                      int32_t* row_off, uint32_t* ent, int64_t ent_rows_capacity,
                                      int64_t* ent_rows_out) {
  constexpr int NT = 1024, WAVE = 64, NW = NT / WAVE;
  constexpr int64_t LDS_BUDGET = 160 * 1024 - 1024;      // dynamic LDS one workgroup may use
  if (!t2s || !tile_out || !ent_rows_out) return DL_ERR_NULL;
  if (n_teacher <= 0 || n_student <= 0) return DL_ERR_SHAPE;
  if (n_teacher > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int64_t marg_bytes = ((n_student + 3) & ~(int64_t)3) * 4;
  int tile = 8192;
  while (tile >= 4096 && marg_bytes + (int64_t)tile * 4 > LDS_BUDGET) tile >>= 1;
  if (tile < 4096) return DL_ERR_LIMIT;                  // marginal + smallest tile do not fit the LDS
  int tile_bits = 0;
  while ((1 << tile_bits) < tile) ++tile_bits;
  if (n_student >= (1LL << (32 - tile_bits)) - 1) return DL_ERR_LIMIT;
  *tile_out = tile;
  const int64_t ntiles = (n_teacher + tile - 1) / tile;
  std::vector<std::vector<uint32_t>> bucket(NT);
  int64_t rows = 0;
  if (row_off) row_off[0] = 0;
  for (int64_t k = 0; k < ntiles; ++k) {
    for (auto& b : bucket) b.clear();
    const int64_t t0 = k * tile, t1 = std::min<int64_t>(n_teacher, t0 + tile);
    for (int64_t t = t0; t < t1; ++t) {
      const int32_t sid = t2s[t];
      if (sid >= n_student) return DL_ERR_SHAPE;
      if (sid >= 0) bucket[sid % NT].push_back(((uint32_t)sid << tile_bits) | (uint32_t)(t - t0));
    }
    for (auto& b : bucket) std::sort(b.begin(), b.end());      // (s, t) ascending: s in the high bits
    for (int w = 0; w < NW; ++w) {
      size_t longest = 0;
      for (int l = 0; l < WAVE; ++l) longest = std::max(longest, bucket[w * WAVE + l].size());
      if (ent) {
        if (rows + (int64_t)longest > ent_rows_capacity) return DL_ERR_SHAPE;
        for (size_t j = 0; j < longest; ++j)
          for (int l = 0; l < WAVE; ++l) {
            const auto& b = bucket[w * WAVE + l];
            ent[(rows + (int64_t)j) * WAVE + l] = j < b.size() ? b[j] : 0xffffffffu;
          }
      }
      rows += (int64_t)longest;
      if (rows > 0x7fffffffLL) return DL_ERR_LIMIT;
      if (row_off) row_off[k * NW + w + 1] = (int32_t)rows;
    }
  }
  *ent_rows_out = rows;
  return DL_OK;
}

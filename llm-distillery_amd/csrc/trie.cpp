// Host-side cross-tokenizer tables: a byte trie over the student vocabulary, the longest-prefix
// map teacher token -> student token, and its CSR form (student id -> teacher ids).
// Plain C++ on host memory; no GPU involved.  No reference counterpart.
#include "distill_hip.h"

#include <cstdint>
#include <algorithm>
#include <cstring>
#include <unordered_map>
#include <utility>
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
// Layout consumed by the planned marginalisation kernels (1024 threads = 16 waves per workgroup).
// Every accumulator word in LDS is touched by one thread only, so no atomics are needed and the
// summation order is fixed.  Accumulator slots: slot s < n_student is student id s; a student id
// that receives far more teacher ids than an even share (real vocabularies: the single-byte and
// other short tokens) gets extra slots n_student_padded + j ("replicas") so that its load can be
// split over several threads; after the last tile the replicas are folded into their id's slot in
// a fixed order (fold table: triples id, first replica slot, replica count).  Slots are dealt to
// threads by descending load onto the least-loaded thread; inside a tile an entry of a replicated
// id goes to the replica whose owner holds the fewest entries of that tile so far.
// The teacher vocabulary is cut into tiles of `tile` ids; for tile k and wave w, rows
// row_off[k*16 + w] .. row_off[k*16 + w + 1] of `ent` hold, 64 entries per row (one per lane), the
// entries (slot << log2(tile) | t - k*tile) of the wave's threads, each thread's entries sorted by
// (slot, t); bit 31 marks the first entry of a slot in the thread's list, bit 30 the last one, and
// 0x80000000 (a first entry that never ends) is padding.
extern "C" int dl_marginal_plan_build(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int* tile_out,
                                      int32_t* row_off, uint32_t* ent, int64_t ent_rows_capacity,
                                      int64_t* ent_rows_out, int32_t* fold, int64_t fold_capacity,
                                      int64_t* n_fold_out, int* n_extra_out) {
  constexpr int NT = 1024, WAVE = 64, NW = NT / WAVE;
  constexpr uint32_t FIRST = 0x80000000u, LAST = 0x40000000u, PAD = FIRST;
  constexpr int64_t LDS_BUDGET = 160 * 1024 - 1024;      // dynamic LDS one workgroup may use
  if (!t2s || !tile_out || !ent_rows_out || !n_fold_out || !n_extra_out) return DL_ERR_NULL;
  if (n_teacher <= 0 || n_student <= 0) return DL_ERR_SHAPE;
  if (n_teacher > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int64_t n_pad = (n_student + 3) & ~(int64_t)3;
  const int64_t marg_bytes = n_pad * 4;
  int tile = 8192;
  while (tile >= 4096 && marg_bytes + (int64_t)tile * 4 > LDS_BUDGET) tile >>= 1;
  if (tile < 4096) return DL_ERR_LIMIT;                  // marginal + smallest tile do not fit the LDS
  int tile_bits = 0;
  while ((1 << tile_bits) < tile) ++tile_bits;
  *tile_out = tile;
  const int64_t ntiles = (n_teacher + tile - 1) / tile;

  // loads per student id
  std::vector<int64_t> count(n_student, 0);
  int64_t n_mapped = 0;
  for (int64_t t = 0; t < n_teacher; ++t) {
    const int32_t sid = t2s[t];
    if (sid >= n_student) return DL_ERR_SHAPE;
    if (sid >= 0) { ++count[sid]; ++n_mapped; }
  }
  // replicas: LDS words left beside the marginal and the tile, handed one at a time to the id with
  // the largest load per slot, down to a quarter of a thread's even share
  int64_t budget = ((LDS_BUDGET - marg_bytes - (int64_t)tile * 4) / 4) & ~(int64_t)3;
  const int64_t slot_limit = (1LL << (30 - tile_bits)) - 1;                 // slot ids must fit between the flags and the tile offset
  if (n_pad >= slot_limit) return DL_ERR_LIMIT;
  budget = std::min<int64_t>(budget, slot_limit - n_pad);
  const double share = (double)n_mapped / NT;
  std::vector<int32_t> reps(n_student, 1);
  {
    auto per_slot = [&](int32_t s) { return (double)count[s] / reps[s]; };
    auto worse = [&](int32_t a, int32_t b) { const double la = per_slot(a), lb = per_slot(b); return la != lb ? la < lb : a > b; };
    std::vector<int32_t> heap;
    for (int64_t s = 0; s < n_student; ++s)
      if ((double)count[s] > std::max(share / 4, 8.0)) heap.push_back((int32_t)s);
    std::make_heap(heap.begin(), heap.end(), worse);
    while (budget > 0 && !heap.empty()) {
      std::pop_heap(heap.begin(), heap.end(), worse);
      const int32_t s = heap.back();
      if (per_slot(s) <= std::max(share / 4, 8.0)) break;                   // the heaviest is light enough: done
      ++reps[s];
      --budget;
      std::push_heap(heap.begin(), heap.end(), worse);
    }
  }
  // slots: own slot of every id that is hit, plus the replicas; fold table in ascending id order
  struct Slot { int32_t slot; double load; };
  std::vector<Slot> slots;
  std::vector<int32_t> first_extra(n_student, -1);
  int64_t n_extra = 0, n_fold = 0;
  for (int64_t s = 0; s < n_student; ++s) {
    if (count[s] == 0) continue;
    const double load = (double)count[s] / reps[s];
    slots.push_back({(int32_t)s, load});
    if (reps[s] > 1) {
      first_extra[s] = (int32_t)(n_pad + n_extra);
      for (int j = 1; j < reps[s]; ++j) slots.push_back({(int32_t)(n_pad + n_extra + j - 1), load});
      if (fold) {
        if (n_fold >= fold_capacity) return DL_ERR_SHAPE;
        fold[3 * n_fold] = (int32_t)s; fold[3 * n_fold + 1] = first_extra[s]; fold[3 * n_fold + 2] = reps[s] - 1;
      }
      n_extra += reps[s] - 1;
      ++n_fold;
    }
  }
  *n_fold_out = n_fold;
  *n_extra_out = (int)n_extra;
  // owners: heaviest slot first onto the least-loaded thread (ties: lower thread number)
  std::stable_sort(slots.begin(), slots.end(), [](const Slot& a, const Slot& b) { return a.load > b.load; });
  std::vector<int32_t> owner(n_pad + n_extra, -1);
  {
    std::vector<std::pair<double, int>> th(NT);
    for (int i = 0; i < NT; ++i) th[i] = {0.0, i};
    auto heavier = [](const std::pair<double, int>& a, const std::pair<double, int>& b) { return a > b; };
    std::make_heap(th.begin(), th.end(), heavier);                          // min-heap on (load, thread)
    for (const Slot& sl : slots) {
      std::pop_heap(th.begin(), th.end(), heavier);
      owner[sl.slot] = th.back().second;
      th.back().first += sl.load;
      std::push_heap(th.begin(), th.end(), heavier);
    }
  }

  std::vector<std::vector<uint32_t>> bucket(NT);
  int64_t rows = 0;
  if (row_off) row_off[0] = 0;
  for (int64_t k = 0; k < ntiles; ++k) {
    for (auto& b : bucket) b.clear();
    const int64_t t0 = k * tile, t1 = std::min<int64_t>(n_teacher, t0 + tile);
    for (int64_t t = t0; t < t1; ++t) {
      const int32_t sid = t2s[t];
      if (sid < 0) continue;
      int32_t slot = sid;
      size_t best = bucket[owner[sid]].size();
      for (int j = 1; j < reps[sid]; ++j) {                                 // the replica whose owner is least busy in this tile
        const int32_t cand = first_extra[sid] + j - 1;
        const size_t sz = bucket[owner[cand]].size();
        if (sz < best) { best = sz; slot = cand; }
      }
      bucket[owner[slot]].push_back(((uint32_t)slot << tile_bits) | (uint32_t)(t - t0));
    }
    for (auto& b : bucket) std::sort(b.begin(), b.end());      // (slot, t) ascending: slot in the high bits
    for (int w = 0; w < NW; ++w) {
      size_t longest = 0;
      for (int l = 0; l < WAVE; ++l) longest = std::max(longest, bucket[w * WAVE + l].size());
      if (ent) {
        if (rows + (int64_t)longest > ent_rows_capacity) return DL_ERR_SHAPE;
        for (size_t j = 0; j < longest; ++j)
          for (int l = 0; l < WAVE; ++l) {
            const auto& b = bucket[w * WAVE + l];
            uint32_t e = PAD;
            if (j < b.size()) {
              e = b[j];
              if (j == 0 || (b[j - 1] >> tile_bits) != (b[j] >> tile_bits)) e |= FIRST;
              if (j + 1 == b.size() || (b[j + 1] >> tile_bits) != (b[j] >> tile_bits)) e |= LAST;
            }
            ent[(rows + (int64_t)j) * WAVE + l] = e;
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

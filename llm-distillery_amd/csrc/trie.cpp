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
// The teacher vocabulary is cut into tiles; the kernel stages one tile of probabilities in LDS at
// a time, with workgroup barriers between tiles.  Inside a tile every accumulator word ("slot") in
// LDS is touched by one thread only, so no atomics are needed and the summation order is fixed;
// from tile to tile a slot may change hands.  Slot s < n_student is student id s.  The entries of
// one id inside one tile are cut into pieces of at most PIECE entries (PIECE = the kernel's batch
// of 8 where the LDS allows); piece 0 goes to the id's own slot, piece j > 0 to replica slot
// first_extra[id] + j - 1 behind the padded marginal, so an id owns as many replicas as its
// busiest tile needs.  After the last tile the replicas are folded into their id's slot in a
// fixed order (fold table: triples id, first replica slot, replica count).  Inside a tile the
// pieces are dealt, largest first, onto the thread that holds the fewest entries so far: lists
// come out level, which matters because every wave of the workgroup waits for the longest one.
// The tile size is chosen among the multiples of 1024 ids from 8192 down to 4096: a smaller tile
// leaves more LDS for replicas (shorter lists when a few ids are very hot) but costs more barriers.
// For tile k and wave w, rows (row_off[k*16 + w] & ~3) .. (row_off[k*16 + w + 1] & ~3) of `ent` (64
// dwords per row) hold the entries of the wave's threads, each thread's entries sorted by (slot, t).
// Threads that hold at most one run in a tile are given the low thread numbers of that tile, the
// others the high ones, so most waves consist of one-run threads only.  Two list formats:
//   * general (bit 0 of row_off[k*16 + w] clear): batches of PLAN_BATCH entries per lane, 8 rows each,
//     lane-major (the entries of lane l are dwords [8l, 8l + 8) of the batch), at least one batch.  A
//     thread adds up a run of entries of one slot and stores slot + running sum after every entry, so
//     only the run's last entry may name the slot: bits 15-30 hold the slot there and the lane's spare
//     slot (behind the replicas, one per lane) on the other entries; bit 31 marks the first entry of a
//     run (the running sum restarts); bits 0-14 hold 4 * (t - k*tile), the byte offset inside the tile.
//     Padding is a first entry on the spare slot with offset 0; a thread's padding comes first and
//     its entries last.
//   * packed (bit 0 set; every lane holds at most one run of at most 8 entries): 4 rows, 4 dwords per
//     lane, lane-major.  A dword holds two 16-bit fields, the lane's entries in order from the low
//     field of dword 0 on; bits 2-15 of a field are the byte offset 4 * (t - k*tile), padding (first)
//     points at the zero words behind the tile, 4 * tile; the low two bits of the eight fields
//     together are the run's slot (the lane's spare slot if it has no entries): field 2j carries slot
//     bits 2j and 2j + 1, field 2j + 1 bits 8 + 2j and 9 + 2j.
namespace {

constexpr int PLAN_NT = 1024, PLAN_WAVE = 64, PLAN_NW = PLAN_NT / PLAN_WAVE;
constexpr int PLAN_BATCH = 8;                                 // entries per batch in the kernels
constexpr int64_t PLAN_LDS_BUDGET = 160 * 1024 - 1024 - 64 * 4 - 16;   // dynamic LDS one workgroup may use, less the spare slots and the zero words behind the tile
constexpr int PLAN_PACKED_ROWS = 4;                           // rows a packed list takes
constexpr int PLAN_SLOT_SHIFT = 15;

struct PlanLayout {
  int tile = 0, tile_bits = 0, piece = 0;
  int64_t ntiles = 0, n_pad = 0, n_extra = 0, n_fold = 0;
  std::vector<int32_t> first_extra;                           // per student id, -1: no replicas
  std::vector<int32_t> reps;                                  // slots per student id (own one included)
};

// Entries of tile k as (student id, t - k*tile), sorted by (id, t).
void tile_entries(const int32_t* t2s, int64_t n_teacher, const PlanLayout& L, int64_t k,
                  std::vector<std::pair<int32_t, int32_t>>& out) {
  out.clear();
  const int64_t t0 = k * L.tile, t1 = std::min<int64_t>(n_teacher, t0 + L.tile);
  for (int64_t t = t0; t < t1; ++t)
    if (t2s[t] >= 0) out.emplace_back(t2s[t], (int32_t)(t - t0));
  std::sort(out.begin(), out.end());
}

// Replica counts for a tile size: the smallest piece size >= PLAN_BATCH whose replicas fit the LDS
// left beside the marginal and the tile.  False: the tile does not fit at all.
bool plan_layout(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int tile, PlanLayout& L) {
  L = PlanLayout();
  L.tile = tile;
  while ((1 << L.tile_bits) < tile) ++L.tile_bits;
  L.ntiles = (n_teacher + tile - 1) / tile;
  L.n_pad = (n_student + 3) & ~(int64_t)3;
  const int64_t marg_bytes = L.n_pad * 4;
  if (marg_bytes + (int64_t)tile * 4 > PLAN_LDS_BUDGET) return false;
  int64_t budget = ((PLAN_LDS_BUDGET - marg_bytes - (int64_t)tile * 4) / 4) & ~(int64_t)3;
  const int64_t slot_limit = (1LL << 16) - PLAN_WAVE - 4;       // slot ids (the spare ones included) take 16 bits of an entry
  if (L.n_pad >= slot_limit) return false;
  budget = std::min<int64_t>(budget, slot_limit - L.n_pad);
  // busiest tile of every id
  std::vector<int32_t> busiest(n_student, 0), in_tile(n_student, 0);
  for (int64_t k = 0; k < L.ntiles; ++k) {
    const int64_t t0 = k * tile, t1 = std::min<int64_t>(n_teacher, t0 + tile);
    for (int64_t t = t0; t < t1; ++t)
      if (t2s[t] >= 0) ++in_tile[t2s[t]];
    for (int64_t t = t0; t < t1; ++t)
      if (t2s[t] >= 0) {
        busiest[t2s[t]] = std::max(busiest[t2s[t]], in_tile[t2s[t]]);
        in_tile[t2s[t]] = 0;
      }
  }
  auto extra_for = [&](int piece) {
    int64_t n = 0;
    for (int64_t s = 0; s < n_student; ++s)
      if (busiest[s] > piece) n += (busiest[s] + piece - 1) / piece - 1;
    return n;
  };
  int piece = PLAN_BATCH;
  while (extra_for(piece) > budget) piece += std::max(1, piece / 8);
  L.piece = piece;
  L.reps.assign(n_student, 1);
  L.first_extra.assign(n_student, -1);
  for (int64_t s = 0; s < n_student; ++s)
    if (busiest[s] > piece) {
      L.reps[s] = (busiest[s] + piece - 1) / piece;
      L.first_extra[s] = (int32_t)(L.n_pad + L.n_extra);
      L.n_extra += L.reps[s] - 1;
      ++L.n_fold;
    }
  return true;
}

// The lists of the 1024 threads for one tile (entries without flags, sorted per thread).
void plan_deal_tile(const PlanLayout& L, const std::vector<std::pair<int32_t, int32_t>>& entries,
                    std::vector<std::vector<uint32_t>>& bucket) {
  struct Piece { int32_t slot; int32_t first, count; };       // entries[first, first + count)
  std::vector<Piece> pieces;
  for (size_t i = 0; i < entries.size();) {
    size_t j = i;
    while (j < entries.size() && entries[j].first == entries[i].first) ++j;
    const int32_t sid = entries[i].first, c = (int32_t)(j - i);
    const int32_t n = (c + L.piece - 1) / L.piece, base = c / n, rem = c % n;
    int32_t at = (int32_t)i;
    for (int32_t q = 0; q < n; ++q) {
      const int32_t len = base + (q < rem ? 1 : 0);
      pieces.push_back({q == 0 ? sid : L.first_extra[sid] + q - 1, at, len});
      at += len;
    }
    i = j;
  }
  std::stable_sort(pieces.begin(), pieces.end(), [](const Piece& a, const Piece& b) { return a.count > b.count; });
  for (auto& b : bucket) b.clear();
  std::vector<std::pair<int32_t, int32_t>> th(PLAN_NT);       // (entries held, thread): min-heap
  for (int i = 0; i < PLAN_NT; ++i) th[i] = {0, i};
  auto heavier = [](const std::pair<int32_t, int32_t>& a, const std::pair<int32_t, int32_t>& b) { return a > b; };
  std::make_heap(th.begin(), th.end(), heavier);
  for (const Piece& pc : pieces) {
    std::pop_heap(th.begin(), th.end(), heavier);
    auto& b = bucket[th.back().second];
    for (int32_t q = 0; q < pc.count; ++q)
      b.push_back(((uint32_t)pc.slot << L.tile_bits) | (uint32_t)entries[pc.first + q].second);
    th.back().first += pc.count;
    std::push_heap(th.begin(), th.end(), heavier);
  }
  for (auto& b : bucket) std::sort(b.begin(), b.end());       // (slot, t) ascending: slot in the high bits
  // threads with at most one run first (in the order they were dealt), the others behind them
  auto one_run = [&](const std::vector<uint32_t>& b) {
    return b.empty() || (b.front() >> L.tile_bits) == (b.back() >> L.tile_bits);
  };
  std::stable_partition(bucket.begin(), bucket.end(), one_run);
}

// True if every thread of wave w holds at most one run and no more than one batch of entries.
bool plan_wave_is_uniform(const PlanLayout& L, const std::vector<std::vector<uint32_t>>& bucket, int w) {
  for (int l = 0; l < PLAN_WAVE; ++l) {
    const auto& b = bucket[w * PLAN_WAVE + l];
    if (b.size() > (size_t)PLAN_BATCH) return false;
    if (!b.empty() && (b.front() >> L.tile_bits) != (b.back() >> L.tile_bits)) return false;
  }
  return true;
}

}  // namespace

extern "C" int dl_marginal_plan_build(const int32_t* t2s, int64_t n_teacher, int64_t n_student, int* tile_out,
                                      int32_t* row_off, uint32_t* ent, int64_t ent_rows_capacity,
                                      int64_t* ent_rows_out, int32_t* fold, int64_t fold_capacity,
                                      int64_t* n_fold_out, int* n_extra_out) {
  constexpr uint32_t FIRST = 0x80000000u;
  if (!t2s || !tile_out || !ent_rows_out || !n_fold_out || !n_extra_out) return DL_ERR_NULL;
  if (n_teacher <= 0 || n_student <= 0) return DL_ERR_SHAPE;
  if (n_teacher > 0x7fffffffLL) return DL_ERR_LIMIT;
  for (int64_t t = 0; t < n_teacher; ++t)
    if (t2s[t] >= n_student) return DL_ERR_SHAPE;

  // tile size: the cheapest of the candidates by an estimate of the kernels' time per tile
  std::vector<std::pair<int32_t, int32_t>> entries;
  std::vector<std::vector<uint32_t>> bucket(PLAN_NT);
  PlanLayout best;
  int64_t best_cost = -1;
  for (int tile = 8192; tile >= 4096; tile -= 1024) {
    PlanLayout L;
    if (!plan_layout(t2s, n_teacher, n_student, tile, L)) continue;
    int64_t cost = 0;
    for (int64_t k = 0; k < L.ntiles; ++k) {
      tile_entries(t2s, n_teacher, L, k, entries);
      plan_deal_tile(L, entries, bucket);
      size_t longest = 0;
      for (const auto& b : bucket) longest = std::max(longest, b.size());
      const int64_t batches = std::max<int64_t>(1, ((int64_t)longest + PLAN_BATCH - 1) / PLAN_BATCH);
      bool all_packed = true;
      for (int w = 0; w < PLAN_NW && all_packed; ++w) all_packed = plan_wave_is_uniform(L, bucket, w);
      // nanoseconds per tile measured on an MI355X: 310 + 130 per 1024 ids when every wave's list is
      // packed, 60 more when a wave takes a general batch (every wave waits for it at the barrier),
      // about 450 for every further batch
      cost += 310 + 130 * (int64_t)tile / 1024 + (all_packed ? 0 : 60) + 450 * (batches - 1);
    }
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = L; }
  }
  if (best_cost < 0) return DL_ERR_LIMIT;                    // marginal + smallest tile do not fit the LDS
  const PlanLayout& L = best;
  *tile_out = L.tile;
  *n_fold_out = L.n_fold;
  *n_extra_out = (int)L.n_extra;
  if (fold) {
    if (L.n_fold > fold_capacity) return DL_ERR_SHAPE;
    int64_t f = 0;
    for (int64_t s = 0; s < n_student; ++s)
      if (L.reps[s] > 1) {
        fold[3 * f] = (int32_t)s; fold[3 * f + 1] = L.first_extra[s]; fold[3 * f + 2] = L.reps[s] - 1;
        ++f;
      }
  }

  const uint32_t spare = (uint32_t)(L.n_pad + ((L.n_extra + 3) & ~(int64_t)3));   // first of the 64 spare slots
  int64_t rows = 0;
  if (row_off) row_off[0] = 0;
  for (int64_t k = 0; k < L.ntiles; ++k) {
    tile_entries(t2s, n_teacher, L, k, entries);
    plan_deal_tile(L, entries, bucket);
    for (int w = 0; w < PLAN_NW; ++w) {
      const bool packed = plan_wave_is_uniform(L, bucket, w);
      size_t longest = 0;
      for (int l = 0; l < PLAN_WAVE; ++l) longest = std::max(longest, bucket[w * PLAN_WAVE + l].size());
      longest = std::max<size_t>(PLAN_BATCH, (longest + PLAN_BATCH - 1) / PLAN_BATCH * PLAN_BATCH);   // whole batches, at least one
      const size_t list_rows = packed ? (size_t)PLAN_PACKED_ROWS : longest;
      if (ent) {
        if (rows + (int64_t)list_rows > ent_rows_capacity) return DL_ERR_SHAPE;
        uint32_t* out = ent + rows * PLAN_WAVE;
        for (int l = 0; l < PLAN_WAVE; ++l) {
          const auto& b = bucket[w * PLAN_WAVE + l];
          if (packed) {
            const uint32_t slot = b.empty() ? spare + (uint32_t)l : b.front() >> L.tile_bits;
            for (int f = 0; f < PLAN_BATCH; ++f) {                              // padding first, the entries last
              const int j = f - (PLAN_BATCH - (int)b.size());
              const uint32_t offset = j >= 0 ? (b[j] & ((1u << L.tile_bits) - 1u)) : (uint32_t)L.tile;
              const int slot_bit = (f & 1) ? 8 + (f & ~1) : f;                   // where the field's two slot bits come from
              const uint32_t field = offset << 2 | ((slot >> slot_bit) & 3u);
              uint32_t& d = out[l * 4 + f / 2];
              d = (f & 1) ? (d | field << 16) : field;
            }
            continue;
          }
          for (size_t row = 0; row < longest; ++row) {
            uint32_t e = FIRST | (spare + (uint32_t)l) << PLAN_SLOT_SHIFT;
            if (row >= longest - b.size()) {                                    // padding first, the entries last
              const size_t j = row - (longest - b.size());
              const uint32_t slot = b[j] >> L.tile_bits, offset = b[j] & ((1u << L.tile_bits) - 1u);
              const bool first = j == 0 || (b[j - 1] >> L.tile_bits) != slot;
              const bool last = j + 1 == b.size() || (b[j + 1] >> L.tile_bits) != slot;
              e = (first ? FIRST : 0u) | (last ? slot : spare + (uint32_t)l) << PLAN_SLOT_SHIFT | offset << 2;
            }
            out[(row / PLAN_BATCH) * PLAN_BATCH * PLAN_WAVE + l * PLAN_BATCH + row % PLAN_BATCH] = e;
          }
        }
      }
      if (row_off && packed) row_off[k * PLAN_NW + w] |= 1;
      rows += (int64_t)list_rows;
      if (rows > 0x7fffffffLL) return DL_ERR_LIMIT;
      if (row_off) row_off[k * PLAN_NW + w + 1] = (int32_t)rows;
    }
  }
  *ent_rows_out = rows;
  return DL_OK;
}

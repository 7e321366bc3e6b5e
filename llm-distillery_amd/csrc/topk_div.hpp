// Forward / reverse KL against a sparse (top-K) teacher: loss and gradient in one sweep.
//
// Forward KL needs the full-vocabulary log-sum-exp of the student row, so the row is pulled
// into registers with 16-byte non-temporal loads (read from HBM once), reduced, and the gradient
//     d kl / d logit_j = (softmax(z)_j - sum_k q_k [j == idx_k]) * inv_T * scale
// is produced from the same registers: a dense softmax sweep, then K sparse corrections after a
// workgroup barrier.  The K teacher entries (id, log-prob, gathered student logit) live in LDS.
//
// A 128256-entry bf16 row is 250 KB, half of a CU's register file, so a workgroup that holds a
// whole row runs alone on its CU and its load / arithmetic / store phases cannot overlap.  The
// split kernel therefore cuts a row into P column parts, one workgroup each; several parts of
// different rows share a CU and hide each other's phases.  The parts of a row exchange their
// (max, sum-exp, partial loss) through a small workspace in global memory; the wait on the
// partner is bounded, and a part that gives up recomputes the row statistics on its own.
//
// Reverse KL (student renormalised over the K ids) touches only the K gathered logits; its
// gradient row is a zero fill plus K sparse values.
//
// Rows that do not fit (or break the 16-byte alignment rules) take the streaming kernel, which
// reads the row twice.
// This header holds the kernels and their launchers; topk_div.hip instantiates them for one stored
// teacher (dl_div_topk), topk_multi.hip for several unmerged teachers (dl_fkl_multi_teacher).
#pragma once
#include "distill_common.hpp"
#include "distill_hip.h"
#include <algorithm>

namespace dl {

// Several teachers handed over unmerged (dl_fkl_multi_teacher): teacher j holds Kt entries per row in
// val[j] / idx[j]; an entry's mass is exp(val + logw[j]); its id goes through id_map (teacher id ->
// student id, negative = dropped).
struct MultiTeacher {
  int n; int Kt;
  const void* val[DL_MAX_TEACHERS]; const void* idx[DL_MAX_TEACHERS];
  float logw[DL_MAX_TEACHERS];
  const int32_t* id_map; int64_t Vt;
};

// The same teachers prepared for the loss kernels (multi_prep_kernel): per teacher row the surviving
// entries as (student id, log of the renormalised mass), dealt into one bucket per column part of
// the loss kernel's row split, in stored order (teacher 0 first).  Bucket h of a row holds its first
// `cap0` entries in first[(row * parts + h) * cap0 ...] -- the part's workgroup fetches all cap0 slots
// by lane before it knows the count, and keeps what lies below it: the slots behind are never written
// -- and whatever exceeds cap0 in the row's share of `more`, buckets back to back.  head[row * 16 + h] = entries of bucket h (h < 8),
// [8] = entries of the row, [9] = float bits of the sum of the renormalised masses (1 up to rounding).
struct TeacherBuckets {
  const uint2* first; const uint2* more; const int* head;
  int cap0; int E;
};

struct TopkParams {
  const void* logits; int64_t row_stride; int64_t n_rows; int64_t V;
  const int32_t* row_map;
  const void* t_val; int t_val_dtype; const void* t_idx; int t_idx_itype; int K;
  int64_t n_trows; const int32_t* t_cnt;
  float inv_T_s, inv_T_t, grad_scale;
  float* row_loss; void* grad; int64_t grad_stride;
  void* workspace; int parts; int spin_limit; int flags;
  TeacherBuckets bk;    // MULTI kernels only; K is then the number of entries a bucket may hold, rounded up to whole slots
};

constexpr int MAX_PARTS = 16;             // parts a row may be cut into (parts of 256 x 4 chunks)
constexpr int MAX_COARSE_PARTS = 8;       // of 256 x 16 chunks

// What one part of a split row tells the others: three floats and a tag that depends on all of
// them.  The four words are written and read with relaxed device-scope accesses (they bypass the
// non-coherent cache levels; no cache-wide flush or invalidate); a reader accepts a record only
// when the tag matches, so no ordering between the words is needed.  A cleared record is invalid.
struct PartStats { unsigned m, s, b, tag; };
__device__ __forceinline__ unsigned part_tag(unsigned m, unsigned s, unsigned b) {
  return m ^ ((s << 7) | (s >> 25)) ^ ((b << 13) | (b >> 19)) ^ 0x5eed1234u;
}
__device__ __forceinline__ void part_publish(PartStats* w, float m, float s, float b) {
  const unsigned um = __float_as_uint(m), us = __float_as_uint(s), ub = __float_as_uint(b);
  __hip_atomic_store(&w->m, um, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->s, us, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->b, ub, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->tag, part_tag(um, us, ub), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Bounded wait for a partner's record; false = gave up after `limit` polls.
__device__ __forceinline__ bool part_collect(PartStats* w, int limit, float& m, float& s, float& b) {
  for (int spins = 0; spins < limit; ++spins) {
    const unsigned um = __hip_atomic_load(&w->m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned us = __hip_atomic_load(&w->s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned ub = __hip_atomic_load(&w->b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned ut = __hip_atomic_load(&w->tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (ut == part_tag(um, us, ub)) {
      m = __uint_as_float(um); s = __uint_as_float(us); b = __uint_as_float(ub);
      return true;
    }
    __builtin_amdgcn_s_sleep(4);
  }
  return false;
}

// Workspace of a split launch: n_rows * parts records, then a counter and the list of (row, part)
// numbers that gave up waiting for a partner and are finished by a second launch.
struct RetryList {
  unsigned* count;
  unsigned* entries;
  __host__ __device__ RetryList(void* workspace, int64_t n_rows, int parts) {
    char* base = reinterpret_cast<char*>(workspace) + n_rows * parts * (int64_t)sizeof(PartStats);
    count = reinterpret_cast<unsigned*>(base);
    entries = reinterpret_cast<unsigned*>(base + 16);
  }
  __host__ __device__ static int64_t bytes(int64_t n_rows, int parts) {
    return n_rows * parts * (int64_t)(sizeof(PartStats) + 4) + 16;
  }
};

// LDS carve-up shared by the kernels of this file.  The id array is padded to a multiple of 16
// with -1 so that it can be scanned four ids per read.
struct TopkLds {
  float* red;        // reduction scratch, 64 floats
  float* xm; float* xs; float* xb; int* xok;    // per-part statistics of a split row, MAX_PARTS each
  int* idx;          // Kp  vocabulary id or -1
  float* t;          // Kp  scaled teacher logit -> teacher log-probability over the K entries
  float* q;          // Kp  teacher probability
  float* z;          // Kp  gathered student logit
  // in-register corrections (kernels that keep the row in registers; owners == 0 elsewhere):
  float* val;        // Kp  final gradient value at the entry's column
  int* next;         // Kp  next entry owned by the same thread, or -1
  int* head;         // CORRECTION_HEADS list heads: first entry of a chunk's list, or -1
  unsigned* own;     // one per thread: bit i set = chunk i of the thread holds an entry
  u32x4* tail;       // ROWS_TAIL: the logits of the row's ragged chunk, kept for the gradient by the one thread that holds it
  int Kp;
  __device__ TopkLds(unsigned char* base, int K, int owners = 0) {
    Kp = (K + 15) & ~15;
    red = reinterpret_cast<float*>(base);
    xm = red + 64; xs = xm + MAX_PARTS; xb = xs + MAX_PARTS; xok = reinterpret_cast<int*>(xb + MAX_PARTS);
    idx = reinterpret_cast<int*>(base + 512);
    t = reinterpret_cast<float*>(idx + Kp);
    q = t + Kp;
    z = q + Kp;
    val = z + Kp;
    next = reinterpret_cast<int*>(val + Kp);
    head = next + Kp;
    own = reinterpret_cast<unsigned*>(head + (owners ? CORRECTION_HEADS : 0));
    tail = reinterpret_cast<u32x4*>(own + owners);
  }
  __host__ __device__ static size_t bytes(int K, int owners = 0) {
    const size_t Kp = (size_t)((K + 15) & ~15);
    return 512 + Kp * 16 + (owners ? Kp * 8 + (size_t)CORRECTION_HEADS * 4 + (size_t)owners * 4 + 16 : 0);
  }
};

// Teacher entries of one row held in registers between issue and use: J entries per thread,
// entry k = tid + j * NT.  Issuing their (tiny) loads before the row's 16 big ones, and the
// dependent gathers right behind those, keeps three global-memory latencies off the critical path.
template <int J>
struct TeacherEntries {
  int id[J];
  float tv[J];
  float z[J];
};

template <int NT, int J>
__device__ __forceinline__ void teacher_issue(const TopkParams& p, int64_t trow, TeacherEntries<J>& t) {
  const int K = p.K;
  const int cnt = p.t_cnt ? min(p.t_cnt[trow], K) : K;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int k = threadIdx.x + j * NT;
    int64_t id = -1;
    float v = -INFINITY;
    if (k < cnt) {
      const int64_t at = trow * (int64_t)K + k;
      id = load_index(p.t_idx, p.t_idx_itype, at);
      v = load_as_float(p.t_val, p.t_val_dtype, at);       // independent of the id: both loads fly together
    }
    const bool ok = id >= 0 && id < p.V && v > -INFINITY;      // an entry of zero mass is no entry
    t.id[j] = ok ? (int)id : -1;
    t.tv[j] = ok ? v * p.inv_T_t : -INFINITY;
  }
}

template <class Tag, int J>
__device__ __forceinline__ void teacher_gather(const char* row, int lo, int hi, TeacherEntries<J>& t) {
#pragma unroll
  for (int j = 0; j < J; ++j)
    t.z[j] = (t.id[j] >= lo && t.id[j] < hi) ? load_as_float(row, Tag::id, t.id[j]) : 0.f;
}

// Prepared teachers (TeacherBuckets): the first J * NT = cap0 entries of this part's bucket, one per
// lane and slot, fetched by position alone (slots behind the count hold whatever was there); the bucket's and the row's entry
// counts and the row's mass sum come along as same-address loads.
struct BucketHead { int n; int total; float qsum; int more_at; };

template <int NT, int J>
__device__ __forceinline__ void bucket_issue(const TopkParams& p, int64_t trow, int h, int P, TeacherEntries<J>& t,
                                             BucketHead& hd) {
  const uint2* first = p.bk.first + (trow * P + h) * (int64_t)p.bk.cap0;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const uint2 e = first[threadIdx.x + j * NT];
    t.id[j] = (int)e.x;
    t.tv[j] = __uint_as_float(e.y);
  }
  const int* head = p.bk.head + trow * 16;
  hd.n = min(max(head[h], 0), p.bk.E);    // counts are clamped to what the workspace and LDS were laid out for
  hd.total = head[8];
  hd.qsum = __int_as_float(head[9]);
  hd.more_at = 0;                         // where this bucket's overflow starts in the row's share of `more`
  for (int g = 0; g < h; ++g) hd.more_at += max(min(head[g], p.bk.E) - p.bk.cap0, 0);
  hd.more_at = min(hd.more_at, p.bk.E - max(hd.n - p.bk.cap0, 0));
}

// Registers -> LDS, then the teacher's log-sum-exp; same result layout as stage_teacher.
// The gathered student logits t.z are the last loads of the workgroup to arrive (they queue behind the
// row's own loads), so they are touched last: everything before overlaps with the row in flight.
template <int NT, int J>
__device__ __forceinline__ float teacher_finish(const TopkLds& s, const TeacherEntries<J>& t) {
  float tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int k = threadIdx.x + j * NT;
    if (k < s.Kp) s.idx[k] = t.id[j];
    tmax = fmaxf(tmax, t.tv[j]);
  }
  tmax = block_max<NT>(tmax, s.red);     // barrier inside: LDS entries visible afterwards
  float tlse = tmax;
  if (tmax != -INFINITY) {
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j) part += expf(t.tv[j] - tmax);
    tlse = tmax + logf(block_sum<NT>(part, s.red));
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int k = threadIdx.x + j * NT;
      if (k < s.Kp) {
        const float lt = t.tv[j] - tlse;
        s.t[k] = lt;
        s.q[k] = expf(lt);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int k = threadIdx.x + j * NT;
    if (k < s.Kp) s.z[k] = t.z[j];      // read back by this thread only
  }
  return tlse;
}

// Stage the teacher row: ids, scaled log-probs, and the student logits at the ids that fall into
// the column range [lo, hi) this workgroup owns.  Returns the log-sum-exp of the scaled teacher
// entries (-inf if the row has none); afterwards s.t holds the teacher log-probabilities and s.q
// the probabilities (0 for padding and ignored entries).
template <class Tag, int NT>
__device__ __forceinline__ float stage_teacher(const TopkParams& p, const TopkLds& s, int64_t trow,
                                               const char* row, int lo, int hi) {
  const int K = p.K;
  const int cnt = p.t_cnt ? min(p.t_cnt[trow], K) : K;
  float tmax = -INFINITY;
  for (int k = threadIdx.x; k < s.Kp; k += NT) {
    const int64_t at = trow * (int64_t)K + k;
    const int64_t id = k < cnt ? load_index(p.t_idx, p.t_idx_itype, at) : -1;
    const bool in = id >= 0 && id < p.V;
    const float tv = in ? load_as_float(p.t_val, p.t_val_dtype, at) * p.inv_T_t : -INFINITY;
    const bool ok = in && tv > -INFINITY;                  // an entry of zero mass is no entry
    s.idx[k] = ok ? (int)id : -1;
    s.t[k] = tv;
    s.z[k] = (ok && id >= lo && id < hi) ? load_as_float(row, Tag::id, id) : 0.f;
    tmax = fmaxf(tmax, tv);
  }
  tmax = block_max<NT>(tmax, s.red);     // barrier inside: LDS entries visible afterwards
  if (tmax == -INFINITY) return tmax;
  float part = 0.f;
  for (int k = threadIdx.x; k < s.Kp; k += NT) part += expf(s.t[k] - tmax);
  const float tlse = tmax + logf(block_sum<NT>(part, s.red));
  for (int k = threadIdx.x; k < s.Kp; k += NT) {      // own entries only: no barrier needed yet
    const float lt = s.t[k] - tlse;
    s.t[k] = lt;
    s.q[k] = expf(lt);
  }
  return tlse;
}

// Partial forward-KL sums over the ids inside [lo, hi):  B = sum q_k (t_k - z_k * inv_T)  and, over
// all ids, Q = sum q_k.  The row value is  sum over parts of B  +  lse * Q.
template <int NT>
__device__ __forceinline__ void fkl_partials(const TopkParams& p, const TopkLds& s, int lo, int hi, float& B,
                                             float& Q) {
  B = 0.f; Q = 0.f;
  for (int k = threadIdx.x; k < s.Kp; k += NT) {
    const int id = s.idx[k];
    if (id >= 0) {
      const float q = s.q[k];
      Q += q;
      if (id >= lo && id < hi) B += q * (s.t[k] - s.z[k] * p.inv_T_s);
    }
  }
  block_sum2<NT>(B, Q, s.red);
}

// Sum of the masses q[e] of the entries on a chunk list that name column `want`, given the largest of
// them (`big` > 0): order-independent.  Every mass is scaled by a power of two taken from the largest
// (exact), rounded to an integer below 2^30 and added as such, so the sum is the same whatever order
// the list was linked in, and good to 2^-30 of the largest term per term.
__device__ __forceinline__ float mass_on_column(const int* next, const int* col, const float* q, int first, int want,
                                                float big) {
  const int shift = 30 - __builtin_amdgcn_frexp_expf(big);      // big * 2^shift in [2^29, 2^30)
  long long acc = 0;
  for (int e = first; e >= 0; e = next[e])
    if (col[e] == want) acc += (long long)__float2int_rn(ldexpf(q[e], shift));
  const float hi = (float)(int)(acc >> 24), lo = (float)(int)(acc & 0xffffff);      // acc < 2^41: both parts exact in fp32
  return ldexpf(fmaf(hi, 16777216.f, lo), -shift);
}

// Prepared teachers, the K-wide part of the row's loss.  Several entries of a row may carry the same
// student id (the same token in two teachers, two teacher ids mapped onto one student id); the
// mixture's mass on the id is their sum Q_id, and the row's forward KL is
//     sum_id Q_id (log Q_id - s_id)  =  sum_k q_k (log Q_id(k) - s_id(k)).
// All entries of a bucket lie inside the part's columns [lo, hi).  They are linked into the lists of
// the 16-byte chunks their columns lie in (the lists the gradient sweep uses anyway); the thread of
// entry k then finds the other entries of its column on that list and sums their masses in fixed
// point, independent of the list's order.  Entries beyond the bucket's first cap0 (rare: the ids of a
// row crowd into one part) are fetched here, from the row's overflow share.
// Leaves q in s.q, Q_id(k) in s.val[k], z in s.z[k]; returns the number of LDS entry slots in use
// (a multiple of NT); B as fkl_partials.
template <class Tag, int NT, int NCH, int J>
__device__ __forceinline__ int bucket_finish(const TopkParams& p, const TopkLds& s, const TeacherEntries<J>& te,
                                             const BucketHead& hd, int64_t trow, const char* row, int lo, int hi, float& B) {
  const int nk = max(J * NT, (hd.n + NT - 1) / NT * NT);
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int k = threadIdx.x + j * NT;
    const bool ok = k < hd.n && te.id[j] >= lo && te.id[j] < hi;      // what lies behind the bucket's count was never written
    s.idx[k] = ok ? te.id[j] : -1;
    s.t[k] = te.tv[j];
    s.q[k] = ok ? expf(te.tv[j]) : 0.f;
    s.z[k] = te.z[j];
  }
  if (nk > J * NT) {
    const uint2* more = p.bk.more + trow * (int64_t)p.bk.E + hd.more_at;
    for (int k = J * NT + threadIdx.x; k < nk; k += NT) {
      uint2 e{0xffffffffu, 0xff800000u};
      if (k < hd.n) e = more[k - J * NT];
      const int id = (int)e.x;
      const bool ok = id >= lo && id < hi;
      const float lq = __uint_as_float(e.y);
      s.idx[k] = ok ? id : -1;
      s.t[k] = lq;
      s.q[k] = ok ? expf(lq) : 0.f;
      s.z[k] = ok ? load_as_float(row, Tag::id, id) : 0.f;
    }
  }
  for (int k = threadIdx.x; k < nk; k += NT) {
    const int id = s.idx[k];                               // this thread's own store
    if (id >= 0) correction_link<Tag, NT, NCH>(s.head, s.own, s.next, k, id - lo);
  }
  __syncthreads();
  B = 0.f;
  for (int k = threadIdx.x; k < nk; k += NT) {
    const int id = s.idx[k];
    if (id < 0) continue;
    const int first = s.head[correction_head_slot<Tag, NT, NCH>(id - lo)];
    int same = 0;
    float big = 0.f;
    for (int e = first; e >= 0; e = s.next[e]) {
      const bool mine = s.idx[e] == id;
      same += mine ? 1 : 0;
      big = fmaxf(big, mine ? s.q[e] : 0.f);
    }
    const float q = s.q[k];
    float Qid = q, l = s.t[k];
    if (same > 1 && big > 0.f) {
      Qid = mass_on_column(s.next, s.idx, s.q, first, id, big);
      l = logf(Qid);
    }
    s.val[k] = Qid;
    B += q * (l - s.z[k] * p.inv_T_s);
  }
  B = block_sum<NT>(B, s.red);
  return nk;
}

// Teacher mass on the id of entry k, summed over every entry that carries the same id.
__device__ __forceinline__ float mass_on_id(const TopkLds& s, int k, int id) {
  int same = 0;
  const int4* ids = reinterpret_cast<const int4*>(s.idx);
#pragma unroll 4
  for (int j = 0; j < s.Kp / 4; ++j) {
    const int4 v = ids[j];
    same += (v.x == id) + (v.y == id) + (v.z == id) + (v.w == id);
  }
  if (same == 1) return s.q[k];
  float q = 0.f;                        // duplicates inside a row are rare: slow path
  for (int j = 0; j < s.Kp; ++j) q += (s.idx[j] == id) ? s.q[j] : 0.f;
  return q;
}

// Sparse corrections of the dense softmax row already written by this workgroup, for the ids
// inside [lo, hi).  b is the row's log2-sum-exp2, a = inv_T * log2(e), c = inv_T * scale.
template <class Tag, int NT>
__device__ __forceinline__ void fkl_sparse_fix(const TopkLds& s, void* grow, int lo, int hi,
                                               float a, float b, float c, bool ids_unique) {
  for (int k = threadIdx.x; k < s.Kp; k += NT) {
    const int id = s.idx[k];
    if (id < lo || id >= hi) continue;
    const float q = ids_unique ? s.q[k] : mass_on_id(s, k, id);
    store_from_float(grow, Tag::id, id, (fast_exp2(fmaf(s.z[k], a, -b)) - q) * c);
  }
}

// The same corrections for a row (part) held in registers, applied by the threads that hold the
// columns before they store them (correction_link / correction_apply).  Entry threads leave the
// student probability at the entry's column in s.val and link the entry into its owner's list; the
// owner subtracts the teacher mass -- of all entries of that column, should ids repeat, which it
// sees from the chunk's list: no scan over the row's ids.
template <class Tag, int NT, int NCH>
__device__ __forceinline__ void fkl_link_corrections(const TopkLds& s, int lo, int hi, float a, float b) {
  for (int k = threadIdx.x; k < s.Kp; k += NT) {
    const int id = s.idx[k];
    if (id < lo || id >= hi) continue;
    s.val[k] = fast_exp2(fmaf(s.z[k], a, -b));
    correction_link<Tag, NT, NCH>(s.head, s.own, s.next, k, id - lo);
  }
}

// Full-row statistics straight from global memory (two uses: the streaming kernel, and a split
// part whose partner did not answer in time).  Returns the row maximum and sum 2^((x - max) a).
// MODE 0: element by element.  MODE 1: rows on the 16-byte grid, a whole number of chunks long.
// MODE 2: any row: its 16-byte chunks by vector loads, the elements before and behind them one by one.
template <class Tag, int NT, int MODE>
__device__ __forceinline__ void row_stats_streamed(const char* row, int64_t V, float a, float* red, float& mx,
                                                   float& sm) {
  using C = Chunk<Tag>;
  float m = -INFINITY;
  sm = 0.f;
  const auto one = [&](float f) {
    if (f > m) { sm *= fast_exp2((m - f) * a); m = f; }
    if (f > -INFINITY) sm += fast_exp2(fmaf(f, a, -m * a));
  };
  if (MODE != 0) {
    const RowSplit<Tag> sp(row, V, MODE == 2);
    const char* body = row + (int64_t)sp.head * Tag::bytes;
    for (int64_t ch = threadIdx.x; ch < sp.nbody; ch += NT) {
      float f[C::N];
      C::unpack(*reinterpret_cast<const u32x4*>(body + ch * 16), f);
      float cm = f[0];
#pragma unroll
      for (int e = 1; e < C::N; ++e) cm = fmaxf(cm, f[e]);
      if (cm > m) { sm *= fast_exp2((m - cm) * a); m = cm; }
      const float mb = m * a;
      if (m > -INFINITY) {
#pragma unroll
        for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[e], a, -mb));
      }
    }
    if (MODE == 2 && (int)threadIdx.x < sp.leftovers()) one(load_as_float(row, Tag::id, sp.column(threadIdx.x)));
  } else {
    for (int64_t j = threadIdx.x; j < V; j += NT) one(load_as_float(row, Tag::id, j));
  }
  mx = block_max<NT>(m, red);
  sm = (m == -INFINITY) ? 0.f : sm * fast_exp2((m - mx) * a);
  sm = block_sum<NT>(sm, red);
}

// How the rows of a register kernel lie in memory (template parameter RAG):
//   ROWS_WHOLE  on the 16-byte grid (base and pitch), a whole number of chunks long
//   ROWS_ANY    anywhere (element-aligned), any length: whole chunks move by unaligned 16-byte accesses
//   ROWS_TAIL   on the 16-byte grid, but V is not a whole number of chunks (a crop of a padded vocabulary,
//               logits[:, :, :crop]): every chunk but the row's last moves like a ROWS_WHOLE one
// In the last two the row's last, partly filled chunk moves element by element, with -inf in the columns
// it lacks (they add nothing to any statistic and are not stored).
constexpr int ROWS_WHOLE = 0, ROWS_ANY = 1, ROWS_TAIL = 2;

// Chunk c of a part that starts at `part`; `ncols` = columns from the part's first to the row's end.
template <class Tag, int RAG>
__device__ __forceinline__ u32x4 load_part_chunk(const char* part, int64_t c, int64_t ncols) {
  // cached, not streaming, loads: the gather of the logits at the teacher ids that follows then
  // finds its lines in L2 instead of fetching them a second time (0.47 GB less per 32768 rows of K = 200)
  if constexpr (RAG == ROWS_WHOLE) return *reinterpret_cast<const u32x4*>(part + c * 16);
  else if ((c + 1) * Chunk<Tag>::N <= ncols) {
    if constexpr (RAG == ROWS_ANY) return load16_unaligned(part + c * 16);
    else return *reinterpret_cast<const u32x4*>(part + c * 16);
  }
  else return load_chunk_elementwise<Tag>(part, (int)c, (int)ncols);
}
template <class Tag, int RAG>
__device__ __forceinline__ void store_part_chunk(char* part, int64_t c, int64_t ncols, const u32x4& v) {
  if constexpr (RAG == ROWS_WHOLE) store16_stream(part + c * 16, v);
  else if ((c + 1) * Chunk<Tag>::N <= ncols) {
    if constexpr (RAG == ROWS_ANY) store16_unaligned(part + c * 16, v);
    else store16_stream(part + c * 16, v);
  }
  else store_chunk_elementwise<Tag>(part, (int)c, (int)ncols, v);
}
template <class Tag, int NT, int RAG>
__device__ __forceinline__ void zero_part(char* gpart, int64_t nch, int64_t ncols) {
  if constexpr (RAG == ROWS_WHOLE) zero_row<Tag, NT>(gpart, nch);
  else for (int64_t ch = threadIdx.x; ch < nch; ch += NT) store_part_chunk<Tag, RAG>(gpart, ch, ncols, u32x4{0u, 0u, 0u, 0u});
}

// ---------------------------------------------------------------------------------------
// Forward KL, (part of) a row resident in registers: NT threads x NCH 16-byte chunks per thread.
// SPLIT: P = p.parts workgroups per row.  Consecutive workgroup ids are dealt round-robin to the 8
// XCDs, each of which dispatches its share in order, so the parts of a row are placed 8 ids apart:
// they land on the same XCD back to back (partners start together and meet through one L2).
// Within a group of 8*P ids, id t serves row 8*group + t % 8, part t / 8.
// ---------------------------------------------------------------------------------------
// J > 0: the K <= J * NT teacher entries travel in registers (loads issued ahead of the row's);
// J == 0: any K, staged by a plain loop.
// RETRY: second launch over the parts that gave up waiting in the first (see split_retry_list):
// every record of the row is published by then, so nothing is waited for.
// MULTI: the row's teachers arrive prepared in buckets (TopkParams::bk), J * NT = cap0 entries in registers.
// RAG: how the rows lie in memory (ROWS_WHOLE / ROWS_ANY / ROWS_TAIL above).
template <class Tag, int NT, int NCH, bool SPLIT, int J, bool RETRY, bool MULTI, int RAG = ROWS_WHOLE>
__device__ __forceinline__ void fkl_topk_part(const TopkParams& p, const TopkLds& s, int64_t r, int h) {
  static_assert(!MULTI || J > 0, "the head of a bucket travels in registers");
  static_assert(RAG != ROWS_ANY || !MULTI, "rows off the 16-byte grid: one stored teacher");
  using C = Chunk<Tag>;
  const int tid = threadIdx.x;
  const int P = SPLIT ? p.parts : 1;
  const int64_t c0 = (int64_t)h * NT * NCH;                       // first chunk of this part
  const int64_t nch_row = RAG != ROWS_WHOLE ? (p.V + C::N - 1) / C::N : p.V / C::N;
  const int64_t nch = min((int64_t)NT * NCH, nch_row - c0);       // chunks of this part
  const int lo = (int)(c0 * C::N);                                // its column range
  const int hi = RAG != ROWS_WHOLE ? (int)min(p.V, (int64_t)lo + nch * C::N) : lo + (int)(nch * C::N);
  const int64_t ncols = p.V - lo;                                 // columns from the part's first to the row's end
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  char* gpart = grow ? grow + c0 * 16 : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (gpart) zero_part<Tag, NT, RAG>(gpart, nch, ncols);
    if (tid == 0 && h == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  const char* rpart = row + c0 * 16;

  correction_clear<NT>(s.head, s.own);      // lists of corrections, filled after the row statistics
  TeacherEntries<(J > 0 ? J : 1)> te;
  BucketHead hd{};
  if constexpr (MULTI) bucket_issue<NT, J>(p, trow, h, P, te, hd);
  else if constexpr (J > 0) teacher_issue<NT, J>(p, trow, te);
  // ROWS_TAIL: the part that holds the row's ragged chunk (part-relative number tail_c, else -1) loads it like the
  // others -- the 16 bytes start inside the row and, aligned as they are, end inside the row's pitch or at least
  // inside the page the row's last column lies in -- and the one thread that holds it puts -inf in the columns
  // beyond the row.  Which of a thread's registers that is, is the same for every thread (a scalar): the
  // unrolled sweeps pay a scalar compare per chunk for it, no vector work and no registers.
  const int64_t tail_c = (RAG == ROWS_TAIL && ncols < nch * C::N) ? nch - 1 : -1;
  const int tail_reg = tail_c >= 0 ? ChunkMap<NT, NCH>::reg((int)tail_c) : -1;
  const bool tail_mine = tail_c >= 0 && ChunkMap<NT, NCH>::owner((int)tail_c) == tid;
  const int64_t nfull = tail_c >= 0 ? nch - 1 : nch;              // chunks of this part that are stored whole
  u32x4 reg[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int64_t c = ChunkMap<NT, NCH>::chunk(i, tid);
    if constexpr (RAG == ROWS_TAIL) reg[i] = c < nch ? load_part_chunk<Tag, ROWS_WHOLE>(rpart, c, ncols) : C::neg_inf();
    else reg[i] = c < nch ? load_part_chunk<Tag, RAG>(rpart, c, ncols) : C::neg_inf();
  }
  u32x4 tail_raw = C::neg_inf();
  if constexpr (RAG == ROWS_TAIL) {
    if (tail_c >= 0) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
        if (i == tail_reg && tail_mine) reg[i] = chunk_keep_first<Tag>(reg[i], (int)(ncols - tail_c * C::N));
    }
    // a second copy of the ragged chunk for the gradient sweep (same line: no traffic), parked in LDS below
    if (tail_mine) tail_raw = load_part_chunk<Tag, ROWS_WHOLE>(rpart, tail_c, ncols);
  }

  // teacher side while the row is in flight
  float tlse = 0.f, B = 0.f, Q = 0.f;
  int nk = s.Kp;                      // LDS entry slots in use
  if constexpr (MULTI) {
    teacher_gather<Tag, J>(row, lo, hi, te);
    if (hd.total > 0) nk = bucket_finish<Tag, NT, NCH, J>(p, s, te, hd, trow, row, lo, hi, B);
    tlse = hd.total > 0 ? 0.f : -INFINITY;
    Q = hd.qsum;
  } else if constexpr (J > 0) {
    teacher_gather<Tag, J>(row, lo, hi, te);
    tlse = teacher_finish<NT, J>(s, te);
  } else {
    tlse = stage_teacher<Tag, NT>(p, s, trow, row, lo, hi);
  }
  if (tlse == -INFINITY) {            // no usable teacher entry: the row contributes nothing
    if (gpart) zero_part<Tag, NT, RAG>(gpart, nch, ncols);
    if (tid == 0 && h == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  if constexpr (!MULTI) fkl_partials<NT>(p, s, lo, hi, B, Q);

  if constexpr (RAG == ROWS_TAIL) {
    if (tail_mine) *s.tail = chunk_keep_first<Tag>(tail_raw, (int)(ncols - tail_c * C::N));      // read back by this thread only
  }
  const float a = p.inv_T_s * LOG2E;
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) mx = fmaxf(mx, f[e]);
  }
  mx = block_max<NT>(mx, s.red);
  // Second sweep: 2^(x a - max a + bias) takes the place of x in the registers; the gradient is
  // that value times a row constant, so each element costs one exp2, not two.
  float mb = (mx == -INFINITY) ? 0.f : mx * a;      // a part that holds only -inf logits: every 2^(.) below is 0, not NaN
  const float mb_own = mb - C::stash_bias;
  float sm = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) {
      f[e] = fast_exp2(fmaf(f[e], a, -mb_own));
      sm += f[e];
    }
    reg[i] = C::stash(f);
    forget(reg[i]);         // pins the schedule chunk by chunk: no pile-up of unpacked values
  }
  sm = block_sum<NT>(sm * __builtin_exp2f(-C::stash_bias), s.red);      // exact: a power of two

  if (SPLIT) {
    // publish this part's statistics, collect the others'
    PartStats* ws = reinterpret_cast<PartStats*>(p.workspace) + r * P;
    if (tid == 0 && !RETRY) part_publish(ws + h, mx, sm, B);
    if (tid < P) {
      float om = mx, os = sm, ob = B;
      const int ok = (tid == h) || part_collect(ws + tid, RETRY ? 0x7fffffff : p.spin_limit, om, os, ob);
      s.xm[tid] = om; s.xs[tid] = os; s.xb[tid] = ob; s.xok[tid] = ok;
    }
    __syncthreads();
    bool all_ok = true;
    for (int j = 0; j < P; ++j) all_ok = all_ok && (s.xok[j] != 0);
    if (!all_ok) {
      // A partner did not answer in time.  Nothing has been written yet: this part puts itself on
      // the retry list and leaves; its own record is published, so the partners can finish.
      if (tid == 0) {
        RetryList list(p.workspace, p.n_rows, P);
        list.entries[atomicAdd(list.count, 1u)] = (unsigned)(r * P + h);
      }
      return;
    }
    float M = s.xm[0];
    for (int j = 1; j < P; ++j) M = fmaxf(M, s.xm[j]);
    float S = 0.f, Bt = 0.f;
    for (int j = 0; j < P; ++j) { S += s.xs[j] * fast_exp2((s.xm[j] - M) * a); Bt += s.xb[j]; }
    mb = M * a; sm = S; B = Bt;
  }
  const float b = mb + fast_log2(sm);      // log2-sum-exp2 of the scaled row
  if (tid == 0 && h == 0 && p.row_loss) p.row_loss[r] = B + (b * LN2) * Q;

  if (gpart) {
    const float c = p.inv_T_s * p.grad_scale;
    const float kc = fast_exp2(mb_own - b) * c;       // stashed value -> gradient
    // 16 chunks of 4-byte logits leave no registers for placing the corrections during the sweep
    // (it spills): those shapes write them behind the dense stores instead.
    constexpr bool IN_REGISTERS = !(Tag::bytes == 4 && NCH == 16);
    if constexpr (MULTI) {
      // the lists exist since bucket_finish, s.val holds the mixture's mass on the entry's id: every
      // entry of a column carries the column's final value, whichever of them the owner meets
      for (int k = tid; k < nk; k += NT) {
        const int id = s.idx[k];
        if (id >= lo && id < hi) s.val[k] = fast_exp2(fmaf(s.z[k], a, -b)) - s.val[k];
      }
      __syncthreads();
    } else if (IN_REGISTERS) {
      fkl_link_corrections<Tag, NT, NCH>(s, lo, hi, a, b);
      __syncthreads();
    }
    const unsigned mine = IN_REGISTERS ? s.own[tid] : 0u;
    const bool may_repeat = !MULTI && (p.flags & DL_TOPK_UNIQUE_IDS) == 0;
    const auto mass = [&](int k) { return MULTI ? 0.f : s.q[k]; };
    const auto value = [&](int k, float q) { return (s.val[k] - q) * c; };
    unsigned repeats = 0u;            // chunks in which an id occurs more than once
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int64_t ch = ChunkMap<NT, NCH>::chunk(i, tid);
      if (ch < nfull) {
        float f[C::N];
        forget(reg[i]);
        C::unstash(reg[i], f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] *= kc;
        if (mine & (1u << i))
          if (correction_apply<Tag, NT, NCH>(s.head, s.next, s.idx, lo, i, f, mass, value)) repeats |= 1u << i;
        if constexpr (RAG == ROWS_TAIL) store16_stream(gpart + ch * 16, C::pack(f));
        else store_part_chunk<Tag, RAG>(gpart, ch, ncols, C::pack(f));
      }
    }
    if constexpr (RAG == ROWS_TAIL) {
      // The ragged chunk, by the one thread that holds it, from the copy of its logits in LDS, stored element by
      // element.  The sweep above covers the whole chunks
      // only and is the sweep of whole rows, instruction for instruction: a second bound inside it, or
      // registers that must outlive it, make the 512 x 16 shape spill.
      if (tail_mine) {
        float f[C::N];
        C::unpack(*s.tail, f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = fast_exp2(fmaf(f[e], a, -b)) * c;
        if (mine & (1u << tail_reg))
          if (correction_apply<Tag, NT, NCH>(s.head, s.next, s.idx, lo, tail_reg, f, mass, value)) repeats |= 1u << tail_reg;
        store_chunk_elementwise<Tag>(gpart, (int)tail_c, (int)ncols, C::pack(f));
      }
    }
    if (may_repeat && repeats)
      correction_repeats<Tag, NT, NCH>(s.head, s.next, s.idx, lo, repeats, NCH, mass, value,
                                  [&](int column, float v) { store_from_float(grow, Tag::id, column, v); });
    if (!IN_REGISTERS) {
      __syncthreads();      // dense stores are ordered before the sparse corrections
      if constexpr (MULTI) {
        for (int k = tid; k < nk; k += NT) {
          const int id = s.idx[k];
          if (id >= lo && id < hi) store_from_float(grow, Tag::id, id, s.val[k] * c);      // entries of one column: the same value
        }
      } else {
        fkl_sparse_fix<Tag, NT>(s, grow, lo, hi, a, b, c, (p.flags & DL_TOPK_UNIQUE_IDS) != 0);
      }
    }
  }
}

template <class Tag, int NT, int NCH, bool SPLIT, int J, bool MULTI = false, int RAG = ROWS_WHOLE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void fkl_topk_reg_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K, NT);
  const int P = SPLIT ? p.parts : 1;
  const unsigned grp = SPLIT ? blockIdx.x / (8u * P) : 0u, t_in = SPLIT ? blockIdx.x % (8u * P) : 0u;
  const int64_t r = SPLIT ? (int64_t)grp * 8 + (t_in & 7u) : xcd_banded_row(blockIdx.x);
  const int h = SPLIT ? (int)(t_in >> 3) : 0;
  if (r >= p.n_rows) return;
  fkl_topk_part<Tag, NT, NCH, SPLIT, J, false, MULTI, RAG>(p, s, r, h);
}

// One listed part, as a real call: the loop around it then costs the body no registers.
template <class Tag, int NT, int NCH, int J, bool MULTI, int RAG>
__device__ __attribute__((noinline)) void fkl_topk_part_again(const TopkParams& p, const TopkLds& s, unsigned at) {
  fkl_topk_part<Tag, NT, NCH, true, J, true, MULTI, RAG>(p, s, (int64_t)(at / (unsigned)p.parts), (int)(at % (unsigned)p.parts));
}

// The parts on the retry list, a fixed grid striding over it (normally the list is empty and
// every workgroup leaves after one load).
template <class Tag, int NT, int NCH, int J, bool MULTI = false, int RAG = ROWS_WHOLE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void fkl_topk_retry_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K, NT);
  const RetryList list(p.workspace, p.n_rows, p.parts);
  const unsigned n = *list.count;
#pragma unroll 1
  for (unsigned e = blockIdx.x; e < n; e += gridDim.x) {
    fkl_topk_part_again<Tag, NT, NCH, J, MULTI, RAG>(p, s, list.entries[e]);
    __syncthreads();      // LDS is reused by the next entry
  }
}

// ---------------------------------------------------------------------------------------
// Forward KL, streaming: any V, any alignment; the row is read twice (second read mostly L2 / MALL).
// MODE as for row_stats_streamed; MODE 2 needs the gradient row to sit on the 16-byte grid as the
// logits row does (same address modulo 16), so that the chunks of both line up.
// ---------------------------------------------------------------------------------------
template <class Tag, int NT, int MODE>
__global__ __launch_bounds__(NT) void fkl_topk_stream_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K);
  using C = Chunk<Tag>;
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  const int64_t V = p.V;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  const RowSplit<Tag> sp(row, V, MODE == 2);
  float tlse = -INFINITY;
  if (trow >= 0) tlse = stage_teacher<Tag, NT>(p, s, trow, row, 0, (int)V);
  if (tlse == -INFINITY) {
    if (grow) {
      if (MODE != 0) {
        zero_row<Tag, NT>(grow + (int64_t)sp.head * Tag::bytes, sp.nbody);
        if (MODE == 2 && tid < sp.leftovers()) store_from_float(grow, Tag::id, sp.column(tid), 0.f);
      } else {
        for (int64_t j = tid; j < V; j += NT) store_from_float(grow, Tag::id, j, 0.f);
      }
    }
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  float B, Q;
  fkl_partials<NT>(p, s, 0, (int)V, B, Q);
  const float a = p.inv_T_s * LOG2E;
  float mx, sm;
  row_stats_streamed<Tag, NT, MODE>(row, V, a, s.red, mx, sm);
  const float b = mx * a + fast_log2(sm);
  if (tid == 0 && p.row_loss) p.row_loss[r] = B + (b * LN2) * Q;

  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
    if (MODE != 0) {
      const char* body = row + (int64_t)sp.head * Tag::bytes;
      char* gbody = grow + (int64_t)sp.head * Tag::bytes;
      for (int64_t ch = tid; ch < sp.nbody; ch += NT) {
        float f[C::N];
        C::unpack(*reinterpret_cast<const u32x4*>(body + ch * 16), f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = fast_exp2(fmaf(f[e], a, -b)) * c;
        store16_stream(gbody + ch * 16, C::pack(f));
      }
      if (MODE == 2 && tid < sp.leftovers()) {
        const int64_t j = sp.column(tid);
        store_from_float(grow, Tag::id, j, fast_exp2(fmaf(load_as_float(row, Tag::id, j), a, -b)) * c);
      }
    } else {
      for (int64_t j = tid; j < V; j += NT)
        store_from_float(grow, Tag::id, j, fast_exp2(fmaf(load_as_float(row, Tag::id, j), a, -b)) * c);
    }
    __syncthreads();
    fkl_sparse_fix<Tag, NT>(s, grow, 0, (int)V, a, b, c, (p.flags & DL_TOPK_UNIQUE_IDS) != 0);
  }
}

// ---------------------------------------------------------------------------------------
// Reverse KL on the teacher's support: K gathered logits per row, gradient = zero row + K values.
// ---------------------------------------------------------------------------------------
// MODE 0: element-wise stores.  MODE 1: gradient rows on the 16-byte grid, a whole number of chunks long.
// MODE 2: any other gradient row: its 16-byte chunks by vector stores (the teacher ids counted from the
// first of them), the columns before and behind them one by one.
template <class Tag, int NT, int MODE>
__global__ __launch_bounds__(NT) void rkl_topk_kernel(const TopkParams p) {
  constexpr bool VEC = MODE != 0;
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K, NT);
  using C = Chunk<Tag>;
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  const int64_t V = p.V;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  const RowSplit<Tag> sp(grow, V, MODE == 2 && grow);              // the row that is written decides
  char* gbody = grow + (int64_t)sp.head * Tag::bytes;
  correction_clear<NT>(s.head, s.own);
  float tlse = -INFINITY;
  if (trow >= 0) tlse = stage_teacher<Tag, NT>(p, s, trow, row, 0, (int)V);
  // Every store comes after the K logits have been gathered (stage_teacher ends in barriers), so
  // the gradient may be written over the logits.
  if (grow && (!VEC || tlse == -INFINITY)) {
    if (VEC) {
      zero_row<Tag, NT>(gbody, sp.nbody);
      if (MODE == 2 && tid < sp.leftovers()) store_from_float(grow, Tag::id, sp.column(tid), 0.f);
    } else {
      for (int64_t j = tid; j < V; j += NT) store_from_float(grow, Tag::id, j, 0.f);
    }
  }
  if (tlse == -INFINITY) {
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  // student renormalised over the staged ids
  float zm = -INFINITY;
  for (int k = tid; k < s.Kp; k += NT)
    if (s.idx[k] >= 0) zm = fmaxf(zm, s.z[k] * p.inv_T_s);
  zm = block_max<NT>(zm, s.red);
  float part = 0.f;
  for (int k = tid; k < s.Kp; k += NT)
    if (s.idx[k] >= 0) part += expf(s.z[k] * p.inv_T_s - zm);
  const float slse = zm + logf(block_sum<NT>(part, s.red));
  part = 0.f;
  for (int k = tid; k < s.Kp; k += NT) {
    if (s.idx[k] >= 0) {
      const float sp = s.z[k] * p.inv_T_s - slse;
      const float d = sp - s.t[k];
      const float rk = expf(sp);
      part += rk * d;
      s.q[k] = rk;      // student mass on the support
      s.z[k] = d;       // log ratio
    }
  }
  const float rkl = block_sum<NT>(part, s.red);     // barriers inside publish s.t / s.z
  if (tid == 0 && p.row_loss) p.row_loss[r] = rkl;
  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
    __syncthreads();    // zero fill precedes the sparse values (scalar path); s.q / s.z complete
    for (int k = tid; k < s.Kp; k += NT) {
      const int id = s.idx[k];
      if (id < 0) continue;
      if (VEC) {
        // placed by the thread that writes the column's chunk; columns beside the body are left to the last step
        const int64_t idb = (int64_t)id - sp.head;
        if (idb >= 0 && idb < sp.nbody * C::N) correction_link<Tag, NT>(s.head, s.own, s.next, k, (int)idb);
      } else {
        float g = 0.f;
        for (int j = 0; j < s.Kp; ++j) g += (s.idx[j] == id) ? s.q[j] * (s.z[j] - rkl) : 0.f;
        store_from_float(grow, Tag::id, id, g * c);
      }
    }
    if (VEC) {
      // the row of zeros, each chunk written once with the support's values already in place
      __syncthreads();
      const unsigned mine = s.own[tid];
      const int64_t nch = sp.nbody;
      const auto term = [&](int k) { return s.q[k] * (s.z[k] - rkl); };
      const auto value = [&](int, float g) { return g * c; };
      unsigned repeats = 0u;
      int n_own = 0;
      for (int64_t ch = tid, i = 0; ch < nch; ch += NT, ++i) {
        float f[C::N];
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = 0.f;
        if (mine & (1u << (i & 31)))
          if (correction_apply<Tag, NT>(s.head, s.next, s.idx, sp.head, (int)i, f, term, value)) repeats |= 1u << (i & 31);
        store16_stream(gbody + ch * 16, C::pack(f));
        n_own = (int)i + 1;
      }
      if (repeats)
        correction_repeats<Tag, NT>(s.head, s.next, s.idx, sp.head, repeats, n_own, term, value,
                                    [&](int column, float v) { store_from_float(grow, Tag::id, column, v); });
      if (MODE == 2 && tid < sp.leftovers()) {
        const int64_t j = sp.column(tid);
        float g = 0.f;
        for (int k = 0; k < s.Kp; ++k) g += (s.idx[k] == j) ? term(k) : 0.f;
        store_from_float(grow, Tag::id, j, g * c);
      }
    }
  }
}

// clears the `ready` words of the split kernel's workspace (a template only so that it may live in a header)
template <int NT>
__global__ __launch_bounds__(NT) void clear_workspace_kernel(u32x4* ws, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i < n16) ws[i] = u32x4{0u, 0u, 0u, 0u};
}

// ---------------------------------------------------------------------------------------
// host dispatch
// ---------------------------------------------------------------------------------------
// Register slots for the entries of a row: J of fkl_topk_reg_kernel.  One stored teacher: 1 or 3 slots
// of NT entries, else 0 (staged by a loop).  Prepared teachers (MULTI): the slots the buckets were laid
// out for, cap0 / NT (1, 2, 4 or 8: bucket_slots).
template <int NT, bool MULTI>
static int entry_slots(const TopkParams& p) {
  if (MULTI) return p.bk.cap0 / NT;
  const int Kp = (p.K + 15) & ~15;
  return Kp <= NT ? 1 : Kp <= 3 * NT ? 3 : 0;
}

// Launches kernel template KERNEL<J, MULTI> for the slot count of this call.
#define DL_LAUNCH_BY_SLOTS(KERNEL_J, grid)                                                                      \
  {                                                                                                             \
    const int j = entry_slots<NT, MULTI>(p);                                                                    \
    const size_t lds = TopkLds::bytes(p.K, NT);                                                                 \
    if constexpr (MULTI) {                                                                                      \
      if (j == 1) hipLaunchKernelGGL((KERNEL_J(1)), dim3(grid), dim3(NT), lds, st, p);                          \
      if constexpr (2 * NT <= DL_MAX_TOPK)                                                                      \
        if (j == 2) hipLaunchKernelGGL((KERNEL_J(2)), dim3(grid), dim3(NT), lds, st, p);                        \
      if constexpr (4 * NT <= DL_MAX_TOPK)                                                                      \
        if (j == 4) hipLaunchKernelGGL((KERNEL_J(4)), dim3(grid), dim3(NT), lds, st, p);                        \
      if constexpr (8 * NT <= DL_MAX_TOPK)                                                                      \
        if (j == 8) hipLaunchKernelGGL((KERNEL_J(8)), dim3(grid), dim3(NT), lds, st, p);                        \
    } else {                                                                                                    \
      if (j == 1) hipLaunchKernelGGL((KERNEL_J(1)), dim3(grid), dim3(NT), lds, st, p);                          \
      else if (j == 3) hipLaunchKernelGGL((KERNEL_J(3)), dim3(grid), dim3(NT), lds, st, p);                     \
      else hipLaunchKernelGGL((KERNEL_J(0)), dim3(grid), dim3(NT), lds, st, p);                                 \
    }                                                                                                           \
  }

template <class Tag, int NT, int NCH, bool SPLIT, bool MULTI, int RAG>
static void launch_reg_j(const TopkParams& p, unsigned grid, hipStream_t st) {
#define DL_REG_KERNEL(J) fkl_topk_reg_kernel<Tag, NT, NCH, SPLIT, J, MULTI, RAG>
  DL_LAUNCH_BY_SLOTS(DL_REG_KERNEL, grid)
#undef DL_REG_KERNEL
}

// one workgroup per row, rows of any alignment and length (one stored teacher)
template <class Tag, int NT, int NCH>
static int launch_reg_any(const TopkParams& p, hipStream_t st) {
  constexpr bool MULTI = false;
  const unsigned grid = xcd_banded_grid(p.n_rows);
#define DL_REG_ANY_KERNEL(J) fkl_topk_reg_kernel<Tag, NT, NCH, false, J, false, ROWS_ANY>
  DL_LAUNCH_BY_SLOTS(DL_REG_ANY_KERNEL, grid)
#undef DL_REG_ANY_KERNEL
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

template <class Tag, int NT, int NCH, bool MULTI, int RAG>
static void launch_retry_j(const TopkParams& p, unsigned grid, hipStream_t st) {
#define DL_RETRY_KERNEL(J) fkl_topk_retry_kernel<Tag, NT, NCH, J, MULTI, RAG>
  DL_LAUNCH_BY_SLOTS(DL_RETRY_KERNEL, grid)
#undef DL_RETRY_KERNEL
}
#undef DL_LAUNCH_BY_SLOTS

static int launch_status() { return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH; }

template <class Tag, int NT, int NCH, bool MULTI, int RAG>
static int launch_reg(const TopkParams& p, hipStream_t st) {
  launch_reg_j<Tag, NT, NCH, false, MULTI, RAG>(p, xcd_banded_grid(p.n_rows), st);
  return launch_status();
}

// 16-byte words at the head of the exchange workspace that must be zero when the split kernels start:
// one PartStats per (row, part), then the retry counter
static int64_t split_clear_words(int64_t n_rows, int parts) { return n_rows * parts + 1; }

// `cleared`: an earlier launch on the same stream has already zeroed those words
template <class Tag, int NT, int NCH, bool MULTI, int RAG>
static int launch_split(TopkParams p, int parts, hipStream_t st, bool cleared) {
  p.parts = parts;
  const int64_t n16 = split_clear_words(p.n_rows, parts);
  if (!cleared)
    hipLaunchKernelGGL(clear_workspace_kernel<256>, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<u32x4*>(p.workspace), n16);
  launch_reg_j<Tag, NT, NCH, true, MULTI, RAG>(p, (unsigned)((p.n_rows + 7) / 8 * 8 * parts), st);
  launch_retry_j<Tag, NT, NCH, MULTI, RAG>(p, (unsigned)std::min<int64_t>(p.n_rows * parts, 256), st);
  return launch_status();
}

// Number of column parts a row of `nch` 16-byte chunks is cut into (1 = one workgroup per row).
// Rows of up to 1024 x 16 chunks are cut into parts of 256 x 16 chunks, as many as hold columns (a
// part without columns would have no maximum to publish); `forced` (the DL_TOPK_PARTS field of the
// call's flags) = 1, 2 or 4 overrides that for such rows where every part still gets columns.
static int split_parts(int64_t nch, int forced, bool fine = false) {
  if (fine && nch > 256 * 4 && nch <= (int64_t)MAX_PARTS * 256 * 4) return (int)((nch + 256 * 4 - 1) / (256 * 4));
  if (nch <= 512 * 16) return 1;
  const int parts = (int)((nch + 256 * 16 - 1) / (256 * 16));      // 3 .. MAX_COARSE_PARTS parts of 256 x 16 chunks
  if (nch > 1024 * 16) return parts;
  if (forced == 1 || forced == 2 || (forced == 4 && parts == 4)) return forced;
  return parts;
}

// The register kernel that serves rows of `nch` 16-byte chunks of `bytes`-wide logits: threads per
// workgroup, chunks per thread, column parts per row (parts > 1: the split kernels, which need the
// exchange workspace: `split_ok`).  NT == 0: none (rows too wide: the streaming kernel).
struct FklShape { int NT, NCH, parts; };
static FklShape fkl_shape(int64_t nch, int bytes, int forced_parts, bool split_ok, bool fine = false, bool thirteen = false) {
  if (nch > (int64_t)MAX_COARSE_PARTS * 256 * 16) return {0, 0, 0};
  if (fine && split_ok && nch > 256 * 4 && nch <= (int64_t)MAX_PARTS * 256 * 4) return {256, 4, split_parts(nch, forced_parts, true)};
  if (nch <= 256 * 4) return {256, 4, 1};
  if (nch <= 256 * 8) return {256, 8, 1};
  // 4-byte logits: 8 chunks per thread from twice the threads keep the corrections in registers
  if (nch <= 256 * 16) return bytes == 4 ? FklShape{512, 8, 1} : FklShape{256, 16, 1};
  // two-byte rows of up to 53248 columns (the 50k vocabularies): 13 chunks per thread.  A workgroup's waves are
  // filled one after the other and the full ones set its time: 13 sweeps instead of 16
  // (16384 x 50304 bf16: 64.6 -> 68.3 % of the HBM peak, 51200 columns: 69 %)
  if (thirteen && bytes != 4 && nch <= 512 * 13) return {512, 13, 1};
  if (nch <= 512 * 16) return {512, 16, 1};
  const int parts = split_parts(nch, forced_parts);
  // The widest rows in half as many parts of 512 threads: fewer partners to wait for.  Measured at 8192
  // rows: four-byte rows of 6 to 8 parts of 256 threads gain 4-11 % that way, two-byte rows of 8 parts
  // 4 %; two-byte rows of 5 to 7 parts lose up to 8 % (the last, partly filled part gets larger).
  if (split_ok && nch > 1024 * 16 && (bytes == 4 ? parts >= 6 : parts == 8)) return {512, 16, (parts + 1) / 2};
  if (parts == 2 && split_ok) return {512, 16, 2};
  if (parts >= 3 && split_ok) {
    // rows that do not fill their parts: as few chunks per thread as hold the row (13 to 15), the parts then equally
    // full -- every wave of every part carries the same share, and that share sets the row's time
    const int64_t per_thread = (nch + (int64_t)parts * 256 - 1) / ((int64_t)parts * 256);
    if (thirteen && per_thread < 16) return {256, per_thread < 13 ? 13 : (int)per_thread, parts};
    return {256, 16, parts};
  }
  if (nch <= 1024 * 16) return {1024, 16, 1};      // no workspace: one workgroup per row
  return {0, 0, 0};
}

// MULTI has no streaming form: the caller checks fkl_shape first.
// RAG = ROWS_WHOLE: `aligned` tells whether the rows are whole chunks on the 16-byte grid (else: the unaligned
// register kernels or the streaming kernel).  RAG = ROWS_TAIL: rows on the grid that end inside a chunk
// (`aligned` is true); the same shapes as whole rows of ceil(V / chunk) chunks.
template <class Tag, bool MULTI, int RAG = ROWS_WHOLE>
static int launch_fkl(const TopkParams& p, bool aligned, int64_t ws_bytes, hipStream_t st, bool ws_cleared = false) {
  const int64_t nch = RAG == ROWS_TAIL ? (p.V + Tag::epc - 1) / Tag::epc : p.V / Tag::epc;
  const int forced = (p.flags >> DL_TOPK_PARTS_SHIFT) & 15;
  const bool fine = !MULTI && (p.flags & DL_TOPK_FINE_PARTS) != 0 &&
                    ws_bytes >= RetryList::bytes(p.n_rows, split_parts(nch, forced, true));
  // the shape a workspace would allow; without room for that shape's records, the shape that needs none
  const FklShape wish = aligned ? fkl_shape(nch, Tag::bytes, forced, true, fine, !MULTI) : FklShape{0, 0, 0};
  const bool split_ok = p.workspace && ws_bytes >= RetryList::bytes(p.n_rows, wish.parts) && p.n_rows * wish.parts <= 0x7fffffffLL;
  const FklShape sh = !aligned || wish.parts <= 1 || split_ok ? wish : fkl_shape(nch, Tag::bytes, forced, false, fine, !MULTI);
  switch (sh.NT * 100 + sh.NCH) {
    case 256 * 100 + 4:
      if constexpr (!MULTI)
        if (sh.parts > 1) return launch_split<Tag, 256, 4, MULTI, RAG>(p, sh.parts, st, ws_cleared);
      return launch_reg<Tag, 256, 4, MULTI, RAG>(p, st);
    case 256 * 100 + 8: return launch_reg<Tag, 256, 8, MULTI, RAG>(p, st);
    case 512 * 100 + 8:
      if constexpr (Tag::bytes == 4) return launch_reg<Tag, 512, 8, MULTI, RAG>(p, st);
      break;
    case 256 * 100 + 16:
      if (sh.parts > 1) return launch_split<Tag, 256, 16, MULTI, RAG>(p, sh.parts, st, ws_cleared);
      if constexpr (Tag::bytes != 4) return launch_reg<Tag, 256, 16, MULTI, RAG>(p, st);
      break;
    case 512 * 100 + 13:
      if constexpr (Tag::bytes != 4 && !MULTI) return launch_reg<Tag, 512, 13, MULTI, RAG>(p, st);
      break;
    case 256 * 100 + 13:
      if constexpr (!MULTI) return launch_split<Tag, 256, 13, MULTI, RAG>(p, sh.parts, st, ws_cleared);
      break;
    case 256 * 100 + 14:
      if constexpr (!MULTI) return launch_split<Tag, 256, 14, MULTI, RAG>(p, sh.parts, st, ws_cleared);
      break;
    case 256 * 100 + 15:
      if constexpr (!MULTI) return launch_split<Tag, 256, 15, MULTI, RAG>(p, sh.parts, st, ws_cleared);
      break;
    case 512 * 100 + 16:
      return sh.parts > 1 ? launch_split<Tag, 512, 16, MULTI, RAG>(p, sh.parts, st, ws_cleared) : launch_reg<Tag, 512, 16, MULTI, RAG>(p, st);
    case 1024 * 100 + 16: return launch_reg<Tag, 1024, 16, MULTI, RAG>(p, st);
    default: break;
  }
  if (MULTI) return aligned ? DL_ERR_LIMIT : DL_ERR_ALIGN;
  // rows off the 16-byte grid: the streaming kernel moves their chunks by aligned vector accesses if logits
  // and gradient rows share their address modulo 16 (the same pitch from 16-byte aligned bases, or the
  // gradient written over the logits)
  const bool same_phase = !p.grad || (reinterpret_cast<uintptr_t>(p.logits) % 16 == reinterpret_cast<uintptr_t>(p.grad) % 16 &&
                                      ((p.row_stride - p.grad_stride) * Tag::bytes) % 16 == 0);
  if constexpr (!MULTI && RAG == ROWS_WHOLE) {
    if (!aligned) {
      // ... or, as far as one workgroup holds a row, the register kernels with unaligned accesses.  Measured
      // (16384 x 32100 bf16: 0.47 ms against 0.75 ms streaming; 16384 x 50257: 1.27 against 0.92): up to
      // 256 x 16 chunks they win; the 512 x 16 shape spills under the extra addressing and only beats the
      // element-wise kernel, which rows on different phases would otherwise take.
      // Beyond 256 x 16 chunks: column parts of that shape (parts of a row start a whole number of chunks behind the
      // row's first element, wherever that lies), where a workspace for their exchange came along.
      const int64_t nch_any = (p.V + Tag::epc - 1) / Tag::epc;
      const int parts_any = (int)((nch_any + 256 * 16 - 1) / (256 * 16));
      if (parts_any >= 2 && parts_any <= MAX_COARSE_PARTS && p.workspace && ws_bytes >= RetryList::bytes(p.n_rows, parts_any) &&
          p.n_rows * parts_any <= 0x7fffffffLL)
        return launch_split<Tag, 256, 16, false, ROWS_ANY>(p, parts_any, st, ws_cleared);
      const FklShape any = fkl_shape(nch_any, Tag::bytes, 0, false);
      if (any.parts == 1) switch (any.NT * 100 + any.NCH) {
        case 256 * 100 + 4: return launch_reg_any<Tag, 256, 4>(p, st);
        case 256 * 100 + 8: return launch_reg_any<Tag, 256, 8>(p, st);
        case 512 * 100 + 8:
          if constexpr (Tag::bytes == 4) return launch_reg_any<Tag, 512, 8>(p, st);
          break;
        case 256 * 100 + 16:
          if constexpr (Tag::bytes != 4) return launch_reg_any<Tag, 256, 16>(p, st);
          break;
        case 512 * 100 + 16:
          if (!same_phase) return launch_reg_any<Tag, 512, 16>(p, st);
          break;
        default: break;
      }
    }
  }
  if (aligned && RAG == ROWS_WHOLE) {
    hipLaunchKernelGGL((fkl_topk_stream_kernel<Tag, 1024, 1>), dim3(xcd_banded_grid(p.n_rows)), dim3(1024),
                       TopkLds::bytes(p.K), st, p);
  } else if (same_phase) {
    hipLaunchKernelGGL((fkl_topk_stream_kernel<Tag, 1024, 2>), dim3(xcd_banded_grid(p.n_rows)), dim3(1024),
                       TopkLds::bytes(p.K), st, p);
  } else {
    hipLaunchKernelGGL((fkl_topk_stream_kernel<Tag, 1024, 0>), dim3(xcd_banded_grid(p.n_rows)), dim3(1024),
                       TopkLds::bytes(p.K), st, p);
  }
  return launch_status();
}

// The ROWS_TAIL instantiations of launch_fkl live in translation units of their own (topk_div_tail.hip,
// topk_multi_tail.hip), so that they compile beside the others.
int launch_fkl_tail(int logits_dtype, const TopkParams& p, int64_t ws_bytes, hipStream_t st);
int launch_fkl_tail_multi(int logits_dtype, const TopkParams& p, int64_t ws_bytes, hipStream_t st, bool ws_cleared);

template <class Tag>
static hipError_t launch_rkl(const TopkParams& p, bool aligned, hipStream_t st) {
  // the logits are only gathered from; what is written decides: MODE 2 takes any gradient row
  if (aligned)
    hipLaunchKernelGGL((rkl_topk_kernel<Tag, 256, 1>), dim3(xcd_banded_grid(p.n_rows)), dim3(256),
                       TopkLds::bytes(p.K, 256), st, p);
  else
    hipLaunchKernelGGL((rkl_topk_kernel<Tag, 256, 2>), dim3(xcd_banded_grid(p.n_rows)), dim3(256),
                       TopkLds::bytes(p.K, 256), st, p);
  return hipGetLastError();
}

// Polls a part of a split row waits for its partners' records before it defers itself to the second launch.
constexpr int SPIN_LIMIT = 20000;

}  // namespace dl


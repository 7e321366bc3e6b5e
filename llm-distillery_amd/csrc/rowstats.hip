// Two-phase path for losses whose per-row weights depend on all rows (the reference's
// alpha-weighted composite): phase 1 returns, per row, the full-vocabulary log-sum-exp and the
// scaled logits at the teacher's ids; the caller combines them (K-wide work) and asks phase 2 for
//     grad[r, j] = ( a_r * softmax(z_r)_j + sum_k c_rk [j == idx_rk] ) * inv_T
// where a_r = dL/d lse_r and c_rk = dL/d zk_rk.  Phase 1 is a read-only streaming reduction,
// phase 2 an element-wise sweep (read row, write gradient) plus K sparse additions.
#include "composite.hpp"

namespace dl {

struct StatsParams {
  const void* logits; int64_t row_stride; int64_t n_rows; int64_t V;
  const int32_t* row_map; const void* t_idx; int t_idx_itype; int K; int64_t n_trows;
  float inv_T;
  float* lse; float* zk;                               // outputs of phase 1 / inputs of phase 2
  const float* coef_lse; const float* coef_zk;         // phase 2
  void* grad; int64_t grad_stride;
};

// ---- phase 1: lse_r = logsumexp_j(x_rj * inv_T),  zk_rk = x[r, idx_rk] * inv_T ------------------
// MODE 0: element-wise loads (rows that are not even element-aligned never get here; kept for reference
// and for rows shorter than a chunk).  MODE 1: rows on the 16-byte grid, a whole number of chunks long.
// MODE 2: any other row: its 16-byte chunks by vector loads, the elements before and behind them one by one.
//
// STASH: the logits at the teacher's ids are not fetched by loads of their own (K random reads of cold lines per
// row, which the sweep then fetches a second time: a quarter more traffic and 9 of the kernel's 50 us on 2048
// rows of 32000 fp32 columns with K = 400) but taken from the sweep itself.  Chunk c of the body belongs to
// thread c % NT in its round c / NT; the ids set one bit per (thread, round) in LDS, a scan over the threads'
// bit counts gives every marked chunk a slot, the sweep drops the marked chunks (16 bytes, as loaded) into their
// slots on its way, and behind the sweep every entry reads its element from its chunk's slot.  At most 64 rounds
// (64 * NT chunks per row) and one slot per entry (K * 16 bytes of LDS from the launch).
constexpr int STASH_ROUNDS = 64;
constexpr int STASH_MAX_K = 1024;

//
// RECORD (with STASH): the row's record of the composite loss (composite_row_record, there by one wave of a launch
// of its own) is made here, by the whole workgroup, behind the sweep: the teacher's K values are fetched before the
// sweep, the logits at its ids are in LDS when the sweep ends, so the record costs three rounds of workgroup
// reductions and no memory round trip.  K <= STASH_MAX_K: at most STASH_MAX_K / NT entries per thread.
template <class Tag, int NT, int MODE, bool STASH, bool RECORD>
__device__ __forceinline__ void rowstats_row(const StatsParams& p, const CompositeParams* cp) {
  static_assert(!RECORD || STASH, "the record is made from the logits the sweep leaves in LDS");
  constexpr int E = STASH_MAX_K / NT;
  __shared__ float red[64];
  __shared__ unsigned long long s_bits[STASH ? NT : 1];
  __shared__ int s_pre[STASH ? NT : 1];
  __shared__ int s_wave[STASH ? NT / 64 : 1];
  extern __shared__ __align__(16) unsigned char smem[];        // STASH: K slots of 16 bytes
  using C = Chunk<Tag>;
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) return;
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  const float a = p.inv_T * LOG2E;
  float m = -INFINITY, sm = 0.f;
  const auto one = [&](float f) {
    if (f > m) { sm *= fast_exp2((m - f) * a); m = f; }
    if (f > -INFINITY) sm += fast_exp2(fmaf(f, a, -m * a));
  };
  unsigned traw[RECORD ? E : 1];      // the teacher's values as stored, converted behind the sweep: all loads in flight together
  if constexpr (RECORD) {
    const int64_t at0 = trow * p.K;
    if (cp->t_val_dtype == F32) {
#pragma unroll
      for (int j = 0; j < E; ++j) traw[j] = reinterpret_cast<const unsigned*>(cp->t_val)[at0 + (tid + j * NT < p.K ? tid + j * NT : 0)];
    } else {
#pragma unroll
      for (int j = 0; j < E; ++j) traw[j] = reinterpret_cast<const unsigned short*>(cp->t_val)[at0 + (tid + j * NT < p.K ? tid + j * NT : 0)];
    }
  }
  if constexpr (!STASH) {
    for (int k = tid; k < p.K; k += NT) {
      const int64_t id = load_index(p.t_idx, p.t_idx_itype, trow * p.K + k);
      p.zk[trow * p.K + k] = (id >= 0 && id < p.V) ? load_as_float(row, Tag::id, id) * p.inv_T : 0.f;
    }
  }
  if (MODE != 0) {
    const RowSplit<Tag> sp(row, p.V, MODE == 2);
    const char* body = row + (int64_t)sp.head * Tag::bytes;
    const int64_t nch = sp.nbody;
    u32x4* stash = reinterpret_cast<u32x4*>(smem);
    unsigned long long mybits = 0;
    int slot = 0;
    int64_t idv[RECORD ? E : 1];      // RECORD: the thread's teacher ids, its row's label and whether that counts: known
    bool want = false;                // before the sweep, so that the record behind it waits for no load
    int64_t label = -1;
    if constexpr (STASH) {
      s_bits[tid] = 0;
      __syncthreads();
      const auto mark = [&](int64_t id) {
        const int64_t rel = id - sp.head;
        if (rel >= 0 && rel < nch * C::N) {
          const int ch = (int)(rel / C::N);
          atomicOr(&s_bits[ch % NT], 1ull << (ch / NT));
        }
      };
      if constexpr (RECORD) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
          const int k = tid + j * NT;
          idv[j] = load_index(p.t_idx, p.t_idx_itype, trow * p.K + (k < p.K ? k : 0));
        }
        const int c = convo_of_row(cp->off, cp->n_convos, trow);
        const int li = (int)(trow - cp->off.row(c));
        want = li < cp->off.label(c + 1) - cp->off.label(c);
        if (want) {
          label = cp->labels[cp->off.label(c) + li];
          for (int av = cp->off.avoid(c); av < cp->off.avoid(c + 1); ++av) want = want && (load_index(cp->avoid, cp->avoid_itype, av) != li);
        }
#pragma unroll
        for (int j = 0; j < E; ++j) {
          if (tid + j * NT < p.K) mark(idv[j]);
          else idv[j] = -1;
        }
      } else {
        for (int k = tid; k < p.K; k += NT) mark(load_index(p.t_idx, p.t_idx_itype, trow * p.K + k));
      }
      __syncthreads();
      mybits = s_bits[tid];
      const int cnt = __popcll(mybits);
      int inc = cnt;                                         // inclusive scan over the wave, then over the waves
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(inc, d, 64);
        if ((tid & 63) >= d) inc += up;
      }
      if ((tid & 63) == 63) s_wave[tid >> 6] = inc;
      __syncthreads();
      int before = 0;
#pragma unroll
      for (int w = 0; w < NT / 64; ++w) before += (w < (tid >> 6)) ? s_wave[w] : 0;
      slot = before + inc - cnt;
      s_pre[tid] = slot;
    }
    for (int64_t c0 = 0; c0 < nch; c0 += 4 * NT) {          // four 16-byte loads in flight per thread
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t ch = c0 + (int64_t)u * NT + tid;
        // streamed, not cached: with cached loads the kernel is slower, whether or not gathers follow that could hit
        v[u] = ch < nch ? load16_stream(body + ch * 16) : C::neg_inf();
      }
      float cm = -INFINITY;
      float f[4][C::N];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        C::unpack(v[u], f[u]);
#pragma unroll
        for (int e = 0; e < C::N; ++e) cm = fmaxf(cm, f[u][e]);
      }
      if constexpr (STASH) {
        const unsigned four = (unsigned)(mybits >> (c0 / NT)) & 15u;
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (four >> u & 1) stash[slot++] = v[u];
      }
      if (cm > m) { sm *= fast_exp2((m - cm) * a); m = cm; }
      const float mb = m * a;
      if (m > -INFINITY) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[u][e], a, -mb));
      }
    }
    if (MODE == 2 && tid < sp.leftovers()) one(load_as_float(row, Tag::id, sp.column(tid)));
    const float mx = block_max<NT>(m, red);
    sm = (m == -INFINITY) ? 0.f : sm * fast_exp2((m - mx) * a);
    sm = block_sum<NT>(sm, red);
    const float lse = (mx * a + fast_log2(sm)) * LN2;
    if (tid == 0) p.lse[trow] = lse;
    if constexpr (STASH) {
      __syncthreads();
      // the logit at teacher entry k out of its chunk's slot (the few columns before and behind the body: from memory)
      const auto logit_at = [&](int64_t id) {
        const int64_t rel = id - sp.head;
        float z = 0.f;
        if (rel >= 0 && rel < nch * C::N) {
          const int ch = (int)(rel / C::N), t = ch % NT, j = ch / NT;
          const int at = s_pre[t] + __popcll(s_bits[t] & ((1ull << j) - 1ull));
          const int e = at * C::N + (int)(rel % C::N);
          if constexpr (Tag::bytes == 4) z = reinterpret_cast<const float*>(smem)[e];
          else z = load_as_float(reinterpret_cast<const unsigned short*>(smem) + e, Tag::id, 0);
        } else if (id >= 0 && id < p.V) {
          z = load_as_float(row, Tag::id, id);
        }
        return z * p.inv_T;
      };
      if constexpr (!RECORD) {
        for (int k = tid; k < p.K; k += NT) p.zk[trow * p.K + k] = logit_at(load_index(p.t_idx, p.t_idx_itype, trow * p.K + k));
      } else {
        const int K = p.K;
        float tv[E], zv[E];
#pragma unroll
        for (int j = 0; j < E; ++j) {
          const int k = tid + j * NT;
          tv[j] = zv[j] = -INFINITY;
          if (j * NT >= K) continue;
          if (k < K) {
            zv[j] = logit_at(idv[j]);
            p.zk[trow * K + k] = zv[j];
            const float t = cp->t_val_dtype == F32 ? __uint_as_float(traw[j])
                            : cp->t_val_dtype == BF16 ? __uint_as_float(traw[j] << 16)
                                                      : (float)__builtin_bit_cast(_Float16, (unsigned short)traw[j]);
            tv[j] = t * cp->inv_T_t;
          }
        }
        // the arithmetic of composite_row_record, entry for entry, with the reductions over the workgroup
        float tmax = -INFINITY, zmax = -INFINITY;
#pragma unroll
        for (int j = 0; j < E; ++j) { tmax = fmaxf(tmax, tv[j]); zmax = fmaxf(zmax, zv[j]); }
        block_max2<NT>(tmax, zmax, red);
        // (rounds j that hold no entry at all are skipped by the whole workgroup; exponentials and logarithms by the
        // hardware's base-2 instructions: a few units in the last place, against a record that is good to 1e-6)
        const auto ex = [](float v) { return fast_exp2(v * LOG2E); };
        float tsum = 0.f, zsum = 0.f;
#pragma unroll
        for (int j = 0; j < E; ++j)
          if (j * NT < K) { tsum += ex(tv[j] - tmax); zsum += ex(zv[j] - zmax); }      // exp(-inf) = 0 beyond K
        block_sum2<NT>(tsum, zsum, red);
        const float t_lse = tmax + fast_log2(tsum) * LN2;
        const float z_lse = zmax + fast_log2(zsum) * LN2;
        const float s_lse = z_lse - lse;
        float kl = 0.f, rkl = 0.f, found = -INFINITY;      // found: minus the first entry that carries the label
#pragma unroll
        for (int j = 0; j < E; ++j) {
          const int k = tid + j * NT;
          if (j * NT >= K) continue;
          if (k < K) {
            const float t = tv[j] - t_lse;
            const float sk = zv[j] - lse;
            const float s2 = sk - s_lse;
            kl += ex(t) * (t - sk);
            rkl += ex(s2) * (s2 - t);
            if (want && idv[j] == label) found = fmaxf(found, -(float)k);
          }
        }
        block_sum2<NT>(kl, rkl, red);
        found = block_max<NT>(found, red);
        const int kstar = found == -INFINITY ? -1 : (int)(-found);
#pragma unroll
        for (int j = 0; j < E; ++j)
          if (kstar >= 0 && tid + j * NT == kstar) { red[0] = zv[j] - lse; red[1] = tv[j] - t_lse; }
        __syncthreads();
        if (tid == 0) {
          RowRec rr;
          rr.kl = kl; rr.rkl = rkl; rr.t_lse = t_lse; rr.s_lse = s_lse;
          rr.valid = kstar >= 0 ? 1 : 0;
          rr.kstar = kstar;
          rr.own_s = kstar >= 0 ? red[0] : 0.f;
          rr.own_t = kstar >= 0 ? red[1] : 0.f;
          cp->rec[trow] = rr;
        }
      }
    }
    return;
  } else {
    for (int64_t j = tid; j < p.V; j += NT) one(load_as_float(row, Tag::id, j));
  }
  const float mx = block_max<NT>(m, red);
  sm = (m == -INFINITY) ? 0.f : sm * fast_exp2((m - mx) * a);
  sm = block_sum<NT>(sm, red);
  if (tid == 0) p.lse[trow] = (mx * a + fast_log2(sm)) * LN2;
}

template <class Tag, int NT, int MODE, bool STASH>
__global__ __launch_bounds__(NT) void rowstats_kernel(const StatsParams p) {
  rowstats_row<Tag, NT, MODE, STASH, false>(p, nullptr);
}
template <class Tag, int NT, int MODE>
__global__ __launch_bounds__(NT) void rowstats_record_kernel(const StatsParams p, const CompositeParams cp) {
  rowstats_row<Tag, NT, MODE, true, true>(p, &cp);
}

// ---- phase 2 -------------------------------------------------------------------------------
// One workgroup per (row, column part of NT*NCH chunks).
// Coefficient on the id of entry k, summed over every entry of the row that carries the same id
// (ids of a row may repeat: each such entry then yields the same total).
__device__ __forceinline__ float coef_on_id(const int* s_idx, const float* s_c, int Kp, int k, int id) {
  const int4* ids4 = reinterpret_cast<const int4*>(s_idx);
  int same = 0;
#pragma unroll 4
  for (int j = 0; j < Kp / 4; ++j) {
    const int4 q = ids4[j];
    same += (q.x == id) + (q.y == id) + (q.z == id) + (q.w == id);
  }
  if (same == 1) return s_c[k];
  float cs = 0.f;
  for (int j = 0; j < Kp; ++j) cs += (s_idx[j] == id) ? s_c[j] : 0.f;
  return cs;
}

// correction_apply for a correction that is added to the dense value: element e of chunk i becomes
// dense + coef(k) * scale for the entry k that names it; true if some element is named more than once.
template <class Tag, int NT, class Coef>
__device__ __forceinline__ bool correction_add(const int* head, const int* next, const int* col, int lo, int i,
                                               float (&f)[Chunk<Tag>::N], float scale, Coef coef) {
  using C = Chunk<Tag>;
  unsigned seen = 0u, again = 0u;
  float dense[C::N];
#pragma unroll
  for (int j = 0; j < C::N; ++j) dense[j] = f[j];
  for (int k = head[(i % (CORRECTION_HEADS / NT)) * NT + threadIdx.x]; k >= 0; k = next[k]) {
    const int off = col[k] - lo;
    if (ChunkMap<NT, 0>::reg(off / C::N) != i) continue;
    const int e = off % C::N;
    again |= seen & (1u << e);
    seen |= 1u << e;
    const float c = coef(k) * scale;
#pragma unroll
    for (int j = 0; j < C::N; ++j) f[j] = (j == e) ? dense[j] + c : f[j];
  }
  return again != 0u;
}

// MODE as for phase 1.  MODE 2 needs the gradient row to sit on the 16-byte grid exactly as the logits row does
// (same address modulo 16): the kernel then works on the rows' bodies, with the teacher ids counted
// from the body's first column, and part 0 adds the few columns before and behind the body one by one.
// MODE 3: logits and gradient rows on the 16-byte grid that end inside a chunk (logits[:, :, :crop] of padded
// rows): the ragged chunk is loaded and converted like the others -- its 16 bytes start inside the row and,
// aligned as they are, end inside the row's pitch or at least inside the page of the row's last column; what
// lies behind the row is computed on and dropped -- and stored element by element.
// COMPOSITE: the coefficients are not read but made here, from the row's record and its conversation's
// coefficients (composite_entry_grad; every part of a row makes all K of them, in the same order: the same bits),
// which saves the launch that would write them and the row's coefficient on the log-sum-exp, their sum.
template <class Tag, int NT, int NCH, int MODE, bool COMPOSITE>
__device__ __forceinline__ void rowcoef_grad_part(const StatsParams& p, int parts, const CompositeParams* cp) {
  constexpr bool VEC = MODE != 0;
  __shared__ float red[64];
  extern __shared__ __align__(16) unsigned char smem[];
  using C = Chunk<Tag>;
  const int Kp = (p.K + 15) & ~15;
  int* s_idx = reinterpret_cast<int*>(smem);
  float* s_c = reinterpret_cast<float*>(s_idx + Kp);
  float* s_z = s_c + Kp;
  float* s_val = s_z + Kp;                         // (spare)
  int* s_next = reinterpret_cast<int*>(s_val + Kp);
  int* s_head = s_next + Kp;
  unsigned* s_own = reinterpret_cast<unsigned*>(s_head + CORRECTION_HEADS);
  // Workgroup ids are dealt round-robin to the 8 XCDs: within a group of 8 * parts ids, id t serves
  // row 8 * group + t % 8, part t / 8, so the parts of a row run on one XCD back to back.
  const unsigned grp = blockIdx.x / (8u * parts), t_in = blockIdx.x % (8u * parts);
  const int64_t r = (int64_t)grp * 8 + (t_in & 7u);
  const int h = (int)(t_in >> 3);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  const int64_t per_part = (int64_t)NT * NCH * C::N;                 // columns per part
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  char* grow_all = reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes;
  const char* row_all = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  // what the sweeps below see as the row: all of it, or (MODE 2) its body
  const RowSplit<Tag> sp(row_all, p.V, MODE == 2);
  const int64_t V = MODE == 2 ? sp.nbody * C::N : p.V;
  const int shift = MODE == 2 ? sp.head : 0;                         // column of the row that is column 0 of the sweeps
  char* grow = grow_all + (int64_t)shift * Tag::bytes;
  const char* row = row_all + (int64_t)shift * Tag::bytes;
  const int64_t lo = min(V, h * per_part), hi = min(V, lo + per_part);
  // chunk `ch` of the row: whole, or (MODE 3) the ragged one at the row's end
  const auto put = [&](int64_t ch, const u32x4& v) {
    if (MODE != 3 || (ch + 1) * C::N <= V) store16_stream(grow + ch * 16, v);
    else store_chunk_elementwise<Tag>(grow, (int)ch, (int)V, v);
  };
  if (trow < 0) {
    if (MODE == 3) for (int64_t ch = lo / C::N + tid; ch * C::N < hi; ch += NT) put(ch, u32x4{0u, 0u, 0u, 0u});
    else if (VEC) zero_row<Tag, NT>(grow + lo * Tag::bytes, (hi - lo) / C::N);
    else for (int64_t j = lo + tid; j < hi; j += NT) store_from_float(grow, Tag::id, j, 0.f);
    if (MODE == 2 && h == 0 && tid < sp.leftovers()) store_from_float(grow_all, Tag::id, sp.column(tid), 0.f);
    return;
  }
  const float a = p.inv_T * LOG2E;
  const float lse = p.lse[trow];
  const float b = lse * LOG2E;
  float w = COMPOSITE ? 0.f : p.coef_lse[trow] * p.inv_T;
  RowRec rec{};
  RowCoef rc{};
  float up = 0.f, acc = 0.f;
  if constexpr (COMPOSITE) {
    rec = cp->rec[trow];
    rc = cp->coef[trow];
    up = cp->g_train[convo_of_row(cp->off, cp->n_convos, trow)];
  }
  // Teacher ids, their coefficients and the logits at the ids of this part go to LDS; issued behind
  // the row's own loads so that their latencies overlap instead of trailing the dense sweep.
  auto stage = [&]() {
    for (int k = tid; k < Kp; k += NT) {
      int64_t id = -1;
      float cv = 0.f;
      bool in_row = false;                                           // ids outside the row name no column
      if (k < p.K) {
        id = load_index(p.t_idx, p.t_idx_itype, trow * p.K + k);
        in_row = id >= 0 && id < p.V;
        id -= shift;
        if constexpr (COMPOSITE) {
          cv = composite_entry_grad(*cp, rec, rc, up, lse, trow, k, cp->zk[trow * p.K + k]);
          acc += cv;
        } else {
          cv = p.coef_zk[trow * p.K + k];
        }
      }
      const bool mine = in_row && id >= lo && id < hi;
      if (MODE == 2 && h == 0 && in_row && (id < 0 || id >= V)) {
        // a column before or behind the body: leftover number li is kept as -2 - li for part 0's last step
        const int64_t li = id < 0 ? id + shift : sp.head + (id - V);
        s_idx[k] = -2 - (int)li;
        s_c[k] = cv;
        s_z[k] = 0.f;
        continue;
      }
      s_idx[k] = mine ? (int)id : -1;
      s_c[k] = cv;
      if (!VEC) s_z[k] = mine ? load_as_float(row, Tag::id, id) : 0.f;      // VEC: the column's owner has it in its registers
    }
  };
  if (VEC) {
    const int64_t c_lo = lo / C::N, c_hi = (hi + (MODE == 3 ? C::N - 1 : 0)) / C::N;
    u32x4 v[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int64_t ch = c_lo + (int64_t)i * NT + tid;
      v[i] = ch < c_hi ? load16_stream(row + ch * 16) : C::neg_inf();
    }
    correction_clear<NT>(s_head, s_own);
    stage();
    if constexpr (COMPOSITE) w = -block_sum<NT>(acc, red) * p.inv_T;      // s_k = z_k - lse: d / d lse = -sum_k
    __syncthreads();
    // the columns that carry a teacher entry, handed to the threads that hold them: those add the entry's coefficient
    // to the dense value they have just made
    for (int k = tid; k < Kp; k += NT) {
      const int id = s_idx[k];
      if (id >= 0) correction_link<Tag, NT>(s_head, s_own, s_next, k, id - (int)lo);
    }
    __syncthreads();
    const unsigned mine = s_own[tid];
    const auto coef = [&](int k) { return s_c[k]; };
    // a column named by several entries (the rare path behind the sweep): its dense value made again, the same bits
    const auto value = [&](int k, float cs) {
      return fast_exp2(fmaf(load_as_float(row, Tag::id, s_idx[k]), a, -b)) * w + cs * p.inv_T;
    };
    unsigned repeats = 0u;            // chunks in which an id occurs more than once
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int64_t ch = c_lo + (int64_t)i * NT + tid;
      if (ch < c_hi) {
        float f[C::N];
        C::unpack(v[i], f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = fast_exp2(fmaf(f[e], a, -b)) * w;
        if (mine & (1u << i))
          if (correction_add<Tag, NT>(s_head, s_next, s_idx, (int)lo, i, f, p.inv_T, coef)) repeats |= 1u << i;
        put(ch, C::pack(f));
      }
    }
    if (repeats)
      correction_repeats<Tag, NT>(s_head, s_next, s_idx, (int)lo, repeats, NCH, coef, value,
                                  [&](int column, float g) { store_from_float(grow, Tag::id, column, g); });
    if (MODE == 2 && h == 0 && tid < sp.leftovers()) {
      // a column before or behind the body: dense value plus the coefficients of every entry that names it
      const int64_t j = sp.column(tid);
      float cs = 0.f;
      for (int k = 0; k < Kp; ++k) cs += s_idx[k] == -2 - tid ? s_c[k] : 0.f;
      store_from_float(grow_all, Tag::id, j, fast_exp2(fmaf(load_as_float(row_all, Tag::id, j), a, -b)) * w + cs * p.inv_T);
    }
    return;
  } else {
    stage();
    if constexpr (COMPOSITE) w = -block_sum<NT>(acc, red) * p.inv_T;
    for (int64_t j = lo + tid; j < hi; j += NT)
      store_from_float(grow, Tag::id, j, fast_exp2(fmaf(load_as_float(row, Tag::id, j), a, -b)) * w);
  }
  __syncthreads();          // LDS entries staged; dense stores ordered before the sparse additions
  for (int k = tid; k < Kp; k += NT) {
    const int id = s_idx[k];
    if (id < 0) continue;
    const float dense = fast_exp2(fmaf(s_z[k], a, -b)) * w;
    store_from_float(grow, Tag::id, id, dense + coef_on_id(s_idx, s_c, Kp, k, id) * p.inv_T);
  }
}

template <class Tag, int NT, int NCH, int MODE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void rowcoef_grad_kernel(const StatsParams p, int parts) {
  rowcoef_grad_part<Tag, NT, NCH, MODE, false>(p, parts, nullptr);
}
template <class Tag, int NT, int NCH, int MODE>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void rowcoef_composite_kernel(const StatsParams p, int parts, const CompositeParams cp) {
  rowcoef_grad_part<Tag, NT, NCH, MODE, true>(p, parts, &cp);
}

static bool aligned16(const void* ptr, int64_t stride, int eb) {
  return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (stride * eb) % 16 == 0;
}

// Rows whose addresses differ by a multiple of 16 bytes, row for row: what the kernels that sweep the
// 16-byte chunks inside unaligned rows need of a (logits, gradient) pair.
static bool same_phase16(const void* a, int64_t stride_a, const void* b, int64_t stride_b, int eb) {
  return reinterpret_cast<uintptr_t>(a) % 16 == reinterpret_cast<uintptr_t>(b) % 16 && ((stride_a - stride_b) * eb) % 16 == 0;
}

// phase 1 with the rows' records of the composite loss made at its tail (the caller has checked stash_fits)
static bool stash_fits(int mode, int K, int64_t V, int epc) {
  return mode != 0 && K <= STASH_MAX_K && (V + epc - 1) / epc <= (int64_t)STASH_ROUNDS * 256;
}
template <class Tag>
static hipError_t launch_stats_record(const StatsParams& p, int mode, const CompositeParams& cp, hipStream_t st) {
  const size_t lds = (size_t)p.K * 16;
  const dim3 grid((unsigned)p.n_rows), block(256);
  if (mode == 1) hipLaunchKernelGGL((rowstats_record_kernel<Tag, 256, 1>), grid, block, lds, st, p, cp);
  else hipLaunchKernelGGL((rowstats_record_kernel<Tag, 256, 2>), grid, block, lds, st, p, cp);
  return hipGetLastError();
}

template <class Tag>
static hipError_t launch_stats(const StatsParams& p, int mode, hipStream_t st) {
  // the logits at the teacher's ids out of the sweep where the row's chunks fit the threads' 64 rounds (the bound holds
  // for every row: a peeled head only shortens the body)
  const bool stash = stash_fits(mode, p.K, p.V, Tag::epc);
  const size_t lds = stash ? (size_t)p.K * 16 : 0;
  const dim3 grid((unsigned)p.n_rows), block(256);
  if (mode == 1 && stash) hipLaunchKernelGGL((rowstats_kernel<Tag, 256, 1, true>), grid, block, lds, st, p);
  else if (mode == 2 && stash) hipLaunchKernelGGL((rowstats_kernel<Tag, 256, 2, true>), grid, block, lds, st, p);
  else if (mode == 1) hipLaunchKernelGGL((rowstats_kernel<Tag, 256, 1, false>), grid, block, 0, st, p);
  else if (mode == 2) hipLaunchKernelGGL((rowstats_kernel<Tag, 256, 2, false>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((rowstats_kernel<Tag, 256, 0, false>), grid, block, 0, st, p);
  return hipGetLastError();
}

template <class Tag>
static hipError_t launch_coef(const StatsParams& p, int mode, hipStream_t st, const CompositeParams* cp = nullptr) {
  // 4 chunks per thread: this kernel keeps nothing of the row beyond the chunk it is converting, and a
  // stream that moves few chunks per thread between its loads and its stores runs 6-9 % faster on this
  // device than one that moves 16 (measured on a plain copy as well: 78 % against 70 % of peak)
  constexpr int NT = 512, NCH = 4;
  const int64_t per_part = (int64_t)NT * NCH * Tag::epc;
  const int parts = (int)((p.V + per_part - 1) / per_part);
  const size_t lds = (size_t)((p.K + 15) & ~15) * 20 + (size_t)CORRECTION_HEADS * 4 + (size_t)NT * 4;   // ids, coefficients, logits, values, links; list heads, chunk masks
  const dim3 grid((unsigned)((p.n_rows + 7) / 8 * 8 * parts));
  if (cp) {
    if (mode == 1) hipLaunchKernelGGL((rowcoef_composite_kernel<Tag, NT, NCH, 1>), grid, dim3(NT), lds, st, p, parts, *cp);
    else if (mode == 2) hipLaunchKernelGGL((rowcoef_composite_kernel<Tag, NT, NCH, 2>), grid, dim3(NT), lds, st, p, parts, *cp);
    else if (mode == 3) hipLaunchKernelGGL((rowcoef_composite_kernel<Tag, NT, NCH, 3>), grid, dim3(NT), lds, st, p, parts, *cp);
    else hipLaunchKernelGGL((rowcoef_composite_kernel<Tag, NT, NCH, 0>), grid, dim3(NT), lds, st, p, parts, *cp);
    return hipGetLastError();
  }
  if (mode == 1) hipLaunchKernelGGL((rowcoef_grad_kernel<Tag, NT, NCH, 1>), grid, dim3(NT), lds, st, p, parts);
  else if (mode == 2) hipLaunchKernelGGL((rowcoef_grad_kernel<Tag, NT, NCH, 2>), grid, dim3(NT), lds, st, p, parts);
  else if (mode == 3) hipLaunchKernelGGL((rowcoef_grad_kernel<Tag, NT, NCH, 3>), grid, dim3(NT), lds, st, p, parts);
  else hipLaunchKernelGGL((rowcoef_grad_kernel<Tag, NT, NCH, 0>), grid, dim3(NT), lds, st, p, parts);
  return hipGetLastError();
}

static int check_common(const void* logits, int dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                        const void* t_idx, int itype, int K, int64_t n_trows) {
  if (!logits || (!t_idx && n_trows > 0)) return DL_ERR_NULL;      // no teacher rows: every row is masked
  if (dtype < DL_F32 || dtype > DL_F16 || (itype != DL_I32 && itype != DL_I64)) return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || K <= 0 || n_trows < 0 || row_stride < V) return DL_ERR_SHAPE;
  if (K > DL_MAX_TOPK || V > 0x7fffffffLL || n_rows > 0x7fffffffLL) return DL_ERR_LIMIT;
  return DL_OK;
}

}  // namespace dl

extern "C" int dl_rowstats_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                                const int32_t* row_map, const void* t_idx, int t_idx_itype, int K,
                                int64_t n_teacher_rows, float inv_T, float* lse, float* zk, void* stream) {
  using namespace dl;
  const int rc = check_common(logits, logits_dtype, row_stride, n_rows, V, t_idx, t_idx_itype, K, n_teacher_rows);
  if (rc != DL_OK) return rc;
  if ((!lse || !zk) && n_teacher_rows > 0) return DL_ERR_NULL;
  if (n_rows == 0) return DL_OK;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(logits) % eb != 0) return DL_ERR_ALIGN;
  const int vec = V % (16 / eb) == 0 && aligned16(logits, row_stride, eb) ? 1 : 2;
  StatsParams p{logits, row_stride, n_rows, V, row_map, t_idx, t_idx_itype, K, n_teacher_rows, inv_T, lse, zk,
                nullptr, nullptr, nullptr, 0};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const hipError_t e = logits_dtype == DL_F32 ? launch_stats<TagF32>(p, vec, st)
                       : logits_dtype == DL_BF16 ? launch_stats<TagBF16>(p, vec, st)
                                                 : launch_stats<TagF16>(p, vec, st);
  return e == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_composite_forward_fused(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                                          const int32_t* row_map, int64_t n_teacher_rows, float inv_T, const void* t_val,
                                          int t_val_dtype, float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                          const int64_t* labels, const void* avoid, int avoid_itype, const int32_t* row_off,
                                          const int32_t* label_off, const int32_t* avoid_off, int offsets_on_host,
                                          int n_convos, float alpha, float* lse, float* zk, void* row_records,
                                          void* row_coef, float* out, void* stream) {
  using namespace dl;
  const int rc = check_common(logits, logits_dtype, row_stride, n_rows, V, t_idx, t_idx_itype, K, n_teacher_rows);
  if (rc != DL_OK) return rc;
  if ((!lse || !zk) && n_teacher_rows > 0) return DL_ERR_NULL;
  CompositeParams cp;
  const int st0 = composite_forward_params(cp, lse, zk, t_val, t_val_dtype, inv_T_teacher, t_idx, t_idx_itype, K, labels, avoid,
                                           avoid_itype, row_off, label_off, avoid_off, offsets_on_host, n_convos,
                                           n_teacher_rows, alpha, row_records, row_coef, out);
  if (st0 != DL_OK) return st0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (n_rows > 0) {
    if (reinterpret_cast<uintptr_t>(logits) % eb != 0) return DL_ERR_ALIGN;
    const int vec = V % (16 / eb) == 0 && aligned16(logits, row_stride, eb) ? 1 : 2;
    StatsParams p{logits, row_stride, n_rows, V, row_map, t_idx, t_idx_itype, K, n_teacher_rows, inv_T, lse, zk,
                  nullptr, nullptr, nullptr, 0};
    // every teacher row has its logits row (no map, as many of the one as of the other): the rows' records at the
    // tail of phase 1; else teacher rows without a logits row need records too: the launch of their own
    if (!row_map && n_teacher_rows == n_rows && stash_fits(vec, K, V, 16 / eb)) {
      const hipError_t e = logits_dtype == DL_F32 ? launch_stats_record<TagF32>(p, vec, cp, st)
                           : logits_dtype == DL_BF16 ? launch_stats_record<TagBF16>(p, vec, cp, st)
                                                     : launch_stats_record<TagF16>(p, vec, cp, st);
      if (e != hipSuccess) return DL_ERR_LAUNCH;
    } else {
      const hipError_t e = logits_dtype == DL_F32 ? launch_stats<TagF32>(p, vec, st)
                           : logits_dtype == DL_BF16 ? launch_stats<TagBF16>(p, vec, st)
                                                     : launch_stats<TagF16>(p, vec, st);
      if (e != hipSuccess) return DL_ERR_LAUNCH;
      if (n_teacher_rows > 0) launch_composite_rows_fwd(cp, st);
    }
  } else if (n_teacher_rows > 0) {
    launch_composite_rows_fwd(cp, st);
  }
  launch_composite_convo(cp, st);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_rowcoef_grad_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                                    int64_t V, const int32_t* row_map, const void* t_idx, int t_idx_itype, int K,
                                    int64_t n_teacher_rows, float inv_T, const float* lse, const float* coef_lse,
                                    const float* coef_zk, void* grad, int64_t grad_stride, void* stream) {
  using namespace dl;
  const int rc = check_common(logits, logits_dtype, row_stride, n_rows, V, t_idx, t_idx_itype, K, n_teacher_rows);
  if (rc != DL_OK) return rc;
  if (((!lse || !coef_lse || !coef_zk) && n_teacher_rows > 0) || !grad) return DL_ERR_NULL;
  if (grad_stride < V) return DL_ERR_SHAPE;
  if (n_rows == 0) return DL_OK;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(logits) % eb != 0 || reinterpret_cast<uintptr_t>(grad) % eb != 0) return DL_ERR_ALIGN;
  const bool on_grid = aligned16(logits, row_stride, eb) && aligned16(grad, grad_stride, eb);
  const int vec = on_grid ? (V % (16 / eb) == 0 ? 1 : 3) : same_phase16(logits, row_stride, grad, grad_stride, eb) ? 2 : 0;
  StatsParams p{logits, row_stride, n_rows, V, row_map, t_idx, t_idx_itype, K, n_teacher_rows, inv_T,
                const_cast<float*>(lse), nullptr, coef_lse, coef_zk, grad, grad_stride};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const hipError_t e = logits_dtype == DL_F32 ? launch_coef<TagF32>(p, vec, st)
                       : logits_dtype == DL_BF16 ? launch_coef<TagBF16>(p, vec, st)
                                                 : launch_coef<TagF16>(p, vec, st);
  return e == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_composite_backward_fused(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                                           int64_t V, const int32_t* row_map, int64_t n_teacher_rows, float inv_T,
                                           const void* t_val, int t_val_dtype,
                                           float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                           const int32_t* row_off, int offsets_on_host, int n_convos, const float* lse,
                                           const float* zk, const void* row_records, const void* row_coef,
                                           const float* g_train, void* grad, int64_t grad_stride, void* stream) {
  using namespace dl;
  const int rc = check_common(logits, logits_dtype, row_stride, n_rows, V, t_idx, t_idx_itype, K, n_teacher_rows);
  if (rc != DL_OK) return rc;
  CompositeParams cp;
  const int st0 = composite_backward_params(cp, lse, zk, t_val, t_val_dtype, inv_T_teacher, t_idx, t_idx_itype, K, row_off,
                                            offsets_on_host, n_convos, n_teacher_rows, row_records, row_coef, g_train);
  if (st0 != DL_OK) return st0;
  if (!grad) return DL_ERR_NULL;
  if (grad_stride < V) return DL_ERR_SHAPE;
  if (n_rows == 0) return DL_OK;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(logits) % eb != 0 || reinterpret_cast<uintptr_t>(grad) % eb != 0) return DL_ERR_ALIGN;
  const bool on_grid = aligned16(logits, row_stride, eb) && aligned16(grad, grad_stride, eb);
  const int vec = on_grid ? (V % (16 / eb) == 0 ? 1 : 3) : same_phase16(logits, row_stride, grad, grad_stride, eb) ? 2 : 0;
  StatsParams p{logits, row_stride, n_rows, V, row_map, t_idx, t_idx_itype, K, n_teacher_rows, inv_T,
                const_cast<float*>(lse), nullptr, nullptr, nullptr, grad, grad_stride};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const hipError_t e = logits_dtype == DL_F32 ? launch_coef<TagF32>(p, vec, st, &cp)
                       : logits_dtype == DL_BF16 ? launch_coef<TagBF16>(p, vec, st, &cp)
                                                 : launch_coef<TagF16>(p, vec, st, &cp);
  return e == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

// Cross-tokenizer marginalisation: a dense teacher distribution over the TEACHER vocabulary is
// summed into the student vocabulary along a many-to-one id map,
//     marg[r, s] = sum over { t : t2s[t] == s } of p[r, t],
// and, fused, the reverse KL of the student against that marginal with its gradient.
//
//   * map form (fast): one workgroup per row streams the teacher row once (16-byte loads of the
//     probabilities and of the id map, which stays L2-resident) and accumulates into an LDS copy
//     of the student vocabulary with ds_add_f32.  The order of the additions is not fixed, so the
//     sums agree to fp32 rounding, not bit for bit.
//   * CSR form (deterministic): one thread per student id adds its segment in ascending
//     teacher-id order.
//   * planned form (fast and deterministic): the host lays the map out as a "plan": the teacher
//     vocabulary is cut into tiles; inside a tile every accumulator slot (a student id, or one of
//     the replicas of a student id that many teacher ids map to) belongs to one thread, and for
//     every (tile, wave) the entries of the wave's 64 threads are stored row-wise (64 entries per
//     row, padded to batches of 8 rows), each thread's entries sorted by (slot, t).  The kernel
//     streams a teacher tile into LDS (coalesced), then every thread walks its entries, reads the
//     tile at random (LDS), and adds runs of equal slot into LDS words only it touches in that
//     tile, so no atomics, and the order of additions is fixed: bit-reproducible.  Replicas are
//     folded into their id's slot after the last tile.
//   * fused reverse KL: the marginal never leaves LDS; its logarithm is the teacher row of the
//     dense-divergence sweeps, the student row sits in registers.
#include "dense_div.hpp"

namespace dl {

constexpr int MARG_NT = 1024;
constexpr int MARG_MAX_VS = 36864;          // fp32 marginal of one row in LDS: 144 KiB of the CU's 160
constexpr int MARG_NU = 5;                  // units of 8 student columns per thread in the fused kernel
static_assert(MARG_MAX_VS / 8 <= MARG_NU * MARG_NT, "the student row must fit the registers of the fused kernel");
constexpr int MARG_MAX_DYN_LDS = 160 * 1024 - 1024;   // dynamic LDS a workgroup may request (planned form: marginal + tile)

struct MargParams {
  const void* probs; int p_dtype; int64_t p_stride; int64_t n_rows; int64_t Vt;
  const int32_t* t2s; int64_t Vs;
  float* marg; int64_t marg_stride; int out_log;
  // fused reverse KL
  const void* logits; int s_dtype; int64_t row_stride; int64_t n_srows; const int32_t* row_map;
  float inv_T_s, inv_T_t, grad_scale; float* row_loss; void* grad; int64_t grad_stride;
  // plan (all NULL/0: accumulate with LDS atomics along t2s instead)
  const int32_t* plan_row_off; const uint32_t* plan_ent; int plan_tile;
  const int32_t* plan_fold; int plan_n_fold; int plan_n_extra;       // replica slots behind the marginal and how they fold
  // compact form of the fused reverse KL (Vs_full > 0): Vs counts the student ids the map reaches, `cols` [Vs] names
  // their columns in the logits rows of Vs_full columns (-1: padding), col_src16 [Vs_full] the compact id of every
  // column (0xffff: none); logits and gradient rows are full-width
  const int32_t* cols; const unsigned short* col_src16; int64_t Vs_full;
};

// LDS words of the planned form behind the tile: the marginal and the replica slots, both padded to
// 16 bytes, and one slot per lane for the run totals that are not final yet
constexpr int PLAN_SPARE_SLOTS = 64;
__host__ __device__ inline int64_t plan_slot_words(int64_t Vs, int n_extra) {
  return ((Vs + 3) & ~(int64_t)3) + (((int64_t)n_extra + 3) & ~(int64_t)3) + PLAN_SPARE_SLOTS;
}

// Plan entry of a general list: bit 31 = first entry of a run of one slot in its thread's list of
// the tile; bits 15-30 = the slot on the last entry of the run, the lane's spare slot on the others;
// bits 0-14 = byte offset of the probability inside the tile.  Padding is a first entry on the spare
// slot.  A batch is 8 entries per lane, lane-major: the entries of lane l are dwords [8l, 8l + 8) of
// the batch's 512, fetched with two 16-byte loads.
constexpr int PLAN_SLOT_SHIFT = 15;
constexpr unsigned PLAN_OFFSET_MASK = 0x7ffcu, PLAN_SLOT_MASK = 0xffffu;
constexpr int PLAN_EB = 8;           // entries per batch
// Packed list (every lane holds at most one run, at most 8 entries): 4 dwords per lane, lane-major, one
// 16-byte load.  Every dword holds two 16-bit fields; bits 2-15 of a field are the byte offset of a
// probability inside the tile, or of the zero words behind the tile for padding (first in the lane's
// list); the low two bits of the eight fields together are the lane's slot: field 2j carries slot bits
// 2j and 2j + 1, field 2j + 1 bits 8 + 2j and 9 + 2j.
constexpr int PLAN_PACKED_ROWS = 4;  // rows of 64 dwords a packed list takes in the entry array
constexpr int PLAN_ZERO_WORDS = 4;   // LDS words behind the tile that stay 0

struct PlanBatch { u32x4 lo, hi; };

__device__ __forceinline__ float plan_tile_value(const float* tile, unsigned byte_offset) {
  return *reinterpret_cast<const float*>(reinterpret_cast<const char*>(tile) + byte_offset);
}

// Marginal of one teacher row into marg[0, Vs) (LDS, zeroed here) along a plan; `tile` is LDS
// scratch of plan_tile floats.  fp32 probabilities, 16-byte aligned rows.
//
// The hot loop is straight-line code: per entry a read of the tile, a read of the entry's slot, the
// running sum of the run (restarted where the entry says so) and a store of slot + running sum.
// Only the store of a run's last entry lands in the run's slot; the others go to the lane's spare
// slot, which nobody reads for its value.  A slot belongs to one thread inside a tile and has one
// run per thread and tile, so reading all slots of a batch before its stores changes nothing.
// The run totals are added as slot + (0 + v0 + v1 + ...), in list order.
__device__ __forceinline__ void plan_consume(const PlanBatch& b, const float* tile, float* marg, float& run) {
  const unsigned e[PLAN_EB] = {b.lo.x, b.lo.y, b.lo.z, b.lo.w, b.hi.x, b.hi.y, b.hi.z, b.hi.w};
  float val[PLAN_EB], base[PLAN_EB];
#pragma unroll
  for (int j = 0; j < PLAN_EB; ++j) val[j] = plan_tile_value(tile, e[j] & PLAN_OFFSET_MASK);
#pragma unroll
  for (int j = 0; j < PLAN_EB; ++j) base[j] = marg[(e[j] >> PLAN_SLOT_SHIFT) & PLAN_SLOT_MASK];
#pragma unroll
  for (int j = 0; j < PLAN_EB; ++j) {
    run = ((int)e[j] < 0 ? 0.f : run) + val[j];          // bit 31: the run starts here
    marg[(e[j] >> PLAN_SLOT_SHIFT) & PLAN_SLOT_MASK] = base[j] + run;
  }
}

// A packed list: the same sum in the same order as plan_consume gives for a lane with one run (its
// padding adds zeros ahead of the run), the slot read and written once.
__device__ __forceinline__ void plan_consume_packed(const u32x4& d, const float* tile, float* marg) {
  const unsigned w[4] = {d.x, d.y, d.z, d.w};
  float val[PLAN_EB];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    val[2 * j] = plan_tile_value(tile, w[j] & 0xfffcu);
    val[2 * j + 1] = plan_tile_value(tile, (w[j] >> 16) & 0xfffcu);
  }
  unsigned u = w[0] & 0x00030003u;
#pragma unroll
  for (int j = 1; j < 4; ++j) u |= (w[j] & 0x00030003u) << (2 * j);
  const unsigned slot = (u & 0xffu) | ((u >> 8) & 0xff00u);
  const float base = marg[slot];
  float run = 0.f;
#pragma unroll
  for (int j = 0; j < PLAN_EB; ++j) run += val[j];
  marg[slot] = base + run;
}

// The loop over the tiles keeps two kinds of loads in flight, always issued in the same order: the
// first batch of the next tile's list (into the entry registers the current tile does not use) and,
// behind it, the 16-byte loads of the tile after the next (into the registers the current tile's data
// has just left for LDS); the loop is unrolled by two so that both register sets are addressed
// statically.  Loads complete in issue order and the hardware counts them per wave, so every wait
// names how many younger loads may stay in flight: the wait for a tile's entries, issued ahead of the
// data of the tile behind it, leaves that data in flight, which gives every tile two iterations to
// arrive.  That only works out if the order is the same on every path into the loop, which the
// scheduling barriers pin.  (With the entries of the first tile issued ahead of its data, as the
// compiler had it, every wait in the loop became a wait for all but one or none of the loads: one
// tile in flight whatever the depth, and the entries' trip to L2 and back waited for in full.)
__device__ __forceinline__ void accumulate_marginal_planned(const MargParams& p, const char* prow, float* marg,
                                                            float* tile) {
  const int tid = threadIdx.x, lane = tid & (WAVE - 1);
  // the wave index as a scalar: plan offsets are then fetched with scalar loads, which have their own
  // counter and do not queue behind the vector prefetches
  const int w = __builtin_amdgcn_readfirstlane(tid / WAVE);
  constexpr int NW = MARG_NT / WAVE;
  const int TS = p.plan_tile;
  const int q_tile = TS / 4;                        // 16-byte loads per tile: 1024 .. 2048, up to two per thread
  const int ntiles = (int)((p.Vt + TS - 1) / TS);
  const int64_t n4 = p.Vt / 4;
  const int n_slots = (int)plan_slot_words(p.Vs, p.plan_n_extra);
  for (int j = tid; j < n_slots; j += MARG_NT) marg[j] = 0.f;
  if (tid < PLAN_ZERO_WORDS) tile[TS + tid] = 0.f;  // the tile's stores never reach these
  // Byte offsets inside a tile are 32-bit and the tile's base is uniform: loads with a scalar base.
  // Unconditional load from a clamped offset: with branch-free loads the compiler knows how many are
  // in flight and never has to drain the whole queue.  What a clamped load brings is never used: no
  // entry points behind the end of the row, and a select on the value here would make the thread
  // wait for the load right away instead of two tiles later.
  u32x4 tbuf[2][2];
  auto fetch_tile = [&](int k, u32x4 (&buf)[2]) {
    const bool in_row = k < ntiles;
    const char* base = prow + (in_row ? (int64_t)k * TS * 4 : 0);
    const int left = in_row ? (int)(n4 - (int64_t)k * q_tile) : 0;      // 16-byte units from the tile's start to the row's end
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = u * MARG_NT + tid;
      const unsigned off = (c < q_tile && c < left) ? (unsigned)c * 16u : 0u;
      buf[u] = load16_stream(base + off);
    }
  };
  // the constant address space tells the compiler that nothing in this kernel writes the offsets:
  // only then does it fetch them with scalar loads
  typedef const __attribute__((address_space(4))) int32_t* ConstI32;
  ConstI32 row_off = (ConstI32)p.plan_row_off;
  // Row numbers are multiples of 4; bit 0 of a list's first row number says that the list is packed.
  // Behind the last tile: the plan's first list, fetched and dropped.
  struct List { int first, end, packed; };
  auto list_of = [&](int k) {
    List l{0, 0, 0};
    if (k < ntiles) {
      const int a = row_off[k * NW + w], b = row_off[k * NW + w + 1];
      l.first = a & ~3;
      l.end = b & ~3;
      l.packed = a & 1;
    }
    return l;
  };
  // (the first batch of) a list: one 16-byte load per lane if packed, else two
  auto fetch_batch = [&](int r_first, int packed, PlanBatch& b) {
    const unsigned* at = p.plan_ent + (int64_t)r_first * WAVE;          // uniform
    if (packed) {
      b.lo = *reinterpret_cast<const u32x4*>(at + (unsigned)lane * 4u);
    } else {
      b.lo = *reinterpret_cast<const u32x4*>(at + (unsigned)lane * 8u);
      b.hi = *reinterpret_cast<const u32x4*>(at + (unsigned)lane * 8u + 4u);
    }
  };
  PlanBatch e_even, e_odd;
  List cur = list_of(0), next = list_of(1);           // the descriptors run two tiles ahead of the entries
  fetch_tile(0, tbuf[0]);
  __builtin_amdgcn_sched_barrier(0);
  fetch_batch(cur.first, cur.packed, e_even);
  __builtin_amdgcn_sched_barrier(0);
  fetch_tile(1, tbuf[1]);
  __builtin_amdgcn_sched_barrier(0);
  float run = 0.f;
  auto do_tile = [&](int k, u32x4 (&buf)[2], PlanBatch& e, PlanBatch& e_next) {
    __syncthreads();                                 // previous tile fully consumed (first pass: marg zeroed)
#pragma unroll
    for (int u = 0; u < 2; ++u)
      if (u * MARG_NT + tid < q_tile) *reinterpret_cast<u32x4*>(tile + ((int64_t)u * MARG_NT + tid) * 4) = buf[u];
    __syncthreads();
    fetch_batch(next.first, next.packed, e_next);
    __builtin_amdgcn_sched_barrier(0);
    fetch_tile(k + 2, buf);
    __builtin_amdgcn_sched_barrier(0);
    const List after = list_of(k + 2);
    if (cur.packed) {                                          // wave-uniform: the flag came by a scalar load
      plan_consume_packed(e.lo, tile, marg);
    } else {
      plan_consume(e, tile, marg, run);
      for (int r = cur.first + PLAN_EB; r < cur.end; r += PLAN_EB) {   // a list longer than one batch (rare: not enough LDS
        fetch_batch(r, 0, e);                                          // for replicas): fetched on the spot
        plan_consume(e, tile, marg, run);
      }
    }
    cur = next;
    next = after;
  };
  // unrolled by two: the registers are addressed statically.  No path may enter the loop body with a
  // different set of loads in flight than the others, or every wait falls back to the worst case: an
  // odd last tile is therefore a third copy behind the loop, not a skipped second half.
  int k = 0;
  for (; k + 1 < ntiles; k += 2) {
    do_tile(k, tbuf[0], e_even, e_odd);
    do_tile(k + 1, tbuf[1], e_odd, e_even);
  }
  if (k < ntiles) do_tile(k, tbuf[0], e_even, e_odd);
  __syncthreads();
  // replicas into their id's slot: own slot first, then the replicas in ascending order
  for (int f = tid; f < p.plan_n_fold; f += MARG_NT) {
    const int sid = p.plan_fold[3 * f], first = p.plan_fold[3 * f + 1], cnt = p.plan_fold[3 * f + 2];
    float a = marg[sid];
    for (int j = 0; j < cnt; ++j) a += marg[first + j];
    marg[sid] = a;
  }
  __syncthreads();
}

// Accumulate the slice [s_lo, s_lo + s_n) of one row's marginal into `acc` (LDS, zeroed here).
template <bool VEC>
__device__ __forceinline__ void accumulate_marginal(const MargParams& p, const char* prow, float* acc, int s_lo,
                                                    int s_n) {
  const int tid = threadIdx.x;
  for (int j = tid; j < s_n; j += MARG_NT) acc[j] = 0.f;
  __syncthreads();
  if (VEC) {       // fp32 probabilities, 16-byte aligned: four columns per load
    // Double-buffered batches of U 16-byte loads of the probabilities and of the id map per thread:
    // the next batch is in flight while the current one is scattered into LDS.
    constexpr int U = 4;
    const int64_t n4 = p.Vt / 4;
    const char* mrow = reinterpret_cast<const char*>(p.t2s);
    u32x4 pa[U], ia[U], pb[U], ib[U];
    auto fetch = [&](int64_t c0, u32x4* pv, u32x4* iv) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t c = c0 + (int64_t)u * MARG_NT + tid;
        if (c < n4) {
          pv[u] = load16_stream(prow + c * 16);
          iv[u] = *reinterpret_cast<const u32x4*>(mrow + c * 16);
        } else {
          pv[u] = u32x4{0u, 0u, 0u, 0u};
          iv[u] = u32x4{~0u, ~0u, ~0u, ~0u};
        }
      }
    };
    auto scatter = [&](u32x4* pv, u32x4* iv) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        forget(pv[u]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int s = (int)iv[u][e] - s_lo;
          if (s >= 0 && s < s_n)
            __hip_atomic_fetch_add(&acc[s], __uint_as_float(pv[u][e]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    };
    constexpr int64_t STEP = (int64_t)U * MARG_NT;
    fetch(0, pa, ia);
    for (int64_t c0 = 0; c0 < n4; c0 += 2 * STEP) {
      fetch(c0 + STEP, pb, ib);            // beyond the row: nothing is loaded, sentinel ids
      scatter(pa, ia);
      fetch(c0 + 2 * STEP, pa, ia);
      scatter(pb, ib);
    }
  } else {
    for (int64_t t = tid; t < p.Vt; t += MARG_NT) {
      const int s = p.t2s[t] - s_lo;
      if (s >= 0 && s < s_n)
        __hip_atomic_fetch_add(&acc[s], load_as_float(prow, p.p_dtype, t), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  __syncthreads();
}

// marg (or log marg) to memory; student vocabularies wider than the LDS slice take several passes.
template <bool VEC>
__global__ __launch_bounds__(MARG_NT) void marginalise_map_kernel(const MargParams p) {
  extern __shared__ __align__(16) float acc[];
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int pb = p.p_dtype == F32 ? 4 : 2;
  const char* prow = reinterpret_cast<const char*>(p.probs) + r * p.p_stride * pb;
  float* out = p.marg + r * p.marg_stride;
  if (VEC && p.plan_ent) {
    float* marg = acc + p.plan_tile + PLAN_ZERO_WORDS;      // the tile sits first: its addresses are then plain offsets
    accumulate_marginal_planned(p, prow, marg, acc);
    for (int j = threadIdx.x; j < p.Vs; j += MARG_NT) out[j] = p.out_log ? logf(marg[j]) : marg[j];
    return;
  }
  for (int64_t s_lo = 0; s_lo < p.Vs; s_lo += MARG_MAX_VS) {
    const int s_n = (int)min((int64_t)MARG_MAX_VS, p.Vs - s_lo);
    accumulate_marginal<VEC>(p, prow, acc, (int)s_lo, s_n);
    for (int j = threadIdx.x; j < s_n; j += MARG_NT) out[s_lo + j] = p.out_log ? logf(acc[j]) : acc[j];
    __syncthreads();
  }
}

// Deterministic form: thread per student id, segment summed in ascending teacher-id order.
__global__ __launch_bounds__(256) void marginalise_csr_kernel(const void* probs, int p_dtype, int64_t p_stride,
                                                             int64_t Vt, const int32_t* offsets,
                                                             const int32_t* indices, int64_t Vs, float* marg,
                                                             int64_t marg_stride, int out_log) {
  const int64_t r = blockIdx.y;
  const int64_t s = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (s >= Vs) return;
  const char* prow = reinterpret_cast<const char*>(probs) + r * p_stride * (p_dtype == F32 ? 4 : 2);
  float m = 0.f;
  for (int e = offsets[s]; e < offsets[s + 1]; ++e) {
    const int t = indices[e];
    if (t >= 0 && t < Vt) m += load_as_float(prow, p_dtype, t);
  }
  marg[r * marg_stride + s] = out_log ? logf(m) : m;
}

// ---- fused: marginal in LDS -> reverse KL against the student row in registers -----------------
// The student row of the fused kernel: NU units of 8 columns per thread, in registers.
// Unit u of a compacted student row: the raw elements at columns cols[8u .. 8u + 7] of the full-width row.
// Unit u of a full-width row seen through `cols`: the logits at columns cols[8u .. 8u + 7] (-inf for a column of -1).
// The ids are fetched apart from the elements, so that a caller with several units has all ids in flight together
// before the first element load waits for them.
struct UnitIds { int4 a, b; };
__device__ __forceinline__ UnitIds unit_ids(const int32_t* cols, int64_t u) {
  return UnitIds{*reinterpret_cast<const int4*>(cols + u * 8), *reinterpret_cast<const int4*>(cols + u * 8 + 4)};
}
template <class TagS>
__device__ __forceinline__ void gather_unit(Unit<TagS>& x, const char* srow, const UnitIds& ids) {
  const int id[8] = {ids.a.x, ids.a.y, ids.a.z, ids.a.w, ids.b.x, ids.b.y, ids.b.z, ids.b.w};
  if constexpr (TagS::bytes == 4) {
#pragma unroll
    for (int e = 0; e < 8; ++e) x.c[e >> 2][e & 3] = id[e] >= 0 ? reinterpret_cast<const unsigned*>(srow)[id[e]] : 0xff800000u;
  } else {
    const u32x4 ninf = Chunk<TagS>::neg_inf();
    unsigned h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
      h[e] = id[e] >= 0 ? (unsigned)reinterpret_cast<const unsigned short*>(srow)[id[e]] : (ninf[0] & 0xffffu);
#pragma unroll
    for (int d = 0; d < 4; ++d) x.c[0][d] = h[2 * d] | (h[2 * d + 1] << 16);
  }
}
template <class TagS>
__device__ __forceinline__ void gather_unit(Unit<TagS>& x, const char* srow, const int32_t* cols, int64_t u) {
  gather_unit<TagS>(x, srow, unit_ids(cols, u));
}

template <class TagS, int NU>
struct StudentRow {
  Unit<TagS> s[NU];
  int64_t nunits;
  __device__ __forceinline__ void load(const char* srow, int64_t nu) {
    nunits = nu;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * MARG_NT + threadIdx.x;
      if (u < nunits) s[i].load(srow, u); else s[i].fill_neg_inf();
    }
  }
  // The same from a full-width row, unit u = the logits at columns cols[8u .. 8u + 7] (-inf for a column of -1).
  __device__ __forceinline__ void load_gathered(const char* srow, const int32_t* cols, int64_t nu) {
    nunits = nu;
    UnitIds ids[NU];
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * MARG_NT + threadIdx.x;
      ids[i] = u < nunits ? unit_ids(cols, u) : UnitIds{int4{-1, -1, -1, -1}, int4{-1, -1, -1, -1}};
    }
#pragma unroll
    for (int i = 0; i < NU; ++i) gather_unit<TagS>(s[i], srow, ids[i]);
  }
};

// Reverse KL of the student row (in registers) against a marginal that sits in LDS as probabilities,
// with its gradient; the same quantities as dense_stats<DL_RKL> + dense_grad_sweep<DL_RKL> on the
// logarithm of the marginal, in fewer instructions (with one 1024-thread workgroup per CU these
// passes run on the vector ALUs alone, no memory traffic to hide behind).  Log2 domain throughout:
//   xt_j = log2(m_j) / T_t - bt        (off the support: XT_OFF, standing for -inf)
//   xs_j = s_j a_s - bs
//   S = sum_on 2^xs, T = sum 2^xt, W = sum_on 2^xs (xs - xt)
//   RKL = (W / S - log2 S + log2 T) ln 2
//   d RKL / d s_j = 2^xs_j (ln 2 / (T_s S)) ((xs_j - xt_j) - W / S)      on the support, else 0
// None of these depends on the biases bs, bt; they only keep the sums in range.  The usual choice, the
// largest marginal and the largest student logit ON THE SUPPORT, costs a pass over the marginal before
// the sums can start.  Instead: bt = 0 (a marginal of probabilities is at most 1, and its largest entry
// is rarely below 2^-20) and bs from the largest student logit of the whole row, which needs the
// registers only.  Pass B: xt (written over the marginal; a log-domain value, exact whatever the
// bias), the three sums.  If T or S then lies outside [2^-64, 2^64] -- the row carries no or hardly any
// mass, an unnormalised teacher, or a student whose mass sits far off the support -- the maxima are
// taken after all, from the stored xt, and the sums are redone on them.  Pass C: gradient.  When a
// gradient follows, pass B leaves 2^xs in the registers of the logits and xs - xt in the marginal's
// slots (rkl_sums_stash), and pass C is a multiply-add and a multiply per column.
// What stands for log2(0) in the stored xt and for a student logit of -inf: finite, so that differences
// of two such values are finite (0 * finite = 0 needs no select), and far below anything a sum notices.
constexpr float XT_OFF = -1e30f;
// 2^24 lifts every positive fp32 value, denormals included (>= 2^-149), into the normal range; marginal
// entries above 2^103 would overflow (probabilities are at most 1).
constexpr float MARG_LOG_SCALE = 0x1p24f, MARG_LOG_SHIFT = 24.f;

template <class TagS, int NU, bool UNIT_T>
__device__ __forceinline__ void rkl_sums_optimistic(Unit<TagS> (&s)[NU], int64_t nunits, float* marg, float a_s, float bs,
                                                    float inv_T_t, float& ss, float& stt, float& w) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int64_t u = (int64_t)i * MARG_NT + tid;
    if (u < nunits) {
      float sv[8], m[8];
      s[i].unpack(sv);
      const float4 m0 = *reinterpret_cast<const float4*>(marg + u * 8), m1 = *reinterpret_cast<const float4*>(marg + u * 8 + 4);
      m[0] = m0.x; m[1] = m0.y; m[2] = m0.z; m[3] = m0.w; m[4] = m1.x; m[5] = m1.y; m[6] = m1.z; m[7] = m1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // the hardware logarithm takes a denormal for zero: the marginal is scaled into the normal range first
        const float l2 = fast_log2(m[e] * MARG_LOG_SCALE);
        const float xt = fmaxf(UNIT_T ? l2 - MARG_LOG_SHIFT : fmaf(l2, inv_T_t, -MARG_LOG_SHIFT * inv_T_t), XT_OFF);
        const float xs = fmaxf(fmaf(sv[e], a_s, -bs), XT_OFF);
        const float eon = m[e] > 0.f ? fast_exp2(xs) : 0.f;
        stt += UNIT_T ? m[e] : fast_exp2(xt);      // 2^xt; 0 off the support
        ss += eon;
        w = fmaf(eon, xs - xt, w);                 // the difference is finite: no 0 * inf
        m[e] = xt;
      }
      *reinterpret_cast<float4*>(marg + u * 8) = float4{m[0], m[1], m[2], m[3]};        // own columns only: no barrier needed
      *reinterpret_cast<float4*>(marg + u * 8 + 4) = float4{m[4], m[5], m[6], m[7]};
    }
  }
}

// The same pass when a gradient follows: it leaves what the gradient is made of, so that the
// gradient pass needs no transcendental and a third of the instructions.  With B = the stash bias of
// the row's type (Chunk<TagS>::stash_bias: 2^xs in fp16 keeps 11 bits down to 2^-29 of the row's
// largest entry; fp32 rows keep all of it) and both biases lifted by B,
//   registers of the logits <- 2^(xs + B)   (0 off the support)
//   marginal's slot         <- xs - xt      (of a column whose 2^xs underflows anyway, xs <= -256: 0 - xt,
//                                            so that xt can be had back exactly enough from any slot)
// ss, stt (unless UNIT_T) and w come out multiplied by 2^B.
constexpr float XS_DEAD = -256.f;
template <class TagS, int NU, bool UNIT_T>
__device__ __forceinline__ void rkl_sums_stash(Unit<TagS> (&s)[NU], int64_t nunits, float* marg, float a_s, float bs2,
                                               float inv_T_t, float& ss, float& stt, float& w) {
  constexpr float B = Chunk<TagS>::stash_bias;
  const int tid = threadIdx.x;
  const float ct = UNIT_T ? B - MARG_LOG_SHIFT : B - MARG_LOG_SHIFT * inv_T_t;
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int64_t u = (int64_t)i * MARG_NT + tid;
    if (u < nunits) {
      float sv[8], m[8];
      s[i].unpack(sv);
      const float4 m0 = *reinterpret_cast<const float4*>(marg + u * 8), m1 = *reinterpret_cast<const float4*>(marg + u * 8 + 4);
      m[0] = m0.x; m[1] = m0.y; m[2] = m0.z; m[3] = m0.w; m[4] = m1.x; m[5] = m1.y; m[6] = m1.z; m[7] = m1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float l2 = fast_log2(m[e] * MARG_LOG_SCALE);
        const float xt = fmaxf(UNIT_T ? l2 + ct : fmaf(l2, inv_T_t, ct), XT_OFF);
        const float xs = fmaf(sv[e], a_s, -bs2);                   // -inf for a logit of -inf
        // 2^xs on the support, 0 off it, without a select: xt is XT_OFF exactly off the support, where
        // xt * 2^-90 = -800 sinks the exponent, and so small on it that the sum rounds back to xs
        const float eon = fast_exp2(fmaf(xt, 0x1p-90f, xs));
        const float d = (xs > XS_DEAD ? xs : 0.f) - xt;            // finite
        stt += UNIT_T ? m[e] : fast_exp2(xt);
        ss += eon;
        w = fmaf(eon, d, w);
        m[e] = d;
        sv[e] = eon;
      }
      *reinterpret_cast<float4*>(marg + u * 8) = float4{m[0], m[1], m[2], m[3]};        // own columns only: no barrier needed
      *reinterpret_cast<float4*>(marg + u * 8 + 4) = float4{m[4], m[5], m[6], m[7]};
#pragma unroll
      for (int k = 0; k < Unit<TagS>::NC; ++k) s[i].c[k] = Chunk<TagS>::stash(sv + k * Chunk<TagS>::N);
    }
  }
}

// The gradient from what rkl_sums_stash left: 2^(xs + B) * (k1 (xs - xt) - k1 wbar), k1 over the sum
// that carries the same 2^B.  The factor is held finite (a column off the support stores 1e30 for its
// difference), so that 0 * factor is 0.
// COMPACT rows leave the gradient of unit u, as fp32, where its differences stood (marg[8u .. 8u + 7], the thread's
// own slots); the caller expands it into the full-width row afterwards.
template <class TagS>
__device__ __forceinline__ void put_gradient_unit(char* grow, float* marg, int64_t u, const float* g, bool to_lds) {
  if (to_lds) {
    *reinterpret_cast<float4*>(marg + u * 8) = float4{g[0], g[1], g[2], g[3]};
    *reinterpret_cast<float4*>(marg + u * 8 + 4) = float4{g[4], g[5], g[6], g[7]};
  } else {
    Unit<TagS>::store(grow, u, g);
  }
}

template <class TagS, int NU>
__device__ __forceinline__ void rkl_gradient_from_stash(Unit<TagS> (&s)[NU], int64_t nunits, float* marg, float k1,
                                                        float wbar, char* grow, bool to_lds) {
  const int tid = threadIdx.x;
  const float k0 = -k1 * wbar;
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int64_t u = (int64_t)i * MARG_NT + tid;
    if (u < nunits) {
      float es[8], d[8], g[8];
#pragma unroll
      for (int k = 0; k < Unit<TagS>::NC; ++k) Chunk<TagS>::unstash(s[i].c[k], es + k * Chunk<TagS>::N);
      const float4 m0 = *reinterpret_cast<const float4*>(marg + u * 8), m1 = *reinterpret_cast<const float4*>(marg + u * 8 + 4);
      d[0] = m0.x; d[1] = m0.y; d[2] = m0.z; d[3] = m0.w; d[4] = m1.x; d[5] = m1.y; d[6] = m1.z; d[7] = m1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = es[e] * __builtin_amdgcn_fmed3f(fmaf(d[e], k1, k0), -3e38f, 3e38f);
      put_gradient_unit<TagS>(grow, marg, u, g, to_lds);
    }
  }
}

// Pass C on the stored xt (rows whose sums were redone on their maxima).
template <class TagS, int NU>
__device__ __forceinline__ void rkl_gradient_pass(Unit<TagS> (&s)[NU], int64_t nunits, float* marg, float a_s, float bs,
                                                  float k1, float wbar, char* grow, bool to_lds) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int64_t u = (int64_t)i * MARG_NT + tid;
    if (u < nunits) {
      float sv[8], xt[8], g[8];
      s[i].unpack(sv);
      const float4 m0 = *reinterpret_cast<const float4*>(marg + u * 8), m1 = *reinterpret_cast<const float4*>(marg + u * 8 + 4);
      xt[0] = m0.x; xt[1] = m0.y; xt[2] = m0.z; xt[3] = m0.w; xt[4] = m1.x; xt[5] = m1.y; xt[6] = m1.z; xt[7] = m1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xs = fmaxf(fmaf(sv[e], a_s, -bs), XT_OFF);     // finite for a logit of -inf: 0 * difference is 0
        g[e] = xt[e] > 0.5f * XT_OFF ? fast_exp2(xs) * k1 * ((xs - xt[e]) - wbar) : 0.f;
      }
      put_gradient_unit<TagS>(grow, marg, u, g, to_lds);
    }
  }
}

// With a gradient asked for, the sums' pass leaves its ingredients behind (rkl_sums_stash).  If the sums
// then turn out to be out of range, the row is put back -- logits read again (nothing of the row has
// been written yet, also when the gradient goes over the logits), xt from the stored differences --
// and takes the passes on its maxima like a row without a gradient.
// Compact rows (p.Vs_full > 0): returns true when the gradient of the compact columns was left in marg for the
// caller to expand; false when there is none to expand (no gradient asked for, or the row was zero-filled here).
template <class TagS, int NU>
__device__ __forceinline__ bool rkl_against_marginal(Unit<TagS> (&s)[NU], int64_t nunits, float* marg, float* red,
                                                     const MargParams& p, int64_t r, char* grow, const char* srow) {
  const int tid = threadIdx.x;
  const bool compact = p.Vs_full > 0;
  const float a_s = p.inv_T_s * LOG2E;
  const auto stored_of = [&](int64_t u, float (&m)[8]) {
    const float4 m0 = *reinterpret_cast<const float4*>(marg + u * 8), m1 = *reinterpret_cast<const float4*>(marg + u * 8 + 4);
    m[0] = m0.x; m[1] = m0.y; m[2] = m0.z; m[3] = m0.w; m[4] = m1.x; m[5] = m1.y; m[6] = m1.z; m[7] = m1.w;
  };
  const auto in_range = [](float v) { return v > 0x1p-64f && v < 0x1p64f; };
  const bool unit_T = p.inv_T_t == 1.f;
  // The row's largest logit (units beyond the row hold -inf).  16-bit rows: non-negative values order like
  // their bit patterns read as signed integers and every negative one reads as a negative integer, so the
  // packed integer maximum of the raw pairs is the maximum whenever that is not negative -- half an
  // instruction per column instead of two.
  float ms = -INFINITY;
  bool have_ms = false;
  if constexpr (TagS::bytes == 2) {
    typedef short i16x2 __attribute__((ext_vector_type(2)));
    i16x2 pm = {(short)-32768, (short)-32768};
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      forget(s[i].c[0]);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w16 = s[i].c[0][d];      // by value: a bit cast straight from a vector element reads element 0
        pm = __builtin_elementwise_max(pm, __builtin_bit_cast(i16x2, w16));
      }
    }
    const float top = block_max<MARG_NT>((float)max((int)pm.x, (int)pm.y), red);      // exact, order-preserving
    if (top >= 0.f) {                                                                 // the same for every thread
      const unsigned bits = (unsigned)(int)top;
      ms = TagS::id == BF16 ? __uint_as_float(bits << 16) : (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
      have_ms = true;
    }
  }
  if (!have_ms) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      float sv[8];
      s[i].unpack(sv);
#pragma unroll
      for (int e = 0; e < 8; ++e) ms = fmaxf(ms, sv[e]);
    }
    ms = block_max<MARG_NT>(ms, red);
  }
  float bs = ms > -INFINITY ? ms * a_s : 0.f;
  float ss = 0.f, stt = 0.f, w = 0.f;
  bool redo;
  // fp32 rows always: for them the stash is free, and a second form of the pass beside it costs registers
  if (TagS::bytes == 4 || grow) {
    constexpr float B = Chunk<TagS>::stash_bias;
    const float bs2 = bs - B;
    if (unit_T) rkl_sums_stash<TagS, NU, true>(s, nunits, marg, a_s, bs2, 1.f, ss, stt, w);
    else rkl_sums_stash<TagS, NU, false>(s, nunits, marg, a_s, bs2, p.inv_T_t, ss, stt, w);
    block_sum3<MARG_NT>(ss, stt, w, red);
    const float unscale = __uint_as_float((unsigned)(127 - (int)B) << 23);      // 2^-B
    const float ss1 = ss * unscale, stt1 = unit_T ? stt : stt * unscale;
    // 16-bit rows: the stash keeps 2^xs down to 2^-29 of the row's largest entry, on the support or off it.
    // If the support holds less than 1/64 of that entry's weight (the student's mass sits off the support),
    // entries that matter would fall below: such a row is redone on the support's maximum as well.
    const bool stash_ok = TagS::bytes == 4 || ss1 >= 0x1p-6f;
    if (stash_ok && in_range(ss1) && in_range(stt1)) {      // the same for every thread
      const float wbar = w / ss;
      if (tid == 0 && p.row_loss) p.row_loss[r] = (wbar - fast_log2(ss1) + fast_log2(stt1)) * LN2;
      if (grow) rkl_gradient_from_stash<TagS, NU>(s, nunits, marg, p.inv_T_s * p.grad_scale * LN2 / ss, wbar, grow, compact);
      return compact && grow;
    }
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * MARG_NT + tid;
      if (u < nunits) {
        if (compact) gather_unit<TagS>(s[i], srow, p.cols, u);
        else s[i].load(srow, u);
        float sv[8], d[8];
        s[i].unpack(sv);
        stored_of(u, d);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xs = fmaf(sv[e], a_s, -bs2);
          d[e] = fmaxf(((xs > XS_DEAD ? xs : 0.f) - d[e]) - B, XT_OFF);
        }
        *reinterpret_cast<float4*>(marg + u * 8) = float4{d[0], d[1], d[2], d[3]};
        *reinterpret_cast<float4*>(marg + u * 8 + 4) = float4{d[4], d[5], d[6], d[7]};
      }
    }
    redo = true;
  } else {
    if (unit_T) rkl_sums_optimistic<TagS, NU, true>(s, nunits, marg, a_s, bs, 1.f, ss, stt, w);
    else rkl_sums_optimistic<TagS, NU, false>(s, nunits, marg, a_s, bs, p.inv_T_t, ss, stt, w);
    block_sum3<MARG_NT>(ss, stt, w, red);
    redo = !(in_range(ss) && in_range(stt));      // the same for every thread
  }
  if (redo) {
    float tmax = -INFINITY;
    ms = -INFINITY;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * MARG_NT + tid;
      if (u < nunits) {
        float sv[8], xt[8];
        s[i].unpack(sv);
        stored_of(u, xt);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          tmax = fmaxf(tmax, xt[e]);
          ms = fmaxf(ms, xt[e] > 0.5f * XT_OFF ? sv[e] : -INFINITY);
        }
      }
    }
    block_max2<MARG_NT>(tmax, ms, red);
    if (!(tmax > 0.5f * XT_OFF)) {                    // the teacher row carried no mass at all
      if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
      if (grow) zero_row<TagS, MARG_NT>(grow, (compact ? p.Vs_full : p.Vs) / TagS::epc);
      return false;
    }
    bs = ms * a_s;
    ss = 0.f, stt = 0.f, w = 0.f;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * MARG_NT + tid;
      if (u < nunits) {
        float sv[8], xt[8];
        s[i].unpack(sv);
        stored_of(u, xt);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bool on = xt[e] > 0.5f * XT_OFF;
          xt[e] = on ? xt[e] - tmax : XT_OFF;
          const float xs = fmaxf(fmaf(sv[e], a_s, -bs), XT_OFF);
          const float eon = on ? fast_exp2(xs) : 0.f;
          stt += fast_exp2(xt[e]);
          ss += eon;
          w = fmaf(eon, xs - xt[e], w);
        }
        *reinterpret_cast<float4*>(marg + u * 8) = float4{xt[0], xt[1], xt[2], xt[3]};
        *reinterpret_cast<float4*>(marg + u * 8 + 4) = float4{xt[4], xt[5], xt[6], xt[7]};
      }
    }
    block_sum3<MARG_NT>(ss, stt, w, red);
  }
  const float wbar = w / ss;
  if (tid == 0 && p.row_loss) p.row_loss[r] = (wbar - fast_log2(ss) + fast_log2(stt)) * LN2;
  if (grow) rkl_gradient_pass<TagS, NU>(s, nunits, marg, a_s, bs, p.inv_T_s * p.grad_scale * LN2 / ss, wbar, grow, compact);
  return compact && grow;
}

// The gradient of a compact row (fp32 in marg, one value per compact id) into the full-width row: column j takes the
// value of compact id col_src16[j], or 0; every chunk of the row is written once, by a 16-byte store.
template <class TagS>
__device__ __forceinline__ void expand_gradient_row(const float* marg, const unsigned short* col_src16, int64_t Vs_full, char* grow) {
  using C = Chunk<TagS>;
  constexpr int U = 8;                                   // chunks in flight per thread: their table loads are issued together
  const int64_t nch = Vs_full / C::N;
  for (int64_t c0 = threadIdx.x; c0 < nch; c0 += (int64_t)U * MARG_NT) {
    u32x4 t[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int64_t ch = c0 + (int64_t)j * MARG_NT;
      if constexpr (C::N == 8) {
        t[j] = ch < nch ? *reinterpret_cast<const u32x4*>(col_src16 + ch * 8) : u32x4{~0u, ~0u, ~0u, ~0u};
      } else {
        const uint2 h = ch < nch ? *reinterpret_cast<const uint2*>(col_src16 + ch * 4) : uint2{~0u, ~0u};
        t[j] = u32x4{h.x, h.y, ~0u, ~0u};
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int64_t ch = c0 + (int64_t)j * MARG_NT;
      if (ch < nch) {
        float g[C::N];
#pragma unroll
        for (int e = 0; e < C::N; ++e) {
          const unsigned id = (t[j][e >> 1] >> ((e & 1) * 16)) & 0xffffu;
          g[e] = id != 0xffffu ? marg[id] : 0.f;
        }
        store16_stream(grow + ch * 16, C::pack(g));
      }
    }
  }
}

template <class TagS, int NU, bool VEC>
__global__ __launch_bounds__(MARG_NT) void rkl_marginalised_kernel(const MargParams p) {
  extern __shared__ __align__(16) float acc[];
  __shared__ float red[64];
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_srows) return;
  const int tid = threadIdx.x;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * TagS::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_rows);
  const bool compact = p.Vs_full > 0;
  if (trow < 0) {
    if (grow) zero_row<TagS, MARG_NT>(grow, (compact ? p.Vs_full : p.Vs) / TagS::epc);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  StudentRow<TagS, NU> rows;
  const char* srow = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * TagS::bytes;
  const int pb = p.p_dtype == F32 ? 4 : 2;
  const char* prow = reinterpret_cast<const char*>(p.probs) + trow * p.p_stride * pb;
  float* marg = acc;
  // the student row is in flight during the accumulation
  if (VEC && p.plan_ent) {
    marg = acc + p.plan_tile + PLAN_ZERO_WORDS;  // the tile sits first: its addresses are then plain offsets
    if (compact) rows.load_gathered(srow, p.cols, p.Vs / 8); else rows.load(srow, p.Vs / 8);
    accumulate_marginal_planned(p, prow, marg, acc);
  } else {
    if (compact) rows.load_gathered(srow, p.cols, p.Vs / 8); else rows.load(srow, p.Vs / 8);
    accumulate_marginal<VEC>(p, prow, acc, 0, (int)p.Vs);
  }
  if (rkl_against_marginal<TagS, NU>(rows.s, rows.nunits, marg, red, p, r, grow, srow)) {      // the same for every thread
    __syncthreads();                             // the gradient of every compact column is in LDS
    expand_gradient_row<TagS>(marg, p.col_src16, p.Vs_full, grow);
  }
}

static bool ok16(const void* ptr, int64_t stride, int eb) {
  return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (stride * eb) % 16 == 0;
}

// More than 64 KiB of dynamic LDS has to be requested per kernel; once per process and device is
// enough (the call is slow, so it must not sit on the launch path).
template <class K>
static void allow_large_lds_for(K kernel) {
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            MARG_MAX_DYN_LDS);
}
static void allow_large_lds() {
  static thread_local int done_for = -1;
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (done_for == dev) return;
  allow_large_lds_for(&marginalise_map_kernel<true>);
  allow_large_lds_for(&marginalise_map_kernel<false>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagF32, MARG_NU, true>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagF32, MARG_NU, false>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagBF16, MARG_NU, true>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagBF16, MARG_NU, false>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagF16, MARG_NU, true>);
  allow_large_lds_for(&rkl_marginalised_kernel<TagF16, MARG_NU, false>);
  done_for = dev;
}

}  // namespace dl

// Fills the plan fields of `p` if a usable plan is given; returns the dynamic LDS bytes to request.
static size_t attach_plan(dl::MargParams& p, const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                          const int32_t* plan_fold, int plan_n_fold, int plan_n_extra, bool vec, size_t lds_without_plan) {
  if (!plan_row_off || !plan_ent || !vec) return lds_without_plan;
  if (plan_tile < 4096 || plan_tile > 8192 || plan_tile % 1024) return lds_without_plan;
  if (plan_n_fold < 0 || plan_n_extra < 0 || (plan_n_fold > 0 && !plan_fold)) return lds_without_plan;
  const size_t need = (size_t)dl::plan_slot_words(p.Vs, plan_n_extra) * 4 + (size_t)(plan_tile + dl::PLAN_ZERO_WORDS) * 4;
  if (need > (size_t)dl::MARG_MAX_DYN_LDS) return lds_without_plan;
  p.plan_row_off = plan_row_off; p.plan_ent = plan_ent; p.plan_tile = plan_tile;
  p.plan_fold = plan_fold; p.plan_n_fold = plan_n_fold; p.plan_n_extra = plan_n_extra;
  return need;
}

extern "C" int dl_marginalise_map(const void* probs, int p_dtype, int64_t p_stride, int64_t n_rows, int64_t Vt,
                                  const int32_t* t2s, int64_t Vs, const int32_t* plan_row_off,
                                  const uint32_t* plan_ent, int plan_tile, const int32_t* plan_fold, int plan_n_fold,
                                  int plan_n_extra, float* marg, int64_t marg_stride,
                                  int out_log, void* stream) {
  using namespace dl;
  if (!probs || !t2s || !marg) return DL_ERR_NULL;
  if (p_dtype < DL_F32 || p_dtype > DL_F16) return DL_ERR_DTYPE;
  if (n_rows < 0 || Vt <= 0 || Vs <= 0 || p_stride < Vt || marg_stride < Vs) return DL_ERR_SHAPE;
  if (n_rows > 0x7fffffffLL || Vt > 0x7fffffffLL || Vs > 0x7fffffffLL) return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  MargParams p{};
  p.probs = probs; p.p_dtype = p_dtype; p.p_stride = p_stride; p.n_rows = n_rows; p.Vt = Vt; p.t2s = t2s; p.Vs = Vs;
  p.marg = marg; p.marg_stride = marg_stride; p.out_log = out_log;
  const bool vec = p_dtype == DL_F32 && Vt % 4 == 0 && ok16(probs, p_stride, 4) && ok16(t2s, 0, 4);
  const size_t lds = attach_plan(p, plan_row_off, plan_ent, plan_tile, plan_fold, plan_n_fold, plan_n_extra, vec,
                                 (size_t)(Vs < MARG_MAX_VS ? Vs : MARG_MAX_VS) * 4);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  allow_large_lds();
  if (vec) hipLaunchKernelGGL((marginalise_map_kernel<true>), dim3(xcd_banded_grid(n_rows)), dim3(MARG_NT), lds, st, p);
  else hipLaunchKernelGGL((marginalise_map_kernel<false>), dim3(xcd_banded_grid(n_rows)), dim3(MARG_NT), lds, st, p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_marginalise_csr(const void* probs, int p_dtype, int64_t p_stride, int64_t n_rows, int64_t Vt,
                                  const int32_t* offsets, const int32_t* indices, int64_t Vs, float* marg,
                                  int64_t marg_stride, int out_log, void* stream) {
  using namespace dl;
  if (!probs || !offsets || !indices || !marg) return DL_ERR_NULL;
  if (p_dtype < DL_F32 || p_dtype > DL_F16) return DL_ERR_DTYPE;
  if (n_rows < 0 || Vt <= 0 || Vs <= 0 || p_stride < Vt || marg_stride < Vs) return DL_ERR_SHAPE;
  if (n_rows > 65535 * 1024LL || Vs > 0x7fffffffLL) return DL_ERR_LIMIT;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  for (int64_t r0 = 0; r0 < n_rows; r0 += 65535) {        // grid.y limit
    const int64_t nr = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
    const int pb = p_dtype == DL_F32 ? 4 : 2;
    hipLaunchKernelGGL(marginalise_csr_kernel, dim3((unsigned)((Vs + 255) / 256), (unsigned)nr), dim3(256), 0, st,
                       reinterpret_cast<const char*>(probs) + r0 * p_stride * pb, p_dtype, p_stride, Vt, offsets,
                       indices, Vs, marg + r0 * marg_stride, marg_stride, out_log);
  }
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

// Shared by dl_rkl_marginalised (cols == NULL: the rows are Vs wide) and dl_rkl_marginalised_compact (logits and
// gradient rows Vs_full wide, the kernel works on the Vs columns `cols` names).
static int rkl_marginalised_launch(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t Vs,
                                   const int32_t* row_map, const void* t_probs, int p_dtype, int64_t p_stride,
                                   int64_t n_teacher_rows, int64_t Vt, const int32_t* t2s,
                                   const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                                   const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                                   float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                                   void* grad, int64_t grad_stride, const int32_t* cols, const unsigned short* col_src16,
                                   int64_t Vs_full, void* stream) {
  using namespace dl;
  if (!logits || !t_probs || !t2s) return DL_ERR_NULL;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || p_dtype < DL_F32 || p_dtype > DL_F16) return DL_ERR_DTYPE;
  const int64_t width = cols ? Vs_full : Vs;      // columns of a logits / gradient row
  if (n_rows < 0 || Vs <= 0 || Vt <= 0 || n_teacher_rows < 0 || width < Vs || row_stride < width || p_stride < Vt ||
      (grad && grad_stride < width))
    return DL_ERR_SHAPE;
  if (Vs > MARG_MAX_VS || n_rows > 0x7fffffffLL || Vt > 0x7fffffffLL || width > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int sb = logits_dtype == DL_F32 ? 4 : 2;
  if (Vs % 8 != 0 || width % 8 != 0 || (grad && !ok16(grad, grad_stride, sb))) return DL_ERR_ALIGN;
  if (cols ? (reinterpret_cast<uintptr_t>(logits) % sb != 0 || reinterpret_cast<uintptr_t>(cols) % 16 != 0 ||
              reinterpret_cast<uintptr_t>(col_src16) % 16 != 0)
           : !ok16(logits, row_stride, sb))
    return DL_ERR_ALIGN;
  if (n_rows == 0) return DL_OK;
  MargParams p{};
  p.cols = cols; p.col_src16 = col_src16; p.Vs_full = cols ? Vs_full : 0;
  p.probs = t_probs; p.p_dtype = p_dtype; p.p_stride = p_stride; p.n_rows = n_teacher_rows; p.Vt = Vt; p.t2s = t2s;
  p.Vs = Vs; p.logits = logits; p.s_dtype = logits_dtype; p.row_stride = row_stride; p.n_srows = n_rows;
  p.row_map = row_map; p.inv_T_s = inv_T_student; p.inv_T_t = inv_T_teacher; p.grad_scale = grad_scale;
  p.row_loss = row_loss; p.grad = grad; p.grad_stride = grad_stride;
  const bool vec = p_dtype == DL_F32 && Vt % 4 == 0 && ok16(t_probs, p_stride, 4) && ok16(t2s, 0, 4);
  const size_t lds = attach_plan(p, plan_row_off, plan_ent, plan_tile, plan_fold, plan_n_fold, plan_n_extra, vec, (size_t)Vs * 4);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(xcd_banded_grid(n_rows)), block(MARG_NT);
  allow_large_lds();
#define DL_LAUNCH_RKLM(TAG)                                                                                  \
  do {                                                                                                       \
    if (vec) hipLaunchKernelGGL((rkl_marginalised_kernel<TAG, MARG_NU, true>), grid, block, lds, st, p);           \
    else hipLaunchKernelGGL((rkl_marginalised_kernel<TAG, MARG_NU, false>), grid, block, lds, st, p);              \
  } while (0)
  if (logits_dtype == DL_F32) DL_LAUNCH_RKLM(TagF32);
  else if (logits_dtype == DL_BF16) DL_LAUNCH_RKLM(TagBF16);
  else DL_LAUNCH_RKLM(TagF16);
#undef DL_LAUNCH_RKLM
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_rkl_marginalised(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t Vs,
                                   const int32_t* row_map, const void* t_probs, int p_dtype, int64_t p_stride,
                                   int64_t n_teacher_rows, int64_t Vt, const int32_t* t2s,
                                   const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                                   const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                                   float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                                   void* grad, int64_t grad_stride, void* stream) {
  return rkl_marginalised_launch(logits, logits_dtype, row_stride, n_rows, Vs, row_map, t_probs, p_dtype, p_stride,
                                 n_teacher_rows, Vt, t2s, plan_row_off, plan_ent, plan_tile, plan_fold, plan_n_fold,
                                 plan_n_extra, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride, nullptr,
                                 nullptr, 0, stream);
}

extern "C" int dl_rkl_marginalised_compact(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                                           int64_t Vs_full, const int32_t* cols, const uint16_t* col_src16, int64_t n_compact,
                                           const int32_t* row_map, const void* t_probs, int p_dtype, int64_t p_stride,
                                           int64_t n_teacher_rows, int64_t Vt, const int32_t* t2c,
                                           const int32_t* plan_row_off, const uint32_t* plan_ent, int plan_tile,
                                           const int32_t* plan_fold, int plan_n_fold, int plan_n_extra,
                                           float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                                           void* grad, int64_t grad_stride, void* stream) {
  if (!cols || !col_src16) return DL_ERR_NULL;
  return rkl_marginalised_launch(logits, logits_dtype, row_stride, n_rows, n_compact, row_map, t_probs, p_dtype, p_stride,
                                 n_teacher_rows, Vt, t2c, plan_row_off, plan_ent, plan_tile, plan_fold, plan_n_fold,
                                 plan_n_extra, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride, cols,
                                 reinterpret_cast<const unsigned short*>(col_src16), Vs_full, stream);
}

// dl_fkl_multi_teacher: forward KL against the weighted mixture of several sparse (top-K) teachers
// whose ids pass through a teacher -> student vocabulary map.
//
// Two launches.  (1) multi_prep_kernel, K-wide, one wave per teacher row: maps the ids, weighs and
// renormalises the masses (teacher temperature 1: the normaliser is the plain sum of the surviving
// masses, whatever ids they land on) and deals the entries, in stored order, into one bucket per
// column part of the loss kernel's row split.  (2) The loss kernels of dl_div_topk, instantiated with
// MULTI = true: a part's workgroup fetches only its own bucket -- a quarter of the row's entries
// for rows cut in four, by lane position, no count needed first -- and settles entries that share a
// student id on the per-chunk lists the gradient sweep keeps anyway (bucket_finish in
// topk_div.hpp).  No sort anywhere; every sum that depends on an order the hardware chooses is
// taken in fixed point.
#include "topk_div.hpp"
#include <cmath>

namespace dl {

constexpr int PREP_ROWS = 4;      // teacher rows per workgroup, one wave each

struct PrepParams {
  MultiTeacher mt; int val_dtype, idx_itype; int64_t V; int64_t n_trows;
  int parts; int part_shift;      // bucket of student id s: s >> part_shift (parts == 1: everything in bucket 0)
  int cap0; int E;
  uint2* first; uint2* more; int* head;
  u32x4* clear; int64_t clear_n16;      // the loss kernels' exchange records, zeroed on the way (clear_n16 == 0: nothing to clear)
};

// Exclusive prefix sum over the lanes of a wave of four 16-bit counters packed into 64 bits (no field
// may overflow: at most DL_MAX_TOPK entries per row); `total` receives the sum over all lanes.
__device__ __forceinline__ unsigned long long wave_scan_packed(unsigned long long v, unsigned long long& total) {
  const int lane = threadIdx.x & (WAVE - 1);
  unsigned long long incl = v;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const unsigned lo = (unsigned)__shfl_up((int)(unsigned)incl, o, WAVE), hi = (unsigned)__shfl_up((int)(unsigned)(incl >> 32), o, WAVE);
    if (lane >= o) incl += ((unsigned long long)hi << 32) | lo;
  }
  const unsigned tl = (unsigned)__shfl((int)(unsigned)incl, WAVE - 1, WAVE), th = (unsigned)__shfl((int)(unsigned)(incl >> 32), WAVE - 1, WAVE);
  total = ((unsigned long long)th << 32) | tl;
  return incl - v;
}

// One wave per teacher row, no barriers: the waves of a workgroup never meet.  J = slots of 64
// entries: slot j holds entries (j % S) * 64 + lane of teacher j / S, S = ceil(Kt / 64) -- the teacher
// behind a slot is the same for the whole wave, its pointers stay scalar.  An entry's place in its
// bucket: the entries of that bucket in lower lanes, then those of its own lane in lower slots -- a
// fixed function of the stored rows, found with one packed prefix sum per four buckets.
// Every load is issued whether or not its lane holds an entry (lanes without one read entry 0 of
// the row and discard it): no branch separates the loads, so all of them are in flight together.
// VD / IT: storage types of the teachers' log-probs and ids, compile-time so that the loads of all
// slots are issued back to back (a run-time switch per load would make every load wait for the one before).
// VEC: Kt is a multiple of 4 and the teachers' arrays are 16-byte aligned: a lane then takes four
// consecutive entries of a teacher with one load per array (slot j = entries 4 * (64 * (j / 4 % S) +
// lane) + j % 4 of teacher j / 4 / S, S = ceil(Kt / 256); J a multiple of 4) -- a quarter of the load
// instructions, which is what bounds this kernel: the CU's vector memory path takes about as long
// for a 4-byte-per-lane load as for a 16-byte one.
// WIDE: more than four buckets per row (a second packed word of counters; with four or fewer every
// reference to it folds away).
template <int J, int VD, int IT, bool VEC, bool WIDE>
__global__ __launch_bounds__(PREP_ROWS * WAVE) void multi_prep_kernel(const PrepParams p) {
  const MultiTeacher& m = p.mt;
  const int lane = threadIdx.x & (WAVE - 1);
  for (int64_t i = (int64_t)blockIdx.x * (PREP_ROWS * WAVE) + threadIdx.x; i < p.clear_n16; i += (int64_t)gridDim.x * (PREP_ROWS * WAVE))
    p.clear[i] = u32x4{0u, 0u, 0u, 0u};
  const int64_t trow = (int64_t)blockIdx.x * PREP_ROWS + threadIdx.x / WAVE;
  if (trow >= p.n_trows) return;
  const int S = (m.Kt + (VEC ? 4 : 1) * WAVE - 1) / ((VEC ? 4 : 1) * WAVE);
  const int P = p.parts;

  int64_t raw[J];
  float tv[J];
  bool live[J];
  if constexpr (VEC) {
    static_assert(J % 4 == 0, "four entries per lane and group");
#pragma unroll
    for (int g = 0; g < J / 4; ++g) {
      const int tj = min(g / S, m.n - 1);
      const int k0 = 4 * ((g - (g / S) * S) * WAVE + lane);
      const bool in = g / S < m.n && k0 < m.Kt;
      const int64_t at = trow * (int64_t)m.Kt + (in ? k0 : 0);
      if constexpr (IT == I32) {
        const int4 v = *reinterpret_cast<const int4*>(reinterpret_cast<const int32_t*>(m.idx[tj]) + at);
        raw[4 * g] = v.x; raw[4 * g + 1] = v.y; raw[4 * g + 2] = v.z; raw[4 * g + 3] = v.w;
      } else {
        const longlong2 a = *reinterpret_cast<const longlong2*>(reinterpret_cast<const int64_t*>(m.idx[tj]) + at);
        const longlong2 b = *reinterpret_cast<const longlong2*>(reinterpret_cast<const int64_t*>(m.idx[tj]) + at + 2);
        raw[4 * g] = a.x; raw[4 * g + 1] = a.y; raw[4 * g + 2] = b.x; raw[4 * g + 3] = b.y;
      }
      if constexpr (VD == F32) {
        const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(m.val[tj]) + at);
        tv[4 * g] = v.x; tv[4 * g + 1] = v.y; tv[4 * g + 2] = v.z; tv[4 * g + 3] = v.w;
      } else {
        const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(m.val[tj]) + at);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const unsigned short u = (unsigned short)((e < 2 ? v.x : v.y) >> (16 * (e & 1)));
          tv[4 * g + e] = VD == BF16 ? __uint_as_float((unsigned)u << 16) : (float)__builtin_bit_cast(_Float16, u);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        live[4 * g + e] = in;
        tv[4 * g + e] += m.logw[tj];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int tj = min(j / S, m.n - 1);
      const int kk = (j - (j / S) * S) * WAVE + lane;
      live[j] = j / S < m.n && kk < m.Kt;
      const int64_t at = trow * (int64_t)m.Kt + (live[j] ? kk : 0);
      if constexpr (IT == I32) raw[j] = (int64_t)reinterpret_cast<const int32_t*>(m.idx[tj])[at];
      else raw[j] = reinterpret_cast<const int64_t*>(m.idx[tj])[at];
      if constexpr (VD == F32) tv[j] = reinterpret_cast<const float*>(m.val[tj])[at];
      else if constexpr (VD == BF16) tv[j] = __uint_as_float((unsigned)reinterpret_cast<const unsigned short*>(m.val[tj])[at] << 16);
      else tv[j] = (float)reinterpret_cast<const _Float16*>(m.val[tj])[at];
      tv[j] += m.logw[tj];
    }
  }
  int id[J];
  if (m.id_map) {
    int32_t got[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      live[j] = live[j] && raw[j] >= 0 && raw[j] < m.Vt;
      got[j] = m.id_map[live[j] ? raw[j] : 0];
    }
#pragma unroll
    for (int j = 0; j < J; ++j) raw[j] = got[j];
  }
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const bool ok = live[j] && raw[j] >= 0 && raw[j] < p.V && tv[j] > -INFINITY;      // dropped, outside the vocabulary, zero weight or mass
    id[j] = ok ? (int)raw[j] : -1;
    tv[j] = ok ? tv[j] : -INFINITY;
  }

  // renormalise over the survivors: log q = tv - logsumexp(tv)
  float tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < J; ++j) tmax = fmaxf(tmax, tv[j]);
  tmax = wave_max(tmax);
  float tlse = 0.f;
  if (tmax > -INFINITY) {
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j) part += fast_exp2((tv[j] - tmax) * LOG2E);
    tlse = tmax + fast_log2(wave_sum(part)) * LN2;
  }

  // buckets: counters of four buckets share a 64-bit word, 16 bits each
  unsigned long long mine[2] = {0ull, 0ull};
#pragma unroll
  for (int j = 0; j < J; ++j) {
    if (id[j] < 0) continue;
    const int h = P == 1 ? 0 : min(id[j] >> p.part_shift, P - 1);
    mine[WIDE ? h >> 2 : 0] += 1ull << (16 * (h & 3));
  }
  unsigned long long total[2] = {0ull, 0ull}, at_lane[2] = {0ull, 0ull};
  at_lane[0] = wave_scan_packed(mine[0], total[0]);
  if (WIDE) at_lane[1] = wave_scan_packed(mine[1], total[1]);
  const auto field = [](const unsigned long long (&w)[2], int h) { return (int)((w[WIDE ? h >> 2 : 0] >> (16 * (h & 3))) & 0xffffull); };

  // The entries go to the wave's own stretch of LDS first, bucket after bucket, and from there to
  // memory in order: a lane's entries of one bucket lie up to J slots apart, so storing them straight
  // from the registers is J instructions of 64 lanes in 64 different lines each, and the vector memory
  // path takes a cycle per line; out of LDS a bucket leaves in whole 512-byte pieces.
  extern __shared__ __align__(16) uint2 staged_rows[];
  uint2* staged = staged_rows + (threadIdx.x / WAVE) * p.E;
  unsigned long long start[2] = {0ull, 0ull};          // where bucket h begins in `staged`, packed like the counters
  {
    int run = 0;
    for (int h = 0; h < P; ++h) {
      start[WIDE ? h >> 2 : 0] |= (unsigned long long)run << (16 * (h & 3));
      run += field(total, h);
    }
  }
#pragma unroll
  for (int j = 0; j < J; ++j) {
    if (id[j] < 0) continue;
    const int h = P == 1 ? 0 : min(id[j] >> p.part_shift, P - 1);
    const int at = field(start, h) + field(at_lane, h);
    at_lane[WIDE ? h >> 2 : 0] += 1ull << (16 * (h & 3));
    staged[at] = uint2{(unsigned)id[j], __float_as_uint(tv[j] - tlse)};
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  uint2* first = p.first + trow * (int64_t)P * p.cap0;
  uint2* more = p.more + trow * (int64_t)p.E;
  int spilled = 0;                                     // entries of lower buckets beyond their cap0: they lie back to back in `more`
  for (int h = 0; h < P; ++h) {
    const int n = field(total, h), from = field(start, h);
    for (int k = lane; k < n; k += WAVE) {
      const uint2 e = staged[from + k];
      if (k < p.cap0) first[(int64_t)h * p.cap0 + k] = e;
      else more[spilled + k - p.cap0] = e;             // rare: a bucket holds more than cap0 entries
    }
    spilled += max(n - p.cap0, 0);
  }
  // no padding: a part's workgroup reads cap0 slots of its bucket and goes by the count in the header
  int n_row = 0;
  for (int h = 0; h < P; ++h) n_row += field(total, h);
  if (lane < 16) {
    int v = lane < P ? field(total, lane & 7) : 0;
    if (lane == 8) v = n_row;
    if (lane == 9) v = __float_as_int(n_row > 0 ? 1.f : 0.f);      // the renormalised masses sum to one
    p.head[trow * 16 + lane] = v;
  }
}

// Slots of NT entries (register-resident in the loss kernel) a bucket is laid out for: enough for one
// and a half times an even share of the row's E entries, never more than hold all of them; 1, 2, 4 or 8.
static int bucket_slots(int E, int parts, int NT) {
  const int all = (E + NT - 1) / NT;
  const int likely = (3 * E / 2 + parts * NT - 1) / (parts * NT);
  const int want = std::min(all, std::max(likely, 1));
  for (int j : {1, 2, 4})
    if (want <= j) return j;
  return 8;      // E <= DL_MAX_TOPK keeps j * NT within the kernels' LDS budget
}

struct MultiPlan { FklShape shape; int cap0; int64_t exchange_bytes, first_bytes, head_bytes, more_bytes; };

static bool multi_plan(int logits_dtype, int64_t n_rows, int64_t V, int E, int64_t n_trows, int flags, MultiPlan& out) {
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  const int64_t nch = (V + 16 / eb - 1) / (16 / eb);      // a row that ends inside a chunk holds that chunk too
  const FklShape sh = fkl_shape(nch, eb, (flags >> DL_TOPK_PARTS_SHIFT) & 15, true);
  if (sh.NT == 0) return false;
  out.shape = sh;
  out.cap0 = bucket_slots(E, sh.parts, sh.NT) * sh.NT;
  const auto pad = [](int64_t b) { return (b + 255) & ~255LL; };
  out.exchange_bytes = sh.parts > 1 ? pad(RetryList::bytes(n_rows, sh.parts)) : 0;
  out.first_bytes = pad(n_trows * sh.parts * (int64_t)out.cap0 * 8);
  out.head_bytes = pad(n_trows * 64);
  out.more_bytes = pad(n_trows * (int64_t)E * 8);
  return true;
}

template <int J, int VD, bool VEC>
static void launch_prep_it(const PrepParams& p, hipStream_t st) {
  const dim3 grid((unsigned)((p.n_trows + PREP_ROWS - 1) / PREP_ROWS)), block(PREP_ROWS * WAVE);
  const size_t lds = (size_t)PREP_ROWS * p.E * sizeof(uint2);      // <= 64 KiB: E <= DL_MAX_TOPK
  if (p.parts > 4) {
    if (p.idx_itype == DL_I32) hipLaunchKernelGGL((multi_prep_kernel<J, VD, I32, VEC, true>), grid, block, lds, st, p);
    else hipLaunchKernelGGL((multi_prep_kernel<J, VD, I64, VEC, true>), grid, block, lds, st, p);
  } else {
    if (p.idx_itype == DL_I32) hipLaunchKernelGGL((multi_prep_kernel<J, VD, I32, VEC, false>), grid, block, lds, st, p);
    else hipLaunchKernelGGL((multi_prep_kernel<J, VD, I64, VEC, false>), grid, block, lds, st, p);
  }
}

template <int J, bool VEC>
static void launch_prep(const PrepParams& p, hipStream_t st) {
  if (p.val_dtype == DL_F16) launch_prep_it<J, F16, VEC>(p, st);
  else if (p.val_dtype == DL_F32) launch_prep_it<J, F32, VEC>(p, st);
  else launch_prep_it<J, BF16, VEC>(p, st);
}

}  // namespace dl

extern "C" int64_t dl_fkl_multi_teacher_workspace_bytes(int logits_dtype, int64_t n_rows, int64_t V, int n_teachers, int K,
                                                       int64_t n_teacher_rows, int flags) {
  using namespace dl;
  if (n_rows <= 0 || V <= 0 || n_teachers < 1 || K <= 0 || n_teacher_rows < 0 || (int64_t)n_teachers * K > DL_MAX_TOPK) return 0;
  MultiPlan plan;
  if (!multi_plan(logits_dtype, n_rows, V, n_teachers * K, n_teacher_rows, flags, plan)) return 0;
  return plan.exchange_bytes + plan.first_bytes + plan.head_bytes + plan.more_bytes;
}

extern "C" int dl_fkl_multi_teacher(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                                    const int32_t* row_map, int n_teachers, const void* const* t_vals,
                                    const void* const* t_idxs, int val_dtype, int idx_itype, int K,
                                    int64_t n_teacher_rows, const float* weights, const int32_t* id_map, int64_t Vt,
                                    float inv_T_student, float grad_scale, float* row_loss, void* grad,
                                    int64_t grad_stride, void* workspace, int64_t workspace_bytes, int flags,
                                    void* stream) {
  using namespace dl;
  if (!logits || ((!t_vals || !t_idxs || !weights) && n_teacher_rows > 0)) return DL_ERR_NULL;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || val_dtype < DL_F32 || val_dtype > DL_F16 ||
      (idx_itype != DL_I32 && idx_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || K <= 0 || n_teacher_rows < 0 || row_stride < V || (grad && grad_stride < V) ||
      (id_map && Vt <= 0))
    return DL_ERR_SHAPE;
  if (n_teachers < 1 || n_teachers > DL_MAX_TEACHERS || (int64_t)n_teachers * K > DL_MAX_TOPK || n_rows > 0x7fffffffLL ||
      n_teacher_rows > 0x7fffffffLL || V > 0x7fffffffLL)
    return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  const int E = n_teachers * K;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  const bool on_grid = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && ((row_stride * eb) % 16 == 0) &&
                       (!grad || (reinterpret_cast<uintptr_t>(grad) % 16 == 0 && (grad_stride * eb) % 16 == 0));
  if (!on_grid) return DL_ERR_ALIGN;
  const bool whole = V % (16 / eb) == 0;      // else the rows end inside a chunk: the ROWS_TAIL kernels
  MultiPlan plan;
  if (!multi_plan(logits_dtype, n_rows, V, E, n_teacher_rows, flags, plan)) return DL_ERR_LIMIT;
  if (!workspace || reinterpret_cast<uintptr_t>(workspace) % 256 != 0 ||
      workspace_bytes < plan.exchange_bytes + plan.first_bytes + plan.head_bytes + plan.more_bytes)
    return DL_ERR_WORKSPACE;
  char* ws = reinterpret_cast<char*>(workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);

  TopkParams p{};
  p.logits = logits; p.row_stride = row_stride; p.n_rows = n_rows; p.V = V; p.row_map = row_map;
  p.t_val_dtype = val_dtype; p.t_idx_itype = idx_itype;
  p.K = (std::max(plan.cap0, E) + plan.shape.NT - 1) / plan.shape.NT * plan.shape.NT;      // LDS entry slots
  p.n_trows = n_teacher_rows; p.t_cnt = nullptr;
  p.inv_T_s = inv_T_student; p.inv_T_t = 1.f; p.grad_scale = grad_scale;
  p.row_loss = row_loss; p.grad = grad; p.grad_stride = grad_stride;
  p.workspace = ws; p.parts = 1; p.spin_limit = (flags & DL_TOPK_NO_WAIT) ? 0 : SPIN_LIMIT;
  p.flags = flags | DL_TOPK_UNIQUE_IDS;      // the kernels settle shared ids themselves
  p.bk.first = reinterpret_cast<const uint2*>(ws + plan.exchange_bytes);
  p.bk.head = reinterpret_cast<const int*>(ws + plan.exchange_bytes + plan.first_bytes);
  p.bk.more = reinterpret_cast<const uint2*>(ws + plan.exchange_bytes + plan.first_bytes + plan.head_bytes);
  p.bk.cap0 = plan.cap0; p.bk.E = E;

  bool ws_cleared = false;
  if (n_teacher_rows > 0) {
    PrepParams q{};
    q.mt.n = n_teachers; q.mt.Kt = K; q.mt.id_map = id_map; q.mt.Vt = Vt;
    for (int j = 0; j < n_teachers; ++j) {
      if (!t_vals[j] || !t_idxs[j]) return DL_ERR_NULL;
      if (!(weights[j] >= 0.f) || !std::isfinite(weights[j])) return DL_ERR_SHAPE;
      q.mt.val[j] = t_vals[j]; q.mt.idx[j] = t_idxs[j];
      q.mt.logw[j] = weights[j] > 0.f ? logf(weights[j]) : -INFINITY;      // weight 0: the teacher's entries carry no mass
    }
    q.val_dtype = val_dtype; q.idx_itype = idx_itype; q.V = V; q.n_trows = n_teacher_rows;
    q.parts = plan.shape.parts;
    q.part_shift = __builtin_ctzll((uint64_t)plan.shape.NT * plan.shape.NCH * (16 / eb));      // columns per part: a power of two
    q.cap0 = plan.cap0; q.E = E;
    if (plan.shape.parts > 1) {      // saves the split kernels' own fill launch
      q.clear = reinterpret_cast<u32x4*>(ws); q.clear_n16 = split_clear_words(n_rows, plan.shape.parts);
      ws_cleared = true;
    }
    q.first = const_cast<uint2*>(p.bk.first); q.more = const_cast<uint2*>(p.bk.more); q.head = const_cast<int*>(p.bk.head);
    bool vec = K % 4 == 0;
    for (int j = 0; j < n_teachers; ++j)
      vec = vec && reinterpret_cast<uintptr_t>(t_vals[j]) % 16 == 0 && reinterpret_cast<uintptr_t>(t_idxs[j]) % 16 == 0;
    if (vec) {
      const int slots = 4 * n_teachers * ((K + 4 * WAVE - 1) / (4 * WAVE));      // <= 4 * (8 + 2048 / 256)
      if (slots <= 8) launch_prep<8, true>(q, st);
      else if (slots <= 16) launch_prep<16, true>(q, st);
      else if (slots <= 32) launch_prep<32, true>(q, st);
      else launch_prep<64, true>(q, st);
    } else {
      const int slots = n_teachers * ((K + WAVE - 1) / WAVE);                    // <= 8 + 2048 / 64
      if (slots <= 8) launch_prep<8, false>(q, st);
      else if (slots <= 16) launch_prep<16, false>(q, st);
      else launch_prep<40, false>(q, st);
    }
  }
  if (!whole) return launch_fkl_tail_multi(logits_dtype, p, plan.exchange_bytes, st, ws_cleared);
  return logits_dtype == DL_F32 ? launch_fkl<TagF32, true>(p, true, plan.exchange_bytes, st, ws_cleared)
         : logits_dtype == DL_BF16 ? launch_fkl<TagBF16, true>(p, true, plan.exchange_bytes, st, ws_cleared)
                                   : launch_fkl<TagF16, true>(p, true, plan.exchange_bytes, st, ws_cleared);
}

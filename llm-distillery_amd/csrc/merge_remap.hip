// Teacher-side preprocessing of sparse (top-K) distributions, one workgroup per token row:
//
//   * weighted multi-teacher merge with an optional teacher->student vocabulary id map:
//     mass = w_teacher * exp(logp); ids go through the map (-1 = dropped); entries that land on the
//     same id are summed in entry order; the survivors come out in ascending id order with
//     log(mass) -- a ragged sparse teacher that dl_div_topk consumes through its t_cnt argument;
//   * the dataset manager's pairwise merge: the same sum for two teachers without map, then the
//     K largest masses in descending order (ties: smaller id first).
//
// Both are a sort of at most 4096 (id, entry) keys in LDS (bitonic network on 64-bit keys), a
// segmented sum in sorted order -- fixed order, so the result is bit-reproducible -- and a
// compaction.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

constexpr int MERGE_NT = 256;
constexpr int MERGE_MAX_E = 4096;

struct MergeParams {
  int n_teachers;
  const void* val[DL_MAX_TEACHERS];
  const void* idx[DL_MAX_TEACHERS];
  float weight[DL_MAX_TEACHERS];
  int64_t rows[DL_MAX_TEACHERS];       // rows each teacher holds (pairwise merge: they may differ)
  int val_dtype, idx_itype, K;
  const int32_t* id_map; int64_t Vt; int64_t Vs;
  int64_t n_rows;
  int top_k;                           // 0: all survivors ascending by id; >0: the top_k largest masses
  int32_t* out_idx32; int64_t* out_idx64; float* out_logm; int32_t* out_cnt; int64_t out_stride;
};

// Sorts keys[0, MERGE_NT * EPL) (LDS) ascending: through registers, see block_sort.
template <class W, int EPL>
__device__ __forceinline__ void sort_keys(W* keys) {
  W c[EPL];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < EPL; ++j) c[j] = keys[threadIdx.x * EPL + j];
  block_sort<W, MERGE_NT, EPL>(c, keys);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < EPL; ++j) keys[threadIdx.x * EPL + j] = c[j];
  __syncthreads();
}

// (id, entry) sort keys: 32-bit `id << log2(Ep) | entry` when the student vocabulary leaves room
// (a third of the instructions of a 64-bit sort), else 64-bit `id << 32 | entry`.
template <class W, int EPL> struct IdEntryKey;
template <int EPL> struct IdEntryKey<unsigned, EPL> {
  static constexpr int EBITS = __builtin_ctz(EPL * MERGE_NT);
  static constexpr unsigned PAD = 0xffffffffu;
  __device__ static __forceinline__ unsigned make(int64_t id, int e) { return ((unsigned)id << EBITS) | (unsigned)e; }
  __device__ static __forceinline__ unsigned id(unsigned k) { return k >> EBITS; }
  __device__ static __forceinline__ unsigned entry(unsigned k) { return k & ((1u << EBITS) - 1u); }
};
template <int EPL> struct IdEntryKey<unsigned long long, EPL> {
  static constexpr unsigned long long PAD = ~0ull;
  __device__ static __forceinline__ unsigned long long make(int64_t id, int e) { return ((unsigned long long)id << 32) | (unsigned)e; }
  __device__ static __forceinline__ unsigned id(unsigned long long k) { return (unsigned)(k >> 32); }
  __device__ static __forceinline__ unsigned entry(unsigned long long k) { return (unsigned)k; }
};

// Exclusive prefix sum over n_pow2 flags (each thread owns a contiguous run); returns the total.
// Wave-level scans with lane shuffles, wave totals combined through LDS.
__device__ __forceinline__ int block_scan_flags(const unsigned char* flag, int* pos, int n_pow2, int* scratch) {
  const int per = n_pow2 / MERGE_NT;              // n_pow2 >= MERGE_NT
  const int begin = threadIdx.x * per;
  int local = 0;
  for (int i = 0; i < per; ++i) local += flag[begin + i];
  int incl = local;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const int up = __shfl_up(incl, o, WAVE);
    if (lane >= o) incl += up;
  }
  if (lane == WAVE - 1) scratch[w] = incl;
  __syncthreads();
  int base = 0, total = 0;
#pragma unroll
  for (int i = 0; i < MERGE_NT / WAVE; ++i) {
    const int v = scratch[i];
    if (i < w) base += v;
    total += v;
  }
  int run = base + incl - local;
  for (int i = 0; i < per; ++i) { pos[begin + i] = run; run += flag[begin + i]; }
  __syncthreads();
  return total;
}

template <int EPL, class W>
__global__ __launch_bounds__(MERGE_NT) void merge_kernel(const MergeParams p, int E) {
  constexpr int Ep = EPL * MERGE_NT;
  using KY = IdEntryKey<W, EPL>;
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned long long* keys = reinterpret_cast<unsigned long long*>(smem);            // Ep
  W* ikeys = reinterpret_cast<W*>(smem);                                              // the (id, entry) keys, same storage
  float* mass = reinterpret_cast<float*>(keys + Ep);                                  // Ep (by entry, later by slot)
  float* umass = mass + Ep;                                                           // Ep (by unique slot)
  int* uid = reinterpret_cast<int*>(umass + Ep);                                      // Ep
  int* pos = uid + Ep;                                                                // Ep
  int* scratch = pos + Ep;                                                            // MERGE_NT + 1
  unsigned char* flag = reinterpret_cast<unsigned char*>(scratch + MERGE_NT + 1);     // Ep
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int K = p.K;

  if (p.top_k > 0 && (r >= p.rows[0] || r >= p.rows[1])) {
    // pairwise merge, row held by one input only: it passes through in its stored order
    const int j = r < p.rows[0] ? 0 : 1;
    for (int k = tid; k < K; k += MERGE_NT) {
      const int64_t at = r * (int64_t)K + k;
      p.out_idx64[r * p.out_stride + k] = load_index(p.idx[j], p.idx_itype, at);
      p.out_logm[r * p.out_stride + k] = logf(expf(load_as_float(p.val[j], p.val_dtype, at)));
    }
    return;
  }

  // stage: key = (id << 32 | entry), mass by entry.  Three rounds of independent loads (ids and
  // values, then the id map) instead of one dependent chain per entry.
  int64_t id[EPL];
  float lv[EPL], wt[EPL];
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int e = u * MERGE_NT + tid;
    const int j = e < E ? e / K : 0, k = e - j * K;
    const bool live = e < E && r < p.rows[j];
    const int64_t at = live ? r * (int64_t)K + k : 0;
    const int64_t got = load_index(p.idx[j], p.idx_itype, at);
    const float v = load_as_float(p.val[j], p.val_dtype, at);
    id[u] = live ? got : -1;
    lv[u] = v;
    wt[u] = p.weight[j];
  }
  if (p.id_map) {
#pragma unroll
    for (int u = 0; u < EPL; ++u) {
      const bool in = id[u] >= 0 && id[u] < p.Vt;
      const int32_t mapped = p.id_map[in ? id[u] : 0];
      id[u] = in ? (int64_t)mapped : -1;
    }
  }
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int e = u * MERGE_NT + tid;
    const bool keep = id[u] >= 0 && id[u] < p.Vs;
    ikeys[e] = keep ? KY::make(id[u], e) : KY::PAD;
    mass[e] = keep ? wt[u] * expf(lv[u]) : 0.f;
  }
  sort_keys<W, EPL>(ikeys);

  // segment heads in sorted order
  for (int i = tid; i < Ep; i += MERGE_NT) {
    const W k = ikeys[i];
    flag[i] = (k != KY::PAD && (i == 0 || KY::id(ikeys[i - 1]) != KY::id(k))) ? 1 : 0;
  }
  __syncthreads();
  const int n_unique = block_scan_flags(flag, pos, Ep, scratch);
  for (int i = tid; i < Ep; i += MERGE_NT) {
    if (flag[i]) {
      const unsigned id = KY::id(ikeys[i]);
      float m = 0.f;
      for (int j = i; j < Ep && ikeys[j] != KY::PAD && KY::id(ikeys[j]) == id; ++j) m += mass[KY::entry(ikeys[j])];   // entry order
      uid[pos[i]] = (int)id;
      umass[pos[i]] = m;
    }
  }
  __syncthreads();

  const int64_t ob = r * p.out_stride;
  if (p.top_k == 0) {
    for (int u = tid; u < (int)p.out_stride; u += MERGE_NT) {
      const bool live = u < n_unique;
      if (p.out_idx32) p.out_idx32[ob + u] = live ? uid[u] : -1;
      if (p.out_idx64) p.out_idx64[ob + u] = live ? (int64_t)uid[u] : -1;
      p.out_logm[ob + u] = live ? logf(umass[u]) : -INFINITY;
    }
    if (tid == 0 && p.out_cnt) p.out_cnt[r] = n_unique;
    return;
  }
  // top_k largest masses, descending; ties towards the smaller id
  for (int i = tid; i < Ep; i += MERGE_NT)
    keys[i] = i < n_unique ? ((unsigned long long)(~__float_as_uint(umass[i])) << 32) | (unsigned)uid[i] : ~0ull;
  sort_keys<unsigned long long, EPL>(keys);
  for (int u = tid; u < p.top_k; u += MERGE_NT) {
    const bool live = u < n_unique;
    const unsigned long long k = keys[u];
    const int id = live ? (int)(unsigned)k : -1;
    const float m = live ? __uint_as_float(~(unsigned)(k >> 32)) : 0.f;
    if (p.out_idx32) p.out_idx32[ob + u] = id;
    if (p.out_idx64) p.out_idx64[ob + u] = id;
    p.out_logm[ob + u] = live ? logf(m) : -INFINITY;
  }
  if (tid == 0 && p.out_cnt) p.out_cnt[r] = n_unique < p.top_k ? n_unique : p.top_k;
}

static int launch_merge(MergeParams& p, hipStream_t st) {
  const int E = p.n_teachers * p.K;
  int Ep = 256;
  while (Ep < E) Ep <<= 1;
  const size_t lds = (size_t)Ep * (8 + 4 + 4 + 4 + 4 + 1) + (MERGE_NT + 1) * 4 + 16;
  const dim3 grid((unsigned)p.n_rows), block(MERGE_NT);
  // 32-bit (id, entry) keys if every id plus the all-ones padding id fits beside log2(Ep) entry bits
  const bool narrow = (uint64_t)p.Vs * (uint64_t)Ep < (1ull << 32) - (uint64_t)Ep;
#define DL_MERGE_CASE(EPL)                                                                              \
  if (narrow) hipLaunchKernelGGL((merge_kernel<EPL, unsigned>), grid, block, lds, st, p, E);             \
  else hipLaunchKernelGGL((merge_kernel<EPL, unsigned long long>), grid, block, lds, st, p, E);          \
  break;
  switch (Ep / MERGE_NT) {
    case 1: DL_MERGE_CASE(1)
    case 2: DL_MERGE_CASE(2)
    case 4: DL_MERGE_CASE(4)
    case 8: DL_MERGE_CASE(8)
    default: DL_MERGE_CASE(16)
  }
#undef DL_MERGE_CASE
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

}  // namespace dl

extern "C" int dl_merge_remap_topk(int n_teachers, const void* const* t_vals, const void* const* t_idxs,
                                   int val_dtype, int idx_itype, int K, const float* weights, int64_t n_rows,
                                   const int32_t* id_map, int64_t Vt, int64_t Vs, int32_t* out_idx,
                                   float* out_logmass, int32_t* out_cnt, void* stream) {
  using namespace dl;
  if (!t_vals || !t_idxs || !weights || !out_idx || !out_logmass || !out_cnt) return DL_ERR_NULL;
  if (n_teachers < 1 || n_teachers > DL_MAX_TEACHERS) return DL_ERR_LIMIT;
  if (val_dtype < DL_F32 || val_dtype > DL_F16 || (idx_itype != DL_I32 && idx_itype != DL_I64)) return DL_ERR_DTYPE;
  if (K <= 0 || n_rows < 0 || Vs <= 0 || (id_map && Vt <= 0)) return DL_ERR_SHAPE;
  if ((int64_t)n_teachers * K > MERGE_MAX_E || n_rows > 0x7fffffffLL || Vs > 0x7fffffffLL) return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  MergeParams p{};
  p.n_teachers = n_teachers;
  for (int j = 0; j < n_teachers; ++j) {
    if (!t_vals[j] || !t_idxs[j]) return DL_ERR_NULL;
    p.val[j] = t_vals[j]; p.idx[j] = t_idxs[j]; p.weight[j] = weights[j]; p.rows[j] = n_rows;
  }
  p.val_dtype = val_dtype; p.idx_itype = idx_itype; p.K = K;
  p.id_map = id_map; p.Vt = Vt; p.Vs = Vs; p.n_rows = n_rows; p.top_k = 0;
  p.out_idx32 = out_idx; p.out_idx64 = nullptr; p.out_logm = out_logmass; p.out_cnt = out_cnt;
  p.out_stride = (int64_t)n_teachers * K;
  return launch_merge(p, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int dl_merge_topk_pair(const void* disk_val, const void* disk_idx, int64_t disk_rows, const void* new_val,
                                  const void* new_idx, int64_t new_rows, int val_dtype, int idx_itype, int K,
                                  int64_t V, float* out_logmass, int64_t* out_idx, void* stream) {
  using namespace dl;
  if (!disk_val || !disk_idx || !new_val || !new_idx || !out_logmass || !out_idx) return DL_ERR_NULL;
  if (val_dtype < DL_F32 || val_dtype > DL_F16 || (idx_itype != DL_I32 && idx_itype != DL_I64)) return DL_ERR_DTYPE;
  if (K <= 0 || disk_rows < 0 || new_rows < 0 || V <= 0) return DL_ERR_SHAPE;
  if (2 * (int64_t)K > MERGE_MAX_E || V > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int64_t n = disk_rows > new_rows ? disk_rows : new_rows;
  if (n == 0) return DL_OK;
  if (n > 0x7fffffffLL) return DL_ERR_LIMIT;
  MergeParams p{};
  p.n_teachers = 2;
  p.val[0] = disk_val; p.idx[0] = disk_idx; p.weight[0] = 1.f; p.rows[0] = disk_rows;
  p.val[1] = new_val; p.idx[1] = new_idx; p.weight[1] = 1.f; p.rows[1] = new_rows;
  p.val_dtype = val_dtype; p.idx_itype = idx_itype; p.K = K;
  p.id_map = nullptr; p.Vt = 0; p.Vs = V; p.n_rows = n; p.top_k = K;
  p.out_idx32 = nullptr; p.out_idx64 = out_idx; p.out_logm = out_logmass; p.out_cnt = nullptr;
  p.out_stride = K;
  return launch_merge(p, reinterpret_cast<hipStream_t>(stream));
}

// Teacher-side producer: full-vocabulary log-softmax and the K largest entries per token row,
// emitted in the dataset's storage layout (log-probs fp16 or fp32, ids int32 or int64, descending).
//
// Two launches.  (1) One workgroup per column part of a row (256 threads x 16 chunks of 16 bytes,
// the part read from HBM once into registers; four workgroups share a CU so that one part's loads
// overlap another's arithmetic).  After the max / sum-exp sweeps the registers are rewritten in place
// as order-preserving unsigned keys and every chunk's largest key is kept.  The K-th largest of those
// chunk maxima is a lower bound L of the part's K-th largest key (K distinct entries reach it), and
// with 4096 chunks per part only ~K..1.2K entries lie at or above it: they are collected into LDS,
// sorted (key descending, column ascending) and the best K written to a per-part record together with
// the part's (max, sum-exp).  (2) One workgroup per row merges the sorted part lists by rank and the
// statistics into the row's log-sum-exp.
// Ties go to the smaller id, deterministically; torch.topk, which the reference calls, leaves tie
// order open.  Rows with more than 2048 entries at or above L (constant or coarsely quantised rows)
// take an exact but slow select by bisection over key bits and then over columns.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

constexpr int PROD_MAX_K = 1024;
constexpr int PROD_NT = 256, PROD_NCH = 16;
constexpr int PROD_CAP = 2048;              // candidates of a part held in LDS
constexpr int PROD_RANK_SORT_MAX = 512;     // at most this many candidates are sorted by counting
constexpr int PROD_MAX_PARTS = 8;

typedef unsigned long long u64;
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

struct PartHeader { float mx; float sm; int cnt; int pad; };     // 16 bytes, then cnt sorted u64 entries

struct ProducerParams {
  const void* logits; int64_t row_stride; int64_t V;
  const int32_t* row_list; int64_t n_out;
  int K; int parts;
  char* ws; int64_t part_stride;            // bytes per (row, part) record
  void* out_val; int out_dtype; void* out_idx; int out_itype;
};

__host__ __device__ inline int64_t producer_part_stride(int K) { return 16 + (((int64_t)K * 8 + 15) & ~15LL); }

// ---- order-preserving keys ---------------------------------------------------------------------
// 16-bit storage types are handled as packed pairs of 16-bit keys, fp32 as 32-bit keys.
template <class Tag> struct Keys;

template <> struct Keys<TagF32> {
  static constexpr int BITS = 32;
  static constexpr int PER_DWORD = 1;
  __device__ static __forceinline__ unsigned encode(unsigned u) {      // dword of raw bits -> dword of keys
    return u ^ ((unsigned)((int)u >> 31) | 0x80000000u);
  }
  __device__ static __forceinline__ unsigned key(unsigned kd, int) { return kd; }
  __device__ static __forceinline__ unsigned dword_max(unsigned a, unsigned b) { return a > b ? a : b; }
  __device__ static __forceinline__ unsigned top_key(unsigned m) { return m; }
  __device__ static __forceinline__ float value(unsigned k) {
    const unsigned u = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
    return __uint_as_float(u);
  }
};

template <bool IS_BF16> struct Keys16 {
  static constexpr int BITS = 16;
  static constexpr int PER_DWORD = 2;
  __device__ static __forceinline__ unsigned encode(unsigned u) {
    const unsigned neg = (u >> 15) & 0x00010001u;            // 1 per negative half
    return u ^ (neg * 0x7fffu) ^ 0x80008000u;                // negative: flip all 16 bits; else flip the sign bit
  }
  __device__ static __forceinline__ unsigned key(unsigned kd, int half) { return half ? (kd >> 16) : (kd & 0xffffu); }
  __device__ static __forceinline__ unsigned dword_max(unsigned a, unsigned b) {     // per 16-bit half
    const u16x2 m = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(unsigned, m);
  }
  __device__ static __forceinline__ unsigned top_key(unsigned m) { const unsigned l = m & 0xffffu, h = m >> 16; return l > h ? l : h; }
  __device__ static __forceinline__ float value(unsigned k) {
    const unsigned h = (k & 0x8000u) ? (k ^ 0x8000u) : (~k & 0xffffu);
    if (IS_BF16) return __uint_as_float(h << 16);
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
  }
};
template <> struct Keys<TagBF16> : Keys16<true> {};
template <> struct Keys<TagF16> : Keys16<false> {};

// Sum of a per-thread integer over the workgroup; two barriers, scratch reusable at once.
template <int NT>
__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  constexpr int NW = NT / WAVE;
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  int r = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) r += scratch[i];
  __syncthreads();
  return r;
}

// Number of entries of the part for which pred(key, column inside the part) holds.
template <class Tag, int NT, int NCH, class Pred>
__device__ __forceinline__ int count_entries(u32x4 (&reg)[NCH], int my_chunks, int* scratch, Pred pred) {
  using KY = Keys<Tag>;
  int c = 0;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    forget(reg[i]);       // the sweep is repeated in bisection loops: keep its unpacked keys from being hoisted out of them
    if (i < my_chunks) {
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < KY::PER_DWORD; ++h) {
          const int col = (i * NT + (int)threadIdx.x) * Chunk<Tag>::N + d * KY::PER_DWORD + h;
          c += pred(KY::key(reg[i][d], h), col) ? 1 : 0;
        }
    }
  }
  return block_sum_int<NT>(c, scratch);
}

// Appends the entries for which pred holds to cand (LDS); slots beyond PROD_CAP are counted, not written.
template <class Tag, int NT, int NCH, class Pred>
__device__ __forceinline__ void collect_entries(const u32x4 (&reg)[NCH], int i, int lo, u64* cand, int* n_cand, Pred pred) {
  using KY = Keys<Tag>;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int h = 0; h < KY::PER_DWORD; ++h) {
      const unsigned k = KY::key(reg[i][d], h);
      const int col = (i * NT + (int)threadIdx.x) * Chunk<Tag>::N + d * KY::PER_DWORD + h;
      if (pred(k, col)) {
        const int slot = atomicAdd(n_cand, 1);
        if (slot < PROD_CAP) cand[slot] = ((u64)(~k) << 32) | (unsigned)(lo + col);     // ascending = key descending, id ascending
      }
    }
}

template <class Tag>
__global__ __launch_bounds__(PROD_NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void topk_part_kernel(const ProducerParams p) {
  constexpr int NT = PROD_NT, NCH = PROD_NCH, NW = NT / WAVE;
  using C = Chunk<Tag>;
  using KY = Keys<Tag>;
  __shared__ float red[64];
  __shared__ int ired[NW];
  __shared__ int slots[2 * NW];
  __shared__ int s_n;
  __shared__ __align__(16) u64 cand[PROD_CAP];

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  const int P = p.parts;
  const int64_t ro = blockIdx.x / (unsigned)P;
  const int h_part = (int)(blockIdx.x % (unsigned)P);
  const int64_t r = p.row_list ? (int64_t)p.row_list[ro] : ro;
  const int64_t c0 = (int64_t)h_part * NT * NCH;
  const int nch = (int)min((int64_t)NT * NCH, p.V / C::N - c0);      // chunks of this part, >= 1
  const int lo = (int)(c0 * C::N);
  const int n_elems = nch * C::N;
  const int Kp = min(p.K, n_elems);
  const char* rpart = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes + c0 * 16;
  char* rec = p.ws + ((int64_t)blockIdx.x) * p.part_stride;

  u32x4 reg[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = i * NT + tid;
    reg[i] = c < nch ? load16_stream(rpart + (int64_t)c * 16) : C::neg_inf();
  }
  if (tid == 0) s_n = 0;

  // max and sum-exp of the part (natural log-softmax; no temperature at collection time)
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) mx = fmaxf(mx, f[e]);
  }
  mx = block_max<NT>(mx, red);
  const float mb = (mx == -INFINITY) ? 0.f : mx * LOG2E;
  float sm = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[e], LOG2E, -mb));
  }
  sm = block_sum<NT>(sm, red);

  // raw bits -> ordered keys, in place; largest key of every chunk
  const int my_chunks = (nch - tid + NT - 1) / NT;                  // chunks i < my_chunks are inside the part
  unsigned gm[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    forget(reg[i]);
#pragma unroll
    for (int d = 0; d < 4; ++d) reg[i][d] = KY::encode(reg[i][d]);
    const unsigned m = KY::dword_max(KY::dword_max(reg[i][0], reg[i][1]), KY::dword_max(reg[i][2], reg[i][3]));
    gm[i] = i < my_chunks ? KY::top_key(m) : 0u;
  }

  // L = Kp-th largest chunk maximum, found bit by bit (0 when the part has fewer chunks than Kp)
  unsigned L = 0;
  if (nch >= Kp) {
#pragma unroll 1
    for (int b = KY::BITS - 1; b >= 0; --b) {
      const unsigned t = L | (1u << b);
      int c = 0;
#pragma unroll
      for (int i = 0; i < NCH; ++i) c += __popcll(__ballot(gm[i] >= t));
      int* sl = slots + (b & 1) * NW;
      if (lane == 0) sl[w] = c;
      __syncthreads();
      int tot = 0;
#pragma unroll
      for (int j = 0; j < NW; ++j) tot += sl[j];
      if (tot >= Kp) L = t;
    }
  }
  __syncthreads();

  // entries at or above L; the chunk maxima tell which chunks hold any
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    if (i < my_chunks && gm[i] >= L)
      collect_entries<Tag, NT, NCH>(reg, i, lo, cand, &s_n, [L](unsigned k, int) { return k >= L; });
  }
  __syncthreads();
  int n = s_n;

  if (n > PROD_CAP) {
    // exact select: T = Kp-th largest key by bisection over key bits, then the smallest columns among its ties
    unsigned T = 0;
#pragma unroll 1
    for (int b = KY::BITS - 1; b >= 0; --b) {
      const unsigned t = T | (1u << b);
      if (count_entries<Tag, NT, NCH>(reg, my_chunks, ired, [t](unsigned k, int) { return k >= t; }) >= Kp) T = t;
    }
    const int n_gt = count_entries<Tag, NT, NCH>(reg, my_chunks, ired, [T](unsigned k, int) { return k > T; });
    const int need = Kp - n_gt;                                     // >= 1 ties to take
    int clo = 0, chi = n_elems - 1;                                 // smallest column bound with `need` ties at or below it
    while (clo < chi) {
      const int mid = clo + (chi - clo) / 2;
      const int cnt = count_entries<Tag, NT, NCH>(reg, my_chunks, ired,
                                                  [T, mid](unsigned k, int col) { return k == T && col <= mid; });
      if (cnt >= need) chi = mid; else clo = mid + 1;
    }
    if (tid == 0) s_n = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < my_chunks)
        collect_entries<Tag, NT, NCH>(reg, i, lo, cand, &s_n,
                                      [T, clo](unsigned k, int col) { return k > T || (k == T && col <= clo); });
    }
    __syncthreads();
    n = s_n;                                                        // == Kp
  }

  // ---- sort the n >= Kp candidates, emit the best Kp -------------------------------------------
  u64* lst = reinterpret_cast<u64*>(rec + 16);
  if (n <= PROD_RANK_SORT_MAX) {
    if (tid == 0 && (n & 1)) cand[n] = ~0ull;
    __syncthreads();
    const int pairs = (n + 1) / 2;
    const ulonglong2* c2 = reinterpret_cast<const ulonglong2*>(cand);
    for (int ai = tid; ai < n; ai += NT) {
      const u64 a = cand[ai];
      int rank = 0;
#pragma unroll 4
      for (int b = 0; b < pairs; ++b) {
        const ulonglong2 v = c2[b];
        rank += (v.x < a ? 1 : 0) + (v.y < a ? 1 : 0);
      }
      if (rank < Kp) lst[rank] = a;
    }
  } else {
    int n2 = 1024;
    while (n2 < n) n2 <<= 1;
    for (int a = n + tid; a < n2; a += NT) cand[a] = ~0ull;
    __syncthreads();
    for (int size = 2; size <= n2; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int t = tid; t < n2 / 2; t += NT) {
          const int lo_i = 2 * t - (t & (stride - 1)), hi_i = lo_i + stride;
          const bool up = (lo_i & size) == 0;
          const u64 a = cand[lo_i], b = cand[hi_i];
          if ((a > b) == up) { cand[lo_i] = b; cand[hi_i] = a; }
        }
        __syncthreads();
      }
    }
    for (int k = tid; k < Kp; k += NT) lst[k] = cand[k];
  }
  if (tid == 0) {
    PartHeader hd{mx, sm, Kp, 0};
    *reinterpret_cast<PartHeader*>(rec) = hd;
  }
}

// Merge of the parts of one row: log-sum-exp from the part statistics; every listed entry's final
// position is its position in its own sorted list plus the number of smaller entries in the others
// (no two entries are equal: the column is part of the sort word).
template <class Tag>
__global__ __launch_bounds__(256) void topk_merge_kernel(const ProducerParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  u64* lists = reinterpret_cast<u64*>(smem_raw);                    // parts x K
  __shared__ int s_cnt[PROD_MAX_PARTS];
  const int tid = threadIdx.x;
  const int64_t ro = blockIdx.x;
  const int P = p.parts, K = p.K;
  const char* rec0 = p.ws + ro * P * p.part_stride;

  float M = -INFINITY;
  for (int q = 0; q < P; ++q) M = fmaxf(M, reinterpret_cast<const PartHeader*>(rec0 + q * p.part_stride)->mx);
  float S = 0.f;
  for (int q = 0; q < P; ++q) {
    const PartHeader hd = *reinterpret_cast<const PartHeader*>(rec0 + q * p.part_stride);
    if (hd.mx != -INFINITY) S += hd.sm * fast_exp2((hd.mx - M) * LOG2E);
    if (tid == 0) s_cnt[q] = hd.cnt;
    const u64* lst = reinterpret_cast<const u64*>(rec0 + q * p.part_stride + 16);
    for (int j = tid; j < hd.cnt; j += 256) lists[q * K + j] = lst[j];
  }
  const float lse = (M * LOG2E + fast_log2(S)) * LN2;
  __syncthreads();

  for (int item = tid; item < P * K; item += 256) {
    const int q = item / K, j = item - q * K;
    if (j >= s_cnt[q]) continue;
    const u64 a = lists[item];
    int rank = j;
    for (int o = 0; o < P; ++o) {
      if (o == q) continue;
      const u64* l = lists + o * K;
      int lo = 0, hi = s_cnt[o];                                    // -> number of entries of list o below a
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (l[mid] < a) lo = mid + 1; else hi = mid;
      }
      rank += lo;
    }
    if (rank < K) {
      const float logp = Keys<Tag>::value(~(unsigned)(a >> 32)) - lse;
      const int col = (int)(unsigned)a;
      store_from_float(p.out_val, p.out_dtype, ro * K + rank, logp);
      if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * K + rank] = col;
      else reinterpret_cast<int64_t*>(p.out_idx)[ro * K + rank] = col;
    }
  }
}

static int producer_parts(int64_t V, int logits_dtype) {
  const int64_t nch = V / (logits_dtype == DL_F32 ? 4 : 8);
  return (int)((nch + PROD_NT * PROD_NCH - 1) / (PROD_NT * PROD_NCH));
}

template <class Tag>
static int launch_producer(const ProducerParams& p, hipStream_t st) {
  hipLaunchKernelGGL((topk_part_kernel<Tag>), dim3((unsigned)(p.n_out * p.parts)), dim3(PROD_NT), 0, st, p);
  hipLaunchKernelGGL((topk_merge_kernel<Tag>), dim3((unsigned)p.n_out), dim3(256), (size_t)p.parts * p.K * 8, st, p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

}  // namespace dl

extern "C" int64_t dl_teacher_topk_workspace_bytes(int logits_dtype, int64_t n_out, int64_t V, int K) {
  if (n_out <= 0 || V <= 0 || K <= 0) return 0;
  return n_out * dl::producer_parts(V, logits_dtype) * dl::producer_part_stride(K);
}

extern "C" int dl_teacher_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                               const int32_t* row_list, int64_t n_out, int K, void* out_val, int out_dtype,
                               void* out_idx, int out_itype, void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace dl;
  if (!logits || !out_val || !out_idx) return DL_ERR_NULL;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || (out_dtype != DL_F32 && out_dtype != DL_F16) ||
      (out_itype != DL_I32 && out_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || n_out < 0 || V <= 0 || K <= 0 || K > V || row_stride < V || (!row_list && n_out > n_rows))
    return DL_ERR_SHAPE;
  const int parts = producer_parts(V, logits_dtype);
  if (K > PROD_MAX_K || parts > PROD_MAX_PARTS || V > 0x7fffffffLL || n_out * parts > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (V % (16 / eb) != 0 || reinterpret_cast<uintptr_t>(logits) % 16 != 0 || (row_stride * eb) % 16 != 0)
    return DL_ERR_ALIGN;
  if (n_out == 0) return DL_OK;
  if (!workspace) return DL_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return DL_ERR_ALIGN;
  if (workspace_bytes < dl_teacher_topk_workspace_bytes(logits_dtype, n_out, V, K)) return DL_ERR_WORKSPACE;
  ProducerParams p{logits, row_stride, V, row_list, n_out, K, parts, reinterpret_cast<char*>(workspace),
                   producer_part_stride(K), out_val, out_dtype, out_idx, out_itype};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  return logits_dtype == DL_F32 ? launch_producer<TagF32>(p, st)
         : logits_dtype == DL_BF16 ? launch_producer<TagBF16>(p, st)
                                   : launch_producer<TagF16>(p, st);
}

// Teacher-side producer: full-vocabulary log-softmax and the K largest entries per token row,
// emitted in the dataset's storage layout (log-probs fp16 or fp32, ids int32 or int64, descending).
//
// One workgroup per output row; the row is read from HBM once into registers.  After the
// max / sum-exp sweeps the registers are rewritten in place as order-preserving unsigned keys, and
// the K-th largest key is found by a radix select from the most significant byte down:
//   * first byte: per-thread register counters over a 4-bin window that starts at the bin of the
//     row maximum and slides down until it holds the K-th entry (the top entries of a logits row
//     share one or two exponents, so one window almost always suffices);
//   * remaining bytes: a 256-bin LDS histogram over the few entries that match the prefix.
// Entries above the threshold key and the lowest-index entries equal to it are collected in LDS and
// sorted (key descending, index ascending) with a bitonic network.  Ties therefore go to the
// smaller id, deterministically; torch.topk, which the reference calls, leaves tie order open.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

constexpr int PROD_MAX_K = 1024;
constexpr int PROD_EQ_CAP = 1024;

struct ProducerParams {
  const void* logits; int64_t row_stride; int64_t V;
  const int32_t* row_list; int64_t n_out;
  int K;
  void* out_val; int out_dtype; void* out_idx; int out_itype;
};

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
  __device__ static __forceinline__ float value(unsigned k) {
    const unsigned h = (k & 0x8000u) ? (k ^ 0x8000u) : (~k & 0xffffu);
    if (IS_BF16) return __uint_as_float(h << 16);
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
  }
};
template <> struct Keys<TagBF16> : Keys16<true> {};
template <> struct Keys<TagF16> : Keys16<false> {};

template <int NT>
__device__ __forceinline__ void block_sum4(int (&c)[4], int* scratch) {
  constexpr int NW = NT / WAVE;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) c[j] += __shfl_xor(c[j], o, WAVE);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) scratch[j * NW + w] = c[j];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int r = 0;
#pragma unroll
    for (int i = 0; i < NW; ++i) r += scratch[j * NW + i];
    c[j] = r;
  }
  __syncthreads();
}

template <int NT>
__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  int c[4] = {v, 0, 0, 0};
  block_sum4<NT>(c, scratch);
  return c[0];
}

template <class Tag, int NT, int NCH>
__global__ __launch_bounds__(NT) void topk_producer_kernel(const ProducerParams p) {
  using C = Chunk<Tag>;
  using KY = Keys<Tag>;
  __shared__ float red[64];
  __shared__ int ired[4 * (NT / WAVE)];
  __shared__ int hist[256];
  __shared__ int s_pick[2];                       // digit chosen by a histogram pass, entries above it
  __shared__ int s_nsel, s_neq;
  __shared__ unsigned long long cand[PROD_MAX_K];
  __shared__ int eq[PROD_EQ_CAP];

  const int tid = threadIdx.x;
  const int64_t ro = blockIdx.x;
  const int64_t r = p.row_list ? (int64_t)p.row_list[ro] : ro;
  const int64_t nch = p.V / C::N;
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  const int K = p.K;

  u32x4 reg[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int64_t c = (int64_t)i * NT + tid;
    reg[i] = c < nch ? load16_stream(row + c * 16) : C::neg_inf();
  }
  if (tid == 0) { s_nsel = 0; s_neq = 0; }

  // log-sum-exp (natural; no temperature at collection time)
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
  const float mb = mx * LOG2E;
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
  const float lse = (mb + fast_log2(sm)) * LN2;

  // raw bits -> ordered keys, in place.  Chunks beyond the row hold -inf: the smallest finite-or-inf key.
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    forget(reg[i]);
#pragma unroll
    for (int d = 0; d < 4; ++d) reg[i][d] = KY::encode(reg[i][d]);
  }
  const int my_chunks = (int)((nch - tid + NT - 1) / NT);          // chunks i < my_chunks are inside the row

  // ---- radix select, most significant byte first ----------------------------------------------
  constexpr int NDIG = KY::BITS / 8;
  unsigned prefix = 0;           // chosen digits so far, right-aligned
  int need = K;                  // entries still to take among keys whose prefix matches
  {
    // first byte: sliding 4-bin window from the bin of the row maximum downwards
    unsigned maxbits;
    if (KY::BITS == 32) maxbits = KY::encode(__float_as_uint(mx));
    else if (Tag::id == BF16) maxbits = KY::key(KY::encode(__float_as_uint(mx) >> 16), 0);
    else maxbits = KY::key(KY::encode((unsigned)__builtin_bit_cast(unsigned short, (_Float16)mx)), 0);
    int top = (int)(maxbits >> (KY::BITS - 8));
    for (;;) {
      int c[4] = {0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if (i < my_chunks) {
#pragma unroll
          for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int h = 0; h < KY::PER_DWORD; ++h) {
              const int dig = (int)(KY::key(reg[i][d], h) >> (KY::BITS - 8));
              const int off = top - dig;
#pragma unroll
              for (int j = 0; j < 4; ++j) c[j] += (off == j) ? 1 : 0;
            }
        }
      }
      block_sum4<NT>(c, ired);
      int found = -1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (found < 0) {
          if (c[j] >= need) found = j; else need -= c[j];
        }
      }
      if (found >= 0) { prefix = (unsigned)(top - found); break; }
      top -= 4;
      if (top < 0) { prefix = 0; break; }       // cannot happen for K <= V; keeps the loop bounded
    }
  }
#pragma unroll 1
  for (int dg = 1; dg < NDIG; ++dg) {
    const int shift = KY::BITS - 8 * (dg + 1);
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < my_chunks) {
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int h = 0; h < KY::PER_DWORD; ++h) {
            const unsigned k = KY::key(reg[i][d], h);
            if ((k >> (shift + 8)) == prefix) atomicAdd(&hist[(k >> shift) & 0xffu], 1);
          }
      }
    }
    __syncthreads();
    if (tid == 0) {
      int n = need, pick = 0;
      for (int b = 255; b >= 0; --b) {
        const int hcnt = hist[b];
        if (hcnt >= n) { pick = b; break; }
        n -= hcnt;
      }
      s_pick[0] = pick;
      s_pick[1] = n;
    }
    __syncthreads();
    prefix = (prefix << 8) | (unsigned)s_pick[0];
    need = s_pick[1];
    __syncthreads();
  }
  const unsigned T = prefix;     // the K-th largest key; `need` of the entries equal to it are taken

  // ---- collect ---------------------------------------------------------------------------------
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    if (i < my_chunks) {
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < KY::PER_DWORD; ++h) {
          const unsigned k = KY::key(reg[i][d], h);
          const int col = (int)(((int64_t)i * NT + tid) * C::N) + d * KY::PER_DWORD + h;
          if (k > T) {
            const int slot = atomicAdd(&s_nsel, 1);
            cand[slot] = ((unsigned long long)(~k) << 32) | (unsigned)col;
          } else if (k == T) {
            const int slot = atomicAdd(&s_neq, 1);
            if (slot < PROD_EQ_CAP) eq[slot] = col;
          }
        }
    }
  }
  __syncthreads();
  const int n_sel = s_nsel, n_eq = s_neq;        // n_sel + need == K
  if (n_eq <= PROD_EQ_CAP) {
    // the `need` smallest indices among the ties: rank by counting (ties are few)
    for (int a = tid; a < n_eq; a += NT) {
      const int col = eq[a];
      int rank = 0;
      for (int b = 0; b < n_eq; ++b) rank += eq[b] < col ? 1 : 0;
      if (rank < need) cand[n_sel + rank] = ((unsigned long long)(~T) << 32) | (unsigned)col;
    }
  } else {
    // very many ties (e.g. a constant row): smallest column bound I with `need` ties at or below it
    int lo = 0, hi = (int)p.V - 1;
    while (lo < hi) {
      const int mid = lo + (hi - lo) / 2;
      int cnt = 0;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if (i < my_chunks) {
#pragma unroll
          for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int h = 0; h < KY::PER_DWORD; ++h) {
              const int col = (int)(((int64_t)i * NT + tid) * C::N) + d * KY::PER_DWORD + h;
              cnt += (KY::key(reg[i][d], h) == T && col <= mid) ? 1 : 0;
            }
        }
      }
      cnt = block_sum_int<NT>(cnt, ired);
      if (cnt >= need) hi = mid; else lo = mid + 1;
    }
    if (tid == 0) s_neq = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < my_chunks) {
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int h = 0; h < KY::PER_DWORD; ++h) {
            const int col = (int)(((int64_t)i * NT + tid) * C::N) + d * KY::PER_DWORD + h;
            if (KY::key(reg[i][d], h) == T && col <= lo) {
              const int slot = atomicAdd(&s_neq, 1);
              cand[n_sel + slot] = ((unsigned long long)(~T) << 32) | (unsigned)col;
            }
          }
      }
    }
  }
  for (int a = K + tid; a < PROD_MAX_K; a += NT) cand[a] = ~0ull;
  __syncthreads();

  // ---- sort: key descending, column ascending --------------------------------------------------
  int n2 = 64;
  while (n2 < K) n2 <<= 1;
  for (int size = 2; size <= n2; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = tid; t < n2 / 2; t += NT) {
        const int lo_i = 2 * t - (t & (stride - 1)), hi_i = lo_i + stride;
        const bool up = (lo_i & size) == 0;
        const unsigned long long a = cand[lo_i], b = cand[hi_i];
        if ((a > b) == up) { cand[lo_i] = b; cand[hi_i] = a; }
      }
      __syncthreads();
    }
  }
  for (int k = tid; k < K; k += NT) {
    const unsigned long long c = cand[k];
    const unsigned key = ~(unsigned)(c >> 32);
    const int col = (int)(unsigned)c;
    const float logp = KY::value(key) - lse;
    store_from_float(p.out_val, p.out_dtype, ro * K + k, logp);
    if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * K + k] = col;
    else reinterpret_cast<int64_t*>(p.out_idx)[ro * K + k] = col;
  }
}

template <class Tag>
static int launch_producer(const ProducerParams& p, hipStream_t st) {
  const int64_t nch = p.V / Tag::epc;
  const dim3 grid((unsigned)p.n_out);
  if (nch <= 256 * 16) hipLaunchKernelGGL((topk_producer_kernel<Tag, 256, 16>), grid, dim3(256), 0, st, p);
  else if (nch <= 1024 * 16) hipLaunchKernelGGL((topk_producer_kernel<Tag, 1024, 16>), grid, dim3(1024), 0, st, p);
  else return DL_ERR_LIMIT;
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

}  // namespace dl

extern "C" int dl_teacher_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                               const int32_t* row_list, int64_t n_out, int K, void* out_val, int out_dtype,
                               void* out_idx, int out_itype, void* stream) {
  using namespace dl;
  if (!logits || !out_val || !out_idx) return DL_ERR_NULL;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || (out_dtype != DL_F32 && out_dtype != DL_F16) ||
      (out_itype != DL_I32 && out_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || n_out < 0 || V <= 0 || K <= 0 || K > V || row_stride < V || (!row_list && n_out > n_rows))
    return DL_ERR_SHAPE;
  if (K > PROD_MAX_K || V > 0x7fffffffLL || n_out > 0x7fffffffLL) return DL_ERR_LIMIT;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (V % (16 / eb) != 0 || reinterpret_cast<uintptr_t>(logits) % 16 != 0 || (row_stride * eb) % 16 != 0)
    return DL_ERR_ALIGN;
  if (n_out == 0) return DL_OK;
  ProducerParams p{logits, row_stride, V, row_list, n_out, K, out_val, out_dtype, out_idx, out_itype};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  return logits_dtype == DL_F32 ? launch_producer<TagF32>(p, st)
         : logits_dtype == DL_BF16 ? launch_producer<TagBF16>(p, st)
                                   : launch_producer<TagF16>(p, st);
}

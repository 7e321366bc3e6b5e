// Kernels and C entry point for divergences against a dense teacher stored in memory.
#include "dense_div.hpp"
#include <algorithm>

namespace dl {

struct DenseParams {
  int kind;
  const void* logits; int s_dtype; int64_t row_stride; int64_t n_rows; int64_t V;
  const int32_t* row_map;
  const void* t_logits; int t_dtype; int64_t t_stride; int64_t n_trows;
  float inv_T_s, inv_T_t, grad_scale;
  float* row_loss; void* grad; int64_t grad_stride;
};

// Both rows in registers: NU units of 8 columns per thread.  ANY: rows of V columns that may start
// anywhere and end inside a unit (unaligned 16-byte accesses; columns beyond the row read as -inf, which
// adds nothing to any statistic, and are not stored).
// BLOCKED (two fp32 rows on the grid): which 8 columns make up a unit is free as long as student, teacher and
// gradient agree, and nothing but the loads and stores ever asks.  A unit of 8 consecutive fp32 columns is two
// chunks side by side, so that a wave's load instruction touches every other 16 bytes: half of each line, and the
// next instruction the other half.  Instead the 128 chunks of 64 consecutive units (one wave's worth) are dealt
// chunk c to lane c % 64, first and second chunk of a unit 64 chunks apart (n apart in a last block of n < 64
// units): every load and store instruction of a wave then covers 1 KiB in one piece.
template <class TagS, class TagT, int NT, int NU, bool ANY = false>
struct RegRows {
  static constexpr bool ONLINE = false;      // sweeps cost no memory traffic: maxima first, then sums
  static constexpr bool BLOCKED = !ANY && TagS::bytes == 4 && TagT::bytes == 4;
  Unit<TagS> s[NU];
  Unit<TagT> t[NU];
  int64_t nunits;
  int64_t V;
  // byte offset of chunk k of unit u in a BLOCKED row
  __device__ __forceinline__ int64_t blocked_at(int64_t u, int k) const {
    const int64_t b = u >> 6;
    const int64_t nb = min((int64_t)64, nunits - (b << 6));
    return ((b << 7) + k * nb + (u & 63)) * 16;
  }
  __device__ __forceinline__ void load(const char* srow, const char* trow, int64_t nu, int64_t n_cols = 0) {
    nunits = nu;
    V = n_cols;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (u < nunits) {
        if constexpr (ANY) { s[i].load_any(srow, u, V); t[i].load_any(trow, u, V); }
        else if constexpr (BLOCKED) {
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const int64_t at = blocked_at(u, k);
            s[i].c[k] = load16_stream(srow + at);
            t[i].c[k] = load16_stream(trow + at);
          }
        }
        else { s[i].load(srow, u); t[i].load(trow, u); }
      } else {
        s[i].fill_neg_inf(); t[i].fill_neg_inf();
      }
    }
  }
  __device__ __forceinline__ void store(char* grow, int64_t u, const float* g) const {
    if constexpr (ANY) Unit<TagS>::store_any(grow, u, V, g);
    else if constexpr (BLOCKED) {
#pragma unroll
      for (int k = 0; k < 2; ++k) store16_stream(grow + blocked_at(u, k), Chunk<TagS>::pack(g + k * 4));
    }
    else Unit<TagS>::store(grow, u, g);
  }
  template <class F>
  __device__ __forceinline__ void sweep(F f) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (u < nunits) {
        float a[8], b[8];
        s[i].unpack(a);
        t[i].unpack(b);
        f(u, a, b);
      }
    }
  }
  // The same, and what f leaves in its arguments goes back into the registers (fp32 rows: bit moves).
  // The branch is per wave, not per lane (lanes beyond the row hold -inf, which f must take): a value
  // rewritten under a per-lane branch would get a second register beside the one that the idle lanes keep.
  static constexpr bool EXACT_STASH = TagS::bytes == 4 && TagT::bytes == 4;
  template <class F>
  __device__ __forceinline__ void sweep_rewrite(F f) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (__builtin_amdgcn_readfirstlane((int)((u & ~(int64_t)63) < nunits))) {
        float a[8], b[8];
        s[i].unpack(a);
        t[i].unpack(b);
        f(u, a, b);
        s[i].repack(a);
        t[i].repack(b);
      }
    }
  }
  // Maxima of both rows from the raw bit patterns, for two 16-bit rows: non-negative 16-bit floats
  // order like their patterns read as signed integers and every negative one reads as a negative
  // integer, so the packed integer maximum is the row's maximum whenever that is not negative (half
  // an instruction per element instead of two).  False -- for every thread alike -- when a row's
  // maximum is negative or the types are not 16-bit: the caller then takes the maxima from the values.
  static constexpr bool RAW_MAXIMA = TagS::bytes == 2 && TagT::bytes == 2;
  __device__ __forceinline__ bool raw_maxima(float& ms, float& mt, float* red) {
    if constexpr (!RAW_MAXIMA) return false;
    typedef short i16x2 __attribute__((ext_vector_type(2)));
    i16x2 a = {(short)-32768, (short)-32768}, b = a;
#pragma unroll
    for (int i = 0; i < NU; ++i) {      // units beyond the row hold -inf: negative patterns
      forget(s[i].c[0]);
      forget(t[i].c[0]);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned ws = s[i].c[0][d], wt = t[i].c[0][d];      // by value: a bit cast straight from a vector element reads element 0
        a = __builtin_elementwise_max(a, __builtin_bit_cast(i16x2, ws));
        b = __builtin_elementwise_max(b, __builtin_bit_cast(i16x2, wt));
      }
    }
    float fa = (float)max((int)a.x, (int)a.y), fb = (float)max((int)b.x, (int)b.y);      // exact, order-preserving
    block_max2<NT>(fa, fb, red);
    if (fa < 0.f || fb < 0.f) return false;
    const auto value = [](int id, unsigned bits) {
      return id == BF16 ? __uint_as_float(bits << 16) : (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
    };
    ms = value(TagS::id, (unsigned)(int)fa);
    mt = value(TagT::id, (unsigned)(int)fb);
    return true;
  }
};

template <int KIND, class TagS, class TagT, int NT, int NU, bool ANY = false>
__global__ __launch_bounds__(NT) void dense_reg_kernel(const DenseParams p) {
  __shared__ float red[64];
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * TagS::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  const int64_t nunits = ANY ? (p.V + 7) / 8 : p.V / 8;
  if (trow < 0) {
    if (grow) {
      if constexpr (!ANY) {
        zero_row<TagS, NT>(grow, p.V / TagS::epc);
      } else {
        const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int64_t u = tid; u < nunits; u += NT) Unit<TagS>::store_any(grow, u, p.V, z);
      }
    }
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  RegRows<TagS, TagT, NT, NU, ANY> rows;
  rows.load(reinterpret_cast<const char*>(p.logits) + r * p.row_stride * TagS::bytes,
            reinterpret_cast<const char*>(p.t_logits) + trow * p.t_stride * TagT::bytes, nunits, p.V);
  if constexpr (KIND == DL_JSD && RegRows<TagS, TagT, NT, NU, ANY>::EXACT_STASH) {
    // The divergence sweep leaves the gradient's ingredients in the rows' registers (at no cost for fp32
    // rows, so also when no gradient is asked for: a second copy of the sweeps for that case costs registers).
    const DenseStats st = dense_stats<KIND, NT, true>(rows, p.inv_T_s, p.inv_T_t, red);
    if (tid == 0 && p.row_loss) p.row_loss[r] = st.loss;
    if (grow) dense_jsd_grad_from_stash<TagS>(rows, st, p.inv_T_s * p.grad_scale, grow);
  } else {
    const DenseStats st = dense_stats<KIND, NT>(rows, p.inv_T_s, p.inv_T_t, red);
    if (tid == 0 && p.row_loss) p.row_loss[r] = st.loss;
    if (grow) dense_grad_sweep<KIND, TagS>(rows, st, p.inv_T_s * p.grad_scale, grow);
  }
}

// ---------------------------------------------------------------------------------------
// Forward / reverse KL on rows cut into column parts.  A workgroup that holds a whole pair of rows is
// 512 or 1024 threads wide, so one or two of them fill a CU and nothing overlaps their load,
// arithmetic and store phases.  Here a row pair is cut into P <= 8 parts of 256 (or 512) threads x NU units
// instead; four (two) parts of different rows share a CU and hide each other's phases, and each part still
// reads its columns once.  The parts of a row exchange (maxima, sums of exponentials, divergence sum on the part's
// own biases) through a 32-byte record per part in a caller-provided workspace: relaxed device-scope stores
// and loads, validated by a tag over the five words; the wait is bounded, and a part that gives up -- it has
// written nothing yet, also when the gradient goes over the logits -- puts itself on a list that a second
// launch finishes from the then complete records.  Every part combines the records in part order: all parts
// of a row arrive at the same bits, and so does the second launch.  Parts of a row sit 8 workgroup ids
// apart, i.e. on one XCD back to back.  JSD is not cut: its divergence needs the row's normalisers inside a
// logarithm, which would take a second exchange.
// ---------------------------------------------------------------------------------------
struct DenseRecord { unsigned ms, mt, ss, st, w, tag, pad0, pad1; };
constexpr int DENSE_MAX_PARTS = 8;
constexpr int DENSE_SPIN_LIMIT = 20000;

struct DenseSplit {
  DenseRecord* records;      // n_rows * parts
  unsigned* retry_count;     // then a counter (16 bytes) and n_rows * parts list slots
  unsigned* retry_list;
  int parts;
  int spin_limit;
  int64_t part_units;        // units of 8 columns per part (the last part takes what is left)
  __host__ __device__ static int64_t bytes(int64_t n_rows, int parts) { return n_rows * parts * (int64_t)(sizeof(DenseRecord) + 4) + 16; }
  // The row is cut evenly, in whole waves of units: a last part that holds a few columns would still take a
  // workgroup, and its partners would wait for it like for a full one.
  __host__ DenseSplit(void* ws, int64_t n_rows, int parts_, int spin, int64_t units, int64_t most_units) {
    part_units = ((units + parts_ - 1) / parts_ + 63) / 64 * 64;
    if (part_units > most_units || (parts_ - 1) * part_units >= units) part_units = most_units;
    records = reinterpret_cast<DenseRecord*>(ws);
    char* base = reinterpret_cast<char*>(ws) + n_rows * parts_ * (int64_t)sizeof(DenseRecord);
    retry_count = reinterpret_cast<unsigned*>(base);
    retry_list = reinterpret_cast<unsigned*>(base + 16);
    parts = parts_;
    spin_limit = spin;
  }
};

__device__ __forceinline__ unsigned dense_record_tag(unsigned a, unsigned b, unsigned c, unsigned d, unsigned e) {
  return a ^ ((b << 5) | (b >> 27)) ^ ((c << 11) | (c >> 21)) ^ ((d << 17) | (d >> 15)) ^ ((e << 23) | (e >> 9)) ^ 0x5eed4321u;
}
__device__ __forceinline__ void dense_record_publish(DenseRecord* w, float ms, float mt, float ss, float st, float wv) {
  const unsigned a = __float_as_uint(ms), b = __float_as_uint(mt), c = __float_as_uint(ss), d = __float_as_uint(st),
                 e = __float_as_uint(wv);
  __hip_atomic_store(&w->ms, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->mt, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->ss, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->st, d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->w, e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&w->tag, dense_record_tag(a, b, c, d, e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Bounded wait for a partner's record; false = gave up after `limit` polls.  A cleared record is invalid.
__device__ __forceinline__ bool dense_record_collect(DenseRecord* w, int limit, float* out) {
  for (int spins = 0; spins < limit; ++spins) {
    const unsigned a = __hip_atomic_load(&w->ms, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned b = __hip_atomic_load(&w->mt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned c = __hip_atomic_load(&w->ss, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned d = __hip_atomic_load(&w->st, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned e = __hip_atomic_load(&w->w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned t = __hip_atomic_load(&w->tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t == dense_record_tag(a, b, c, d, e)) {
      out[0] = __uint_as_float(a); out[1] = __uint_as_float(b); out[2] = __uint_as_float(c);
      out[3] = __uint_as_float(d); out[4] = __uint_as_float(e);
      return true;
    }
    __builtin_amdgcn_s_sleep(4);
  }
  return false;
}

template <int KIND, class TagS, class TagT, int NT, int NU, bool RETRY>
__device__ __forceinline__ void dense_split_part(const DenseParams& p, const DenseSplit& x, int64_t r, int h, float* red,
                                                 float (*xch)[DENSE_MAX_PARTS], int* xok) {
  static_assert(KIND == DL_FKL || KIND == DL_RKL, "JSD rows are not cut into parts");
  const int tid = threadIdx.x;
  const int P = x.parts;
  const int64_t u0 = (int64_t)h * x.part_units;                        // first unit of this part
  const int64_t nu = min(x.part_units, p.V / 8 - u0);                   // its units
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + (r * p.grad_stride + u0 * 8) * TagS::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (grow) zero_row<TagS, NT>(grow, nu * 8 / TagS::epc);
    if (tid == 0 && h == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  using Rows = RegRows<TagS, TagT, NT, NU>;
  Rows rows;
  rows.load(reinterpret_cast<const char*>(p.logits) + (r * p.row_stride + u0 * 8) * TagS::bytes,
            reinterpret_cast<const char*>(p.t_logits) + (trow * p.t_stride + u0 * 8) * TagT::bytes, nu);
  const float a_s = p.inv_T_s * LOG2E, a_t = p.inv_T_t * LOG2E;
  float ms = -INFINITY, mt = -INFINITY;
  bool have = false;
  if constexpr (KIND != DL_RKL && Rows::RAW_MAXIMA) have = rows.raw_maxima(ms, mt, red);
  if (!have) {
    rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        mt = fmaxf(mt, t[e]);
        ms = fmaxf(ms, (KIND == DL_RKL && t[e] == -INFINITY) ? -INFINITY : s[e]);
      }
    });
    block_max2<NT>(ms, mt, red);
  }
  // a part that holds no finite logit (a masked stretch of the vocabulary): bias 0 keeps 2^(-inf - bias) = 0
  const float bs = ms == -INFINITY ? 0.f : ms * a_s, bt = mt == -INFINITY ? 0.f : mt * a_t;
  float ss = 0.f, stt = 0.f, w = 0.f;
  rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xs = fmaf(s[e], a_s, -bs), xt = fmaf(t[e], a_t, -bt);
      const float es = fast_exp2(xs), et = fast_exp2(xt);
      stt += et;
      if (KIND == DL_RKL) {
        const bool on = t[e] != -INFINITY;
        ss += on ? es : 0.f;
        w += (on && es > 0.f) ? es * (xs - xt) : 0.f;
      } else {
        ss += es;
        w += et > 0.f ? et * (xt - xs) : 0.f;
      }
    }
  });
  block_sum3<NT>(ss, stt, w, red);

  DenseRecord* ws = x.records + r * P;
  if (tid == 0 && !RETRY) dense_record_publish(ws + h, ms, mt, ss, stt, w);
  if (tid < P) {
    float rec[5] = {ms, mt, ss, stt, w};
    const int ok = (tid == h) || dense_record_collect(ws + tid, RETRY ? 0x7fffffff : x.spin_limit, rec);
#pragma unroll
    for (int k = 0; k < 5; ++k) xch[k][tid] = rec[k];
    xok[tid] = ok;
  }
  __syncthreads();
  bool all_ok = true;
  for (int j = 0; j < P; ++j) all_ok = all_ok && (xok[j] != 0);
  if (!all_ok) {
    if (tid == 0) x.retry_list[atomicAdd(x.retry_count, 1u)] = (unsigned)(r * P + h);
    return;
  }
  // the row's statistics from the parts', in part order (the same bits in every part)
  float Ms = xch[0][0], Mt = xch[1][0];
  for (int j = 1; j < P; ++j) { Ms = fmaxf(Ms, xch[0][j]); Mt = fmaxf(Mt, xch[1][j]); }
  float S = 0.f, T = 0.f, W = 0.f;
  for (int j = 0; j < P; ++j) {
    const float pms = xch[0][j], pmt = xch[1][j], pss = xch[2][j], pst = xch[3][j], pw = xch[4][j];
    // shifts of the part's biases to the row's (log2 domain, >= 0); a part without a finite maximum summed nothing on that side
    const float ds = pms == -INFINITY ? 0.f : (Ms - pms) * a_s, dt = pmt == -INFINITY ? 0.f : (Mt - pmt) * a_t;
    const float fs = fast_exp2(-ds), ft = fast_exp2(-dt);
    if (KIND == DL_FKL) W += ft * (pw - (dt - ds) * pst);
    else W += fs * (pw - (ds - dt) * pss);
    S += pss * fs;
    T += pst * ft;
  }
  DenseStats st;
  st.a_s = a_s; st.a_t = a_t;
  const float l2s = fast_log2(S), l2t = fast_log2(T);
  st.ls = (Ms == -INFINITY ? 0.f : Ms * a_s) + l2s;
  st.lt = (Mt == -INFINITY ? 0.f : Mt * a_t) + l2t;
  st.loss = (KIND == DL_FKL ? W / T - l2t + l2s : W / S - l2s + l2t) * LN2;
  st.aux = st.loss;
  st.tmax = Mt;
  if (tid == 0 && h == 0 && p.row_loss) p.row_loss[r] = st.loss;
  if (grow) dense_grad_sweep<KIND, TagS>(rows, st, p.inv_T_s * p.grad_scale, grow);
}

template <int KIND, class TagS, class TagT, int NT, int NU>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void dense_split_kernel(const DenseParams p, const DenseSplit x) {
  __shared__ float red[64];
  __shared__ float xch[5][DENSE_MAX_PARTS];
  __shared__ int xok[DENSE_MAX_PARTS];
  const unsigned P = (unsigned)x.parts;
  const unsigned grp = blockIdx.x / (8u * P), t_in = blockIdx.x % (8u * P);
  const int64_t r = (int64_t)grp * 8 + (t_in & 7u);
  if (r >= p.n_rows) return;
  dense_split_part<KIND, TagS, TagT, NT, NU, false>(p, x, r, (int)(t_in >> 3), red, xch, xok);
}

// One listed part, as a real call: the loop around it then costs the body no registers.
template <int KIND, class TagS, class TagT, int NT, int NU>
__device__ __attribute__((noinline)) void dense_split_part_again(const DenseParams& p, const DenseSplit& x, unsigned at, float* red,
                                                                 float (*xch)[DENSE_MAX_PARTS], int* xok) {
  dense_split_part<KIND, TagS, TagT, NT, NU, true>(p, x, (int64_t)(at / (unsigned)x.parts), (int)(at % (unsigned)x.parts), red, xch, xok);
}

// The parts that gave up waiting, a fixed grid striding over their list (normally empty).
template <int KIND, class TagS, class TagT, int NT, int NU>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 8)))
void dense_split_retry_kernel(const DenseParams p, const DenseSplit x) {
  __shared__ float red[64];
  __shared__ float xch[5][DENSE_MAX_PARTS];
  __shared__ int xok[DENSE_MAX_PARTS];
  const unsigned n = *x.retry_count;
#pragma unroll 1
  for (unsigned e = blockIdx.x; e < n; e += gridDim.x) {
    dense_split_part_again<KIND, TagS, TagT, NT, NU>(p, x, x.retry_list[e], red, xch, xok);
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void dense_clear_kernel(u32x4* ws, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) ws[i] = u32x4{0u, 0u, 0u, 0u};
}

// Units per thread of the split kernels for a dtype pair (0: the pair has no register kernel).
static int dense_split_units(int s_dtype, int t_dtype) {
  if (s_dtype == t_dtype) return s_dtype == F32 ? 4 : 8;
  return t_dtype == F32 ? 6 : s_dtype == F32 ? 4 : 0;
}
// How a row of V columns is cut: threads per part and parts (parts == 0: not cut).  Measured (forward KL, 512 and
// 8192 rows, 32000 to 262144 columns, fp32 pairs, 16-bit pairs and a 16-bit student against an fp32 teacher):
//   * a row that half a workgroup's registers hold (512 threads) stays whole;
//   * with a 16-bit student up to four parts of 256 threads beat half as many of 512 (more workgroups per CU to
//     hide the exchange behind), beyond that the partners to wait for cost more than they bring: parts of 512
//     threads, at most 8; fp32 students (a part of 256 threads holds 8192 columns only) take parts of 512 from the start;
//   * wider still, pairs with an fp32 row take parts of 1024 threads (beyond 8 of those, and beyond 262144
//     columns of a 16-bit pair, one workgroup per row streams the row from the caches);
//   * on fewer than 1024 rows the cut pays only from 256 KiB of row pair upwards (one workgroup per row keeps
//     the CUs busy by itself below that, and has no partners to wait for).
// `forced_nt` (256 / 512 / 1024, a tuning hook) fixes the thread count and cuts wherever two parts or more come out.
struct DenseCut { int nt, parts; };
static DenseCut dense_split_cut(int kind, int s_dtype, int t_dtype, int64_t n_rows, int64_t V, int forced_nt = 0) {
  const int nu = dense_split_units(s_dtype, t_dtype);
  if (kind == DL_JSD || nu == 0 || V % 8 != 0) return {0, 0};
  const int64_t units = V / 8;
  const auto parts_of = [&](int nt) { return (units + (int64_t)nt * nu - 1) / ((int64_t)nt * nu); };
  const auto cut_of = [&](int nt) {
    const int64_t parts = parts_of(nt);
    return parts >= 2 && parts <= DENSE_MAX_PARTS && (nt != 1024 || t_dtype == F32 || s_dtype == F32) ? DenseCut{nt, (int)parts} : DenseCut{0, 0};
  };
  if (forced_nt) return cut_of(forced_nt);
  if (parts_of(512) < 2) return {0, 0};
  const int64_t pair_bytes = V * ((s_dtype == F32 ? 4 : 2) + (t_dtype == F32 ? 4 : 2));
  if (n_rows < 1024 && pair_bytes < 256 * 1024) return {0, 0};
  if (parts_of(256) <= 4 && s_dtype != F32) return cut_of(256);      // (fp32 students: 8192 columns per such part only)
  if (parts_of(512) <= DENSE_MAX_PARTS) return cut_of(512);
  return cut_of(1024);
}

template <int KIND, class TagS, class TagT, int NT, int NU>
static void launch_dense_split_kind(const DenseParams& p, const DenseSplit& x, hipStream_t st) {
  const int64_t n16 = p.n_rows * x.parts * 2 + 1;      // records, then the retry counter
  hipLaunchKernelGGL(dense_clear_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, st,
                     reinterpret_cast<u32x4*>(x.records), n16);
  hipLaunchKernelGGL((dense_split_kernel<KIND, TagS, TagT, NT, NU>), dim3((unsigned)((p.n_rows + 7) / 8 * 8 * x.parts)),
                     dim3(NT), 0, st, p, x);
  hipLaunchKernelGGL((dense_split_retry_kernel<KIND, TagS, TagT, NT, NU>),
                     dim3((unsigned)std::min<int64_t>(p.n_rows * x.parts, 256)), dim3(NT), 0, st, p, x);
}
template <class TagS, class TagT, int NU>
static void launch_dense_split(const DenseParams& p, const DenseSplit& x, int nt, hipStream_t st) {
  if (nt == 256) {
    if (p.kind == DL_FKL) launch_dense_split_kind<DL_FKL, TagS, TagT, 256, NU>(p, x, st);
    else launch_dense_split_kind<DL_RKL, TagS, TagT, 256, NU>(p, x, st);
  } else if (nt == 1024) {
    if constexpr (TagT::bytes == 4 || TagS::bytes == 4) {      // 16-bit pairs reach 262144 columns with parts of 512 threads
      if (p.kind == DL_FKL) launch_dense_split_kind<DL_FKL, TagS, TagT, 1024, NU>(p, x, st);
      else launch_dense_split_kind<DL_RKL, TagS, TagT, 1024, NU>(p, x, st);
    }
  } else {
    if (p.kind == DL_FKL) launch_dense_split_kind<DL_FKL, TagS, TagT, 512, NU>(p, x, st);
    else launch_dense_split_kind<DL_RKL, TagS, TagT, 512, NU>(p, x, st);
  }
}
static void launch_dense_split_pair(const DenseParams& p, const DenseSplit& x, int nt, hipStream_t st) {
  if (p.s_dtype == F32 && p.t_dtype == F32) launch_dense_split<TagF32, TagF32, 4>(p, x, nt, st);
  else if (p.s_dtype == BF16 && p.t_dtype == BF16) launch_dense_split<TagBF16, TagBF16, 8>(p, x, nt, st);
  else if (p.s_dtype == F16 && p.t_dtype == F16) launch_dense_split<TagF16, TagF16, 8>(p, x, nt, st);
  else if (p.s_dtype == BF16 && p.t_dtype == F32) launch_dense_split<TagBF16, TagF32, 6>(p, x, nt, st);
  else if (p.s_dtype == F16 && p.t_dtype == F32) launch_dense_split<TagF16, TagF32, 6>(p, x, nt, st);
  else if (p.s_dtype == F32 && p.t_dtype == BF16) launch_dense_split<TagF32, TagBF16, 4>(p, x, nt, st);
  else launch_dense_split<TagF32, TagF16, 4>(p, x, nt, st);
}

// Rows too wide for the registers, 16-byte aligned: the same sweeps, every one of them over global
// memory with 16-byte loads, two units per thread in flight (2-3 reads of both rows; all but the first
// come from L2 / the memory-side cache as far as the rows of the workgroups in flight fit there).
template <class TagS, class TagT, int NT>
struct StreamRows {
  static constexpr bool ONLINE = true;       // every sweep reads both rows: maxima and sums share one
  const char* srow;
  const char* trow;
  int64_t nunits;
  __device__ __forceinline__ void store(char* grow, int64_t u, const float* g) const { Unit<TagS>::store(grow, u, g); }
  template <class Tag>
  static __device__ __forceinline__ void fetch(Unit<Tag>& x, const char* row, int64_t u) {
#pragma unroll
    for (int k = 0; k < Unit<Tag>::NC; ++k) x.c[k] = *reinterpret_cast<const u32x4*>(row + (u * Unit<Tag>::NC + k) * 16);
  }
  template <class F>
  __device__ __forceinline__ void sweep(F f) {
    constexpr int U = 2;
    for (int64_t u0 = threadIdx.x; u0 < nunits; u0 += (int64_t)U * NT) {
      Unit<TagS> s[U];
      Unit<TagT> t[U];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const int64_t u = u0 + (int64_t)j * NT;
        if (u < nunits) { fetch(s[j], srow, u); fetch(t[j], trow, u); }
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const int64_t u = u0 + (int64_t)j * NT;
        if (u < nunits) {
          float a[8], b[8];
          s[j].unpack(a);
          t[j].unpack(b);
          f(u, a, b);
        }
      }
    }
  }
};

template <int KIND, class TagS, class TagT, int NT>
__global__ __launch_bounds__(NT) void dense_stream_vec_kernel(const DenseParams p) {
  __shared__ float red[64];
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * TagS::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (grow) zero_row<TagS, NT>(grow, p.V / TagS::epc);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  StreamRows<TagS, TagT, NT> rows{reinterpret_cast<const char*>(p.logits) + r * p.row_stride * TagS::bytes,
                                  reinterpret_cast<const char*>(p.t_logits) + trow * p.t_stride * TagT::bytes, p.V / 8};
  const DenseStats st = dense_stats<KIND, NT>(rows, p.inv_T_s, p.inv_T_t, red);
  if (tid == 0 && p.row_loss) p.row_loss[r] = st.loss;
  if (grow) dense_grad_sweep<KIND, TagS>(rows, st, p.inv_T_s * p.grad_scale, grow);
}

// Rows too wide for both to sit in registers, but not for the student's alone: the student row is
// read from HBM once and kept on the CU, half of it in registers (NUS / 2 units per thread) and half
// in LDS (128 KiB; all of it in registers leaves too few for the sweeps: the compiler spills).  The
// teacher row is streamed through a ring of D units per thread in every sweep (its later reads come
// from L2 as far as the rows in flight fit there).  Against streaming both rows this saves one or
// two reads of the student row.
template <class TagS, class TagT, int NT, int NUS>
struct StudentRegRows {
  static constexpr bool ONLINE = true;       // every sweep reads the teacher row: maxima and sums share one
  static constexpr int D = Unit<TagT>::NC == 1 ? 4 : 2;      // teacher units in flight per thread
  static constexpr int NR = NUS / 2;                         // student units in registers; the rest in LDS
  static constexpr int NC = Unit<TagS>::NC;
  static constexpr size_t LDS_BYTES = (size_t)(NUS - NR) * NC * NT * 16;
  Unit<TagS> s[NR];
  u32x4* lds;
  const char* trow;
  int64_t nunits;
  __device__ __forceinline__ void store(char* grow, int64_t u, const float* g) const { Unit<TagS>::store(grow, u, g); }
  __device__ __forceinline__ void load(const char* srow, const char* trow_, int64_t nu, u32x4* lds_) {
    trow = trow_;
    nunits = nu;
    lds = lds_;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (u < nunits) s[i].load(srow, u);
      else s[i].fill_neg_inf();
    }
#pragma unroll
    for (int i = NR; i < NUS; ++i) {         // every thread reads back only what it wrote: no barrier needed
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      Unit<TagS> x;
      if (u < nunits) x.load(srow, u);
      else x.fill_neg_inf();
#pragma unroll
      for (int k = 0; k < NC; ++k) lds[((i - NR) * NC + k) * NT + threadIdx.x] = x.c[k];
    }
  }
  template <class F>
  __device__ __forceinline__ void sweep(F f) {
    Unit<TagT> t[D];
#pragma unroll
    for (int d = 0; d < D && d < NUS; ++d) {
      const int64_t u = (int64_t)d * NT + threadIdx.x;
      if (u < nunits) StreamRows<TagS, TagT, NT>::fetch(t[d], trow, u);
    }
#pragma unroll
    for (int i = 0; i < NUS; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (u < nunits) {
        float a[8], b[8];
        if (i < NR) {
          s[i].unpack(a);
        } else {
          Unit<TagS> x;
#pragma unroll
          for (int k = 0; k < NC; ++k) x.c[k] = lds[((i - NR) * NC + k) * NT + threadIdx.x];
          x.unpack(a);
        }
        t[i % D].unpack(b);
        f(u, a, b);
      }
      if (i + D < NUS) {                     // refill the slot just used
        const int64_t un = (int64_t)(i + D) * NT + threadIdx.x;
        if (un < nunits) StreamRows<TagS, TagT, NT>::fetch(t[i % D], trow, un);
      }
      // no memory access moves across this point: without it the compiler issues the loads of all
      // units up front and spills the registers that hold them
      asm volatile("" ::: "memory");
    }
  }
};

template <int KIND, class TagS, class TagT, int NT, int NUS>
__global__ __launch_bounds__(NT) void dense_student_reg_kernel(const DenseParams p) {
  extern __shared__ __align__(16) u32x4 student_half[];
  __shared__ float red[64];
  const int64_t r = xcd_banded_row(blockIdx.x);
  if (r >= p.n_rows) return;
  const int tid = threadIdx.x;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * TagS::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (grow) zero_row<TagS, NT>(grow, p.V / TagS::epc);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  StudentRegRows<TagS, TagT, NT, NUS> rows;
  rows.load(reinterpret_cast<const char*>(p.logits) + r * p.row_stride * TagS::bytes,
            reinterpret_cast<const char*>(p.t_logits) + trow * p.t_stride * TagT::bytes, p.V / 8, student_half);
  const DenseStats st = dense_stats<KIND, NT>(rows, p.inv_T_s, p.inv_T_t, red);
  if (tid == 0 && p.row_loss) p.row_loss[r] = st.loss;
  if (grow) dense_grad_sweep<KIND, TagS>(rows, st, p.inv_T_s * p.grad_scale, grow);
}

// Any size, any alignment, any dtype pair: four scalar passes over global memory.
template <int NT>
__global__ __launch_bounds__(NT) void dense_stream_kernel(const DenseParams p) {
  __shared__ float red[64];
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t V = p.V;
  const int sb = p.s_dtype == F32 ? 4 : 2, tb = p.t_dtype == F32 ? 4 : 2;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * sb : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (grow) for (int64_t j = tid; j < V; j += NT) store_from_float(grow, p.s_dtype, j, 0.f);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  const char* srow = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * sb;
  const char* trw = reinterpret_cast<const char*>(p.t_logits) + trow * p.t_stride * tb;
  const int kind = p.kind;
  const float a_s = p.inv_T_s * LOG2E, a_t = p.inv_T_t * LOG2E;
  float ms = -INFINITY, mt = -INFINITY;
  for (int64_t j = tid; j < V; j += NT) {
    const float s = load_as_float(srow, p.s_dtype, j), t = load_as_float(trw, p.t_dtype, j);
    mt = fmaxf(mt, t);
    ms = fmaxf(ms, (kind == DL_RKL && t == -INFINITY) ? -INFINITY : s);
  }
  block_max2<NT>(ms, mt, red);
  const float bs = ms * a_s, bt = mt * a_t;
  float ss = 0.f, stt = 0.f;
  for (int64_t j = tid; j < V; j += NT) {
    const float s = load_as_float(srow, p.s_dtype, j), t = load_as_float(trw, p.t_dtype, j);
    ss += (kind == DL_RKL && t == -INFINITY) ? 0.f : fast_exp2(fmaf(s, a_s, -bs));
    stt += fast_exp2(fmaf(t, a_t, -bt));
  }
  block_sum2<NT>(ss, stt, red);
  const float ls = bs + fast_log2(ss), lt = bt + fast_log2(stt);
  float x = 0.f, y = 0.f;
  for (int64_t j = tid; j < V; j += NT) {
    const float lp = fmaf(load_as_float(srow, p.s_dtype, j), a_s, -ls);
    const float lq = fmaf(load_as_float(trw, p.t_dtype, j), a_t, -lt);
    if (kind == DL_FKL) fkl_term(lp, lq, x);
    else if (kind == DL_RKL) rkl_term(lp, lq, x);
    else jsd_term(lp, lq, x, y);
  }
  block_sum2<NT>(x, y, red);
  const float loss = kind == DL_JSD ? 0.5f * LN2 * (x + y) : x * LN2;
  const float aux = x * LN2;
  if (tid == 0 && p.row_loss) p.row_loss[r] = loss;
  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
    for (int64_t j = tid; j < V; j += NT) {
      const float lp = fmaf(load_as_float(srow, p.s_dtype, j), a_s, -ls);
      const float lq = fmaf(load_as_float(trw, p.t_dtype, j), a_t, -lt);
      store_from_float(grow, p.s_dtype, j, dense_grad(kind, lp, lq, aux) * c);
    }
  }
}

template <int KIND, class TagS, class TagT, int NU>
static bool launch_dense_kind(const DenseParams& p, hipStream_t st) {
  const int64_t units = p.V / 8;
  constexpr int NUS = 256 / (16 * Unit<TagS>::NC);      // the student row alone: 256 bytes of registers per thread
  const dim3 grid(xcd_banded_grid(p.n_rows));
  if (units <= 256 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, TagS, TagT, 256, NU>), grid, dim3(256), 0, st, p);
  else if (units <= 512 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, TagS, TagT, 512, NU>), grid, dim3(512), 0, st, p);
  else if (units <= 1024 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, TagS, TagT, 1024, NU>), grid, dim3(1024), 0, st, p);
  else if (units <= 1024 * NUS) {
    // more than 64 KiB of dynamic LDS has to be requested per kernel, once per device (the call is slow)
    constexpr size_t lds = StudentRegRows<TagS, TagT, 1024, NUS>::LDS_BYTES;
    static thread_local int allowed_on = -1;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (allowed_on != dev) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&dense_student_reg_kernel<KIND, TagS, TagT, 1024, NUS>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return false;
      allowed_on = dev;
    }
    hipLaunchKernelGGL((dense_student_reg_kernel<KIND, TagS, TagT, 1024, NUS>), grid, dim3(1024), lds, st, p);
  }
  else hipLaunchKernelGGL((dense_stream_vec_kernel<KIND, TagS, TagT, 1024>), grid, dim3(1024), 0, st, p);
  return true;
}

// Rows off the 16-byte grid or not a whole number of units long, student and teacher of one dtype: the
// register kernel with unaligned accesses, as far as a workgroup holds the pair of rows.
template <int KIND, class Tag, int NU>
static bool launch_dense_any_kind(const DenseParams& p, hipStream_t st) {
  const int64_t units = (p.V + 7) / 8;
  const dim3 grid(xcd_banded_grid(p.n_rows));
  if (units <= 256 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, Tag, Tag, 256, NU, true>), grid, dim3(256), 0, st, p);
  else if (units <= 512 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, Tag, Tag, 512, NU, true>), grid, dim3(512), 0, st, p);
  else if (units <= 1024 * NU) hipLaunchKernelGGL((dense_reg_kernel<KIND, Tag, Tag, 1024, NU, true>), grid, dim3(1024), 0, st, p);
  else return false;
  return true;
}
template <class Tag, int NU>
static bool launch_dense_any(const DenseParams& p, hipStream_t st) {
  if (p.kind == DL_FKL) return launch_dense_any_kind<DL_FKL, Tag, NU>(p, st);
  if (p.kind == DL_RKL) return launch_dense_any_kind<DL_RKL, Tag, NU>(p, st);
  return launch_dense_any_kind<DL_JSD, Tag, NU>(p, st);
}
static bool launch_dense_any_pair(const DenseParams& p, hipStream_t st) {
  if (p.s_dtype == F32 && p.t_dtype == F32) return launch_dense_any<TagF32, 4>(p, st);
  if (p.s_dtype == BF16 && p.t_dtype == BF16) return launch_dense_any<TagBF16, 8>(p, st);
  if (p.s_dtype == F16 && p.t_dtype == F16) return launch_dense_any<TagF16, 8>(p, st);
  return false;
}

template <class TagS, class TagT, int NU>
static bool launch_dense_reg(const DenseParams& p, hipStream_t st) {
  if (p.kind == DL_FKL) return launch_dense_kind<DL_FKL, TagS, TagT, NU>(p, st);
  if (p.kind == DL_RKL) return launch_dense_kind<DL_RKL, TagS, TagT, NU>(p, st);
  return launch_dense_kind<DL_JSD, TagS, TagT, NU>(p, st);
}

// Register path for the dtype pairs that occur: teacher stored like the student, or in fp32, or a 16-bit teacher
// against a student that the caller has already cast to fp32 (as the reference does with its logits).
static bool launch_dense_pair(const DenseParams& p, hipStream_t st) {
  if (p.s_dtype == F32 && p.t_dtype == F32) return launch_dense_reg<TagF32, TagF32, 4>(p, st);
  if (p.s_dtype == BF16 && p.t_dtype == BF16) return launch_dense_reg<TagBF16, TagBF16, 8>(p, st);
  if (p.s_dtype == F16 && p.t_dtype == F16) return launch_dense_reg<TagF16, TagF16, 8>(p, st);
  if (p.s_dtype == BF16 && p.t_dtype == F32) return launch_dense_reg<TagBF16, TagF32, 4>(p, st);
  if (p.s_dtype == F16 && p.t_dtype == F32) return launch_dense_reg<TagF16, TagF32, 4>(p, st);
  if (p.s_dtype == F32 && p.t_dtype == BF16) return launch_dense_reg<TagF32, TagBF16, 4>(p, st);
  if (p.s_dtype == F32 && p.t_dtype == F16) return launch_dense_reg<TagF32, TagF16, 4>(p, st);
  return false;
}

}  // namespace dl

extern "C" int64_t dl_div_dense_workspace_bytes(int kind, int logits_dtype, int t_dtype, int64_t n_rows, int64_t V) {
  if (n_rows <= 0 || V <= 0) return 0;
  // enough for every cut the flags of dl_div_dense_ws may ask for
  int parts = 0;
  for (int nt : {0, 256, 512, 1024}) parts = std::max(parts, dl::dense_split_cut(kind, logits_dtype, t_dtype, n_rows, V, nt).parts);
  return parts ? dl::DenseSplit::bytes(n_rows, parts) : 0;
}

extern "C" int dl_div_dense(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                            int64_t V, const int32_t* row_map, const void* t_logits, int t_dtype, int64_t t_stride,
                            int64_t n_teacher_rows, float inv_T_student, float inv_T_teacher, float grad_scale,
                            float* row_loss, void* grad, int64_t grad_stride, void* stream) {
  return dl_div_dense_ws(kind, logits, logits_dtype, row_stride, n_rows, V, row_map, t_logits, t_dtype, t_stride,
                         n_teacher_rows, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride, nullptr, 0, 0,
                         stream);
}

extern "C" int dl_div_dense_ws(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                               int64_t V, const int32_t* row_map, const void* t_logits, int t_dtype, int64_t t_stride,
                               int64_t n_teacher_rows, float inv_T_student, float inv_T_teacher, float grad_scale,
                               float* row_loss, void* grad, int64_t grad_stride, void* workspace, int64_t workspace_bytes,
                               int flags, void* stream) {
  using namespace dl;
  if (!logits || (!t_logits && n_teacher_rows > 0)) return DL_ERR_NULL;      // no teacher rows: every row is masked
  if (kind < DL_FKL || kind > DL_JSD || logits_dtype < DL_F32 || logits_dtype > DL_F16 || t_dtype < DL_F32 ||
      t_dtype > DL_F16)
    return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || n_teacher_rows < 0 || row_stride < V || t_stride < V || (grad && grad_stride < V))
    return DL_ERR_SHAPE;
  if (n_rows > 0x7fffffffLL || V > 0x7fffffffLL) return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  const int sb = logits_dtype == DL_F32 ? 4 : 2, tb = t_dtype == DL_F32 ? 4 : 2;
  auto ok16 = [](const void* ptr, int64_t stride, int eb) {
    return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (stride * eb) % 16 == 0;
  };
  const bool vec = V % 8 == 0 && ok16(logits, row_stride, sb) && ok16(t_logits, t_stride, tb) &&
                   (!grad || ok16(grad, grad_stride, sb));
  DenseParams p{kind, logits, logits_dtype, row_stride, n_rows, V, row_map, t_logits, t_dtype, t_stride,
                n_teacher_rows, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool elem = reinterpret_cast<uintptr_t>(logits) % sb == 0 && reinterpret_cast<uintptr_t>(t_logits) % tb == 0 &&
                    (!grad || reinterpret_cast<uintptr_t>(grad) % sb == 0);
  if (!elem) return DL_ERR_ALIGN;
  // rows cut into column parts, where a workspace for their exchange came along
  const int hook = (flags >> DL_TOPK_PARTS_SHIFT) & 15;      // 1 / 2: parts of 256 / 512 threads wherever the row can be cut
  const DenseCut cut = vec ? dense_split_cut(kind, logits_dtype, t_dtype, n_rows, V, hook == 1 ? 256 : hook == 2 ? 512 : hook == 3 ? 1024 : 0) : DenseCut{0, 0};
  if (cut.parts && workspace && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
      workspace_bytes >= DenseSplit::bytes(n_rows, cut.parts) && n_rows * cut.parts <= 0x7fffffffLL) {
    const DenseSplit x(workspace, n_rows, cut.parts, (flags & DL_TOPK_NO_WAIT) ? 0 : DENSE_SPIN_LIMIT, V / 8,
                       (int64_t)cut.nt * dense_split_units(logits_dtype, t_dtype));
    launch_dense_split_pair(p, x, cut.nt, st);
    return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
  }
  if (!(vec ? launch_dense_pair(p, st) : launch_dense_any_pair(p, st)))
    hipLaunchKernelGGL((dense_stream_kernel<1024>), dim3((unsigned)n_rows), dim3(1024), 0, st, p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

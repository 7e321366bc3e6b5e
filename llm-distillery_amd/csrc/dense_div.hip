// Kernels and C entry point for divergences against a dense teacher stored in memory.
#include "dense_div.hpp"

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
template <class TagS, class TagT, int NT, int NU, bool ANY = false>
struct RegRows {
  static constexpr bool ONLINE = false;      // sweeps cost no memory traffic: maxima first, then sums
  Unit<TagS> s[NU];
  Unit<TagT> t[NU];
  int64_t nunits;
  int64_t V;
  __device__ __forceinline__ void load(const char* srow, const char* trow, int64_t nu, int64_t n_cols = 0) {
    nunits = nu;
    V = n_cols;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int64_t u = (int64_t)i * NT + threadIdx.x;
      if (u < nunits) {
        if constexpr (ANY) { s[i].load_any(srow, u, V); t[i].load_any(trow, u, V); }
        else { s[i].load(srow, u); t[i].load(trow, u); }
      } else {
        s[i].fill_neg_inf(); t[i].fill_neg_inf();
      }
    }
  }
  __device__ __forceinline__ void store(char* grow, int64_t u, const float* g) const {
    if constexpr (ANY) Unit<TagS>::store_any(grow, u, V, g);
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

// Register path for the dtype pairs that occur: teacher stored like the student, or in fp32.
static bool launch_dense_pair(const DenseParams& p, hipStream_t st) {
  if (p.s_dtype == F32 && p.t_dtype == F32) return launch_dense_reg<TagF32, TagF32, 4>(p, st);
  if (p.s_dtype == BF16 && p.t_dtype == BF16) return launch_dense_reg<TagBF16, TagBF16, 8>(p, st);
  if (p.s_dtype == F16 && p.t_dtype == F16) return launch_dense_reg<TagF16, TagF16, 8>(p, st);
  if (p.s_dtype == BF16 && p.t_dtype == F32) return launch_dense_reg<TagBF16, TagF32, 4>(p, st);
  if (p.s_dtype == F16 && p.t_dtype == F32) return launch_dense_reg<TagF16, TagF32, 4>(p, st);
  return false;
}

}  // namespace dl

extern "C" int dl_div_dense(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                            int64_t V, const int32_t* row_map, const void* t_logits, int t_dtype, int64_t t_stride,
                            int64_t n_teacher_rows, float inv_T_student, float inv_T_teacher, float grad_scale,
                            float* row_loss, void* grad, int64_t grad_stride, void* stream) {
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
  if (!(vec ? launch_dense_pair(p, st) : launch_dense_any_pair(p, st)))
    hipLaunchKernelGGL((dense_stream_kernel<1024>), dim3((unsigned)n_rows), dim3(1024), 0, st, p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

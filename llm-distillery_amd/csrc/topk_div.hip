// Forward / reverse KL against a sparse (top-K) teacher: loss and gradient in one sweep.
//
// One workgroup per token row.  Forward KL needs the full-vocabulary
// log-sum-exp of the student row, so the row is pulled into registers with
// 16-byte non-temporal loads (read from HBM once), reduced, and the gradient
//     d kl / d logit_j = (softmax(z)_j - sum_k q_k [j == idx_k]) * inv_T * scale
// is produced from the same registers: a dense softmax sweep, then K sparse
// corrections after a workgroup barrier.  The K teacher entries (id, log-prob,
// gathered student logit) live in LDS.
//
// Reverse KL (student renormalised over the K ids) touches only the K gathered
// logits; its gradient row is a zero fill plus K sparse values.
//
// Rows that do not fit the register file (or break the 16-byte alignment rules)
// take the streaming kernel, which reads the row twice.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

struct TopkParams {
  const void* logits; int64_t row_stride; int64_t n_rows; int64_t V;
  const int32_t* row_map;
  const void* t_val; int t_val_dtype; const void* t_idx; int t_idx_itype; int K;
  int64_t n_trows; const int32_t* t_cnt;
  float inv_T_s, inv_T_t, grad_scale;
  float* row_loss; void* grad; int64_t grad_stride;
};

// LDS carve-up shared by the kernels of this file.
struct TopkLds {
  float* red;   // 2 * (NT/64) floats, padded to 64
  int* idx;     // K   vocabulary id or -1
  float* t;     // K   scaled teacher logit -> teacher prob q_k
  float* z;     // K   gathered student logit -> student prob at the id
  __device__ TopkLds(unsigned char* base, int K) {
    red = reinterpret_cast<float*>(base);
    idx = reinterpret_cast<int*>(base + 256);
    t = reinterpret_cast<float*>(idx + K);
    z = t + K;
  }
  static size_t bytes(int K) { return 256 + (size_t)K * 12; }
};

// Stage the teacher row: ids, scaled log-probs and the student logits at those ids.
// Returns log-sum-exp of the scaled teacher entries (-inf if the row has none).
template <class Tag, int NT>
__device__ __forceinline__ float stage_teacher(const TopkParams& p, const TopkLds& s, int64_t trow,
                                               const char* row) {
  const int K = p.K;
  const int cnt = p.t_cnt ? min(p.t_cnt[trow], K) : K;
  float tmax = -INFINITY;
  for (int k = threadIdx.x; k < K; k += NT) {
    const int64_t at = trow * (int64_t)K + k;
    const int64_t id = k < cnt ? load_index(p.t_idx, p.t_idx_itype, at) : -1;
    const bool ok = id >= 0 && id < p.V;
    const float tv = ok ? load_as_float(p.t_val, p.t_val_dtype, at) * p.inv_T_t : -INFINITY;
    s.idx[k] = ok ? (int)id : -1;
    s.t[k] = tv;
    s.z[k] = ok ? load_as_float(row, Tag::id, id) : 0.f;
    tmax = fmaxf(tmax, tv);
  }
  tmax = block_max<NT>(tmax, s.red);     // barrier inside: LDS entries visible afterwards
  if (tmax == -INFINITY) return tmax;
  float part = 0.f;
  for (int k = threadIdx.x; k < K; k += NT) part += expf(s.t[k] - tmax);
  const float tsum = block_sum<NT>(part, s.red);
  return tmax + logf(tsum);
}

// Forward-KL row value; leaves q_k in s.t and the student probability at the id in s.z.
template <int NT>
__device__ __forceinline__ float fkl_from_staged(const TopkParams& p, const TopkLds& s, float tlse, float lse) {
  float part = 0.f;
  for (int k = threadIdx.x; k < p.K; k += NT) {
    if (s.idx[k] >= 0) {
      const float tk = s.t[k] - tlse;
      const float sk = s.z[k] * p.inv_T_s - lse;
      const float q = expf(tk);
      part += q * (tk - sk);
      s.t[k] = q;
      s.z[k] = expf(sk);
    } else {
      s.t[k] = 0.f;
    }
  }
  return block_sum<NT>(part, s.red);
}

// K sparse corrections of the dense softmax row already written by this workgroup.
// Ids that occur more than once receive the summed teacher mass (every duplicate
// writes the same value).
template <class Tag, int NT>
__device__ __forceinline__ void fkl_sparse_fix(const TopkParams& p, const TopkLds& s, void* grow, float c) {
  for (int k = threadIdx.x; k < p.K; k += NT) {
    const int id = s.idx[k];
    if (id < 0) continue;
    float q = 0.f;
    for (int j = 0; j < p.K; ++j) q += (s.idx[j] == id) ? s.t[j] : 0.f;
    store_from_float(grow, Tag::id, id, (s.z[k] - q) * c);
  }
}

// ---------------------------------------------------------------------------------------
// Forward KL, row resident in registers: NT threads x NCH 16-byte chunks per thread.
// ---------------------------------------------------------------------------------------
template <class Tag, int NT, int NCH>
__global__ __launch_bounds__(NT) void fkl_topk_reg_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K);
  using C = Chunk<Tag>;
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t nch = p.V / C::N;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  if (trow < 0) {
    if (grow) zero_row<Tag, NT>(grow, nch);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;

  u32x4 reg[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int64_t c = (int64_t)i * NT + tid;
    reg[i] = c < nch ? load16_stream(row + c * 16) : C::neg_inf();
  }

  // teacher side while the row is in flight
  const float tlse = stage_teacher<Tag, NT>(p, s, trow, row);
  if (tlse == -INFINITY) {            // no usable teacher entry: the row contributes nothing
    if (grow) zero_row<Tag, NT>(grow, nch);
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
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
  const float mb = mx * a;
  float sm = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[e], a, -mb));
  }
  sm = block_sum<NT>(sm, s.red);
  const float b = mb + fast_log2(sm);      // log2-sum-exp2 of the scaled row
  const float lse = b * LN2;

  const float kl = fkl_from_staged<NT>(p, s, tlse, lse);
  if (tid == 0 && p.row_loss) p.row_loss[r] = kl;

  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int64_t ch = (int64_t)i * NT + tid;
      if (ch < nch) {
        float f[C::N];
        forget(reg[i]);
        C::unpack(reg[i], f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = fast_exp2(fmaf(f[e], a, -b)) * c;
        store16_stream(grow + ch * 16, C::pack(f));
      }
    }
    __syncthreads();      // dense row stores are ordered before the sparse corrections
    fkl_sparse_fix<Tag, NT>(p, s, grow, c);
  }
}

// ---------------------------------------------------------------------------------------
// Forward KL, streaming: any V, any alignment; the row is read twice (second read mostly L2 / MALL).
// ---------------------------------------------------------------------------------------
template <class Tag, int NT, bool VEC>
__global__ __launch_bounds__(NT) void fkl_topk_stream_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K);
  using C = Chunk<Tag>;
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t V = p.V;
  const int64_t nch = V / C::N;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  float tlse = -INFINITY;
  if (trow >= 0) tlse = stage_teacher<Tag, NT>(p, s, trow, row);
  if (tlse == -INFINITY) {
    if (grow) {
      if (VEC) zero_row<Tag, NT>(grow, nch);
      else for (int64_t j = tid; j < V; j += NT) store_from_float(grow, Tag::id, j, 0.f);
    }
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  const float a = p.inv_T_s * LOG2E;
  // pass 1: per-thread running (max, sum) in the exp2 domain
  float m = -INFINITY, sm = 0.f;
  if (VEC) {
    for (int64_t ch = tid; ch < nch; ch += NT) {
      float f[C::N];
      C::unpack(*reinterpret_cast<const u32x4*>(row + ch * 16), f);
      float cm = f[0];
#pragma unroll
      for (int e = 1; e < C::N; ++e) cm = fmaxf(cm, f[e]);
      if (cm > m) { sm *= fast_exp2((m - cm) * a); m = cm; }
      const float mb = m * a;
#pragma unroll
      for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[e], a, -mb));
    }
  } else {
    for (int64_t j = tid; j < V; j += NT) {
      const float f = load_as_float(row, Tag::id, j);
      if (f > m) { sm *= fast_exp2((m - f) * a); m = f; }
      sm += fast_exp2(fmaf(f, a, -m * a));
    }
  }
  const float mx = block_max<NT>(m, s.red);
  const float mb = mx * a;
  sm = (m == -INFINITY) ? 0.f : sm * fast_exp2(fmaf(m, a, -mb));
  sm = block_sum<NT>(sm, s.red);
  const float b = mb + fast_log2(sm);
  const float lse = b * LN2;

  const float kl = fkl_from_staged<NT>(p, s, tlse, lse);
  if (tid == 0 && p.row_loss) p.row_loss[r] = kl;

  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
    if (VEC) {
      for (int64_t ch = tid; ch < nch; ch += NT) {
        float f[C::N];
        C::unpack(*reinterpret_cast<const u32x4*>(row + ch * 16), f);
#pragma unroll
        for (int e = 0; e < C::N; ++e) f[e] = fast_exp2(fmaf(f[e], a, -b)) * c;
        store16_stream(grow + ch * 16, C::pack(f));
      }
    } else {
      for (int64_t j = tid; j < V; j += NT)
        store_from_float(grow, Tag::id, j, fast_exp2(fmaf(load_as_float(row, Tag::id, j), a, -b)) * c);
    }
    __syncthreads();
    fkl_sparse_fix<Tag, NT>(p, s, grow, c);
  }
}

// ---------------------------------------------------------------------------------------
// Reverse KL on the teacher's support: K gathered logits per row, gradient = zero row + K values.
// ---------------------------------------------------------------------------------------
template <class Tag, int NT, bool VEC>
__global__ __launch_bounds__(NT) void rkl_topk_kernel(const TopkParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const TopkLds s(smem, p.K);
  using C = Chunk<Tag>;
  const int64_t r = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t V = p.V;
  char* grow = p.grad ? reinterpret_cast<char*>(p.grad) + r * p.grad_stride * Tag::bytes : nullptr;
  if (grow) {
    if (VEC) zero_row<Tag, NT>(grow, V / C::N);
    else for (int64_t j = tid; j < V; j += NT) store_from_float(grow, Tag::id, j, 0.f);
  }
  const int64_t trow = teacher_row(p.row_map, r, p.n_trows);
  const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
  float tlse = -INFINITY;
  if (trow >= 0) tlse = stage_teacher<Tag, NT>(p, s, trow, row);
  if (tlse == -INFINITY) {
    if (tid == 0 && p.row_loss) p.row_loss[r] = 0.f;
    return;
  }
  // student renormalised over the staged ids
  float zm = -INFINITY;
  for (int k = tid; k < p.K; k += NT)
    if (s.idx[k] >= 0) zm = fmaxf(zm, s.z[k] * p.inv_T_s);
  zm = block_max<NT>(zm, s.red);
  float part = 0.f;
  for (int k = tid; k < p.K; k += NT)
    if (s.idx[k] >= 0) part += expf(s.z[k] * p.inv_T_s - zm);
  const float slse = zm + logf(block_sum<NT>(part, s.red));
  part = 0.f;
  for (int k = tid; k < p.K; k += NT) {
    if (s.idx[k] >= 0) {
      const float sp = s.z[k] * p.inv_T_s - slse;
      const float d = sp - (s.t[k] - tlse);
      const float rk = expf(sp);
      part += rk * d;
      s.t[k] = rk;      // student mass on the support
      s.z[k] = d;       // log ratio
    }
  }
  const float rkl = block_sum<NT>(part, s.red);     // barriers inside publish s.t / s.z
  if (tid == 0 && p.row_loss) p.row_loss[r] = rkl;
  if (grow) {
    const float c = p.inv_T_s * p.grad_scale;
    __syncthreads();    // zero fill precedes the sparse values
    for (int k = tid; k < p.K; k += NT) {
      const int id = s.idx[k];
      if (id < 0) continue;
      float g = 0.f;
      for (int j = 0; j < p.K; ++j) g += (s.idx[j] == id) ? s.t[j] * (s.z[j] - rkl) : 0.f;
      store_from_float(grow, Tag::id, id, g * c);
    }
  }
}

// ---------------------------------------------------------------------------------------
// host dispatch
// ---------------------------------------------------------------------------------------
template <class Tag, int NT, int NCH>
static hipError_t launch_reg(const TopkParams& p, hipStream_t st) {
  hipLaunchKernelGGL((fkl_topk_reg_kernel<Tag, NT, NCH>), dim3((unsigned)p.n_rows), dim3(NT),
                     TopkLds::bytes(p.K), st, p);
  return hipGetLastError();
}

template <class Tag>
static hipError_t launch_fkl(const TopkParams& p, bool aligned, hipStream_t st) {
  const int64_t nch = p.V / Tag::epc;
  if (aligned) {
    if (nch <= 256 * 4) return launch_reg<Tag, 256, 4>(p, st);
    if (nch <= 256 * 8) return launch_reg<Tag, 256, 8>(p, st);
    if (nch <= 256 * 16) return launch_reg<Tag, 256, 16>(p, st);
    if (nch <= 512 * 16) return launch_reg<Tag, 512, 16>(p, st);
    if (nch <= 1024 * 16) return launch_reg<Tag, 1024, 16>(p, st);
    hipLaunchKernelGGL((fkl_topk_stream_kernel<Tag, 1024, true>), dim3((unsigned)p.n_rows), dim3(1024),
                       TopkLds::bytes(p.K), st, p);
  } else {
    hipLaunchKernelGGL((fkl_topk_stream_kernel<Tag, 1024, false>), dim3((unsigned)p.n_rows), dim3(1024),
                       TopkLds::bytes(p.K), st, p);
  }
  return hipGetLastError();
}

template <class Tag>
static hipError_t launch_rkl(const TopkParams& p, bool aligned, hipStream_t st) {
  if (aligned)
    hipLaunchKernelGGL((rkl_topk_kernel<Tag, 256, true>), dim3((unsigned)p.n_rows), dim3(256),
                       TopkLds::bytes(p.K), st, p);
  else
    hipLaunchKernelGGL((rkl_topk_kernel<Tag, 256, false>), dim3((unsigned)p.n_rows), dim3(256),
                       TopkLds::bytes(p.K), st, p);
  return hipGetLastError();
}

}  // namespace dl

extern "C" int dl_div_topk(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                           int64_t V, const int32_t* row_map, const void* t_val, int t_val_dtype,
                           const void* t_idx, int t_idx_itype, int K, int64_t n_teacher_rows,
                           const int32_t* t_cnt, float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                           void* grad, int64_t grad_stride, void* stream) {
  using namespace dl;
  if (!logits || !t_val || !t_idx) return DL_ERR_NULL;
  if (kind != DL_FKL && kind != DL_RKL) return DL_ERR_DTYPE;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || t_val_dtype < DL_F32 || t_val_dtype > DL_F16 ||
      (t_idx_itype != DL_I32 && t_idx_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || K <= 0 || n_teacher_rows < 0 || row_stride < V || (grad && grad_stride < V)) return DL_ERR_SHAPE;
  if (K > DL_MAX_TOPK || n_rows > 0x7fffffffLL || V > 0x7fffffffLL) return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  const int epc = 16 / eb;
  const bool aligned = (V % epc == 0) && (reinterpret_cast<uintptr_t>(logits) % 16 == 0) &&
                       ((row_stride * eb) % 16 == 0) &&
                       (!grad || (reinterpret_cast<uintptr_t>(grad) % 16 == 0 && (grad_stride * eb) % 16 == 0));
  TopkParams p{logits, row_stride, n_rows, V, row_map, t_val, t_val_dtype, t_idx, t_idx_itype, K, n_teacher_rows,
               t_cnt, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  hipError_t e;
  if (kind == DL_FKL) {
    e = logits_dtype == DL_F32 ? launch_fkl<TagF32>(p, aligned, st)
        : logits_dtype == DL_BF16 ? launch_fkl<TagBF16>(p, aligned, st)
                                  : launch_fkl<TagF16>(p, aligned, st);
  } else {
    e = logits_dtype == DL_F32 ? launch_rkl<TagF32>(p, aligned, st)
        : logits_dtype == DL_BF16 ? launch_rkl<TagBF16>(p, aligned, st)
                                  : launch_rkl<TagF16>(p, aligned, st);
  }
  return e == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

// The K-wide half of the reference's composite loss (utils/finetuning_utils.py:58-124) for all
// conversations of a batch: forward KL and reverse KL per token, the top-K cross entropies of
// student and teacher, the alpha-weighted means, the nine logged values, and the backward
// coefficients that dl_rowcoef_grad_topk turns into the gradient of the logits.
//
// Inputs are phase 1's outputs (lse [N], zk [N, K]: the student's full-vocabulary log-probs on the
// teacher's support are zk - lse) and the teacher rows as stored.  Three launches:
//   rows forward   one wave per token row: log-softmax of the teacher over K, kl, rkl, label hit;
//   conversations  one workgroup per conversation: max / valid-mean / weights / the nine values,
//                  and per row the three coefficients dL/dkl, dL/drkl, dL/d(own log-prob);
//   rows backward  one wave per token row: dL/dzk [N, K] and dL/dlse [N].
// A conversation's rows couple through max(kl), the valid-mean of the cross entropy and the means,
// which is why the middle launch exists.  Sums over a conversation are accumulated in double in a
// fixed order: bit-reproducible.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

constexpr int CMP_ROWS_PER_WG = 4;            // one wave each
constexpr int CMP_NT = 256;

// per-row record written by the forward row kernel, read by the other two
struct RowRec { float kl, rkl, own_s, own_t, t_lse, s_lse; int kstar; int valid; };       // 32 bytes
// per-row coefficients for a unit upstream gradient on the conversation's train loss
struct RowCoef { float g_kl, g_rkl, g_own; float pad; };                                  // 16 bytes

struct CompositeParams {
  const float* lse; const float* zk;
  const void* t_val; int t_val_dtype; float inv_T_t;
  const void* t_idx; int t_idx_itype; int K;
  const int64_t* labels; const int32_t* avoid;
  const int32_t* row_off; const int32_t* label_off; const int32_t* avoid_off;   // [C + 1] each
  int n_convos; int64_t n_rows; float alpha;
  RowRec* rec; RowCoef* coef; float* out;         // out [C, 9]
  const float* g_train; float* g_lse; float* g_zk;
};

__device__ __forceinline__ int wave_min_int(int v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, WAVE));
  return v;
}

// conversation that holds row i: last c with row_off[c] <= i
__device__ __forceinline__ int convo_of_row(const int32_t* row_off, int n_convos, int64_t i) {
  int lo = 0, hi = n_convos - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (row_off[mid] <= i) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// ---- rows, forward ---------------------------------------------------------------------------------
__global__ __launch_bounds__(CMP_NT) void composite_rows_fwd_kernel(const CompositeParams p) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t i = (int64_t)blockIdx.x * CMP_ROWS_PER_WG + threadIdx.x / WAVE;
  if (i >= p.n_rows) return;
  const int K = p.K;
  const float* z = p.zk + i * K;
  const float lse = p.lse[i];
  // maxima
  float tmax = -INFINITY, zmax = -INFINITY;
  for (int k = lane; k < K; k += WAVE) {
    tmax = fmaxf(tmax, load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t);
    zmax = fmaxf(zmax, z[k]);
  }
  tmax = wave_max(tmax);
  zmax = wave_max(zmax);
  float tsum = 0.f, zsum = 0.f;
  for (int k = lane; k < K; k += WAVE) {
    tsum += expf(load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t - tmax);
    zsum += expf(z[k] - zmax);
  }
  const float t_lse = tmax + logf(wave_sum(tsum));          // teacher renormalised over its K entries
  const float z_lse = zmax + logf(wave_sum(zsum));          // log-sum-exp of the student over the support
  const float s_lse = z_lse - lse;                          // = logsumexp_k(s_k), s_k = z_k - lse

  // label of this row, if it has one: conversation-local row li carries label li, for li < #labels
  const int c = convo_of_row(p.row_off, p.n_convos, i);
  const int li = (int)(i - p.row_off[c]);
  const int n_lab = p.label_off[c + 1] - p.label_off[c];
  bool want = li < n_lab;
  int64_t label = -1;
  if (want) {
    label = p.labels[p.label_off[c] + li];
    for (int a = p.avoid_off[c]; a < p.avoid_off[c + 1]; ++a) want = want && (p.avoid[a] != li);
  }
  float kl = 0.f, rkl = 0.f;
  int kfound = 0x7fffffff;
  for (int k = lane; k < K; k += WAVE) {
    const float t = load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t - t_lse;
    const float s = z[k] - lse;
    const float s2 = s - s_lse;
    kl += expf(t) * (t - s);
    rkl += expf(s2) * (s2 - t);
    if (want && load_index(p.t_idx, p.t_idx_itype, i * K + k) == label) kfound = min(kfound, k);
  }
  kl = wave_sum(kl);
  rkl = wave_sum(rkl);
  kfound = wave_min_int(kfound);
  if (lane == 0) {
    RowRec r;
    r.kl = kl; r.rkl = rkl; r.t_lse = t_lse; r.s_lse = s_lse;
    r.valid = kfound != 0x7fffffff ? 1 : 0;
    r.kstar = r.valid ? kfound : -1;
    r.own_s = r.valid ? z[kfound] - lse : 0.f;
    r.own_t = r.valid ? load_as_float(p.t_val, p.t_val_dtype, i * K + kfound) * p.inv_T_t - t_lse : 0.f;
    p.rec[i] = r;
  }
}

// ---- conversations -----------------------------------------------------------------------------------
// N sums over the workgroup at once (wave butterflies, then the wave totals in wave order): one pair of barriers for all of them.
template <int NT, int N>
__device__ __forceinline__ void block_sums_f64(double (&v)[N], double* scratch) {
  constexpr int NW = NT / WAVE;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
#pragma unroll
  for (int k = 0; k < N; ++k) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v[k] += __shfl_xor(v[k], o, WAVE);
    if (lane == 0) scratch[k * NW + w] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < N; ++k) {
    double r = 0.0;
#pragma unroll
    for (int i = 0; i < NW; ++i) r += scratch[k * NW + i];
    v[k] = r;
  }
  __syncthreads();
}

// x^alpha and x^(alpha - 1) for the weights; alpha = 2 (the reference's configuration) and 1 need no powf
__device__ __forceinline__ void weight_powers(float x, float alpha, float& pa, float& pa1) {
  if (alpha == 2.f) { pa = x * x; pa1 = x; }
  else if (alpha == 1.f) { pa = x; pa1 = 1.f; }
  else { pa1 = powf(x, alpha - 1.f); pa = powf(x, alpha); }
}

constexpr int CONVO_NT = 256;

__global__ __launch_bounds__(CONVO_NT) void composite_convo_kernel(const CompositeParams p) {
  constexpr int CMP_NT = CONVO_NT;  // (shadows the row kernels' size inside this kernel)
  __shared__ float red[64];
  __shared__ double dred[10 * CMP_NT / WAVE];
  const int c = blockIdx.x, tid = threadIdx.x;
  const int r0 = p.row_off[c], n = p.row_off[c + 1] - r0;
  const int m = p.label_off[c + 1] - p.label_off[c];          // labels; the host guarantees m == n - 1
  const RowRec* rec = p.rec + r0;
  float* out = p.out + (int64_t)c * 9;
  if (n <= 0) {
    if (tid < 9) out[tid] = NAN;
    return;
  }
  const float alpha = p.alpha;

  // maxima (with their multiplicity: the gradient of max() is shared evenly among ties), valid sums
  float mk = -INFINITY, mr = -INFINITY;
  for (int i = tid; i < n; i += CMP_NT) { mk = fmaxf(mk, rec[i].kl); mr = fmaxf(mr, rec[i].rkl); }
  block_max2<CMP_NT>(mk, mr, red);
  double nv = 0.0, sum_s = 0.0, sum_t = 0.0, tie_k = 0.0, tie_r = 0.0;
  for (int i = tid; i < n; i += CMP_NT) {
    const RowRec r = rec[i];
    if (i < m && r.valid) { nv += 1.0; sum_s += (double)r.own_s; sum_t += (double)r.own_t; }
    tie_k += r.kl == mk ? 1.0 : 0.0;
    tie_r += r.rkl == mr ? 1.0 : 0.0;
  }
  {
    double v[5] = {nv, sum_s, sum_t, tie_k, tie_r};
    block_sums_f64<CMP_NT>(v, dred);
    nv = v[0]; sum_s = v[1]; sum_t = v[2]; tie_k = v[3]; tie_r = v[4];
  }
  const float mean_s = (float)(sum_s / nv), mean_t = (float)(sum_t / nv);       // 0 / 0 = NaN: no valid row

  // weighted sums, logged means, and the two sums the gradient of the maxima needs
  double a_wkl = 0.0, a_wrkl = 0.0, a_kl = 0.0, a_rkl = 0.0, a_ces = 0.0, a_cet = 0.0, a_d = 0.0;
  double a_gmk = 0.0, a_gmr = 0.0, a_ginv = 0.0;
  const float inv_n = 1.f / (float)n;
  for (int i = tid; i < n; i += CMP_NT) {
    const RowRec r = rec[i];
    float cpos = 0.f;
    if (i < m) {
      const float ce_s = -(r.valid ? r.own_s : mean_s), ce_t = -(r.valid ? r.own_t : mean_t);
      const float d = ce_s - ce_t;
      cpos = d < 0.f ? 0.f : d;
      a_ces += (double)ce_s; a_cet += (double)ce_t; a_d += (double)d;
      // gradient that reaches the valid rows through the mean substituted into invalid rows
      if (!r.valid && !(d < 0.f)) a_ginv += (double)(0.5f * inv_n * (r.kl + r.rkl));
    }
    const float Ak = r.kl / mk + 1.f, Ar = r.rkl / mr + 1.f;
    float pk, pk1, pr, pr1;
    weight_powers(Ak, alpha, pk, pk1);
    weight_powers(Ar, alpha, pr, pr1);
    const float wk = pk + cpos, wr = pr + cpos;
    a_wkl += (double)(r.kl * wk); a_wrkl += (double)(r.rkl * wr);
    a_kl += (double)r.kl; a_rkl += (double)r.rkl;
    a_gmk += (double)(r.kl * alpha * pk1 * (-r.kl / (mk * mk)));
    a_gmr += (double)(r.rkl * alpha * pr1 * (-r.rkl / (mr * mr)));
  }
  {
    double v[10] = {a_wkl, a_wrkl, a_kl, a_rkl, a_ces, a_cet, a_d, a_gmk, a_gmr, a_ginv};
    block_sums_f64<CMP_NT>(v, dred);
    a_wkl = v[0]; a_wrkl = v[1]; a_kl = v[2]; a_rkl = v[3]; a_ces = v[4]; a_cet = v[5]; a_d = v[6];
    a_gmk = v[7]; a_gmr = v[8]; a_ginv = v[9];
  }
  if (tid == 0) {
    const float wkl = (float)(a_wkl / n), wrkl = (float)(a_wrkl / n);
    const float total = (wkl + wrkl) * 0.5f;
    out[0] = total;                         // train_loss
    out[1] = total;                         // custom loss
    out[2] = (float)(a_ces / m);            // CE loss
    out[3] = (float)(a_kl / n);             // kl_div
    out[4] = (float)(a_rkl / n);            // reverse kl_div
    out[5] = wkl;                           // weighted kl_div
    out[6] = wrkl;                          // weighted rev. kl_div
    out[7] = (float)(a_cet / m);            // teacher CE loss
    out[8] = (float)(a_d / m);              // CE diff
  }
  if (!p.coef) return;
  // coefficients for a unit gradient on train_loss = (wkl + wrkl) / 2, wkl = mean(kl * w)
  const float gmk = 0.5f * inv_n * (float)a_gmk / (float)tie_k, gmr = 0.5f * inv_n * (float)a_gmr / (float)tie_r;
  const float ginv_share = (float)(a_ginv / nv);
  RowCoef* coef = p.coef + r0;
  for (int i = tid; i < n; i += CMP_NT) {
    const RowRec r = rec[i];
    float cpos = 0.f, g_own = 0.f;
    if (i < m) {
      const float d = -(r.valid ? r.own_s : mean_s) + (r.valid ? r.own_t : mean_t);
      cpos = d < 0.f ? 0.f : d;
      if (r.valid) {
        const float g_ce = (d < 0.f) ? 0.f : 0.5f * inv_n * (r.kl + r.rkl);        // dL / d ce_s of this row
        g_own = -(g_ce + ginv_share);                                              // ce_s = -own log-prob
      }
    }
    const float Ak = r.kl / mk + 1.f, Ar = r.rkl / mr + 1.f;
    float pk, pk1, pr, pr1;
    weight_powers(Ak, alpha, pk, pk1);
    weight_powers(Ar, alpha, pr, pr1);
    RowCoef o;
    o.g_kl = 0.5f * inv_n * (pk + cpos + r.kl * alpha * pk1 / mk) + (r.kl == mk ? gmk : 0.f);
    o.g_rkl = 0.5f * inv_n * (pr + cpos + r.rkl * alpha * pr1 / mr) + (r.rkl == mr ? gmr : 0.f);
    o.g_own = g_own;
    o.pad = 0.f;
    coef[i] = o;
  }
}

// ---- rows, backward ----------------------------------------------------------------------------------
__global__ __launch_bounds__(CMP_NT) void composite_rows_bwd_kernel(const CompositeParams p) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t i = (int64_t)blockIdx.x * CMP_ROWS_PER_WG + threadIdx.x / WAVE;
  if (i >= p.n_rows) return;
  const int K = p.K;
  const int c = convo_of_row(p.row_off, p.n_convos, i);
  const float up = p.g_train[c];
  const RowRec r = p.rec[i];
  const RowCoef g = p.coef[i];
  const float lse = p.lse[i];
  const float* z = p.zk + i * K;
  float* gz = p.g_zk + i * K;
  float acc = 0.f;
  for (int k = lane; k < K; k += WAVE) {
    const float t = load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t - r.t_lse;
    const float s2 = z[k] - lse - r.s_lse;
    // d kl / d s_k = -q_k ;  d rkl / d s_k = r_k ((s'_k - t_k) - rkl)
    float gs = g.g_kl * (-expf(t)) + g.g_rkl * expf(s2) * ((s2 - t) - r.rkl);
    if (k == r.kstar) gs += g.g_own;
    gs = up == 0.f ? 0.f : gs * up;             // a conversation that is not part of the loss gets exact zeros, NaN or not
    gz[k] = gs;
    acc += gs;
  }
  acc = wave_sum(acc);
  if (lane == 0) p.g_lse[i] = -acc;             // s_k = z_k - lse
}

}  // namespace dl

static int composite_check(const float* lse, const float* zk, const void* t_val, int t_val_dtype, const void* t_idx,
                           int t_idx_itype, int K, const int32_t* row_off, const int32_t* label_off,
                           const int32_t* avoid_off, int n_convos, int64_t n_rows, const void* rec) {
  if (!lse || !zk || !t_val || !t_idx || !row_off || !label_off || !avoid_off || !rec) return DL_ERR_NULL;
  if (t_val_dtype < DL_F32 || t_val_dtype > DL_F16 || (t_idx_itype != DL_I32 && t_idx_itype != DL_I64)) return DL_ERR_DTYPE;
  if (K <= 0 || n_convos <= 0 || n_rows < 0) return DL_ERR_SHAPE;
  if (n_rows > 0x7fffffffLL) return DL_ERR_LIMIT;
  return DL_OK;
}

extern "C" int dl_composite_forward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                                    float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                    const int64_t* labels, const int32_t* avoid, const int32_t* row_off,
                                    const int32_t* label_off, const int32_t* avoid_off, int n_convos,
                                    int64_t n_rows, float alpha, void* row_records, void* row_coef, float* out,
                                    void* stream) {
  using namespace dl;
  const int st0 = composite_check(lse, zk, t_val, t_val_dtype, t_idx, t_idx_itype, K, row_off, label_off, avoid_off,
                                  n_convos, n_rows, row_records);
  if (st0 != DL_OK) return st0;
  if (!out || !labels) return DL_ERR_NULL;
  CompositeParams p{};
  p.lse = lse; p.zk = zk; p.t_val = t_val; p.t_val_dtype = t_val_dtype; p.inv_T_t = inv_T_teacher;
  p.t_idx = t_idx; p.t_idx_itype = t_idx_itype; p.K = K; p.labels = labels; p.avoid = avoid;
  p.row_off = row_off; p.label_off = label_off; p.avoid_off = avoid_off; p.n_convos = n_convos; p.n_rows = n_rows;
  p.alpha = alpha; p.rec = reinterpret_cast<RowRec*>(row_records); p.coef = reinterpret_cast<RowCoef*>(row_coef);
  p.out = out;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (n_rows > 0)
    hipLaunchKernelGGL(composite_rows_fwd_kernel, dim3((unsigned)((n_rows + CMP_ROWS_PER_WG - 1) / CMP_ROWS_PER_WG)),
                       dim3(CMP_NT), 0, st, p);
  hipLaunchKernelGGL(composite_convo_kernel, dim3((unsigned)n_convos), dim3(CONVO_NT), 0, st, p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_composite_backward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                                     float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                     const int32_t* row_off, int n_convos, int64_t n_rows, const void* row_records,
                                     const void* row_coef, const float* g_train, float* g_lse, float* g_zk,
                                     void* stream) {
  using namespace dl;
  const int st0 = composite_check(lse, zk, t_val, t_val_dtype, t_idx, t_idx_itype, K, row_off, row_off, row_off,
                                  n_convos, n_rows, row_records);
  if (st0 != DL_OK) return st0;
  if (!row_coef || !g_train || !g_lse || !g_zk) return DL_ERR_NULL;
  if (n_rows == 0) return DL_OK;
  CompositeParams p{};
  p.lse = lse; p.zk = zk; p.t_val = t_val; p.t_val_dtype = t_val_dtype; p.inv_T_t = inv_T_teacher;
  p.t_idx = t_idx; p.t_idx_itype = t_idx_itype; p.K = K; p.row_off = row_off; p.n_convos = n_convos; p.n_rows = n_rows;
  p.rec = reinterpret_cast<RowRec*>(const_cast<void*>(row_records));
  p.coef = reinterpret_cast<RowCoef*>(const_cast<void*>(row_coef));
  p.g_train = g_train; p.g_lse = g_lse; p.g_zk = g_zk;
  hipLaunchKernelGGL(composite_rows_bwd_kernel, dim3((unsigned)((n_rows + CMP_ROWS_PER_WG - 1) / CMP_ROWS_PER_WG)),
                     dim3(CMP_NT), 0, reinterpret_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

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
#include "composite.hpp"

namespace dl {

constexpr int CMP_ROWS_PER_WG = 4;            // one wave each
constexpr int CMP_NT = 256;

// ---- rows, forward ---------------------------------------------------------------------------------
// One wave per token row (composite_row_record).
template <int VD, int IT, int R>
__global__ __launch_bounds__(CMP_NT) void composite_rows_fwd_kernel(const CompositeParams p) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t i = (int64_t)blockIdx.x * CMP_ROWS_PER_WG + threadIdx.x / WAVE;
  if (i >= p.n_rows) return;
  composite_row_record<VD, IT, R>(p, i, p.zk + i * p.K, p.lse[i], lane);
}

// ---- conversations -----------------------------------------------------------------------------------
// N sums over the workgroup at once (wave butterflies, then the wave totals in wave order): one pair of barriers for all of them.
template <int NT, int N>
__device__ __forceinline__ void block_sums_f64(double (&v)[N], double* scratch) {
  constexpr int NW = NT / WAVE;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
#pragma unroll
  for (int k = 0; k < N; ++k) v[k] = wave_sum(v[k]);
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) scratch[k * NW + w] = v[k];
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

constexpr int CONVO_NT = 512;
constexpr int CONVO_R = 4;      // rows per thread kept in registers between the passes: conversations of up to 2048 rows are read once

// f(i, record of row i) for the rows this thread serves: the first CONVO_R of them from registers
template <class F>
__device__ __forceinline__ void convo_rows(const RowRec (&mine)[CONVO_R], const RowRec* rec, int n, F f) {
#pragma unroll
  for (int j = 0; j < CONVO_R; ++j) {
    const int i = threadIdx.x + j * CONVO_NT;
    if (i < n) f(i, mine[j]);
  }
  for (int i = threadIdx.x + CONVO_R * CONVO_NT; i < n; i += CONVO_NT) f(i, rec[i]);
}

__global__ __launch_bounds__(CONVO_NT) void composite_convo_kernel(const CompositeParams p) {
  constexpr int CMP_NT = CONVO_NT;  // (shadows the row kernels' size inside this kernel)
  __shared__ float red[64];
  __shared__ double dred[10 * CMP_NT / WAVE];
  const int c = blockIdx.x, tid = threadIdx.x;
  const int r0 = p.off.row(c), n = p.off.row(c + 1) - r0;
  const int m = p.off.label(c + 1) - p.off.label(c);          // labels; the host guarantees m == n - 1
  const RowRec* rec = p.rec + r0;
  float* out = p.out + (int64_t)c * 9;
  if (n <= 0) {
    if (tid < 9) out[tid] = NAN;
    return;
  }
  const float alpha = p.alpha;
  RowRec mine[CONVO_R];
#pragma unroll
  for (int j = 0; j < CONVO_R; ++j) {
    const int i = tid + j * CMP_NT;
    mine[j] = rec[i < n ? i : 0];
  }

  // maxima (with their multiplicity: the gradient of max() is shared evenly among ties), valid sums
  float mk = -INFINITY, mr = -INFINITY;
  convo_rows(mine, rec, n, [&](int, const RowRec& r) { mk = fmaxf(mk, r.kl); mr = fmaxf(mr, r.rkl); });
  block_max2<CMP_NT>(mk, mr, red);
  double nv = 0.0, sum_s = 0.0, sum_t = 0.0, tie_k = 0.0, tie_r = 0.0;
  convo_rows(mine, rec, n, [&](int i, const RowRec& r) {
    if (i < m && r.valid) { nv += 1.0; sum_s += (double)r.own_s; sum_t += (double)r.own_t; }
    tie_k += r.kl == mk ? 1.0 : 0.0;
    tie_r += r.rkl == mr ? 1.0 : 0.0;
  });
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
  const float inv_mk2 = 1.f / (mk * mk), inv_mr2 = 1.f / (mr * mr), inv_mk = 1.f / mk, inv_mr = 1.f / mr;      // for the gradient's terms; the weights themselves divide
  convo_rows(mine, rec, n, [&](int i, const RowRec& r) {
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
    a_gmk += (double)(r.kl * alpha * pk1 * (-r.kl * inv_mk2));
    a_gmr += (double)(r.rkl * alpha * pr1 * (-r.rkl * inv_mr2));
  });
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
  convo_rows(mine, rec, n, [&](int i, const RowRec& r) {
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
    o.g_kl = 0.5f * inv_n * (pk + cpos + r.kl * alpha * pk1 * inv_mk) + (r.kl == mk ? gmk : 0.f);
    o.g_rkl = 0.5f * inv_n * (pr + cpos + r.rkl * alpha * pr1 * inv_mr) + (r.rkl == mr ? gmr : 0.f);
    o.g_own = g_own;
    o.pad = 0.f;
    coef[i] = o;
  });
}

// ---- rows, backward ----------------------------------------------------------------------------------
__global__ __launch_bounds__(CMP_NT) void composite_rows_bwd_kernel(const CompositeParams p) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t i = (int64_t)blockIdx.x * CMP_ROWS_PER_WG + threadIdx.x / WAVE;
  if (i >= p.n_rows) return;
  const int K = p.K;
  const int c = convo_of_row(p.off, p.n_convos, i);
  const float up = p.g_train[c];
  const RowRec r = p.rec[i];
  const RowCoef g = p.coef[i];
  const float lse = p.lse[i];
  const float* z = p.zk + i * K;
  float* gz = p.g_zk + i * K;
  float acc = 0.f;
  for (int k = lane; k < K; k += WAVE) {
    const float gs = composite_entry_grad(p, r, g, up, lse, i, k, z[k]);
    gz[k] = gs;
    acc += gs;
  }
  acc = wave_sum(acc);
  if (lane == 0) p.g_lse[i] = -acc;             // s_k = z_k - lse
}

}  // namespace dl

namespace dl {
template <int VD, int IT>
static void launch_rows_fwd_k(const CompositeParams& p, hipStream_t st) {
  const dim3 grid((unsigned)((p.n_rows + CMP_ROWS_PER_WG - 1) / CMP_ROWS_PER_WG)), block(CMP_NT);
  if (p.K <= 2 * WAVE) hipLaunchKernelGGL((composite_rows_fwd_kernel<VD, IT, 2>), grid, block, 0, st, p);
  else if (p.K <= 4 * WAVE) hipLaunchKernelGGL((composite_rows_fwd_kernel<VD, IT, 4>), grid, block, 0, st, p);
  else if (p.K <= 8 * WAVE) hipLaunchKernelGGL((composite_rows_fwd_kernel<VD, IT, 8>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((composite_rows_fwd_kernel<VD, IT, 0>), grid, block, 0, st, p);
}
template <int VD>
static void launch_rows_fwd_v(const CompositeParams& p, hipStream_t st) {
  if (p.t_idx_itype == DL_I32) launch_rows_fwd_k<VD, I32>(p, st);
  else launch_rows_fwd_k<VD, I64>(p, st);
}
static void launch_rows_fwd(const CompositeParams& p, hipStream_t st) {
  if (p.t_val_dtype == DL_F32) launch_rows_fwd_v<F32>(p, st);
  else if (p.t_val_dtype == DL_BF16) launch_rows_fwd_v<BF16>(p, st);
  else launch_rows_fwd_v<F16>(p, st);
}
}  // namespace dl

static int composite_check(const float* lse, const float* zk, const void* t_val, int t_val_dtype, const void* t_idx,
                           int t_idx_itype, int K, const int32_t* row_off, const int32_t* label_off,
                           const int32_t* avoid_off, int offsets_on_host, int n_convos, int64_t n_rows, const void* rec) {
  if (!lse || !zk || !t_val || !t_idx || !row_off || !label_off || !avoid_off || !rec) return DL_ERR_NULL;
  if (t_val_dtype < DL_F32 || t_val_dtype > DL_F16 || (t_idx_itype != DL_I32 && t_idx_itype != DL_I64)) return DL_ERR_DTYPE;
  if (K <= 0 || n_convos <= 0 || n_rows < 0) return DL_ERR_SHAPE;
  if (n_rows > 0x7fffffffLL || (offsets_on_host && n_convos > DL_MAX_HOST_CONVOS)) return DL_ERR_LIMIT;
  if (offsets_on_host) {
    // host arrays can be checked here: non-decreasing, rows cover exactly n_rows
    if (row_off[0] != 0 || row_off[n_convos] != n_rows || label_off[0] < 0 || avoid_off[0] < 0) return DL_ERR_SHAPE;
    for (int c = 0; c < n_convos; ++c)
      if (row_off[c + 1] < row_off[c] || label_off[c + 1] < label_off[c] || avoid_off[c + 1] < avoid_off[c]) return DL_ERR_SHAPE;
  }
  return DL_OK;
}

static void set_offsets(dl::ConvoOffsets& off, const int32_t* row_off, const int32_t* label_off, const int32_t* avoid_off,
                        int offsets_on_host, int n_convos) {
  const int32_t* src[3] = {row_off, label_off, avoid_off};
  for (int a = 0; a < 3; ++a) {
    off.dev[a] = offsets_on_host ? nullptr : src[a];
    if (offsets_on_host)
      for (int c = 0; c <= n_convos; ++c) off.inl[a][c] = src[a][c];
  }
}

namespace dl {

int composite_forward_params(CompositeParams& p, const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                             float inv_T_teacher, const void* t_idx, int t_idx_itype, int K, const int64_t* labels,
                             const void* avoid, int avoid_itype, const int32_t* row_off, const int32_t* label_off,
                             const int32_t* avoid_off, int offsets_on_host, int n_convos, int64_t n_rows, float alpha,
                             void* row_records, void* row_coef, float* out) {
  const int st0 = composite_check(lse, zk, t_val, t_val_dtype, t_idx, t_idx_itype, K, row_off, label_off, avoid_off,
                                  offsets_on_host, n_convos, n_rows, row_records);
  if (st0 != DL_OK) return st0;
  if (!out) return DL_ERR_NULL;
  if (avoid_itype != DL_I32 && avoid_itype != DL_I64) return DL_ERR_DTYPE;
  if (offsets_on_host && ((label_off[n_convos] > label_off[0] && !labels) || (avoid_off[n_convos] > avoid_off[0] && !avoid)))
    return DL_ERR_NULL;                       // without labels / ignore entries the pointers may be NULL
  if (!offsets_on_host && (!labels || !avoid)) return DL_ERR_NULL;
  p = CompositeParams{};
  p.lse = lse; p.zk = zk; p.t_val = t_val; p.t_val_dtype = t_val_dtype; p.inv_T_t = inv_T_teacher;
  p.t_idx = t_idx; p.t_idx_itype = t_idx_itype; p.K = K; p.labels = labels; p.avoid = avoid; p.avoid_itype = avoid_itype;
  set_offsets(p.off, row_off, label_off, avoid_off, offsets_on_host, n_convos);
  p.n_convos = n_convos; p.n_rows = n_rows;
  p.alpha = alpha; p.rec = reinterpret_cast<RowRec*>(row_records); p.coef = reinterpret_cast<RowCoef*>(row_coef);
  p.out = out;
  return DL_OK;
}

int composite_backward_params(CompositeParams& p, const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                              float inv_T_teacher, const void* t_idx, int t_idx_itype, int K, const int32_t* row_off,
                              int offsets_on_host, int n_convos, int64_t n_rows, const void* row_records,
                              const void* row_coef, const float* g_train) {
  const int st0 = composite_check(lse, zk, t_val, t_val_dtype, t_idx, t_idx_itype, K, row_off, row_off, row_off,
                                  offsets_on_host, n_convos, n_rows, row_records);
  if (st0 != DL_OK) return st0;
  if (!row_coef || !g_train) return DL_ERR_NULL;
  p = CompositeParams{};
  p.lse = lse; p.zk = zk; p.t_val = t_val; p.t_val_dtype = t_val_dtype; p.inv_T_t = inv_T_teacher;
  p.t_idx = t_idx; p.t_idx_itype = t_idx_itype; p.K = K; p.n_convos = n_convos; p.n_rows = n_rows;
  set_offsets(p.off, row_off, row_off, row_off, offsets_on_host, n_convos);
  p.rec = reinterpret_cast<RowRec*>(const_cast<void*>(row_records));
  p.coef = reinterpret_cast<RowCoef*>(const_cast<void*>(row_coef));
  p.g_train = g_train;
  return DL_OK;
}

void launch_composite_rows_fwd(const CompositeParams& p, hipStream_t st) { launch_rows_fwd(p, st); }

void launch_composite_convo(const CompositeParams& p, hipStream_t st) {
  hipLaunchKernelGGL(composite_convo_kernel, dim3((unsigned)p.n_convos), dim3(CONVO_NT), 0, st, p);
}

}  // namespace dl

extern "C" int dl_composite_forward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                                    float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                    const int64_t* labels, const void* avoid, int avoid_itype, const int32_t* row_off,
                                    const int32_t* label_off, const int32_t* avoid_off, int offsets_on_host, int n_convos,
                                    int64_t n_rows, float alpha, void* row_records, void* row_coef, float* out,
                                    void* stream) {
  using namespace dl;
  CompositeParams p;
  const int st0 = composite_forward_params(p, lse, zk, t_val, t_val_dtype, inv_T_teacher, t_idx, t_idx_itype, K, labels, avoid,
                                           avoid_itype, row_off, label_off, avoid_off, offsets_on_host, n_convos, n_rows,
                                           alpha, row_records, row_coef, out);
  if (st0 != DL_OK) return st0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (n_rows > 0) launch_rows_fwd(p, st);
  launch_composite_convo(p, st);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_composite_backward(const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                                     float inv_T_teacher, const void* t_idx, int t_idx_itype, int K,
                                     const int32_t* row_off, int offsets_on_host, int n_convos, int64_t n_rows,
                                     const void* row_records, const void* row_coef, const float* g_train, float* g_lse,
                                     float* g_zk, void* stream) {
  using namespace dl;
  CompositeParams p;
  const int st0 = composite_backward_params(p, lse, zk, t_val, t_val_dtype, inv_T_teacher, t_idx, t_idx_itype, K, row_off,
                                            offsets_on_host, n_convos, n_rows, row_records, row_coef, g_train);
  if (st0 != DL_OK) return st0;
  if (!g_lse || !g_zk) return DL_ERR_NULL;
  if (n_rows == 0) return DL_OK;
  p.g_lse = g_lse; p.g_zk = g_zk;
  hipLaunchKernelGGL(composite_rows_bwd_kernel, dim3((unsigned)((n_rows + CMP_ROWS_PER_WG - 1) / CMP_ROWS_PER_WG)),
                     dim3(CMP_NT), 0, reinterpret_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

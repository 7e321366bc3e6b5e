// Shared between the K-wide kernels of the composite loss (composite.hip) and the two-phase kernels that
// take their row steps along (rowstats.hip): the per-row state, the conversation offsets, and the work of one
// wave on one token row, forward (its record) and backward (the coefficient of one teacher entry).
#pragma once
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

// per-row record written by the forward row kernel, read by the other two
struct RowRec { float kl, rkl, own_s, own_t, t_lse, s_lse; int kstar; int valid; };       // 32 bytes
// per-row coefficients for a unit upstream gradient on the conversation's train loss
struct RowCoef { float g_kl, g_rkl, g_own; float pad; };                                  // 16 bytes

// First row / label / ignore entry of every conversation, [C + 1] each: device arrays, or -- for up to
// DL_MAX_HOST_CONVOS conversations -- copies that travel with the launch (a caller with one
// conversation, or a handful, then needs no upload of three tiny arrays per call).
struct ConvoOffsets {
  const int32_t* dev[3];                          // row, label, avoid; NULL = use `inl`
  int32_t inl[3][DL_MAX_HOST_CONVOS + 1];
  __device__ __forceinline__ int row(int c) const { return dev[0] ? dev[0][c] : inl[0][c]; }
  __device__ __forceinline__ int label(int c) const { return dev[1] ? dev[1][c] : inl[1][c]; }
  __device__ __forceinline__ int avoid(int c) const { return dev[2] ? dev[2][c] : inl[2][c]; }
};

struct CompositeParams {
  const float* lse; const float* zk;
  const void* t_val; int t_val_dtype; float inv_T_t;
  const void* t_idx; int t_idx_itype; int K;
  const int64_t* labels; const void* avoid; int avoid_itype;
  ConvoOffsets off;
  int n_convos; int64_t n_rows; float alpha;
  RowRec* rec; RowCoef* coef; float* out;         // out [C, 9]
  const float* g_train; float* g_lse; float* g_zk;
};

__device__ __forceinline__ int wave_min_int(int v) { return wave_min(v); }

// conversation that holds row i: last c whose first row is <= i
__device__ __forceinline__ int convo_of_row(const ConvoOffsets& off, int n_convos, int64_t i) {
  int lo = 0, hi = n_convos - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (off.row(mid) <= i) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The record of token row i, by one wave: `z` are the row's K scaled logits at the teacher's ids, `lse` its
// full-vocabulary log-sum-exp.  R > 0: K <= 64 * R and the storage types are known at compile time: the
// row's teacher values, ids and gathered logits are fetched once, all loads in flight together, and
// stay in registers for the three passes (maxima, sums, divergences).  R == 0: any K, any types,
// three passes over memory.
template <int VD, int IT, int R>
__device__ __forceinline__ void composite_row_record(const CompositeParams& p, int64_t i, const float* z, float lse, int lane) {
  const int K = p.K;
  constexpr int RR = R > 0 ? R : 1;
  float tv[RR], zv[RR];
  int64_t id[RR];
  if constexpr (R > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int k = lane + j * WAVE;
      const int64_t at = i * K + (k < K ? k : 0);      // lanes beyond K read entry 0 and discard it: no branch between the loads
      float t;
      if constexpr (VD == F32) t = reinterpret_cast<const float*>(p.t_val)[at];
      else if constexpr (VD == BF16) t = __uint_as_float((unsigned)reinterpret_cast<const unsigned short*>(p.t_val)[at] << 16);
      else t = (float)reinterpret_cast<const _Float16*>(p.t_val)[at];
      if constexpr (IT == I32) id[j] = reinterpret_cast<const int32_t*>(p.t_idx)[at];
      else id[j] = reinterpret_cast<const int64_t*>(p.t_idx)[at];
      const float zz = z[k < K ? k : 0];
      tv[j] = k < K ? t * p.inv_T_t : -INFINITY;
      zv[j] = k < K ? zz : -INFINITY;
      id[j] = k < K ? id[j] : -1;
    }
  }
  // maxima
  float tmax = -INFINITY, zmax = -INFINITY;
  if constexpr (R > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) { tmax = fmaxf(tmax, tv[j]); zmax = fmaxf(zmax, zv[j]); }
  } else {
    for (int k = lane; k < K; k += WAVE) {
      tmax = fmaxf(tmax, load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t);
      zmax = fmaxf(zmax, z[k]);
    }
  }
  tmax = wave_max(tmax);
  zmax = wave_max(zmax);
  float tsum = 0.f, zsum = 0.f;
  if constexpr (R > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) { tsum += expf(tv[j] - tmax); zsum += expf(zv[j] - zmax); }      // exp(-inf) = 0 beyond K
  } else {
    for (int k = lane; k < K; k += WAVE) {
      tsum += expf(load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t - tmax);
      zsum += expf(z[k] - zmax);
    }
  }
  const float t_lse = tmax + logf(wave_sum(tsum));          // teacher renormalised over its K entries
  const float z_lse = zmax + logf(wave_sum(zsum));          // log-sum-exp of the student over the support
  const float s_lse = z_lse - lse;                          // = logsumexp_k(s_k), s_k = z_k - lse

  // label of this row, if it has one: conversation-local row li carries label li, for li < #labels
  const int c = convo_of_row(p.off, p.n_convos, i);
  const int li = (int)(i - p.off.row(c));
  const int n_lab = p.off.label(c + 1) - p.off.label(c);
  bool want = li < n_lab;
  int64_t label = -1;
  if (want) {
    label = p.labels[p.off.label(c) + li];
    for (int a = p.off.avoid(c); a < p.off.avoid(c + 1); ++a) want = want && (load_index(p.avoid, p.avoid_itype, a) != li);
  }
  float kl = 0.f, rkl = 0.f;
  int kfound = 0x7fffffff;
  if constexpr (R > 0) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int k = lane + j * WAVE;
      if (k < K) {
        const float t = tv[j] - t_lse;
        const float s = zv[j] - lse;
        const float s2 = s - s_lse;
        kl += expf(t) * (t - s);
        rkl += expf(s2) * (s2 - t);
        if (want && id[j] == label) kfound = min(kfound, k);
      }
    }
  } else {
    for (int k = lane; k < K; k += WAVE) {
      const float t = load_as_float(p.t_val, p.t_val_dtype, i * K + k) * p.inv_T_t - t_lse;
      const float s = z[k] - lse;
      const float s2 = s - s_lse;
      kl += expf(t) * (t - s);
      rkl += expf(s2) * (s2 - t);
      if (want && load_index(p.t_idx, p.t_idx_itype, i * K + k) == label) kfound = min(kfound, k);
    }
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

// d(train loss of the row's conversation, times its upstream gradient `up`) / d(scaled logit at teacher entry k)
// of token row i: d kl / d s_k = -q_k,  d rkl / d s_k = r_k ((s'_k - t_k) - rkl), the label's own log-prob on entry kstar.
__device__ __forceinline__ float composite_entry_grad(const CompositeParams& p, const RowRec& r, const RowCoef& g, float up,
                                                      float lse, int64_t i, int k, float zk) {
  const float t = load_as_float(p.t_val, p.t_val_dtype, i * p.K + k) * p.inv_T_t - r.t_lse;
  const float s2 = zk - lse - r.s_lse;
  float gs = g.g_kl * (-expf(t)) + g.g_rkl * expf(s2) * ((s2 - t) - r.rkl);
  if (k == r.kstar) gs += g.g_own;
  return up == 0.f ? 0.f : gs * up;             // a conversation that is not part of the loss gets exact zeros, NaN or not
}

// Host side (composite.hip): argument checks of dl_composite_forward / dl_composite_backward that fill the kernels'
// parameters, and the launch of the per-conversation kernel.
int composite_forward_params(CompositeParams& p, const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                             float inv_T_teacher, const void* t_idx, int t_idx_itype, int K, const int64_t* labels,
                             const void* avoid, int avoid_itype, const int32_t* row_off, const int32_t* label_off,
                             const int32_t* avoid_off, int offsets_on_host, int n_convos, int64_t n_rows, float alpha,
                             void* row_records, void* row_coef, float* out);
int composite_backward_params(CompositeParams& p, const float* lse, const float* zk, const void* t_val, int t_val_dtype,
                              float inv_T_teacher, const void* t_idx, int t_idx_itype, int K, const int32_t* row_off,
                              int offsets_on_host, int n_convos, int64_t n_rows, const void* row_records,
                              const void* row_coef, const float* g_train);
void launch_composite_rows_fwd(const CompositeParams& p, hipStream_t st);
void launch_composite_convo(const CompositeParams& p, hipStream_t st);

}  // namespace dl

// Forward KL, reverse KL and Jensen-Shannon divergence against a DENSE (full-vocabulary) teacher:
// loss and gradient in one launch.
//
// One workgroup per token row.  Student and teacher rows are pulled into registers with 16-byte
// non-temporal loads (each read from HBM once) and swept four times from there: maxima, sums of
// exponentials, divergence sums, gradient.  All arithmetic runs in the log2 domain
// (lp = x * inv_T * log2(e) - log2-sum-exp2), natural logs appear only in the results.
//
// The same sweeps serve the byte-trie path, where the teacher row is not read from memory but is
// the log of a marginal that the workgroup has just accumulated in LDS (marginalise.hip).
#pragma once
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

// ---- a unit = 8 consecutive columns: one 16-byte chunk of a 16-bit row, two of an fp32 row ----
template <class Tag> struct Unit {
  static constexpr int NC = Tag::bytes == 4 ? 2 : 1;
  u32x4 c[NC];
  __device__ __forceinline__ void load(const char* row, int64_t u) {
#pragma unroll
    for (int k = 0; k < NC; ++k) c[k] = load16_stream(row + (u * NC + k) * 16);
  }
  __device__ __forceinline__ void fill_neg_inf() {
#pragma unroll
    for (int k = 0; k < NC; ++k) c[k] = Chunk<Tag>::neg_inf();
  }
  __device__ __forceinline__ void unpack(float* f) {
#pragma unroll
    for (int k = 0; k < NC; ++k) { forget(c[k]); Chunk<Tag>::unpack(c[k], f + k * Chunk<Tag>::N); }
  }
  __device__ static __forceinline__ void store(char* row, int64_t u, const float* f) {
#pragma unroll
    for (int k = 0; k < NC; ++k) store16_stream(row + (u * NC + k) * 16, Chunk<Tag>::pack(f + k * Chunk<Tag>::N));
  }
};

// Per-row results of the statistic sweeps, log2 domain.
struct DenseStats {
  float a_s, a_t;        // inv_T * log2(e) of student / teacher
  float ls, lt;          // log2-sum-exp2 of the scaled student (over the support for RKL) / teacher row
  float loss;            // natural-log divergence of the row
  float aux;             // FKL: unused; RKL: rkl; JSD: KL(P || M)
  float tmax;            // largest teacher logit of the row (-inf: the teacher row carries no mass)
};

// Divergence terms of one column.  lp / lq: log2-probabilities of student / teacher.
__device__ __forceinline__ void fkl_term(float lp, float lq, float& acc) {
  const float q = fast_exp2(lq);
  acc += q > 0.f ? q * (lq - lp) : 0.f;
}
__device__ __forceinline__ void rkl_term(float lp, float lq, float& acc) {
  const float r = fast_exp2(lp);
  acc += (lq > -INFINITY && r > 0.f) ? r * (lp - lq) : 0.f;
}
__device__ __forceinline__ float log2_mix(float lp, float lq) {      // log2((2^lp + 2^lq) / 2)
  const float hi = fmaxf(lp, lq), lo = fminf(lp, lq);
  return hi + fast_log2(0.5f + 0.5f * fast_exp2(lo - hi));
}
__device__ __forceinline__ void jsd_term(float lp, float lq, float& kl_pm, float& kl_qm) {
  if (lp == -INFINITY && lq == -INFINITY) return;
  const float lm = log2_mix(lp, lq);
  const float pr = fast_exp2(lp), q = fast_exp2(lq);
  kl_pm += pr > 0.f ? pr * (lp - lm) : 0.f;
  kl_qm += q > 0.f ? q * (lq - lm) : 0.f;
}

// Gradient of one column (before the common factor c = inv_T * scale).
__device__ __forceinline__ float dense_grad(int kind, float lp, float lq, float aux) {
  if (kind == DL_FKL) return fast_exp2(lp) - fast_exp2(lq);
  if (kind == DL_RKL) return lq > -INFINITY ? fast_exp2(lp) * ((lp - lq) * LN2 - aux) : 0.f;
  if (lp == -INFINITY) return 0.f;
  return 0.5f * fast_exp2(lp) * ((lp - log2_mix(lp, lq)) * LN2 - aux);
}

// The four sweeps over a row pair.  `Rows` provides
//   template <class F> void sweep(F f)       calls f(u, s[8], t[8]) for every unit this thread owns
// (values already unpacked to fp32, -inf beyond the row), and `red` is LDS scratch of 64 floats.
template <int NT, class Rows>
__device__ __forceinline__ DenseStats dense_stats(int kind, Rows& rows, float inv_T_s, float inv_T_t, float* red) {
  DenseStats st;
  st.a_s = inv_T_s * LOG2E;
  st.a_t = inv_T_t * LOG2E;
  // maxima (for RKL the student maximum is taken over the teacher's support)
  float ms = -INFINITY, mt = -INFINITY;
  rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      mt = fmaxf(mt, t[e]);
      ms = fmaxf(ms, (kind == DL_RKL && t[e] == -INFINITY) ? -INFINITY : s[e]);
    }
  });
  block_max2<NT>(ms, mt, red);
  st.tmax = mt;
  const float bs = ms * st.a_s, bt = mt * st.a_t;
  float ss = 0.f, stt = 0.f;
  rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float es = fast_exp2(fmaf(s[e], st.a_s, -bs));
      ss += (kind == DL_RKL && t[e] == -INFINITY) ? 0.f : es;
      stt += fast_exp2(fmaf(t[e], st.a_t, -bt));
    }
  });
  block_sum2<NT>(ss, stt, red);
  st.ls = bs + fast_log2(ss);
  st.lt = bt + fast_log2(stt);
  // divergence sums
  float x = 0.f, y = 0.f;
  rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float lp = fmaf(s[e], st.a_s, -st.ls), lq = fmaf(t[e], st.a_t, -st.lt);
      if (kind == DL_FKL) fkl_term(lp, lq, x);
      else if (kind == DL_RKL) rkl_term(lp, lq, x);
      else jsd_term(lp, lq, x, y);
    }
  });
  block_sum2<NT>(x, y, red);
  if (kind == DL_JSD) { st.loss = 0.5f * LN2 * (x + y); st.aux = x * LN2; }
  else { st.loss = x * LN2; st.aux = st.loss; }
  return st;
}

template <class TagS, class Rows>
__device__ __forceinline__ void dense_grad_sweep(int kind, Rows& rows, const DenseStats& st, float c, char* grow) {
  rows.sweep([&](int64_t u, const float* s, const float* t) {
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float lp = fmaf(s[e], st.a_s, -st.ls), lq = fmaf(t[e], st.a_t, -st.lt);
      g[e] = dense_grad(kind, lp, lq, st.aux) * c;
    }
    Unit<TagS>::store(grow, u, g);
  });
}

}  // namespace dl

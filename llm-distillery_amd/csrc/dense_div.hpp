// Forward KL, reverse KL and Jensen-Shannon divergence against a DENSE (full-vocabulary) teacher:
// loss and gradient in one launch.
//
// One workgroup per token row.  Student and teacher rows are pulled into registers with 16-byte
// non-temporal loads (each read from HBM once) and swept from there: maxima, sums of exponentials
// (with the divergence sum of forward / reverse KL riding along; JSD takes a sweep of its own),
// gradient.  Rows too wide for the registers are swept from memory, maxima and sums in one sweep.  All arithmetic runs in the log2 domain
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
  // A unit of a 4-byte row is two chunks side by side: a wave's load (or store) instruction then touches
  // every other 16 bytes, half of each 64-byte line, and the instruction for the other chunk the other
  // half.  With streaming accesses the halves travel separately (8192 x 32000 fp32 forward KL: 52 % of the
  // HBM peak); through the cache they meet there (64 %).  Units of one chunk keep the streaming hints.
  __device__ __forceinline__ void load(const char* row, int64_t u) {
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      if constexpr (NC == 1) c[k] = load16_stream(row + (u * NC + k) * 16);
      else c[k] = *reinterpret_cast<const u32x4*>(row + (u * NC + k) * 16);
    }
  }
  __device__ __forceinline__ void fill_neg_inf() {
#pragma unroll
    for (int k = 0; k < NC; ++k) c[k] = Chunk<Tag>::neg_inf();
  }
  __device__ __forceinline__ void unpack(float* f) {
#pragma unroll
    for (int k = 0; k < NC; ++k) { forget(c[k]); Chunk<Tag>::unpack(c[k], f + k * Chunk<Tag>::N); }
  }
  __device__ __forceinline__ void repack(const float* f) {
#pragma unroll
    for (int k = 0; k < NC; ++k) c[k] = Chunk<Tag>::pack(f + k * Chunk<Tag>::N);
  }
  __device__ static __forceinline__ void store(char* row, int64_t u, const float* f) {
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      if constexpr (NC == 1) store16_stream(row + (u * NC + k) * 16, Chunk<Tag>::pack(f + k * Chunk<Tag>::N));
      else *reinterpret_cast<u32x4*>(row + (u * NC + k) * 16) = Chunk<Tag>::pack(f + k * Chunk<Tag>::N);
    }
  }
  // The same for rows of V columns that may start anywhere (element-aligned) and end inside a chunk:
  // whole chunks by unaligned 16-byte accesses, a partly filled one element by element (-inf / not
  // stored beyond the row), nothing for chunks wholly beyond it.
  __device__ __forceinline__ void load_any(const char* row, int64_t u, int64_t V) {
    constexpr int N = Chunk<Tag>::N;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int64_t ch = u * NC + k;
      c[k] = (ch + 1) * N <= V ? load16_unaligned(row + ch * 16)
             : ch * N < V      ? load_chunk_elementwise<Tag>(row, (int)ch, (int)V)
                               : Chunk<Tag>::neg_inf();
    }
  }
  __device__ static __forceinline__ void store_any(char* row, int64_t u, int64_t V, const float* f) {
    constexpr int N = Chunk<Tag>::N;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int64_t ch = u * NC + k;
      const u32x4 v = Chunk<Tag>::pack(f + k * N);
      if ((ch + 1) * N <= V) store16_unaligned(row + ch * 16, v);
      else if (ch * N < V) store_chunk_elementwise<Tag>(row, (int)ch, (int)V, v);
    }
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
// Three transcendentals per column: the mixture's logarithm is taken of the probabilities themselves.
// Columns where a probability underflows contribute nothing for it: log2 p - log2 m is at most 1
// (m >= p / 2) and is held inside [LOG_FLOOR, 1], so that 0 * difference is 0 without a select.  One
// median instruction does it for every case: -inf (p = 0 < m) -> the floor, +inf (m underflows, log2 p
// finite) -> 1, and the NaN of -inf - -inf -> the floor (the median of a NaN is the smaller bound).
constexpr float LOG_FLOOR = -1e30f;
__device__ __forceinline__ float log_ratio_to_mixture(float lp, float lm) {
  return __builtin_amdgcn_fmed3f(lp - lm, LOG_FLOOR, 1.f);
}
__device__ __forceinline__ void jsd_term(float lp, float lq, float& kl_pm, float& kl_qm) {
  const float pr = fast_exp2(lp), q = fast_exp2(lq);
  const float lm = fast_log2(0.5f * pr + 0.5f * q);
  kl_pm = fmaf(pr, log_ratio_to_mixture(lp, lm), kl_pm);
  kl_qm = fmaf(q, log_ratio_to_mixture(lq, lm), kl_qm);
}

// Gradient of one column (before the common factor c = inv_T * scale).
// A student column of -inf (a masked vocabulary entry) where the teacher has mass carries no student mass:
// its log ratio is held finite so that 0 * ratio is 0, as in the loss sweeps.  The mixture's logarithm goes
// through log_ratio_to_mixture here as everywhere: a student mass so small that half of it is a denormal,
// on a column without teacher mass, gives log2 m = -inf (the hardware logarithm takes denormals for zero).
__device__ __forceinline__ float rkl_log_ratio(float lp, float lq) {
  return __builtin_amdgcn_fmed3f(lp - lq, LOG_FLOOR, -LOG_FLOOR);
}
__device__ __forceinline__ float dense_grad(int kind, float lp, float lq, float aux) {
  if (kind == DL_FKL) return fast_exp2(lp) - fast_exp2(lq);
  if (kind == DL_RKL) return lq > -INFINITY ? fast_exp2(lp) * (rkl_log_ratio(lp, lq) * LN2 - aux) : 0.f;
  const float pr = fast_exp2(lp);
  return 0.5f * pr * (log_ratio_to_mixture(lp, fast_log2(0.5f * pr + 0.5f * fast_exp2(lq))) * LN2 - aux);
}

// The same with the kind a compile-time constant and the row's constants folded:
//   FKL  c (p - q)                                             kb, k0 unused
//   RKL  r (kb (lp - lq) + k0)            kb = c ln 2,         k0 = -c RKL
//   JSD  p (kb (lp - lm) + k0)            kb = c ln 2 / 2,     k0 = -c KL(P || M) / 2
template <int KIND>
__device__ __forceinline__ float dense_grad_column(float lp, float lq, float c, float kb, float k0) {
  if (KIND == DL_FKL) return (fast_exp2(lp) - fast_exp2(lq)) * c;
  if (KIND == DL_RKL) return lq > -INFINITY ? fast_exp2(lp) * fmaf(rkl_log_ratio(lp, lq), kb, k0) : 0.f;
  const float pr = fast_exp2(lp);
  return pr * fmaf(log_ratio_to_mixture(lp, fast_log2(0.5f * pr + 0.5f * fast_exp2(lq))), kb, k0);
}

// The sweeps over a row pair held in registers.  `Rows` provides
//   template <class F> void sweep(F f)       calls f(u, s[8], t[8]) for every unit this thread owns
// (values already unpacked to fp32, -inf beyond the row), and `red` is LDS scratch of 64 floats.
// KIND is a compile-time constant: the per-column code carries no branch on it.
//
// Forward and reverse KL need three sweeps, not four: with es = 2^(s a_s - bs), et = 2^(t a_t - bt)
// (bs, bt the scaled maxima) and S = sum es, T = sum et,
//   FKL = sum q (lq - lp) = (1/T) sum et ((t a_t - bt) - (s a_s - bs)) - log2 T + log2 S      (q = et / T)
//   RKL = sum r (lp - lq) = (1/S) sum es ((s a_s - bs) - (t a_t - bt)) - log2 S + log2 T      (r = es / S, support only)
// so the divergence sum rides along with the sums of exponentials.  JSD needs the normalised
// probabilities inside a logarithm and keeps its own sweep.
//
// STASH (JSD on rows of fp32 pairs held in registers): the divergence sweep leaves p and
// log2 p - log2 m in the registers of the logits, exactly, and the gradient
//   g = c p / 2 ((log2 p - log2 m) ln 2 - KL(P || M))
// takes two instructions per column (dense_jsd_grad_from_stash) instead of recomputing three
// transcendentals (8192 x 32000: 0.70 -> 0.67 ms).  The same for forward and reverse KL (their
// exponentials kept) shortened the arithmetic by a third and the kernel not at all: with fp32 rows
// those two are not bound by the vector ALU.
template <int KIND, int NT, bool STASH = false, class Rows>
__device__ __forceinline__ DenseStats dense_stats(Rows& rows, float inv_T_s, float inv_T_t, float* red) {
  DenseStats st;
  st.a_s = inv_T_s * LOG2E;
  st.a_t = inv_T_t * LOG2E;
  const float a_s = st.a_s, a_t = st.a_t;
  float ms = -INFINITY, mt = -INFINITY;     // maxima (for RKL the student maximum is taken over the teacher's support)
  float ss = 0.f, stt = 0.f, w = 0.f;
  if constexpr (Rows::ONLINE) {
    // Rows that are read from memory in every sweep: maxima and sums in ONE sweep.  Each thread keeps
    // running maxima; when a unit raises one, what has been summed so far is carried over to the new
    // bias: with shifts ds, dt >= 0 of the two biases (log2 domain), es scales by 2^-ds, et by 2^-dt,
    // and the divergence terms et (xt - xs) / es (xs - xt) follow from xs -= ds, xt -= dt.  A maximum
    // of -inf means that nothing has been summed on that side yet (bias 0 keeps 2^(-inf - bias) = 0).
    const auto carry = [&](float nms, float nmt) {
      const float ds = ms == -INFINITY ? 0.f : (nms - ms) * a_s, dt = mt == -INFINITY ? 0.f : (nmt - mt) * a_t;
      const float fs = fast_exp2(-ds), ft = fast_exp2(-dt);
      if (KIND == DL_FKL) w = ft * (w - (dt - ds) * stt);
      if (KIND == DL_RKL) w = fs * (w - (ds - dt) * ss);
      ss *= fs;
      stt *= ft;
      ms = nms;
      mt = nmt;
    };
    rows.sweep([&](int64_t, const float* s, const float* t) {
      float ums = -INFINITY, umt = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        umt = fmaxf(umt, t[e]);
        ums = fmaxf(ums, (KIND == DL_RKL && t[e] == -INFINITY) ? -INFINITY : s[e]);
      }
      if (ums > ms || umt > mt) carry(fmaxf(ms, ums), fmaxf(mt, umt));
      const float bs = ms == -INFINITY ? 0.f : ms * a_s, bt = mt == -INFINITY ? 0.f : mt * a_t;
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
          if (KIND == DL_FKL) w += et > 0.f ? et * (xt - xs) : 0.f;
        }
      }
    });
    float gs = ms, gt = mt;
    block_max2<NT>(gs, gt, red);
    carry(gs, gt);                          // this thread's sums on the row's biases
  } else {
    bool have = false;
    if constexpr (KIND != DL_RKL && Rows::RAW_MAXIMA) have = rows.raw_maxima(ms, mt, red);      // RKL: the student's maximum is over the support
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
    const float bs = ms * a_s, bt = mt * a_t;
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
          if (KIND == DL_FKL) w += et > 0.f ? et * (xt - xs) : 0.f;
        }
      }
    });
  }
  st.tmax = mt;
  const float bs = ms * a_s, bt = mt * a_t;
  block_sum2<NT>(ss, stt, red);
  const float l2s = fast_log2(ss), l2t = fast_log2(stt);
  st.ls = bs + l2s;
  st.lt = bt + l2t;
  if (KIND != DL_JSD) {
    w = block_sum<NT>(w, red);
    const float x = KIND == DL_FKL ? w / stt - l2t + l2s : w / ss - l2s + l2t;
    st.loss = x * LN2;
    st.aux = st.loss;
    return st;
  }
  float x = 0.f, y = 0.f;
  if constexpr (STASH) {
    rows.sweep_rewrite([&](int64_t, float* s, float* t) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float lp = fmaf(s[e], a_s, -st.ls), lq = fmaf(t[e], a_t, -st.lt);
        const float pr = fast_exp2(lp), q = fast_exp2(lq);
        const float lm = fast_log2(0.5f * pr + 0.5f * q);
        const float d = log_ratio_to_mixture(lp, lm);       // finite: pr = 0 then gives a gradient of 0
        x = fmaf(pr, d, x);
        y = fmaf(q, log_ratio_to_mixture(lq, lm), y);
        s[e] = pr;
        t[e] = d;
      }
    });
  } else {
    rows.sweep([&](int64_t, const float* s, const float* t) {
#pragma unroll
      for (int e = 0; e < 8; ++e) jsd_term(fmaf(s[e], a_s, -st.ls), fmaf(t[e], a_t, -st.lt), x, y);
    });
  }
  block_sum2<NT>(x, y, red);
  st.loss = 0.5f * LN2 * (x + y);
  st.aux = x * LN2;
  return st;
}

template <int KIND, class TagS, class Rows>
__device__ __forceinline__ void dense_grad_sweep(Rows& rows, const DenseStats& st, float c, char* grow) {
  const float a_s = st.a_s, a_t = st.a_t, ls = st.ls, lt = st.lt;
  const float kb = (KIND == DL_JSD ? 0.5f : 1.f) * c * LN2, k0 = (KIND == DL_JSD ? -0.5f : -1.f) * c * st.aux;
  rows.sweep([&](int64_t u, const float* s, const float* t) {
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = dense_grad_column<KIND>(fmaf(s[e], a_s, -ls), fmaf(t[e], a_t, -lt), c, kb, k0);
    rows.store(grow, u, g);
  });
}

// The JSD gradient from what dense_stats<DL_JSD, NT, true> left in the registers.
template <class TagS, class Rows>
__device__ __forceinline__ void dense_jsd_grad_from_stash(Rows& rows, const DenseStats& st, float c, char* grow) {
  const float kb = 0.5f * c * LN2, k0 = -0.5f * c * st.aux;
  rows.sweep([&](int64_t u, const float* pr, const float* d) {
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = pr[e] * fmaf(d[e], kb, k0);
    rows.store(grow, u, g);
  });
}

}  // namespace dl

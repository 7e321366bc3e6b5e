"""CPU restatement of the reference's distillation-loss arithmetic.

TEST INFRASTRUCTURE ONLY -- the checker, never the product.  The shipped
package must not import this module; only tests, the smoke check and the
CPU-baseline leg of the benchmark do.

Every function names the reference lines (relative to the reference tree) it
follows.  The arithmetic itself lives in PyTorch library routines
(`F.log_softmax`, `torch.gather`, `F.kl_div(log_target=True)`, `torch.topk`,
`torch.unique`, `index_add_`), exactly as in the reference, so this file calls
the same routines.  `dtype=torch.float64` gives the "truth" variant used for
tolerances, `torch.float32` the reference-precision variant.

Parity status (what pins each function besides reading the reference):
  * student/teacher log-softmax, forward KL, reverse KL (top-K): closed forms,
    gradient identities, invariants and the golden fixture written from the
    reference's `calculate_divergence`            -> pinned.
  * top-K cross entropy, alpha-weighted composite, 9-key dict: golden fixture
    plus brute-force loops                        -> pinned.
  * pairwise top-K merge: dict brute force, mass conservation -> pinned
    (tie order inside `torch.topk` is implementation defined in the reference;
    here ties break towards the smaller id -- "parity unpinned" for ties).
  * dense-teacher forward/reverse KL: the reference's training side cannot run
    with `indices=None` (it raises), so these follow the formula of
    `custom_kl_div` and reduce to the top-K functions at K=V    -> pinned by
    that reduction only.
  * forward KL against a ragged, already-normalised sparse teacher
    (`fwd_kl_sparse_rows`, the checker of the merged multi-teacher loss):
    reduces to the golden-pinned top-K form on full rows, to `F.kl_div` on the
    live prefix of ragged rows, gradient identity   -> pinned.
  * JSD, weighted multi-teacher merge, vocabulary remap, byte-trie map and CSR
    marginalisation have NO counterpart in the reference: "parity unpinned";
    they are pinned by textbook formulas, brute force and invariants.
"""
from __future__ import annotations

import math
from typing import Iterable, Sequence

import numpy as np
import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# ---------------------------------------------------------------------------
# a0 -- caller prologue (row selection, temperature, label construction)
# ---------------------------------------------------------------------------

def content_indices(content_ranges: Sequence[tuple[int, int]]) -> np.ndarray:
    """Rows of a conversation that carry content.

    Follows classes/student/model.py:87-91 and
    classes/teacher/result_processor_worker.py:27-31: the concatenation of
    `arange(start, end)` over the content ranges.
    """
    return np.concatenate([np.arange(a, b) for a, b in content_ranges]).astype(np.int64)


def ce_indices(content_ranges: Sequence[tuple[int, int]], context_len: int,
               convo_len: int) -> tuple[np.ndarray, np.ndarray]:
    """Label positions (content rows shifted by one) and the rows to ignore.

    Follows classes/student/model.py:93-116.  Ranges that start at or beyond
    the context length are skipped; with more than one range the last row of
    every range is ignored for the cross entropy (its label belongs to the next
    turn's header); a final label at or after the conversation length is
    dropped together with its ignore entry.
    """
    labels, avoid = [], []
    many = len(content_ranges) > 1
    cursor = 0
    for start, end in content_ranges:
        if start + 1 > context_len:
            continue
        labels.append(np.arange(start + 1, end + 1))
        last = cursor + (end - start) - 1
        if many:
            avoid.append(last)
        cursor = last + 1
    lab = np.concatenate(labels)
    if lab[-1] >= convo_len:
        lab = lab[:-1]
        if avoid:
            avoid.pop()
    return lab.astype(np.int64), np.asarray(avoid, dtype=np.int64)


def scaled_student_logits(model_logits: torch.Tensor, crop: int, T: float,
                          dtype=torch.float32) -> torch.Tensor:
    """`logits[..., :crop].float() / T` -- classes/student/model.py:408."""
    return model_logits[..., :crop].to(dtype) / T


# ---------------------------------------------------------------------------
# a1..a4 -- per-token divergences on a top-K teacher
# ---------------------------------------------------------------------------

def student_logprobs_on_support(z: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """Full-vocabulary log-softmax of the student, gathered at the teacher ids.

    utils/finetuning_utils.py:88,92.  The result does not sum to one over K.
    """
    return torch.gather(F.log_softmax(z, dim=-1), 1, idx.long())


def teacher_logprobs_topk(stored: torch.Tensor, T: float = 1.0, dtype=torch.float32) -> torch.Tensor:
    """Teacher renormalised over its K stored entries.

    classes/student/model.py:421 (divide the stored log-probs by T) followed by
    utils/finetuning_utils.py:91 (log-softmax over K).  Mass outside the top-K
    is discarded, not spread.
    """
    return F.log_softmax(stored.to(dtype) / T, dim=-1)


def _kl_rows(inp_logp: torch.Tensor, tgt_logp: torch.Tensor) -> torch.Tensor:
    """`custom_kl_div(per_token=True)` -- utils/finetuning_utils.py:49-56."""
    return F.kl_div(inp_logp, tgt_logp, reduction="none", log_target=True).sum(dim=-1)


def fwd_kl_topk_rows(z: torch.Tensor, t_logp: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """KL(teacher || student) per token on the teacher's support.

    utils/finetuning_utils.py:104.  `z` are the scaled student logits [N,V],
    `t_logp` the renormalised teacher log-probs [N,K].
    """
    return _kl_rows(student_logprobs_on_support(z, idx), t_logp)


def rev_kl_topk_rows(z: torch.Tensor, t_logp: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """KL(student restricted+renormalised to the support || teacher) per token.

    utils/finetuning_utils.py:105: the gathered student log-probs go through a
    second log-softmax over K before the divergence.
    """
    s_sup = F.log_softmax(student_logprobs_on_support(z, idx), dim=-1)
    return _kl_rows(t_logp, s_sup)


# ---------------------------------------------------------------------------
# dense teacher (full-vocabulary) divergences
# ---------------------------------------------------------------------------

def fwd_kl_dense_rows(z: torch.Tensor, t_logits: torch.Tensor) -> torch.Tensor:
    """KL(teacher || student) with a dense teacher.

    Formula of utils/finetuning_utils.py:49-56,94,104 with K = V.  Teacher
    entries of zero mass (logit -inf) contribute 0 (0 log 0 = 0); the
    reference's `F.kl_div(log_target=True)` would give NaN there, and its
    training side never runs dense, so that convention is this build's.
    """
    s = F.log_softmax(z, dim=-1)
    t = F.log_softmax(t_logits, dim=-1)
    zero = torch.isneginf(t)
    t_safe = torch.where(zero, torch.zeros_like(t), t)
    term = torch.exp(t_safe) * (t_safe - s)
    return torch.where(zero, torch.zeros_like(term), term).sum(dim=-1)


def rev_kl_dense_rows(z: torch.Tensor, t_logits: torch.Tensor) -> torch.Tensor:
    """Reverse KL with a dense teacher, on the teacher's support.

    utils/finetuning_utils.py:105 with the support = {j : teacher mass > 0}:
    the student is renormalised over the support exactly as the reference
    renormalises it over the top-K ids, so a teacher with exact zeros (as a
    byte-trie marginal has) stays finite.  With a strictly positive teacher
    this is the textbook KL(student || teacher).
    """
    t = F.log_softmax(t_logits, dim=-1)
    sup = ~torch.isneginf(t)
    s_sup = F.log_softmax(z.masked_fill(~sup, NEG_INF), dim=-1)
    sup = sup & ~torch.isneginf(s_sup)       # a masked student entry (-inf) carries no student mass: 0 log 0 = 0
    # off the support both operands are replaced by finite stand-ins before the product, so that
    # autograd does not turn 0 * inf into NaN gradients
    s_safe = torch.where(sup, s_sup, torch.zeros_like(s_sup))
    t_safe = torch.where(sup, t, torch.zeros_like(t))
    term = torch.exp(s_safe) * (s_safe - t_safe)
    return torch.where(sup, term, torch.zeros_like(term)).sum(dim=-1)


def jsd_dense_rows(z: torch.Tensor, t_logits: torch.Tensor) -> torch.Tensor:
    """Jensen-Shannon divergence 0.5 KL(P||M) + 0.5 KL(Q||M), M = (P+Q)/2.

    Not in the reference (parity unpinned): textbook definition, natural log,
    P = softmax(student), Q = softmax(teacher).
    """
    s = F.log_softmax(z, dim=-1)
    t = F.log_softmax(t_logits, dim=-1)
    p, q = torch.exp(s), torch.exp(t)
    m = 0.5 * (p + q)
    logm = torch.log(m)
    a = torch.where(p > 0, p * (s - logm), torch.zeros_like(p))
    b = torch.where(q > 0, q * (t - logm), torch.zeros_like(q))
    return 0.5 * (a.sum(dim=-1) + b.sum(dim=-1))


DENSE_ROWS = {"fkl": fwd_kl_dense_rows, "rkl": rev_kl_dense_rows, "jsd": jsd_dense_rows}
TOPK_ROWS = {"fkl": fwd_kl_topk_rows, "rkl": rev_kl_topk_rows}


def mean_loss_and_grad(kind: str, logits: torch.Tensor, T: float, *,
                       t_vals: torch.Tensor | None = None, t_idx: torch.Tensor | None = None,
                       t_logits: torch.Tensor | None = None, t_T: float | None = None,
                       valid: torch.Tensor | None = None, dtype=torch.float32):
    """Mean-over-valid-tokens loss and d(loss)/d(logits), the op sequence of the
    reference: cast -> /T -> log_softmax -> gather -> kl_div -> per-token sum
    -> mean -> backward (classes/student/model.py:408,420-425,441 with
    utils/finetuning_utils.py:88-105).

    `logits` [R,V] in its storage dtype; rows with `valid == False` are removed
    before the loss (the reference index_selects content rows) and get a zero
    gradient.  Top-K teacher: `t_vals` [Nv,K] stored log-probs, `t_idx` [Nv,K].
    Dense teacher: `t_logits` [Nv,Vt==V].  Returns (loss, rows[Nv], grad[R,V]
    in the compute dtype, i.e. before the cast back to the storage dtype of `logits`).
    """
    R = logits.shape[0]
    if valid is None:
        valid = torch.ones(R, dtype=torch.bool)
    sel = torch.nonzero(valid).squeeze(-1)
    leaf = logits.detach().to(dtype).requires_grad_(True)      # the `.float()` of the caller
    z = torch.index_select(leaf, 0, sel) / T
    if t_T is None:
        t_T = T
    if t_logits is not None:
        rows = DENSE_ROWS[kind](z, t_logits.to(dtype) / t_T)
    else:
        rows = TOPK_ROWS[kind](z, teacher_logprobs_topk(t_vals, t_T, dtype), t_idx)
    loss = rows.mean()
    loss.backward()
    return loss.detach(), rows.detach(), leaf.grad.detach()


F32_HALF_ULP = 2.0 ** -24


def storage_tolerance(ref: torch.Tensor, storage_dtype, rtol: float, terms: torch.Tensor | None = None) -> torch.Tensor:
    """Element-wise bound for comparing a gradient stored in `storage_dtype` with an
    unrounded float64 reference: `rtol` on the entry's own value plus the half-ulp the
    round-to-nearest store may add (bf16 2^-8, fp16 2^-11 relative; fp16 also its subnormal
    spacing), plus `terms`: an absolute, per-entry bound on what fp32 evaluation loses where
    the entry is a difference of larger quantities (built by the helpers below from the
    entry's own operands).  Nothing in the bound depends on other entries' size: an entry
    that is 1e-6 of the tensor's largest is still held to `rtol` of itself."""
    half_ulp = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[storage_dtype]
    floor = {torch.float32: 1e-30, torch.bfloat16: 1e-30, torch.float16: 2.0 ** -25}[storage_dtype]
    bound = ref.abs() * (rtol + half_ulp) + floor
    return bound if terms is None else bound + terms


def softmax_rounding(z: torch.Tensor) -> torch.Tensor:
    """Relative error that fp32 evaluation leaves on the entries of softmax(z), `z` [n, V] the scaled
    logits in float64.  The exponent z_j - max is a difference of fp32 numbers of size |z_j| and |max|,
    each rounded to half an ulp, and an absolute error of the exponent is a relative error of the
    exponential; the exponential, the row sum, its reciprocal and the product add about eight more
    half-ulps.  (The reference's own fp32 log-softmax carries the same.)"""
    zmax = z.max(-1, keepdim=True).values
    mag = torch.nan_to_num(z.abs(), posinf=0.0) + zmax.abs()
    return F32_HALF_ULP * (8.0 + mag)


def _support_sum(idx: torch.Tensor, vals: torch.Tensor, V: int) -> torch.Tensor:
    """[n, V] with vals[i, k] summed at column idx[i, k]; ids outside [0, V) are ignored."""
    ok = (idx >= 0) & (idx < V)
    out = torch.zeros(idx.shape[0], V, dtype=vals.dtype)
    out.scatter_add_(1, torch.where(ok, idx, torch.zeros_like(idx)).long(), torch.where(ok, vals, torch.zeros_like(vals)))
    return out


def sparse_gradient_tolerance(grad64: torch.Tensor, logits: torch.Tensor, T: float, idx: torch.Tensor, storage_dtype,
                              rtol: float, support_scale: float = 0.0, row_coef=None) -> torch.Tensor:
    """Element-wise bound for a gradient of the form g_ij = a_i softmax(z_i)_j + c_ij with c_i zero off the
    K ids of row i (forward KL on a sparse teacher: a_i = scale / T, c_ik = -q_ik scale / T; the alpha-weighted
    composite: a_i, c_ik its row coefficients).  `grad64`, `logits` [n, V] (rows already selected),
    `idx` [n, K] (ids outside [0, V) ignored), `T` the student temperature.

    a_i is `row_coef` where the caller knows it (a number or [n, 1]), else read off the float64 gradient on the
    columns outside the support; c_ij = g_ij - a_i p_ij on the support.
    The bound is `storage_tolerance` of the entry itself plus, per entry,
      |a_i| p_ij softmax_rounding(z)_ij          the dense term as fp32 computes it,
      |c_ij| 2^-24 (8 + 32)                      the sparse term: a teacher mass exp(t - lse_K) from stored
                                                 log-probs of magnitude up to 32, rounded like the softmax,
      |a_i| 2^-40 max_j p_ij  (16-bit rows)      the kernel keeps 2^(z_j - max) of a 16-bit row between its sum
                                                 and gradient sweeps as fp16 scaled by 2^15: 11 bits (inside
                                                 `rtol`) down to 2^-29 of the row's largest probability, below
                                                 that fp16's subnormal spacing, 2^-39 of the largest,
    so off the support an entry is held to `rtol` (+ half an ulp of the store) of itself, and on the support to
    that plus fp32 rounding of its two cancelling terms.  `support_scale` > 0 adds, on the support only,
    that fraction of the row's largest coefficient max(|a_i|, max_k |c_ik|): for gradients whose sparse term is
    itself a sum of cancelling pieces the float64 gradient does not show (the composite's reverse-KL and
    cross-entropy parts)."""
    z = logits.double() / T
    p = torch.softmax(z, -1)
    n, V = p.shape
    on = _support_sum(idx.long(), torch.ones(idx.shape, dtype=torch.float64), V) > 0
    off_mass = torch.where(on, torch.zeros_like(p), p).sum(-1, keepdim=True)
    off_grad = torch.where(on, torch.zeros_like(p), grad64).sum(-1, keepdim=True)
    if row_coef is not None:
        a = torch.as_tensor(row_coef, dtype=torch.float64) * torch.ones(n, 1, dtype=torch.float64)
    else:
        # rows whose whole vocabulary is support have nothing to read a_i from and take their largest entry as the scale
        a = torch.where(off_mass > 1e-12, off_grad / off_mass.clamp_min(1e-300), grad64.abs().max(-1, keepdim=True).values)
    c = torch.where(on, grad64 - a * p, torch.zeros_like(p))
    terms = a.abs() * p * softmax_rounding(z) + c.abs() * (F32_HALF_ULP * 40.0)
    if storage_dtype != torch.float32:
        terms = terms + a.abs() * p.max(-1, keepdim=True).values * 2.0 ** -40
    if support_scale:
        row_scale = torch.maximum(a.abs(), c.abs().max(-1, keepdim=True).values)
        terms = terms + on * (support_scale * row_scale)
    return storage_tolerance(grad64, storage_dtype, rtol, terms)


def rkl_topk_gradient_tolerance(grad64: torch.Tensor, logits: torch.Tensor, t_vals: torch.Tensor, t_idx: torch.Tensor,
                                T: float, t_T: float, scale: float, storage_dtype, rtol: float) -> torch.Tensor:
    """Element-wise bound for the reverse-KL gradient on a sparse teacher,
    g_ij = sum_{k: idx_ik = j} r_k ((s'_k - t_k) - rkl_i) scale / T (utils/finetuning_utils.py:105): zero off the
    support (exactly in the kernel, to float64 rounding in the reference); on it `storage_tolerance` plus fp32 rounding of the pieces the bracket is a difference of:
    r_k to `softmax_rounding`, s'_k and t_k (log-softmaxes over K) to half-ulps of their operands, rkl_i to the
    r-weighted sum of those."""
    n, V = logits.shape
    idx = t_idx.long()
    ok = (idx >= 0) & (idx < V)
    z = torch.gather(logits.double() / T, 1, torch.where(ok, idx, torch.zeros_like(idx)))
    z = z.masked_fill(~ok, NEG_INF)
    t_in = (t_vals.double() / t_T).masked_fill(~ok, NEG_INF)
    live = ok & ~torch.isneginf(t_in)
    z = z.masked_fill(~live, NEG_INF)
    s = F.log_softmax(z, -1)
    t = F.log_softmax(t_in, -1)
    r = torch.exp(s)
    diff = torch.where(live, s - t, torch.zeros_like(s))
    rkl = (r * diff).sum(-1, keepdim=True)
    e_r = torch.where(live, softmax_rounding(z), torch.zeros_like(z))
    tmax = t_in.max(-1, keepdim=True).values
    d_diff = e_r + F32_HALF_ULP * (8.0 + torch.nan_to_num(t_in.abs(), posinf=0.0) + tmax.abs())
    d_rkl = (r * (d_diff + e_r * diff.abs())).sum(-1, keepdim=True)
    per_entry = r * (e_r * (diff.abs() + rkl.abs()) + d_diff + d_rkl) * (abs(scale) / T)
    terms = _support_sum(idx, torch.where(live, per_entry, torch.zeros_like(per_entry)), V)
    # the float64 reference itself: its backward through the full-vocabulary log-softmax leaves
    # softmax_j * (sum_k g_k), a sum that is zero only up to float64 rounding, on every column
    pieces = (r * (diff.abs() + rkl.abs())).sum(-1, keepdim=True) * (abs(scale) / T)
    terms = terms + torch.softmax(logits.double() / T, -1) * pieces * 2.0 ** -46
    return storage_tolerance(grad64, storage_dtype, rtol, terms)


def composite_gradient_tolerance(gref: torch.Tensor, logits: torch.Tensor, T: float, storage_dtype, rtol: float, rows,
                                 idx: torch.Tensor, crop: int | None = None) -> torch.Tensor:
    """Entry-by-entry bound for the gradient of the alpha-weighted composite (utils/finetuning_utils.py:107-110) over
    one sequence of logits: `gref`, `logits` [S, Vm]; `rows` the content rows (None: all), `idx` [N, K] their teacher
    ids, `crop` the vocabulary in use.  Every entry is a_i softmax_j + (K sparse corrections): `rtol` of the entry
    itself, the store's half ulp, fp32 rounding of the entry's two parts, and on the K support columns 4e-6 of the
    row's largest coefficient (the correction there is a sum of forward-KL, reverse-KL and cross-entropy pieces that
    cancel).  Rows outside `rows`, rows beyond the teacher's and columns beyond `crop` must be exactly zero."""
    bound = storage_tolerance(gref, storage_dtype, rtol)
    rows = torch.arange(gref.shape[0]) if rows is None else rows
    n = min(len(rows), len(idx))
    crop = gref.shape[1] if crop is None else crop
    r = rows[:n].long()
    bound[r, :crop] = sparse_gradient_tolerance(gref[r, :crop].double(), logits[r, :crop], T, idx[:n].long(), storage_dtype,
                                                rtol, support_scale=4e-6)
    return bound


def topk_gradient_tolerance(kind: str, grad64: torch.Tensor, logits: torch.Tensor, t_vals: torch.Tensor, t_idx: torch.Tensor,
                            T: float, t_T: float | None, scale: float, storage_dtype, rtol: float,
                            valid: torch.Tensor | None = None) -> torch.Tensor:
    """The bound of `sparse_gradient_tolerance` (forward KL) or `rkl_topk_gradient_tolerance` (reverse KL) for
    the arguments of `mean_loss_and_grad`: `grad64`, `logits` [R, V]; teacher rows for the valid rows only; rows
    with `valid == False` must be exactly zero."""
    bound = storage_tolerance(grad64, storage_dtype, rtol)
    sel = torch.arange(logits.shape[0]) if valid is None else torch.nonzero(valid).squeeze(-1)
    if kind == "fkl":
        bound[sel] = sparse_gradient_tolerance(grad64[sel], logits[sel], T, t_idx, storage_dtype, rtol, row_coef=scale / T)
    else:
        bound[sel] = rkl_topk_gradient_tolerance(grad64[sel], logits[sel], t_vals, t_idx, T, T if t_T is None else t_T,
                                                 scale, storage_dtype, rtol)
    return bound


def dense_gradient_tolerance(grad64: torch.Tensor, logits: torch.Tensor, t_logits: torch.Tensor, rows64: torch.Tensor,
                             T: float, t_T: float, scale: float, storage_dtype, rtol: float, stash: bool = False,
                             kind: str = "fkl") -> torch.Tensor:
    """Element-wise bound for the gradient of a dense-teacher divergence, rows already selected
    (`logits`, `t_logits`, `grad64` [n, V]; `rows64` [n] the per-row losses; `scale` the factor the
    gradient carries, e.g. 1 / n_valid).  `storage_tolerance` of the entry itself plus fp32 rounding of the
    terms the entry is a difference of, (p_j + q_j)(1 + |log p_j / q_j| + loss_i) scale / T: 4e-6 of them (the
    logarithms, the row sums and the loss each carry a few half-ulps, and where the terms cancel the result
    keeps that much of the TERMS -- the reference's fp32 evaluation as well) plus `softmax_rounding` of the two
    rows (logits of large magnitude lose absolute precision in the exponent).  `kind` "rkl": p is the student
    renormalised over the teacher's support.  `stash`: the fused
    marginal kernel keeps 2^(z_j - max) of a 16-bit student row between its passes as fp16 scaled by 2^15, which
    below 2^-29 of the row's largest logit's weight resolves 2^-40 exp(max - z_j) of the entry."""
    zs, zt = logits.double() / T, t_logits.double() / t_T
    lq = torch.log_softmax(zt, -1)
    zs_all = zs
    if kind == "rkl":      # the student renormalised over the teacher's support, as `rev_kl_dense_rows` takes it
        zs = zs.masked_fill(torch.isneginf(lq), NEG_INF)
    lp = torch.log_softmax(zs, -1)
    ratio = torch.nan_to_num((lp - lq).abs(), nan=0.0, posinf=0.0)
    terms = (lp.exp() + lq.exp()) * (1 + ratio + rows64.unsqueeze(-1)) * (abs(scale) / T)
    terms = terms * (4e-6 + softmax_rounding(zs) + softmax_rounding(zt))
    if stash:
        # the teacher row is the logarithm of a marginal that the kernel sums in fp32 (a few dozen terms per
        # student id) and takes through the hardware logarithm (an ulp of |log2 m|), divided by T_t
        eps_t = F32_HALF_ULP * (4.0 * torch.nan_to_num(zt.abs(), posinf=0.0) + 64.0 / t_T)
        terms = terms + (lp.exp() + lq.exp()) * eps_t * (abs(scale) / T)
    if stash and storage_dtype != torch.float32:
        gap = torch.nan_to_num(zs_all.max(-1, keepdim=True).values - zs_all, posinf=0.0)     # from the row's largest logit, on the support or off it
        terms = terms + grad64.abs() * 2.0 ** -40 * torch.exp(gap.clamp_max(600.0))
    return storage_tolerance(grad64, storage_dtype, rtol, terms)


def marginal_rkl_gradient_tolerance(grad64: torch.Tensor, logits: torch.Tensor, t_logits: torch.Tensor, rows64: torch.Tensor,
                                    T: float, t_T: float, scale: float, storage_dtype, rtol: float) -> torch.Tensor:
    """`dense_gradient_tolerance` for the fused marginal + reverse-KL kernel (which stashes, see there)."""
    return dense_gradient_tolerance(grad64, logits, t_logits, rows64, T, t_T, scale, storage_dtype, rtol, stash=True, kind="rkl")


# ---------------------------------------------------------------------------
# a5, a6 -- top-K cross entropy, alpha-weighted composite, the 9-key dict
# ---------------------------------------------------------------------------

def topk_cross_entropy(logprobs: torch.Tensor, labels: torch.Tensor, idx: torch.Tensor,
                       ignore_rows: torch.Tensor) -> torch.Tensor:
    """Negative log-prob of the label where the label is among the row's ids.

    utils/finetuning_utils.py:68-84.  The last row is cropped iff there are
    fewer labels than rows; rows listed in `ignore_rows` and rows whose label
    is not among their K ids count as invalid and receive the mean of the
    valid rows.  With as many labels as rows the crop is `[:0]`, an empty
    slice, and the comparison raises exactly as the reference does.
    """
    n_rows = logprobs.size(0)
    stop = -1 if labels.size(-1) < n_rows else 0
    hit = labels.unsqueeze(-1) == idx[:stop]
    hit[ignore_rows] = False
    valid = hit.any(dim=-1)
    # the reference allocates float32 here; the float64 "truth" variant keeps its precision
    picked = torch.zeros_like(valid, dtype=torch.float64 if logprobs.dtype == torch.float64 else torch.float32)
    picked[valid] = logprobs[:stop][hit].squeeze(-1)
    picked[~valid] = picked[valid].mean()
    return -picked


def alpha_weighted(per_token: torch.Tensor, alpha, ce_per_token: torch.Tensor) -> torch.Tensor:
    """mean(kl * ((kl / max(kl) + 1)^alpha + ce)); utils/finetuning_utils.py:58-66.

    The cross-entropy vector is extended by a single zero when shorter; the
    maximum is part of the autograd graph (not detached).
    """
    if ce_per_token.numel() < per_token.numel():
        ce_per_token = torch.cat((ce_per_token, torch.zeros(1, device=ce_per_token.device, dtype=ce_per_token.dtype)))
    w = (per_token / per_token.max() + 1).pow(alpha) + ce_per_token
    return (per_token * w).mean()


LOSS_KEYS = ("train_loss", "custom loss", "CE loss", "kl_div", "reverse kl_div",
             "weighted kl_div", "weighted rev. kl_div", "teacher CE loss", "CE diff")


def calculate_divergence(student_logits: torch.Tensor, teacher_logits: torch.Tensor,
                         indices: torch.Tensor | None, convo_CE_tokens: torch.Tensor,
                         alpha, avoid_indices: torch.Tensor) -> dict[str, torch.Tensor]:
    """The reference's per-conversation loss, utils/finetuning_utils.py:47-124.

    Inputs as the caller provides them (classes/student/model.py:420-425):
    student logits [N,V] already cast to fp32 and divided by T, teacher stored
    log-probs [N,K] already divided by T, ids [N,K], labels [N-1], ignore rows.
    """
    n = min(student_logits.size(0), teacher_logits.size(0),
            indices.size(0) if indices is not None else student_logits.size(0))
    s = F.log_softmax(student_logits[:n], dim=-1)
    t = F.log_softmax(teacher_logits[:n], dim=-1)
    if indices is not None:
        s = torch.gather(s, 1, indices[:n])
    labels = convo_CE_tokens[:n]
    ce_s = topk_cross_entropy(s, labels, indices, avoid_indices)
    ce_t = topk_cross_entropy(t, labels, indices, avoid_indices)
    ce_diff = ce_s - ce_t
    ce_pos = torch.where(ce_diff < 0, torch.zeros_like(ce_diff), ce_diff)
    kl = _kl_rows(s, t)
    rkl = _kl_rows(t, F.log_softmax(s, dim=-1))
    wkl = alpha_weighted(kl, alpha, ce_pos)
    wrkl = alpha_weighted(rkl, alpha, ce_pos)
    total = (wkl + wrkl) / 2
    return dict(zip(LOSS_KEYS, (total, total, ce_s.mean(), kl.mean(), rkl.mean(), wkl, wrkl,
                                ce_t.mean(), ce_diff.mean())))


# ---------------------------------------------------------------------------
# a9 -- teacher producer
# ---------------------------------------------------------------------------

def teacher_topk_producer(logits: torch.Tensor, crop: int, K: int):
    """Full-vocabulary log-softmax then the K largest entries per row.

    classes/teacher/inference_worker.py:73-80: values fp32 in descending order
    and int64 ids.  Temperature is NOT applied at collection time.
    """
    logp = F.log_softmax(logits[..., :crop].float(), dim=-1)
    return torch.topk(logp, K, dim=-1)


def to_storage(vals: torch.Tensor, idx: torch.Tensor):
    """fp16 log-probs + uint32 ids as written to disk, classes/data_manager.py:306,312."""
    return vals.to(torch.float16), idx.to(torch.int64).numpy().astype(np.uint32)


def from_storage(vals16, idx_u32):
    """fp32 / int64 as loaded for training, classes/data_manager.py:323-324."""
    return torch.as_tensor(np.asarray(vals16, dtype=np.float32)), \
        torch.as_tensor(np.asarray(idx_u32, dtype=np.int64))


# ---------------------------------------------------------------------------
# a7 -- pairwise multi-teacher merge as the dataset manager performs it
# ---------------------------------------------------------------------------

def merge_topk_pair(disk_logp: np.ndarray, new_logp: np.ndarray, disk_idx: np.ndarray,
                    new_idx: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Sum two top-K teachers in probability space and keep the K largest.

    classes/data_manager.py:210-246,249-261: exp -> per row concat + unique
    (sorted) + index_add -> topk(K) -> log.  Rows beyond the shorter input pass
    through unmerged.  Result is unnormalised (sums to about the number of
    teachers) and in descending-probability order.  Ties: the reference leaves
    them to `torch.topk`; here the smaller id wins (stable sort).
    """
    a = torch.as_tensor(np.exp(np.asarray(disk_logp, dtype=np.float32)))
    b = torch.as_tensor(np.exp(np.asarray(new_logp, dtype=np.float32)))
    ia = torch.as_tensor(np.asarray(disk_idx, dtype=np.int64))
    ib = torch.as_tensor(np.asarray(new_idx, dtype=np.int64))
    n = min(a.size(0), b.size(0))
    K = a.size(-1)
    rest_v, rest_i = (a[n:], ia[n:]) if a.size(0) > n else (b[n:], ib[n:])
    out_v = torch.zeros((n, K), dtype=torch.float32)
    out_i = torch.zeros((n, K), dtype=torch.int64)
    for r in range(n):
        ids, inv = torch.unique(torch.cat((ia[r], ib[r])), return_inverse=True)
        mass = torch.zeros(ids.numel(), dtype=torch.float32)
        mass.index_add_(0, inv, torch.cat((a[r], b[r])))
        order = torch.sort(mass, descending=True, stable=True).indices[:K]
        out_v[r] = mass[order]
        out_i[r] = ids[order]
    out_v = torch.cat((out_v, rest_v))
    out_i = torch.cat((out_i, rest_i))
    return np.log(out_v.numpy()), out_i.numpy()


def merge_dense_pair(disk_logp: np.ndarray, new_logp: np.ndarray) -> np.ndarray:
    """Dense merge: exp, zero-pad the shorter one, add, log.

    classes/data_manager.py:200-208,249-261.
    """
    a = np.exp(np.asarray(disk_logp, dtype=np.float32))
    b = np.exp(np.asarray(new_logp, dtype=np.float32))
    n = max(a.shape[0], b.shape[0])
    a = np.pad(a, ((0, n - a.shape[0]), (0, 0)))
    b = np.pad(b, ((0, n - b.shape[0]), (0, 0)))
    with np.errstate(divide="ignore"):
        return np.log(a + b)


# ---------------------------------------------------------------------------
# a10 -- weighted multi-teacher merge + vocabulary remap (no reference function)
# ---------------------------------------------------------------------------

def merge_remap_rows(vals: Sequence[np.ndarray], idxs: Sequence[np.ndarray],
                     weights: Sequence[float], id_map: np.ndarray | None,
                     T: float = 1.0, n_student: int | None = None):
    """Weighted sum of several top-K teachers after mapping their ids.

    Parity unpinned (no reference counterpart; generalises
    classes/data_manager.py:231-240 with weights and an id map).  Per row:
    mass_e = w_teacher * exp(logp_e) in fp32; the id goes through `id_map`
    (teacher id -> student id, -1 = dropped, its mass is removed; ids outside
    the map, and student ids outside [0, n_student) when that is given, are
    dropped as well); entries that
    land on the same student id are summed in entry order (teacher 0's entries
    first); the surviving ids are listed in ascending order; the teacher
    distribution is log_softmax(log(mass) / T) over the survivors.

    Returns a list (one item per row) of (ids int32[n_r], mass fp32[n_r],
    logq fp64[n_r]).  A row with no survivor yields empty arrays.
    """
    n_rows = vals[0].shape[0]
    out = []
    for r in range(n_rows):
        acc: dict[int, np.float32] = {}
        for v, ix, w in zip(vals, idxs, weights):
            m = (np.float32(w) * np.exp(np.asarray(v[r], dtype=np.float32))).astype(np.float32)
            for e in range(m.shape[0]):
                tid = int(ix[r][e])
                if id_map is None:
                    sid = tid
                else:
                    sid = int(id_map[tid]) if 0 <= tid < len(id_map) else -1      # outside the teacher vocabulary: dropped
                if sid < 0 or (n_student is not None and sid >= n_student):
                    continue
                acc[sid] = np.float32(acc.get(sid, np.float32(0.0)) + m[e])
        ids = np.asarray(sorted(acc), dtype=np.int32)
        mass = np.asarray([acc[i] for i in ids], dtype=np.float32)
        if ids.size:
            with np.errstate(divide="ignore"):                    # an id all of whose entries carry zero mass: log 0 = -inf
                lg = np.log(mass.astype(np.float64)) / T
            if np.isfinite(lg.max()):                             # all mass zero (a teacher of weight 0 alone): stays -inf
                lg = lg - (lg.max() + math.log(np.exp(lg - lg.max()).sum()))
        else:
            lg = np.zeros(0, dtype=np.float64)
        out.append((ids, mass, lg))
    return out


def merge_remap_padded(vals, idxs, weights, id_map, T: float = 1.0, n_student: int | None = None):
    """`merge_remap_rows` packed into padded arrays: ids int32 [N,E] (pad -1),
    logq fp32 [N,E] (pad -inf), count int32 [N]; E = total entries per row."""
    rows = merge_remap_rows(vals, idxs, weights, id_map, T, n_student)
    E = sum(v.shape[1] for v in vals)
    N = len(rows)
    ids = np.full((N, E), -1, dtype=np.int32)
    lq = np.full((N, E), -np.inf, dtype=np.float32)
    cnt = np.zeros(N, dtype=np.int32)
    for r, (i, _, l) in enumerate(rows):
        ids[r, :i.size] = i
        lq[r, :i.size] = l
        cnt[r] = i.size
    return ids, lq, cnt


def fwd_kl_sparse_rows(z: torch.Tensor, ids: np.ndarray, logq: np.ndarray, cnt: np.ndarray):
    """Forward KL against an already-normalised ragged sparse teacher
    (utils/finetuning_utils.py:92,104 with a per-row entry count).  An entry of zero mass
    (log-probability -inf: a merged id all of whose teachers carry weight 0) contributes 0,
    the convention of this build for forward KL (the library routine would give 0 * inf = NaN)."""
    s = F.log_softmax(z, dim=-1)
    rows = []
    for r in range(z.shape[0]):
        n = int(cnt[r])
        if n == 0:
            rows.append(z.new_zeros(()))
            continue
        sk = s[r, torch.as_tensor(ids[r, :n].astype(np.int64))]
        t = torch.as_tensor(logq[r, :n]).to(z.dtype)
        live = ~torch.isneginf(t)
        rows.append((torch.exp(t[live]) * (t[live] - sk[live])).sum())
    return torch.stack(rows)


# ---------------------------------------------------------------------------
# a11 -- byte-trie longest-prefix map, CSR, marginalisation (no reference function)
# ---------------------------------------------------------------------------

def trie_map_bruteforce(student_vocab: Sequence[bytes], teacher_vocab: Sequence[bytes],
                        byte_fallback: Sequence[int] | None = None) -> np.ndarray:
    """Teacher token -> the student token that is the longest prefix of its bytes.

    Parity unpinned (no reference counterpart).  Brute force with a dict,
    scanning prefixes longest to shortest.  Duplicate student strings: the
    smallest id owns the string.  No student token is a prefix: the
    `byte_fallback[first byte]` id if given and >= 0, else -1.  Empty teacher
    strings map to -1.
    """
    owner: dict[bytes, int] = {}
    for i, b in enumerate(student_vocab):
        if len(b) and b not in owner:
            owner[b] = i
    longest = max((len(b) for b in student_vocab), default=0)
    out = np.full(len(teacher_vocab), -1, dtype=np.int32)
    for t, b in enumerate(teacher_vocab):
        if not len(b):
            continue
        for L in range(min(len(b), longest), 0, -1):
            hit = owner.get(bytes(b[:L]))
            if hit is not None:
                out[t] = hit
                break
        else:
            if byte_fallback is not None and byte_fallback[b[0]] >= 0:
                out[t] = byte_fallback[b[0]]
    return out


def csr_from_map(t2s: np.ndarray, n_student: int) -> tuple[np.ndarray, np.ndarray]:
    """Group teacher ids by student id: offsets int32 [Vs+1], indices int32
    [#mapped], teacher ids ascending inside a segment; ids mapped to -1 are
    left out."""
    offsets = np.zeros(n_student + 1, dtype=np.int32)
    segs: list[list[int]] = [[] for _ in range(n_student)]
    for t, s in enumerate(t2s):
        if s >= 0:
            segs[int(s)].append(t)
    flat: list[int] = []
    for s in range(n_student):
        flat.extend(segs[s])
        offsets[s + 1] = len(flat)
    return offsets, np.asarray(flat, dtype=np.int32)


def marginalise_csr(p_teacher: np.ndarray, offsets: np.ndarray, indices: np.ndarray,
                    dtype=np.float64) -> np.ndarray:
    """marg[r, s] = sum of p_teacher[r, t] over the teacher ids t of segment s."""
    p = np.asarray(p_teacher, dtype=dtype)
    out = np.zeros((p.shape[0], offsets.shape[0] - 1), dtype=dtype)
    for s in range(offsets.shape[0] - 1):
        a, b = int(offsets[s]), int(offsets[s + 1])
        if b > a:
            out[:, s] = p[:, indices[a:b]].sum(axis=1)
    return out


def marginalise_map(p_teacher: np.ndarray, t2s: np.ndarray, n_student: int,
                    dtype=np.float64) -> np.ndarray:
    """The same marginal computed by scattering along the teacher->student map."""
    p = np.asarray(p_teacher, dtype=dtype)
    out = np.zeros((p.shape[0], n_student), dtype=dtype)
    keep = t2s >= 0
    np.add.at(out, (slice(None), t2s[keep]), p[:, keep])
    return out


def marginal_to_teacher_logits(marg: torch.Tensor) -> torch.Tensor:
    """log of the marginal (zero mass -> -inf), the 'stored log-prob' a dense
    teacher row would hold; temperature is applied afterwards as in
    classes/student/model.py:421."""
    return torch.log(marg)

"""Cross-tokenizer vocabulary tables and marginalisation.

The reference's `utils/vocab_utils.py` only names tokenizer families and rejects distillation
across vocabularies (collect_and_finetune.py:83-101); this module supplies what that case needs:
a byte-trie longest-prefix map from teacher tokens to student tokens, its CSR form, the
marginalisation of a dense teacher distribution into the student vocabulary, and the reverse KL
against it.  The table builders are host C++ (libdistill_hip.so, no GPU needed); the
marginalisation and the loss are HIP kernels.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import numpy as np
import torch

from . import _lib
from .ops import _DT, _dev, _grad_target, _opt_i32, _rows_2d, _stream_ptr


def _pack(vocab: Sequence[bytes]):
    lens = np.fromiter((len(b) for b in vocab), dtype=np.int64, count=len(vocab))
    offsets = np.zeros(len(vocab) + 1, dtype=np.int64)
    np.cumsum(lens, out=offsets[1:])
    blob = np.frombuffer(b"".join(bytes(b) for b in vocab), dtype=np.uint8) if offsets[-1] else np.zeros(1, np.uint8)
    return np.ascontiguousarray(blob), offsets


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def longest_prefix_map(student_vocab: Sequence[bytes], teacher_vocab: Sequence[bytes],
                       byte_fallback: Sequence[int] | None = None) -> np.ndarray:
    """int32 [len(teacher_vocab)]: for every teacher token the id of the student token whose bytes
    are the longest prefix of the teacher token's bytes; `byte_fallback[first byte]` (256 ids, -1 =
    none) when no student token is a prefix; -1 otherwise."""
    sb, so = _pack(student_vocab)
    tb, to = _pack(teacher_vocab)
    fb = None
    if byte_fallback is not None:
        fb = np.ascontiguousarray(np.asarray(byte_fallback, dtype=np.int32))
        if fb.shape != (256,):
            raise ValueError("byte_fallback must hold 256 ids")
    out = np.empty(len(teacher_vocab), dtype=np.int32)
    st = _lib.load().dl_trie_longest_prefix_map(_p(sb), _p(so), len(student_vocab), _p(tb), _p(to), len(teacher_vocab),
                                                _p(fb) if fb is not None else None, _p(out))
    _lib.check(st, "dl_trie_longest_prefix_map")
    return out


def csr_from_map(t2s: np.ndarray, n_student: int) -> tuple[np.ndarray, np.ndarray]:
    """(offsets int32 [n_student + 1], indices int32 [#mapped]): teacher ids grouped by student id,
    ascending inside a group; ids mapped to -1 are left out."""
    t2s = np.ascontiguousarray(np.asarray(t2s, dtype=np.int32))
    offsets = np.empty(n_student + 1, dtype=np.int32)
    indices = np.empty(max(t2s.size, 1), dtype=np.int32)
    n = ctypes.c_int64(0)
    st = _lib.load().dl_csr_from_map(_p(t2s), t2s.size, n_student, _p(offsets), _p(indices), ctypes.byref(n))
    _lib.check(st, "dl_csr_from_map")
    return offsets, indices[:n.value].copy()


class _PlanArrays:
    """Device copies of what dl_marginal_plan_build lays out for one map: list offsets, entries, fold table."""

    def __init__(self, row_off, ent, fold, tile: int, n_fold: int, n_extra: int, device):
        self.tile, self.n_fold, self.n_extra = tile, n_fold, n_extra
        self.row_off = torch.as_tensor(row_off, device=device)
        self.ent = torch.as_tensor(ent.view(np.int32), device=device)     # same bits; torch has no uint32 arithmetic need
        self.fold = torch.as_tensor(fold, device=device)

    def args(self):
        """(row_off, ent, tile, fold, n_fold, n_extra) as the C ABI takes them."""
        return self.row_off.data_ptr(), self.ent.data_ptr(), self.tile, self.fold.data_ptr(), self.n_fold, self.n_extra


def _build_plan(t2s: np.ndarray, n_student: int, device) -> "_PlanArrays | None":
    """dl_marginal_plan_build for `t2s` onto `n_student` ids; None where the library says too wide."""
    lib = _lib.load()
    tile, rows, n_fold, n_extra = ctypes.c_int(0), ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_int(0)
    st = lib.dl_marginal_plan_build(_p(t2s), t2s.size, n_student, ctypes.byref(tile), None, None, 0, ctypes.byref(rows),
                                    None, 0, ctypes.byref(n_fold), ctypes.byref(n_extra))
    if st == -4:          # DL_ERR_LIMIT: student vocabulary too wide for a plan
        return None
    _lib.check(st, "dl_marginal_plan_build")
    ntiles = -(-t2s.size // tile.value)
    row_off = np.zeros(16 * ntiles + 1, dtype=np.int32)
    ent = np.empty((max(rows.value, 1), 64), dtype=np.uint32)
    fold = np.zeros((max(n_fold.value, 1), 3), dtype=np.int32)
    st = lib.dl_marginal_plan_build(_p(t2s), t2s.size, n_student, ctypes.byref(tile), _p(row_off), _p(ent), rows.value,
                                    ctypes.byref(rows), _p(fold), n_fold.value, ctypes.byref(n_fold),
                                    ctypes.byref(n_extra))
    _lib.check(st, "dl_marginal_plan_build")
    return _PlanArrays(row_off, ent, fold, tile.value, int(n_fold.value), int(n_extra.value), device)


class MarginalPlan:
    """A teacher->student id map laid out for the planned marginalisation kernels (fixed summation
    order, no atomics): build once per tokenizer pair, reuse for every batch.  Holds the device
    copies of the map and of the plan arrays.  Up to two plans are built:

    * `full`: over the student ids themselves, where the kernels' marginal can hold them all (at most
      36864 ids).  `marginalise` uses it, and `rkl_marginalised` where there is no compact one.
    * `compact`: over the map's image -- the student ids some teacher id maps to, ascending, `cols`; every
      other column lies off the marginal's support in every row.  `rkl_marginalised` then gathers those
      columns of the logits inside the kernel, runs the passes behind the marginal on them alone and
      expands the gradient row (`col_src`: compact column of every student id, -1 outside the image).
      The passes behind the marginal cost time in proportion to the marginal's width, the expansion in
      proportion to the full vocabulary (about 0.45 of a pass column per column); the compact plan is
      therefore built where the image holds at most half of the student ids (and the vocabulary is a
      multiple of 8 ids, the compact kernel's alignment), or where the full width does not fit.

    `compact=True` builds the compact plan only, `compact=False` the full one only.  `row_off`, `ent`, `fold`,
    `tile`, `n_fold` and `n_extra` describe the full plan, or the compact one where that is the only one."""

    COMPACT_AT_MOST = 0.5          # image size / student vocabulary below which the compact plan pays

    def __init__(self, t2s: np.ndarray, n_student: int, device, compact: bool | None = None):
        t2s = np.ascontiguousarray(np.asarray(t2s, dtype=np.int32))
        self.n_student = int(n_student)
        self.n_teacher = int(t2s.size)
        self.t2s = torch.as_tensor(t2s, device=device)
        self.full = self.compact = None
        self.cols = self.col_src = self.col_src16 = self.t2c = None
        self.n_compact = 0
        if compact is not True:
            self.full = _build_plan(t2s, self.n_student, device)
        ok = (t2s >= 0) & (t2s < self.n_student)
        used = np.unique(t2s[ok])
        if compact is None:
            compact = self.full is None or (self.n_student % 8 == 0 and
                                            used.size <= self.COMPACT_AT_MOST * self.n_student)
        if compact:
            n_compact = max(8, -(-used.size // 8) * 8)
            t2c = np.full(t2s.size, -1, dtype=np.int32)
            t2c[ok] = np.searchsorted(used, t2s[ok]).astype(np.int32)
            self.compact = _build_plan(t2c, n_compact, device)     # None: the image itself is too wide (the atomic path still works)
            if self.compact is not None:
                cols = np.full(n_compact, -1, dtype=np.int32)
                cols[:used.size] = used
                col_src = np.full(-(-self.n_student // 8) * 8, -1, dtype=np.int32)
                col_src[used] = np.arange(used.size, dtype=np.int32)
                self.n_compact = n_compact
                self.cols = torch.as_tensor(cols, device=device)
                self.col_src = torch.as_tensor(col_src, device=device)
                self.col_src16 = torch.as_tensor(col_src.astype(np.uint16).view(np.int16), device=device)      # -1 reads 0xffff
                self.t2c = torch.as_tensor(t2c, device=device)
        main = self.full if self.full is not None else self.compact
        self.row_off, self.ent, self.fold = (main.row_off, main.ent, main.fold) if main else (None, None, None)
        self.tile, self.n_fold, self.n_extra = (main.tile, main.n_fold, main.n_extra) if main else (0, 0, 0)

    def check(self, n_student: int, n_teacher: int, device) -> None:
        """Raises unless the plan was built for these vocabulary sizes and lives on `device`: the
        kernels index LDS by what the plan says and cannot check it themselves."""
        if self.n_student != int(n_student) or self.n_teacher != int(n_teacher):
            raise RuntimeError(f"the plan maps {self.n_teacher} teacher ids onto {self.n_student} student ids, "
                               f"the call has {int(n_teacher)} and {int(n_student)}")
        if self.t2s.device != torch.device(device):
            raise RuntimeError(f"the plan lives on {self.t2s.device}, the call runs on {device}")

    def _args(self):
        """The full plan's (row_off, ent, tile, fold, n_fold, n_extra) as the C ABI takes them; zeros without one."""
        return self.full.args() if self.full is not None else (0, 0, 0, 0, 0, 0)


def marginalise(probs: torch.Tensor, *, t2s: torch.Tensor | None = None, csr=None, plan: MarginalPlan | None = None,
                n_student: int, log: bool = False) -> torch.Tensor:
    """marg[r, s] = sum of probs[r, t] over the teacher ids mapped to s (fp32 [rows, n_student]).
    `plan` (a MarginalPlan) selects the planned form: fast and bit-reproducible; `t2s` (int32 [Vt],
    on the GPU) the LDS-atomic form; `csr=(offsets, indices)` the thread-per-id deterministic one.
    `log=True` returns log(marg)."""
    _dev(probs, "probs")
    x = _rows_2d(probs)
    if x.dtype not in _DT:
        raise RuntimeError("unsupported dtype")
    R, Vt = x.shape
    if csr is None and plan is None and t2s is None:
        raise ValueError("marginalise needs one of plan=, t2s= or csr=")
    out = torch.empty((R, n_student), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        if csr is not None:
            off, ind = csr
            _dev(off, "offsets", x.device), _dev(ind, "indices", x.device)
            if off.dtype != torch.int32 or ind.dtype != torch.int32 or off.numel() != n_student + 1:
                raise RuntimeError("csr must be (int32 offsets [n_student + 1], int32 indices)")
            if int(off[-1].item()) > ind.numel():
                raise RuntimeError("csr offsets run past the indices array")
            st = lib.dl_marginalise_csr(x.data_ptr(), _DT[x.dtype], x.stride(0), R, Vt, off.contiguous().data_ptr(),
                                        ind.contiguous().data_ptr(), n_student, out.data_ptr(), out.stride(0), int(log),
                                        _stream_ptr(x.device))
            _lib.check(st, "dl_marginalise_csr")
        else:
            plan_args = (0, 0, 0, 0, 0, 0)
            if plan is not None:
                plan.check(n_student, Vt, x.device)
                t2s = plan.t2s
                plan_args = plan._args()                # the full plan; without one the LDS-atomic form runs
            _, _ = _opt_i32(t2s, Vt, "t2s", x.device)
            st = lib.dl_marginalise_map(x.data_ptr(), _DT[x.dtype], x.stride(0), R, Vt, t2s.data_ptr(), n_student,
                                        *plan_args, out.data_ptr(), out.stride(0), int(log), _stream_ptr(x.device))
            _lib.check(st, "dl_marginalise_map")
    return out


class _CompactView:
    """A compact MarginalPlan seen from the compact side: the map onto compact ids and the plan over them."""

    def __init__(self, plan: "MarginalPlan"):
        self.plan = plan


def gather_columns(x: torch.Tensor, cols: torch.Tensor) -> torch.Tensor:
    """out[r, c] = x[r, cols[c]] (-inf where cols[c] < 0): dl_gather_columns."""
    R, V = x.shape
    out = torch.empty((R, cols.numel()), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        for a in range(0, R, 65535):
            n = min(65535, R - a)
            st = lib.dl_gather_columns(x[a:].data_ptr(), _DT[x.dtype], x.stride(0), n, V, cols.data_ptr(), cols.numel(),
                                       out[a:].data_ptr(), out.stride(0), _stream_ptr(x.device))
            _lib.check(st, "dl_gather_columns")
    return out


def expand_columns(xc: torch.Tensor, col_src: torch.Tensor, V: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[r, j] = xc[r, col_src[j]] for j < V (0 where col_src[j] < 0): dl_expand_columns."""
    R, n = xc.shape
    if out is None:
        out = torch.empty((R, V), dtype=xc.dtype, device=xc.device)
    lib = _lib.load()
    with torch.cuda.device(xc.device):
        for a in range(0, R, 65535):
            m = min(65535, R - a)
            st = lib.dl_expand_columns(xc[a:].data_ptr(), _DT[xc.dtype], xc.stride(0), m, n, col_src.data_ptr(), V,
                                       out[a:].data_ptr(), out.stride(0), _stream_ptr(xc.device))
            _lib.check(st, "dl_expand_columns")
    return out


def rkl_marginalised(logits: torch.Tensor, teacher_probs: torch.Tensor, t2s: "torch.Tensor | MarginalPlan", *,
                     row_map: torch.Tensor | None = None, T: float = 1.0, teacher_T: float | None = None,
                     grad_scale: float = 1.0, want_grad: bool = True, grad_out: torch.Tensor | None = None):
    """Reverse KL of the student (logits [rows, Vs]) against the teacher's distribution
    (teacher_probs [N, Vt]) marginalised into the student vocabulary along `t2s`, loss and gradient
    in one launch; the marginal stays in LDS.  `t2s` is the int32 [Vt] map on the GPU or, better, a
    MarginalPlan built from it.  Returns (row_loss fp32 [rows], grad or None)."""
    _dev(logits, "logits")
    x, tp = _rows_2d(logits), _rows_2d(teacher_probs)
    R, Vs = x.shape
    N, Vt = tp.shape
    dev = x.device
    _dev(teacher_probs, "teacher_probs", dev)
    plan_args = (0, 0, 0, 0, 0, 0)
    if x.dtype not in _DT or tp.dtype not in _DT:
        raise RuntimeError("unsupported dtype")
    if isinstance(t2s, MarginalPlan):
        t2s.check(Vs, Vt, dev)
        if t2s.compact is not None:
            # the student vocabulary compacted to the map's image (dl_rkl_marginalised_compact)
            plan = t2s
            if row_map is None and N < R:
                raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
            _, rm_ptr = _opt_i32(row_map, R, "row_map", dev)
            row_loss = torch.empty(R, dtype=torch.float32, device=dev)
            grad, g_ptr, g_stride = None, 0, Vs
            if want_grad:
                grad = _grad_target(grad_out, R, Vs, x.dtype, dev)
                g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
            with torch.cuda.device(dev):
                st = _lib.load().dl_rkl_marginalised_compact(
                    x.data_ptr(), _DT[x.dtype], x.stride(0), R, Vs, plan.cols.data_ptr(), plan.col_src16.data_ptr(),
                    plan.n_compact, rm_ptr, tp.data_ptr(), _DT[tp.dtype], tp.stride(0), N, Vt, plan.t2c.data_ptr(),
                    *plan.compact.args(), 1.0 / T, 1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                    row_loss.data_ptr(), g_ptr, g_stride, _stream_ptr(dev))
            _lib.check(st, "dl_rkl_marginalised_compact")
            if grad is not None and logits.dim() != 2 and grad_out is None:
                grad = grad.view(logits.shape)
            return row_loss, grad
        plan_args = t2s._args()
        t2s = t2s.t2s
    elif isinstance(t2s, _CompactView):
        plan_args = t2s.plan.compact.args()
        t2s = t2s.plan.t2c
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    _, rm_ptr = _opt_i32(row_map, R, "row_map", dev)
    _opt_i32(t2s, Vt, "t2s", dev)
    row_loss = torch.empty(R, dtype=torch.float32, device=dev)
    grad, g_ptr, g_stride = None, 0, Vs
    if want_grad:
        grad = _grad_target(grad_out, R, Vs, x.dtype, dev)
        g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
    with torch.cuda.device(dev):
        st = _lib.load().dl_rkl_marginalised(x.data_ptr(), _DT[x.dtype], x.stride(0), R, Vs, rm_ptr, tp.data_ptr(),
                                             _DT[tp.dtype], tp.stride(0), N, Vt, t2s.data_ptr(), *plan_args, 1.0 / T,
                                             1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                                             row_loss.data_ptr(), g_ptr, g_stride, _stream_ptr(dev))
    _lib.check(st, "dl_rkl_marginalised")
    return row_loss, grad

"""Teacher-distribution preprocessing on the GPU: multi-teacher merge, vocabulary remap, and the
losses fed by them.  Thin wrappers over the C ABI; all arithmetic runs in the HIP kernels."""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from . import _lib, ops
from .ops import _DT, _IT, _dev, _stream_ptr


def _ptr_array(tensors: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def merge_remap_topk(vals: Sequence[torch.Tensor], idxs: Sequence[torch.Tensor], weights: Sequence[float],
                     id_map: torch.Tensor | None = None, student_vocab: int | None = None):
    """Weighted sum of several top-K teachers after mapping their ids into the student vocabulary.

    vals[j] / idxs[j]: [N, K] stored log-probs and ids of teacher j (same dtype for all teachers);
    id_map: int32 [Vt] teacher id -> student id, -1 = dropped (None = same vocabulary).
    Returns (ids int32 [N, E] ascending, -1 padded; log-mass fp32 [N, E]; count int32 [N]) with
    E = len(vals) * K -- the ragged sparse teacher `ops.div_topk(..., t_cnt=count)` consumes.
    """
    n = len(vals)
    if n == 0 or len(idxs) != n or len(weights) != n:
        raise ValueError("vals, idxs and weights must have one entry per teacher")
    vals = [v.contiguous() for v in vals]
    idxs = [i.contiguous() for i in idxs]
    for v, i in zip(vals, idxs):
        _dev(v, "vals", vals[0].device), _dev(i, "idxs", vals[0].device)
        if v.shape != vals[0].shape or i.shape != vals[0].shape or v.dtype != vals[0].dtype or i.dtype != idxs[0].dtype:
            raise RuntimeError("all teachers must share shape [N, K] and dtypes")
    N, K = vals[0].shape
    dev = vals[0].device
    if id_map is not None:
        _dev(id_map, "id_map", dev)
        if id_map.dtype != torch.int32 or id_map.dim() != 1 or not id_map.is_contiguous():
            raise RuntimeError("id_map must be a contiguous int32 vector")
        if student_vocab is None:
            raise ValueError("student_vocab is required with an id_map")
    elif student_vocab is None:
        raise ValueError("student_vocab (number of ids) is required")
    E = n * K
    out_idx = torch.empty((N, E), dtype=torch.int32, device=dev)
    out_lm = torch.empty((N, E), dtype=torch.float32, device=dev)
    out_cnt = torch.empty((N,), dtype=torch.int32, device=dev)
    w = (ctypes.c_float * n)(*[float(x) for x in weights])
    with torch.cuda.device(dev):
        st = _lib.load().dl_merge_remap_topk(n, _ptr_array(vals), _ptr_array(idxs), _DT[vals[0].dtype],
                                             _IT[idxs[0].dtype], K, w, N,
                                             id_map.data_ptr() if id_map is not None else 0,
                                             id_map.numel() if id_map is not None else 0, int(student_vocab),
                                             out_idx.data_ptr(), out_lm.data_ptr(), out_cnt.data_ptr(),
                                             _stream_ptr(dev))
    _lib.check(st, "dl_merge_remap_topk")
    return out_idx, out_lm, out_cnt


def merge_topk_pair(disk_val: torch.Tensor, disk_idx: torch.Tensor, new_val: torch.Tensor, new_idx: torch.Tensor,
                    vocab: int):
    """The dataset manager's merge of a stored teacher with a newly collected one
    (classes/data_manager.py:198-261): returns (log-mass fp32 [n, K], ids int64 [n, K]) in
    descending-mass order, n = the longer of the two inputs."""
    for t, name in ((disk_val, "disk_val"), (disk_idx, "disk_idx"), (new_val, "new_val"), (new_idx, "new_idx")):
        _dev(t, name, disk_val.device if disk_val.is_cuda else None)
    disk_val, disk_idx, new_val, new_idx = (t.contiguous() for t in (disk_val, disk_idx, new_val, new_idx))
    if disk_val.dtype != new_val.dtype or disk_idx.dtype != new_idx.dtype or disk_val.shape[1] != new_val.shape[1]:
        raise RuntimeError("both teachers must share K and dtypes")
    K = disk_val.shape[1]
    n = max(disk_val.shape[0], new_val.shape[0])
    dev = disk_val.device
    out_lm = torch.empty((n, K), dtype=torch.float32, device=dev)
    out_idx = torch.empty((n, K), dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        st = _lib.load().dl_merge_topk_pair(disk_val.data_ptr(), disk_idx.data_ptr(), disk_val.shape[0],
                                            new_val.data_ptr(), new_idx.data_ptr(), new_val.shape[0],
                                            _DT[disk_val.dtype], _IT[disk_idx.dtype], K, int(vocab),
                                            out_lm.data_ptr(), out_idx.data_ptr(), _stream_ptr(dev))
    _lib.check(st, "dl_merge_topk_pair")
    return out_lm, out_idx


def _check_teachers(vals, idxs, weights):
    n = len(vals)
    if n == 0 or len(idxs) != n or len(weights) != n:
        raise ValueError("vals, idxs and weights must have one entry per teacher")
    vals = [v.contiguous() for v in vals]
    idxs = [i.contiguous() for i in idxs]
    for v, i in zip(vals, idxs):
        _dev(v, "vals", vals[0].device), _dev(i, "idxs", vals[0].device)
        if v.dim() != 2 or v.shape != vals[0].shape or i.shape != vals[0].shape or v.dtype != vals[0].dtype \
                or i.dtype != idxs[0].dtype:
            raise RuntimeError("all teachers must share shape [N, K] and dtypes")
    if vals[0].dtype not in _DT or idxs[0].dtype not in _IT:
        raise RuntimeError("unsupported dtype")
    return vals, idxs


def fkl_multi_teacher(logits: torch.Tensor, vals: Sequence[torch.Tensor], idxs: Sequence[torch.Tensor],
                      weights: Sequence[float], id_map: torch.Tensor | None = None, *,
                      row_map: torch.Tensor | None = None, T: float = 1.0, teacher_T: float | None = None,
                      grad_scale: float = 1.0, want_grad: bool = True, grad_out: torch.Tensor | None = None,
                      fused: bool | None = None, no_wait: bool = False):
    """Forward KL of the student against the weighted, remapped, renormalised mixture of several
    top-K teachers.  Returns (row_loss, grad) like `ops.div_topk`.

    With teacher temperature 1 (`teacher_T`, default = `T`) this is dl_fkl_multi_teacher: a K-wide
    launch maps, weighs and renormalises the entries and deals them, unsorted, into one bucket per
    column part of the loss kernel's rows; the loss kernel's workgroups each fetch only their own
    bucket and sum the entries that share a student id on their per-chunk lists.  Other temperatures
    and unaligned or very wide rows take the sorting form: `merge_remap_topk` (ascending unique ids
    through memory) feeding `ops.div_topk`.  `fused=True` insists on the first form (raises where it
    does not apply), `fused=False` on the second."""
    tT = T if teacher_T is None else teacher_T
    if fused is None or fused:
        got = _fkl_multi_fused(logits, vals, idxs, weights, id_map, row_map, T, grad_scale, want_grad, grad_out, no_wait) \
            if tT == 1.0 else None
        if got is not None:
            return got
        if fused:
            raise RuntimeError("the bucketed multi-teacher form needs teacher temperature 1 and 16-byte aligned rows of at most "
                               "262144 two-byte (131072 four-byte) columns")
    V = logits.shape[-1]
    ids, logmass, cnt = merge_remap_topk(vals, idxs, weights, id_map, student_vocab=V)
    return ops.div_topk("fkl", logits, logmass, ids, row_map=row_map, t_cnt=cnt, T=T, teacher_T=teacher_T,
                        grad_scale=grad_scale, want_grad=want_grad, grad_out=grad_out, unique_ids=True, no_wait=no_wait)


def _fkl_multi_fused(logits, vals, idxs, weights, id_map, row_map, T, grad_scale, want_grad, grad_out, no_wait):
    """dl_fkl_multi_teacher; None where the library says the one-pass form does not apply."""
    _dev(logits, "logits")
    x = ops._rows_2d(logits)
    R, V = x.shape
    dev = x.device
    vals, idxs = _check_teachers(vals, idxs, weights)
    _dev(vals[0], "vals", dev)
    if x.dtype not in _DT:
        raise RuntimeError("unsupported dtype")
    N, K = vals[0].shape
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    _, rm_ptr = ops._opt_i32(row_map, R, "row_map", dev)
    _, map_ptr = ops._opt_i32(id_map, None, "id_map", dev)
    row_loss = torch.empty(R, dtype=torch.float32, device=dev)
    grad, g_ptr, g_stride = None, 0, V
    if want_grad:
        grad = ops._grad_target(grad_out, R, V, x.dtype, dev, like=x)
        g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
    lib = _lib.load()
    n = len(vals)
    flags = _lib.DL_TOPK_NO_WAIT if no_wait else 0
    ws_bytes = lib.dl_fkl_multi_teacher_workspace_bytes(_DT[x.dtype], R, V, n, K, N, flags)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    w = (ctypes.c_float * n)(*[float(v) for v in weights])
    with torch.cuda.device(dev):
        st = lib.dl_fkl_multi_teacher(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr, n, _ptr_array(vals),
                                      _ptr_array(idxs), _DT[vals[0].dtype], _IT[idxs[0].dtype], K, N, w, map_ptr,
                                      id_map.numel() if id_map is not None else 0, 1.0 / T, grad_scale,
                                      row_loss.data_ptr(), g_ptr, g_stride, ws.data_ptr() if ws is not None else 0,
                                      ws_bytes, flags, ops._stream_ptr(dev))
    if st in (-4, -6):              # DL_ERR_LIMIT / ALIGN: rows too wide or unaligned for the register kernels
        return None
    _lib.check(st, "dl_fkl_multi_teacher")
    if grad is not None and logits.dim() != 2 and grad_out is None:
        grad = grad.view(logits.shape)
    return row_loss, grad


def teacher_topk(logits: torch.Tensor, K: int, *, crop_to_size: int | None = None, rows: torch.Tensor | None = None,
                 val_dtype=torch.float16, idx_dtype=torch.int32):
    """What the teacher's inference worker produces (classes/teacher/inference_worker.py:73-80) in
    the dataset's storage layout: per row the K largest full-vocabulary log-probs, descending, and
    their ids.  `rows` (int32 positions, e.g. the content rows) selects and orders the output rows.
    Returns (log-probs [n, K] val_dtype, ids [n, K] idx_dtype)."""
    _dev(logits, "logits")
    x = ops._rows_2d(logits if crop_to_size is None else logits[..., :crop_to_size])
    if x.dtype not in _DT or val_dtype not in (torch.float16, torch.float32) or idx_dtype not in _IT:
        raise RuntimeError("unsupported dtype")
    R, V = x.shape
    dev = x.device
    n_out, rl_ptr = R, 0
    if rows is not None:
        ops._opt_i32(rows, None, "rows", dev)
        n_out, rl_ptr = rows.numel(), rows.data_ptr()
    out_v = torch.empty((n_out, K), dtype=val_dtype, device=dev)
    out_i = torch.empty((n_out, K), dtype=idx_dtype, device=dev)
    lib = _lib.load()
    ws = torch.empty((max(16, lib.dl_teacher_topk_workspace_bytes(_DT[x.dtype], n_out, V, K)),), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        st = lib.dl_teacher_topk(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rl_ptr, n_out, K,
                                 out_v.data_ptr(), _DT[val_dtype], out_i.data_ptr(), _IT[idx_dtype],
                                 ws.data_ptr(), ws.numel(), _stream_ptr(dev))
    _lib.check(st, "dl_teacher_topk")
    return out_v, out_i

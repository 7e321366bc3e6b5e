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


def fkl_multi_teacher(logits: torch.Tensor, vals: Sequence[torch.Tensor], idxs: Sequence[torch.Tensor],
                      weights: Sequence[float], id_map: torch.Tensor | None = None, *,
                      row_map: torch.Tensor | None = None, T: float = 1.0, teacher_T: float | None = None,
                      grad_scale: float = 1.0, want_grad: bool = True, grad_out: torch.Tensor | None = None):
    """Forward KL of the student against the weighted, remapped, renormalised mixture of several
    top-K teachers: one merge launch (K-wide work, once per row) feeding the fused loss+gradient
    kernel.  Returns (row_loss, grad) like `ops.div_topk`."""
    V = logits.shape[-1]
    ids, logmass, cnt = merge_remap_topk(vals, idxs, weights, id_map, student_vocab=V)
    return ops.div_topk("fkl", logits, logmass, ids, row_map=row_map, t_cnt=cnt, T=T, teacher_T=teacher_T,
                        grad_scale=grad_scale, want_grad=want_grad, grad_out=grad_out, unique_ids=True)


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

"""Tensor-level wrappers over the C ABI.  PyTorch supplies device memory and the
stream; all arithmetic happens in the HIP kernels.  No fallbacks: a CPU tensor or
a missing library raises."""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib

_DT = {torch.float32: _lib.DL_F32, torch.bfloat16: _lib.DL_BF16, torch.float16: _lib.DL_F16}
_IT = {torch.int32: _lib.DL_I32, torch.int64: _lib.DL_I64}
KINDS = {"fkl": _lib.DL_FKL, "rkl": _lib.DL_RKL, "jsd": _lib.DL_JSD}


def _stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _dev(t: torch.Tensor, name: str, dev: torch.device | None = None) -> None:
    """`t` must live on the GPU -- on `dev`, when given: the kernels take raw pointers and run on the
    device of the logits, so a tensor on another GPU would be read through a foreign address."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); this library has no CPU path")
    if dev is not None and t.device != dev:
        raise RuntimeError(f"{name} lives on {t.device}, the logits on {dev}: all tensors of a call must share one device")


def _grad_target(grad_out, R: int, V: int, dtype, dev, like: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The gradient buffer of a launch over [R, V] logits: `grad_out` checked against what the kernel
    will write (shape, dtype, dense along V, same device), or a fresh one.  A fresh buffer for logits
    `like` whose rows do not all start on 16-byte boundaries (a column slice, an odd pitch) copies their
    pitch and their offset on the 16-byte grid: the kernels use vector accesses inside such rows only when
    logits and gradient rows line up."""
    if grad_out is None:
        if like is not None and like.dim() == 2:
            eb = like.element_size()
            phase = (like.data_ptr() % 16) // eb
            if phase or (like.stride(0) * eb) % 16 or (V * eb) % 16:
                pitch = like.stride(0)
                buf = torch.empty(R * pitch + phase + 8, dtype=dtype, device=dev)      # torch allocations start on 16-byte boundaries
                return buf.as_strided((R, V), (pitch, 1), phase)
        return torch.empty((R, V), dtype=dtype, device=dev)
    if grad_out.dim() != 2 or tuple(grad_out.shape) != (R, V) or grad_out.dtype != dtype or grad_out.stride(1) != 1 \
            or grad_out.device != dev:
        raise RuntimeError(f"grad_out must be a [{R}, {V}] {dtype} tensor on {dev}, dense along the vocabulary axis")
    return grad_out


def _rows_2d(logits: torch.Tensor) -> torch.Tensor:
    """View [..., V] logits as [R, V] without copying; the last dim must be dense."""
    if logits.dim() < 2:
        raise RuntimeError("logits must have shape [..., rows, vocab]")
    if logits.stride(-1) != 1:
        raise RuntimeError("logits must be contiguous along the vocabulary axis")
    if logits.dim() == 2:
        return logits
    V = logits.shape[-1]
    try:
        return logits.view(-1, V)
    except RuntimeError:
        flat = logits.as_strided((logits.numel() // V, V), (logits.stride(-2), 1), logits.storage_offset())
        lead = 1
        for d in range(logits.dim() - 2, -1, -1):      # accept only a uniform row pitch
            if logits.stride(d) != lead * logits.stride(-2) and logits.shape[d] != 1:
                raise RuntimeError("logits rows are not evenly strided; make them contiguous first")
            lead *= logits.shape[d]
        return flat


def _opt_i32(t, n, name, dev):
    if t is None:
        return None, 0
    _dev(t, name)
    if t.dtype != torch.int32 or t.dim() != 1 or not t.is_contiguous() or t.device != dev:
        raise RuntimeError(f"{name} must be a contiguous int32 vector on {dev}")
    if n is not None and t.numel() != n:
        raise RuntimeError(f"{name} has {t.numel()} entries, expected {n}")
    return t, t.data_ptr()


def div_topk(kind: str, logits: torch.Tensor, t_val: torch.Tensor, t_idx: torch.Tensor, *,
             row_map: torch.Tensor | None = None, t_cnt: torch.Tensor | None = None,
             T: float = 1.0, teacher_T: float | None = None, grad_scale: float = 1.0,
             want_grad: bool = True, grad_out: torch.Tensor | None = None, unique_ids: bool = False,
             no_wait: bool = False, parts: int = 0):
    """Per-token forward ("fkl") or reverse ("rkl") KL against a top-K teacher and,
    in the same launch, d(sum of row losses)/d(logits) * grad_scale.

    logits [..., V] bf16/fp16/fp32 (native model dtype, rows evenly strided);
    t_val/t_idx [N, K] stored teacher log-probs and ids; row_map int32 [rows]
    gives the teacher row of each logits row (negative = masked row).  `unique_ids=True` promises
    that no id repeats within a row (skips the check for repeated ids).  `no_wait` / `parts` are the
    library's per-call test hooks for rows cut into column parts (DL_TOPK_NO_WAIT, DL_TOPK_PARTS).
    Returns (row_loss fp32 [rows], grad like logits or None).
    """
    if kind not in ("fkl", "rkl"):
        raise ValueError("kind must be 'fkl' or 'rkl' for a top-K teacher")
    _dev(logits, "logits")
    x = _rows_2d(logits)
    R, V = x.shape
    dev = x.device
    _dev(t_val, "t_val", dev), _dev(t_idx, "t_idx", dev)
    if x.dtype not in _DT or t_val.dtype not in _DT or t_idx.dtype not in _IT:
        raise RuntimeError("unsupported dtype")
    if t_val.dim() != 2 or t_val.shape != t_idx.shape:
        raise RuntimeError("t_val and t_idx must both be [N, K]")
    t_val, t_idx = t_val.contiguous(), t_idx.contiguous()
    N, K = t_val.shape
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    _, rm_ptr = _opt_i32(row_map, R, "row_map", dev)
    _, cnt_ptr = _opt_i32(t_cnt, N, "t_cnt", dev)
    row_loss = torch.empty(R, dtype=torch.float32, device=dev)
    grad, g_ptr, g_stride = None, 0, V
    if want_grad:
        grad = _grad_target(grad_out, R, V, x.dtype, dev, like=x)
        g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
    if parts not in (0, 1, 2, 4, 16):
        raise ValueError("parts must be 0 (automatic), 1, 2, 4 or 16 (parts of 1024 chunks, up to 16 per row)")
    flags = (_lib.DL_TOPK_UNIQUE_IDS if unique_ids else 0) | (_lib.DL_TOPK_NO_WAIT if no_wait else 0) | \
        (_lib.DL_TOPK_FINE_PARTS if parts == 16 else parts << _lib.DL_TOPK_PARTS_SHIFT)
    lib = _lib.load()
    ws_bytes = lib.dl_div_topk_workspace_bytes(KINDS[kind], _DT[x.dtype], R, V) if want_grad else 0
    if parts == 16 and want_grad:
        ws_bytes = R * 16 * 20 + 16
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        st = lib.dl_div_topk(KINDS[kind], x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr,
                             t_val.data_ptr(), _DT[t_val.dtype], t_idx.data_ptr(), _IT[t_idx.dtype], K, N,
                             cnt_ptr, 1.0 / T, 1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                             row_loss.data_ptr(), g_ptr, g_stride,
                             ws.data_ptr() if ws is not None else 0, ws_bytes,
                             flags, _stream_ptr(dev))
    _lib.check(st, "dl_div_topk")
    if grad is not None and logits.dim() != 2 and grad_out is None:
        grad = grad.view(logits.shape)
    return row_loss, grad


def div_topk_static(kind: str, logits: torch.Tensor, t_val: torch.Tensor, t_idx: torch.Tensor, row_loss: torch.Tensor,
                    grad: torch.Tensor | None, *, row_map: torch.Tensor | None = None, t_cnt: torch.Tensor | None = None,
                    T: float = 1.0, teacher_T: float | None = None, grad_scale: float = 1.0, unique_ids: bool = False,
                    no_wait: bool = False, parts: int = 0) -> None:
    """`div_topk` for callers that cannot allocate (dl_div_topk_static): the caller brings `row_loss`
    fp32 [rows] and `grad` like the logits (or None), the split-row scratch is the library's static
    device array, and neither this wrapper nor the library allocates.  Calls that may overlap in time
    on one GPU must not use it (they would share the array); limit: DL_STATIC_SCRATCH_BYTES."""
    if kind not in ("fkl", "rkl"):
        raise ValueError("kind must be 'fkl' or 'rkl' for a top-K teacher")
    if parts not in (0, 1, 2, 4):
        raise ValueError("parts must be 0 (automatic), 1, 2 or 4")
    _dev(logits, "logits")
    x = _rows_2d(logits)
    R, V = x.shape
    dev = x.device
    _dev(t_val, "t_val", dev), _dev(t_idx, "t_idx", dev), _dev(row_loss, "row_loss", dev)
    if x.dtype not in _DT or t_val.dtype not in _DT or t_idx.dtype not in _IT:
        raise RuntimeError("unsupported dtype")
    if t_val.dim() != 2 or t_val.shape != t_idx.shape or not (t_val.is_contiguous() and t_idx.is_contiguous()):
        raise RuntimeError("t_val and t_idx must both be contiguous [N, K]")
    N, K = t_val.shape
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    if row_loss.dtype != torch.float32 or row_loss.dim() != 1 or row_loss.numel() != R or not row_loss.is_contiguous():
        raise RuntimeError(f"row_loss must be a contiguous fp32 vector of {R} entries")
    _, rm_ptr = _opt_i32(row_map, R, "row_map", dev)
    _, cnt_ptr = _opt_i32(t_cnt, N, "t_cnt", dev)
    g_ptr, g_stride = 0, V
    if grad is not None:
        g = _grad_target(grad, R, V, x.dtype, dev)
        g_ptr, g_stride = g.data_ptr(), g.stride(0)
    flags = (_lib.DL_TOPK_UNIQUE_IDS if unique_ids else 0) | (_lib.DL_TOPK_NO_WAIT if no_wait else 0) | \
        (parts << _lib.DL_TOPK_PARTS_SHIFT)
    with torch.cuda.device(dev):
        st = _lib.load().dl_div_topk_static(KINDS[kind], x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr,
                                            t_val.data_ptr(), _DT[t_val.dtype], t_idx.data_ptr(), _IT[t_idx.dtype], K, N,
                                            cnt_ptr, 1.0 / T, 1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                                            row_loss.data_ptr(), g_ptr, g_stride, flags, _stream_ptr(dev))
    _lib.check(st, "dl_div_topk_static")


def div_dense(kind: str, logits: torch.Tensor, t_logits: torch.Tensor, *, row_map: torch.Tensor | None = None,
              T: float = 1.0, teacher_T: float | None = None, grad_scale: float = 1.0, want_grad: bool = True,
              grad_out: torch.Tensor | None = None, split: bool = True, no_wait: bool = False, part_threads: int = 0):
    """Per-token "fkl", "rkl" or "jsd" against a dense teacher [N, V] and, in the same launch,
    d(sum of row losses)/d(logits) * grad_scale.  Returns (row_loss fp32 [rows], grad or None).
    `split=False` withholds the workspace that lets wide forward / reverse-KL rows be cut into column parts
    (dl_div_dense_ws); `no_wait` and `part_threads` (256 / 512 / 1024) are the library's test hooks for those parts
    (DL_TOPK_NO_WAIT, DL_TOPK_PARTS)."""
    if kind not in KINDS:
        raise ValueError("kind must be 'fkl', 'rkl' or 'jsd'")
    _dev(logits, "logits")
    x = _rows_2d(logits)
    t = _rows_2d(t_logits)
    R, V = x.shape
    dev = x.device
    _dev(t_logits, "t_logits", dev)
    if x.dtype not in _DT or t.dtype not in _DT:
        raise RuntimeError("unsupported dtype")
    if t.shape[1] != V:
        raise RuntimeError(f"teacher has {t.shape[1]} columns, logits {V}")
    N = t.shape[0]
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    _, rm_ptr = _opt_i32(row_map, R, "row_map", dev)
    row_loss = torch.empty(R, dtype=torch.float32, device=dev)
    grad, g_ptr, g_stride = None, 0, V
    if want_grad:
        grad = _grad_target(grad_out, R, V, x.dtype, dev)
        g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
    lib = _lib.load()
    ws_bytes = lib.dl_div_dense_workspace_bytes(KINDS[kind], _DT[x.dtype], _DT[t.dtype], R, V) if split else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        st = lib.dl_div_dense_ws(KINDS[kind], x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr,
                                 t.data_ptr(), _DT[t.dtype], t.stride(0), N, 1.0 / T,
                                 1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                                 row_loss.data_ptr(), g_ptr, g_stride, ws.data_ptr() if ws is not None else 0, ws_bytes,
                                 (_lib.DL_TOPK_NO_WAIT if no_wait else 0) |
                                 ({0: 0, 256: 1, 512: 2, 1024: 3}[part_threads] << _lib.DL_TOPK_PARTS_SHIFT), _stream_ptr(dev))
    _lib.check(st, "dl_div_dense_ws")
    if grad is not None and logits.dim() != 2 and grad_out is None:
        grad = grad.view(logits.shape)
    return row_loss, grad


def _rowstats_raw(x: torch.Tensor, t_idx: torch.Tensor, row_map, inv_T: float):
    """Phase 1 launch: (lse [N], zk [N, K]) for the valid rows of x [R, V]."""
    _dev(x, "logits"), _dev(t_idx, "t_idx", x.device)
    if x.dim() != 2 or x.stride(1) != 1 or x.dtype not in _DT:
        raise RuntimeError("logits must be [rows, V] bf16/fp16/fp32, dense along V")
    if t_idx.dim() != 2 or t_idx.dtype not in _IT:
        raise RuntimeError("t_idx must be [N, K] int32/int64")
    t_idx = t_idx.contiguous()
    R, V = x.shape
    N, K = t_idx.shape
    if row_map is None and N < R:
        raise RuntimeError(f"{R} logits rows but only {N} teacher rows and no row_map")
    _, rm_ptr = _opt_i32(row_map, R, "row_map", x.device)
    # every teacher row is written by the kernel unless a row map leaves some out, or there are more
    # teacher rows than logits rows (rows R .. N-1 are then nobody's): no zero fill in that case only
    make = torch.empty if row_map is None and N == R else torch.zeros
    lse = make(N, dtype=torch.float32, device=x.device)
    zk = make((N, K), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        st = _lib.load().dl_rowstats_topk(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr, t_idx.data_ptr(),
                                          _IT[t_idx.dtype], K, N, inv_T, lse.data_ptr(), zk.data_ptr(),
                                          _stream_ptr(x.device))
    _lib.check(st, "dl_rowstats_topk")
    return lse, zk


def _rowcoef_grad_raw(x: torch.Tensor, t_idx: torch.Tensor, row_map, inv_T: float, lse: torch.Tensor,
                      g_lse: torch.Tensor, g_zk: torch.Tensor, grad_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Phase 2 launch: d L / d x from dL/d lse and dL/d zk (into `grad_out` [R, V], dense along V, if given)."""
    t_idx = t_idx.contiguous()
    R, V = x.shape
    N, K = t_idx.shape
    _, rm_ptr = _opt_i32(row_map, R, "row_map", x.device)
    g_lse = g_lse.to(torch.float32).contiguous()
    g_zk = g_zk.to(torch.float32).contiguous()
    for name, t in (("t_idx", t_idx), ("lse", lse), ("g_lse", g_lse), ("g_zk", g_zk)):
        _dev(t, name, x.device)
    grad = _grad_target(grad_out, R, V, x.dtype, x.device, like=x)
    with torch.cuda.device(x.device):
        st = _lib.load().dl_rowcoef_grad_topk(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr, t_idx.data_ptr(),
                                              _IT[t_idx.dtype], K, N, inv_T, lse.data_ptr(), g_lse.data_ptr(),
                                              g_zk.data_ptr(), grad.data_ptr(), grad.stride(0),
                                              _stream_ptr(x.device))
    _lib.check(st, "dl_rowcoef_grad_topk")
    return grad


def _cropped(logits: torch.Tensor, crop: int) -> torch.Tensor:
    return logits[:, :crop] if 0 < crop < logits.shape[1] else logits


@torch.library.custom_op("distillery_amd::rowstats_topk", mutates_args=())
def rowstats_topk(logits: torch.Tensor, t_idx: torch.Tensor, row_map: Optional[torch.Tensor],
                  inv_T: float, crop: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """(lse [N] fp32, zk [N, K] fp32): full-vocabulary log-sum-exp of logits * inv_T and the scaled
    logits at the teacher ids, for the rows selected by row_map.  Differentiable w.r.t. logits.
    `crop` > 0 uses only the first `crop` columns (the reference's `[:, :, :crop_to_size]`,
    classes/student/model.py:408) without a slice in the autograd graph, whose backward would
    zero-fill and copy a second full-width gradient buffer."""
    return _rowstats_raw(_cropped(logits, crop), t_idx, row_map, inv_T)


@rowstats_topk.register_fake
def _(logits, t_idx, row_map, inv_T, crop=0):
    N, K = t_idx.shape
    return (logits.new_empty((N,), dtype=torch.float32), logits.new_empty((N, K), dtype=torch.float32))


@torch.library.custom_op("distillery_amd::rowcoef_grad_topk", mutates_args=())
def rowcoef_grad_topk(logits: torch.Tensor, t_idx: torch.Tensor, row_map: Optional[torch.Tensor], inv_T: float,
                      lse: torch.Tensor, g_lse: torch.Tensor, g_zk: torch.Tensor, crop: int = 0) -> torch.Tensor:
    x = _cropped(logits, crop)
    if x is logits:
        return _rowcoef_grad_raw(logits, t_idx, row_map, inv_T, lse, g_lse, g_zk)
    grad = torch.empty_like(logits)                      # full width; the kernel fills [:, :crop]
    grad[:, crop:].zero_()
    _rowcoef_grad_raw(x, t_idx, row_map, inv_T, lse, g_lse, g_zk, grad_out=grad[:, :crop])
    return grad


@rowcoef_grad_topk.register_fake
def _(logits, t_idx, row_map, inv_T, lse, g_lse, g_zk, crop=0):
    return torch.empty_like(logits)


def _rowstats_setup(ctx, inputs, output):
    logits, t_idx, row_map, inv_T, crop = inputs
    lse, _ = output
    ctx.save_for_backward(logits, t_idx, lse, *([row_map] if row_map is not None else []))
    ctx.has_map = row_map is not None
    ctx.inv_T = inv_T
    ctx.crop = crop


def _rowstats_backward(ctx, g_lse, g_zk):
    saved = ctx.saved_tensors
    logits, t_idx, lse = saved[:3]
    row_map = saved[3] if ctx.has_map else None
    if g_lse is None:
        g_lse = torch.zeros_like(lse)
    if g_zk is None:
        g_zk = torch.zeros((t_idx.shape[0], t_idx.shape[1]), dtype=torch.float32, device=lse.device)
    return rowcoef_grad_topk(logits, t_idx, row_map, ctx.inv_T, lse, g_lse, g_zk, ctx.crop), None, None, None, None


rowstats_topk.register_autograd(_rowstats_backward, setup_context=_rowstats_setup)


def _offsets_arg(offsets):
    """(row, label, avoid) offsets for dl_composite_*: three ctypes int32 arrays that travel with the
    launch when `offsets` is a host list of three lists (at most DL_MAX_HOST_CONVOS conversations), or
    the rows of a device int32 [3, C + 1] tensor."""
    if isinstance(offsets, torch.Tensor):
        return (offsets[0].data_ptr(), offsets[1].data_ptr(), offsets[2].data_ptr()), 0, offsets.shape[1] - 1
    C = len(offsets[0]) - 1
    arr = ctypes.c_int32 * (C + 1)
    return (arr(*offsets[0]), arr(*offsets[1]), arr(*offsets[2])), 1, C


# True: phase 1 and the K-wide epilogue of the composite loss as the two entry points a caller with launches of its own
# uses (dl_rowstats_topk, dl_composite_forward) instead of the one call that stands for them; the tests compare the two.
SEPARATE_COMPOSITE_FORWARD = False


def _composite_forward_raw(logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T, inv_T_teacher, alpha, crop, need_grad):
    """Phase 1 over the logits + the K-wide epilogue: (nine values [C, 9], lse, zk, rec, coef or None)."""
    x = _cropped(logits, crop)
    dev = x.device
    R, V = x.shape
    N, K = t_idx.shape
    lib = _lib.load()
    offs, on_host, C = _offsets_arg(offsets)
    if not on_host:      # with offsets on the device the library cannot see that a list is empty and wants both pointers
        labels = labels if labels.numel() else torch.zeros(1, dtype=torch.int64, device=dev)
        avoid = avoid if avoid.numel() else torch.zeros(1, dtype=avoid.dtype, device=dev)
    # every teacher row is written by phase 1 unless a row map leaves some out or teacher rows outnumber the logits rows
    make = torch.empty if row_map is None and N == R else torch.zeros
    lse = make(N, dtype=torch.float32, device=dev)
    zk = make((N, K), dtype=torch.float32, device=dev)
    rec = torch.empty((N, 8), dtype=torch.float32, device=dev)
    coef = torch.empty((N, 4), dtype=torch.float32, device=dev) if need_grad else None
    out = torch.empty((C, 9), dtype=torch.float32, device=dev)
    rm_ptr = row_map.data_ptr() if row_map is not None else 0
    stream = _stream_ptr(dev)
    with torch.cuda.device(dev):
        if SEPARATE_COMPOSITE_FORWARD:
            st = lib.dl_rowstats_topk(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr, t_idx.data_ptr(), _IT[t_idx.dtype],
                                      K, N, inv_T, lse.data_ptr(), zk.data_ptr(), stream)
            _lib.check(st, "dl_rowstats_topk")
            st = lib.dl_composite_forward(
                lse.data_ptr(), zk.data_ptr(), t_val.data_ptr(), _DT[t_val.dtype], inv_T_teacher, t_idx.data_ptr(),
                _IT[t_idx.dtype], K, labels.data_ptr() if labels.numel() else 0, avoid.data_ptr() if avoid.numel() else 0,
                _IT[avoid.dtype], offs[0], offs[1], offs[2], on_host, C, N, alpha, rec.data_ptr(),
                coef.data_ptr() if need_grad else 0, out.data_ptr(), stream)
            _lib.check(st, "dl_composite_forward")
        else:
            st = lib.dl_composite_forward_fused(
                x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr, N, inv_T, t_val.data_ptr(), _DT[t_val.dtype],
                inv_T_teacher, t_idx.data_ptr(), _IT[t_idx.dtype], K, labels.data_ptr() if labels.numel() else 0,
                avoid.data_ptr() if avoid.numel() else 0, _IT[avoid.dtype], offs[0], offs[1], offs[2], on_host, C, alpha,
                lse.data_ptr(), zk.data_ptr(), rec.data_ptr(), coef.data_ptr() if need_grad else 0, out.data_ptr(), stream)
            _lib.check(st, "dl_composite_forward_fused")
    return out, lse, zk, rec, coef


# The composite loss's backward is one launch (dl_composite_backward_fused) or two (dl_composite_backward +
# dl_rowcoef_grad_topk), chosen by the rows' width; "fused" / "separate" here fixes the form (the tests compare them).
FORCE_COMPOSITE_BACKWARD = None


def _composite_backward_raw(logits, t_val, t_idx, lse, zk, rec, coef, g_train, offsets, row_map, inv_T, inv_T_teacher, crop):
    """The epilogue's backward + phase 2: d(sum_c g_train[c] * train_loss[c]) / d logits, full width."""
    x = _cropped(logits, crop)
    dev = x.device
    R, V = x.shape
    N, K = t_idx.shape
    lib = _lib.load()
    offs, on_host, C = _offsets_arg(offsets)
    g = g_train.to(torch.float32).contiguous()
    grad = torch.empty_like(logits)                      # full width; the kernel fills [:, :crop]
    if x is not logits:
        grad[:, crop:].zero_()
    gx = _cropped(grad, crop)
    stream = _stream_ptr(dev)
    # Phase 2 making the rows' coefficients itself saves a launch and two K-wide arrays, but every column part of a row
    # (32 KiB of logits) makes all K of them: it pays up to four parts per row (0.664 against 0.676 ms on 8192 x 32000
    # fp32 rows, K = 400) and costs beyond (4.01 against 3.95 ms on 32768 x 128256 bf16 rows, K = 200: eight parts)
    fused = V * x.element_size() <= 4 * 32768 if FORCE_COMPOSITE_BACKWARD is None else FORCE_COMPOSITE_BACKWARD == "fused"
    if fused:
        with torch.cuda.device(dev):
            st = lib.dl_composite_backward_fused(
                x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, row_map.data_ptr() if row_map is not None else 0, N, inv_T,
                t_val.data_ptr(), _DT[t_val.dtype], inv_T_teacher,
                t_idx.data_ptr(), _IT[t_idx.dtype], K, offs[0], on_host, C, lse.data_ptr(), zk.data_ptr(), rec.data_ptr(),
                coef.data_ptr(), g.data_ptr(), gx.data_ptr(), gx.stride(0), stream)
            _lib.check(st, "dl_composite_backward_fused")
        return grad
    g_lse = torch.empty_like(lse)
    g_zk = torch.empty_like(zk)
    with torch.cuda.device(dev):
        st = lib.dl_composite_backward(
            lse.data_ptr(), zk.data_ptr(), t_val.data_ptr(), _DT[t_val.dtype], inv_T_teacher, t_idx.data_ptr(),
            _IT[t_idx.dtype], K, offs[0], on_host, C, N, rec.data_ptr(), coef.data_ptr(), g.data_ptr(),
            g_lse.data_ptr(), g_zk.data_ptr(), stream)
        _lib.check(st, "dl_composite_backward")
        st = lib.dl_rowcoef_grad_topk(x.data_ptr(), _DT[x.dtype], x.stride(0), R, V,
                                      row_map.data_ptr() if row_map is not None else 0, t_idx.data_ptr(),
                                      _IT[t_idx.dtype], K, N, inv_T, lse.data_ptr(), g_lse.data_ptr(), g_zk.data_ptr(),
                                      gx.data_ptr(), gx.stride(0), stream)
        _lib.check(st, "dl_rowcoef_grad_topk")
    return grad


class _CompositeLoss(torch.autograd.Function):
    """The reference's composite loss of C conversations as ONE autograd node: phase 1 over the logits and the
    K-wide epilogue (dl_composite_forward_fused), and in backward their counterpart (dl_composite_backward_fused:
    the epilogue's backward inside phase 2, or dl_composite_backward + dl_rowcoef_grad_topk on wide rows).  Returns (train_loss [C], the nine
    values [C, 9]); only train_loss is differentiable, and only with respect to the logits.
    The eager path goes through this class rather than through the registered ops below (which run the
    same launches): a call through the dispatcher costs tens of microseconds of host time more, which at
    the reference's default shape (one conversation of 2048 x 32000 logits: 0.17 ms of kernels) is what
    decides whether the host keeps ahead of the device."""

    @staticmethod
    def forward(ctx, logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T: float, inv_T_teacher: float,
                alpha: float, crop: int):
        need_grad = ctx.needs_input_grad[0]          # False under torch.no_grad() (the validation loop) and for detached logits
        out, lse, zk, rec, coef = _composite_forward_raw(logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T,
                                                         inv_T_teacher, alpha, crop, need_grad)
        if need_grad:
            on_host = not isinstance(offsets, torch.Tensor)
            ctx.save_for_backward(logits, t_val, t_idx, lse, zk, rec, coef, *([row_map] if row_map is not None else []),
                                  *([] if on_host else [offsets]))
            ctx.host_offsets = offsets if on_host else None
            ctx.has_map = row_map is not None
            ctx.scalars = (inv_T, inv_T_teacher, crop)
        train = out[:, 0].clone()      # its own storage: the differentiable output must not alias the logged one
        ctx.mark_non_differentiable(out)
        return train, out

    @staticmethod
    def backward(ctx, g_train, _g_logged):
        saved = ctx.saved_tensors
        logits, t_val, t_idx, lse, zk, rec, coef = saved[:7]
        row_map = saved[7] if ctx.has_map else None
        offsets = ctx.host_offsets if ctx.host_offsets is not None else saved[-1]
        inv_T, inv_T_teacher, crop = ctx.scalars
        grad = _composite_backward_raw(logits, t_val, t_idx, lse, zk, rec, coef, g_train, offsets, row_map, inv_T,
                                       inv_T_teacher, crop)
        return (grad,) + (None,) * 10


# The same two halves as registered operators (torch.library): visible to torch.compile, FakeTensor tracing and
# torch.library.opcheck.  The forward returns what its backward needs as extra outputs; offsets are the device form.
@torch.library.custom_op("distillery_amd::composite_forward", mutates_args=())
def composite_forward_op(logits: torch.Tensor, t_val: torch.Tensor, t_idx: torch.Tensor, labels: torch.Tensor,
                         avoid: torch.Tensor, offsets: torch.Tensor, row_map: Optional[torch.Tensor], inv_T: float,
                         inv_T_teacher: float, alpha: float, crop: int = 0
                         ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(train_loss [C], nine values [C, 9], lse [N], zk [N, K], per-row records [N, 8], per-row coefficients [N, 4])."""
    out, lse, zk, rec, coef = _composite_forward_raw(logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T,
                                                     inv_T_teacher, alpha, crop, True)
    return out[:, 0].clone(), out, lse, zk, rec, coef


@composite_forward_op.register_fake
def _(logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T, inv_T_teacher, alpha, crop=0):
    N, K = t_idx.shape
    C = offsets.shape[1] - 1
    f32 = dict(dtype=torch.float32)
    return (logits.new_empty((C,), **f32), logits.new_empty((C, 9), **f32), logits.new_empty((N,), **f32),
            logits.new_empty((N, K), **f32), logits.new_empty((N, 8), **f32), logits.new_empty((N, 4), **f32))


@torch.library.custom_op("distillery_amd::composite_backward", mutates_args=())
def composite_backward_op(logits: torch.Tensor, t_val: torch.Tensor, t_idx: torch.Tensor, lse: torch.Tensor, zk: torch.Tensor,
                          rec: torch.Tensor, coef: torch.Tensor, g_train: torch.Tensor, offsets: torch.Tensor,
                          row_map: Optional[torch.Tensor], inv_T: float, inv_T_teacher: float, crop: int = 0) -> torch.Tensor:
    return _composite_backward_raw(logits, t_val, t_idx, lse, zk, rec, coef, g_train, offsets, row_map, inv_T, inv_T_teacher, crop)


@composite_backward_op.register_fake
def _(logits, t_val, t_idx, lse, zk, rec, coef, g_train, offsets, row_map, inv_T, inv_T_teacher, crop=0):
    return torch.empty_like(logits)


def _composite_op_setup(ctx, inputs, output):
    logits, t_val, t_idx, labels, avoid, offsets, row_map, inv_T, inv_T_teacher, alpha, crop = inputs
    _, _, lse, zk, rec, coef = output
    ctx.save_for_backward(logits, t_val, t_idx, lse, zk, rec, coef, offsets, *([row_map] if row_map is not None else []))
    ctx.has_map = row_map is not None
    ctx.scalars = (inv_T, inv_T_teacher, crop)


def _composite_op_backward(ctx, g_train, *_unused):
    saved = ctx.saved_tensors
    logits, t_val, t_idx, lse, zk, rec, coef, offsets = saved[:8]
    row_map = saved[8] if ctx.has_map else None
    inv_T, inv_T_teacher, crop = ctx.scalars
    if g_train is None:
        g_train = torch.zeros(offsets.shape[1] - 1, dtype=torch.float32, device=logits.device)
    grad = composite_backward_op(logits, t_val, t_idx, lse, zk, rec, coef, g_train, offsets, row_map, inv_T, inv_T_teacher, crop)
    return (grad,) + (None,) * 10


composite_forward_op.register_autograd(_composite_op_backward, setup_context=_composite_op_setup)


def composite_loss(logits: torch.Tensor, t_val: torch.Tensor, t_idx: torch.Tensor, labels: torch.Tensor,
                   avoid: torch.Tensor, offsets, row_map: Optional[torch.Tensor], inv_T: float, inv_T_teacher: float,
                   alpha: float, crop: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """(train_loss [C], nine values [C, 9]) of C conversations straight from the logits [rows, V]:
    `t_val` / `t_idx` [N, K] the stored teacher rows of all conversations back to back, `labels` int64
    and `avoid` int32 / int64 concatenated, `offsets` = three host lists (first row, first label,
    first ignore entry of every conversation, C + 1 entries each; C <= DL_MAX_HOST_CONVOS) or a device
    int32 [3, C + 1] tensor, `row_map` as for `div_topk`.  See dl_rowstats_topk / dl_composite_forward."""
    _dev(logits, "logits")
    dev = logits.device
    for name, t in (("t_val", t_val), ("t_idx", t_idx), ("labels", labels), ("avoid", avoid)):
        _dev(t, name, dev)
    if logits.dim() != 2 or logits.stride(1) != 1 or logits.dtype not in _DT:
        raise RuntimeError("logits must be [rows, V] bf16/fp16/fp32, dense along V")
    if t_val.dtype not in _DT or t_idx.dtype not in _IT or labels.dtype != torch.int64 or avoid.dtype not in _IT:
        raise RuntimeError("unsupported dtype")
    if t_idx.dim() != 2 or t_val.shape != t_idx.shape or not (t_val.is_contiguous() and t_idx.is_contiguous()
                                                             and labels.is_contiguous() and avoid.is_contiguous()):
        raise RuntimeError("t_val / t_idx must be contiguous [N, K], labels and avoid contiguous vectors")
    N = t_idx.shape[0]
    if row_map is None and N < logits.shape[0]:
        raise RuntimeError(f"{logits.shape[0]} logits rows but only {N} teacher rows and no row_map")
    if row_map is not None:
        _opt_i32(row_map, logits.shape[0], "row_map", dev)
    if isinstance(offsets, torch.Tensor):
        _dev(offsets, "offsets", dev)
        if offsets.dtype != torch.int32 or offsets.dim() != 2 or offsets.shape[0] != 3 or not offsets.is_contiguous():
            raise RuntimeError("device offsets must be a contiguous int32 [3, C + 1] tensor")
    elif len(offsets) != 3 or len(offsets[0]) - 1 > _lib.DL_MAX_HOST_CONVOS or offsets[0][-1] != N:
        raise RuntimeError("host offsets: three lists of C + 1 entries, C <= DL_MAX_HOST_CONVOS, rows ending at N")
    if torch.compiler.is_compiling():      # traced: the registered operators (device offsets only)
        if not isinstance(offsets, torch.Tensor):
            offsets = torch.tensor(offsets, dtype=torch.int32, device=dev)
        res = composite_forward_op(logits, t_val, t_idx, labels, avoid, offsets, row_map, float(inv_T), float(inv_T_teacher),
                                   float(alpha), int(crop))
        return res[0], res[1].detach()
    return _CompositeLoss.apply(logits, t_val, t_idx, labels, avoid, offsets, row_map, float(inv_T), float(inv_T_teacher),
                                float(alpha), int(crop))


def reduce_sum(values: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Deterministic sum(values) * scale as a 0-d fp32 tensor."""
    _dev(values, "values")
    v = values.contiguous().view(-1)
    if v.dtype != torch.float32:
        raise RuntimeError("reduce_sum takes fp32 values")
    out = torch.empty((), dtype=torch.float32, device=v.device)
    with torch.cuda.device(v.device):
        st = _lib.load().dl_reduce_sum(v.data_ptr(), v.numel(), scale, out.data_ptr(), _stream_ptr(v.device))
    _lib.check(st, "dl_reduce_sum")
    return out


def copy16(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Streaming copy of src's bytes into dst (the calibration kernel for HBM counters)."""
    _dev(src, "src"), _dev(dst, "dst", src.device)
    n = src.numel() * src.element_size()
    if not (src.is_contiguous() and dst.is_contiguous()) or dst.numel() * dst.element_size() != n:
        raise RuntimeError("copy16 needs two contiguous buffers of the same byte size")
    with torch.cuda.device(src.device):
        st = _lib.load().dl_copy16(src.data_ptr(), dst.data_ptr(), n, _stream_ptr(src.device))
    _lib.check(st, "dl_copy16")


def copy_rows(src: torch.Tensor, dst: torch.Tensor, threads: int, chunks: int, parts_on_one_xcd: bool = True,
              wave_major: bool = True, lds_kb: int = 0) -> None:
    """Copy of a contiguous [rows, width] tensor in the access shape of the row kernels (dl_copy_rows):
    the yardstick for what a bare copy reaches with `threads` x `chunks` 16-byte chunks per workgroup.
    `wave_major`: every wave owns `chunks` KiB in one piece; `lds_kb`: LDS held per workgroup, which
    bounds the workgroups per CU at 160 / lds_kb."""
    _dev(src, "src"), _dev(dst, "dst", src.device)
    if src.dim() != 2 or not (src.is_contiguous() and dst.is_contiguous()) or src.shape != dst.shape or src.dtype != dst.dtype:
        raise RuntimeError("copy_rows needs two contiguous [rows, width] tensors of one shape and dtype")
    if not 0 <= int(lds_kb) <= 64:
        raise ValueError("lds_kb must be 0..64")
    flags = (1 if parts_on_one_xcd else 0) | (2 if wave_major else 0) | (int(lds_kb) << 8)
    with torch.cuda.device(src.device):
        st = _lib.load().dl_copy_rows(src.data_ptr(), dst.data_ptr(), src.shape[0], src.shape[1] * src.element_size(), int(threads),
                                      int(chunks), flags, _stream_ptr(src.device))
    _lib.check(st, "dl_copy_rows")

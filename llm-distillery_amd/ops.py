"""Tensor-level wrappers over the C ABI.  PyTorch supplies device memory and the
stream; all arithmetic happens in the HIP kernels.  No fallbacks: a CPU tensor or
a missing library raises."""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.float32: _lib.DL_F32, torch.bfloat16: _lib.DL_BF16, torch.float16: _lib.DL_F16}
_IT = {torch.int32: _lib.DL_I32, torch.int64: _lib.DL_I64}
KINDS = {"fkl": _lib.DL_FKL, "rkl": _lib.DL_RKL, "jsd": _lib.DL_JSD}


def _stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _dev(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); this library has no CPU path")


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
             want_grad: bool = True, grad_out: torch.Tensor | None = None):
    """Per-token forward ("fkl") or reverse ("rkl") KL against a top-K teacher and,
    in the same launch, d(sum of row losses)/d(logits) * grad_scale.

    logits [..., V] bf16/fp16/fp32 (native model dtype, rows evenly strided);
    t_val/t_idx [N, K] stored teacher log-probs and ids; row_map int32 [rows]
    gives the teacher row of each logits row (negative = masked row).
    Returns (row_loss fp32 [rows], grad like logits or None).
    """
    if kind not in ("fkl", "rkl"):
        raise ValueError("kind must be 'fkl' or 'rkl' for a top-K teacher")
    _dev(logits, "logits"), _dev(t_val, "t_val"), _dev(t_idx, "t_idx")
    x = _rows_2d(logits)
    R, V = x.shape
    dev = x.device
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
        grad = grad_out if grad_out is not None else torch.empty((R, V), dtype=x.dtype, device=dev)
        if grad.shape != (R, V) or grad.dtype != x.dtype or grad.stride(1) != 1 or grad.device != dev:
            raise RuntimeError("grad_out must match logits as a [rows, V] tensor")
        g_ptr, g_stride = grad.data_ptr(), grad.stride(0)
    lib = _lib.load()
    ws_bytes = lib.dl_div_topk_workspace_bytes(KINDS[kind], _DT[x.dtype], R, V) if want_grad else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        st = lib.dl_div_topk(KINDS[kind], x.data_ptr(), _DT[x.dtype], x.stride(0), R, V, rm_ptr,
                             t_val.data_ptr(), _DT[t_val.dtype], t_idx.data_ptr(), _IT[t_idx.dtype], K, N,
                             cnt_ptr, 1.0 / T, 1.0 / (T if teacher_T is None else teacher_T), grad_scale,
                             row_loss.data_ptr(), g_ptr, g_stride,
                             ws.data_ptr() if ws is not None else 0, ws_bytes, _stream_ptr(dev))
    _lib.check(st, "dl_div_topk")
    if grad is not None and logits.dim() != 2 and grad_out is None:
        grad = grad.view(logits.shape)
    return row_loss, grad


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
    _dev(src, "src"), _dev(dst, "dst")
    n = src.numel() * src.element_size()
    if not (src.is_contiguous() and dst.is_contiguous()) or dst.numel() * dst.element_size() != n:
        raise RuntimeError("copy16 needs two contiguous buffers of the same byte size")
    with torch.cuda.device(src.device):
        st = _lib.load().dl_copy16(src.data_ptr(), dst.data_ptr(), n, _stream_ptr(src.device))
    _lib.check(st, "dl_copy16")


def set_option(name: str, value: int) -> None:
    """Process-wide tuning / test hooks of the library ("split_parts", "spin_limit")."""
    _lib.check(_lib.load().dl_set_option(name.encode(), int(value)), f"dl_set_option({name!r})")

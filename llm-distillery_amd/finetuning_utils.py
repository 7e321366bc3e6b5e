"""Drop-in for the loss entry point of the reference, `utils/finetuning_utils.py`.

`calculate_divergence` keeps the reference's name, positional arguments and its
nine result keys (utils/finetuning_utils.py:47,112-122).  The two full-vocabulary
steps of the reference -- `F.log_softmax` over V and `torch.gather` at the teacher
ids (:88,:92), and their autograd replay -- run in the HIP kernels behind the
`distillery_amd::rowstats_topk` custom op; what is left is K-wide arithmetic on
[N, K] tensors, written with the same torch routines the reference uses so that
its quirks carry over unchanged (crop rule and valid-mean fill of the top-K cross
entropy, pad-by-one and non-detached max of the alpha weighting).

`distill_loss` is the extended entry point: it takes the model's logits in their
native dtype, un-gathered, with the row selection and the temperature folded
into the kernels (classes/student/model.py:408,420-421).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor

from . import ops
from .losses import LossDict

LOSS_KEYS = ("train_loss", "custom loss", "CE loss", "kl_div", "reverse kl_div",
             "weighted kl_div", "weighted rev. kl_div", "teacher CE loss", "CE diff")


def _kl_per_token(inp_logp: Tensor, tgt_logp: Tensor) -> Tensor:
    return F.kl_div(inp_logp, tgt_logp, reduction="none", log_target=True).sum(dim=-1)


def _topk_cross_entropy(logprobs: Tensor, labels: Tensor, indices: Tensor, ignore_rows: Tensor) -> Tensor:
    """utils/finetuning_utils.py:68-84 on K-wide tensors."""
    stop = -1 if labels.size(-1) < logprobs.size(0) else 0
    hit = labels.unsqueeze(-1) == indices[:stop]
    hit[ignore_rows] = False
    valid = hit.any(dim=-1)
    # masked sums instead of the reference's boolean-mask gathers (`picked[valid] = logprobs[hit]`,
    # `picked[~valid] = picked[valid].mean()`): the same values, but nothing here makes the host wait
    # for the device.  A row's ids are distinct, so at most one entry per row is hit.
    own = torch.where(hit, logprobs[:stop], torch.zeros((), dtype=logprobs.dtype, device=logprobs.device)).sum(dim=-1)
    mean_valid = own.sum() / valid.sum()              # no valid row: 0 / 0 = NaN, like the mean of nothing
    return -torch.where(valid, own, mean_valid)


def _alpha_weighted(per_token: Tensor, alpha, ce_per_token: Tensor) -> Tensor:
    """utils/finetuning_utils.py:58-66."""
    if ce_per_token.numel() < per_token.numel():
        ce_per_token = torch.cat((ce_per_token, torch.zeros(1, device=ce_per_token.device)))
    w = (per_token / per_token.max() + 1).pow(alpha) + ce_per_token
    return (per_token * w).mean()


def _assemble(s_sup: Tensor, t: Tensor, indices: Tensor, labels: Tensor, alpha, avoid: Tensor) -> dict[str, Tensor]:
    ce_s = _topk_cross_entropy(s_sup, labels, indices, avoid)
    ce_t = _topk_cross_entropy(t, labels, indices, avoid)
    ce_diff = ce_s - ce_t
    ce_pos = torch.where(ce_diff < 0, torch.zeros_like(ce_diff), ce_diff)
    kl = _kl_per_token(s_sup, t)
    rkl = _kl_per_token(t, F.log_softmax(s_sup, dim=-1))
    wkl = _alpha_weighted(kl, alpha, ce_pos)
    wrkl = _alpha_weighted(rkl, alpha, ce_pos)
    total = (wkl + wrkl) / 2
    return dict(zip(LOSS_KEYS, (total, total, ce_s.mean(), kl.mean(), rkl.mean(), wkl, wrkl, ce_t.mean(),
                                ce_diff.mean())))


def _packed_rows(tensors) -> Tensor:
    """The row-wise concatenation of 2-D tensors; no copy when they already lie back to back in
    memory (consecutive slices of one packed tensor, as `teachers_from_outgoing_batch` returns)."""
    if len(tensors) == 1:
        return tensors[0].contiguous()
    first = tensors[0]
    at = first.data_ptr()
    for t in tensors:
        if not t.is_contiguous() or t.dtype != first.dtype or t.data_ptr() != at or \
                t.untyped_storage().data_ptr() != first.untyped_storage().data_ptr():
            return torch.cat(tensors, dim=0)
        at += t.numel() * t.element_size()
    rows = sum(t.shape[0] for t in tensors)
    return torch.as_strided(first, (rows, first.shape[1]), (first.shape[1], 1))


def _fusable(counts, labels, alpha) -> bool:
    """The fused epilogue covers what the reference's code can run: a Python-number alpha and, per
    conversation, exactly one label fewer than rows (anything else raises inside the reference's
    cross entropy or weighting, and the torch form below reproduces that)."""
    return not isinstance(alpha, Tensor) and all(lab.dim() == 1 and lab.numel() == n - 1 for n, lab in zip(counts, labels))


def _fused_dicts(x: Tensor, row_map, inv_T: float, crop: int, counts, t_vals, t_idxs, labels, avoids,
                 inv_T_teacher: float, alpha):
    """Nine-key dicts of all conversations from one autograd node (`ops.composite_loss`: one phase-1
    launch over the logits, the K-wide epilogue, and in backward their two counterparts);
    `train_loss` / `custom loss` carry the autograd history, the seven logged values do not (the
    reference's `Losses.add_losses` detaches them before any use, classes/losses.py:35-37).
    The conversations' row / label / ignore offsets travel with the launch: nothing is uploaded."""
    dev = x.device
    C = len(counts)
    n_lab = [int(lab.numel()) for lab in labels]
    n_avoid = [int(a.numel()) for a in avoids]
    if C <= ops._lib.DL_MAX_HOST_CONVOS:
        offs = ([0] + list(_cumsum(counts)), [0] + list(_cumsum(n_lab)), [0] + list(_cumsum(n_avoid)))
    else:
        offs = torch.tensor([[0] + list(_cumsum(counts)), [0] + list(_cumsum(n_lab)), [0] + list(_cumsum(n_avoid))],
                            dtype=torch.int32).to(dev)
    lab_cat = (torch.cat([lab.to(torch.int64) for lab in labels]) if C > 1 else labels[0].to(torch.int64)).contiguous()
    if C > 1:
        avoid_cat = torch.cat([a.to(torch.int64) for a in avoids])
    else:
        avoid_cat = avoids[0] if avoids[0].dtype in ops._IT else avoids[0].to(torch.int64)
    train, nine = ops.composite_loss(x, _packed_rows(t_vals), _packed_rows(t_idxs), lab_cat, avoid_cat.contiguous(), offs,
                                     row_map, inv_T, inv_T_teacher, alpha, crop)
    out = []
    for c in range(C):
        row = nine[c]
        d = LossDict(zip(LOSS_KEYS, row.unbind(0)))
        d["train_loss"] = d["custom loss"] = train[c]      # one tensor under both keys, with its graph, as in the reference
        d.packed, d.keys_packed = row, LOSS_KEYS
        out.append(d)
    return out


def _cumsum(values):
    total = 0
    for v in values:
        total += int(v)
        yield total


def calculate_divergence(student_logits: Tensor, teacher_logits: Tensor, indices: Tensor | None,
                         convo_CE_tokens: Tensor, alpha, avoid_indices: Tensor) -> dict[str, Tensor]:
    """Same contract as the reference's `calculate_divergence`: `student_logits` [N, V] (already
    divided by the temperature, any floating dtype), `teacher_logits` [N, K] stored log-probs divided
    by the temperature, `indices` [N, K], the cross-entropy labels and the rows to ignore.  Returns
    the nine-key dict; `train_loss` carries autograd history back to `student_logits`.

    `indices=None` (dense teacher) raises, as the reference's own training path does.
    """
    if indices is None:
        raise TypeError("calculate_divergence needs top-K indices: the dense-teacher form of the reference "
                        "composite is not executable (use dense_divergence for dense teachers)")
    n = min(student_logits.size(0), teacher_logits.size(0), indices.size(0))
    idx = indices[:n]
    # Rows beyond n are masked through the row map instead of sliced away: the backward of a slice
    # would zero-fill a second [N, V] buffer and copy the gradient into it.
    row_map = None
    if n < student_logits.size(0):
        row_map = torch.full((student_logits.size(0),), -1, dtype=torch.int32, device=student_logits.device)
        row_map[:n] = torch.arange(n, dtype=torch.int32, device=student_logits.device)
    labels = convo_CE_tokens[:n]
    if _fusable([n], [labels], alpha) and teacher_logits.dtype in ops._DT:
        return _fused_dicts(student_logits, row_map, 1.0, 0, [n], [teacher_logits[:n]], [idx], [labels], [avoid_indices], 1.0,
                            alpha)[0]
    lse, zk = ops.rowstats_topk(student_logits, idx, row_map, 1.0)
    s_sup = zk - lse.unsqueeze(-1)                       # log_softmax over V, gathered at the ids
    t = F.log_softmax(teacher_logits[:n].float(), dim=-1)
    return _assemble(s_sup, t, idx, labels, alpha, avoid_indices)


def distill_loss(model_logits: Tensor, content_rows: Tensor, teacher_logprobs: Tensor, indices: Tensor,
                 convo_CE_tokens: Tensor, alpha, avoid_indices: Tensor, temperature: float = 1.0,
                 crop_to_size: int | None = None, teacher_temperature: float | None = None) -> dict[str, Tensor]:
    """The composite loss of one conversation straight from the model output.

    model_logits [S, V_model] in the model's dtype; `content_rows` int [N] positions of the content
    tokens (classes/student/model.py:87-91); `teacher_logprobs` [N, K] as stored (not yet divided by
    the temperature).  Slice, cast, temperature and row selection happen inside the kernels.
    `teacher_temperature=1` reproduces the validation loop, which scales only the student
    (classes/student/model.py:501-502).
    """
    x = model_logits
    S = x.shape[0]
    n = min(content_rows.numel(), teacher_logprobs.size(0), indices.size(0))
    row_map = torch.full((S,), -1, dtype=torch.int32, device=x.device)
    row_map[content_rows[:n].long()] = torch.arange(n, dtype=torch.int32, device=x.device)
    tT = temperature if teacher_temperature is None else teacher_temperature
    labels = convo_CE_tokens[:n]
    if _fusable([n], [labels], alpha) and teacher_logprobs.dtype in ops._DT:
        return _fused_dicts(x, row_map, 1.0 / temperature, int(crop_to_size or 0), [n], [teacher_logprobs[:n]], [indices[:n]],
                            [labels], [avoid_indices], 1.0 / tT, alpha)[0]
    lse, zk = ops.rowstats_topk(x, indices[:n], row_map, 1.0 / temperature, int(crop_to_size or 0))
    s_sup = zk - lse.unsqueeze(-1)
    t = F.log_softmax(teacher_logprobs[:n].float() / tT, dim=-1)
    return _assemble(s_sup, t, indices[:n], labels, alpha, avoid_indices)


def distill_loss_batch(model_logits: Tensor, convos, alpha, temperature: float = 1.0,
                       crop_to_size: int | None = None, teacher_temperature: float | None = None,
                       row_map: Tensor | None = None) -> list[dict[str, Tensor]]:
    """The per-conversation composite losses of a whole batch with ONE pass over the logits.

    Replaces the Python loop of classes/student/model.py:415-436 (one `calculate_divergence` call,
    i.e. one full-vocabulary log-softmax + gather and its autograd replay, per conversation): the
    V-wide work of all conversations runs as a single phase-1 launch over `model_logits`
    [B, S, V_model] and, in backward, a single phase-2 launch; only the K-wide epilogue stays per
    conversation, because its weights (max of the per-token KL, mean of the valid cross entropies)
    are per-conversation quantities in the reference.

    `convos[i]` = (content_rows int [N_i] positions inside sequence i, teacher_logprobs [N_i, K] as
    stored, indices [N_i, K], convo_CE_tokens [N_i - 1], avoid_indices).  All conversations share K.
    Returns one nine-key dict per conversation, in order; feed them to `Losses.add_losses` as the
    reference does and call `Losses.backward` once.  `row_map` (int32 [B * S], from `BatchIndex`)
    saves rebuilding the row map on the device; it is ignored if a teacher holds fewer rows than its
    conversation has content rows.
    """
    if model_logits.dim() != 3:
        raise RuntimeError("model_logits must be [batch, seq, vocab]")
    B, S, _ = model_logits.shape
    if len(convos) != B:
        raise ValueError(f"{len(convos)} conversations for a batch of {B} sequences")
    x = model_logits
    dev = x.device
    counts = [min(rows.numel(), t_lp.size(0), idx.size(0)) for rows, t_lp, idx, _, _ in convos]
    if row_map is None or row_map.numel() != B * S or any(n != rows.numel() for n, (rows, *_) in zip(counts, convos)):
        row_map = torch.full((B * S,), -1, dtype=torch.int32, device=dev)
        where = torch.cat([rows[:n].long() + b * S for b, ((rows, *_), n) in enumerate(zip(convos, counts))])
        row_map[where] = torch.arange(where.numel(), dtype=torch.int32, device=dev)      # one scatter for the batch
    idx_cat = _packed_rows([idx[:n] for (_, _, idx, _, _), n in zip(convos, counts)])
    tT = temperature if teacher_temperature is None else teacher_temperature
    labels_all = [labels[:n] for (_, _, _, labels, _), n in zip(convos, counts)]
    if _fusable(counts, labels_all, alpha) and all(c[1].dtype in ops._DT for c in convos):
        return _fused_dicts(ops._rows_2d(x), row_map, 1.0 / temperature, int(crop_to_size or 0), counts,
                            [t_lp[:n] for (_, t_lp, _, _, _), n in zip(convos, counts)], [idx_cat], labels_all,
                            [c[4] for c in convos], 1.0 / tT, alpha)
    lse, zk = ops.rowstats_topk(ops._rows_2d(x), idx_cat, row_map, 1.0 / temperature, int(crop_to_size or 0))
    out, base = [], 0
    for (rows, t_lp, idx, labels, avoid), n in zip(convos, counts):
        s_sup = zk[base:base + n] - lse[base:base + n].unsqueeze(-1)
        t = F.log_softmax(t_lp[:n].float() / tT, dim=-1)
        out.append(_assemble(s_sup, t, idx[:n], labels[:n], alpha, avoid))
        base += n
    return out


def distill_loss_batch_indexed(model_logits: Tensor, index, tokens: Tensor, teachers, alpha,
                               temperature: float = 1.0, crop_to_size: int | None = None,
                               teacher_temperature: float | None = None) -> list[dict[str, Tensor]]:
    """`distill_loss_batch` from a `BatchIndex` (all row / label / ignore indices of the batch built
    and uploaded once), the batch's token ids [B, S] and `teachers[b]` = (stored log-probs [N_b, K],
    ids [N_b, K]).  Covers classes/student/model.py:415-436 including the index construction of
    `:87-116` and the label gather of `:423`."""
    labels = index.labels(tokens)
    convos = [(index.rows[b], t_lp, idx, labels[b], index.avoid[b]) for b, (t_lp, idx) in enumerate(teachers)]
    return distill_loss_batch(model_logits, convos, alpha, temperature, crop_to_size, teacher_temperature,
                              row_map=index.row_map)


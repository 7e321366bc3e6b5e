"""Row and label index construction for a batch of conversations.

Mirrors `StudentModel._get_content_indices_tensor` (classes/student/model.py:87-91) and
`StudentModel._get_CE_indices_tensor` (classes/student/model.py:93-116), which the reference runs per
conversation with one host-to-device copy each, and adds a batched form: every index array of a
batch is built in one host pass and uploaded in ONE copy, in the layout `distill_loss_batch` and
the kernels' `row_map` argument consume.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

Ranges = Sequence[tuple[int, int]]


def content_rows(content_ranges: Ranges) -> np.ndarray:
    """Positions of the content tokens of one conversation: the concatenation of
    `arange(start, end)` over its content ranges (classes/student/model.py:87-91).
    Raises ValueError for an empty range list, like the reference's `np.concatenate`."""
    return np.concatenate([np.arange(a, b, dtype=np.int64) for a, b in content_ranges])


def ce_rows(content_ranges: Ranges, context_len: int, convo_len: int) -> tuple[np.ndarray, np.ndarray]:
    """Label positions and cross-entropy rows to ignore (classes/student/model.py:93-116).

    The label of content row `p` is the token at `p + 1`.  Ranges that start at or beyond the
    context length are skipped.  With more than one range the last row of every range is ignored
    (its label is the first token of the next turn's header).  A final label at or after the
    conversation length is dropped, together with the last ignore entry."""
    labels, avoid = [], []
    several = len(content_ranges) > 1
    first = 0                                   # row number (among the content rows) of the range's first row
    for start, end in content_ranges:
        if start + 1 > context_len:
            continue
        labels.append(np.arange(start + 1, end + 1, dtype=np.int64))
        last = first + (end - start) - 1
        if several:
            avoid.append(last)
        first = last + 1
    lab = np.concatenate(labels)
    if lab[-1] >= convo_len:
        lab = lab[:-1]
        if avoid:
            avoid.pop()
    return lab, np.asarray(avoid, dtype=np.int64)


class BatchIndex:
    """All index arrays of one batch, built on the host in one pass and uploaded in one copy.

    `content_ranges[b]` are the content ranges of sequence b of a `[B, S, V]` batch, `lengths[b]`
    its unpadded token count.  Device tensors afterwards:

    * `row_map` int32 [B * S]: teacher row of every logits row (rows are numbered through the batch
      in conversation order), -1 for rows without content — the `row_map` of the loss kernels;
    * `rows[b]` int64 [N_b]: content positions inside sequence b;
    * `label_pos[b]` int64: positions whose tokens are the cross-entropy labels of conversation b;
    * `avoid[b]` int64: content rows of conversation b to ignore in the cross entropy;
    * `counts[b]`, `offsets[b]`: N_b and the first teacher row of conversation b (host ints).
    """

    def __init__(self, content_ranges: Sequence[Ranges], lengths: Sequence[int], seq_len: int, context_len: int,
                 device):
        if len(content_ranges) != len(lengths):
            raise ValueError("one length per conversation")
        B, S = len(content_ranges), int(seq_len)
        rows = [content_rows(r) for r in content_ranges]
        ce = [ce_rows(r, context_len, n) for r, n in zip(content_ranges, lengths)]
        for b, r in enumerate(rows):
            if r.size and (r.min() < 0 or r.max() >= S):
                raise ValueError(f"conversation {b}: content range outside the sequence length {S}")
        self.counts = [int(r.size) for r in rows]
        self.offsets = [0] * B
        row_map = np.full(B * S, -1, dtype=np.int64)
        base = 0
        for b, r in enumerate(rows):
            self.offsets[b] = base
            row_map[b * S + r] = np.arange(base, base + r.size)
            base += r.size
        self.total = base
        parts = [row_map] + rows + [c[0] for c in ce] + [c[1] for c in ce]
        sizes = [p.size for p in parts]
        host = torch.from_numpy(np.concatenate(parts))
        dev = torch.device(device)
        if dev.type == "cuda":
            host = host.pin_memory()
        flat = host.to(dev, non_blocking=True)
        cuts = np.cumsum([0] + sizes)
        pieces = [flat[cuts[i]:cuts[i + 1]] for i in range(len(parts))]
        self.row_map = pieces[0].to(torch.int32)
        self.rows = pieces[1:1 + B]
        self.label_pos = pieces[1 + B:1 + 2 * B]
        self.avoid = pieces[1 + 2 * B:1 + 3 * B]
        self.seq_len = S

    def labels(self, tokens: torch.Tensor) -> list[torch.Tensor]:
        """Cross-entropy labels per conversation from the batch's token ids [B, S]
        (classes/student/model.py:423: `batch_tokenized[i][CE_indices]`)."""
        return [tokens[b][pos] for b, pos in enumerate(self.label_pos)]


def teachers_from_outgoing_batch(padded_batch: np.ndarray, batch_indices: Sequence[np.ndarray],
                                 batch_padding: Sequence[int], device, storage: bool = True):
    """Device-side teacher tensors from the tuple the dataset manager ships per batch
    (`H5DataManager._make_outgoing_batch`, classes/data_manager.py:332-353): `padded_batch`
    [B, max_len, K] log-probs zero-padded to the longest conversation, `batch_indices[b]` [N_b, K] ids,
    `batch_padding[b]` = N_b.  Zero padding means log-prob 0, which is why the reference must slice
    `[:batch_padding[i]]` before use (classes/student/model.py:421); here the padding never reaches
    the device: the valid rows of all conversations are packed back to back and uploaded in two copies.

    `storage=True` ships the dataset's own dtypes (fp16 log-probs — the cast back is exact because
    that is what the file holds, classes/data_manager.py:306 — and int32 ids), a third of the
    reference's fp32 + int64 bytes; the kernels read both layouts.
    Returns `teachers` = [(log-probs [N_b, K], ids [N_b, K])] as views of the two packed tensors,
    in the form `distill_loss_batch_indexed` takes."""
    B = len(batch_padding)
    if padded_batch.shape[0] != B or len(batch_indices) != B:
        raise ValueError("one padding and one index array per conversation")
    counts = [int(n) for n in batch_padding]
    for b, n in enumerate(counts):
        if n > padded_batch.shape[1] or batch_indices[b].shape[0] < n:
            raise ValueError(f"conversation {b}: {n} rows announced, fewer shipped")
    vals = np.concatenate([padded_batch[b, :n] for b, n in enumerate(counts)], axis=0)
    ids = np.concatenate([np.asarray(batch_indices[b][:n]) for b, n in enumerate(counts)], axis=0)
    if ids.size and (ids.min() < 0 or ids.max() > np.iinfo(np.int32).max):
        raise ValueError("token ids outside int32")
    vals = vals.astype(np.float16 if storage else np.float32, copy=False)
    ids = ids.astype(np.int32 if storage else np.int64, copy=False)
    dev = torch.device(device)
    hv, hi = torch.from_numpy(np.ascontiguousarray(vals)), torch.from_numpy(np.ascontiguousarray(ids))
    if dev.type == "cuda":
        hv, hi = hv.pin_memory(), hi.pin_memory()
    dv, di = hv.to(dev, non_blocking=True), hi.to(dev, non_blocking=True)
    cuts = np.cumsum([0] + counts)
    return [(dv[cuts[b]:cuts[b + 1]], di[cuts[b]:cuts[b + 1]]) for b in range(B)]

"""Host index construction of the product (content rows, label positions, ignore rows, batch row map)
against the oracle's restatement of classes/student/model.py:87-116 and against a position-by-position
brute force; bit-exact."""
import numpy as np
import pytest
import torch

import llm_distillery_amd.batch_index as BI
from oracle import oracle as O

CASES = [
    ([(3, 7), (10, 14)], 2048, 20),
    ([(3, 7), (10, 14)], 2048, 14),        # last label falls off the conversation: dropped with its ignore entry
    ([(2, 6)], 2048, 6),                   # single range: nothing ignored
    ([(0, 5), (9, 10), (30, 47)], 2048, 64),
    ([(0, 5), (9, 10), (30, 47)], 20, 64),   # a range that starts beyond the context length is skipped
    ([(5, 6)], 2048, 7),
]


def _brute(ranges, context_len, convo_len):
    """Row by row: which positions are content, what each row's label position is, which rows end a turn."""
    rows, labels, avoid = [], [], []
    kept = [(a, b) for a, b in ranges if a + 1 <= context_len]
    n = 0
    for a, b in kept:
        for pos in range(a, b):
            labels.append(pos + 1)
            if pos == b - 1 and len(ranges) > 1:
                avoid.append(n)
            n += 1
    for a, b in ranges:
        rows.extend(range(a, b))
    if labels[-1] >= convo_len:
        labels.pop()
        if avoid:
            avoid.pop()
    return rows, labels, avoid


@pytest.mark.parametrize("ranges,ctx,clen", CASES)
def test_rows_labels_and_ignore_rows(ranges, ctx, clen):
    rows = BI.content_rows(ranges)
    lab, avoid = BI.ce_rows(ranges, ctx, clen)
    assert rows.dtype == np.int64 and lab.dtype == np.int64 and avoid.dtype == np.int64
    assert rows.tolist() == O.content_indices(ranges).tolist()
    olab, oavoid = O.ce_indices(ranges, ctx, clen)
    assert lab.tolist() == olab.tolist() and avoid.tolist() == oavoid.tolist()
    brows, blab, bavoid = _brute(ranges, ctx, clen)
    assert rows.tolist() == brows and lab.tolist() == blab and avoid.tolist() == bavoid


def test_empty_range_list_raises_like_numpy_concatenate():
    with pytest.raises(ValueError):
        BI.content_rows([])
    with pytest.raises(ValueError):
        BI.ce_rows([(5000, 5010)], 2048, 6000)      # every range skipped: the reference concatenates nothing


def test_batch_index_layout():
    specs = [[(4, 20), (30, 41)], [(0, 55)], [(10, 16), (20, 30), (44, 59)]]
    lens = [41, 55, 59]
    S = 60
    ix = BI.BatchIndex(specs, lens, S, 2048, "cpu")
    assert ix.row_map.dtype == torch.int32 and ix.row_map.numel() == 3 * S
    expect = np.full(3 * S, -1)
    base = 0
    for b, sp in enumerate(specs):
        r = O.content_indices(sp)
        expect[b * S + r] = np.arange(base, base + r.size)
        assert ix.rows[b].tolist() == r.tolist() and ix.offsets[b] == base and ix.counts[b] == r.size
        lab, avoid = O.ce_indices(sp, 2048, lens[b])
        assert ix.label_pos[b].tolist() == lab.tolist() and ix.avoid[b].tolist() == avoid.tolist()
        base += r.size
    assert ix.row_map.tolist() == expect.tolist() and ix.total == base
    tokens = torch.arange(3 * S).reshape(3, S)
    for b, lab in enumerate(ix.labels(tokens)):
        assert lab.tolist() == (b * S + ix.label_pos[b]).tolist()
    with pytest.raises(ValueError):
        BI.BatchIndex([[(0, 70)]], [70], S, 2048, "cpu")


def test_teachers_from_outgoing_batch_drops_the_zero_padding():
    # the tuple classes/data_manager.py:332-353 ships: zero-padded fp32 [B, max_len, K], ids and lengths
    rng = np.random.default_rng(0)
    K, lens = 6, [5, 9, 1]
    stored = [np.log(rng.random((n, K))).astype(np.float16) for n in lens]          # what the file holds
    ids = [rng.integers(0, 50000, (n, K)).astype(np.int64) for n in lens]
    padded = np.array([np.pad(d.astype(np.float32), ((0, max(lens) - len(d)), (0, 0))) for d in stored])
    teachers = BI.teachers_from_outgoing_batch(padded, ids, lens, "cpu")
    for (v, i), d, ix in zip(teachers, stored, ids):
        assert v.dtype == torch.float16 and i.dtype == torch.int32
        assert np.array_equal(v.numpy(), d) and np.array_equal(i.numpy(), ix)       # fp32 -> fp16 is exact here
    wide = BI.teachers_from_outgoing_batch(padded, ids, lens, "cpu", storage=False)
    assert wide[1][0].dtype == torch.float32 and wide[1][1].dtype == torch.int64
    assert np.array_equal(wide[1][0].numpy(), padded[1, :9])
    with pytest.raises(ValueError):
        BI.teachers_from_outgoing_batch(padded, ids, [5, 10, 1], "cpu")

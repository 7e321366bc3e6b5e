"""Property tests (hypothesis) of the index handling on the CPU side: the oracle's merge / remap
against a dict brute force under duplicate and colliding ids, dropped ids, all-dropped rows and
K larger than the number of distinct ids; the product's host index construction against a
position-by-position brute force on random content ranges; the C++ byte trie against the dict
brute force on random byte vocabularies."""
import numpy as np
from hypothesis import given, settings, strategies as st

import llm_distillery_amd.batch_index as BI
from oracle import oracle as O

SET = settings(max_examples=60, deadline=None, derandomize=True)


@st.composite
def sparse_teachers(draw):
    n_teachers = draw(st.integers(1, 3))
    K = draw(st.integers(1, 6))
    Vt = draw(st.integers(2, 12))
    Vs = draw(st.integers(1, 8))
    rows = draw(st.integers(1, 3))
    idxs = [np.array(draw(st.lists(st.lists(st.integers(-1, Vt), min_size=K, max_size=K), min_size=rows, max_size=rows)),
                     dtype=np.int64) for _ in range(n_teachers)]                      # duplicates and ids outside [0, Vt) allowed
    vals = [np.log(np.array(draw(st.lists(st.lists(st.floats(0.01, 1.0), min_size=K, max_size=K), min_size=rows,
                                          max_size=rows)), dtype=np.float32)) for _ in range(n_teachers)]
    weights = [draw(st.floats(0.1, 1.0)) for _ in range(n_teachers)]
    id_map = np.array(draw(st.lists(st.integers(-1, Vs - 1), min_size=Vt, max_size=Vt)), dtype=np.int32)
    return vals, idxs, weights, id_map, Vs


@SET
@given(sparse_teachers())
def test_merge_remap_equals_dict_bruteforce(case):
    vals, idxs, weights, id_map, Vs = case
    rows = O.merge_remap_rows(vals, idxs, weights, id_map)
    Vt = id_map.size
    for r, (ids, mass, logq) in enumerate(rows):
        acc: dict[int, float] = {}
        for v, ix, w in zip(vals, idxs, weights):
            for k in range(ix.shape[1]):
                t = int(ix[r, k])
                if 0 <= t < Vt and id_map[t] >= 0:
                    s = int(id_map[t])
                    acc[s] = acc.get(s, 0.0) + float(np.float32(w) * np.exp(v[r, k]))
        assert ids.tolist() == sorted(acc)                       # survivors, ascending, no duplicates
        assert all(0 <= s < Vs for s in ids)
        np.testing.assert_allclose(mass, [acc[s] for s in sorted(acc)], rtol=1e-5)
        if ids.size:
            np.testing.assert_allclose(np.exp(logq.astype(np.float64)).sum(), 1.0, rtol=1e-5)   # renormalised
    ids_p, lq_p, cnt_p = O.merge_remap_padded(vals, idxs, weights, id_map)
    for r, (ids, _, _) in enumerate(rows):
        assert cnt_p[r] == ids.size and (ids_p[r, ids.size:] == -1).all() and np.isneginf(lq_p[r, ids.size:]).all()


@st.composite
def content_ranges(draw):
    n = draw(st.integers(1, 5))
    cuts = sorted(draw(st.lists(st.integers(0, 60), min_size=2 * n, max_size=2 * n, unique=True)))
    ranges = [(cuts[2 * i], cuts[2 * i + 1]) for i in range(n)]
    ctx = draw(st.integers(ranges[0][0] + 1, 70))                 # the first range always starts inside the context
    last_label = max(b for a, b in ranges if a + 1 <= ctx)
    clen = draw(st.integers(max(1, last_label - 1), 70))
    return ranges, ctx, clen


@SET
@given(content_ranges())
def test_rows_and_labels_equal_bruteforce(case):
    ranges, ctx, clen = case
    rows = BI.content_rows(ranges)
    lab, avoid = BI.ce_rows(ranges, ctx, clen)
    assert rows.tolist() == [p for a, b in ranges for p in range(a, b)]
    olab, oavoid = O.ce_indices(ranges, ctx, clen)
    assert lab.tolist() == olab.tolist() and avoid.tolist() == oavoid.tolist()
    exp_lab, exp_avoid, n = [], [], 0
    for a, b in ranges:
        if a + 1 > ctx:
            continue
        for pos in range(a, b):
            exp_lab.append(pos + 1)
            if pos == b - 1 and len(ranges) > 1:
                exp_avoid.append(n)
            n += 1
    if exp_lab[-1] >= clen:
        exp_lab.pop()
        if exp_avoid:
            exp_avoid.pop()
    assert lab.tolist() == exp_lab and avoid.tolist() == exp_avoid


@SET
@given(st.lists(st.binary(min_size=0, max_size=3), min_size=1, max_size=12),
       st.lists(st.binary(min_size=0, max_size=5), min_size=1, max_size=20), st.booleans())
def test_trie_equals_dict_bruteforce(student, teacher, with_fallback):
    from llm_distillery_amd import vocab_utils as VU
    fallback = None
    if with_fallback:
        fallback = np.full(256, -1, dtype=np.int32)
        for i, s in enumerate(student):
            if len(s) == 1 and fallback[s[0]] < 0:
                fallback[s[0]] = i
    got = VU.longest_prefix_map(student, teacher, byte_fallback=fallback)
    ref = O.trie_map_bruteforce(student, teacher, fallback)
    assert got.tolist() == ref.tolist()
    off, ind = VU.csr_from_map(got, len(student))
    roff, rind = O.csr_from_map(ref, len(student))
    assert off.tolist() == roff.tolist() and ind.tolist() == rind.tolist()

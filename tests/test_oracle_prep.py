"""Pins the CPU oracle of the teacher-side preprocessing: the pairwise merge
against vectors written from the reference's own _merge_data, and the parts the
reference does not have (weighted merge + remap, byte-trie map, CSR marginal)
against dict/loop brute force and conservation laws."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O


@pytest.mark.parametrize("case", ["equal", "disk_longer", "new_longer"])
def test_merge_topk_pair_matches_reference_golden(golden_dir, case):
    d = np.load(os.path.join(golden_dir, "merge_data.npz"))
    v, i = O.merge_topk_pair(d[f"{case}/disk_val"], d[f"{case}/new_val"], d[f"{case}/disk_idx"], d[f"{case}/new_idx"])
    assert np.array_equal(i, d[f"{case}/merged_idx"])
    np.testing.assert_allclose(v, d[f"{case}/merged_val"], rtol=1e-6, atol=1e-7)


def test_reference_dense_merge_is_not_executable(golden_dir):
    # the reference's dense branch never binds `merged_indices`; the oracle's
    # dense merge therefore follows the formula of merge_full only
    d = np.load(os.path.join(golden_dir, "merge_data.npz"))
    assert "dense/raises_unbound_local" in d.files
    out = O.merge_dense_pair(d["dense/disk_val"], d["dense/new_val"])
    assert out.shape == (6, 20)
    np.testing.assert_allclose(np.exp(out[:4]).sum(-1), 2.0, rtol=1e-5)
    np.testing.assert_allclose(np.exp(out[4:]).sum(-1), 1.0, rtol=1e-5)


def test_merge_topk_pair_against_dict_bruteforce():
    g = torch.Generator().manual_seed(0)
    N, K, V = 7, 5, 23
    def draw():
        v, i = torch.topk(torch.log_softmax(torch.randn(N, V, generator=g) * 2, -1), K)
        return v.numpy(), i.numpy()
    av, ai = draw()
    bv, bi = draw()
    mv, mi = O.merge_topk_pair(av, bv, ai, bi)
    for r in range(N):
        acc = {}
        for v, i in list(zip(av[r], ai[r])) + list(zip(bv[r], bi[r])):
            acc[int(i)] = acc.get(int(i), 0.0) + float(np.exp(np.float32(v)))
        top = sorted(acc.items(), key=lambda kv: -kv[1])[:K]
        assert [k for k, _ in top] == mi[r].tolist()
        np.testing.assert_allclose(np.exp(mv[r]), [v for _, v in top], rtol=1e-5)
        # nothing is lost before truncation
        assert abs(sum(acc.values()) - (np.exp(av[r]).sum() + np.exp(bv[r]).sum())) < 1e-5


def _teachers(N, K, Vt, n, seed):
    g = torch.Generator().manual_seed(seed)
    vals, idxs = [], []
    for _ in range(n):
        v, i = torch.topk(torch.log_softmax(torch.randn(N, Vt, generator=g) * 2, -1), K)
        vals.append(v.to(torch.float16).numpy())
        idxs.append(i.numpy().astype(np.int32))
    return vals, idxs


def test_merge_remap_mass_conservation_and_canonical_order():
    N, K, Vt, Vs = 6, 8, 60, 20
    vals, idxs = _teachers(N, K, Vt, 3, 1)
    rng = np.random.default_rng(1)
    id_map = rng.integers(0, Vs, Vt).astype(np.int32)
    id_map[rng.random(Vt) < 0.1] = -1
    w = (0.5, 0.3, 0.2)
    rows = O.merge_remap_rows(vals, idxs, w, id_map)
    for r, (ids, mass, lq) in enumerate(rows):
        assert np.all(np.diff(ids) > 0) and ids.dtype == np.int32
        kept = sum(wt * np.exp(v[r].astype(np.float64))[id_map[i[r]] >= 0].sum() for v, i, wt in zip(vals, idxs, w))
        np.testing.assert_allclose(mass.astype(np.float64).sum(), kept, rtol=1e-5)
        np.testing.assert_allclose(np.exp(lq).sum(), 1.0, rtol=1e-12)
        np.testing.assert_allclose(np.exp(lq), mass / mass.sum(), rtol=1e-5)
        assert set(ids.tolist()) == {int(id_map[t]) for i in idxs for t in i[r] if id_map[t] >= 0}


def test_merge_remap_identity_single_teacher_is_plain_renormalisation():
    vals, idxs = _teachers(4, 6, 30, 1, 2)
    rows = O.merge_remap_rows(vals, idxs, (1.0,), None, T=2.0)
    for r, (ids, mass, lq) in enumerate(rows):
        order = np.argsort(idxs[0][r])
        assert np.array_equal(ids, idxs[0][r][order])
        ref = O.teacher_logprobs_topk(torch.tensor(vals[0][r:r + 1]), 2.0, torch.float64)[0].numpy()[order]
        np.testing.assert_allclose(lq, ref, atol=1e-6)


def test_merge_remap_all_dropped_row_and_padded_layout():
    vals, idxs = _teachers(3, 4, 12, 2, 3)
    id_map = np.arange(12, dtype=np.int32)
    id_map[idxs[0][1]] = -1
    id_map[idxs[1][1]] = -1
    ids, lq, cnt = O.merge_remap_padded(vals, idxs, (0.5, 0.5), id_map)
    assert cnt[1] == 0 and np.all(ids[1] == -1) and np.all(np.isneginf(lq[1]))
    assert ids.shape == (3, 8) and cnt[0] > 0


def test_fwd_kl_sparse_rows_reduces_to_the_topk_form_and_to_the_library():
    # (1) full rows (cnt == K, normalised log-probs): the value of fwd_kl_topk_rows, which the golden
    #     vectors written from the reference's calculate_divergence pin
    g = torch.Generator().manual_seed(11)
    N, K, V = 9, 7, 41
    z = torch.randn(N, V, generator=g, dtype=torch.float64) * 2
    stored, idx = torch.topk(torch.log_softmax(torch.randn(N, V, generator=g, dtype=torch.float64), -1), K)
    t = O.teacher_logprobs_topk(stored, 1.3, torch.float64)
    full = O.fwd_kl_sparse_rows(z, idx.numpy().astype(np.int32), t.numpy(), np.full(N, K, dtype=np.int32))
    np.testing.assert_allclose(full.numpy(), O.fwd_kl_topk_rows(z, t, idx).numpy(), rtol=1e-12)
    # (2) ragged rows with padding behind the count: per row the library's kl_div on the live prefix;
    #     the padding (-1 ids, -inf log-probs, and garbage behind a count of 0) must not be read
    cnt = np.array([K, 3, 0, 1, 5, K, 2, 0, 4], dtype=np.int32)
    ids = idx.numpy().astype(np.int32).copy()
    lq = np.full((N, K), -np.inf)
    for r in range(N):
        n = int(cnt[r])
        ids[r, n:] = -1
        if n:
            lq[r, :n] = torch.log_softmax(stored[r, :n], -1).numpy()
    ids[2, :] = 12345                                        # count 0: whatever lies there is ignored
    z.requires_grad_(True)
    got = O.fwd_kl_sparse_rows(z, ids, lq, cnt)
    s = torch.log_softmax(z.detach(), -1)
    for r in range(N):
        n = int(cnt[r])
        if n == 0:
            assert got[r].item() == 0.0
            continue
        want = F.kl_div(s[r, idx[r, :n]], torch.as_tensor(lq[r, :n]), reduction="none", log_target=True).sum()
        np.testing.assert_allclose(got[r].item(), want.item(), rtol=1e-12)
    # (3) gradient identity of the forward KL: softmax(z) - scatter(q) on rows with entries, 0 elsewhere
    got.sum().backward()
    want_g = torch.softmax(z.detach(), -1)
    for r in range(N):
        n = int(cnt[r])
        if n == 0:
            want_g[r] = 0
        else:
            want_g[r, idx[r, :n]] -= torch.exp(torch.as_tensor(lq[r, :n]))
    np.testing.assert_allclose(z.grad.numpy(), want_g.numpy(), atol=1e-12)


def _rand_vocab(rng, n, lo=1, hi=16, alphabet=256):
    return [bytes(rng.integers(0, alphabet, rng.integers(lo, hi + 1)).astype(np.uint8)) for _ in range(n)]


def test_trie_bruteforce_known_answers():
    student = [b"a", b"ab", b"abc", b"b", b"\xff", b"ab"]       # id 5 duplicates id 1
    teacher = [b"abcd", b"abx", b"a", b"b", b"c", b"", b"\xff\x00", b"ba"]
    fb = [-1] * 256
    fb[ord("c")] = 4
    got = O.trie_map_bruteforce(student, teacher, fb)
    assert got.tolist() == [2, 1, 0, 3, 4, -1, 4, 3]
    assert O.trie_map_bruteforce(student, teacher).tolist() == [2, 1, 0, 3, -1, -1, 4, 3]


def test_csr_and_marginal_invariants():
    rng = np.random.default_rng(4)
    student = [bytes([b]) for b in range(256)] + _rand_vocab(rng, 300, 2, 4, alphabet=4)
    teacher = _rand_vocab(rng, 900, 1, 6, alphabet=4)
    t2s = O.trie_map_bruteforce(student, teacher)
    assert (t2s >= 0).all()
    off, ind = O.csr_from_map(t2s, len(student))
    assert off[0] == 0 and off[-1] == len(teacher) and np.all(np.diff(off) >= 0)
    assert sorted(ind.tolist()) == list(range(len(teacher)))
    for s in range(len(student)):
        seg = ind[off[s]:off[s + 1]]
        assert np.all(np.diff(seg) > 0) and np.all(t2s[seg] == s)
    p = torch.softmax(torch.randn(5, len(teacher), dtype=torch.float64), -1).numpy()
    m1 = O.marginalise_csr(p, off, ind)
    m2 = O.marginalise_map(p, t2s, len(student))
    np.testing.assert_allclose(m1, m2, rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(m1.sum(-1), 1.0, rtol=1e-12)
    # longest-prefix property: the mapped student string is a prefix, and no longer one exists
    sset = {}
    for i, b in enumerate(student):
        sset.setdefault(b, i)
    for t, b in enumerate(teacher):
        sb = student[t2s[t]]
        assert b.startswith(sb) and sset[sb] == t2s[t]
        assert not any(b[:L] in sset for L in range(len(sb) + 1, len(b) + 1))


def test_teacher_producer_roundtrip_storage():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(2, 7, 50, generator=g)
    v, i = O.teacher_topk_producer(logits, 40, 6)
    assert v.shape == (2, 7, 6) and int(i.max()) < 40
    assert (v[..., :-1] >= v[..., 1:]).all()
    full = torch.log_softmax(logits[..., :40], -1)
    torch.testing.assert_close(torch.gather(full, -1, i), v)
    v16, i32 = O.to_storage(v.reshape(-1, 6), i.reshape(-1, 6))
    v2, i2 = O.from_storage(v16.numpy(), i32)
    assert v2.dtype == torch.float32 and i2.dtype == torch.int64 and torch.equal(i2, i.reshape(-1, 6))


def test_content_and_ce_indices():
    ranges = [(3, 7), (10, 14)]
    assert O.content_indices(ranges).tolist() == [3, 4, 5, 6, 10, 11, 12, 13]
    lab, avoid = O.ce_indices(ranges, context_len=2048, convo_len=20)
    assert lab.tolist() == [4, 5, 6, 7, 11, 12, 13, 14] and avoid.tolist() == [3, 7]
    # the last label falls at the conversation end -> dropped with its ignore entry
    lab, avoid = O.ce_indices(ranges, context_len=2048, convo_len=14)
    assert lab.tolist() == [4, 5, 6, 7, 11, 12, 13] and avoid.tolist() == [3]
    lab, avoid = O.ce_indices([(2, 6)], context_len=2048, convo_len=6)
    assert lab.tolist() == [3, 4, 5] and avoid.size == 0

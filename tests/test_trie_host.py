"""The host C++ byte trie and CSR builder (inside the C-ABI library; no GPU needed) against the
dict-based brute force of the oracle: integer maps must be bit-exact."""
import numpy as np
import pytest

import llm_distillery_amd as D
from llm_distillery_amd import synthetic as S
from oracle import oracle as O


@pytest.mark.parametrize("alphabet,n_s,n_t,seed", [(256, 2000, 5000, 1), (4, 600, 3000, 2), (2, 300, 2000, 3), (16, 5000, 20000, 4)])
def test_trie_map_equals_bruteforce(alphabet, n_s, n_t, seed):
    student = S.random_byte_vocab(n_s, seed, alphabet=alphabet, all_single_bytes=(alphabet == 256))
    teacher = S.random_byte_vocab(n_t, seed + 100, alphabet=alphabet, min_len=0)
    got = D.vocab_utils.longest_prefix_map(student, teacher)
    ref = O.trie_map_bruteforce(student, teacher)
    assert got.dtype == np.int32 and np.array_equal(got, ref)
    rng = np.random.default_rng(seed)
    fb = rng.integers(-1, n_s, 256).astype(np.int32)
    assert np.array_equal(D.vocab_utils.longest_prefix_map(student, teacher, fb), O.trie_map_bruteforce(student, teacher, fb))


def test_trie_edge_cases():
    student = [b"", b"ab", b"ab", b"abc", b"\x00", b"\x00\x00"]
    teacher = [b"", b"a", b"ab", b"abcd", b"\x00\x00\x00", b"\x00a", b"zz"]
    got = D.vocab_utils.longest_prefix_map(student, teacher)
    assert got.tolist() == [-1, -1, 1, 3, 5, 4, -1] == O.trie_map_bruteforce(student, teacher).tolist()
    assert D.vocab_utils.longest_prefix_map([], teacher).tolist() == [-1] * 7
    assert D.vocab_utils.longest_prefix_map(student, []).size == 0
    with pytest.raises(ValueError):
        D.vocab_utils.longest_prefix_map(student, teacher, [0] * 10)


def test_csr_equals_bruteforce_and_is_valid():
    rng = np.random.default_rng(5)
    t2s = rng.integers(-1, 400, 7000).astype(np.int32)
    off, ind = D.vocab_utils.csr_from_map(t2s, 400)
    roff, rind = O.csr_from_map(t2s, 400)
    assert np.array_equal(off, roff) and np.array_equal(ind, rind)
    assert off[0] == 0 and off[-1] == (t2s >= 0).sum() and np.all(np.diff(off) >= 0)
    assert sorted(ind.tolist()) == np.nonzero(t2s >= 0)[0].tolist()
    with pytest.raises(RuntimeError):
        D.vocab_utils.csr_from_map(np.array([5], dtype=np.int32), 3)       # id beyond the student vocabulary


def test_config5_vocabularies_at_full_size():
    """152064 teacher tokens against a 32000-token student trie: every teacher token finds a student
    prefix (all single bytes are student tokens), checked against the brute force on a sample."""
    student = S.random_byte_vocab(32000, 501, all_single_bytes=True)
    teacher = S.random_byte_vocab(152064, 502)
    t2s = D.vocab_utils.longest_prefix_map(student, teacher)
    assert t2s.shape == (152064,) and (t2s >= 0).all() and t2s.max() < 32000
    sample = np.random.default_rng(0).choice(152064, 3000, replace=False)
    ref = O.trie_map_bruteforce(student, [teacher[i] for i in sample])
    assert np.array_equal(t2s[sample], ref)
    off, ind = D.vocab_utils.csr_from_map(t2s, 32000)
    assert off[-1] == 152064 and np.array_equal(np.sort(ind), np.arange(152064))


def test_marginal_plan_covers_every_mapped_id_once_in_owner_order():
    rng = np.random.default_rng(7)
    Vt, Vs = 20000, 3000
    t2s = rng.integers(-1, Vs, Vt).astype(np.int32)
    t2s[rng.random(Vt) < 0.5] = rng.integers(0, 8)            # a few very hot student ids
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, "cpu")
    tile, bits = plan.tile, int(np.log2(plan.tile))
    assert tile in (4096, 8192)
    row_off = plan.row_off.numpy()
    ent = plan.ent.numpy().view(np.uint32)
    ntiles = -(-Vt // tile)
    assert row_off.shape == (16 * ntiles + 1,) and row_off[0] == 0 and row_off[-1] == ent.shape[0]
    seen = np.zeros(Vt, dtype=np.int32)
    for k in range(ntiles):
        for w in range(16):
            rows = ent[row_off[16 * k + w]:row_off[16 * k + w + 1]]
            for lane in range(64):
                col = rows[:, lane]
                live = col[col != 0xffffffff]
                assert (col[len(live):] == 0xffffffff).all()            # padding only at the tail
                assert (np.diff(live.astype(np.int64)) > 0).all()         # sorted by (s, t), no repeats
                sid = (live >> bits).astype(np.int64)
                t = (live & (tile - 1)).astype(np.int64) + k * tile
                assert (sid % 1024 == w * 64 + lane).all()                # owned by this thread
                assert (t2s[t] == sid).all()
                seen[t] += 1
    assert np.array_equal(seen, (t2s >= 0).astype(np.int32))
    # too wide a student vocabulary: no plan, the atomic form remains
    wide = D.vocab_utils.MarginalPlan(np.zeros(100, dtype=np.int32), 40000, "cpu")
    assert wide.ent is None and wide.tile == 0

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


ZERO = -1        # tile index of a packed list's padding: the words the kernels keep at zero behind the tile


def _plan_lists(plan, Vs):
    """Decodes a plan into what the kernels do with it: for every (tile, wave, lane) the list of steps
    (restart, tile index or ZERO, slot stored to or None), for both list formats, with the format's own
    invariants checked on the way.  Yields (k, w, lane, packed, steps, rows of the list)."""
    tile = plan.tile
    raw_off = plan.row_off.numpy()
    assert ((raw_off & 2) == 0).all() and raw_off[-1] & 1 == 0
    packed_flag, row_off = raw_off & 1, raw_off & ~3
    ent = plan.ent.numpy().view(np.uint32).astype(np.int64)
    assert row_off[0] == 0 and row_off[-1] == ent.shape[0]
    n_pad = (Vs + 3) & ~3
    spare0 = n_pad + ((plan.n_extra + 3) & ~3)
    for kw in range(len(row_off) - 1):
        k, w = divmod(kw, 16)
        rows = ent[row_off[kw]:row_off[kw + 1]]
        if packed_flag[kw]:
            assert rows.shape[0] == 4                                        # 4 dwords per lane, lane-major
            words = rows.reshape(64, 4)
            for lane in range(64):
                fields = [(int(words[lane, f // 2]) >> (16 * (f & 1))) & 0xffff for f in range(8)]
                slot = 0
                for f, v in enumerate(fields):
                    slot |= (v & 3) << ((8 + (f & ~1)) if f & 1 else f)
                offs = [v >> 2 for v in fields]
                n_padding = sum(o == tile for o in offs)
                assert all(o == tile for o in offs[:n_padding]) and all(o < tile for o in offs[n_padding:])   # padding first
                assert n_padding < 8 or slot == spare0 + lane               # an idle lane parks on its spare slot
                steps = [(f == 0, ZERO if o == tile else o, slot if f == 7 else None) for f, o in enumerate(offs)]
                yield k, w, lane, True, steps, 4
        else:
            assert rows.shape[0] >= 8 and rows.shape[0] % 8 == 0            # whole batches of 8 entries per lane
            batches = rows.reshape(-1, 64, 8)                                # [batch, lane, entry]
            for lane in range(64):
                col = batches[:, lane, :].reshape(-1)
                first, slot, offset = (col >> 31).astype(bool), (col >> 15) & 0xffff, col & 0x7fff
                assert (offset % 4 == 0).all() and (offset // 4 < tile).all()
                steps = [(bool(f), int(o) // 4, None if sl == spare0 + lane else int(sl)) for f, o, sl in zip(first, offset, slot)]
                yield k, w, lane, False, steps, rows.shape[0]


def test_marginal_plan_covers_every_mapped_id_once_with_single_owner_slots():
    rng = np.random.default_rng(7)
    Vt, Vs = 20000, 3000
    t2s = rng.integers(-1, Vs, Vt).astype(np.int32)
    t2s[rng.random(Vt) < 0.5] = rng.integers(0, 8)            # a few very hot student ids
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, "cpu")
    tile = plan.tile
    assert 4096 <= tile <= 8192 and tile % 1024 == 0
    fold = plan.fold.numpy()[:plan.n_fold]
    ntiles = -(-Vt // tile)
    assert plan.row_off.shape == (16 * ntiles + 1,)
    # replica slots sit behind the padded marginal, each belongs to exactly one hot id
    n_pad = (Vs + 3) & ~3
    slot_id = np.arange(n_pad + plan.n_extra)
    slot_id[Vs:] = -1
    assert plan.n_extra == fold[:, 2].sum() and (np.diff(fold[:, 0]) > 0).all()
    cursor = n_pad
    for sid, first, cnt in fold:
        assert first == cursor and cnt >= 1 and 0 <= sid < Vs
        slot_id[first:first + cnt] = sid
        cursor += cnt
    assert cursor == n_pad + plan.n_extra and plan.n_fold > 0       # the hot ids did get replicas
    seen = np.zeros(Vt, dtype=np.int32)
    longest, n_packed = [], 0
    owner = {}                                                            # (tile, slot) -> thread: slots may change hands between tiles
    runs_in_wave = {}
    for k, w, lane, packed, steps, n_rows in _plan_lists(plan, Vs):
        if lane == 0:
            longest.append(n_rows)
            n_packed += packed
        # cut the steps into runs: a run starts where the running sum restarts and ends where a real slot is stored
        runs, at = [], None
        for restart, t, slot in steps:
            if restart:
                at = []
            assert at is not None                                         # every list starts with a restart
            at.append(t)
            if slot is not None:
                runs.append((slot, at))
                at = None                                                 # the next entry must restart
        live = [(slot, [t for t in ts if t != ZERO]) for slot, ts in runs if slot < n_pad + plan.n_extra]
        live = [(slot, ts) for slot, ts in live if ts]
        if not packed:
            runs_in_wave[(k, w)] = (max(runs_in_wave.get((k, w), (0, 0))[0], len(live)), n_rows)
        assert [sl for sl, _ in live] == sorted({sl for sl, _ in live})    # one run per slot, ascending
        if live:
            assert steps[-1][2] == live[-1][0]                            # padding comes first: the last run ends on the last row
        for slot, ts in live:
            t = np.asarray(ts) + k * tile
            assert (np.diff(t) > 0).all() and (t < Vt).all()
            assert (t2s[t] == slot_id[slot]).all()                        # the entries land on a slot of their own id
            assert owner.setdefault((k, slot), w * 64 + lane) == w * 64 + lane      # one thread per LDS word inside a tile
            seen[t] += 1
        if packed:
            assert len(live) <= 1
    assert np.array_equal(seen, (t2s >= 0).astype(np.int32))
    # a list is packed exactly when every lane of the wave holds at most one run and no more than 8 entries
    assert all(most > 1 or n_rows > 8 for most, n_rows in runs_in_wave.values())
    assert n_packed >= 4 * ntiles                 # one-run threads are gathered in the low waves: half the entries sit on 8 ids
    # half of the entries sit on 8 ids: without replicas one thread would hold > 1200 entries of a tile
    assert max(longest) <= 4 * (tile // 1024)
    # too wide a student vocabulary: the plan is built over the map's image (the student ids it reaches) ...
    wide_map = rng.integers(-1, 90000, 5000).astype(np.int32)
    wide = D.vocab_utils.MarginalPlan(wide_map, 90000, "cpu")
    used = np.unique(wide_map[wide_map >= 0])
    assert wide.full is None and wide.compact is not None and wide.ent is wide.compact.ent
    assert wide.n_compact == -(-used.size // 8) * 8
    cols, col_src, t2c = wide.cols.numpy(), wide.col_src.numpy(), wide.t2c.numpy()
    assert np.array_equal(cols[:used.size], used) and (cols[used.size:] == -1).all()
    assert np.array_equal(np.nonzero(col_src >= 0)[0], used) and np.array_equal(col_src[used], np.arange(used.size))
    assert np.array_equal(t2c >= 0, wide_map >= 0) and np.array_equal(cols[t2c[wide_map >= 0]], wide_map[wide_map >= 0])
    # ... unless the caller rules that out, or the image itself is too wide: no plan, the atomic form remains
    none = D.vocab_utils.MarginalPlan(np.zeros(100, dtype=np.int32), 40000, "cpu", compact=False)
    assert none.ent is None and none.tile == 0 and none.cols is None
    huge = D.vocab_utils.MarginalPlan(np.arange(60000, dtype=np.int32), 60000, "cpu")
    assert huge.ent is None and huge.cols is None
    # a vocabulary that fits gets the full plan, and the compact one beside it where the image is at most half of it
    narrow = rng.integers(-1, 3000, 9000).astype(np.int32)
    both = D.vocab_utils.MarginalPlan(narrow, 8000, "cpu")
    assert both.full is not None and both.compact is not None and both.ent is both.full.ent and both.n_compact <= 3000
    assert D.vocab_utils.MarginalPlan(narrow, 8004, "cpu").compact is None          # not a multiple of 8 ids
    assert D.vocab_utils.MarginalPlan(narrow, 4000, "cpu").compact is None          # image above half of the vocabulary
    assert D.vocab_utils.MarginalPlan(narrow, 8000, "cpu", compact=False).compact is None
    only = D.vocab_utils.MarginalPlan(narrow, 4000, "cpu", compact=True)
    assert only.full is None and only.compact is not None and only._args() == (0, 0, 0, 0, 0, 0)


def _apply_plan(plan, probs, Vs):
    """What the planned kernels compute, step by step in numpy: per tile and thread the running sum
    restarts where the list says so, a general list stores slot + running sum after every entry (spare
    slots on unfinished runs), a packed list once, behind its last entry; replicas are folded into their
    id after the last tile."""
    tile = plan.tile
    n_pad = (Vs + 3) & ~3
    slots = np.zeros(n_pad + ((plan.n_extra + 3) & ~3) + 64, dtype=np.float32)
    touched, seg, seg_k = {}, None, -1
    for k, w, lane, packed, steps, _ in _plan_lists(plan, Vs):
        if k != seg_k:
            seg = np.zeros(tile, dtype=np.float32)
            part = probs[k * tile:(k + 1) * tile]
            seg[:part.size] = part
            seg_k, touched = k, {}
        run = np.float32(0)
        for restart, t, slot in steps:
            run = np.float32((0 if restart else run) + (np.float32(0) if t == ZERO else seg[t]))
            if slot is not None and slot < n_pad + plan.n_extra:   # a real slot: only this thread may touch it in this tile
                assert touched.setdefault(int(slot), (w, lane)) == (w, lane)
                slots[slot] = slots[slot] + run                    # one store per run: slot value read before the batch == before the run
    for sid, first, cnt in plan.fold.numpy()[:plan.n_fold]:
        for j in range(cnt):
            slots[sid] = slots[sid] + slots[first + j]
    return slots[:Vs]


@pytest.mark.parametrize("case", ["uniform", "one_hot_id", "all_dropped", "short", "tiny_student", "wide_student", "zipf"])
def test_marginal_plan_applied_in_numpy_equals_the_marginal(case):
    rng = np.random.default_rng(3)
    Vs, Vt = 3000, 20000
    if case == "uniform":
        t2s = rng.integers(-1, Vs, Vt)
    elif case == "one_hot_id":
        t2s = np.where(rng.random(Vt) < 0.95, 17, rng.integers(0, Vs, Vt))
    elif case == "all_dropped":
        t2s = np.full(Vt, -1)
    elif case == "short":
        Vt = 1000
        t2s = rng.integers(0, Vs, Vt)
    elif case == "tiny_student":
        Vs = 4
        t2s = rng.integers(0, Vs, Vt)
    elif case == "wide_student":
        Vs, Vt = 36500, 9000
        t2s = np.where(rng.random(Vt) < 0.8, rng.integers(0, 6, Vt) * 5000, rng.integers(0, Vs, Vt))
    else:
        t2s = np.minimum(rng.zipf(1.2, Vt) - 1, Vs - 1)
    t2s = t2s.astype(np.int32)
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, "cpu")
    assert plan.ent is not None
    probs = rng.random(Vt).astype(np.float32)
    got = _apply_plan(plan, probs, Vs)
    want = np.zeros(Vs, dtype=np.float64)
    np.add.at(want, t2s[t2s >= 0], probs[t2s >= 0].astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-6)
    assert np.array_equal(got == 0, want == 0)

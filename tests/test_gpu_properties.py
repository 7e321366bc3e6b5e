"""Property tests (hypothesis) of index handling in the kernels, against the oracle: duplicate and
colliding ids, dropped ids, ids outside the vocabulary, all-dropped rows, ragged entry counts, K larger
than the number of distinct ids, empty row masks.  Integer outputs bit-exact."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SET = settings(max_examples=40, deadline=None, derandomize=True)


@pytest.fixture(scope="module")
def D():
    import llm_distillery_amd as d
    d._lib.load()
    return d


@st.composite
def merge_case(draw):
    n_teachers = draw(st.integers(1, 4))
    K = draw(st.integers(1, 40))
    Vt = draw(st.integers(2, 300))
    Vs = draw(st.integers(1, 200))
    rows = draw(st.integers(1, 4))
    seed = draw(st.integers(0, 2 ** 31 - 1))
    rng = np.random.default_rng(seed)
    lo = draw(st.sampled_from([0, -2]))                         # -2: some ids fall outside the teacher vocabulary
    idxs = [rng.integers(lo, Vt + (3 if lo else 0), (rows, K)) for _ in range(n_teachers)]      # with repeats
    vals = [np.log(rng.random((rows, K)).astype(np.float32) * 0.9 + 0.05).astype(np.float16) for _ in range(n_teachers)]
    weights = [float(w) for w in rng.random(n_teachers) + 0.1]
    id_map = rng.integers(0, Vs, Vt).astype(np.int32)
    id_map[rng.random(Vt) < draw(st.sampled_from([0.0, 0.3, 1.0]))] = -1      # 1.0: every id dropped
    return vals, idxs, weights, id_map, Vs, draw(st.booleans())


@SET
@given(merge_case())
def test_merge_remap_kernel_equals_oracle(D, case):
    vals, idxs, weights, id_map, Vs, wide_ids = case
    it = torch.int64 if wide_ids else torch.int32
    ids, lm, cnt = D.merge_remap_topk([torch.tensor(v, device=DEV) for v in vals],
                                      [torch.tensor(i, dtype=it, device=DEV) for i in idxs], weights,
                                      torch.tensor(id_map, device=DEV), student_vocab=Vs)
    ref = O.merge_remap_rows([v.astype(np.float32) for v in vals], idxs, weights, id_map, n_student=Vs)
    ids, lm, cnt = ids.cpu().numpy(), lm.cpu().numpy(), cnt.cpu().numpy()
    for r, (rid, rmass, _) in enumerate(ref):
        assert cnt[r] == rid.size
        assert np.array_equal(ids[r, :cnt[r]], rid)
        assert (ids[r, cnt[r]:] == -1).all() and np.isneginf(lm[r, cnt[r]:]).all()
        np.testing.assert_allclose(np.exp(lm[r, :cnt[r]].astype(np.float64)), rmass, rtol=3e-6)


@st.composite
def topk_case(draw):
    V = draw(st.sampled_from([8, 64, 520, 4096]))
    K = draw(st.integers(1, 24))
    rows = draw(st.integers(1, 6))
    seed = draw(st.integers(0, 2 ** 31 - 1))
    rng = np.random.default_rng(seed)
    ids = rng.integers(-1, V + 2, (rows, K))                    # repeats, -1 and ids >= V are ignored entries
    ids[:, 0] = rng.integers(0, V, rows) if draw(st.booleans()) else ids[:, 0]
    cnt = rng.integers(0, K + 1, rows).astype(np.int32)         # ragged; 0 = a row without teacher
    mask = rng.random(rows) < draw(st.sampled_from([0.0, 0.5, 1.0]))      # 0.0: empty mask
    return V, K, rows, seed, ids, cnt, mask, draw(st.sampled_from(["fkl", "rkl"])), draw(st.sampled_from([1.0, 2.5]))


@SET
@given(topk_case())
def test_topk_divergence_index_handling(D, case):
    V, K, rows, seed, ids, cnt, mask, kind, T = case
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, V, generator=g) * 2
    tv = torch.randn(rows, K, generator=g)
    n_valid = int(mask.sum())
    row_map = np.full(rows, -1, dtype=np.int32)
    row_map[mask] = np.arange(n_valid)
    rl, grad = D.div_topk(kind, logits.to(DEV), tv[torch.as_tensor(mask)].to(DEV).contiguous(),
                          torch.tensor(ids[mask], dtype=torch.int32, device=DEV).contiguous(),
                          row_map=torch.tensor(row_map, device=DEV), t_cnt=torch.tensor(cnt[mask], device=DEV), T=T)
    rl, grad = rl.cpu(), grad.cpu()
    for r in range(rows):
        keep = [k for k in range(int(cnt[r])) if 0 <= int(ids[r, k]) < V] if mask[r] else []
        if not keep:
            assert rl[r] == 0 and torch.count_nonzero(grad[r]) == 0
            continue
        z = (logits[r:r + 1].double() / T).requires_grad_(True)
        t = O.teacher_logprobs_topk(tv[r:r + 1, keep], T, torch.float64)
        idx = torch.as_tensor(ids[r:r + 1, keep])
        ref = (O.fwd_kl_topk_rows if kind == "fkl" else O.rev_kl_topk_rows)(z, t, idx)
        np.testing.assert_allclose(rl[r].item(), ref.item(), rtol=3e-5, atol=3e-6)
        (gref,) = torch.autograd.grad(ref.sum(), z)
        gref = gref[0] / T
        err = (grad[r].double() - gref).abs()
        if kind == "fkl":
            bound = O.sparse_gradient_tolerance(gref[None], logits[r:r + 1], T, idx, torch.float32, 2e-4, row_coef=1.0 / T)[0]
        else:
            bound = O.rkl_topk_gradient_tolerance(gref[None], logits[r:r + 1], tv[r:r + 1, keep], idx, T, T, 1.0,
                                                  torch.float32, 2e-4)[0]
        assert (err <= bound).all(), float((err / bound).max())


@pytest.mark.parametrize("threads,chunks", [(256, 2), (256, 4), (256, 8), (256, 12), (256, 16), (512, 4), (512, 8), (512, 16),
                                            (1024, 4), (1024, 16)])
@pytest.mark.parametrize("one_xcd,wave_major,lds_kb", [(True, True, 0), (False, False, 0), (True, False, 40), (False, True, 64)])
def test_row_shaped_copy_is_a_copy(D, threads, chunks, one_xcd, wave_major, lds_kb):
    # the bandwidth yardstick moves every byte exactly once: ragged last part, a row count that is not a multiple of 8
    g = torch.Generator().manual_seed(threads + chunks)
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (13, 4 * 5003), generator=g, dtype=torch.int32).to(DEV)
    dst = torch.full_like(src, 7)
    D.copy_rows(src, dst, threads, chunks, one_xcd, wave_major, lds_kb)
    assert torch.equal(src, dst)
    with pytest.raises(RuntimeError):
        D.copy_rows(src, dst, 128, 3, one_xcd)

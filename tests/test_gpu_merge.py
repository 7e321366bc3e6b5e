"""GPU parity of the teacher-side merge kernels: integer outputs bit-exact, masses within fp32
tolerance, against the reference's own merge vectors, dict brute force and conservation laws."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def D():
    import llm_distillery_amd as d
    d._lib.load()
    return d


@pytest.mark.parametrize("case", ["equal", "disk_longer", "new_longer"])
def test_pair_merge_matches_reference_golden(D, golden_dir, case):
    d = np.load(os.path.join(golden_dir, "merge_data.npz"))
    V = int(max(d[f"{case}/disk_idx"].max(), d[f"{case}/new_idx"].max())) + 1
    lm, idx = D.merge_topk_pair(torch.tensor(d[f"{case}/disk_val"], device=DEV), torch.tensor(d[f"{case}/disk_idx"], device=DEV),
                                torch.tensor(d[f"{case}/new_val"], device=DEV), torch.tensor(d[f"{case}/new_idx"], device=DEV), V)
    assert idx.dtype == torch.int64 and np.array_equal(idx.cpu().numpy(), d[f"{case}/merged_idx"])
    np.testing.assert_allclose(lm.cpu().numpy(), d[f"{case}/merged_val"], rtol=1e-5, atol=1e-6)


def _teachers(N, K, Vt, n, seed, idx_dtype=torch.int32, val_dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    vals, idxs = [], []
    for _ in range(n):
        v, i = torch.topk(torch.log_softmax(torch.randn(N, Vt, generator=g) * 2, -1), K)
        vals.append(v.to(val_dtype))
        idxs.append(i.to(idx_dtype))
    return vals, idxs


def test_pair_merge_storage_dtypes_against_oracle(D):
    # as stored on disk (fp16 / int32) and with K = 400, the reference's default save_topK
    (av, bv), (ai, bi) = _teachers(40, 400, 32000, 2, 1)
    lm, idx = D.merge_topk_pair(av.to(DEV), ai.to(DEV), bv[:33].to(DEV), bi[:33].to(DEV), 32000)
    rv, ri = O.merge_topk_pair(av.float().numpy(), bv[:33].float().numpy(), ai.numpy(), bi[:33].numpy())
    got_i, got_v = idx.cpu().numpy(), lm.cpu().numpy()
    np.testing.assert_allclose(got_v, rv, rtol=1e-5, atol=2e-6)
    # fp16 storage produces exact ties between masses; order inside a tie is the only freedom
    for r in range(40):
        if not np.array_equal(got_i[r], ri[r]):
            assert sorted(got_i[r]) == sorted(ri[r]) or np.allclose(np.sort(got_v[r]), np.sort(rv[r]), rtol=1e-6)
            ties = got_i[r] != ri[r]
            assert np.allclose(got_v[r][ties], rv[r][ties], rtol=1e-6)
    assert (np.diff(got_v[:33], axis=1) <= 1e-7).all()          # descending


@pytest.mark.parametrize("n,K,Vt,Vs,use_map,idx_dtype", [(3, 50, 3000, 1000, True, torch.int32), (2, 64, 5000, 5000, False, torch.int64),
                                                         (1, 200, 152064, 128256, True, torch.int32), (5, 400, 152064, 128256, True, torch.int32)])
def test_merge_remap_ids_bit_exact_masses_close(D, n, K, Vt, Vs, use_map, idx_dtype):
    N = 12
    vals, idxs = _teachers(N, K, Vt, n, 2, idx_dtype)
    rng = np.random.default_rng(3)
    id_map = None
    if use_map:
        id_map = rng.integers(0, Vs, Vt).astype(np.int32)
        id_map[rng.random(Vt) < 0.05] = -1
        id_map[idxs[0][3].numpy()] = -1                    # a row that loses a whole teacher
    w = [0.5, 0.3, 0.2, 0.7, 0.1][:n]
    ids, lm, cnt = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], w,
                                      torch.tensor(id_map, device=DEV) if use_map else None, student_vocab=Vs)
    ref = O.merge_remap_rows([v.numpy() for v in vals], [i.numpy() for i in idxs], w, id_map)
    ids, lm, cnt = ids.cpu().numpy(), lm.cpu().numpy(), cnt.cpu().numpy()
    assert ids.dtype == np.int32 and ids.shape == (N, n * K)
    for r, (rid, rmass, _) in enumerate(ref):
        assert cnt[r] == rid.size
        assert np.array_equal(ids[r, :cnt[r]], rid)                     # bit-exact, canonical ascending order
        assert (ids[r, cnt[r]:] == -1).all() and np.isneginf(lm[r, cnt[r]:]).all()
        np.testing.assert_allclose(np.exp(lm[r, :cnt[r]].astype(np.float64)), rmass, rtol=2e-6)


def test_merge_remap_all_dropped_row_and_out_of_range_ids(D):
    vals, idxs = _teachers(4, 8, 64, 2, 4)
    id_map = np.arange(64, dtype=np.int32)
    id_map[idxs[0][1].numpy()] = -1
    id_map[idxs[1][1].numpy()] = -1
    idxs[0][2, 0] = 9999                                     # outside the teacher vocabulary: dropped
    ids, lm, cnt = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [0.5, 0.5],
                                      torch.tensor(id_map, device=DEV), student_vocab=64)
    assert cnt[1].item() == 0 and (ids[1] == -1).all()
    logits = torch.randn(4, 64)
    rl, grad = D.div_topk("fkl", logits.to(DEV), lm, ids, t_cnt=cnt)
    assert rl[1].item() == 0 and torch.count_nonzero(grad[1]) == 0 and torch.isfinite(rl).all()


def test_fused_multi_teacher_loss_against_oracle(D):
    """Config-4 semantics at reduced rows: merge -> remap -> renormalise -> forward KL, loss 1e-5,
    gradients within the bf16 tolerance, against the dict/loop oracle."""
    from llm_distillery_amd import synthetic as S
    c = S.config4(DEV, rows=24, V=32000, Vt=40000, K=200)
    T = 1.0
    rl, grad = D.fkl_multi_teacher(c["logits"], c["t_vals"], c["t_idxs"], c["weights"], c["id_map"], T=T,
                                   grad_scale=1.0 / 24)
    loss = D.reduce_sum(rl, 1.0 / 24).item()
    ids, lq, cnt = O.merge_remap_padded([v.cpu().numpy() for v in c["t_vals"]], [i.cpu().numpy() for i in c["t_idxs"]],
                                        c["weights"], c["id_map"].cpu().numpy(), T)
    z = (c["logits"].cpu().double() / T).requires_grad_(True)
    rows = O.fwd_kl_sparse_rows(z, ids, lq.astype(np.float64), cnt)
    rows.mean().backward()
    np.testing.assert_allclose(loss, rows.mean().item(), rtol=1e-5)
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows.detach().numpy(), rtol=3e-5, atol=3e-6)
    gref = z.grad / T
    err = (grad.cpu().double() - gref).abs()
    assert (err <= O.storage_tolerance(gref, torch.bfloat16, 2e-3)).all()
    # mass conservation: the renormalised mixture sums to one on every row with survivors
    assert np.allclose(np.exp(lq.astype(np.float64)).sum(-1)[cnt > 0], 1.0, atol=1e-5)


def test_merge_is_bit_reproducible(D):
    vals, idxs = _teachers(64, 200, 152064, 3, 5)
    m = torch.randint(0, 128256, (152064,), dtype=torch.int32)
    a = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [0.5, 0.3, 0.2], m.to(DEV), student_vocab=128256)
    b = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [0.5, 0.3, 0.2], m.to(DEV), student_vocab=128256)
    assert all(torch.equal(x, y) for x, y in zip(a, b))

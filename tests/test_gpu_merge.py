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
    bound = O.sparse_gradient_tolerance(gref, c["logits"].cpu(), T, torch.as_tensor(ids).long(), torch.bfloat16, 2e-3,
                                        row_coef=1.0 / (24 * T))
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    # mass conservation: the renormalised mixture sums to one on every row with survivors
    assert np.allclose(np.exp(lq.astype(np.float64)).sum(-1)[cnt > 0], 1.0, atol=1e-5)


def _oracle_multi(logits, vals, idxs, weights, id_map, T, valid=None):
    """Loss rows and gradient of the mixture against the dict/loop merge + the pinned ragged forward KL."""
    V = logits.shape[1]
    ids, lq, cnt = O.merge_remap_padded([v.float().numpy() for v in vals], [i.numpy() for i in idxs], weights,
                                        None if id_map is None else id_map.numpy(), 1.0, n_student=V)
    sel = torch.arange(logits.shape[0]) if valid is None else torch.nonzero(valid).squeeze(-1)
    z = (logits[sel].double() / T).requires_grad_(True)
    rows = O.fwd_kl_sparse_rows(z, ids, lq.astype(np.float64), cnt)
    rows.sum().backward()
    grad = torch.zeros(logits.shape, dtype=torch.float64)
    grad[sel] = z.grad / T
    return rows.detach(), grad, cnt, torch.as_tensor(ids).long()


@pytest.mark.parametrize("V,dtype,n,K,Vt,T", [
    (128256, torch.bfloat16, 3, 200, 152064, 1.0),      # rows cut into 4 parts, 3 slots of 256 entries
    (32000, torch.bfloat16, 3, 200, 40000, 2.0),        # one workgroup per row
    (2048, torch.float16, 2, 100, 3000, 1.0),           # narrowest shape
    (40000, torch.float32, 2, 400, 50000, 1.3),         # 3 parts of fp32 (corrections behind the dense stores), 2 slots per teacher
    (16000, torch.float32, 3, 200, 20000, 1.0),         # 512 threads x 8 chunks
    (152064, torch.float16, 1, 200, 152064, 1.0),       # a single teacher through the map, 5 parts
    (65536, torch.bfloat16, 4, 128, 70000, 0.7),        # 512 x 16, one workgroup per row
    (100000, torch.bfloat16, 8, 64, 120000, 1.0),       # 8 teachers: 8 slots
    (128256, torch.float32, 2, 100, 152064, 1.0),       # 4 parts of 512 threads x 16 chunks
    (262144, torch.bfloat16, 2, 100, 152064, 1.0),      # the same for two-byte rows
])
def test_bucketed_multi_teacher_against_oracle(D, V, dtype, n, K, Vt, T):
    """dl_fkl_multi_teacher (entries mapped, renormalised and dealt into per-part buckets by a K-wide
    launch, shared ids summed inside the loss kernel) against the dict/loop merge + ragged forward KL
    of the oracle, and against the sorting form of the library, with masked rows; waiting and
    deferred parts give the same bits."""
    g = torch.Generator().manual_seed(V + n)
    R = 14
    logits = (torch.randn(R, V, generator=g) * 3).to(dtype)
    valid = torch.ones(R, dtype=torch.bool)
    valid[[1, 9]] = False
    nv = int(valid.sum())
    vals, idxs = _teachers(nv, K, Vt, n, V + 1)
    weights = [0.5, 0.3, 0.2, 0.1, 0.25, 0.05, 0.4, 0.15][:n]
    id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
    id_map[torch.rand(Vt, generator=g) < 0.05] = -1
    id_map[idxs[0][0, :40].long()] = 7                      # forty entries of one row land on one student id
    if n > 1:
        id_map[idxs[1][2, :3].long()] = id_map[idxs[0][2, :3].long()]
    rm = torch.full((R,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(nv, dtype=torch.int32)
    args = (logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights, id_map.to(DEV))
    rl, grad = D.fkl_multi_teacher(*args, row_map=rm.to(DEV), T=T, teacher_T=1.0, grad_scale=1.0 / nv, fused=True)
    rows64, grad64, cnt, ids = _oracle_multi(logits, vals, idxs, weights, id_map, T, valid)
    assert (cnt > 0).all()
    np.testing.assert_allclose(D.reduce_sum(rl, 1.0 / nv).item(), rows64.mean().item(), rtol=1e-5)
    np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    assert torch.count_nonzero(rl.cpu()[~valid]) == 0 and torch.count_nonzero(grad.cpu()[~valid]) == 0
    grad64 = grad64 / nv                                    # the scale the kernel stored its gradient with
    err = (grad.cpu().double() - grad64).abs()
    rtol = 1e-4 if dtype == torch.float32 else 2e-3
    bound = O.storage_tolerance(grad64, dtype, rtol)
    vrows = torch.nonzero(valid).squeeze(-1)
    bound[vrows] = O.sparse_gradient_tolerance(grad64[vrows], logits[vrows], T, ids, dtype, rtol, row_coef=1.0 / (nv * T))
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    rl2, grad2 = D.fkl_multi_teacher(*args, row_map=rm.to(DEV), T=T, teacher_T=1.0, grad_scale=1.0 / nv, fused=True, no_wait=True)
    assert torch.equal(rl, rl2) and torch.equal(grad, grad2)
    # the two-launch form (sorted merge through memory, then the loss kernel) agrees to rounding
    rl3, grad3 = D.fkl_multi_teacher(*args, row_map=rm.to(DEV), T=T, teacher_T=1.0, grad_scale=1.0 / nv, fused=False)
    np.testing.assert_allclose(rl.cpu().numpy(), rl3.cpu().numpy(), rtol=2e-5, atol=2e-6)
    assert ((grad3.cpu().double() - grad64).abs() <= bound).all()


@pytest.mark.parametrize("V,pitch,dtype", [(151665, 151936, torch.bfloat16), (50257, 50304, torch.float16), (32003, 32064, torch.float32)])
def test_bucketed_multi_teacher_on_a_crop_of_padded_rows(D, V, pitch, dtype):
    """Rows on the 16-byte grid that end inside a chunk (logits[:, :, :crop], classes/student/model.py:408) stay in the
    bucketed form: entries in the ragged last chunk, masked rows, waiting or not."""
    g = torch.Generator().manual_seed(V)
    R, K, n, Vt = 9, 100, 3, V + 4000
    logits = (torch.randn(R, V, generator=g) * 3).to(dtype)
    valid = torch.ones(R, dtype=torch.bool)
    valid[4] = False
    nv = int(valid.sum())
    vals, idxs = _teachers(nv, K, Vt, n, V + 1)
    weights = [0.5, 0.3, 0.2]
    id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
    id_map[torch.rand(Vt, generator=g) < 0.05] = -1
    id_map[idxs[0][:, :3].long()] = V - 1                     # entries of every row in the last column
    id_map[idxs[1][:, :2].long()] = V - 2
    rm = torch.full((R,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(nv, dtype=torch.int32)
    full = torch.full((R, pitch), 3.0, dtype=dtype, device=DEV)
    x = full[:, :V]
    x.copy_(logits.to(DEV))
    args = (x, [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights, id_map.to(DEV))
    rl, grad = D.fkl_multi_teacher(*args, row_map=rm.to(DEV), T=1.2, teacher_T=1.0, grad_scale=1.0 / nv, fused=True)
    rows64, grad64, cnt, ids = _oracle_multi(logits, vals, idxs, weights, id_map, 1.2, valid)
    np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    assert torch.count_nonzero(rl.cpu()[~valid]) == 0 and torch.count_nonzero(grad.cpu()[~valid]) == 0
    grad64 = grad64 / nv
    rtol = 1e-4 if dtype == torch.float32 else 2e-3
    bound = O.storage_tolerance(grad64, dtype, rtol)
    vrows = torch.nonzero(valid).squeeze(-1)
    bound[vrows] = O.sparse_gradient_tolerance(grad64[vrows], logits[vrows], 1.2, ids, dtype, rtol, row_coef=1.0 / (nv * 1.2))
    err = (grad.cpu().double() - grad64).abs()
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    assert (full[:, V:] == 3.0).all()
    rl2, grad2 = D.fkl_multi_teacher(*args, row_map=rm.to(DEV), T=1.2, teacher_T=1.0, grad_scale=1.0 / nv, fused=True, no_wait=True)
    assert torch.equal(rl, rl2) and torch.equal(grad, grad2)


def test_bucketed_multi_teacher_edge_rows(D):
    """Rows whose entries are all dropped (loss 0, zero gradient), a teacher of weight 0, ids outside
    the teacher vocabulary, int64 ids with fp32 values, no map at all."""
    g = torch.Generator().manual_seed(91)
    R, V, Vt, K = 6, 4096, 6000, 48
    logits = torch.randn(R, V, generator=g) * 2
    vals, idxs = _teachers(R, K, Vt, 3, 92, idx_dtype=torch.int64, val_dtype=torch.float32)
    id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
    for i in idxs:
        id_map[i[1].long()] = -1                              # row 1: nothing survives
    idxs[0][3, :5] = Vt + 11                                  # outside the map: dropped
    idxs[1][3, 5] = -4
    weights = [0.7, 0.0, 0.3]
    rl, grad = D.fkl_multi_teacher(logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights,
                                   id_map.to(DEV), fused=True)
    assert rl[1].item() == 0 and torch.count_nonzero(grad[1]) == 0
    rows64, grad64, cnt, ids = _oracle_multi(logits, [vals[0], vals[2]], [idxs[0], idxs[2]], [0.7, 0.3], id_map, 1.0)
    assert cnt[1] == 0
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    assert ((grad.cpu().double() - grad64).abs() <= O.sparse_gradient_tolerance(grad64, logits, 1.0, ids, torch.float32, 1e-4)).all()
    # same vocabulary, no map: ids collide only where two teachers chose the same token
    small = [i.clamp(0, V - 1) for i in idxs]
    rl, grad = D.fkl_multi_teacher(logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in small], [1.0, 1.0, 1.0], None,
                                   fused=True)
    rows64, grad64, _, ids = _oracle_multi(logits, vals, small, [1.0, 1.0, 1.0], None, 1.0)
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    assert ((grad.cpu().double() - grad64).abs() <= O.sparse_gradient_tolerance(grad64, logits, 1.0, ids, torch.float32, 1e-4)).all()


def test_multi_teacher_with_a_teacher_of_weight_zero(D):
    """A teacher of weight 0 contributes no entries (its ids stay in the merged id list with mass 0, which the
    loss takes as no entry): both forms against the oracle, whose forward KL follows the same convention."""
    g = torch.Generator().manual_seed(91)
    R, V, Vt, K = 6, 40000, 45000, 100
    logits = (torch.randn(R, V, generator=g) * 3).to(torch.bfloat16)
    vals, idxs = _teachers(R, K, Vt, 3, 92)
    weights = [0.6, 0.0, 0.4]
    id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
    rows64, grad64, _, ids = _oracle_multi(logits, vals, idxs, weights, id_map, 1.0)
    assert torch.isfinite(rows64).all()
    args = (logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights, id_map.to(DEV))
    bound = O.sparse_gradient_tolerance(grad64 / R, logits, 1.0, ids, torch.bfloat16, 2e-3, row_coef=1.0 / R)
    for fused in (True, False):
        rl, grad = D.fkl_multi_teacher(*args, T=1.0, teacher_T=1.0, grad_scale=1.0 / R, fused=fused)
        np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
        assert ((grad.cpu().double() - grad64 / R).abs() <= bound).all()


def test_bucketed_multi_teacher_crowded_buckets_and_many_entries(D):
    """Every entry of a row inside one column part (its bucket overflows the slots laid out for an
    even share), 7 teachers x 290 entries, the largest entry count the library takes."""
    g = torch.Generator().manual_seed(94)
    R, V, Vt = 6, 128256, 140000
    logits = (torch.randn(R, V, generator=g) * 3).to(torch.bfloat16)
    for n, K in ((3, 200), (7, 290), (8, 256)):
        vals, idxs = _teachers(R, K, Vt, n, 95 + n)
        id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
        crowd = torch.randint(70000, 75000, (Vt,), generator=g, dtype=torch.int32)      # part 2 of 4, many shared ids
        for i in idxs:
            id_map[i[1].long()] = crowd[i[1].long()]
            id_map[i[4].long()] = crowd[i[4].long()] % 16 + 98300                       # sixteen ids astride the boundary of parts 2 and 3
        weights = [1.0 / (j + 1) for j in range(n)]
        args = (logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights, id_map.to(DEV))
        rl, grad = D.fkl_multi_teacher(*args, fused=True)
        rows64, grad64, _, ids = _oracle_multi(logits, vals, idxs, weights, id_map, 1.0)
        np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
        err = (grad.cpu().double() - grad64).abs()
        bound = O.sparse_gradient_tolerance(grad64, logits, 1.0, ids, torch.bfloat16, 2e-3, row_coef=1.0)
        assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
        rl2, grad2 = D.fkl_multi_teacher(*args, fused=True, no_wait=True)
        assert torch.equal(rl, rl2) and torch.equal(grad, grad2)


def test_bucketed_multi_teacher_refuses_what_it_cannot_take(D):
    vals, idxs = _teachers(4, 32, 5000, 2, 93)
    x = torch.randn(4, 4096, device=DEV)
    args = ([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [1.0, 1.0], None)
    with pytest.raises(RuntimeError, match="bucketed"):       # teacher temperature other than 1
        D.fkl_multi_teacher(x, *args, T=2.0, fused=True)
    with pytest.raises(RuntimeError, match="bucketed"):       # odd vocabulary
        D.fkl_multi_teacher(torch.randn(4, 4097, device=DEV), *args, fused=True)
    rl, _ = D.fkl_multi_teacher(torch.randn(4, 4097, device=DEV), *args)      # automatic: the sorting form
    assert torch.isfinite(rl).all()
    with pytest.raises(RuntimeError):
        D.fkl_multi_teacher(x, *args[:2], [1.0, -0.5], None, fused=True)      # negative weight
    lib = D._lib.load()
    assert lib.dl_fkl_multi_teacher_workspace_bytes(1, 64, 128256, 3, 200, 64, 0) > 0
    assert lib.dl_fkl_multi_teacher_workspace_bytes(1, 64, 300000, 3, 200, 64, 0) == 0      # too wide for the register kernels


def test_merge_is_bit_reproducible(D):
    vals, idxs = _teachers(64, 200, 152064, 3, 5)
    m = torch.randint(0, 128256, (152064,), dtype=torch.int32)
    a = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [0.5, 0.3, 0.2], m.to(DEV), student_vocab=128256)
    b = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], [0.5, 0.3, 0.2], m.to(DEV), student_vocab=128256)
    assert all(torch.equal(x, y) for x, y in zip(a, b))

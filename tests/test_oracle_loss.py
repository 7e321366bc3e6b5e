"""Pins the CPU oracle of the loss arithmetic: golden vectors written from the
reference's own calculate_divergence, closed forms, invariants and special cases
chosen so that a dropped term, a wrong sign or a wrong index fails."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O

CASES = ["two_ranges", "one_range", "alpha0", "alpha_half"]


def _load(golden_dir, case):
    d = np.load(os.path.join(golden_dir, "calculate_divergence.npz"))
    return {k[len(case) + 1:]: d[k] for k in d.files if k.startswith(case + "/")}


@pytest.mark.parametrize("case", CASES)
def test_calculate_divergence_matches_reference_golden(golden_dir, case):
    g = _load(golden_dir, case)
    s = torch.tensor(g["student"], requires_grad=True)
    res = O.calculate_divergence(s, torch.tensor(g["teacher"]), torch.tensor(g["indices"]),
                                 torch.tensor(g["labels"]), float(g["alpha"]),
                                 torch.tensor(g["avoid"], dtype=torch.long))
    assert tuple(res.keys()) == O.LOSS_KEYS
    for k in O.LOSS_KEYS:
        np.testing.assert_allclose(res[k].detach().numpy(), g[f"out/{k}"], rtol=2e-6, atol=1e-7, err_msg=k)
    res["train_loss"].backward()
    np.testing.assert_allclose(s.grad.numpy(), g["grad"], rtol=2e-5, atol=1e-8)


def test_calculate_divergence_raises_with_as_many_labels_as_rows():
    # reference: crop = 0 -> indices[:0] is empty -> the comparison cannot broadcast
    N, K, V = 6, 4, 20
    z = torch.randn(N, V)
    tv, ti = torch.topk(torch.log_softmax(torch.randn(N, V), -1), K)
    with pytest.raises((RuntimeError, IndexError)):
        O.calculate_divergence(z, tv, ti, torch.randint(0, V, (N,)), 2.0, torch.zeros(0, dtype=torch.long))


def _rand_topk(N, V, K, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(N, V, generator=g, dtype=dtype) * 2
    tl = torch.log_softmax(z + torch.randn(N, V, generator=g, dtype=dtype), -1)
    tv, ti = torch.topk(tl, K)
    return z, tv, ti


def test_fwd_kl_closed_form_and_gradient_identity():
    z, tv, ti = _rand_topk(7, 50, 9, 1)
    z.requires_grad_(True)
    t = O.teacher_logprobs_topk(tv, 1.3, torch.float64)
    zz = z / 1.3
    kl = O.fwd_kl_topk_rows(zz, t, ti)
    q = t.exp()
    lse = torch.logsumexp(zz, -1)
    closed = (q * t).sum(-1) - (q * torch.gather(zz, 1, ti)).sum(-1) + lse
    torch.testing.assert_close(kl, closed, rtol=1e-12, atol=1e-12)
    kl.sum().backward()
    p = torch.softmax(zz, -1)
    expect = (p - torch.zeros_like(p).scatter_add_(1, ti, q)) / 1.3
    torch.testing.assert_close(z.grad, expect.detach(), rtol=1e-10, atol=1e-12)


def test_fwd_kl_bound_and_decomposition():
    z, tv, ti = _rand_topk(11, 80, 12, 2)
    t = O.teacher_logprobs_topk(tv, 1.0, torch.float64)
    kl = O.fwd_kl_topk_rows(z, t, ti)
    rsup = F.log_softmax(torch.gather(z, 1, ti), -1)
    m = torch.gather(torch.softmax(z, -1), 1, ti).sum(-1)
    kl_qr = (t.exp() * (t - rsup)).sum(-1)
    torch.testing.assert_close(kl, kl_qr - torch.log(m), rtol=1e-10, atol=1e-12)
    assert (kl >= -torch.log(m) - 1e-12).all() and (kl >= 0).all()


def test_rev_kl_closed_form_gradient_and_locality():
    z, tv, ti = _rand_topk(6, 40, 7, 3)
    t = O.teacher_logprobs_topk(tv, 0.7, torch.float64)
    zr = z.clone().requires_grad_(True)
    rkl = O.rev_kl_topk_rows(zr, t, ti)
    zk = torch.gather(z, 1, ti)
    sp = zk - torch.logsumexp(zk, -1, keepdim=True)
    closed = (sp.exp() * (sp - t)).sum(-1)
    torch.testing.assert_close(rkl, closed, rtol=1e-11, atol=1e-12)
    assert (rkl >= -1e-12).all()
    rkl.sum().backward()
    r = sp.exp()
    gk = r * ((sp - t) - closed.unsqueeze(-1))
    expect = torch.zeros_like(z).scatter_add_(1, ti, gk)
    torch.testing.assert_close(zr.grad, expect, rtol=1e-9, atol=1e-12)
    # independent of every logit off the support
    z2 = z.clone()
    off = torch.ones_like(z, dtype=torch.bool).scatter_(1, ti, False)
    z2[off] += 5.0
    torch.testing.assert_close(O.rev_kl_topk_rows(z2, t, ti), rkl.detach(), rtol=1e-11, atol=1e-12)
    # zero iff the restricted student equals the teacher
    torch.testing.assert_close(O.rev_kl_topk_rows(z, sp, ti), torch.zeros(6, dtype=torch.float64), atol=1e-12, rtol=0)


def test_invariances_permutation_shift_temperature():
    z, tv, ti = _rand_topk(5, 30, 6, 4)
    t = O.teacher_logprobs_topk(tv, 2.0, torch.float64)
    base_f = O.fwd_kl_topk_rows(z / 2.0, t, ti)
    base_r = O.rev_kl_topk_rows(z / 2.0, t, ti)
    perm = torch.randperm(6)
    torch.testing.assert_close(O.fwd_kl_topk_rows(z / 2.0, t[:, perm], ti[:, perm]), base_f, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(O.rev_kl_topk_rows(z / 2.0, t[:, perm], ti[:, perm]), base_r, rtol=1e-12, atol=1e-13)
    shift = torch.randn(5, 1, dtype=torch.float64) * 10
    torch.testing.assert_close(O.fwd_kl_topk_rows((z + shift) / 2.0, t, ti), base_f, rtol=1e-10, atol=1e-11)
    # a per-row constant added to the stored teacher log-probs is irrelevant
    t2 = O.teacher_logprobs_topk(tv + shift, 2.0, torch.float64)
    torch.testing.assert_close(t2, t, rtol=1e-10, atol=1e-11)
    # fp16 -> fp32 storage cast is exact
    v16 = tv.to(torch.float16)
    assert torch.equal(v16.float().to(torch.float16), v16)


def test_topk_with_full_support_equals_dense_and_library():
    g = torch.Generator().manual_seed(5)
    N, V = 4, 25
    z = torch.randn(N, V, generator=g, dtype=torch.float64)
    tl = torch.randn(N, V, generator=g, dtype=torch.float64)
    ti = torch.arange(V).repeat(N, 1)
    t = F.log_softmax(tl, -1)
    lib = F.kl_div(F.log_softmax(z, -1), t, reduction="none", log_target=True).sum(-1)
    torch.testing.assert_close(O.fwd_kl_topk_rows(z, t, ti), lib)
    torch.testing.assert_close(O.fwd_kl_dense_rows(z, tl), lib)
    lib_r = F.kl_div(t, F.log_softmax(z, -1), reduction="none", log_target=True).sum(-1)
    torch.testing.assert_close(O.rev_kl_topk_rows(z, t, ti), lib_r)
    torch.testing.assert_close(O.rev_kl_dense_rows(z, tl), lib_r)


def test_dense_teacher_with_zero_mass_matches_topk_on_support():
    g = torch.Generator().manual_seed(6)
    N, V, K = 5, 40, 9
    z = torch.randn(N, V, generator=g, dtype=torch.float64)
    ti = torch.stack([torch.randperm(V, generator=g)[:K] for _ in range(N)])
    tv = torch.randn(N, K, generator=g, dtype=torch.float64)
    dense = torch.full((N, V), float("-inf"), dtype=torch.float64).scatter_(1, ti, tv)
    t = F.log_softmax(tv, -1)
    torch.testing.assert_close(O.fwd_kl_dense_rows(z, dense), O.fwd_kl_topk_rows(z, t, ti))
    torch.testing.assert_close(O.rev_kl_dense_rows(z, dense), O.rev_kl_topk_rows(z, t, ti))


def test_jsd_properties_and_gradient():
    g = torch.Generator().manual_seed(7)
    N, V = 6, 35
    z = torch.randn(N, V, generator=g, dtype=torch.float64) * 3
    tl = torch.randn(N, V, generator=g, dtype=torch.float64) * 3
    j = O.jsd_dense_rows(z, tl)
    torch.testing.assert_close(j, O.jsd_dense_rows(tl, z))
    assert (j >= 0).all() and (j <= math.log(2) + 1e-12).all()
    torch.testing.assert_close(O.jsd_dense_rows(z, z), torch.zeros(N, dtype=torch.float64), atol=1e-14, rtol=0)
    # disjoint supports -> ln 2
    a = torch.full((1, 6), float("-inf"), dtype=torch.float64)
    b = a.clone()
    a[0, :3] = 0.0
    b[0, 3:] = 1.0
    torch.testing.assert_close(O.jsd_dense_rows(a, b), torch.tensor([math.log(2)], dtype=torch.float64))
    # library cross-check: entropy form H(M) - (H(P)+H(Q))/2
    p, q = torch.softmax(z, -1), torch.softmax(tl, -1)
    m = 0.5 * (p + q)
    H = lambda x: -(x * x.log()).sum(-1)
    torch.testing.assert_close(j, H(m) - 0.5 * (H(p) + H(q)))
    # gradient closed form: 0.5 p_j (log(p_j/m_j) - KL(P||M))
    zr = z.clone().requires_grad_(True)
    O.jsd_dense_rows(zr, tl).sum().backward()
    klpm = (p * (p.log() - m.log())).sum(-1, keepdim=True)
    torch.testing.assert_close(zr.grad, 0.5 * p * (p.log() - m.log() - klpm), rtol=1e-9, atol=1e-13)


def test_gradcheck_all_row_losses():
    z, tv, ti = _rand_topk(3, 12, 4, 8)
    t = O.teacher_logprobs_topk(tv, 1.0, torch.float64)
    tl = torch.randn(3, 12, dtype=torch.float64)
    zr = z.clone().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda x: O.fwd_kl_topk_rows(x, t, ti), (zr,))
    assert torch.autograd.gradcheck(lambda x: O.rev_kl_topk_rows(x, t, ti), (zr,))
    for kind in ("fkl", "rkl", "jsd"):
        assert torch.autograd.gradcheck(lambda x: O.DENSE_ROWS[kind](x, tl), (zr,))


def test_topk_cross_entropy_against_loop():
    g = torch.Generator().manual_seed(9)
    N, K, V = 14, 5, 30
    lp = torch.randn(N, K, generator=g)
    idx = torch.stack([torch.randperm(V, generator=g)[:K] for _ in range(N)])
    labels = torch.randint(0, V, (N - 1,), generator=g)
    labels[::2] = idx[: N - 1: 2, 2]            # force hits on even rows
    ignore = torch.tensor([2, 8])
    got = O.topk_cross_entropy(lp, labels, idx, ignore)
    vals, valid = [], []
    for r in range(N - 1):
        pos = [k for k in range(K) if int(idx[r, k]) == int(labels[r])]
        ok = bool(pos) and r not in (2, 8)
        valid.append(ok)
        vals.append(float(lp[r, pos[0]]) if ok else None)
    mean = np.mean(np.array([v for v in vals if v is not None], dtype=np.float32))
    expect = np.array([-(v if v is not None else mean) for v in vals], dtype=np.float32)
    np.testing.assert_allclose(got.numpy(), expect, rtol=1e-6)
    assert got.shape == (N - 1,)


def test_alpha_weighted_special_cases():
    kl = torch.tensor([0.5, 2.0, 1.0], dtype=torch.float64)
    ce = torch.tensor([0.0, 0.0], dtype=torch.float64)
    # alpha = 0, CE = 0 -> weights 1 -> plain mean
    torch.testing.assert_close(O.alpha_weighted(kl, 0.0, ce), kl.mean())
    ce = torch.tensor([1.0, 3.0], dtype=torch.float64)    # padded with ONE zero
    expect = (kl * ((kl / 2.0 + 1) ** 2 + torch.tensor([1.0, 3.0, 0.0], dtype=torch.float64))).mean()
    torch.testing.assert_close(O.alpha_weighted(kl, 2.0, ce), expect)
    # the max is part of the graph: d/d kl_max has the extra -sum term
    k = kl.clone().requires_grad_(True)
    O.alpha_weighted(k, 2.0, torch.zeros(3, dtype=torch.float64)).backward()
    u = kl / 2.0
    dm = -(2 * kl * (u + 1) * kl / 4.0).sum()            # d/dmax of sum kl (kl/max+1)^2
    own = ((u + 1) ** 2 + 2 * kl * (u + 1) / 2.0)
    own[1] += dm
    torch.testing.assert_close(k.grad, own / 3)


def test_mean_loss_and_grad_masks_rows():
    g = torch.Generator().manual_seed(10)
    R, V, K = 8, 64, 6
    logits = (torch.randn(R, V, generator=g) * 2).to(torch.bfloat16)
    valid = torch.tensor([1, 1, 0, 1, 0, 1, 1, 0], dtype=torch.bool)
    nv = int(valid.sum())
    tv, ti = torch.topk(torch.log_softmax(torch.randn(nv, V, generator=g), -1), K)
    loss, rows, grad = O.mean_loss_and_grad("fkl", logits, 2.0, t_vals=tv, t_idx=ti, valid=valid)
    assert grad.dtype == torch.float32 and rows.shape == (nv,)
    assert torch.count_nonzero(grad[~valid]) == 0
    torch.testing.assert_close(loss, rows.mean())
    # every valid row's gradient sums to ~0 (softmax minus a distribution)
    assert grad[valid].float().sum(-1).abs().max() < 1e-6

"""GPU parity of the cross-tokenizer marginalisation and the fused reverse KL against it."""
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


def _case(R, Vs, Vt, seed, alphabet=4, drop=0.0):
    from llm_distillery_amd import synthetic as S
    import llm_distillery_amd as d
    student = S.random_byte_vocab(Vs, seed, alphabet=alphabet, max_len=6, all_single_bytes=(alphabet == 256))
    teacher = S.random_byte_vocab(Vt, seed + 1, alphabet=alphabet, max_len=8)
    t2s = d.vocab_utils.longest_prefix_map(student, teacher)
    if drop:
        t2s = t2s.copy()
        t2s[np.random.default_rng(seed).random(Vt) < drop] = -1
    g = torch.Generator().manual_seed(seed)
    probs = torch.softmax(torch.randn(R, Vt, generator=g) * 2, -1)
    return t2s, probs


def _map_in_the_form(D, planned, t2s, Vs):
    """False: the bare map on the GPU (LDS atomics); "full": the plan over the student ids only; "auto": what
    MarginalPlan builds by itself (the compact plan beside the full one where the map's image is small)."""
    if not planned:
        return torch.tensor(t2s, device=DEV)
    return D.vocab_utils.MarginalPlan(t2s, Vs, DEV, compact=False if planned == "full" else None)



@pytest.mark.parametrize("Vs,Vt,alphabet", [(1000, 5000, 4), (32000, 152064, 256), (40000, 50001, 16)])
def test_marginal_map_and_csr_forms(D, Vs, Vt, alphabet):
    t2s, probs = _case(6, Vs, Vt, 1, alphabet, drop=0.02)
    ref = O.marginalise_map(probs.numpy(), t2s, Vs)
    off, ind = D.vocab_utils.csr_from_map(t2s, Vs)
    np.testing.assert_allclose(ref, O.marginalise_csr(probs.numpy(), off, ind), rtol=1e-12, atol=1e-15)
    m_map = D.vocab_utils.marginalise(probs.to(DEV), t2s=torch.tensor(t2s, device=DEV), n_student=Vs).cpu().numpy()
    m_csr = D.vocab_utils.marginalise(probs.to(DEV), csr=(torch.tensor(off, device=DEV), torch.tensor(ind, device=DEV)),
                                      n_student=Vs).cpu().numpy()
    # marginal sums within fp32 tolerance; exact zeros where no teacher token maps
    np.testing.assert_allclose(m_map, ref, rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(m_csr, ref, rtol=2e-6, atol=1e-9)
    assert np.array_equal(m_map == 0, ref == 0) and np.array_equal(m_csr == 0, ref == 0)
    np.testing.assert_allclose(m_map.astype(np.float64).sum(-1), probs.double().numpy()[:, t2s >= 0].sum(-1), rtol=1e-5)
    # the CSR form is bit-reproducible
    again = D.vocab_utils.marginalise(probs.to(DEV), csr=(torch.tensor(off, device=DEV), torch.tensor(ind, device=DEV)),
                                      n_student=Vs).cpu().numpy()
    assert np.array_equal(m_csr, again)
    if Vs <= 36000:
        plan = D.vocab_utils.MarginalPlan(t2s, Vs, DEV)
        m_plan = D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy()
        np.testing.assert_allclose(m_plan, ref, rtol=2e-6, atol=1e-9)
        assert np.array_equal(m_plan == 0, ref == 0)
        assert np.array_equal(m_plan, D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy())
    lg = D.vocab_utils.marginalise(probs.to(DEV), t2s=torch.tensor(t2s, device=DEV), n_student=Vs, log=True).cpu().numpy()
    with np.errstate(divide="ignore"):
        np.testing.assert_allclose(lg[ref > 0], np.log(ref[ref > 0]), rtol=1e-5, atol=1e-5)
    assert np.isneginf(lg[ref == 0]).all()


def test_planned_marginal_with_lists_longer_than_one_batch(D):
    """A student vocabulary that leaves the LDS almost no room for replicas, and a few very hot ids:
    the per-thread lists of a tile then run over several batches of the kernel."""
    Vs, Vt, R = 36500, 30000, 5
    rng = np.random.default_rng(11)
    t2s = rng.integers(-1, Vs, Vt).astype(np.int32)
    hot = rng.random(Vt) < 0.9
    t2s[hot] = rng.integers(0, 16, int(hot.sum())) * 977
    probs = torch.softmax(torch.randn(R, Vt, generator=torch.Generator().manual_seed(11)) * 2, -1)
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, DEV)
    assert plan.ent is not None and int(np.diff(plan.row_off.cpu().numpy()).max()) > 8
    ref = O.marginalise_map(probs.numpy(), t2s, Vs)
    m_plan = D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy()
    np.testing.assert_allclose(m_plan, ref, rtol=4e-6, atol=1e-9)
    assert np.array_equal(m_plan == 0, ref == 0)
    assert np.array_equal(m_plan, D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy())


@pytest.mark.parametrize("case", ["one_hot_id", "all_dropped", "short", "tiny_student", "zipf"])
def test_planned_marginal_on_degenerate_maps(D, case):
    rng = np.random.default_rng(3)
    Vs, Vt, R = 3000, 20000, 4
    if case == "one_hot_id":
        t2s = np.where(rng.random(Vt) < 0.95, 17, rng.integers(0, Vs, Vt))
    elif case == "all_dropped":
        t2s = np.full(Vt, -1)
    elif case == "short":
        Vt = 1000
        t2s = rng.integers(0, Vs, Vt)
    elif case == "tiny_student":
        Vs = 4
        t2s = rng.integers(0, Vs, Vt)
    else:
        t2s = np.minimum(rng.zipf(1.2, Vt) - 1, Vs - 1)
    t2s = t2s.astype(np.int32)
    probs = torch.softmax(torch.randn(R, Vt, generator=torch.Generator().manual_seed(5)) * 2, -1)
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, DEV)
    ref = O.marginalise_map(probs.numpy(), t2s, Vs)
    m_plan = D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy()
    np.testing.assert_allclose(m_plan, ref, rtol=2e-5, atol=1e-9)
    assert np.array_equal(m_plan == 0, ref == 0)


def test_a_plan_built_for_other_vocabularies_is_refused(D):
    t2s = np.random.default_rng(0).integers(0, 1000, 5000).astype(np.int32)
    plan = D.vocab_utils.MarginalPlan(t2s, 1000, DEV)
    probs = torch.rand(2, 5000, device=DEV)
    with pytest.raises(RuntimeError, match="the plan maps"):
        D.vocab_utils.marginalise(probs, plan=plan, n_student=1008)
    with pytest.raises(RuntimeError, match="the plan maps"):
        D.vocab_utils.marginalise(torch.rand(2, 6000, device=DEV), plan=plan, n_student=1000)
    with pytest.raises(RuntimeError, match="the plan maps"):
        D.vocab_utils.rkl_marginalised(torch.randn(2, 1008, device=DEV), probs, plan)


def test_marginal_of_16bit_probabilities(D):
    t2s, probs = _case(4, 512, 2048, 2)
    got = D.vocab_utils.marginalise(probs.to(torch.bfloat16).to(DEV), t2s=torch.tensor(t2s, device=DEV), n_student=512)
    ref = O.marginalise_map(probs.to(torch.bfloat16).double().numpy(), t2s, 512)
    np.testing.assert_allclose(got.cpu().numpy(), ref, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("planned", [False, "full", "auto"])
@pytest.mark.parametrize("dtype,Vs,Vt,alphabet,T", [(torch.bfloat16, 32000, 152064, 256, 1.5), (torch.float32, 2048, 9000, 4, 1.0),
                                                    (torch.float16, 8192, 30000, 8, 0.8)])
def test_fused_reverse_kl_against_marginal(D, dtype, Vs, Vt, alphabet, T, planned):
    R = 12
    t2s, probs = _case(R, Vs, Vt, 3, alphabet, drop=0.01)
    g = torch.Generator().manual_seed(9)
    logits = (torch.randn(R + 3, Vs, generator=g) * 2).to(dtype)
    valid = torch.ones(R + 3, dtype=torch.bool)
    valid[[2, 5, 14]] = False
    rm = torch.full((R + 3,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(R, dtype=torch.int32)
    tmap = _map_in_the_form(D, planned, t2s, Vs)
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, row_map=rm.to(DEV), T=T,
                                              grad_scale=1.0 / R)
    if planned:       # fixed summation order: bit-reproducible
        rl2, grad2 = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, row_map=rm.to(DEV), T=T,
                                                    grad_scale=1.0 / R)
        assert torch.equal(rl, rl2) and torch.equal(grad, grad2)
    marg = torch.tensor(O.marginalise_map(probs.numpy(), t2s, Vs))
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg)
    loss64, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, T, t_logits=t_logits, valid=valid, dtype=torch.float64)
    np.testing.assert_allclose(D.reduce_sum(rl, 1.0 / R).item(), loss64.item(), rtol=1e-5)
    np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    assert torch.count_nonzero(grad.cpu()[~valid]) == 0 and torch.count_nonzero(rl.cpu()[~valid]) == 0
    err = (grad.cpu().double() - grad64).abs()
    rtol = 1e-4 if dtype == torch.float32 else 2e-3
    bound = O.storage_tolerance(grad64, dtype, rtol)
    sel = torch.nonzero(valid).squeeze(-1)
    bound[sel] = O.marginal_rkl_gradient_tolerance(grad64[sel], logits[sel], t_logits, rows64, T, T, 1.0 / R, dtype, rtol)
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    # the gradient is confined to the marginal's support
    assert torch.count_nonzero(grad.cpu()[valid][:, (marg.sum(0) == 0)]) == 0


@pytest.mark.parametrize("planned", [False, "full", "auto"])
@pytest.mark.parametrize("T", [1.0, 2.0, 0.5])
def test_fused_reverse_kl_on_rows_whose_sums_leave_the_range(D, T, planned):
    """Rows for which a bias of 0 for the teacher and the row's largest logit for the student do not keep
    the sums in range: hardly any teacher mass (down to denormal entries), an unnormalised teacher, a student
    whose mass sits on a column outside the marginal's support, and a teacher row without mass (zero loss,
    zero gradient)."""
    R, Vs, Vt = 6, 2048, 9000
    t2s, probs = _case(R, Vs, Vt, 5, 4, drop=0.01)
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(R, Vs, generator=g) * 2
    probs = probs.clone()
    probs[0] *= 1e-25
    probs[1] *= 1e25
    probs[5] *= 1e-33                                # most of the marginal's entries are denormal: their logarithms still count
    off = int(t2s[t2s >= 0][0])                      # a student column that is taken off the support of row 2
    probs[2, torch.tensor(t2s == off)] = 0.0
    logits[2, off] = 300.0
    probs[3] = 0.0
    tmap = _map_in_the_form(D, planned, t2s, Vs)
    with_mass = torch.tensor([0, 1, 2, 4, 5])
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, T=T, grad_scale=1.0 / len(with_mass))
    rl, grad = rl.cpu(), grad.cpu()
    assert rl[3] == 0 and torch.count_nonzero(grad[3]) == 0
    marg = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))[with_mass]
    assert marg[2, off] == 0
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg)
    _, rows64, grad64 = O.mean_loss_and_grad("rkl", logits[with_mass], T, t_logits=t_logits, dtype=torch.float64)
    np.testing.assert_allclose(rl[with_mass].double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    err = (grad[with_mass].double() - grad64).abs()
    bound = 1e-4 * grad64.abs() + 2e-6 * grad64.abs().amax(-1, keepdim=True)
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    assert torch.count_nonzero(grad[with_mass][marg == 0]) == 0
    # without a gradient the loss takes other passes over the row: the same values to rounding
    rl_only, none = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, T=T, want_grad=False)
    assert none is None
    np.testing.assert_allclose(rl_only.cpu().numpy(), rl.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lift", [3.0, 6.0, 12.0, 30.0])
def test_fused_reverse_kl_16bit_student_with_its_largest_logits_off_the_support(D, dtype, lift):
    """The student's largest logits sit on columns without teacher mass, `lift` above the rest: reverse KL
    renormalises the student over the support, so the columns that carry the gradient lie far below the
    row's maximum (what the kernel keeps of 2^logit between its passes must still resolve them)."""
    R, Vs, Vt = 5, 4096, 12000
    t2s, probs = _case(R, Vs, Vt, 7, 16, drop=0.01)
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(R, Vs, generator=g) * 2
    marg0 = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))
    on = torch.nonzero(marg0[0] > 0).squeeze(-1)
    off_cols = on[:6]                                # taken off the support of every row
    probs = probs.clone()
    probs[:, torch.isin(torch.tensor(t2s), off_cols)] = 0.0
    logits[:, off_cols] += lift
    logits = logits.to(dtype)
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), torch.tensor(t2s, device=DEV), T=0.7,
                                              teacher_T=1.0, grad_scale=1.0 / R)
    marg = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))
    assert (marg[:, off_cols] == 0).all()
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg)
    _, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, 0.7, t_logits=t_logits, t_T=1.0, dtype=torch.float64)
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    err = (grad.cpu().double() - grad64).abs()
    bound = O.marginal_rkl_gradient_tolerance(grad64, logits, t_logits, rows64, 0.7, 1.0, 1.0 / R, dtype, 2e-3)
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    assert torch.count_nonzero(grad.cpu()[:, off_cols]) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_reverse_kl_16bit_rows_whose_maximum_is_negative_zero_or_towering(D, dtype):
    """16-bit student rows take a non-negative maximum from the raw bit patterns, else from the values: rows
    of negative logits only, maxima of exactly +0 and -0, and one logit far above the rest at every position
    inside a 16-byte chunk in turn (a maximum that missed it would let the sums overflow)."""
    R, Vs, Vt = 12, 4096, 12000
    t2s, probs = _case(R, Vs, Vt, 9, 16, drop=0.01)
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(R, Vs, generator=g) * 2
    logits[0] = -logits[0].abs() - 0.5
    logits[1] = -logits[1].abs() - 1.0
    logits[1, 77] = 0.0
    logits[2] = -logits[2].abs() - 1.0
    logits[2, 1234] = -0.0
    marg0 = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))
    for r in range(4, 12):
        on = torch.nonzero(marg0[r] > 0).squeeze(-1)
        col = int(on[(on % 8) == (r - 4)][5])          # a column of the support at position r - 4 of its chunk
        logits[r, col] = 120.0
    logits = logits.to(dtype)
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), torch.tensor(t2s, device=DEV), T=1.0,
                                              grad_scale=1.0 / R)
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg0)
    _, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, 1.0, t_logits=t_logits, dtype=torch.float64)
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    err = (grad.cpu().double() - grad64).abs()
    bound = O.marginal_rkl_gradient_tolerance(grad64, logits, t_logits, rows64, 1.0, 1.0, 1.0 / R, dtype, 2e-3)
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("planned", [False, "full", "auto"])
def test_fused_reverse_kl_gradient_may_overwrite_the_logits(D, dtype, planned):
    """The gradient written over the logits, also for rows that are put back and redone (their logits are
    read a second time before anything of the row is written): the same bits as into a buffer of its own."""
    R, Vs, Vt = 6, 4096, 12000
    t2s, probs = _case(R, Vs, Vt, 7, 16, drop=0.01)
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(R, Vs, generator=g) * 2
    marg0 = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))
    off_cols = torch.nonzero(marg0[0] > 0).squeeze(-1)[:4]
    probs = probs.clone()
    probs[:, torch.isin(torch.tensor(t2s), off_cols)] = 0.0
    logits[1::2, off_cols] += 40.0                   # every other row has its mass off the support
    probs[4] *= 1e-30                                # and one hardly any teacher mass
    x = logits.to(dtype).to(DEV)
    tmap = _map_in_the_form(D, planned, t2s, Vs)
    rl, grad = D.vocab_utils.rkl_marginalised(x, probs.to(DEV), tmap, T=1.3, grad_scale=0.5)
    y = x.clone()
    rl2, g2 = D.vocab_utils.rkl_marginalised(y, probs.to(DEV), tmap, T=1.3, grad_scale=0.5, grad_out=y)
    assert g2.data_ptr() == y.data_ptr()
    if planned:                                      # fixed summation order: the same bits
        assert torch.equal(rl, rl2) and torch.equal(grad, y)
    else:                                            # LDS atomics: the marginal's sums come in any order
        np.testing.assert_allclose(rl2.cpu().numpy(), rl.cpu().numpy(), rtol=1e-5)
        tol = 1e-4 if dtype == torch.float32 else 2.0 ** -7
        diff = (grad.float() - y.float()).abs()
        assert (diff <= tol * grad.float().abs() + 1e-6 * grad.float().abs().max()).all()
    assert torch.isfinite(rl).all() and torch.isfinite(grad.float()).all() and grad.float().abs().max() > 0


def test_fused_path_limits_are_reported(D):
    with pytest.raises(RuntimeError, match="exceeds"):
        D.vocab_utils.rkl_marginalised(torch.zeros(2, 40000, device=DEV), torch.zeros(2, 64, device=DEV),
                                       torch.zeros(64, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_column_gather_and_expansion(D, dtype):
    """dl_gather_columns / dl_expand_columns move raw elements: a subset of the columns out (padding reads -inf)
    and back in (columns outside the subset read 0), every bit as it was."""
    g = torch.Generator().manual_seed(3)
    R, V = 7, 4104
    x = (torch.randn(R, V + 8, generator=g) * 3).to(dtype).to(DEV)[:, :V]           # rows of another pitch
    used = torch.sort(torch.randperm(V, generator=g)[:1001]).values
    cols = torch.full((1008,), -1, dtype=torch.int32)
    cols[:1001] = used.to(torch.int32)
    col_src = torch.full((V,), -1, dtype=torch.int32)
    col_src[used] = torch.arange(1001, dtype=torch.int32)
    xc = D.vocab_utils.gather_columns(x, cols.to(DEV))
    assert torch.equal(xc[:, :1001], x[:, used.to(DEV)]) and torch.isneginf(xc[:, 1001:].float()).all()
    back = D.vocab_utils.expand_columns(xc, col_src.to(DEV), V)
    want = torch.zeros_like(x)
    want[:, used.to(DEV)] = x[:, used.to(DEV)]
    assert torch.equal(back, want)


@pytest.mark.parametrize("dtype,Vs,Vt,alphabet", [(torch.bfloat16, 128256, 152064, 256), (torch.float32, 50000, 60000, 8),
                                                  (torch.float16, 8192, 30000, 16)])
def test_fused_reverse_kl_on_a_student_vocabulary_compacted_to_the_map_s_image(D, dtype, Vs, Vt, alphabet):
    """Student vocabularies wider than the fused kernel's marginal (and, on request, narrower ones): the plan is
    built over the student ids the map reaches, the logits' columns are gathered, the gradient expanded.  Loss
    and gradient against the oracle on the full vocabulary; columns outside the image get exactly 0; masked
    rows; bit-reproducible."""
    R = 9
    t2s, probs = _case(R, Vs, Vt, 5, alphabet, drop=0.01)
    g = torch.Generator().manual_seed(11)
    logits = (torch.randn(R + 2, Vs, generator=g) * 2).to(dtype)
    valid = torch.ones(R + 2, dtype=torch.bool)
    valid[[1, 7]] = False
    rm = torch.full((R + 2,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(R, dtype=torch.int32)
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, DEV, compact=True)
    assert plan.cols is not None and plan.n_compact % 8 == 0 and plan.n_compact < Vs
    T = 1.5
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), plan, row_map=rm.to(DEV), T=T, grad_scale=1.0 / R)
    rl2, grad2 = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), plan, row_map=rm.to(DEV), T=T, grad_scale=1.0 / R)
    assert torch.equal(rl, rl2) and torch.equal(grad, grad2) and grad.shape == logits.shape and grad.dtype == dtype
    marg = torch.tensor(O.marginalise_map(probs.numpy(), t2s, Vs))
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg)
    loss64, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, T, t_logits=t_logits, valid=valid, dtype=torch.float64)
    np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    assert torch.count_nonzero(grad.cpu()[~valid]) == 0 and torch.count_nonzero(rl.cpu()[~valid]) == 0
    rtol = 1e-4 if dtype == torch.float32 else 2e-3
    bound = O.storage_tolerance(grad64, dtype, rtol)
    sel = torch.nonzero(valid).squeeze(-1)
    bound[sel] = O.marginal_rkl_gradient_tolerance(grad64[sel], logits[sel], t_logits, rows64, T, T, 1.0 / R, dtype, rtol)
    err = (grad.cpu().double() - grad64).abs()
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    outside = torch.ones(Vs, dtype=torch.bool)
    outside[torch.as_tensor(np.unique(t2s[t2s >= 0])).long()] = False
    assert torch.count_nonzero(grad.cpu()[:, outside]) == 0
    rl3, _ = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), plan, row_map=rm.to(DEV), T=T, want_grad=False)
    np.testing.assert_allclose(rl3.cpu().numpy(), rl.cpu().numpy(), rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("Vs,dtype", [(4008, torch.float32), (4000, torch.bfloat16)])
def test_a_plan_that_holds_the_compact_form_only(D, Vs, dtype):
    """No full plan to fall back to: the fused kernel runs on the compact ids, and `marginalise` gives the full-width marginal from the bare map."""
    R, Vt = 5, 9000
    t2s, probs = _case(R, Vs, Vt, 9, 16)
    plan = D.vocab_utils.MarginalPlan(t2s, Vs, DEV, compact=True)
    assert plan.full is None and plan.compact is not None
    g = torch.Generator().manual_seed(4)
    logits = (torch.randn(R, Vs, generator=g) * 2).to(dtype)
    rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), plan, T=1.2, grad_scale=1.0 / R)
    marg = torch.tensor(O.marginalise_map(probs.numpy(), t2s, Vs))
    with np.errstate(divide="ignore"):
        t_logits = O.marginal_to_teacher_logits(marg)
    _, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, 1.2, t_logits=t_logits, dtype=torch.float64)
    np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=3e-5, atol=3e-6)
    bound = O.marginal_rkl_gradient_tolerance(grad64, logits, t_logits, rows64, 1.2, 1.2, 1.0 / R, dtype,
                                              1e-4 if dtype == torch.float32 else 2e-3)
    err = (grad.cpu().double() - grad64).abs()
    assert (err <= bound).all(), f"worst ratio {(err / bound).max():.2f}"
    m = D.vocab_utils.marginalise(probs.to(DEV), plan=plan, n_student=Vs).cpu().numpy()
    np.testing.assert_allclose(m, marg.numpy(), rtol=2e-6, atol=1e-9)

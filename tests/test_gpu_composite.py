"""GPU parity of the two-phase path and the drop-in `calculate_divergence` (through the custom op
and the C ABI) against the golden vectors written from the reference and against the CPU oracle."""
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


_bound = O.composite_gradient_tolerance


def _golden(golden_dir, case):
    d = np.load(os.path.join(golden_dir, "calculate_divergence.npz"))
    return {k[len(case) + 1:]: d[k] for k in d.files if k.startswith(case + "/")}


@pytest.mark.parametrize("case", ["two_ranges", "one_range", "alpha0", "alpha_half"])
def test_calculate_divergence_matches_reference_golden(D, golden_dir, case):
    g = _golden(golden_dir, case)
    s = torch.tensor(g["student"], device=DEV, requires_grad=True)
    res = D.calculate_divergence(s, torch.tensor(g["teacher"], device=DEV), torch.tensor(g["indices"], device=DEV),
                                 torch.tensor(g["labels"], device=DEV), float(g["alpha"]),
                                 torch.tensor(g["avoid"], dtype=torch.long, device=DEV))
    assert tuple(res.keys()) == D.LOSS_KEYS
    for k in D.LOSS_KEYS:
        np.testing.assert_allclose(res[k].item(), g[f"out/{k}"], rtol=1e-5, atol=1e-6, err_msg=k)
    res["train_loss"].backward()
    ref = torch.tensor(g["grad"])
    err = (s.grad.cpu() - ref).abs()
    bound = _bound(ref.double(), torch.tensor(g["student"]), 1.0, torch.float32, 1e-4, None, torch.tensor(g["indices"]))
    assert (err <= bound).all(), (err / bound).max()


def _convo(N, V, K, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    student = (torch.randn(N, V, generator=g) * 2).to(dtype)
    tfull = torch.log_softmax(student.float() + torch.randn(N, V, generator=g), -1)
    tv, ti = torch.topk(tfull, K)
    tv = tv.to(torch.float16).float()
    labels = ti[:N - 1, 0].clone()
    miss = torch.rand(N - 1, generator=g) < 0.3
    labels[miss] = torch.randint(0, V, (int(miss.sum()),), generator=g)
    return student, tv, ti, labels


@pytest.mark.parametrize("V,K,N", [(32000, 200, 130), (128256, 64, 21), (1000, 16, 50), (32003, 200, 40), (1001, 16, 50), (5, 3, 9)])
def test_calculate_divergence_against_oracle_fp32(D, V, K, N):
    student, tv, ti, labels = _convo(N, V, K, 5)
    avoid = torch.tensor([3, N // 2])
    ref_in = student.double().requires_grad_(True)
    ref = O.calculate_divergence(ref_in, tv.double(), ti, labels, 2.0, avoid)
    ref["train_loss"].backward()
    s = student.to(DEV).requires_grad_(True)
    res = D.calculate_divergence(s, tv.to(DEV), ti.to(DEV), labels.to(DEV), 2.0, avoid.to(DEV))
    for k in D.LOSS_KEYS:
        np.testing.assert_allclose(res[k].item(), ref[k].item(), rtol=1e-5, atol=1e-6, err_msg=k)
    res["train_loss"].backward()
    err = (s.grad.cpu().double() - ref_in.grad).abs()
    bound = _bound(ref_in.grad, student, 1.0, torch.float32, 1e-4, None, ti)
    assert (err <= bound).all(), (err / bound).max()


def test_student_rows_beyond_the_teacher_are_dropped_with_zero_gradient(D):
    """utils/finetuning_utils.py:87-88: only the first min(#student, #teacher, #indices) rows count.
    The extra student rows are masked inside the kernels (no slice of the [N, V] logits, whose
    backward would cost a zero fill and a copy of that size); their gradient rows are zero."""
    student, tv, ti, labels = _convo(30, 4096, 16, 8)
    n = 23
    avoid = torch.tensor([4])
    ref_in = student.double().requires_grad_(True)
    ref = O.calculate_divergence(ref_in, tv[:n].double(), ti[:n], labels[:n - 1], 2.0, avoid)
    ref["train_loss"].backward()
    s = student.to(DEV).requires_grad_(True)
    res = D.calculate_divergence(s, tv[:n].to(DEV), ti[:n].to(DEV), labels[:n - 1].to(DEV), 2.0, avoid.to(DEV))
    for k in D.LOSS_KEYS:
        np.testing.assert_allclose(res[k].item(), ref[k].item(), rtol=1e-5, atol=1e-6, err_msg=k)
    res["train_loss"].backward()
    assert s.grad.shape == student.shape and torch.count_nonzero(s.grad[n:]) == 0
    err = (s.grad.cpu().double() - ref_in.grad).abs()
    bound = _bound(ref_in.grad, student, 1.0, torch.float32, 1e-4, None, ti[:n])
    assert (err <= bound).all(), (err / bound).max()


def test_under_no_grad_and_reference_error_behaviour(D):
    student, tv, ti, labels = _convo(12, 512, 8, 6)
    with torch.no_grad():
        res = D.calculate_divergence(student.to(DEV), tv.to(DEV), ti.to(DEV), labels.to(DEV), 2.0,
                                     torch.zeros(0, dtype=torch.long, device=DEV))
    assert not res["train_loss"].requires_grad and torch.isfinite(res["train_loss"])
    # as many labels as rows: the reference's comparison cannot broadcast and raises; so does this
    with pytest.raises((RuntimeError, IndexError)):
        D.calculate_divergence(student.to(DEV), tv.to(DEV), ti.to(DEV), torch.zeros(12, dtype=torch.long, device=DEV),
                               2.0, torch.zeros(0, dtype=torch.long, device=DEV))
    with pytest.raises(TypeError):
        D.calculate_divergence(student.to(DEV), tv.to(DEV), None, labels.to(DEV), 2.0,
                               torch.zeros(0, dtype=torch.long, device=DEV))


@pytest.mark.parametrize("teacher_T", [None, 1.0])
def test_distill_loss_fuses_crop_cast_temperature_and_row_selection(D, teacher_T):
    """The extended entry point against the reference's caller sequence restated on the CPU:
    logits[:, :crop].float() / T -> index_select(content rows) -> teacher / T -> calculate_divergence
    (classes/student/model.py:408,420-425; validation twin :501-502 leaves the teacher unscaled)."""
    g = torch.Generator().manual_seed(7)
    S, Vm, crop, K, T = 88, 32064, 32000, 100, 1.5      # the last label falls at the conversation end and is dropped
    ranges = [(5, 30), (41, 88)]
    model_logits = (torch.randn(S, Vm, generator=g) * 2).to(torch.bfloat16)
    rows = torch.as_tensor(O.content_indices(ranges))
    lab_pos, avoid = O.ce_indices(ranges, 2048, S)
    tokens = torch.randint(0, crop, (S,), generator=g)
    N = rows.numel()
    tfull = torch.log_softmax(model_logits[rows, :crop].float() + torch.randn(N, crop, generator=g), -1)
    tv, ti = torch.topk(tfull, K)
    tokens[torch.as_tensor(lab_pos)] = ti[:len(lab_pos), 1]            # most labels are among the ids
    labels = tokens[torch.as_tensor(lab_pos)]
    tT = T if teacher_T is None else teacher_T
    z = O.scaled_student_logits(model_logits, crop, T, torch.float64).requires_grad_(True)
    ref = O.calculate_divergence(torch.index_select(z, 0, rows), tv.double() / tT, ti, labels, 2.0, torch.as_tensor(avoid))
    ref["train_loss"].backward()
    x = model_logits.to(DEV).requires_grad_(True)
    res = D.distill_loss(x, rows.to(DEV), tv.to(torch.float16).to(DEV), ti.to(torch.int32).to(DEV), labels.to(DEV),
                         2.0, torch.as_tensor(avoid).to(DEV), temperature=T, crop_to_size=crop,
                         teacher_temperature=teacher_T)
    ref16 = O.calculate_divergence(torch.index_select(z.detach(), 0, rows), tv.to(torch.float16).double() / tT, ti, labels,
                                   2.0, torch.as_tensor(avoid))
    for k in D.LOSS_KEYS:
        np.testing.assert_allclose(res[k].item(), ref16[k].item(), rtol=2e-5, atol=2e-6, err_msg=k)
    res["train_loss"].backward()
    assert x.grad.shape == model_logits.shape and x.grad.dtype == torch.bfloat16
    assert torch.count_nonzero(x.grad[:, crop:]) == 0
    gref = torch.zeros(S, Vm, dtype=torch.float64)
    gref[:, :crop] = z.grad / T
    err = (x.grad.cpu().double() - gref).abs()
    # fp16 teacher storage moves the loss by ~1e-4; compare gradients against the same-teacher oracle
    z2 = O.scaled_student_logits(model_logits, crop, T, torch.float64).requires_grad_(True)
    O.calculate_divergence(torch.index_select(z2, 0, rows), tv.to(torch.float16).double() / tT, ti, labels, 2.0,
                           torch.as_tensor(avoid))["train_loss"].backward()
    gref[:, :crop] = z2.grad / T
    err = (x.grad.cpu().double() - gref).abs()
    bound = _bound(gref, model_logits, T, torch.bfloat16, 2e-3, rows, ti, crop)
    assert (err <= bound).all(), (err / bound).max()


def test_rowstats_raw_outputs_and_losses_accumulator_on_gpu(D):
    g = torch.Generator().manual_seed(8)
    R, V, K = 33, 50264, 40
    x = (torch.randn(R, V, generator=g) * 3).to(torch.bfloat16)
    idx = torch.randint(0, V, (R, K), generator=g, dtype=torch.int32)
    lse, zk = D.rowstats_topk(x.to(DEV), idx.to(DEV), None, 0.5)
    ref_lse = torch.logsumexp(x.double() * 0.5, -1)
    np.testing.assert_allclose(lse.cpu().double().numpy(), ref_lse.numpy(), rtol=1e-6, atol=1e-6)
    assert torch.equal(zk.cpu(), torch.gather(x.float(), 1, idx.long()) * 0.5)
    # a batch of two conversations through the accumulator: sum / grad_accum, as the training loop does
    L = D.Losses(None)
    leafs = []
    for seed in (1, 2):
        gg = torch.Generator().manual_seed(seed)
        s = torch.randn(9, 256, generator=gg).to(DEV).requires_grad_(True)
        tv, ti = torch.topk(torch.log_softmax(torch.randn(9, 256, generator=gg), -1), 6)
        L.add_losses(D.calculate_divergence(s, tv.to(DEV), ti.to(DEV), ti[:8, 0].to(DEV), 2.0,
                                            torch.zeros(0, dtype=torch.long, device=DEV)))
        leafs.append(s)
    total = L.loss_dict["train_loss"].item()
    L.backward(divisor=2)
    assert all(s.grad is not None and torch.isfinite(s.grad).all() for s in leafs)
    assert total > 0 and L.num_steps_accumulated == 2


def test_rowstats_with_more_teacher_rows_than_logits_rows(D):
    """utils/finetuning_utils.py:87: only min(#student, #teacher) rows count.  Teacher rows beyond the logits'
    are nobody's: their statistics come back as zeros, not as whatever the allocation held."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 4096, generator=g).to(DEV)
    idx = torch.randint(0, 4096, (9, 12), generator=g, dtype=torch.int32).to(DEV)
    junk = torch.full((9, 12), float("nan"), device=DEV)          # make the allocator's next block dirty
    del junk
    lse, zk = D.rowstats_topk(x, idx, None, 1.0)
    assert lse.shape == (9,) and zk.shape == (9, 12)
    assert torch.count_nonzero(lse[5:]) == 0 and torch.count_nonzero(zk[5:]) == 0
    np.testing.assert_allclose(lse[:5].cpu().numpy(), torch.logsumexp(x.cpu().double(), -1).numpy(), rtol=1e-6)


@pytest.mark.parametrize("dtype,V,pitch,offset", [(torch.bfloat16, 32003, 32003, 0), (torch.float32, 1003, 1003, 0),
                                                  (torch.bfloat16, 5001, 5120, 3), (torch.float16, 7, 7, 0),
                                                  # crops of padded rows: on the 16-byte grid, the last chunk ragged
                                                  (torch.bfloat16, 5001, 5120, 0), (torch.float32, 32003, 32064, 0),
                                                  (torch.bfloat16, 50257, 50304, 0), (torch.float16, 16385, 16392, 0)])
@pytest.mark.parametrize("grad_mode", ["fresh", "other_phase"])
def test_two_phase_kernels_on_rows_off_the_16_byte_grid(D, dtype, V, pitch, offset, grad_mode):
    """Phase 1 and phase 2 on rows that do not start or end on 16-byte boundaries (vector accesses to the
    chunks inside them, element-wise beside; element-wise throughout when the gradient buffer sits on
    another phase of the grid), with repeated ids, ids in the first and last columns and masked rows."""
    from llm_distillery_amd import ops
    R, K = 9, min(12, V)
    g = torch.Generator().manual_seed(V)
    xs = (torch.randn(R, V, generator=g) * 3).to(dtype)
    idx = torch.randint(0, V, (R - 2, K), generator=g, dtype=torch.int32)
    idx[:, 0] = 0
    idx[:, 1] = V - 1
    idx[:, 2] = idx[:, 1]                                         # a repeated id in the last column
    rm = torch.tensor([0, 1, -1, 2, 3, 4, -1, 5, 6], dtype=torch.int32)
    full = torch.zeros(R, pitch + 8, dtype=dtype, device=DEV)
    x = full[:, offset:offset + V] if pitch != V else xs.to(DEV)
    if pitch != V:
        x.copy_(xs.to(DEV))
    inv_T = 0.7
    lse, zk = ops._rowstats_raw(x, idx.to(DEV), rm.to(DEV), inv_T)
    sel = rm >= 0
    ref_lse = torch.logsumexp(xs[sel].double() * inv_T, -1)
    np.testing.assert_allclose(lse.cpu().double().numpy(), ref_lse.numpy(), rtol=2e-6, atol=2e-6)
    assert torch.equal(zk.cpu(), torch.gather(xs[sel].float(), 1, idx.long()) * inv_T)
    g_lse = torch.randn(R - 2, generator=g)
    g_zk = torch.randn(R - 2, K, generator=g)
    out = None if grad_mode == "fresh" else torch.empty(R, x.stride(0) + 1, dtype=dtype, device=DEV)[:, 1:1 + V]
    grad = ops._rowcoef_grad_raw(x, idx.to(DEV), rm.to(DEV), inv_T, lse, g_lse.to(DEV), g_zk.to(DEV), grad_out=out)
    ref = torch.zeros(R, V, dtype=torch.float64)
    p = torch.softmax(xs[sel].double() * inv_T, -1) * g_lse.double().unsqueeze(-1)
    p.scatter_add_(1, idx.long(), g_zk.double())
    ref[sel] = p * inv_T
    err = (grad.cpu().double() - ref).abs()
    # a_i = g_lse inv_T is known here; the corrections are random numbers, two of them on a repeated id: on the
    # support, fp32 rounding of their sum on the scale of the row's largest coefficient
    bound = O.storage_tolerance(ref, dtype, 1e-4 if dtype == torch.float32 else 2e-3)
    bound[sel] = O.sparse_gradient_tolerance(ref[sel], xs[sel], 1.0 / inv_T, idx.long(), dtype, 1e-4 if dtype == torch.float32 else 2e-3,
                                             support_scale=4e-7, row_coef=(g_lse.double() * inv_T).unsqueeze(-1))
    assert (err <= bound).all(), f"worst {(err / bound).max():.2f}"
    assert torch.count_nonzero(grad.cpu()[~sel]) == 0


def test_batched_caller_equals_the_per_conversation_loop(D):
    """One pass over [B, S, V] for all conversations of a batch gives, conversation by conversation, the
    dicts the reference's loop gives (restated on the CPU), and after Losses.backward the same gradient."""
    g = torch.Generator().manual_seed(11)
    B, S, Vm, crop, K, T, accum = 3, 60, 4160, 4096, 24, 1.3, 2
    model_logits = (torch.randn(B, S, Vm, generator=g) * 2).to(torch.bfloat16)
    specs = [[(4, 20), (30, 41)], [(0, 55)], [(10, 16), (20, 30), (44, 59)]]
    lens = [41, 55, 59]
    convos_cpu, convos_gpu = [], []
    for b in range(B):
        rows = torch.as_tensor(O.content_indices(specs[b]))
        lab_pos, avoid = O.ce_indices(specs[b], 2048, lens[b])
        N = rows.numel()
        tfull = torch.log_softmax(model_logits[b, rows, :crop].float() + torch.randn(N, crop, generator=g), -1)
        tv, ti = torch.topk(tfull, K)
        tv = tv.to(torch.float16)
        tokens = torch.randint(0, crop, (S + 1,), generator=g)
        tokens[torch.as_tensor(lab_pos)] = ti[:len(lab_pos), 0]
        labels = tokens[torch.as_tensor(lab_pos)]
        convos_cpu.append((rows, tv, ti, labels, torch.as_tensor(avoid)))
        convos_gpu.append((rows.to(DEV), tv.to(DEV), ti.to(torch.int32).to(DEV), labels.to(DEV), torch.as_tensor(avoid).to(DEV)))
    # reference loop on the CPU in float64
    z = O.scaled_student_logits(model_logits, crop, T, torch.float64).requires_grad_(True)
    ref_dicts, total = [], 0
    for b, (rows, tv, ti, labels, avoid) in enumerate(convos_cpu):
        d = O.calculate_divergence(torch.index_select(z[b], 0, rows), tv.double() / T, ti, labels, 2.0, avoid)
        ref_dicts.append(d)
        total = total + d["train_loss"]
    (total / accum).backward()
    x = model_logits.to(DEV).requires_grad_(True)
    L = D.Losses(None)
    dicts = D.distill_loss_batch(x, convos_gpu, 2.0, temperature=T, crop_to_size=crop)
    values = [{k: d[k].item() for k in D.LOSS_KEYS} for d in dicts]
    for d, r in zip(dicts, ref_dicts):
        for k in D.LOSS_KEYS:
            np.testing.assert_allclose(d[k].item(), r[k].item(), rtol=2e-5, atol=2e-6, err_msg=k)
        L.add_losses(d)
    L.backward(divisor=accum)
    gref = torch.zeros(B, S, Vm, dtype=torch.float64)
    gref[:, :, :crop] = z.grad / T
    err = (x.grad.cpu().double() - gref).abs()
    for b, (rows, tv, ti, labels, avoid) in enumerate(convos_cpu):
        bound = _bound(gref[b], model_logits[b], T, torch.bfloat16, 2e-3, rows, ti, crop)
        assert (err[b] <= bound).all(), (b, (err[b] / bound).max())
    assert torch.count_nonzero(x.grad[0, 41:]) == 0            # rows outside every content range
    # the same batch from content ranges: every index array built on the host and uploaded once
    x2 = model_logits.to(DEV).requires_grad_(True)
    index = D.BatchIndex(specs, lens, S, 2048, DEV)
    tokens_b = torch.zeros(B, S + 1, dtype=torch.long)
    for b, (_, _, _, labels, _) in enumerate(convos_cpu):
        tokens_b[b, torch.as_tensor(O.ce_indices(specs[b], 2048, lens[b])[0])] = labels
    dicts2 = D.distill_loss_batch_indexed(x2, index, tokens_b.to(DEV), [(c[1], c[2]) for c in convos_gpu], 2.0,
                                          temperature=T, crop_to_size=crop)
    L2 = D.Losses(None)
    for v, d2 in zip(values, dicts2):
        for k in D.LOSS_KEYS:
            assert v[k] == d2[k].item(), k
        L2.add_losses(d2)
    L2.backward(divisor=accum)
    assert torch.equal(x.grad, x2.grad)



def _ranged_convo(g, S, V, K, ranges, convo_len, label_hits=0.8):
    """One conversation's pieces (CPU): content rows, stored teacher rows, labels, ignore rows."""
    rows = torch.as_tensor(O.content_indices(ranges))
    lab_pos, avoid = O.ce_indices(ranges, 2048, convo_len)
    N = rows.numel()
    ti = torch.stack([torch.randperm(V, generator=g)[:K] for _ in range(N)])
    tv = torch.log_softmax(torch.randn(N, K, generator=g) * 2, -1).to(torch.float16)
    labels = torch.where(torch.rand(len(lab_pos), generator=g) < label_hits, ti[:len(lab_pos), 3],
                         torch.full((len(lab_pos),), V + 7))          # a label outside the row's ids: invalid row
    return rows, tv, ti, labels, torch.as_tensor(avoid)


@pytest.mark.parametrize("alpha", [2.0, 0.7])
def test_fused_epilogue_equals_the_torch_epilogue(D, alpha):
    """The fused K-wide epilogue (three launches per batch) against the same arithmetic written with
    the torch routines the reference uses (taken when alpha is a tensor): all nine values per
    conversation and the gradient of the logits, including an all-invalid conversation (NaN cross
    entropies, as in the reference) and tied maxima (duplicated rows: max's gradient is shared)."""
    g = torch.Generator().manual_seed(21)
    B, S, V, K, T = 4, 48, 2048, 16, 1.7
    specs = [[(2, 20), (25, 40)], [(0, 33)], [(5, 9), (12, 30), (31, 44)], [(1, 30)]]
    lens = [40, 33, 44, 30]
    convos = [_ranged_convo(g, S, V, K, specs[b], lens[b], label_hits=0.0 if b == 3 else 0.8) for b in range(B)]
    logits = torch.randn(B, S, V, generator=g) * 2                # fp32: the gradients compare unrounded
    logits[1, 7] = logits[1, 3]                                   # two identical rows ...
    r, tv, ti, lab, av = convos[1]
    tv[7], ti[7] = tv[3], ti[3]                                   # ... with identical teachers: tied kl and rkl
    dev_convos = [tuple(t.to(DEV) for t in c) for c in convos]

    def run(a):
        x = logits.to(DEV).requires_grad_(True)
        dicts = D.distill_loss_batch(x, dev_convos, a, temperature=T)
        vals = [{k: d[k].item() for k in D.LOSS_KEYS} for d in dicts]
        total = sum(d["train_loss"] for d in dicts[:3])          # conversation 3 is NaN by construction
        total.backward()
        return vals, x.grad, dicts

    fused, g_fused, dicts = run(alpha)
    plain, g_plain, _ = run(torch.tensor(alpha, device=DEV))      # a tensor alpha takes the torch epilogue
    assert dicts[0]["train_loss"].requires_grad and not dicts[0]["kl_div"].requires_grad
    assert type(dicts[0]["train_loss"].grad_fn).__name__ == "SelectBackward0"
    for b in range(B):
        for k in D.LOSS_KEYS:
            if b == 3 and k not in ("kl_div", "reverse kl_div"):
                assert np.isnan(fused[b][k]) and np.isnan(plain[b][k]), k
            else:
                np.testing.assert_allclose(fused[b][k], plain[b][k], rtol=3e-6, atol=1e-7, err_msg=f"{b} {k}")
    err = (g_fused.float() - g_plain.float()).abs().cpu()
    for b in range(B):
        bound = _bound(g_plain[b].double().cpu(), logits[b], T, torch.float32, 1e-4, convos[b][0], convos[b][2])
        assert (err[b] <= bound).all(), (b, float((err[b] / bound).max()))
    assert torch.count_nonzero(g_fused[3]) == 0


def test_registered_composite_operators_equal_the_eager_node(D):
    """distillery_amd::composite_forward / composite_backward (torch.library operators with fake implementations and a
    registered autograd formula) run the launches of the eager autograd node: the same bits forward and backward;
    torch.library.opcheck accepts schema, fake tensors and autograd registration."""
    from llm_distillery_amd import ops
    g = torch.Generator().manual_seed(31)
    S, V, K = 40, 4096, 16
    specs, lens = [[(2, 17)], [(20, 38)]], [17, 38]
    logits = (torch.randn(S, V, generator=g) * 2).to(torch.bfloat16).to(DEV)
    convos = [_ranged_convo(g, S, V, K, specs[b], lens[b]) for b in range(2)]
    rows = torch.cat([c[0] for c in convos])
    rm = torch.full((S,), -1, dtype=torch.int32)
    rm[rows] = torch.arange(rows.numel(), dtype=torch.int32)
    t_val = torch.cat([c[1] for c in convos]).to(DEV)
    t_idx = torch.cat([c[2] for c in convos]).to(torch.int32).to(DEV)
    labels = torch.cat([c[3] for c in convos]).to(DEV)
    avoid = torch.cat([c[4] for c in convos]).to(DEV)
    counts = [c[0].numel() for c in convos]
    offs = [[0, counts[0], sum(counts)], [0, convos[0][3].numel(), labels.numel()], [0, convos[0][4].numel(), avoid.numel()]]
    offs_dev = torch.tensor(offs, dtype=torch.int32, device=DEV)
    x1 = logits.clone().requires_grad_(True)
    train1, nine1 = ops.composite_loss(x1, t_val, t_idx, labels, avoid, offs, rm.to(DEV), 1 / 1.3, 1 / 1.3, 2.0, 0)
    train1.sum().backward()
    x2 = logits.clone().requires_grad_(True)
    res = ops.composite_forward_op(x2, t_val, t_idx, labels, avoid, offs_dev, rm.to(DEV), 1 / 1.3, 1 / 1.3, 2.0, 0)
    res[0].sum().backward()
    assert torch.equal(train1, res[0]) and torch.equal(nine1, res[1]) and torch.equal(x1.grad, x2.grad)
    torch.library.opcheck(ops.composite_forward_op, (x2.detach(), t_val, t_idx, labels, avoid, offs_dev, rm.to(DEV), 1 / 1.3, 1 / 1.3, 2.0, 0),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))


def test_fused_epilogue_under_no_grad_and_label_count_mismatch(D):
    g = torch.Generator().manual_seed(5)
    rows, tv, ti, labels, avoid = _ranged_convo(g, 40, 1024, 8, [(3, 19)], 19)
    z = (torch.randn(rows.numel(), 1024, generator=g)).to(DEV)
    with torch.no_grad():
        d = D.calculate_divergence(z, tv.float().to(DEV), ti.to(DEV), labels.to(DEV), 2.0, avoid.to(DEV))
    ref = O.calculate_divergence(z.cpu().double(), tv.double(), ti, labels, 2.0, avoid)
    for k in D.LOSS_KEYS:
        np.testing.assert_allclose(d[k].item(), ref[k].item(), rtol=2e-5, atol=2e-6, err_msg=k)
    # as many labels as rows: the reference raises (empty crop); so does the drop-in, from the same torch ops
    with pytest.raises(RuntimeError):
        D.calculate_divergence(z, tv.float().to(DEV), ti.to(DEV), torch.cat([labels, labels[:1]]).to(DEV), 2.0, avoid.to(DEV))


@pytest.mark.parametrize("dtype,V,pitch,K,lens,host_offsets", [
    (torch.float32, 32000, 32000, 400, [130], True),            # the reference's default width and K, one conversation
    (torch.bfloat16, 5001, 5120, 37, [20, 1, 33], False),       # a crop of padded rows, K off the wave size, device offsets
    (torch.float16, 1003, 1003, 16, [9, 40], True),             # rows off the 16-byte grid
    (torch.bfloat16, 128256, 128256, 200, [5, 6], True),
    (torch.float32, 4096, 4096, 600, [12, 7], True)])
def test_coefficients_made_inside_phase_two_equal_the_separate_launches(D, dtype, V, pitch, K, lens, host_offsets):
    """Phase 2 makes the K coefficients of a row itself (dl_composite_backward_fused), or reads what
    dl_composite_backward wrote: ops.FORCE_COMPOSITE_BACKWARD sends the same problem through either form.  With and without a row map (one that scatters
    the teacher rows over more logits rows, some of them masked).  Forward: the same launches, the same bits.
    Backward: the sum of the K coefficients is taken in another order, so the gradients agree to fp32 rounding of
    the dense term; masked rows get zeros."""
    from llm_distillery_amd import ops
    N = sum(lens)
    g = torch.Generator().manual_seed(V + K)
    xs = (torch.randn(N, V, generator=g) * 2).to(dtype)
    tfull = torch.log_softmax(xs.float() + torch.randn(N, V, generator=g), -1)
    tv, ti = torch.topk(tfull, K)
    tv = tv.to(torch.float16).contiguous()
    labels, row_off, label_off, avoid_off, avoid = [], [0], [0], [0], []
    for n in lens:
        r0 = row_off[-1]
        lab = ti[r0:r0 + n - 1, 0].clone()
        miss = torch.rand(max(n - 1, 0), generator=g) < 0.3
        lab[miss] = torch.randint(0, V, (int(miss.sum()),), generator=g)
        labels.append(lab)
        row_off.append(r0 + n)
        label_off.append(label_off[-1] + n - 1)
        if n > 4:
            avoid.append(n // 2)
        avoid_off.append(len(avoid))
    labels = torch.cat(labels).to(DEV)
    avoid = torch.tensor(avoid, dtype=torch.int64, device=DEV)
    offsets = [row_off, label_off, avoid_off]
    if not host_offsets:
        offsets = torch.tensor(offsets, dtype=torch.int32, device=DEV)
    same = lambda a, b: torch.equal(a.nan_to_num(nan=-7.0), b.nan_to_num(nan=-7.0))      # a conversation of one row has no labels: its CE means are 0 / 0
    # logits rows: as many as teacher rows, or more of them with the teacher rows scattered over every third but one
    R = N + N // 2 + 3
    place = torch.sort(torch.randperm(R, generator=g)[:N]).values
    scatter = torch.full((R,), -1, dtype=torch.int32)
    scatter[place] = torch.arange(N, dtype=torch.int32)
    for rm, rows in ((None, torch.arange(N)), (scatter.to(DEV), place)):
        full = torch.randn(N if rm is None else R, pitch, generator=g).to(dtype).to(DEV)      # masked rows hold logits too
        full[rows.to(DEV), :V] = xs.to(DEV)
        res = {}
        for name in ("fused", "separate"):
            ops.FORCE_COMPOSITE_BACKWARD = name
            try:
                x = full.clone().requires_grad_(True)
                train, nine = ops.composite_loss(x, tv.to(DEV), ti.to(DEV), labels, avoid, offsets, rm, 1.0 / 1.3, 1.0, 2.0, crop=V if pitch != V else 0)
                w = torch.arange(1, len(lens) + 1, dtype=torch.float32, device=DEV)
                (train * w).sum().backward()
            finally:
                ops.FORCE_COMPOSITE_BACKWARD = None
            res[name] = (train.detach(), nine, x.grad)
        assert same(res["fused"][0], res["separate"][0]) and same(res["fused"][1], res["separate"][1])
        gf, gs = res["fused"][2].float(), res["separate"][2].float()
        assert torch.count_nonzero(gf[:, V:]) == 0
        if rm is not None:
            masked = torch.ones(R, dtype=torch.bool)
            masked[place] = False
            assert torch.count_nonzero(gf[masked.to(DEV)]) == 0
        tol = gs.abs() * (2e-5 if dtype == torch.float32 else 2.0 ** -7) + gs.abs().amax(-1, keepdim=True) * 1e-6
        assert ((gf - gs).abs() <= tol).all(), ((gf - gs).abs() / tol).max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_phase_one_logits_at_clustered_repeated_and_outlying_teacher_ids(D, dtype):
    """Rows whose ids all fall on every 256th chunk, rows with one id K times, ids in the first and the last column
    and ids outside the row: zk bit for bit the gathered logits times 1/T, zeros for ids outside."""
    from llm_distillery_amd import ops
    R, V, K = 6, 32768, 40
    n = 16 // torch.empty(0, dtype=dtype).element_size()           # columns per 16-byte chunk
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(R, V, generator=g) * 3).to(dtype)
    idx = torch.randint(0, V, (R, K), generator=g, dtype=torch.int64)
    idx[0] = (torch.arange(K) % (V // (256 * n))) * 256 * n + 5 * n + 1      # every 256th chunk (some ids twice)
    idx[1] = idx[1, 0]                                                      # one id K times
    idx[2, :4] = torch.tensor([0, V - 1, -1, V])                            # first and last column, two ids outside the row
    idx[3] = torch.arange(K) * n                                           # consecutive chunks, one id each
    lse, zk = ops._rowstats_raw(x.to(DEV), idx.to(DEV), None, 0.7)
    inside = (idx >= 0) & (idx < V)
    want = torch.where(inside, torch.gather(x.float(), 1, idx.clamp(0, V - 1)) * 0.7, torch.zeros(()))
    assert torch.equal(zk.cpu(), want)
    np.testing.assert_allclose(lse.cpu().double().numpy(), torch.logsumexp(x.double() * 0.7, -1).numpy(), rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("dtype,V,K", [(torch.bfloat16, 131072, 64),      # 64 rounds of 256 chunks: the widest row whose ids come out of the sweep
                                       (torch.bfloat16, 131080, 64),      # one chunk more: gathered directly
                                       (torch.float32, 65536, 300), (torch.float32, 65540, 300),
                                       (torch.bfloat16, 50257, 200),      # rows off the 16-byte grid: ids before and behind the aligned body
                                       (torch.float32, 32003, 1100),      # more entries than the sweep keeps slots for
                                       (torch.float16, 4104, 1024)])
def test_phase_one_ids_out_of_the_sweep_or_gathered(D, dtype, V, K):
    """zk is the logit at the teacher's id times 1/T, bit for bit, whichever way phase 1 fetches it: out of its sweep
    (rows of up to 64 rounds, up to 1024 entries), by loads of its own beyond, element by element in the columns before
    and behind the aligned body of a row off the 16-byte grid."""
    from llm_distillery_amd import ops
    R = 5
    g = torch.Generator().manual_seed(V + K)
    x = (torch.randn(R, V, generator=g) * 3).to(dtype)
    idx = torch.randint(0, V, (R, K), generator=g, dtype=torch.int64)
    idx[0, :16] = torch.arange(16)                                         # the row's first columns
    idx[1, :16] = V - 1 - torch.arange(16)                                 # and its last
    idx[2, :8] = torch.tensor([-5, V, V + 7, 2 ** 31 - 1, -1, 0, V - 1, V // 2])
    idx[3] = idx[3, 0] // 8 * 8 + torch.arange(K) % 8                      # every entry in one chunk or two
    lse, zk = ops._rowstats_raw(x.to(DEV), idx.to(DEV), None, 1.0 / 1.3)
    inside = (idx >= 0) & (idx < V)
    want = torch.where(inside, torch.gather(x.float(), 1, idx.clamp(0, V - 1)) * np.float32(1.0 / 1.3), torch.zeros(()))
    assert torch.equal(zk.cpu(), want)
    np.testing.assert_allclose(lse.cpu().double().numpy(), torch.logsumexp(x.double() / 1.3, -1).numpy(), rtol=3e-6, atol=3e-6)


@pytest.mark.parametrize("dtype,V,pitch,K,lens,host_offsets", [
    (torch.float32, 32000, 32000, 400, [130], True),            # the reference's default width and K
    (torch.bfloat16, 5001, 5120, 37, [20, 1, 33], False),       # a crop of padded rows, K off the wave size, device offsets
    (torch.float16, 1003, 1003, 16, [9, 40], True),             # rows off the 16-byte grid
    (torch.bfloat16, 128256, 128256, 200, [5, 6], True),
    (torch.float32, 4096, 4096, 1024, [12, 7], True),           # four entries per thread
    (torch.float32, 4096, 4096, 1100, [12, 7], True)])          # beyond what the tail of phase 1 takes: three launches
def test_records_made_at_the_tail_of_phase_one_equal_the_separate_launches(D, dtype, V, pitch, K, lens, host_offsets):
    """dl_composite_forward_fused against dl_rowstats_topk + dl_composite_forward (ops.SEPARATE_COMPOSITE_FORWARD):
    lse and zk bit for bit, the nine values and the gradient to fp32 rounding (the sums over K are taken by a
    workgroup instead of a wave); teacher values in every storage type, labels that hit and miss the support."""
    from llm_distillery_amd import ops
    N = sum(lens)
    g = torch.Generator().manual_seed(V + K)
    xs = (torch.randn(N, V, generator=g) * 2).to(dtype)
    tfull = torch.log_softmax(xs.float() + torch.randn(N, V, generator=g), -1)
    tv, ti = torch.topk(tfull, K)
    labels, row_off, label_off, avoid_off, avoid = [], [0], [0], [0], []
    for n in lens:
        r0 = row_off[-1]
        lab = ti[r0:r0 + n - 1, K // 3].clone()
        miss = torch.rand(max(n - 1, 0), generator=g) < 0.3
        lab[miss] = torch.randint(0, V, (int(miss.sum()),), generator=g)
        labels.append(lab)
        row_off.append(r0 + n)
        label_off.append(label_off[-1] + n - 1)
        if n > 4:
            avoid.append(n // 2)
        avoid_off.append(len(avoid))
    labels = torch.cat(labels).to(DEV)
    avoid = torch.tensor(avoid, dtype=torch.int64, device=DEV)
    offsets = [row_off, label_off, avoid_off]
    if not host_offsets:
        offsets = torch.tensor(offsets, dtype=torch.int32, device=DEV)
    full = torch.zeros(N, pitch, dtype=dtype, device=DEV)
    full[:, :V] = xs.to(DEV)
    same = lambda a, b: torch.equal(a.nan_to_num(nan=-7.0), b.nan_to_num(nan=-7.0))
    for tdt, idt in ((torch.float32, torch.int64), (torch.float16, torch.int32), (torch.bfloat16, torch.int64)):
        res = {}
        for name in ("fused", "separate"):
            ops.SEPARATE_COMPOSITE_FORWARD = name == "separate"
            try:
                x = full.clone().requires_grad_(True)
                crop = V if pitch != V else 0
                out, lse, zk, rec, coef = ops._composite_forward_raw(x.detach(), tv.to(tdt).to(DEV), ti.to(idt).to(DEV), labels, avoid,
                                                                     offsets, None, 1.0 / 1.3, 1.0, 2.0, crop, True)
                train, nine = ops.composite_loss(x, tv.to(tdt).to(DEV), ti.to(idt).to(DEV), labels, avoid, offsets, None, 1.0 / 1.3, 1.0, 2.0, crop=crop)
                w = torch.arange(1, len(lens) + 1, dtype=torch.float32, device=DEV)
                (train * w).sum().backward()
            finally:
                ops.SEPARATE_COMPOSITE_FORWARD = False
            res[name] = (lse, zk, rec, out, nine, x.grad)
        f, s_ = res["fused"], res["separate"]
        assert torch.equal(f[0], s_[0]) and torch.equal(f[1], s_[1])                      # lse, zk
        assert torch.equal(f[2].view(torch.int32)[:, 6:], s_[2].view(torch.int32)[:, 6:])  # kstar, valid
        np.testing.assert_allclose(f[2][:, :6].cpu().numpy(), s_[2][:, :6].cpu().numpy(), rtol=2e-5, atol=2e-6)
        np.testing.assert_allclose(f[3].nan_to_num(nan=-7.0).cpu().numpy(), s_[3].nan_to_num(nan=-7.0).cpu().numpy(), rtol=2e-5, atol=2e-6)
        assert same(f[3], f[4])
        gf, gs = f[5].float(), s_[5].float()
        tol = gs.abs() * (1e-4 if dtype == torch.float32 else 2.0 ** -7) + gs.abs().amax(-1, keepdim=True) * 2e-6
        assert ((gf - gs).abs() <= tol).all(), ((gf - gs).abs() / tol).max()

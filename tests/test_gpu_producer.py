"""GPU parity of the teacher producer (log-softmax over V + top-K, storage layout) against the oracle."""
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


def _ref(logits, crop, K):
    """torch.topk semantics with the tie rule made explicit: equal log-probs -> smaller id first
    (a stable descending sort of the full-vocabulary log-softmax)."""
    logp = torch.log_softmax(logits[..., :crop].double(), dim=-1)
    order = torch.sort(logits[..., :crop].float(), dim=-1, descending=True, stable=True).indices[..., :K]
    return torch.gather(logp, -1, order), order


@pytest.mark.parametrize("dtype,V,K", [(torch.bfloat16, 32000, 200), (torch.bfloat16, 128256, 400), (torch.float16, 32000, 64),
                                       (torch.float32, 32000, 200), (torch.float32, 50264, 1024), (torch.bfloat16, 2048, 17)])
def test_topk_ids_bit_exact_values_close(D, dtype, V, K):
    g = torch.Generator().manual_seed(V + K)
    logits = (torch.randn(9, V, generator=g) * 3).to(dtype)
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int64)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu(), ri), "ids (including tie order: smaller id first) must match exactly"
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), rtol=0, atol=2e-6 * max(1.0, float(rv.abs().max())))
    assert (val[:, :-1] >= val[:, 1:]).all()
    # the oracle's producer (torch.topk) returns the same value set
    ov, _ = O.teacher_topk_producer(logits, V, K)
    np.testing.assert_allclose(val.cpu().numpy(), ov.numpy(), rtol=0, atol=3e-6 * max(1.0, float(ov.abs().max())))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rows_whose_largest_logit_is_negative_or_zero(D, dtype):
    """16-bit rows take their maximum from the raw bit patterns when it is not negative, else from the
    values: rows of negative logits only, rows whose maximum is +0 or -0, and ordinary rows between them."""
    g = torch.Generator().manual_seed(5)
    V, K = 40000, 64
    logits = torch.randn(8, V, generator=g) * 3
    logits[0] = -logits[0].abs() - 0.5
    logits[1] = -logits[1].abs() - 20.0
    logits[2] = torch.minimum(logits[2], torch.zeros(()))                    # maximum +0, many times
    logits[3] = -logits[3].abs() - 1.0
    logits[3, 777] = -0.0
    logits[5, :] = -7.25
    logits = logits.to(dtype)
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int64)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu(), ri)
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), rtol=0, atol=2e-6 * max(1.0, float(rv.abs().max())))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rows_with_one_towering_logit(D, dtype):
    """A logit far above the rest of its row, at every position inside a 16-byte chunk in turn: a maximum
    that missed it would let the sum of exponentials overflow."""
    g = torch.Generator().manual_seed(6)
    V, K = 40000, 32
    logits = torch.randn(8, V, generator=g) * 2
    for r in range(8):
        logits[r, 8 * (100 + 37 * r) + r] = 150.0
    logits = logits.to(dtype)
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int64)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu(), ri) and torch.isfinite(val).all()
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), rtol=0, atol=3e-6 * float(rv.abs().max()))


def test_storage_layout_crop_and_content_rows(D):
    g = torch.Generator().manual_seed(3)
    B, S, Vm, crop, K = 2, 40, 32064, 32000, 100
    logits = (torch.randn(B, S, Vm, generator=g) * 2).to(torch.bfloat16)
    rows = torch.as_tensor(np.concatenate([O.content_indices([(3, 9), (20, 31)]), S + O.content_indices([(0, 40)])]), dtype=torch.int32)
    val, idx = D.teacher_topk(logits.to(DEV), K, crop_to_size=crop, rows=rows.to(DEV))
    assert val.dtype == torch.float16 and idx.dtype == torch.int32 and val.shape == (rows.numel(), K)
    flat = logits.reshape(B * S, Vm)[rows.long()]
    rv, ri = _ref(flat, crop, K)
    assert torch.equal(idx.cpu().long(), ri) and int(idx.max()) < crop
    assert torch.equal(val.cpu(), rv.to(torch.float32).to(torch.float16)) or \
        (val.cpu().float() - rv.float()).abs().max() <= 2e-3 * rv.abs().max()
    # round trip through the dataset's dtypes and into the loss: producer output is a valid sparse teacher
    rl, _ = D.div_topk("fkl", logits.reshape(B * S, Vm)[:, :crop].to(DEV)[rows.long().to(DEV)].contiguous(), val, idx, unique_ids=True)
    # a model distilled from itself: KL(q || p) = -log(student mass on the top-K support)
    mass = torch.gather(torch.softmax(flat[:, :crop].double(), -1), 1, ri).sum(-1)
    np.testing.assert_allclose(rl.cpu().double().numpy(), -torch.log(mass).numpy(), rtol=2e-3, atol=2e-3)


def test_heavy_ties_and_constant_rows(D):
    # quantised logits: thousands of entries share the threshold value; constant rows: all equal
    g = torch.Generator().manual_seed(4)
    V, K = 16384, 300
    logits = torch.randint(-3, 4, (5, V), generator=g).to(torch.bfloat16)
    logits[3] = 1.5
    logits[4, ::2] = float("-inf")
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int32)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu().long(), ri)
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), atol=1e-5)
    assert idx[3].cpu().tolist() == list(range(K))


@pytest.mark.parametrize("n_tied", [300, 1000, 3000])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tie_plateaus_of_every_size(D, dtype, n_tied):
    # a plateau of equal top values wider than K: the candidate set of a part outgrows its record
    # (sorted and cut inside the part: in one wave, in LDS, or through the exact bisection select)
    g = torch.Generator().manual_seed(n_tied)
    V, K = 65536, 64
    logits = (torch.randn(4, V, generator=g).clamp(max=3.0)).to(dtype)
    for r in range(4):
        pos = torch.randperm(V // 2, generator=g)[:n_tied] + (0 if r % 2 == 0 else V // 2)
        logits[r, pos] = 5.0
        logits[r, int(pos[0])] = 6.0
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int32)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu().long(), ri)
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n_blocks", [12, 20, 28])
def test_a_plateau_packed_into_few_stretches_of_the_row(D, dtype, n_blocks):
    """Hundreds of equal entries that fill a few contiguous stretches of the row: few chunk groups hold them, so the
    bound taken from the group maxima lies below the plateau and the selection meets more candidates than one wave
    sorts (between 512 and the list's size), all of them tied at the K-th value but a few."""
    g = torch.Generator().manual_seed(n_blocks)
    V, K = 128256, 200
    logits = (torch.randn(6, V, generator=g) * 2).clamp(max=7.5)
    for r in range(6):
        starts = torch.randperm(V // 64 - 1, generator=g)[:n_blocks] * 64
        for s0 in starts.tolist():
            logits[r, s0:s0 + 32] = 8.0
        above = torch.randperm(V, generator=g)[: 5 * r]
        logits[r, above] = 9.0 + torch.rand(above.numel(), generator=g)
    logits = logits.to(dtype)
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int32)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu().long(), ri)
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), atol=1e-5)


@pytest.mark.parametrize("dtype,V,K", [(torch.bfloat16, 50257, 200), (torch.float32, 50257, 400), (torch.float16, 1001, 10),
                                       (torch.bfloat16, 131073, 64), (torch.float32, 7, 7)])
def test_any_vocabulary_size(D, dtype, V, K):
    """The reference's producer takes any `crop_distr_to_size` (classes/teacher/inference_worker.py:73-77):
    vocabularies that are not a whole number of 16-byte chunks, rows on odd pitches."""
    g = torch.Generator().manual_seed(V)
    logits = (torch.randn(6, V, generator=g) * 3).to(dtype)
    logits[2, V - 1] = 9.0                                   # the last column of the padded tail chunk wins a row
    logits[4, V - 3:] = float("-inf")
    val, idx = D.teacher_topk(logits.to(DEV), K, val_dtype=torch.float32, idx_dtype=torch.int64)
    rv, ri = _ref(logits, V, K)
    assert torch.equal(idx.cpu(), ri) and int(idx.max()) < V
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), rtol=0, atol=2e-6 * max(1.0, float(rv[torch.isfinite(rv)].abs().max())))


def test_odd_crop_of_a_wider_vocabulary_and_tied_tails(D):
    g = torch.Generator().manual_seed(12)
    B, S, Vm, crop, K = 2, 7, 32003, 31999, 120
    logits = (torch.randn(B, S, Vm, generator=g) * 2).to(torch.bfloat16)
    logits[..., crop:] = 20.0                                # beyond the crop: must never be seen
    logits[0, 3, crop - 40:crop] = 4.0                       # a tie plateau that runs into the padded tail
    val, idx = D.teacher_topk(logits.to(DEV), K, crop_to_size=crop, val_dtype=torch.float32, idx_dtype=torch.int32)
    rv, ri = _ref(logits.reshape(B * S, Vm), crop, K)
    assert torch.equal(idx.cpu().long(), ri) and int(idx.max()) < crop
    np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), atol=1e-5)
    # a constant row of odd width: every column ties, the first K ids win
    const = torch.full((3, 4099), 0.25, dtype=torch.float16)
    _, ci = D.teacher_topk(const.to(DEV), 300, idx_dtype=torch.int32)
    assert ci[1].cpu().tolist() == list(range(300))


def test_row_list_entries_outside_the_logits_give_masked_rows(D):
    g = torch.Generator().manual_seed(5)
    logits = (torch.randn(10, 4096, generator=g) * 2).to(torch.bfloat16)
    rows = torch.tensor([3, -1, 9, 10, 0, 2 ** 31 - 1, -(2 ** 31)], dtype=torch.int32)
    val, idx = D.teacher_topk(logits.to(DEV), 32, rows=rows.to(DEV), val_dtype=torch.float32)
    good = torch.tensor([0, 2, 4])
    rv, ri = _ref(logits[rows[good].long()], 4096, 32)
    assert torch.equal(idx.cpu()[good].long(), ri)
    np.testing.assert_allclose(val.cpu()[good].double().numpy(), rv.numpy(), atol=1e-5)
    bad = torch.tensor([1, 3, 5, 6])
    assert (idx.cpu()[bad] == -1).all() and torch.isneginf(val.cpu()[bad]).all()


def test_producer_limits(D):
    with pytest.raises(RuntimeError):
        D.teacher_topk(torch.zeros(2, 4096, device=DEV), 2000)
    with pytest.raises(RuntimeError):
        D.teacher_topk(torch.zeros(2, 100, device=DEV), 101)              # K > V

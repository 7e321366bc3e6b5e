"""GPU parity of the sparse-teacher kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-3, torch.float16: 2e-3}


@pytest.fixture(scope="module")
def D():
    import llm_distillery_amd as d
    d._lib.load()
    return d


def _case(R, V, K, dtype, seed, std=2.0, idx_dtype=torch.int32, val_dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(R, V, generator=g) * std).to(dtype)
    tl = torch.log_softmax(logits.float() + torch.randn(R, V, generator=g), -1)
    tv, ti = torch.topk(tl, K)
    return logits, tv.to(val_dtype), ti.to(idx_dtype)


def _check(D, kind, logits, tv, ti, T, valid=None, teacher_T=None, hooks=None, **tol_over):
    R, V = logits.shape
    n_valid = R if valid is None else int(valid.sum())
    loss64, rows64, grad64 = O.mean_loss_and_grad(kind, logits, T, t_vals=tv, t_idx=ti, valid=valid, t_T=teacher_T,
                                             dtype=torch.float64)
    row_map = None
    if valid is not None:
        rm = torch.full((R,), -1, dtype=torch.int32)
        rm[valid] = torch.arange(n_valid, dtype=torch.int32)
        row_map = rm.to(DEV)
    rl, grad = D.div_topk(kind, logits.to(DEV), tv.to(DEV), ti.to(DEV), row_map=row_map, T=T, teacher_T=teacher_T,
                          grad_scale=1.0 / n_valid, **(hooks or {}))
    loss = D.reduce_sum(rl, 1.0 / n_valid)
    torch.cuda.synchronize()
    rows_gpu = rl.cpu()
    if valid is not None:
        assert torch.count_nonzero(rows_gpu[~valid]) == 0
        assert torch.count_nonzero(grad.cpu()[~valid]) == 0
        rows_gpu = rows_gpu[valid]
    # loss: 1e-5 relative against the float64 oracle (fp32 accumulation in the kernel)
    np.testing.assert_allclose(loss.item(), loss64.item(), rtol=1e-5)
    np.testing.assert_allclose(rows_gpu.double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    # gradients, entry by entry: 1e-4 (fp32 logits) / 2e-3 (16-bit logits) of the entry's own value, the half
    # ulp that storing it in the logits' dtype may add, and fp32 rounding of the entry's own cancelling terms
    rtol = tol_over.get("rtol", TOL[logits.dtype])
    err = (grad.cpu().double() - grad64).abs()
    bound = O.topk_gradient_tolerance(kind, grad64, logits, tv, ti, T, teacher_T, 1.0 / n_valid, logits.dtype, rtol, valid)
    bad = err > bound
    assert not bad.any(), f"{int(bad.sum())} gradient entries off; worst ratio {(err / bound).max().item():.3f}"
    return grad


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["fkl", "rkl"])
def test_topk_small(D, dtype, kind):
    logits, tv, ti = _case(37, 1024, 24, dtype, 1)
    _check(D, kind, logits, tv, ti, T=1.0)


@pytest.mark.parametrize("V,K", [(32000, 200), (128256, 200), (50264, 64), (8192, 400), (32000, 2048), (128256, 1024),
                                 (65536, 2048), (40968, 200), (49152, 1000), (53248, 400), (53256, 16)])      # 512 x 13 chunks up to 53248 columns
def test_fkl_topk_register_path_sizes(D, V, K):
    logits, tv, ti = _case(24, V, K, torch.bfloat16, 2, std=3.0)
    _check(D, "fkl", logits, tv, ti, T=1.0)


def test_fkl_topk_fp32_vocab_32000_temperature_and_mask(D):
    logits, tv, ti = _case(40, 32000, 100, torch.float32, 3)
    valid = torch.ones(40, dtype=torch.bool)
    valid[[3, 4, 17, 39]] = False
    _check(D, "fkl", logits, tv[:36], ti[:36], T=2.0, valid=valid)
    _check(D, "rkl", logits, tv[:36], ti[:36], T=0.7, valid=valid)


def test_validation_asymmetry_teacher_not_scaled(D):
    # classes/student/model.py:501-502: the student is divided by T, the teacher is not
    logits, tv, ti = _case(16, 4096, 32, torch.float32, 4)
    _check(D, "fkl", logits, tv, ti, T=1.7, teacher_T=1.0)


@pytest.mark.parametrize("V", [1000, 32003, 130001])
def test_streaming_path_odd_vocab_and_int64_fp32_teacher(D, V):
    # V not a multiple of the 16-byte chunk -> streaming kernel; teacher as the reference loads it (fp32/int64)
    logits, tv, ti = _case(9, V, 50, torch.bfloat16, 5, idx_dtype=torch.int64, val_dtype=torch.float32)
    _check(D, "fkl", logits, tv, ti, T=1.3)
    _check(D, "rkl", logits, tv, ti, T=1.3)


@pytest.mark.parametrize("dtype,V,pitch,offset", [(torch.bfloat16, 32003, 32003, 0),      # contiguous odd rows: every row starts elsewhere on the grid
                                                  (torch.float32, 1003, 1003, 0),
                                                  (torch.bfloat16, 5001, 5120, 3),          # a column slice of aligned rows: one phase for all rows
                                                  (torch.float16, 7, 7, 0),                 # rows shorter than a chunk
                                                  (torch.float32, 4099, 4104, 2),
                                                  (torch.bfloat16, 50257, 50257, 0),        # wider than 256 x 16 chunks: two column parts
                                                  (torch.float16, 151665, 151665, 0),       # five
                                                  (torch.float32, 40003, 40003, 0),         # three, of four-byte chunks
                                                  (torch.float32, 10001, 10001, 0)])        # 512 threads x 8 chunks of fp32
@pytest.mark.parametrize("grad_mode", ["fresh", "in_place", "other_phase"])
@pytest.mark.parametrize("kind", ["fkl", "rkl"])
def test_rows_off_the_16_byte_grid(D, kind, dtype, V, pitch, offset, grad_mode):
    """Rows that do not start on 16-byte boundaries or do not end on one.  Forward KL: rows of up to
    256 x 16 chunks stay in the register kernels (unaligned 16-byte accesses, the last, partly filled chunk
    element by element); wider ones stream, their 16-byte chunks through aligned vector accesses when
    logits and gradient rows share their address modulo 16 (a fresh gradient of the same pitch, or the
    gradient written over the logits), else through the unaligned register kernel as far as that holds a
    row.  Reverse KL, which only gathers from the logits, goes by the gradient rows alone.  All against
    the oracle."""
    R, K = 7, min(24, V)
    logits, tv, ti = _case(R, V, K, dtype, 61, std=3.0)
    valid = torch.ones(R, dtype=torch.bool)
    valid[2] = False
    rm = torch.full((R,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(R - 1, dtype=torch.int32)
    tv, ti = tv[valid], ti[valid]
    ti[:, 0] = 0                                                  # entries in the first and the last column
    ti[:, 1] = V - 1
    if K > 3:
        ti[:, 2] = V - 1                                          # and a repeated id there
    tl = torch.log_softmax(logits[valid].float() * 1.1, -1)       # teacher values that belong to those ids
    tv = torch.gather(tl, 1, ti.long()).to(tv.dtype)
    loss64, rows64, grad64 = O.mean_loss_and_grad(kind, logits, 1.3, t_vals=tv, t_idx=ti, valid=valid, dtype=torch.float64)
    full = torch.zeros(R, pitch + 8, dtype=dtype, device=DEV)
    x = full[:, offset:offset + V] if pitch != V else logits.to(DEV)
    if pitch != V:
        x.copy_(logits.to(DEV))
    assert x.stride(0) == (pitch + 8 if pitch != V else V)
    if grad_mode == "fresh":
        out = None
    elif grad_mode == "in_place":
        out = x
    else:
        out = torch.empty(R, x.stride(0) + 1, dtype=dtype, device=DEV)[:, 1:1 + V]
    rl, grad = D.div_topk(kind, x, tv.to(DEV), ti.to(DEV), row_map=rm.to(DEV), T=1.3, grad_scale=1.0 / (R - 1), grad_out=out)
    assert grad_mode == "fresh" or grad.data_ptr() == out.data_ptr()
    np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    assert rl[2].item() == 0 and torch.count_nonzero(grad[2]) == 0
    err = (grad.cpu().double() - grad64).abs()
    bound = O.topk_gradient_tolerance(kind, grad64, logits, tv, ti, 1.3, None, 1.0 / (R - 1), dtype, TOL[dtype], valid)
    assert (err <= bound).all(), f"worst {(err / bound).max():.2f}"
    if pitch != V and grad_mode != "in_place":      # nothing outside the slice was touched
        assert torch.count_nonzero(full[:, :offset]) == 0 and torch.count_nonzero(full[:, offset + V:]) == 0


@pytest.mark.parametrize("dtype,V,pitch", [(torch.bfloat16, 50257, 50304),      # GPT-2's vocabulary in its padded rows: 512 x 13, one workgroup per row
                                           (torch.bfloat16, 151665, 151936),    # Qwen's: five column parts, the last one ragged
                                           (torch.float16, 100277, 100352),     # four parts of 13 chunks per thread
                                           (torch.float32, 32003, 32064),       # 512 x 16 of four-byte chunks
                                           (torch.float16, 4099, 4104),         # 256 x 4
                                           (torch.bfloat16, 65537, 65544),      # one column more than two parts hold: the third part is one ragged chunk
                                           (torch.float32, 70001, 70008),       # five parts of four-byte chunks
                                           (torch.bfloat16, 262139, 262144)])   # eight parts in four workgroups of 512 threads
@pytest.mark.parametrize("grad_mode", ["fresh", "in_place", "other_pitch", "other_phase"])
def test_crop_of_a_padded_vocabulary(D, dtype, V, pitch, grad_mode):
    """logits[:, :, :crop] of rows padded to a multiple of 16 bytes (classes/student/model.py:408): rows start on
    the 16-byte grid and end inside a chunk.  The register kernels take them like whole rows, one workgroup per
    row or cut into column parts, and move only the row's last chunk element by element; nothing beyond the crop
    is written.  A gradient buffer off the grid (other_phase) falls back to the unaligned / streaming kernels.
    With and without waiting for the partners: the oracle's numbers and the same bits."""
    R, K = 11, 48
    logits, tv, ti = _case(R, V, K, dtype, 71, std=3.0)
    valid = torch.ones(R, dtype=torch.bool)
    valid[[2, 10]] = False
    nv = int(valid.sum())
    rm = torch.full((R,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(nv, dtype=torch.int32)
    tv, ti = tv[valid], ti[valid]
    ti[:, 0] = 0                                                  # entries in the first and the last column
    ti[:, 1] = V - 1
    ti[:, 2] = V - 1                                              # a repeated id in the ragged chunk
    ti[:, 3] = V - V % (8 if dtype != torch.float32 else 4)       # the ragged chunk's first column
    tl = torch.log_softmax(logits[valid].float() * 1.1, -1)
    tv = torch.gather(tl, 1, ti.long()).to(tv.dtype)
    _, rows64, grad64 = O.mean_loss_and_grad("fkl", logits, 1.3, t_vals=tv, t_idx=ti, valid=valid, dtype=torch.float64)
    bound = O.topk_gradient_tolerance("fkl", grad64, logits, tv, ti, 1.3, None, 1.0 / nv, dtype, TOL[dtype], valid)
    results = []
    for no_wait in (False, True):
        full = torch.full((R, pitch), 7.0, dtype=dtype, device=DEV)
        x = full[:, :V]
        x.copy_(logits.to(DEV))
        assert x.data_ptr() % 16 == 0 and (x.stride(0) * x.element_size()) % 16 == 0
        if grad_mode == "fresh":
            out = None
        elif grad_mode == "in_place":
            out = x
        elif grad_mode == "other_pitch":
            out = torch.full((R, pitch + 64), 5.0, dtype=dtype, device=DEV)[:, :V]
        else:
            out = torch.full((R, pitch + 1), 5.0, dtype=dtype, device=DEV)[:, 1:1 + V]
        rl, grad = D.div_topk("fkl", x, tv.to(DEV), ti.to(DEV), row_map=rm.to(DEV), T=1.3, grad_scale=1.0 / nv, grad_out=out,
                              no_wait=no_wait)
        assert grad_mode == "fresh" or grad.data_ptr() == out.data_ptr()
        np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
        assert torch.count_nonzero(rl[~valid.to(DEV)]) == 0 and torch.count_nonzero(grad[~valid.to(DEV)]) == 0
        err = (grad.cpu().double() - grad64).abs()
        assert (err <= bound).all(), f"worst {(err / bound).max():.2f}"
        assert (full[:, V:] == 7.0).all()                         # nothing beyond the crop was touched
        if grad_mode == "other_pitch":
            assert (out.as_strided((R, pitch + 64 - V), (pitch + 64, 1), out.storage_offset() + V) == 5.0).all()
        results.append((rl.clone(), grad.clone()))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])


def test_streaming_path_rows_larger_than_register_file(D):
    logits, tv, ti = _case(6, 152064, 200, torch.bfloat16, 6)
    _check(D, "fkl", logits, tv, ti, T=1.0)
    logits, tv, ti = _case(4, 100000, 64, torch.float32, 7)
    _check(D, "fkl", logits, tv, ti, T=1.0)


def test_cropped_view_of_wider_model_vocab(D):
    # classes/student/model.py:408 slices [:, :, :crop] out of the model's vocabulary
    g = torch.Generator().manual_seed(8)
    full = (torch.randn(2, 10, 32064, generator=g) * 2).to(torch.bfloat16)
    crop = full[:, :, :32000]
    flat = crop.reshape(20, 32000)
    tl = torch.log_softmax(flat.float() + torch.randn(20, 32000, generator=g), -1)
    tv, ti = torch.topk(tl, 40)
    loss64, rows64, grad_ref = O.mean_loss_and_grad("fkl", flat, 1.0, t_vals=tv, t_idx=ti, dtype=torch.float32)
    dev_full = full.to(DEV)
    rl, grad = D.div_topk("fkl", dev_full[:, :, :32000], tv.to(DEV), ti.to(torch.int32).to(DEV), grad_scale=1 / 20)
    assert grad.shape == (2, 10, 32000)
    np.testing.assert_allclose(rl.cpu().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6)
    err = (grad.cpu().float().reshape(20, -1) - grad_ref).abs()
    assert (err <= O.sparse_gradient_tolerance(grad_ref.double(), flat, 1.0, ti, torch.bfloat16, 2e-3)).all()


def test_duplicate_ids_ragged_counts_and_out_of_range_ids(D):
    g = torch.Generator().manual_seed(9)
    R, V, K = 12, 2048, 16
    logits = (torch.randn(R, V, generator=g) * 2)
    ti = torch.randint(0, V, (R, K), generator=g)
    ti[:, 5] = ti[:, 2]                  # duplicates inside a row accumulate
    tv = torch.randn(R, K, generator=g)
    _check(D, "fkl", logits, tv, ti.to(torch.int32), T=1.0)
    _check(D, "rkl", logits, tv, ti.to(torch.int32), T=1.0)
    # ragged: only the first cnt entries count; ids outside [0, V) are ignored; empty rows give 0
    cnt = torch.tensor([16, 1, 0, 7, 16, 3, 0, 9, 2, 16, 5, 11], dtype=torch.int32)
    ti2 = ti.clone()
    ti2[4, 3] = V + 5
    ti2[9, 0] = -3
    rl, grad = D.div_topk("fkl", logits.to(DEV), tv.to(DEV), ti2.to(torch.int32).to(DEV), t_cnt=cnt.to(DEV))
    rl, grad = rl.cpu(), grad.cpu()
    for r in range(R):
        keep = [k for k in range(int(cnt[r])) if 0 <= int(ti2[r, k]) < V]
        if not keep:
            assert rl[r] == 0 and torch.count_nonzero(grad[r]) == 0
            continue
        z = logits[r:r + 1].double()
        t = O.teacher_logprobs_topk(tv[r:r + 1, keep], 1.0, torch.float64)
        ref = O.fwd_kl_topk_rows(z, t, ti2[r:r + 1, keep])
        np.testing.assert_allclose(rl[r].item(), ref.item(), rtol=2e-5, atol=2e-6)


def test_forward_only_and_bit_reproducible(D):
    logits, tv, ti = _case(64, 32000, 200, torch.bfloat16, 10)
    a = D.div_topk("fkl", logits.to(DEV), tv.to(DEV), ti.to(DEV), want_grad=False)
    assert a[1] is None
    b = D.div_topk("fkl", logits.to(DEV), tv.to(DEV), ti.to(DEV))
    c = D.div_topk("fkl", logits.to(DEV), tv.to(DEV), ti.to(DEV))
    assert torch.equal(a[0], b[0]) and torch.equal(b[0], c[0]) and torch.equal(b[1], c[1])
    assert torch.equal(D.reduce_sum(b[0]), D.reduce_sum(c[0]))


def test_errors_are_python_exceptions(D):
    logits, tv, ti = _case(4, 512, 8, torch.float32, 11)
    with pytest.raises(RuntimeError):
        D.div_topk("fkl", logits, tv, ti)                         # CPU tensors: no fallback
    with pytest.raises(RuntimeError):
        D.div_topk("fkl", logits.to(DEV), tv.to(DEV), ti.to(DEV)[:, :4])
    big = torch.zeros(2, 4096, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="exceeds"):
        D.div_topk("fkl", torch.zeros(2, 8192, device=DEV), big, torch.zeros(2, 4096, dtype=torch.int32, device=DEV))
    with pytest.raises(ValueError):
        D.div_topk("jsd", logits.to(DEV), tv.to(DEV), ti.to(DEV))


@pytest.mark.parametrize("parts", [1, 2, 4])
def test_split_row_parts_agree_and_give_up_path(D, parts):
    """A 128256-wide row is cut into column parts that exchange statistics through the workspace.
    Every setting must give the oracle's numbers, also when no part waits for its partners
    (the no-wait flag: every part that finds a record missing leaves and is finished by the second
    launch), and the same bits as with waiting.  The hooks travel with the call: the library keeps
    no state."""
    logits, tv, ti = _case(40, 128256, 200, torch.bfloat16, 12, std=3.0)
    valid = torch.ones(40, dtype=torch.bool)
    valid[[0, 7, 33]] = False
    _check(D, "fkl", logits, tv[:37], ti[:37], T=1.0, valid=valid, hooks={"parts": parts})
    waited = _check(D, "fkl", logits, tv[:37], ti[:37], T=2.0, valid=valid, hooks={"parts": parts})
    retried = _check(D, "fkl", logits, tv[:37], ti[:37], T=2.0, valid=valid, hooks={"parts": parts, "no_wait": True})
    assert torch.equal(waited, retried)
    with pytest.raises(ValueError):
        D.div_topk("fkl", logits[:2].to(DEV), tv[:2].to(DEV), ti[:2].to(DEV), parts=3)


@pytest.mark.parametrize("kind,V,dtype", [("fkl", 128256, torch.bfloat16), ("fkl", 32000, torch.bfloat16), ("fkl", 152064, torch.float16),
                                          ("fkl", 1001, torch.float32), ("rkl", 32000, torch.bfloat16)])
def test_gradient_may_overwrite_the_logits(D, kind, V, dtype):
    """grad == logits (same buffer): every kernel holds, or has consumed, what it still needs of a
    row before it writes there, and a split part that gives up leaves its columns untouched for the
    retry launch; results are the bits of the out-of-place call."""
    logits, tv, ti = _case(24, V, 64, dtype, 31)
    x = logits.to(DEV)
    rl, g = D.div_topk(kind, x, tv.to(DEV), ti.to(DEV), T=1.5)
    for no_wait in (False, True):
        y = x.clone()
        rl2, g2 = D.div_topk(kind, y, tv.to(DEV), ti.to(DEV), T=1.5, grad_out=y, no_wait=no_wait)
        assert g2.data_ptr() == y.data_ptr() and torch.equal(rl, rl2) and torch.equal(g, y)



@pytest.mark.parametrize("V,dtype", [(152064, torch.bfloat16), (128256, torch.float32), (262144, torch.float16),
                                     (100000, torch.float32), (98304, torch.float32), (229376, torch.bfloat16),
                                     (100352, torch.bfloat16), (114688, torch.float16), (200064, torch.bfloat16),
                                     (50304, torch.float32), (57344, torch.float32)])
def test_rows_cut_into_five_to_eight_parts(D, V, dtype):
    """Vocabularies beyond 131072 two-byte (65536 four-byte) entries are cut into 5..8 parts of 4096
    chunks, or (four-byte rows of 6 parts and more, two-byte rows of 8) into 3..4 parts of 8192; two-byte rows that do
    not fill their parts -- and four-byte rows of up to five -- into parts of 13 to 15 chunks per thread (100352
    two-byte columns: 4 x 256 x 13, 114688: 4 x 14, 152064: 5 x 15, 200064: 7 x 14; 50304 four-byte columns: 4 x 13); with and without waiting for the partners the oracle's numbers and the same bits."""
    logits, tv, ti = _case(10, V, 48, dtype, 41, std=3.0)
    valid = torch.ones(10, dtype=torch.bool)
    valid[4] = False
    waited = _check(D, "fkl", logits, tv[:9], ti[:9], T=1.3, valid=valid)
    retried = _check(D, "fkl", logits, tv[:9], ti[:9], T=1.3, valid=valid, hooks={"no_wait": True})
    assert torch.equal(waited, retried)


@pytest.mark.parametrize("V,dtype", [(40000, torch.float32), (70000, torch.bfloat16), (98304, torch.float16), (98312, torch.bfloat16)])
def test_rows_cut_into_three_parts(D, V, dtype):
    """Rows of 8193-12288 chunks fill three parts of 4096 chunks, not four: no part may be left
    without columns."""
    logits, tv, ti = _case(11, V, 48, dtype, 43, std=3.0)
    waited = _check(D, "fkl", logits, tv, ti, T=1.1)
    retried = _check(D, "fkl", logits, tv, ti, T=1.1, hooks={"no_wait": True})
    forced = _check(D, "fkl", logits, tv, ti, T=1.1, hooks={"parts": 4})      # not honoured here: same launch, same bits
    assert torch.equal(waited, retried) and torch.equal(waited, forced)
    _check(D, "fkl", logits, tv, ti, T=1.1, hooks={"parts": 2})
    _check(D, "fkl", logits, tv, ti, T=1.1, hooks={"parts": 1})


@pytest.mark.parametrize("V,dtype,K", [(128256, torch.bfloat16, 200), (32000, torch.bfloat16, 400), (32000, torch.float32, 300),
                                       (8200, torch.float16, 64), (40000, torch.float32, 700), (131072, torch.float16, 32)])
def test_rows_cut_into_parts_of_1024_chunks(D, V, dtype, K):
    """The finer cut (up to 16 parts of 256 threads x 4 chunks per row): the oracle's numbers, with
    repeated ids, masked rows, waiting or not."""
    logits, tv, ti = _case(21, V, K, dtype, 47, std=3.0)
    ti[3, 5] = ti[3, 9]
    ti[6, :] = ti[6, 0]
    valid = torch.ones(21, dtype=torch.bool)
    valid[[2, 20]] = False
    waited = _check(D, "fkl", logits, tv[:19], ti[:19], T=1.2, valid=valid, hooks={"parts": 16})
    retried = _check(D, "fkl", logits, tv[:19], ti[:19], T=1.2, valid=valid, hooks={"parts": 16, "no_wait": True})
    assert torch.equal(waited, retried)


def test_a_column_part_that_holds_only_minus_infinity(D):
    """A masked stretch of the vocabulary (-inf logits) as wide as a whole column part: that part has
    no finite maximum; its columns get zero gradient and the row's statistics come from the others."""
    g = torch.Generator().manual_seed(44)
    R, V, K = 9, 128256, 64
    logits = torch.randn(R, V, generator=g) * 3
    logits[:5, 65536:98304] = float("-inf")                   # part 2 of 4, whole
    logits[5:, 120000:] = float("-inf")                       # the tail of the last part
    logits = logits.to(torch.bfloat16)
    tl = torch.log_softmax(logits.float() + torch.randn(R, V, generator=g), -1)
    tv, ti = torch.topk(tl, K)
    grad = _check(D, "fkl", logits, tv.to(torch.float16), ti.to(torch.int32), T=1.0)
    assert torch.count_nonzero(grad[:5, 65536:98304]) == 0 and torch.isfinite(grad.float()).all()
    _check(D, "fkl", logits, tv.to(torch.float16), ti.to(torch.int32), T=1.0, hooks={"no_wait": True})


@pytest.mark.parametrize("kind", ["fkl", "rkl"])
@pytest.mark.parametrize("V,K", [(4096, 24), (128256, 300), (32000, 900)])
def test_entries_of_zero_mass_are_no_entries(D, kind, V, K):
    """A stored log-prob of -inf (a teacher that masks part of its vocabulary) carries no mass: the
    entry counts neither for the loss nor for the support, exactly as if it were not there."""
    logits, tv, ti = _case(7, V, K, torch.bfloat16, 51)
    tv = tv.float()
    dead = torch.zeros(7, K, dtype=torch.bool)
    dead[:, 3::4] = True
    dead[5, 1:] = True                                        # one live entry
    tv_dead = tv.masked_fill(dead, float("-inf"))
    rl, g = D.div_topk(kind, logits.to(DEV), tv_dead.to(DEV), ti.to(DEV), T=1.2)
    # the same rows with the dead entries pointed outside the vocabulary (ignored by contract)
    ti_out = ti.masked_fill(dead, -1)
    rl2, g2 = D.div_topk(kind, logits.to(DEV), tv.to(DEV), ti_out.to(DEV), T=1.2)
    assert torch.isfinite(rl).all() and torch.equal(rl, rl2) and torch.equal(g, g2)


def test_repeated_ids_on_wide_four_byte_rows(D):
    # 16 chunks of fp32 per thread: the shapes that write their corrections behind the dense stores
    g = torch.Generator().manual_seed(78)
    R, V, K = 5, 32000, 96
    logits = torch.randn(R, V, generator=g) * 2
    ti = torch.randint(0, 40, (R, K), generator=g) * 797 + 5
    tv = torch.randn(R, K, generator=g)
    a = _check(D, "fkl", logits, tv, ti.to(torch.int32), T=0.9)
    b = _check(D, "fkl", logits, tv, ti.to(torch.int32), T=0.9)
    assert torch.equal(a, b)
    wide = torch.randn(3, 60000, generator=g) * 2                  # cut into 4 parts
    ti = torch.randint(0, 30, (3, K), generator=g) * 1999 + 11
    _check(D, "fkl", wide, tv[:3], ti.to(torch.int32), T=1.0)


@pytest.mark.parametrize("kind", ["fkl", "rkl"])
def test_rows_whose_ids_all_repeat(D, kind):
    """Every entry of a row on one id, on two ids of one 16-byte chunk, on a handful of ids: the
    masses add per id (the thread that holds the chunk sums them from its list), the result is the
    oracle's and the same bits on every run."""
    g = torch.Generator().manual_seed(77)
    R, V, K = 6, 4096, 512
    logits = (torch.randn(R, V, generator=g) * 2).to(torch.bfloat16)
    ti = torch.empty(R, K, dtype=torch.int64)
    ti[0] = 1234
    ti[1] = torch.where(torch.arange(K) % 2 == 0, 801, 806)
    ti[2] = torch.randint(0, 5, (K,), generator=g) * 1000 + 3
    ti[3] = torch.randint(0, V, (K,), generator=g)
    ti[4] = torch.arange(K) % 16 + 64
    ti[5] = V - 1
    if kind == "rkl":
        # on a single id the reverse-KL gradient is an exact zero made of 512 cancelling terms: nothing
        # for a relative tolerance to hold on to; two ids instead
        ti[0] = torch.where(torch.arange(K) % 3 == 0, 1234, 77)
        ti[5] = torch.where(torch.arange(K) % 5 == 0, V - 1, 0)
    tv = torch.randn(R, K, generator=g)
    a = _check(D, kind, logits, tv, ti.to(torch.int32), T=1.2)
    b = _check(D, kind, logits, tv, ti.to(torch.int32), T=1.2)
    assert torch.equal(a, b)

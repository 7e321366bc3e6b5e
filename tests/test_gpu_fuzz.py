"""Seeded random shapes and contents through every kernel family (through the C ABI), each case against the
CPU oracle with the entry-by-entry gradient bounds of the oracle's helpers.  The generators are fixed-seed, so a
run is reproducible; a failure names its case.  What the draws are chosen to reach:

  * sparse-teacher kernels: one workgroup per row, rows cut into 2 / 3 / 4 / 5-8 / 16 column parts, rows off the
    16-byte grid (odd vocabularies), the streaming kernel, parts that do not wait for their partners (the
    second launch finishes them), ids that repeat and crowd a few chunks, masked rows;
  * dense kernels: the three divergences, mixed dtypes, offsets that move the maxima, zero-mass teacher columns;
  * fused marginal + reverse KL: the planned (full-width and compact) and the atomic accumulation, and all three ways a row is finished --
    from the values kept between the passes, put back and redone on its maxima (sums that leave the range: teachers
    scaled by 1e+-30; a student whose largest logits sit off the support), and without a gradient;
  * weighted merge + remap: ids bit-exact; the bucketed multi-teacher loss with maps that crowd every entry of a row
    into one column part (buckets overflow into the row's spill area) or onto a handful of student ids;
  * the producer: ties, plateaus, constant rows, -inf halves, crops of wider rows; ids bit-exact;
  * the composite: repeated ids, sliced logits, labels off the support."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = {torch.float32: 1e-4, torch.bfloat16: 2e-3, torch.float16: 2e-3}
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


@pytest.fixture(scope="module")
def D():
    import llm_distillery_amd as d
    d._lib.load()
    return d


def _row_map(valid):
    rm = torch.full((valid.numel(),), -1, dtype=torch.int32)
    rm[valid] = torch.arange(int(valid.sum()), dtype=torch.int32)
    return rm


def _worst(err, bound):
    ratio = err / bound
    i = int(ratio.argmax())
    r, c = divmod(i, err.shape[-1])
    return f"worst ratio {ratio.flatten()[i].item():.2f} at row {r} column {c}: error {err[r, c].item():.3e}, bound {bound[r, c].item():.3e}"


def test_sparse_teacher_divergences(D):
    rng = np.random.default_rng(2024)
    widths = [512, 4096, 8192, 16384, 32000, 32768, 50264, 65536, 100000, 128256, 152064, 200064, 9, 1001, 4099, 32003, 50257,
              130001, 262144, 229376, 40000, 70000, 98304]
    for case in range(220):
        V = int(rng.choice(widths))
        dtype = DTYPES[int(rng.integers(0, 3))]
        K = int(min(V, rng.choice([1, 7, 16, 64, 200, 257, 600, 1000])))
        R = int(rng.integers(1, 7))
        kind = "fkl" if rng.random() < 0.75 else "rkl"
        span = int(min(V, rng.choice([V, max(8, V // 1000), 64, 8])))         # a small span: many repeats, entries crowd a few chunks
        base = int(rng.integers(0, V - span + 1))
        ti = torch.tensor(rng.integers(base, base + span, (R, K)), dtype=torch.int32)
        if rng.random() < 0.3:
            ti[:, 0] = V - 1
        g = torch.Generator().manual_seed(int(rng.integers(0, 2 ** 31)))
        logits = (torch.randn(R, V, generator=g) * 2.5).to(dtype)
        tv = torch.randn(R, K, generator=g) * 2
        T = float(rng.choice([1.0, 0.7, 2.0]))
        valid = torch.ones(R, dtype=torch.bool)
        if rng.random() < 0.4 and R > 1:
            valid = torch.tensor(rng.random(R) < 0.7)
            valid[0] = True
        nv = int(valid.sum())
        hooks = {"no_wait": bool(rng.random() < 0.3), "parts": int(rng.choice([0, 0, 1, 2, 4, 16]))} if kind == "fkl" else {}
        what = f"case {case}: {kind} V={V} {dtype} K={K} R={R} span={span} T={T} valid={nv} {hooks}"
        _, rows64, grad64 = O.mean_loss_and_grad(kind, logits, T, t_vals=tv[:nv], t_idx=ti[:nv], valid=valid, dtype=torch.float64)
        rl, grad = D.div_topk(kind, logits.to(DEV), tv[:nv].to(DEV), ti[:nv].to(DEV), row_map=_row_map(valid).to(DEV), T=T,
                              grad_scale=1.0 / nv, **hooks)
        rl, grad = rl.cpu(), grad.cpu()
        assert torch.count_nonzero(rl[~valid]) == 0 and torch.count_nonzero(grad[~valid]) == 0, what
        np.testing.assert_allclose(rl[valid].double().numpy(), rows64.numpy(), rtol=2e-5, atol=2e-6, err_msg=what)
        err = (grad.double() - grad64).abs()
        bound = O.topk_gradient_tolerance(kind, grad64, logits, tv[:nv], ti[:nv], T, None, 1.0 / nv, dtype, RTOL[dtype], valid)
        assert (err <= bound).all(), f"{what}: {_worst(err, bound)}"


def test_dense_teacher_divergences(D):
    rng = np.random.default_rng(1)
    for case in range(200):
        kind = ["fkl", "rkl", "jsd"][int(rng.integers(0, 3))]
        V = int(rng.choice([8, 1000, 2048, 8192, 32000, 50264, 65536, 50257, 32003, 100000]))
        R = int(rng.integers(1, 9))
        dtype = DTYPES[int(rng.integers(0, 3))]
        t_dtype = dtype if rng.random() < 0.7 else torch.float32
        T = float(rng.choice([0.5, 1.0, 2.0]))
        tT = float(rng.choice([T, T, 1.0]))
        std = float(rng.choice([0.5, 2, 6, 15]))
        off = float(rng.choice([0, 0, -30, 30, -200]))
        g = torch.Generator().manual_seed(case)
        s = torch.randn(R, V, generator=g) * std + off
        t = s * 0.8 + torch.randn(R, V, generator=g) * float(rng.choice([0.3, 1.5, 5])) + float(rng.choice([0, -50, 50]))
        if rng.random() < 0.3:
            t[:, torch.randperm(V, generator=g)[: V // 3]] = -float("inf")       # a teacher without mass on a third of the columns
        s, t = s.clamp(-6e4, 6e4).to(dtype), t.clamp(max=6e4).to(t_dtype)
        what = f"case {case}: {kind} V={V} R={R} {dtype} {t_dtype} T={T} teacher T={tT} std={std} offset={off}"
        _, rows64, grad64 = O.mean_loss_and_grad(kind, s, T, t_logits=t, t_T=tT, dtype=torch.float64)
        if not torch.isfinite(rows64).all():
            continue
        rl, grad = D.div_dense(kind, s.to(DEV), t.to(DEV), T=T, teacher_T=tT, grad_scale=1.0 / R)
        np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=5e-5, atol=1e-5, err_msg=what)
        err = (grad.cpu().double() - grad64).abs()
        bound = O.dense_gradient_tolerance(grad64, s, t, rows64, T, tT, 1.0 / R, dtype, RTOL[dtype], kind=kind)
        assert (err <= bound).all(), f"{what}: {_worst(err, bound)}"


def test_fused_marginal_reverse_kl(D):
    from llm_distillery_amd import synthetic as S
    rng = np.random.default_rng(0)
    maps = {}
    for case in range(200):
        Vs = int(rng.choice([1000, 2048, 8192, 32000]))
        Vt = int(Vs * rng.choice([2, 3, 5])) + int(rng.integers(0, 9))
        alphabet = int(rng.choice([4, 16, 256]))
        R = int(rng.integers(1, 7))
        dtype = DTYPES[int(rng.integers(0, 3))]
        T = float(rng.choice([0.5, 0.7, 1.0, 1.5, 2.0]))
        tT = float(rng.choice([T, T, 1.0, 0.25, 3.0]))
        planned = (False, "full", "auto")[int(rng.integers(0, 3))]
        vocab_seed = int(rng.integers(0, 6))                      # a handful of tokenizer pairs, built once each
        key = (Vs, Vt, alphabet, vocab_seed)
        if key not in maps:
            student = S.random_byte_vocab(Vs, vocab_seed, alphabet=alphabet, max_len=6, all_single_bytes=(alphabet == 256))
            teacher = S.random_byte_vocab(Vt, vocab_seed + 1, alphabet=alphabet, max_len=8)
            t2s = D.vocab_utils.longest_prefix_map(student, teacher).copy()
            t2s[np.random.default_rng(vocab_seed).random(Vt) < 0.02] = -1
            maps[key] = (t2s, {"full": D.vocab_utils.MarginalPlan(t2s, Vs, DEV, compact=False),
                               "auto": D.vocab_utils.MarginalPlan(t2s, Vs, DEV)}, torch.tensor(t2s, device=DEV))
        t2s, plans, t2s_dev = maps[key]
        g = torch.Generator().manual_seed(case)
        probs = torch.softmax(torch.randn(R, Vt, generator=g) * float(rng.choice([1, 3, 8])), -1)
        # unnormalised teachers: the sums of such rows leave the range the optimistic pass covers
        scale = torch.tensor(np.where(rng.random(R) < 0.4, 10.0 ** rng.uniform(-30, 30, R), 1.0), dtype=torch.float32)
        probs = probs * scale.unsqueeze(-1)
        logits = torch.randn(R, Vs, generator=g) * float(rng.choice([1, 3, 10])) + float(rng.choice([0, -40, 40]))
        marg = torch.tensor(O.marginalise_map(probs.double().numpy(), t2s, Vs))
        if rng.random() < 0.3:
            # the student's largest logits on columns without teacher mass: the support lies far below the row's maximum
            dead = torch.nonzero(marg.sum(0) == 0).squeeze(-1)
            if dead.numel() >= 2:
                logits[:, dead[:2]] += float(rng.choice([10, 25, 60]))
        logits = logits.to(dtype)
        what = f"case {case}: Vs={Vs} Vt={Vt} alphabet={alphabet} R={R} {dtype} T={T} teacher T={tT} planned={planned}"
        tmap = plans[planned] if planned else t2s_dev
        rl, grad = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, T=T, teacher_T=tT, grad_scale=1.0 / R)
        rl0, _ = D.vocab_utils.rkl_marginalised(logits.to(DEV), probs.to(DEV), tmap, T=T, teacher_T=tT, want_grad=False)
        with np.errstate(divide="ignore"):
            t_logits = O.marginal_to_teacher_logits(marg)
        _, rows64, grad64 = O.mean_loss_and_grad("rkl", logits, T, t_logits=t_logits, t_T=tT, dtype=torch.float64)
        if not torch.isfinite(rows64).all():
            continue
        np.testing.assert_allclose(rl.cpu().double().numpy(), rows64.numpy(), rtol=5e-5, atol=1e-5, err_msg=what)
        np.testing.assert_allclose(rl0.cpu().numpy(), rl.cpu().numpy(), rtol=2e-5, atol=1e-5, err_msg=what + " (no gradient)")
        err = (grad.cpu().double() - grad64).abs()
        bound = O.marginal_rkl_gradient_tolerance(grad64, logits, t_logits, rows64, T, tT, 1.0 / R, dtype, RTOL[dtype])
        assert (err <= bound).all(), f"{what}: {_worst(err, bound)}"


def _teachers(N, K, Vt, n, g, rng, idx_dtype=torch.int32, val_dtype=torch.float16, one_id=0.0):
    vals, idxs = [], []
    for _ in range(n):
        v, i = torch.topk(torch.log_softmax(torch.randn(N, Vt, generator=g) * float(rng.choice([1, 3])), -1), K)
        if rng.random() < one_id:
            i[:, :] = i[:, :1]                                     # every entry of a row names one id
        vals.append(v.to(val_dtype))
        idxs.append(i.to(idx_dtype))
    return vals, idxs


def test_weighted_merge_and_remap(D):
    rng = np.random.default_rng(4)
    for case in range(200):
        n = int(rng.integers(1, 9))
        K = int(rng.choice([1, 4, 33, 64, 100, 200, 256]))
        if n * K > 2048:
            K = 2048 // n
        Vt = int(rng.choice([64, 3000, 32000, 152064]))
        K = min(K, Vt)
        Vs = int(rng.choice([Vt, max(8, Vt // 3), Vt + 500]))
        N = int(rng.integers(1, 8))
        idt = torch.int32 if rng.random() < 0.6 else torch.int64
        vdt = [torch.float16, torch.float32, torch.bfloat16][int(rng.integers(0, 3))]
        g = torch.Generator().manual_seed(case)
        vals, idxs = _teachers(N, K, Vt, n, g, rng, idt, vdt, one_id=0.3)
        mode = str(rng.choice(["none", "random", "crowded", "identity"]))
        id_map = None
        if mode == "random":
            id_map = rng.integers(0, Vs, Vt).astype(np.int32)
        if mode == "crowded":
            id_map = rng.integers(0, min(Vs, 7), Vt).astype(np.int32)
        if mode == "identity":
            id_map = np.minimum(np.arange(Vt), Vs - 1).astype(np.int32)
        if id_map is not None:
            id_map[rng.random(Vt) < 0.1] = -1
        else:
            Vs = max(Vs, Vt)
        w = list(rng.random(n) + 0.01)
        if rng.random() < 0.2:
            w[int(rng.integers(0, n))] = 0.0
        what = f"case {case}: n={n} K={K} Vt={Vt} Vs={Vs} N={N} {idt} {vdt} map={mode}"
        ids, lm, cnt = D.merge_remap_topk([v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], w,
                                          torch.tensor(id_map, device=DEV) if id_map is not None else None, student_vocab=Vs)
        ref = O.merge_remap_rows([v.float().numpy() for v in vals], [i.numpy() for i in idxs], w, id_map)
        ids, lm, cnt = ids.cpu().numpy(), lm.cpu().numpy(), cnt.cpu().numpy()
        for r, (rid, rmass, _) in enumerate(ref):
            keep = rmass > 0                                       # an entry of zero mass (a teacher of weight 0) may be listed or not
            assert cnt[r] in (rid.size, int(keep.sum())), f"{what}: row {r} count {cnt[r]}"
            want, mass = (rid, rmass) if cnt[r] == rid.size else (rid[keep], rmass[keep])
            assert np.array_equal(ids[r, :cnt[r]], want), f"{what}: row {r} ids"
            assert (ids[r, cnt[r]:] == -1).all() and np.isneginf(lm[r, cnt[r]:]).all(), f"{what}: row {r} padding"
            np.testing.assert_allclose(np.exp(lm[r, :cnt[r]].astype(np.float64)), mass, rtol=4e-6, atol=1e-30, err_msg=what)


def test_bucketed_multi_teacher_loss(D):
    rng = np.random.default_rng(77)
    for case in range(200):
        dtype = DTYPES[int(rng.integers(0, 3))]
        V = int(rng.choice([2048, 8192, 16000, 32000, 40000, 65536, 100000, 128256, 152064, 200000 if dtype != torch.float32 else 120000]))
        n = int(rng.integers(1, 9))
        K = int(rng.choice([4, 33, 64, 100, 200, 256]))
        while n * K > 2048:
            n -= 1
        Vt = int(rng.choice([V, V + 5000, max(K + 1, V // 3)]))
        R = int(rng.integers(1, 8))
        T = float(rng.choice([1.0, 0.7, 2.0]))
        g = torch.Generator().manual_seed(int(rng.integers(0, 2 ** 31)))
        logits = (torch.randn(R, V, generator=g) * 3).to(dtype)
        valid = torch.ones(R, dtype=torch.bool)
        if R > 2 and rng.random() < 0.5:
            valid[int(rng.integers(1, R))] = False
        nv = int(valid.sum())
        vals, idxs = _teachers(nv, K, Vt, n, g, rng)
        weights = list(rng.random(n) + 0.05)
        if n > 1 and rng.random() < 0.2:
            weights[1] = 0.0
        mode = str(rng.choice(["random", "crowded", "identity", "few"]))
        if mode == "identity" and Vt <= V:
            id_map = None
        else:
            if mode == "crowded":          # every id of the map inside one column part: that part's bucket overflows
                lo = int(rng.integers(0, max(1, V - 3000)))
                id_map = torch.randint(lo, min(V, lo + 3000), (Vt,), generator=g, dtype=torch.int32)
            elif mode == "few":            # many teacher ids share a handful of student ids
                id_map = torch.randint(0, 11, (Vt,), generator=g, dtype=torch.int32) * (V // 11)
            else:
                id_map = torch.randint(0, V, (Vt,), generator=g, dtype=torch.int32)
            id_map[torch.rand(Vt, generator=g) < float(rng.choice([0.0, 0.05, 0.5]))] = -1
        what = f"case {case}: V={V} {dtype} n={n} K={K} Vt={Vt} R={R} T={T} map={mode}"
        args = (logits.to(DEV), [v.to(DEV) for v in vals], [i.to(DEV) for i in idxs], weights, None if id_map is None else id_map.to(DEV))
        # the bucketed form wherever the library takes it (wider four-byte rows go through the sorting form)
        bucketed = True if V <= (131072 if dtype == torch.float32 else 262144) else None
        kw = dict(row_map=_row_map(valid).to(DEV), T=T, teacher_T=1.0, grad_scale=1.0 / nv, fused=bucketed)
        rl, grad = D.fkl_multi_teacher(*args, **kw)
        ids, lq, cnt = O.merge_remap_padded([v.float().numpy() for v in vals], [i.numpy() for i in idxs], weights,
                                            None if id_map is None else id_map.numpy(), 1.0, n_student=V)
        sel = torch.nonzero(valid).squeeze(-1)
        z = (logits[sel].double() / T).requires_grad_(True)
        rows64 = O.fwd_kl_sparse_rows(z, ids, lq.astype(np.float64), cnt)
        rows64.sum().backward()
        grad64 = torch.zeros(R, V, dtype=torch.float64)
        grad64[sel] = z.grad / (T * nv)
        np.testing.assert_allclose(rl.cpu()[valid].double().numpy(), rows64.detach().numpy(), rtol=3e-5, atol=3e-6, err_msg=what)
        assert torch.count_nonzero(rl.cpu()[~valid]) == 0 and torch.count_nonzero(grad.cpu()[~valid]) == 0, what
        err = (grad.cpu().double() - grad64).abs()
        bound = O.storage_tolerance(grad64, dtype, RTOL[dtype])
        bound[sel] = O.sparse_gradient_tolerance(grad64[sel], logits[sel], T, torch.as_tensor(ids).long(), dtype, RTOL[dtype])
        assert (err <= bound).all(), f"{what}: {_worst(err, bound)}"
        rl2, grad2 = D.fkl_multi_teacher(*args, **kw, no_wait=True)
        assert torch.equal(rl, rl2) and torch.equal(grad, grad2), what + " (parts that do not wait)"


def test_teacher_producer(D):
    rng = np.random.default_rng(2)
    for case in range(200):
        V = int(rng.choice([17, 255, 1000, 2048, 4099, 32000, 50257, 65536, 128256, 151936, 200003]))
        K = int(min(V, rng.choice([1, 4, 33, 64, 200, 256, 257, 400, 1000])))
        R = int(rng.integers(1, 6))
        dtype = DTYPES[int(rng.integers(0, 3))]
        std = float(rng.choice([0.01, 1, 3, 10]))
        off = float(rng.choice([0, 0, -20, 20, -300]))
        mode = str(rng.choice(["randn", "quant", "const", "plateau"]))
        g = torch.Generator().manual_seed(case)
        x = torch.randn(R, V, generator=g) * std + off
        if mode == "quant":
            x = (x * 2).round() / 2
        if mode == "const":
            x[:] = off
        if mode == "plateau":
            x[:, torch.randperm(V, generator=g)[:int(rng.integers(1, V + 1))]] = off + 3 * std
        if rng.random() < 0.2:
            x[:, torch.randperm(V, generator=g)[: V // 2]] = -float("inf")
        x = x.clamp(max=6e4).to(dtype)
        x = torch.where(x == 0, torch.zeros_like(x), x)             # -0.0 -> +0.0: the kernel orders the two by their bits
        Vm = V + int(rng.choice([0, 0, 3, 64]))
        full = torch.full((R, Vm), 7.0, dtype=dtype)
        full[:, :V] = x
        what = f"case {case}: V={V} of {Vm} K={K} R={R} {dtype} {mode} std={std} offset={off}"
        parts = -(-V // (16384 if dtype == torch.float32 else 32768))
        if K > 1024 or K * parts > 4096 or V > (131072 if dtype == torch.float32 else 262144):
            with pytest.raises(RuntimeError, match="exceeds"):    # the stated limits of dl_teacher_topk
                D.teacher_topk(full.to(DEV), K, crop_to_size=V, val_dtype=torch.float32, idx_dtype=torch.int64)
            continue
        val, idx = D.teacher_topk(full.to(DEV), K, crop_to_size=V, val_dtype=torch.float32, idx_dtype=torch.int64)
        # classes/teacher/inference_worker.py:73-77: log-softmax over the cropped vocabulary, then the K largest;
        # ties towards the smaller id (a stable sort)
        logp = torch.log_softmax(x.double(), dim=-1)
        order = torch.sort(x.float(), dim=-1, descending=True, stable=True).indices[..., :K]
        rv = torch.gather(logp, -1, order)
        assert torch.equal(idx.cpu(), order), what
        finite = torch.isfinite(x.float())
        scale = max(1.0, float(rv[torch.isfinite(rv)].abs().max()) if torch.isfinite(rv).any() else 1.0,
                    float(x.float()[finite].abs().max()) if finite.any() else 1.0)
        np.testing.assert_allclose(val.cpu().double().numpy(), rv.numpy(), rtol=0, atol=3e-6 * scale, equal_nan=True, err_msg=what)


def test_composite_loss(D):
    rng = np.random.default_rng(7)
    for case in range(150):
        V = int(rng.choice([512, 4096, 32000, 32768, 65536, 128256, 152064, 7, 1001, 32003, 50257, 100003]))
        dtype = [torch.bfloat16, torch.float32, torch.float16][int(rng.integers(0, 3))]
        K = int(min(V, rng.choice([4, 16, 64, 200, 400])))
        N = int(rng.integers(3, 40))
        span = int(min(V, rng.choice([V, 64, 16])))
        base = int(rng.integers(0, V - span + 1))
        g = torch.Generator().manual_seed(int(rng.integers(0, 2 ** 31)))
        logits = (torch.randn(N, V, generator=g) * 2).to(dtype)
        if span == V:
            tv, ti = torch.topk(torch.log_softmax(logits.float() + torch.randn(N, V, generator=g), -1), K)
        else:
            ti = torch.tensor(rng.integers(base, base + span, (N, K)))
            tv = torch.log_softmax(torch.randn(N, K, generator=g), -1)
            if span + N + 6 < V:
                ti[:, 0] = (base + span + 5 + torch.arange(N)) % V
        labels = ti[:-1, 0].clone()
        miss = torch.tensor(rng.random(N - 1) < 0.3)
        labels[miss] = (labels[miss] + 1) % V
        avoid = torch.tensor(sorted(set(rng.integers(0, N - 1, int(rng.integers(0, 3))).tolist())), dtype=torch.long)
        alpha = float(rng.choice([2.0, 1.0, 0.5]))
        sliced = bool(rng.random() < 0.5)
        off = int(rng.integers(0, 9))
        what = f"case {case}: V={V} {dtype} K={K} N={N} span={span} alpha={alpha} sliced={sliced} at {off}"
        ref_in = logits.double().requires_grad_(True)
        ref = O.calculate_divergence(ref_in, tv.double(), ti, labels, alpha, avoid)
        if not torch.isfinite(ref["train_loss"]):
            continue
        ref["train_loss"].backward()
        if sliced:
            wide = torch.zeros(N, V + 11, dtype=dtype, device=DEV)
            wide[:, off:off + V] = logits.to(DEV)
            s = wide[:, off:off + V].detach().requires_grad_(True)
        else:
            s = logits.to(DEV).requires_grad_(True)
        res = D.calculate_divergence(s, tv.to(DEV), ti.to(DEV), labels.to(DEV), alpha, avoid.to(DEV))
        for k in D.LOSS_KEYS:
            np.testing.assert_allclose(res[k].item(), ref[k].item(), rtol=2e-5, atol=2e-6, err_msg=f"{what}: {k}")
        res["train_loss"].backward()
        err = (s.grad.cpu().double() - ref_in.grad).abs()
        bound = O.composite_gradient_tolerance(ref_in.grad, logits, 1.0, dtype, RTOL[dtype], None, ti)
        assert (err <= bound).all(), f"{what}: {_worst(err, bound)}"

"""Benchmark of the distillation-loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3]

One step = one pass of the fused loss + gradient over one batch of synthetic input followed by the
deterministic mean reduction.  The default workload is the one the headline metric is quoted on
(C3: 8 x 4096 tokens x 128256-vocabulary bf16 student logits, top-K=200 fp16/int32 teacher, T=1);
`--workload c1|c2|c4|c4-merge|c5|producer|composite|dropin|dropin-batch|copyshape` measures the other configurations and the teacher producer with the
same harness.  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E


# ---------------------------------------------------------------------------------------------
# workloads: build(device, rows) -> (step_fn, main_launch_fn, algorithmic_bytes, tokens, description, kernel)
# step_fn runs the whole step and returns the loss tensor; main_launch_fn launches only the dominant kernel.
# ---------------------------------------------------------------------------------------------
INPLACE = False        # --inplace: the gradient is written over the logits (C3 only; see main)
PARTS = 0              # --parts: column parts per row of the C3 loss kernel (0 = the library's choice)


NO_SPLIT = False       # --no-split: dense rows are not cut into column parts (dl_div_dense without a workspace)
VOCAB = 0              # --vocab / --pitch: C3 on logits[:, :vocab] of rows `pitch` columns wide (a crop of a padded vocabulary)
PITCH = 0


def _wl_c3(D, S, dev, rows):
    import torch
    rows = rows or 8 * 4096
    V, K = VOCAB or 128256, 200
    c = S.config3(dev, rows=rows, seed=3, V=V)
    if PITCH and PITCH != V:
        wide = torch.zeros((rows, PITCH), dtype=c["logits"].dtype, device=dev)
        wide[:, :V] = c["logits"]
        c["logits"] = wide[:, :V]
    if INPLACE:
        grad = c["logits"]
    elif PITCH and PITCH != V:
        grad = torch.empty((rows, PITCH), dtype=c["logits"].dtype, device=dev)[:, :V]
    else:
        grad = torch.empty_like(c["logits"])
    scale = 1.0 / rows
    if VOCAB or PITCH:
        def main_crop():
            return D.div_topk("fkl", c["logits"], c["t_val"], c["t_idx"], T=1.0, grad_scale=scale, grad_out=grad, parts=PARTS)[0]
        return (lambda: D.reduce_sum(main_crop(), scale), main_crop, rows * (V * 2 + V * 2 + K * 6), rows,
                f"forward-KL fwd+bwd, top-K={K} fp16/int32 teacher, {rows} tokens x {V} vocab bf16 logits in rows of "
                f"{PITCH or V} columns, T=1, bf16 gradient", "fkl_topk_reg_kernel<bf16,...>", c, grad)

    def main():
        return D.div_topk("fkl", c["logits"], c["t_val"], c["t_idx"], T=1.0, grad_scale=scale, grad_out=grad, parts=PARTS)[0]

    shape = {0: "256,16,split> (4 column parts per row)", 1: "1024,16> (one workgroup per row)", 2: "512,16,split> (2 column parts per row)",
             4: "256,16,split> (4 column parts per row)", 16: "256,4,split> (16 column parts per row)"}[PARTS]
    return (lambda: D.reduce_sum(main(), scale), main, rows * (V * 2 + V * 2 + K * 6), rows,
            f"C3 forward-KL fwd+bwd, top-K={K} fp16/int32 teacher, {rows} tokens x {V} vocab bf16 logits, T=1, "
            "bf16 gradient" + (" written over the logits" if INPLACE else ""),
            "fkl_topk_reg_kernel<bf16," + shape, c, grad)


def _wl_c4(D, S, dev, rows):
    """dl_fkl_multi_teacher: K-wide preparation (map, weigh, renormalise, bucket per column part) + the loss kernel."""
    import torch
    rows = rows or 4 * 8192
    V, Vt, K = 128256, 152064, 200
    c = S.config4(dev, rows=rows, V=V, Vt=Vt, K=K)
    grad = torch.empty_like(c["logits"])
    scale = 1.0 / rows

    def main():
        return D.fkl_multi_teacher(c["logits"], c["t_vals"], c["t_idxs"], c["weights"], c["id_map"], T=1.0, grad_scale=scale,
                                   grad_out=grad, fused=True)[0]

    return (lambda: D.reduce_sum(main(), scale), main, rows * (V * 2 + V * 2 + 3 * K * 6) + Vt * 4, rows,
            f"C4 3-teacher weighted merge + vocab remap ({Vt}->{V}) + forward-KL fwd+bwd, {rows} tokens, bf16",
            "fkl_topk_reg_kernel<bf16,256,16,split,bucketed teachers> (4 column parts per row) fed by multi_prep_kernel", c, grad)


def _wl_c4_merge(D, S, dev, rows):
    """The two-launch form of C4: sorted merge through memory (bit-exact id output), then the loss kernel."""
    import torch
    rows = rows or 4 * 8192
    V, Vt, K = 128256, 152064, 200
    c = S.config4(dev, rows=rows, V=V, Vt=Vt, K=K)
    grad = torch.empty_like(c["logits"])
    scale = 1.0 / rows
    state = {}

    def merge():
        state["m"] = D.merge_remap_topk(c["t_vals"], c["t_idxs"], c["weights"], c["id_map"], student_vocab=V)

    def main():
        ids, lm, cnt = state["m"]
        return D.div_topk("fkl", c["logits"], lm, ids, t_cnt=cnt, T=1.0, grad_scale=scale, grad_out=grad, unique_ids=True)[0]

    def step():
        merge()
        return D.reduce_sum(main(), scale)

    merge()
    return (step, main, rows * (V * 2 + V * 2 + 3 * K * 6) + Vt * 4, rows,
            f"C4 in two launches: merge_kernel (3 teachers, remap {Vt}->{V}) feeding the forward-KL kernel, {rows} tokens, bf16",
            "fkl_topk_reg_kernel<bf16,256,16,split> fed by merge_kernel", c, grad)


def _wl_dense(kind_name):
    def build(D, S, dev, rows):
        import torch
        if kind_name == "c1":
            c = S.config1(dev) if not rows else S.config1(dev, B=1, S=rows)
            eb, desc = 4, "C1 dense forward-KL fwd+bwd, fp32, T=1, last 10% of positions masked"
        else:
            c = S.config2(dev) if not rows else S.config2(dev, B=1, S=rows)
            eb, desc = 2, "C2 dense JSD fwd+bwd, bf16, T=2, ragged valid lengths"
        R, V = c["logits"].shape
        nv = int(c["valid"].sum())
        grad = torch.empty_like(c["logits"])
        scale = 1.0 / nv

        def main():
            return D.div_dense(c["kind"], c["logits"], c["t_logits"], row_map=c["row_map"], T=c["T"], grad_scale=scale,
                               grad_out=grad, split=not NO_SPLIT)[0]

        return (lambda: D.reduce_sum(main(), scale), main, nv * V * 2 * eb + R * V * eb, R,
                f"{desc}; {R} tokens ({nv} valid) x {V} vocab", f"dense_reg_kernel ({c['kind']})", c, grad)
    return build


ALPHABET = 256         # --alphabet: byte alphabet of C5's random vocabularies (256: nearly all teacher ids fall back to the
                       # 256 single-byte student tokens; 4-16: a flat map, thousands of student ids in use)
STUDENT_VOCAB = 0      # --student-vocab: C5's student vocabulary (default 32000)
UNFUSED = False        # --unfused: C5 as two launches, the marginal through memory


def _wl_c5(D, S, dev, rows):
    import torch
    rows = rows or 2 * 4096
    Vs, Vt = STUDENT_VOCAB or 32000, 152064
    c = S.config5(dev, rows=rows, Vs=Vs, Vt=Vt, alphabet=ALPHABET)
    grad = torch.empty_like(c["logits"])
    scale = 1.0 / rows
    plan = D.vocab_utils.MarginalPlan(c["t2s_host"], Vs, dev)       # built once per tokenizer pair
    used = int(torch.unique(c["t2s"][c["t2s"] >= 0]).numel())
    fused = not UNFUSED and plan.ent is not None
    what = (f"C5 byte-trie marginalisation ({Vt}->{Vs}, alphabet {ALPHABET}: {used} student ids in use) + reverse-KL fwd+bwd, "
            f"{rows} tokens, fp32 teacher softmax, bf16 student, T=1.5")

    if fused:
        def main():
            return D.vocab_utils.rkl_marginalised(c["logits"], c["t_probs"], plan, T=c["T"], grad_scale=scale,
                                                  grad_out=grad)[0]
        kernel = "rkl_marginalised_kernel<bf16> (planned marginal)"
    else:
        # the marginal's logarithm through memory (fp32 [rows, Vs]), then the dense reverse KL on it: what student
        # vocabularies beyond the fused kernel's 36864 ids take
        def main():
            lm = D.vocab_utils.marginalise(c["t_probs"], plan=plan if plan.ent is not None else None, t2s=c["t2s"],
                                           n_student=Vs, log=True)
            return D.div_dense("rkl", c["logits"], lm, T=c["T"], grad_scale=scale, grad_out=grad)[0]
        kernel = "marginalise_map_kernel + dense reverse-KL kernel (the marginal through memory)"
        what += "; in two launches"

    return (lambda: D.reduce_sum(main(), scale), main, rows * (Vt * 4 + Vs * 2 + Vs * 2) + Vt * 4, rows, what, kernel, c, grad)


def _wl_producer(D, S, dev, rows):
    import torch
    rows = rows or 8 * 4096
    V, K = 128256, 200
    c = S.config3(dev, rows=rows, seed=3)
    out = {}

    def main():
        out["v"], out["i"] = D.teacher_topk(c["logits"], K)
        return out["v"]

    def step():
        return main()[0, 0].float()

    return (step, main, rows * (V * 2 + K * 6), rows,
            f"teacher producer: log-softmax over {V} + top-{K}, {rows} rows bf16 -> fp16/int32", "topk_part_kernel<bf16> (4 column parts per row) + topk_merge_kernel",
            c, torch.empty_like(c["logits"]))


def _composite_batch(torch, S, dev, B, seq, V, K, seed=7):
    """A batch as the reference's training loop sees it: [B, seq, V] bf16 logits, per conversation two
    content ranges, stored fp16 / int32 teacher rows with distinct ids, labels mostly among the ids."""
    c = S.config3(dev, rows=B * seq, seed=seed)
    logits = c["logits"].view(B, seq, V)
    convos = []
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    a, b = seq // 16, seq // 2
    for i in range(B):
        rows = torch.cat([torch.arange(a, b - a, device=dev), torch.arange(b, seq - 1, device=dev)])
        ti = c["t_idx"].view(B, seq, K)[i][rows]
        tv = c["t_val"].view(B, seq, K)[i][rows]
        labels = ti[:-1, 1].long()
        avoid = torch.tensor([b - 2 * a - 1], dtype=torch.long, device=dev)
        convos.append((rows, tv, ti, labels, avoid))
    return logits, convos


def _wl_composite(D, S, dev, rows):
    import torch
    B, seq, V, K, T, alpha = 8, (rows // 8) if rows else 4096, 128256, 200, 1.0, 2.0
    logits, convos = _composite_batch(torch, S, dev, B, seq, V, K)
    x = logits.requires_grad_(True)
    n_content = sum(c[0].numel() for c in convos)

    def main():
        x.grad = None
        L = D.Losses(None)
        L.add_batch(D.distill_loss_batch(x, convos, alpha, temperature=T))
        total = L.loss_dict["train_loss"].detach()
        L.backward(divisor=1)
        return total

    # phase 1 reads the content rows, phase 2 reads them again and writes every row of the gradient
    algo = n_content * V * 2 * 2 + B * seq * V * 2 + n_content * K * (6 + 4 + 4 + 4)
    return (main, main, algo, B * seq,
            f"composite loss of the reference (calculate_divergence per conversation, Losses.backward) over a batch: "
            f"{B} x {seq} tokens ({n_content} content) x {V} vocab bf16, K={K}, alpha={alpha}",
            "rowstats_kernel + composite epilogue + rowcoef_grad_kernel (two-phase, whole fwd+bwd)", {"logits": logits}, x)


def _wl_dropin(batched):
    """The reference's own call pattern at its default shape (config.json: context_len 2048, crop 32000,
    save_topK 400, batch 4): per conversation `calculate_divergence` on fp32 logits + `Losses.add_losses`,
    then one `Losses.backward` for the batch (classes/student/model.py:415-441) -- or, `batched`, the same
    batch through `distill_loss_batch` + `Losses.add_batch`.  The dominant-kernel figure is the library's
    launches alone (phase 1, the epilogue, phase 2 with the rows' coefficients made in it, per conversation) on
    preallocated buffers."""
    def build(D, S, dev, rows):
        import torch
        from llm_distillery_amd import ops
        B, N, V, K, alpha = 4, (rows // 4) if rows else 2048, 32000, 400, 2.0
        g = torch.Generator(device=dev)
        g.manual_seed(11)
        xs, tvs, tis, labs = [], [], [], []
        for _ in range(B):
            x = torch.randn(N, V, generator=g, device=dev) * 2
            tl = torch.log_softmax(x + torch.randn(N, V, generator=g, device=dev), -1)
            tv, ti = torch.topk(tl, K)
            xs.append(x.requires_grad_(True)); tvs.append(tv.contiguous()); tis.append(ti.contiguous())
            labs.append(ti[:-1, 1].contiguous())
        avoid = torch.tensor([N // 2], dtype=torch.long, device=dev)
        xb = torch.stack([x.detach() for x in xs]).requires_grad_(True)
        rows_all = torch.arange(N, device=dev)

        def step():
            L = D.Losses(None)
            if batched:
                xb.grad = None
                L.add_batch(D.distill_loss_batch(xb, [(rows_all, tvs[i], tis[i], labs[i], avoid) for i in range(B)], alpha))
            else:
                for i in range(B):
                    xs[i].grad = None
                    L.add_losses(D.calculate_divergence(xs[i], tvs[i], tis[i], labs[i], alpha, avoid))
            total = L.loss_dict["train_loss"].detach()
            L.backward(divisor=1)
            return total

        lib = D._lib.load()
        bufs = [dict(lse=torch.empty(N, device=dev), zk=torch.empty(N, K, device=dev), rec=torch.empty(N, 8, device=dev),
                     coef=torch.empty(N, 4, device=dev), out=torch.empty(1, 9, device=dev), g=torch.ones(1, device=dev),
                     grad=torch.empty(N, V, device=dev))
                for _ in range(B)]
        import ctypes
        arr = ctypes.c_int32 * 2
        offs = (arr(0, N), arr(0, N - 1), arr(0, 1))

        def launches():
            st = torch.cuda.current_stream().cuda_stream
            for i in range(B):
                x, b = xs[i].detach(), bufs[i]
                lib.dl_composite_forward_fused(x.data_ptr(), 0, V, N, V, 0, N, 1.0, tvs[i].data_ptr(), 0, 1.0, tis[i].data_ptr(), 1, K,
                                               labs[i].data_ptr(), avoid.data_ptr(), 1, offs[0], offs[1], offs[2], 1, 1, alpha,
                                               b["lse"].data_ptr(), b["zk"].data_ptr(), b["rec"].data_ptr(), b["coef"].data_ptr(),
                                               b["out"].data_ptr(), st)
            for i in range(B):
                x, b = xs[i].detach(), bufs[i]
                lib.dl_composite_backward_fused(x.data_ptr(), 0, V, N, V, 0, N, 1.0, tvs[i].data_ptr(), 0, 1.0, tis[i].data_ptr(), 1, K,
                                                offs[0], 1, 1, b["lse"].data_ptr(), b["zk"].data_ptr(), b["rec"].data_ptr(),
                                                b["coef"].data_ptr(), b["g"].data_ptr(), b["grad"].data_ptr(), V, st)
            return bufs[0]["out"]

        algo = B * (N * V * 4 * 3 + N * K * (4 + 8 + 4 + 4 + 4))
        return (step, launches, algo, B * N,
                f"the reference's call pattern at its default shape: {B} conversations x {N} tokens x {V} vocab fp32, K={K}: "
                + ("distill_loss_batch + Losses.add_batch" if batched else "calculate_divergence + Losses.add_losses per conversation")
                + " + Losses.backward", "library launches alone: rowstats with the rows' records + conversation epilogue + rowcoef_grad with the rows' coefficients, per conversation",
                {"logits": xb.detach()}, torch.empty_like(xb))
    return build


COPY_SHAPE = {"threads": 256, "chunks": 16, "one_xcd": True, "wave_major": True, "lds_kb": 0}      # --workload copyshape: see main


def _wl_copyshape(D, S, dev, rows):
    """A bare copy of the C3 logits buffer in the access shape of a row kernel: what the memory system gives
    a kernel that moves `--chunks` 16-byte chunks per thread between its loads and its stores."""
    import torch
    rows = rows or 8 * 4096
    V = 128256
    src = torch.empty((rows, V), dtype=torch.bfloat16, device=dev).normal_()
    dst = torch.empty_like(src)
    cs = COPY_SHAPE

    def main():
        D.copy_rows(src, dst, cs["threads"], cs["chunks"], cs["one_xcd"], cs["wave_major"], cs["lds_kb"])
        return dst[0, :1].float().sum()

    parts = -(-(V * 2 // 16) // (cs["threads"] * cs["chunks"]))
    return (main, main, rows * V * 2 * 2, rows,
            f"bare copy of {rows} x {V} bf16 rows, {cs['threads']} threads x {cs['chunks']} chunks per workgroup ({parts} parts per row, "
            + ("parts of a row on one XCD" if cs["one_xcd"] else "row-major workgroup order") + ", "
            + ("wave-major" if cs["wave_major"] else "striped") + " chunks"
            + (f", at most {160 // cs['lds_kb']} workgroups per CU" if cs["lds_kb"] else "") + ")",
            f"copy_rows_kernel<{cs['threads']},{cs['chunks']}>", {"logits": src}, dst)


WORKLOADS = {"copyshape": _wl_copyshape, "dropin": _wl_dropin(False), "dropin-batch": _wl_dropin(True), "composite": _wl_composite, "producer": _wl_producer, "c1": _wl_dense("c1"), "c2": _wl_dense("c2"), "c3": _wl_c3, "c4": _wl_c4, "c4-merge": _wl_c4_merge, "c5": _wl_c5}


# ---------------------------------------------------------------------------------------------
def cpu_baseline(workload: str, rows: int, reps: int):
    """The reference's op sequence (cast -> /T -> log_softmax -> gather -> kl_div -> mean -> backward) in
    PyTorch eager on the host cores, on a bounded row sample of the same workload (rows are independent, so
    tokens/s carries over to the full row count)."""
    import numpy as np
    import torch
    from llm_distillery_amd import synthetic as S
    from oracle import oracle as O

    if workload == "c3":
        c = S.config3("cpu", rows=rows, seed=3)
        fn = lambda: O.mean_loss_and_grad("fkl", c["logits"], 1.0, t_vals=c["t_val"], t_idx=c["t_idx"].long())
        what = f"{rows} of 32768 rows at V=128256, K=200"
    elif workload in ("c4", "c4-merge"):
        c = S.config4("cpu", rows=rows)
        def fn():
            ids, lq, cnt = O.merge_remap_padded([v.numpy() for v in c["t_vals"]], [i.numpy() for i in c["t_idxs"]],
                                                c["weights"], c["id_map"].numpy())
            z = c["logits"].float().requires_grad_(True)
            O.fwd_kl_sparse_rows(z, ids, lq, cnt).mean().backward()
        what = f"{rows} of 32768 rows at V=128256, 3 teachers x K=200 (dict/loop merge)"
    elif workload in ("c1", "c2"):
        c = S.config1("cpu", B=1, S=rows) if workload == "c1" else S.config2("cpu", B=1, S=rows)
        fn = lambda: O.mean_loss_and_grad(c["kind"], c["logits"], c["T"], t_logits=c["t_logits"], valid=c["valid"])
        what = f"{rows} rows at V=32000, dense teacher"
    elif workload == "composite":
        seq = max(64, rows // 2)
        logits, convos = _composite_batch(torch, S, "cpu", 2, seq, 128256, 200)
        def fn():
            z = O.scaled_student_logits(logits, 128256, 1.0).requires_grad_(True)
            total = 0
            for i, (r, tv, ti, labels, avoid) in enumerate(convos):
                total = total + O.calculate_divergence(torch.index_select(z[i], 0, r), tv.float(), ti.long(), labels, 2.0,
                                                       avoid)["train_loss"]
            total.backward()
        rows = 2 * seq
        what = f"2 conversations x {seq} tokens at V=128256, K=200 (the reference's per-conversation loop)"
    elif workload == "producer":
        c = S.config3("cpu", rows=rows, seed=3)
        fn = lambda: O.to_storage(*[t.reshape(-1, 200) for t in O.teacher_topk_producer(c["logits"], 128256, 200)])
        what = f"{rows} of 32768 rows at V=128256, K=200 (log_softmax + torch.topk)"
    else:
        c = S.config5("cpu", rows=rows)
        def fn():
            marg = torch.tensor(O.marginalise_map(c["t_probs"].numpy(), c["t2s_host"], 32000, dtype=np.float32))
            with np.errstate(divide="ignore"):
                O.mean_loss_and_grad("rkl", c["logits"], c["T"], t_logits=torch.log(marg))
        what = f"{rows} of 8192 rows, Vt=152064 -> Vs=32000 (numpy scatter + torch eager)"
    fn()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": rows / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{what}, fp32 eager oracle fwd+bwd, median of {reps} ({med:.2f} s each; "
                      f"os.cpu_count()={os.cpu_count()})"}


def kernel_source_hash() -> str:
    """sha256 over the kernel sources and the C header, in path order: what the counter summaries were taken on."""
    import glob
    import hashlib
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(ROOT, "llm-distillery_amd", "csrc", "*")) + glob.glob(os.path.join(ROOT, "include", "*.h")))
    for path in files:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str):
    """HBM bytes per launch of this workload from the committed rocprofv3 counter summary -- a figure measured
    in an earlier profiled run of this same command, not in this run (the counters need the profiler) -- and
    only while the kernel sources are still the ones it was measured on (their hash is stored beside it):
    after any change to the kernels it reads null until the counter runs are repeated."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("kernel_source_hash") != kernel_source_hash():
        return None
    return rec.get(f"{workload}_bytes_per_launch")


def measured_valu_busy(workload: str):
    """Share of the dominant kernel's time its vector ALUs were busy, from the committed SQ counter summary (same
    rule as measured_traffic: null once the kernel sources have changed)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("kernel_source_hash") != kernel_source_hash():
        return None
    return rec.get(f"{workload}_valu_busy")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c3")
    ap.add_argument("--rows", type=int, default=0, help="override the workload's token count")
    ap.add_argument("--cpu-rows", type=int, default=-1, help="row sample for the CPU baseline (0 = skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the library's plain copy kernel over the logits buffer (known traffic: its "
                         "byte size each way), the yardstick for rocprofv3 FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--threads", type=int, default=256, help="copyshape: threads per workgroup (256 / 512 / 1024)")
    ap.add_argument("--chunks", type=int, default=16, help="copyshape: 16-byte chunks per thread (2 / 4 / 8 / 12 / 16)")
    ap.add_argument("--row-major", action="store_true", help="copyshape: workgroups in row-major order instead of a row's "
                                                              "parts on one XCD")
    ap.add_argument("--striped", action="store_true", help="copyshape: chunk c of a part belongs to thread c %% threads "
                                                            "instead of every wave owning `chunks` KiB in one piece")
    ap.add_argument("--lds-kb", type=int, default=0, help="copyshape: LDS held per workgroup (bounds workgroups per CU at 160 / n)")
    ap.add_argument("--parts", type=int, default=0, choices=(0, 1, 2, 4, 16),
                    help="c3 only: column parts per row of the loss kernel (0 = the library's choice)")
    ap.add_argument("--vocab", type=int, default=0, help="c3: vocabulary size (default 128256)")
    ap.add_argument("--pitch", type=int, default=0, help="c3: columns per stored row, >= --vocab: the logits are the crop "
                    "[:, :vocab] of such rows")
    ap.add_argument("--alphabet", type=int, default=256, help="c5: byte alphabet of the random vocabularies (256 / 4..16)")
    ap.add_argument("--student-vocab", type=int, default=0, help="c5: student vocabulary size (default 32000)")
    ap.add_argument("--unfused", action="store_true", help="c5: marginalise and reverse KL as two launches")
    ap.add_argument("--no-split", action="store_true", help="c1 / dense: one workgroup per row pair (no workspace)")
    ap.add_argument("--source-hash", action="store_true", help="print the hash of the kernel sources (the value "
                    "profiles/traffic.json carries as kernel_source_hash) and exit")
    ap.add_argument("--inplace", action="store_true",
                    help="c3 only: write the gradient over the logits (same DRAM pages: about 4 %% faster).  After the "
                         "first step the buffer holds gradients, not logits, so the printed loss means nothing; the "
                         "traffic and the arithmetic per step are unchanged.  Not the default for that reason")
    args = ap.parse_args()
    if args.source_hash:
        print(kernel_source_hash())
        return
    global INPLACE, PARTS
    global VOCAB, PITCH, NO_SPLIT, ALPHABET, STUDENT_VOCAB, UNFUSED
    NO_SPLIT = args.no_split
    ALPHABET, STUDENT_VOCAB, UNFUSED = args.alphabet, args.student_vocab, args.unfused
    VOCAB, PITCH = (args.vocab, args.pitch) if args.workload == "c3" else (0, 0)
    PARTS = args.parts if args.workload == "c3" else 0
    INPLACE = bool(args.inplace and args.workload == "c3")
    COPY_SHAPE.update(threads=args.threads, chunks=args.chunks, one_xcd=not args.row_major, wave_major=not args.striped,
                      lds_kb=args.lds_kb)
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path is row-parallel and every configuration fits one "
                 "MI355X; run with --gpus 1")

    import torch
    import llm_distillery_amd as D
    from llm_distillery_amd import synthetic as S

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    step, main_launch, algo_bytes, tokens, desc, kernel, c, grad = WORKLOADS[args.workload](D, S, dev, args.rows)

    for _ in range(args.warmup):
        loss = step()
    torch.cuda.synchronize()
    if args.calibrate_copy:
        for _ in range(3):
            D.copy16(c["logits"], grad)
        torch.cuda.synchronize()

    # whole step, wall clock between synchronisations
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # dominant kernel alone: events on the stream it is launched on (torch's current stream)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in ev:
        a.record()
        main_launch()
        b.record()
    torch.cuda.synchronize()
    kern_ms = sum(a.elapsed_time(b) for a, b in ev) / args.steps
    achieved = algo_bytes / (kern_ms * 1e-3) / 1e9

    cpu_rows = args.cpu_rows if args.cpu_rows >= 0 else {"c3": 4096, "c4": 256, "c4-merge": 256, "dropin": 0, "dropin-batch": 0, "copyshape": 0, "c1": 512, "c2": 4096, "c5": 512, "producer": 2048, "composite": 2048}[args.workload]
    out = {
        "metric": "tokens/sec fused KL fwd+bwd @ vocab 128256 bf16; % of HBM peak GB/s",
        "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp32" if args.workload in ("c1", "dropin", "dropin-batch") else "bf16", "data": "synthetic",
        "config": {"workload": desc, "rows": tokens},
        "loss": loss.item(),
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(args.workload),
                     "traffic_from": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, committed; "
                                     "null when the kernel sources have changed since)",
                     "kernel": kernel, "kernel_ms": kern_ms, "algorithmic_bytes": algo_bytes},
        "cpu_baseline": cpu_baseline(args.workload, cpu_rows, 7 if args.workload == "c3" else 3) if cpu_rows > 0 else None,
    }
    busy = measured_valu_busy(args.workload)
    if busy is not None and busy >= 0.6:
        # a kernel whose vector ALUs are busy most of its time is held by instruction issue before it is held by memory
        out["roofline"]["bound_secondary"] = {"bound": "valu", "busy": busy,
                                              "from": "profiles/traffic.json (rocprofv3 --pmc SQ_ACTIVE_INST_VALU of this command, committed)"}
    if args.workload.startswith("dropin"):
        out["step_over_launches"] = ms_per_step / kern_ms
    print(json.dumps(out))


if __name__ == "__main__":
    main()

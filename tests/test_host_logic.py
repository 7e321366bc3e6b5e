"""CPU-side checks: the Losses accumulator mirrors classes/losses.py, the C-ABI library loads and
exports every symbol the header declares, and the Python layer refuses to run without a GPU."""
import os
import re

import pytest
import torch

import llm_distillery_amd as D

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class _Log:
    def __init__(self):
        self.rows = []

    def log(self, d, step=None):
        self.rows.append((d, step))


def _dict(v, leaf):
    out = {k: torch.tensor(float(v + i)) for i, k in enumerate(D.LOSS_KEYS)}
    out["train_loss"] = leaf * v
    return out


def test_losses_accumulates_sums_and_backward_divides():
    leaf = torch.tensor(2.0, requires_grad=True)
    L = D.Losses(_Log())
    with pytest.raises(ValueError):
        L.add_losses({})
    L.add_losses(_dict(1.0, leaf))
    L.add_losses(_dict(3.0, leaf))
    assert L.num_steps_accumulated == 2
    assert L.loss_dict["kl_div"].item() == (1 + 3) + (3 + 3) and not L.loss_dict["kl_div"].requires_grad
    L.backward(divisor=4)
    assert "train_loss" not in L.loss_dict
    assert leaf.grad.item() == pytest.approx((1.0 + 3.0) / 4)      # sum over conversations / divisor
    L.log(step=7)
    keys = [list(d)[0] for d, _ in L.logger.rows]
    assert keys == [f"Loss/{k}" for k in D.LOSS_KEYS if k != "train_loss"]
    d0, step = L.logger.rows[0]
    assert step == 7 and d0["Loss/custom loss"].item() == pytest.approx(((1 + 1) + (3 + 1)) / 2)
    L.empty()
    assert L.loss_dict == {} and L.num_steps_accumulated == 0


def test_losses_add_batch_equals_adding_one_by_one():
    leaf_a, leaf_b = torch.tensor(2.0, requires_grad=True), torch.tensor(2.0, requires_grad=True)
    one, many = D.Losses(None), D.Losses(None)
    one.add_losses(_dict(0.5, leaf_a))                         # something accumulated before the batch
    many.add_losses(_dict(0.5, leaf_b))
    for v in (1.0, 3.0, 4.0):
        one.add_losses(_dict(v, leaf_a))
    many.add_batch([_dict(v, leaf_b) for v in (1.0, 3.0, 4.0)])
    assert one.num_steps_accumulated == many.num_steps_accumulated == 4
    assert set(one.loss_dict) == set(many.loss_dict)
    for k in one.loss_dict:
        assert one.loss_dict[k].item() == pytest.approx(many.loss_dict[k].item())
        assert k == "train_loss" or not many.loss_dict[k].requires_grad
    one.backward(divisor=2)
    many.backward(divisor=2)
    assert leaf_a.grad.item() == pytest.approx(leaf_b.grad.item()) == pytest.approx(8.5 / 2)
    with pytest.raises(ValueError):
        many.add_batch([])
    single = D.Losses(None)
    single.add_batch([_dict(1.0, leaf_b)])
    assert single.num_steps_accumulated == 1


def test_losses_validation_prefix_and_scaling_operators():
    L = D.Losses(_Log(), validation=True)
    L.add_losses({"train_loss": torch.tensor(1.0), "kl_div": torch.tensor(4.0)})
    L.log(step=1, average=False)
    assert list(L.logger.rows[0][0]) == ["Val Loss/kl_div"]
    half = L / 2
    assert half.loss_dict["kl_div"].item() == 2.0 and half.validation
    L *= 3
    assert L.loss_dict["kl_div"].item() == 12.0
    assert "Validation Losses" in str(L)


def test_losses_packed_dicts_accumulate_like_plain_ones():
    """`calculate_divergence` hands out dicts whose values are views of one [9] tensor; `Losses` sums
    those with one addition per conversation.  Totals, step count, backward and logging must be what
    the key-by-key form gives, also when packed and plain dicts are mixed."""
    from llm_distillery_amd.losses import LossDict
    keys = D.LOSS_KEYS
    leafs = [torch.tensor(float(i + 1), requires_grad=True) for i in range(3)]

    def make(i, packed):
        row = torch.arange(9, dtype=torch.float32) * (i + 1)
        train = leafs[i] * 2
        d = LossDict(zip(keys, row.unbind(0))) if packed else dict(zip(keys, row.clone().unbind(0)))
        d["train_loss"] = train
        if packed:
            d.packed, d.keys_packed = row, keys
        return d

    for pattern in ((True, True, True), (False, False, False), (True, False, True), (False, True, True)):
        for leaf in leafs:
            leaf.grad = None
        L = D.Losses(_Log())
        for i, packed in enumerate(pattern):
            L.add_losses(make(i, packed))
        assert L.num_steps_accumulated == 3
        got = L.loss_dict
        assert list(got)[0] == "train_loss" and set(got) == set(keys)
        assert got["train_loss"].item() == 2 * (1 + 2 + 3)
        for j, k in enumerate(keys[1:], start=1):
            assert got[k].item() == j * (1 + 2 + 3) and not got[k].requires_grad
        L.backward(divisor=2)
        assert all(leaf.grad.item() == 1.0 for leaf in leafs) and "train_loss" not in L.loss_dict
        L.log(step=3)
        assert L.logger.rows[0][0]["Loss/custom loss"].item() == pytest.approx(1 * 6 / 3)
        L.empty()
        assert L.loss_dict == {} and L.num_steps_accumulated == 0
    # the batch form: stack + sum
    L = D.Losses(None)
    L.add_batch([make(i, True) for i in range(3)])
    assert L.num_steps_accumulated == 3 and L.loss_dict["kl_div"].item() == 3 * 6 and L.loss_dict["train_loss"].item() == 12
    half = L / 2
    assert half.loss_dict["kl_div"].item() == 9.0


def test_losses_loss_dict_is_a_plain_writable_dict_also_after_packed_additions():
    """classes/losses.py:22 keeps a plain dict attribute that callers may write into, delete from or scale in
    place; the packed accumulation must not turn such writes into no-ops, and a second backward finds the key
    gone (KeyError) as in the reference (classes/losses.py:77-79)."""
    from llm_distillery_amd.losses import LossDict
    keys = D.LOSS_KEYS
    leaf = torch.tensor(1.0, requires_grad=True)

    def make(i):
        row = torch.arange(9, dtype=torch.float32) * (i + 1)
        d = LossDict(zip(keys, row.unbind(0)))
        d["train_loss"] = leaf * (i + 1)
        d.packed, d.keys_packed = row, keys
        return d

    L = D.Losses(_Log())
    L.add_losses(make(0))
    L.add_losses(make(1))
    L.loss_dict["kl_div"] = torch.tensor(100.0)
    L.loss_dict["CE loss"] /= 2
    del L.loss_dict["CE diff"]
    assert L.loss_dict["kl_div"].item() == 100.0 and L.loss_dict["CE loss"].item() == 2 * 3 / 2 and "CE diff" not in L.loss_dict
    L.add_losses(make(2))                                     # a packed dict after the write: added key by key
    assert L.loss_dict["kl_div"].item() == 100.0 + 3 * 3 and L.loss_dict["CE diff"].item() == 8 * 3
    assert L.loss_dict["train_loss"].item() == 6.0 and L.num_steps_accumulated == 3
    L.backward(divisor=3)
    assert leaf.grad.item() == pytest.approx(2.0)
    with pytest.raises(KeyError):
        L.backward()
    P = D.Losses(None)                                        # never touched from outside: still packed at the second backward
    P.add_losses(make(0))
    P.backward()
    with pytest.raises(KeyError):
        P.backward()


def test_registered_operators_trace_with_fake_tensors():
    """The V-wide launches are registered torch.library operators with fake (shape-only) implementations, so that
    FakeTensor tracing / torch.compile see through them without touching a GPU."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from llm_distillery_amd import ops
    with FakeTensorMode():
        logits = torch.empty(10, 64, dtype=torch.bfloat16)
        t_val = torch.empty(7, 5, dtype=torch.float16)
        t_idx = torch.empty(7, 5, dtype=torch.int32)
        labels = torch.empty(5, dtype=torch.int64)
        avoid = torch.empty(1, dtype=torch.int64)
        offsets = torch.empty(3, 3, dtype=torch.int32)                  # two conversations
        row_map = torch.empty(10, dtype=torch.int32)
        train, nine, lse, zk, rec, coef = ops.composite_forward_op(logits, t_val, t_idx, labels, avoid, offsets, row_map, 1.0, 1.0, 2.0, 48)
        assert train.shape == (2,) and nine.shape == (2, 9) and lse.shape == (7,) and zk.shape == (7, 5)
        assert rec.shape == (7, 8) and coef.shape == (7, 4) and train.dtype == torch.float32
        grad = ops.composite_backward_op(logits, t_val, t_idx, lse, zk, rec, coef, train, offsets, row_map, 1.0, 1.0, 48)
        assert grad.shape == logits.shape and grad.dtype == logits.dtype
        lse2, zk2 = ops.rowstats_topk(logits, t_idx, row_map, 1.0, 48)
        assert lse2.shape == (7,) and zk2.shape == (7, 5)


def test_library_exports_every_symbol_the_header_declares():
    header = open(os.path.join(ROOT, "include", "distill_hip.h")).read()
    declared = set(re.findall(r"\b(dl_[a-z0-9_]+)\s*\(", header))
    lib = D._lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(D._lib.exported_symbols())
    assert lib.dl_abi_version() >= 1
    assert lib.dl_status_string(0) == b"ok" and b"NULL" in lib.dl_status_string(-1)


def test_argument_errors_are_reported_before_any_gpu_work():
    """Host-side validation of the entry points that take host arrays: every call below returns its
    status before the first HIP call, so the (never dereferenced) device pointers can be anything."""
    import ctypes
    lib = D._lib.load()
    fake = ctypes.c_void_p(4096)
    i32 = lambda *v: (ctypes.c_int32 * len(v))(*v)
    # composite: offsets that travel with the launch are checked on the host
    def fwd(row, lab, av, C, N):
        return lib.dl_composite_forward(fake, fake, fake, 2, 1.0, fake, 0, 8, fake, fake, 1, row, lab, av, 1, C, N, 2.0, fake, fake,
                                        fake, None)
    assert fwd(i32(0, 5, 3), i32(0, 4, 6), i32(0, 0, 0), 2, 3) == -3            # rows not non-decreasing
    assert fwd(i32(0, 5, 9), i32(0, 4, 7), i32(0, 0, 0), 2, 10) == -3           # rows do not end at n_rows
    assert fwd(i32(1, 5), i32(0, 4), i32(0, 0), 1, 5) == -3                     # rows do not start at 0
    many = i32(*range(66))
    assert fwd(many, many, many, 65, 65) == -4                                  # more conversations than a launch carries
    assert lib.dl_composite_forward(fake, fake, fake, 2, 1.0, fake, 0, 8, fake, fake, 7, i32(0, 5), i32(0, 4), i32(0, 0), 1, 1, 5,
                                    2.0, fake, fake, fake, None) == -2          # ignore entries of an unknown integer type
    assert lib.dl_composite_backward(fake, fake, fake, 2, 1.0, fake, 0, 8, i32(0, 4), 1, 1, 5, fake, fake, fake, fake, fake,
                                     None) == -3
    # multi-teacher loss: limits, weights, workspace
    ptrs = (ctypes.c_void_p * 3)(4096, 4096, 4096)
    w = lambda *v: (ctypes.c_float * len(v))(*v)
    def multi(V=128256, n=3, K=200, ws=fake, ws_bytes=1 << 40, weights=w(0.5, 0.3, 0.2), stride=None):
        return lib.dl_fkl_multi_teacher(fake, 1, stride or V, 64, V, None, n, ptrs, ptrs, 2, 0, K, 64, weights, None, 0, 1.0, 1.0,
                                        fake, fake, V, ws, ws_bytes, 0, None)
    assert multi(n=3, K=700) == -4                                              # more than DL_MAX_TOPK entries per row
    assert multi(V=300000) == -4                                                # rows too wide for the register kernels
    assert multi(V=128257, stride=128264) == -6                                 # odd vocabulary
    assert multi(ws=None) == -7 and multi(ws_bytes=1000) == -7                  # no / too small a workspace
    assert multi(weights=w(0.5, -0.1, 0.2)) == -3 and multi(weights=w(0.5, float("nan"), 0.2)) == -3
    need = lib.dl_fkl_multi_teacher_workspace_bytes(1, 64, 128256, 3, 200, 64, 0)
    assert need > 64 * 4 * 256 * 8 and multi(ws_bytes=need - 1) == -7
    assert lib.dl_fkl_multi_teacher_workspace_bytes(1, 64, 300000, 3, 200, 64, 0) == 0


def test_no_cpu_fallback():
    x = torch.randn(4, 64)
    tv, ti = torch.randn(4, 8), torch.randint(0, 64, (4, 8), dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        D.div_topk("fkl", x, tv, ti)
    with pytest.raises(RuntimeError, match="no CPU path"):
        D.calculate_divergence(x, tv, ti.long(), torch.zeros(3, dtype=torch.long), 2.0, torch.zeros(0, dtype=torch.long))


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "llm-distillery_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "synthetic.py", f"{f} mentions the oracle"

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


def test_library_exports_every_symbol_the_header_declares():
    header = open(os.path.join(ROOT, "include", "distill_hip.h")).read()
    declared = set(re.findall(r"\b(dl_[a-z0-9_]+)\s*\(", header))
    lib = D._lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(D._lib.exported_symbols())
    assert lib.dl_abi_version() >= 1
    assert lib.dl_status_string(0) == b"ok" and b"NULL" in lib.dl_status_string(-1)


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

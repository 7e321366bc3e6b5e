"""Writes the golden vectors under tests/golden/ from the reference's own code.

Runs only in the build container, where the reference tree is mounted at
/root/reference; the fixtures it writes are committed and are what the tests
read.  Two functions of the path have quirks no closed form fixes (the crop rule
and valid-mean fill of the top-K cross entropy, the pad-by-one and non-detached
max of the alpha weighting, tie/tail behaviour of the pairwise merge), so their
input/output vectors are taken from the reference itself:

  * utils/finetuning_utils.py:47-124  calculate_divergence   -> calculate_divergence.npz
  * classes/data_manager.py:198-261   H5DataManager._merge_data -> merge_data.npz

`bitsandbytes`, `wandb` and `h5py` are not installed here and are not used by
those two functions; empty placeholder modules satisfy the module-level imports.
"""
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def _placeholder(name):
    mod = types.ModuleType(name)
    sys.modules[name] = mod
    return mod


def make_calculate_divergence():
    _placeholder("bitsandbytes")
    sys.path.insert(0, REF)
    from utils.finetuning_utils import calculate_divergence  # noqa: E402

    out = {}
    cases = [
        # name, N, K, V, labels, avoid rows, alpha, seed
        ("two_ranges", 17, 8, 64, 16, [6, 15], 2.0, 101),
        ("one_range", 12, 6, 40, 11, [], 2.0, 202),
        ("alpha0", 9, 5, 33, 8, [], 0.0, 303),
        ("alpha_half", 21, 10, 128, 20, [4, 11, 19], 0.5, 404),
    ]
    for name, N, K, V, L, avoid, alpha, seed in cases:
        g = torch.Generator().manual_seed(seed)
        student = (torch.randn(N, V, generator=g) * 2.0)
        teacher_full = torch.log_softmax(student + torch.randn(N, V, generator=g), dim=-1)
        t_val, t_idx = torch.topk(teacher_full, K, dim=-1)
        t_val = t_val.to(torch.float16).float()      # as stored on disk then loaded
        labels = torch.empty(L, dtype=torch.long)
        for r in range(L):
            # ~70 % of labels are among the row's ids (valid rows), the rest are not
            if torch.rand((), generator=g) < 0.7:
                labels[r] = t_idx[r, int(torch.randint(0, K, (), generator=g))]
            else:
                cand = int(torch.randint(0, V, (), generator=g))
                labels[r] = cand
        avoid_t = torch.as_tensor(np.array(avoid), dtype=torch.long)
        s_in = student.clone().requires_grad_(True)
        res = calculate_divergence(s_in, t_val.clone(), t_idx.clone(), labels, alpha, avoid_t)
        res["train_loss"].backward()
        out[f"{name}/student"] = student.numpy()
        out[f"{name}/teacher"] = t_val.numpy()
        out[f"{name}/indices"] = t_idx.numpy()
        out[f"{name}/labels"] = labels.numpy()
        out[f"{name}/avoid"] = avoid_t.numpy()
        out[f"{name}/alpha"] = np.float64(alpha)
        out[f"{name}/grad"] = s_in.grad.numpy()
        for k, v in res.items():
            out[f"{name}/out/{k}"] = v.detach().numpy()
    np.savez_compressed(os.path.join(HERE, "calculate_divergence.npz"), **out)
    print("calculate_divergence.npz:", len(out), "arrays")


def make_merge_data():
    _placeholder("h5py").File = object
    sys.path.insert(0, REF)
    from classes.data_manager import H5DataManager  # noqa: E402

    class _Dist:
        pass

    class _Self:
        def __init__(self, disk):
            self._disk = disk

        def _load_id(self, hdf_file, id):
            return self._disk

    out = {}
    cases = [("equal", 9, 9, 6, 50, 11), ("disk_longer", 12, 7, 5, 40, 22),
             ("new_longer", 5, 10, 8, 64, 33)]
    for name, n_disk, n_new, K, V, seed in cases:
        g = torch.Generator().manual_seed(seed)

        def draw(n):
            lp = torch.log_softmax(torch.randn(n, V, generator=g) * 2.0, dim=-1)
            v, i = torch.topk(lp, K, dim=-1)
            return v.to(torch.float16).numpy().astype(np.float32), i.numpy().astype(np.int64)

        dv, di = draw(n_disk)
        nv, ni = draw(n_new)
        d = _Dist()
        d.distribution = nv.copy()
        d.indices = ni.copy()
        mv, mi = H5DataManager._merge_data(_Self((dv.copy(), di.copy())), None, d, 0)
        out[f"{name}/disk_val"], out[f"{name}/disk_idx"] = dv, di
        out[f"{name}/new_val"], out[f"{name}/new_idx"] = nv, ni
        out[f"{name}/merged_val"], out[f"{name}/merged_idx"] = np.asarray(mv), np.asarray(mi)
    # dense merge (indices None)
    g = torch.Generator().manual_seed(44)
    dv = torch.log_softmax(torch.randn(6, 20, generator=g), -1).numpy()
    nv = torch.log_softmax(torch.randn(4, 20, generator=g), -1).numpy()
    d = _Dist()
    d.distribution = nv.copy()
    d.indices = None
    try:
        mv, mi = H5DataManager._merge_data(_Self((dv.copy(), None)), None, d, 0)
        out["dense/merged_val"] = np.asarray(mv)
    except UnboundLocalError:
        # the reference never binds `merged_indices` on the dense branch
        out["dense/raises_unbound_local"] = np.int32(1)
    out["dense/disk_val"], out["dense/new_val"] = dv, nv
    np.savez_compressed(os.path.join(HERE, "merge_data.npz"), **out)
    print("merge_data.npz:", len(out), "arrays")


if __name__ == "__main__":
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    if which in ("all", "loss"):
        make_calculate_divergence()
    if which in ("all", "merge"):
        make_merge_data()

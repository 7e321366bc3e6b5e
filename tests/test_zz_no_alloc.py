"""dl_div_topk_static -- the entry point that allocates nothing: its split-row scratch is a static
device array of the library -- against dl_div_topk with a caller-owned workspace.  Both run the same
kernels, so the results must agree bit for bit; two calls in a row, the second on a smaller input,
show that what one call leaves in the shared array does not reach the next."""
import ctypes

import pytest
import torch

DEV = "cuda:0"


@pytest.fixture(scope="module")
def D():
    import llm_distillery_amd as d
    d._lib.load()
    return d


def _case(R, V, K, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(R, V, generator=g) * 3).to(dtype)
    tl = torch.log_softmax(logits.float() + torch.randn(R, V, generator=g), -1)
    tv, ti = torch.topk(tl, K)
    return logits.to(DEV), tv.to(torch.float16).to(DEV), ti.to(torch.int32).to(DEV)


def _masked_map(R, masked):
    valid = torch.ones(R, dtype=torch.bool)
    valid[masked] = False
    rm = torch.full((R,), -1, dtype=torch.int32)
    rm[valid] = torch.arange(int(valid.sum()), dtype=torch.int32)
    return rm.to(DEV), int(valid.sum())


@pytest.mark.gpu
@pytest.mark.parametrize("V,dtype,hooks", [(128256, torch.bfloat16, {}), (128256, torch.bfloat16, {"no_wait": True}),
                                           (152064, torch.float16, {}), (40000, torch.float32, {"no_wait": True}),
                                           (32000, torch.bfloat16, {})])
def test_static_scratch_entry_point_matches_the_workspace_one(D, V, dtype, hooks):
    """Rows cut into 4 parts (128256 bf16), 3 (40000 fp32: 10000 chunks in parts of 256 x 14) and 5 (152064 fp16)
    meet through the scratch; 32000-wide rows need none.  With `no_wait` every part also goes through the list of
    deferred parts that lives in the same array."""
    K = 200
    big = _case(72, V, K, dtype, 5)
    small = _case(19, V, K, dtype, 6)
    for (x, tv, ti), masked in ((big, [0, 17, 71]), (small, [3])):
        R = x.shape[0]
        rm, nv = _masked_map(R, masked)
        want_rl, want_g = D.div_topk("fkl", x, tv[:nv], ti[:nv], row_map=rm, T=1.3, grad_scale=1.0 / nv, **hooks)
        rl = torch.full((R,), float("nan"), device=DEV)
        g = torch.full_like(x, float("nan"))
        before = torch.cuda.memory_allocated()
        D.div_topk_static("fkl", x, tv[:nv], ti[:nv], rl, g, row_map=rm, T=1.3, grad_scale=1.0 / nv, **hooks)
        assert torch.cuda.memory_allocated() == before            # nothing came from torch's allocator either
        torch.cuda.synchronize()
        assert torch.equal(rl, want_rl) and torch.equal(g, want_g)
    # reverse KL needs no scratch; the entry point serves it all the same
    x, tv, ti = small
    want_rl, want_g = D.div_topk("rkl", x, tv, ti, T=0.9)
    rl, g = torch.empty(x.shape[0], device=DEV), torch.empty_like(x)
    D.div_topk_static("rkl", x, tv, ti, rl, g, T=0.9)
    assert torch.equal(rl, want_rl) and torch.equal(g, want_g)


@pytest.mark.gpu
@pytest.mark.parametrize("no_wait", [False, True])
def test_static_scratch_close_to_its_limit(D, no_wait):
    """52000 rows of 128256 bf16 columns need 4.16 MB of the 4 MiB array (records of 4 parts, a counter and a
    list slot per part): offsets and the clear at a realistic size, with and without the list of deferred parts,
    bit for bit against the workspace entry point; then a small call, which must not see what the large one left."""
    from llm_distillery_amd import synthetic as S
    lib = D._lib.load()
    rows, V = 52000, 128256
    assert 0.95 * D._lib.DL_STATIC_SCRATCH_BYTES < lib.dl_div_topk_workspace_bytes(0, D._lib.DL_BF16, rows, V) <= D._lib.DL_STATIC_SCRATCH_BYTES
    c = S.config3(DEV, rows=rows, V=V, K=64)
    want_rl, want_g = D.div_topk("fkl", c["logits"], c["t_val"], c["t_idx"], grad_scale=1.0 / rows, no_wait=no_wait)
    rl = torch.full((rows,), float("nan"), device=DEV)
    g = torch.empty_like(c["logits"])
    D.div_topk_static("fkl", c["logits"], c["t_val"], c["t_idx"], rl, g, grad_scale=1.0 / rows, no_wait=no_wait)
    assert torch.equal(rl, want_rl) and torch.equal(g, want_g)
    del g, want_g
    x, tv, ti = _case(9, V, 64, torch.bfloat16, 12)
    want_rl, want_g = D.div_topk("fkl", x, tv, ti, no_wait=no_wait)
    rl, g = torch.empty(9, device=DEV), torch.empty_like(x)
    D.div_topk_static("fkl", x, tv, ti, rl, g, no_wait=no_wait)
    assert torch.equal(rl, want_rl) and torch.equal(g, want_g)


@pytest.mark.gpu
def test_static_scratch_forward_only_and_in_place(D):
    x, tv, ti = _case(33, 128256, 64, torch.bfloat16, 9)
    want_rl, want_g = D.div_topk("fkl", x, tv, ti, T=2.0)
    rl = torch.empty(33, device=DEV)
    D.div_topk_static("fkl", x, tv, ti, rl, None, T=2.0)
    assert torch.equal(rl, want_rl)
    y = x.clone()
    D.div_topk_static("fkl", y, tv, ti, rl, y, T=2.0)              # gradient over the logits
    assert torch.equal(rl, want_rl) and torch.equal(y, want_g)


def test_problems_beyond_the_static_array_are_refused_before_any_gpu_work():
    """Host-side check, no GPU needed: the size test comes before the first HIP call, so the
    (never dereferenced) pointers can be anything non-null."""
    import llm_distillery_amd as d
    lib = d._lib.load()
    limit = d._lib.DL_STATIC_SCRATCH_BYTES
    V, dt = 128256, d._lib.DL_BF16
    rows_ok = 1
    while lib.dl_div_topk_workspace_bytes(0, dt, rows_ok * 2, V) <= limit:
        rows_ok *= 2
    rows_bad = rows_ok * 2
    assert lib.dl_div_topk_workspace_bytes(0, dt, rows_bad, V) > limit
    fake = ctypes.c_void_p(4096)
    st = lib.dl_div_topk_static(0, fake, dt, V, rows_bad, V, None, fake, d._lib.DL_F16, fake, d._lib.DL_I32, 8, rows_bad,
                                None, 1.0, 1.0, 1.0, fake, fake, V, 0, None)
    assert st == -8 and b"static" in lib.dl_status_string(st)
    # narrow rows need no scratch: no row limit applies (argument errors are still reported)
    assert lib.dl_div_topk_static(0, fake, dt, 100, 10 ** 6, 32000, None, fake, d._lib.DL_F16, fake, d._lib.DL_I32, 8,
                                  10 ** 6, None, 1.0, 1.0, 1.0, fake, fake, 32000, 0, None) == -3      # row_stride < V

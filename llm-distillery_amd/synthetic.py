"""Seeded synthetic inputs for the five benchmark configurations.

Everything is generated in row chunks on the target device so the largest config
(32768 x 128256 bf16) never needs more than one fp32 chunk of scratch.  The same
seed on the same device type gives the same tensors.
"""
from __future__ import annotations

import numpy as np
import torch

CHUNK_ROWS = 1024


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _gumbel(shape, g, device):
    u = torch.rand(shape, generator=g, device=device).clamp_(1e-10, 1.0 - 1e-7)
    return -torch.log(-torch.log(u))


def topk_teacher_for(student_chunk: torch.Tensor, K: int, n_hot: int, g, teacher_vocab: int | None = None):
    """K unique int32 ids per row (the row's `n_hot` largest logits plus uniform
    draws without replacement) and fp16 log-probs = log-softmax of
    Gumbel-perturbed scores over those K entries."""
    R, V = student_chunk.shape
    dev = student_chunk.device
    Vt = V if teacher_vocab is None else teacher_vocab
    sf = student_chunk.float()
    hot = sf.topk(n_hot, dim=-1).indices if n_hot > 0 else torch.empty((R, 0), dtype=torch.long, device=dev)
    noise = torch.rand((R, Vt), generator=g, device=dev)
    if n_hot > 0:
        noise.scatter_(1, hot, -1.0)
    rest = noise.topk(K - n_hot, dim=-1).indices
    ids = torch.cat((hot, rest), dim=1)
    base = torch.gather(sf, 1, ids.clamp(max=V - 1))
    scores = base + _gumbel((R, K), g, dev)
    logp = torch.log_softmax(scores, dim=-1)
    return logp.to(torch.float16), ids.to(torch.int32)


def config3(device, rows: int = 8 * 4096, V: int = 128256, K: int = 200, seed: int = 3, std: float = 3.0,
            dtype=torch.bfloat16):
    """Sparse top-K teacher, forward KL: student ~ N(0, 3^2) bf16, K=200 ids per
    token (argmax-20 of the student row + 180 uniform), fp16 teacher log-probs, T=1."""
    g = _gen(device, seed)
    logits = torch.empty((rows, V), dtype=dtype, device=device)
    t_val = torch.empty((rows, K), dtype=torch.float16, device=device)
    t_idx = torch.empty((rows, K), dtype=torch.int32, device=device)
    for a in range(0, rows, CHUNK_ROWS):
        b = min(rows, a + CHUNK_ROWS)
        chunk = (torch.randn((b - a, V), generator=g, device=device) * std).to(dtype)
        logits[a:b] = chunk
        t_val[a:b], t_idx[a:b] = topk_teacher_for(chunk, K, min(20, K), g)
    return {"logits": logits, "t_val": t_val, "t_idx": t_idx, "T": 1.0, "kind": "fkl"}


def row_map_from_valid(valid: torch.Tensor) -> torch.Tensor:
    """int32 map for the kernels: position of each valid row among the valid rows, -1 elsewhere."""
    rm = torch.full((valid.numel(),), -1, dtype=torch.int32, device=valid.device)
    rm[valid] = torch.arange(int(valid.sum()), dtype=torch.int32, device=valid.device)
    return rm


def config1(device, B: int = 1, S: int = 512, V: int = 32000, seed: int = 1):
    """Plumbing config: forward KL over the full vocabulary, fp32.  Student ~ N(0, 2^2), teacher =
    student + N(0, 1), T = 1; the last ceil(10 %) positions of the sequence are padding (for
    S = 512: 461 valid, 51 masked).  The dense teacher holds only the valid rows."""
    g = _gen(device, seed)
    logits = torch.randn((B * S, V), generator=g, device=device) * 2.0
    teacher = logits + torch.randn((B * S, V), generator=g, device=device)
    n_pad = -(-S // 10)
    valid = (torch.arange(S, device=device) < S - n_pad).repeat(B)
    return {"logits": logits, "t_logits": teacher[valid].contiguous(), "valid": valid,
            "row_map": row_map_from_valid(valid), "T": 1.0, "kind": "fkl"}


def config2(device, B: int = 4, S: int = 2048, V: int = 32000, seed: int = 2, dtype=torch.bfloat16):
    """JSD over the full vocabulary, dense bf16 teacher, T = 2: student ~ N(0, 2^2), teacher =
    0.8 * student + N(0, 1.5^2); per-sequence valid length uniform in [S/2, S], the rest masked."""
    g = _gen(device, seed)
    s32 = torch.randn((B * S, V), generator=g, device=device) * 2.0
    teacher = (0.8 * s32 + torch.randn((B * S, V), generator=g, device=device) * 1.5).to(dtype)
    logits = s32.to(dtype)
    del s32
    lengths = torch.randint(S // 2, S + 1, (B,), generator=g, device=device)
    valid = (torch.arange(S, device=device).unsqueeze(0) < lengths.unsqueeze(1)).reshape(-1)
    return {"logits": logits, "t_logits": teacher[valid].contiguous(), "valid": valid,
            "row_map": row_map_from_valid(valid), "T": 2.0, "kind": "jsd", "lengths": lengths}


def vocab_id_map(device, Vt: int = 152064, Vs: int = 128256, drop: float = 0.05, seed: int = 40) -> torch.Tensor:
    """Seeded int32 teacher->student id map: ~`drop` of the teacher ids map to -1 (dropped), the rest
    to uniform student ids, so many teacher ids collide on one student id."""
    g = _gen(device, seed)
    m = torch.randint(0, Vs, (Vt,), generator=g, device=device, dtype=torch.int32)
    m[torch.rand((Vt,), generator=g, device=device) < drop] = -1
    return m


def config4(device, rows: int = 4 * 8192, V: int = 128256, Vt: int = 152064, K: int = 200, n_teachers: int = 3,
            seed: int = 4, dtype=torch.bfloat16):
    """Multi-teacher merge + vocabulary remap, forward KL: three top-K=200 teachers over a
    152064-id teacher vocabulary, weights (0.5, 0.3, 0.2), seeded id map into the 128256-id student
    vocabulary (~5 % dropped, collisions sum), bf16 student logits ~ N(0, 3^2), T = 1."""
    g = _gen(device, seed)
    logits = torch.empty((rows, V), dtype=dtype, device=device)
    vals = [torch.empty((rows, K), dtype=torch.float16, device=device) for _ in range(n_teachers)]
    idxs = [torch.empty((rows, K), dtype=torch.int32, device=device) for _ in range(n_teachers)]
    for a in range(0, rows, CHUNK_ROWS):
        b = min(rows, a + CHUNK_ROWS)
        chunk = (torch.randn((b - a, V), generator=g, device=device) * 3.0).to(dtype)
        logits[a:b] = chunk
        for j in range(n_teachers):
            vals[j][a:b], idxs[j][a:b] = topk_teacher_for(chunk, K, 20, g, teacher_vocab=Vt)
    return {"logits": logits, "t_vals": vals, "t_idxs": idxs, "weights": (0.5, 0.3, 0.2)[:n_teachers],
            "id_map": vocab_id_map(device, Vt, V, seed=seed + 36), "T": 1.0, "kind": "fkl"}


def random_byte_vocab(n: int, seed: int, min_len: int = 1, max_len: int = 16, alphabet: int = 256,
                      all_single_bytes: bool = False) -> list[bytes]:
    """n random byte strings with lengths uniform in [min_len, max_len]; with `all_single_bytes`
    the first 256 entries are the 256 one-byte strings (the byte-fallback tokens)."""
    rng = np.random.default_rng(seed)
    out: list[bytes] = [bytes([b]) for b in range(256)] if all_single_bytes else []
    lens = rng.integers(min_len, max_len + 1, n - len(out))
    blob = rng.integers(0, alphabet, int(lens.sum()), dtype=np.uint8).tobytes()
    at = 0
    for L in lens:
        out.append(blob[at:at + int(L)])
        at += int(L)
    return out


def config5(device, rows: int = 2 * 4096, Vs: int = 32000, Vt: int = 152064, seed: int = 5, dtype=torch.bfloat16,
            alphabet: int = 256):
    """Cross-tokenizer byte-trie marginalisation, then reverse KL: student vocabulary of `Vs` random
    byte strings (lengths 1-16, all 256 single bytes included), teacher vocabulary of `Vt` random byte
    strings; dense fp32 teacher softmax [rows, Vt]; bf16 student logits ~ N(0, 2^2); T = 1.5.
    The id map / CSR come from the host trie."""
    from . import vocab_utils
    student_vocab = random_byte_vocab(Vs, seed * 100 + 1, all_single_bytes=True, alphabet=alphabet)
    teacher_vocab = random_byte_vocab(Vt, seed * 100 + 2, alphabet=alphabet)
    t2s = vocab_utils.longest_prefix_map(student_vocab, teacher_vocab)
    g = _gen(device, seed)
    logits = (torch.randn((rows, Vs), generator=g, device=device) * 2.0).to(dtype)
    probs = torch.empty((rows, Vt), dtype=torch.float32, device=device)
    for a in range(0, rows, CHUNK_ROWS):
        b = min(rows, a + CHUNK_ROWS)
        probs[a:b] = torch.softmax(torch.randn((b - a, Vt), generator=g, device=device) * 2.0, dim=-1)
    return {"logits": logits, "t_probs": probs, "t2s": torch.as_tensor(t2s, device=device), "t2s_host": t2s,
            "student_vocab": student_vocab, "teacher_vocab": teacher_vocab, "T": 1.5, "kind": "rkl"}

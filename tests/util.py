"""Seeded synthetic inputs shared by the tests (seed 42, the reference's: tests/test_decompress.py:20)."""
import numpy as np
import torch


def gen(seed=42):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def rand_codes(numel, seed=42):
    """Uniform 32-bit words as int32 (full entropy, top bit included)."""
    lo = torch.randint(0, 1 << 16, (numel,), generator=gen(seed), dtype=torch.int64)
    hi = torch.randint(0, 1 << 16, (numel,), generator=gen(seed + 1), dtype=torch.int64)
    w = (hi << 16) | lo
    w = torch.where(w >= (1 << 31), w - (1 << 32), w)
    return w.to(torch.int32)


def rand_half(numel, seed=7, scale=1.0):
    return (torch.randn(numel, generator=gen(seed), dtype=torch.float32) * scale).to(torch.float16)


def np_u32(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def np_f16(t):
    return t.detach().cpu().contiguous().numpy()


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300))

"""Seeded random shapes through every op, against the CPU oracle: the fixed shapes of the other GPU tests are
the layer sizes and hand-picked corners; these look for what nobody picked (odd row counts, one-lane ragged
slabs, row counts around the CU count, batches around 16)."""
import numpy as np
import pytest
import torch

from util import np_f16, np_u32, rand_codes, rand_half, rel_l2

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-3


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return rptc_kernels


def _mode(rk, mode):
    class _Ctx:
        def __enter__(self):
            self.prev = rk.set_carry_mode(mode)

        def __exit__(self, *a):
            rk.set_carry_mode(self.prev)
    return _Ctx()




@pytest.mark.parametrize("case", range(24))
def test_matvec_and_dense_export_random_shapes(rk, oracle, case):
    rng = np.random.default_rng(1000 + case)
    m = int(rng.choice([1, 2, 31, 255, 256, 257, 511, 513, int(rng.integers(1, 1200))]))
    n = 64 * int(rng.choice([1, 2, 31, 32, 33, 63, 65, int(rng.integers(1, 200))]))
    S, mode, bits = int(rng.choice([6, 8])), int(rng.integers(0, 2)), int(rng.choice([2, 2, 3, 4]))
    print(f"\n[case] matvec m={m} n={n} S={S} mode={mode} bits={bits}", flush=True)
    comp = rand_codes(m * n * bits // 32, seed=case)
    cb = rand_half(2 << S, seed=case + 1)
    x = rand_half(n, seed=case + 2)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    out = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    with _mode(rk, mode):
        rk.matvec_bits_dense(comp.cuda(), cb.cuda(), W, bits)
        rk.decompress_matvec_bits(comp.cuda(), cb.cuda(), x.cuda(), out, bits)
    want = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=mode)
    assert np.array_equal(np_f16(W).view(np.uint16), want.view(np.uint16))
    assert rel_l2(np_f16(out), oracle.dense_matvec(want, np_f16(x))) < REL_L2_TOL


@pytest.mark.parametrize("case", range(20))
def test_matmul_random_shapes(rk, oracle, case):
    rng = np.random.default_rng(2000 + case)
    m = int(rng.choice([1, 15, 16, 17, 255, 257, int(rng.integers(1, 900))]))
    n = 64 * int(rng.choice([1, 31, 32, 33, 64, int(rng.integers(1, 150))]))
    batch = int(rng.choice([1, 2, 15, 16, 17, 31, 32]))
    S, mode, bits = int(rng.choice([6, 8])), int(rng.integers(0, 2)), int(rng.choice([2, 2, 3, 4]))
    print(f"\n[case] matmul m={m} n={n} batch={batch} S={S} mode={mode} bits={bits}", flush=True)
    comp = rand_codes(m * n * bits // 32, seed=case + 10)
    cb = rand_half(2 << S, seed=case + 11)
    x = rand_half(batch * n, seed=case + 12).reshape(batch, n)
    out = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
    with _mode(rk, mode):
        rk.decompress_matmul_bits(comp.cuda(), cb.cuda(), x.cuda(), out, bits)
    W = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=mode)
    want = np_f16(x).astype(np.float64) @ W.astype(np.float64).T
    got = np_f16(out).astype(np.float64)
    assert np.all(np.isfinite(got)) and rel_l2(got, want) < REL_L2_TOL


@pytest.mark.parametrize("case", range(16))
def test_matvec_t_random_shapes(rk, oracle, case):
    rng = np.random.default_rng(3000 + case)
    m = int(rng.choice([1, 63, 64, 65, 255, 256, 1000, int(rng.integers(1, 3000))]))
    n = 64 * int(rng.choice([1, 7, 8, 9, 16, 64, int(rng.integers(1, 128))]))
    L, mode = int(rng.choice([14, 16])), int(rng.integers(0, 2))
    print(f"\n[case] matvec_t m={m} n={n} L={L} mode={mode}", flush=True)
    comp = rand_codes(m * n // 16, seed=case + 20)
    cb = rand_half(1 << L, seed=case + 21)
    x = rand_half(n, seed=case + 22)
    out0 = rand_half(m, seed=case + 23)
    out = out0.cuda()
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    with _mode(rk, mode):
        getattr(rk, f"decompress_matvec_t_{L}")(comp.cuda(), cb.cuda(), x.cuda(), out)
        rk.matvec_t_dense(comp.cuda(), cb.cuda(), W, L)
    wantW = oracle.matvec_t_dense(np_u32(comp), np_f16(cb), m, n, L, mode=mode)
    assert np.array_equal(np_f16(W).view(np.uint16), wantW.view(np.uint16))
    want = oracle.matvec_t(np_u32(comp), np_f16(cb), np_f16(x), m, L, mode=mode) + np_f16(out0).astype(np.float64)
    assert rel_l2(np_f16(out), want) < REL_L2_TOL


@pytest.mark.parametrize("case", range(10))
def test_decompress_random_shapes(rk, oracle, case):
    rng = np.random.default_rng(4000 + case)
    m = int(rng.choice([1, 2, 255, 257, int(rng.integers(1, 600))]))
    cn = 32 * int(rng.integers(1, 9))
    mode = int(rng.integers(0, 2))
    print(f"\n[case] decompress m={m} cn={cn} mode={mode}", flush=True)
    comp = rand_codes(m * 4 * cn, seed=case + 30).reshape(m, 4 * cn)
    cb = rand_half(65536, seed=case + 31)
    out = torch.full((m, 64 * cn), float("nan"), dtype=torch.float16, device="cuda")
    with _mode(rk, mode):
        rk.decompress(comp.cuda(), cb.cuda(), out)
    want = oracle.decompress(np_u32(comp), np_f16(cb), mode=mode)
    assert np.array_equal(np_f16(out).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("case", range(10))
def test_fused_prologues_random_shapes(rk, oracle, case):
    """silu / add + rms-norm prologues against the double-precision definition through the oracle's dense matrix."""
    rng = np.random.default_rng(5000 + case)
    m = int(rng.choice([1, 33, 256, 300, int(rng.integers(1, 700))]))
    n = 64 * int(rng.choice([1, 4, 33, 64, 172, int(rng.integers(1, 200))]))
    S, mode = int(rng.choice([6, 8])), int(rng.integers(0, 2))
    print(f"\n[case] fused prologues m={m} n={n} S={S} mode={mode}", flush=True)
    comp = rand_codes(m * n // 16, seed=case + 40)
    cb = rand_half(2 << S, seed=case + 41)
    W = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode).astype(np.float64)
    gu = rand_half(2 * n, seed=case + 42)
    x, delta = rand_half(n, seed=case + 43), rand_half(n, seed=case + 44, scale=0.3)
    w = (1.0 + 0.1 * rand_half(n, seed=case + 45).float()).half()
    out_s = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    out_n = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    x_out = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
    with _mode(rk, mode):
        rk.decompress_matvec_silu(comp.cuda(), cb.cuda(), gu.cuda(), out_s)
        rk.decompress_matvec_rmsnorm(comp.cuda(), cb.cuda(), x.cuda(), delta.cuda(), w.cuda(), x_out, out_n, eps=1e-5)
    g, u = gu[:n].double(), gu[n:].double()
    act = (g / (1.0 + torch.exp(-g))).half().double() * u           # the gate is rounded to fp16 before the product
    assert rel_l2(np_f16(out_s), W @ act.half().double().numpy()) < 2 * REL_L2_TOL
    r = (x.float() + delta.float()).half()
    assert torch.equal(x_out.cpu().view(torch.int16), r.view(torch.int16))
    rd = r.double()
    h = ((rd * torch.rsqrt((rd * rd).mean() + 1e-5)).half().double() * w.double()).half().double()
    assert rel_l2(np_f16(out_n), W @ h.numpy()) < 2 * REL_L2_TOL

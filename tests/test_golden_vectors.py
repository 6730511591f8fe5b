"""The committed vectors of tests/golden/vectors_small.npz: the oracle must still reproduce them
(CPU), and the HIP kernels must reproduce them through the C ABI (GPU): decoded weights bit for bit,
products within rel-L2 1e-3."""
import os

import numpy as np
import pytest
import torch

from util import rel_l2

HERE = os.path.dirname(os.path.abspath(__file__))
REL_L2_TOL = 1e-3


@pytest.fixture(scope="module")
def vec():
    with np.load(os.path.join(HERE, "golden", "vectors_small.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def f16(a):
    return np.ascontiguousarray(a).view(np.float16)


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a).view(dtype)).cuda()


# ------------------------------------------------------------------------------- oracle (CPU)

@pytest.mark.parametrize("mode", [0, 1])
def test_oracle_reproduces_the_vectors(oracle, vec, mode):
    got = oracle.decompress(vec["decompress.comp"], f16(vec["decompress.codebook"]), mode=mode)
    assert np.array_equal(got.view(np.uint16), vec[f"decompress.out.mode{mode}"])
    for name, S in (("matvec_s6", 6), ("matvec_s8_ragged", 8)):
        W = vec[f"{name}.W.mode{mode}"]
        m, n = W.shape
        cb = f16(vec[f"{name}.codebook"])
        assert np.array_equal(oracle.matvec_dense(vec[f"{name}.comp"], cb, m, n, S, mode=mode).view(np.uint16), W)
        y = oracle.matvec(vec[f"{name}.comp"], cb, f16(vec[f"{name}.x"]), m, S, mode=mode)
        assert np.array_equal(y, vec[f"{name}.y.mode{mode}"])
        # the stored product is the double-precision product of the stored weights
        assert rel_l2(f16(W).astype(np.float64) @ f16(vec[f"{name}.x"]).astype(np.float64), y) < 1e-12
    for name, L in (("matvec_t_16", 16), ("matvec_t_14", 14)):
        W = vec[f"{name}.W.mode{mode}"]
        m, n = W.shape
        cb = f16(vec[f"{name}.codebook"])
        assert np.array_equal(oracle.matvec_t_dense(vec[f"{name}.comp"], cb, m, n, L, mode=mode).view(np.uint16), W)
        y = oracle.matvec_t(vec[f"{name}.comp"], cb, f16(vec[f"{name}.x"]), m, L, mode=mode)
        assert np.array_equal(y, vec[f"{name}.y.mode{mode}"])
        assert rel_l2(f16(W).astype(np.float64) @ f16(vec[f"{name}.x"]).astype(np.float64), y) < 1e-12
    for name, S, bits in (("bits3", 8, 3), ("bits4", 6, 4)):
        W = vec[f"{name}.W.mode{mode}"]
        m, n = W.shape
        got = oracle.bits_dense(vec[f"{name}.comp"], f16(vec[f"{name}.codebook"]), m, n, S, bits, mode=mode)
        assert np.array_equal(got.view(np.uint16), W)


def test_oracle_reproduces_the_hadamard_vector(oracle, vec):
    y = oracle.sign_hadamard(f16(vec["hadamard.x"]), f16(vec["hadamard.signs"]), 256)
    assert np.array_equal(y, vec["hadamard.y"])


# --------------------------------------------------------------------------------- kernels (GPU)

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


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [0, 1])
def test_kernels_reproduce_the_vectors(rk, vec, mode):
    print(f"\n[case] golden vectors, mode {mode}", flush=True)
    with _mode(rk, mode):
        want = vec[f"decompress.out.mode{mode}"]
        out = torch.zeros(want.shape, dtype=torch.float16, device="cuda")
        rk.decompress(dev(vec["decompress.comp"], np.int32), dev(vec["decompress.codebook"], np.float16), out)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want)

        for name, S in (("matvec_s6", 6), ("matvec_s8_ragged", 8)):
            Wn = vec[f"{name}.W.mode{mode}"]
            m, n = Wn.shape
            comp, cb = dev(vec[f"{name}.comp"], np.int32), dev(vec[f"{name}.codebook"], np.float16)
            W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
            rk.matvec_dense(comp, cb, W, S)
            assert np.array_equal(W.cpu().numpy().view(np.uint16), Wn)
            y = torch.zeros(m, dtype=torch.float16, device="cuda")
            c3 = comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp
            getattr(rk, f"decompress_matvec_16_{S}_1")(c3, cb, dev(vec[f"{name}.x"], np.float16), y)
            assert rel_l2(y.cpu().numpy(), vec[f"{name}.y.mode{mode}"]) < REL_L2_TOL

        for name, L in (("matvec_t_16", 16), ("matvec_t_14", 14)):
            Wn = vec[f"{name}.W.mode{mode}"]
            m, n = Wn.shape
            comp, cb = dev(vec[f"{name}.comp"], np.int32), dev(vec[f"{name}.codebook"], np.float16)
            W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
            rk.matvec_t_dense(comp, cb, W, L)
            assert np.array_equal(W.cpu().numpy().view(np.uint16), Wn)
            y = torch.zeros(m, dtype=torch.float16, device="cuda")     # the op adds to out
            getattr(rk, f"decompress_matvec_t_{L}")(comp, cb, dev(vec[f"{name}.x"], np.float16), y)
            assert rel_l2(y.cpu().numpy(), vec[f"{name}.y.mode{mode}"]) < REL_L2_TOL

        for name, bits in (("bits3", 3), ("bits4", 4)):
            Wn = vec[f"{name}.W.mode{mode}"]
            m, n = Wn.shape
            comp, cb = dev(vec[f"{name}.comp"], np.int32), dev(vec[f"{name}.codebook"], np.float16)
            W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
            rk.matvec_bits_dense(comp, cb, W, bits)
            assert np.array_equal(W.cpu().numpy().view(np.uint16), Wn)
            y = torch.zeros(m, dtype=torch.float16, device="cuda")
            rk.decompress_matvec_bits(comp, cb, dev(vec[f"{name}.x"], np.float16), y, bits)
            assert rel_l2(y.cpu().numpy(), vec[f"{name}.y.mode{mode}"]) < REL_L2_TOL


@pytest.mark.gpu
def test_hadamard_kernel_reproduces_the_vector(rk, vec):
    print("\n[case] golden vector, sign-Hadamard", flush=True)
    x, s = dev(vec["hadamard.x"], np.float16), dev(vec["hadamard.signs"], np.float16)
    out = torch.zeros_like(x)
    rk.sign_hadamard(x, s, out, block=256)
    assert rel_l2(out.cpu().numpy(), vec["hadamard.y"]) < REL_L2_TOL

"""rptc_lite_dequantize on the GPU against the CPU restatement of rptc_lite.py:63-73 (orc_lite_dequantize), bit for bit:
every output is an entry of the alphabet, so float bits are compared, not values."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    assert rptc_kernels.library().rptc_init() == 0
    return rptc_kernels


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def _want(oracle, alphabet, L, S, R, sym):
    return np.stack([oracle.lite_dequantize(alphabet, L, S, R, np.ascontiguousarray(row)) for row in sym])


# (L, S, R, V): the reference's own setting first (rptc_lite.py:141-146), then other symbol widths (R that does not
# divide 32 included: the oldest symbol is cut by the register's end), a single output per step, V that is no pair
CONFIGS = [(16, 9, 4, 2), (16, 9, 2, 2), (12, 8, 3, 1), (20, 10, 5, 3), (16, 8, 1, 2), (31, 16, 16, 8), (9, 9, 7, 2)]


@pytest.mark.parametrize("L,S,R,V", CONFIGS)
@pytest.mark.parametrize("rows,length", [(1, 1), (3, 7), (2, 1024), (5, 2049), (1, 100003)])
def test_lite_dequantize_equals_the_oracle(rk, oracle, L, S, R, V, rows, length):
    g = np.random.default_rng(1000 * L + 10 * R + length)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    sym = g.integers(0, 1 << R, (rows, length), dtype=np.int32)
    out, ms = rk.lite_dequantize(torch.from_numpy(alphabet).cuda(), L, S, R, torch.from_numpy(sym).cuda(), timed=True)
    assert ms > 0 and out.shape == (rows, length, V) and out.dtype == torch.float32
    want = _want(oracle, alphabet, L, S, R, sym)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_lite_dequantize_of_one_sequence_and_of_the_reference_batch(rk, oracle):
    """A 1-D sequence returns [length, V]; the reference's evaluation batch (rptc_lite.py:122: 2^20 / T sequences of
    T = 1024 steps) in one call, more sequences than the launch has rows of workgroups."""
    L, S, R, V, T = 16, 9, 4, 2, 1024
    g = np.random.default_rng(42)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    a = torch.from_numpy(alphabet).cuda()
    one = g.integers(0, 1 << R, T, dtype=np.int32)
    out, _ = rk.lite_dequantize(a, L, S, R, torch.from_numpy(one).cuda())
    assert out.shape == (T, V)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.lite_dequantize(alphabet, L, S, R, one).view(np.uint32))
    rows = 70000                                   # > 65535 sequences: the launch strides over them
    sym = g.integers(0, 1 << R, (rows, 64), dtype=np.int32)
    out, _ = rk.lite_dequantize(a, L, S, R, torch.from_numpy(sym).cuda())
    got = out.cpu().numpy()
    pick = np.concatenate([np.arange(0, 40), np.arange(65500, 65600), np.arange(rows - 40, rows)])
    assert np.array_equal(got[pick].view(np.uint32), _want(oracle, alphabet, L, S, R, sym[pick]).view(np.uint32))
    # every output is an alphabet entry chosen by the last L bits: the same window gives the same output in any row
    states = np.zeros((rows, 64), dtype=np.int64)
    st = np.zeros(rows, dtype=np.int64)
    for t in range(64):
        st = ((st << R) | sym[:, t]) & 0xFFFF
        states[:, t] = st
    flat_s, flat_o = states.reshape(-1), got.reshape(-1, V).view(np.uint64).reshape(-1)
    order = np.argsort(flat_s, kind="stable")
    s_sorted, o_sorted = flat_s[order], flat_o[order]
    same_state = s_sorted[1:] == s_sorted[:-1]
    assert np.array_equal(o_sorted[1:][same_state], o_sorted[:-1][same_state])


def test_lite_dequantize_uses_symbols_as_the_reference_does(rk, oracle):
    """A symbol outside [0, 2^R) is OR-ed into the register with all its bits (rptc_lite.py:65), negative ones
    included, and spoils the steps behind it until it has left the register."""
    L, S, R, V = 16, 9, 4, 2
    g = np.random.default_rng(7)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    sym = g.integers(0, 1 << R, (2, 300), dtype=np.int32)
    sym[0, 17], sym[0, 200], sym[1, 0] = -5, 0x12345, -(1 << 31)
    out, _ = rk.lite_dequantize(torch.from_numpy(alphabet).cuda(), L, S, R, torch.from_numpy(sym).cuda())
    assert np.array_equal(out.cpu().numpy().view(np.uint32), _want(oracle, alphabet, L, S, R, sym).view(np.uint32))


def test_lite_dequantize_rejects_bad_arguments(rk):
    lib = rk.library()
    a = torch.zeros((512, 2), dtype=torch.float32, device="cuda")
    q = torch.zeros((2, 64), dtype=torch.int32, device="cuda")
    o = torch.zeros((2, 64, 2), dtype=torch.float32, device="cuda")
    args = lambda **kw: [kw.get("a", a.data_ptr()), kw.get("L", 16), kw.get("S", 9), kw.get("R", 4), kw.get("V", 2),
                         kw.get("q", q.data_ptr()), kw.get("rows", 2), kw.get("length", 64), kw.get("o", o.data_ptr()), None, None]
    assert lib.rptc_lite_dequantize(*args()) == 0
    assert lib.rptc_lite_dequantize(*args(a=None)) == -1
    assert lib.rptc_lite_dequantize(*args(L=8)) == -2          # L < S
    assert lib.rptc_lite_dequantize(*args(L=32)) == -2
    assert lib.rptc_lite_dequantize(*args(R=0)) == -2
    assert lib.rptc_lite_dequantize(*args(R=17)) == -2
    assert lib.rptc_lite_dequantize(*args(V=9)) == -2
    assert lib.rptc_lite_dequantize(*args(rows=0)) == -2
    assert lib.rptc_lite_dequantize(*args(o=o.data_ptr() + 4)) == -3
    with pytest.raises(RuntimeError):
        rk.lite_dequantize(a, 16, 8, 4, q)                      # alphabet.size(0) != 1 << S
    with pytest.raises(RuntimeError):
        rk.lite_dequantize(a, 16, 9, 4, q.to(torch.int64))
    torch.cuda.synchronize()

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


# ------------------------------------------------------------------ the search (rptc_lite.py:19-60)

@pytest.mark.parametrize("S", [9, 8, 5])
@pytest.mark.parametrize("rows,steps,weights", [(1, 1, "none"), (3, 17, "own"), (2, 64, "shared"), (1, 200, "none")])
def test_lite_quantize_equals_the_oracle(rk, oracle, S, rows, steps, weights):
    """`rptc_lite_viterbi` against the CPU restatement of rptc_lite.quantize, bit for bit: symbols, cost (every sum is
    fp32 in the same order, so the path and its price are the oracle's) — and the decoder's output of the symbols has
    that price."""
    L, R, V = 16, 4, 2
    g = np.random.default_rng(100 * S + steps)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    samples = g.standard_normal((rows, steps, V)).astype(np.float32)
    imp = None
    if weights == "own":
        imp = (g.random((rows, steps, V)) + 0.25).astype(np.float32)
    elif weights == "shared":
        imp = (g.random((steps, V)) + 0.25).astype(np.float32)
    a = torch.from_numpy(alphabet).cuda()
    q, cost = rk.lite_quantize(a, L, S, R, None if imp is None else torch.from_numpy(imp).cuda(), torch.from_numpy(samples).cuda())
    assert q.shape == (rows, steps) and q.dtype == torch.int32 and cost.shape == (rows,)
    for r in range(rows):
        w = None if imp is None else (imp if imp.ndim == 2 else imp[r])
        want_q, want_cost = oracle.lite_quantize(alphabet, L, S, R, w, samples[r])
        assert np.array_equal(q[r].cpu().numpy(), want_q), (r, S, steps)
        assert cost[r].cpu().numpy().view(np.uint32) == np.float32(want_cost).view(np.uint32)
    deq, _ = rk.lite_dequantize(a, L, S, R, q)
    ww = np.ones_like(samples) if imp is None else np.broadcast_to(imp, samples.shape)
    price = (ww.astype(np.float64) * (samples.astype(np.float64) - deq.cpu().numpy()) ** 2).sum(axis=(1, 2))
    assert np.allclose(price, cost.cpu().numpy(), rtol=1e-4, atol=1e-5)


def test_lite_quantize_of_one_sequence_and_the_reference_length(rk, oracle):
    """A 2-D `samples` returns a 1-D sequence and a scalar loss, as the reference does; T = 1024 steps is the length its
    driver trains and evaluates on (rptc_lite.py:141)."""
    L, S, R, V, T = 16, 9, 4, 2, 1024
    g = np.random.default_rng(3)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    samples = g.standard_normal((T, V)).astype(np.float32)
    q, cost = rk.lite_quantize(torch.from_numpy(alphabet).cuda(), L, S, R, torch.ones((T, V), device="cuda"), torch.from_numpy(samples).cuda())
    assert q.shape == (T,) and cost.dim() == 0
    want_q, want_cost = oracle.lite_quantize(alphabet, L, S, R, None, samples)
    assert np.array_equal(q.cpu().numpy(), want_q)
    assert abs(float(cost) - float(want_cost)) <= 1e-6 * float(want_cost)
    # a 2-bit-per-value code of unit Gaussians: the distortion sits a little above the rate-distortion bound 2^-4
    assert 0.06 < float(cost) / (T * V) < 0.12


def test_lite_quantize_rejects_what_the_kernel_is_not_built_for(rk):
    a = torch.zeros((512, 2), dtype=torch.float32, device="cuda")
    x = torch.zeros((8, 2), dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(a, 20, 9, 4, None, x)                  # L
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(a, 16, 9, 2, None, x)                  # R
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(torch.zeros((1024, 2), dtype=torch.float32, device="cuda"), 16, 10, 4, None, x)     # S
    with pytest.raises(RuntimeError):
        rk.lite_quantize(a, 16, 8, 4, None, x)                  # alphabet.size(0) != 1 << S
    with pytest.raises(RuntimeError):
        rk.lite_quantize(a, 16, 9, 4, torch.zeros((7, 2), dtype=torch.float32, device="cuda"), x)
    torch.cuda.synchronize()

"""rptc_lite_viterbi on the GPU against the CPU restatement of rptc_lite.quantize (rptc_lite.py:19-60), bit for bit: the
search's sums are fp32 in one fixed order on both sides, so symbols and cost must be identical."""
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


@pytest.mark.parametrize("L,S,R,V,rows,steps,weights", [(16, 10, 4, 2, 2, 9, "own"), (16, 9, 2, 2, 1, 12, "none"), (12, 8, 4, 3, 3, 40, "shared"),
                                                         (8, 8, 8, 1, 2, 5, "own"), (14, 6, 1, 4, 1, 33, "none"), (20, 9, 4, 2, 1, 3, "own"),
                                                         (4, 2, 2, 2, 5, 100, "shared")])
def test_lite_quantize_with_other_parameters_equals_the_oracle(rk, oracle, L, S, R, V, rows, steps, weights):
    """Parameters other than the reference driver's go through the plain kernel (path costs in the scratch buffer): the
    same symbols and cost as the CPU restatement, bit for bit, and the decoder's output of the symbols has that price."""
    g = np.random.default_rng(1000 * L + 10 * R + V)
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
        assert np.array_equal(q[r].cpu().numpy(), want_q), (r, L, S, R, V)
        assert cost[r].cpu().numpy().view(np.uint32) == np.float32(want_cost).view(np.uint32)
    deq, _ = rk.lite_dequantize(a, L, S, R, q)
    ww = np.ones_like(samples) if imp is None else np.broadcast_to(imp, samples.shape)
    price = (ww.astype(np.float64) * (samples.astype(np.float64) - deq.cpu().numpy().reshape(samples.shape)) ** 2).sum(axis=(1, 2))
    assert np.allclose(price, cost.cpu().numpy(), rtol=1e-4, atol=1e-5)


def test_lite_quantize_rejects_what_the_kernels_are_not_built_for(rk):
    a = torch.zeros((512, 2), dtype=torch.float32, device="cuda")
    x = torch.zeros((8, 2), dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(torch.zeros((2, 2), dtype=torch.float32, device="cuda"), 21, 1, 4, None, x)      # L
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(a, 16, 9, 16, None, x)                 # R
    with pytest.raises(RuntimeError, match="status -5"):
        rk.lite_quantize(torch.zeros((512, 5), dtype=torch.float32, device="cuda"), 16, 9, 4, None,
                         torch.zeros((8, 5), dtype=torch.float32, device="cuda"))                          # V
    with pytest.raises(RuntimeError):
        rk.lite_quantize(a, 16, 8, 4, None, x)                  # alphabet.size(0) != 1 << S
    with pytest.raises(RuntimeError):
        rk.lite_quantize(a, 16, 9, 4, torch.zeros((7, 2), dtype=torch.float32, device="cuda"), x)
    torch.cuda.synchronize()

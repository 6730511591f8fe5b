"""rptc_decompress_matvec_chain on the GPU: a chain of independent fused decode + mat-vecs in one launch.  Every layer's
output is held to the double-precision product of the bit-exact dense matrix (rel-L2 1e-3, the mat-vec's bar) on its
input, to the per-launch kernel on the same input, and to itself from run to run (bit for bit).  Chains with
dependencies are refused by the library (RPTC_EDEPEND) and run by `MatvecChain` as one launch per layer."""
import ctypes

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
    assert rptc_kernels.library().rptc_init() == 0
    return rptc_kernels


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def dense_of(rk, comp, cb, m, n, S, mode):
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        rk.matvec_dense(comp, cb, W, S)
    finally:
        rk.set_carry_mode(prev)
    return W


def check_layer(rk, comp, cb, x, out, S, mode):
    m, n = out.numel(), x.numel()
    W = dense_of(rk, comp, cb, m, n, S, mode)
    want = (W.double() @ x.double()).cpu().numpy()
    assert rel_l2(np_f16(out), want) < REL_L2_TOL
    # the per-launch kernel on the same input (another order of the same fp32 sums)
    y = torch.zeros(m, dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        getattr(rk, f"decompress_matvec_16_{S}_1")(comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp, cb, x, y)
    finally:
        rk.set_carry_mode(prev)
    assert rel_l2(np_f16(out), np_f16(y).astype(np.float64)) < REL_L2_TOL


SHAPES = [(64, 2048), (33, 4096 + 768), (7, 704), (512, 6144), (300, 64), (1024, 2048 + 64), (5, 16384), (2000, 1984)]


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("S", [6, 8])
def test_chain_of_independent_layers(rk, oracle, S, mode):
    """Layers of many shapes (ragged rows, odd row counts, fewer rows than workgroups, the longest row) with
    inputs and outputs of their own: nothing orders them, so waves run from one into the next."""
    cb = rand_half(2 << S, seed=5).cuda()
    layers = []
    for i, (m, n) in enumerate(SHAPES * 2):
        comp = rand_codes(m * n // 16, seed=100 + i).cuda()
        x = rand_half(n, seed=200 + i).cuda()
        out = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
        layers.append((comp, x, out))
    chain = rk.MatvecChain(layers, cb)
    chain.run(carry_mode=mode)
    assert chain.one_launch
    first = [out.clone() for _, _, out in layers]
    for comp, x, out in layers:
        assert not torch.isnan(out).any()
        check_layer(rk, comp, cb, x, out, S, mode)
    # decoded weights through the fused path, bit for bit: one-hot activations read single matrix entries
    m, n = SHAPES[1]
    comp = layers[1][0]
    Wd = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode)
    cols = [0, 1, 63, 64, 2047, 2048, 4095, 4096, n - 1]
    hot = []
    for c in cols:
        x = torch.zeros(n, dtype=torch.float16, device="cuda")
        x[c] = 1.0
        hot.append((comp, x, torch.zeros(m, dtype=torch.float16, device="cuda")))
    rk.MatvecChain(hot, cb).run(carry_mode=mode)
    for c, (_, _, out) in zip(cols, hot):
        assert np.array_equal(np_f16(out).astype(np.float32), Wd[:, c].astype(np.float32))
    # again: every sum has a fixed order, so the bits repeat
    for _, _, out in layers:
        out.fill_(float("nan"))
    chain.run(carry_mode=mode)
    assert chain.one_launch
    for (_, _, out), ref in zip(layers, first):
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("mode", [0, 1])
def test_chain_of_dependent_layers_at_the_llama_shapes(rk, mode):
    """out of one layer is the next one's input (4096 -> 4096 -> 11008 -> 4096 -> 4096): the library refuses the one-launch
    form and the chain runs as a launch per layer, in order.  Each layer is checked on the input the chain gave it."""
    S = 8
    cb = (rand_half(2 << S, seed=6).float() * 0.02).half().cuda()       # keeps the activations in fp16 range
    dims = [4096, 4096, 11008, 4096, 4096]
    bufs = [rand_half(dims[0], seed=7).cuda()] + [torch.full((d,), float("nan"), dtype=torch.float16, device="cuda") for d in dims[1:]]
    layers = []
    for i in range(len(dims) - 1):
        n, m = dims[i], dims[i + 1]
        layers.append((rand_codes(m * n // 16, seed=300 + i).cuda(), bufs[i], bufs[i + 1]))
    chain = rk.MatvecChain(layers, cb)
    assert not chain.one_launch
    for rep in range(3):
        for b in bufs[1:]:
            b.fill_(float("nan"))
        chain.run(carry_mode=mode)
        for comp, x, out in layers:
            assert not torch.isnan(out).any()
            check_layer(rk, comp, cb, x, out, S, mode)
        if rep == 0:
            first = [b.clone() for b in bufs[1:]]
        else:
            for b, ref in zip(bufs[1:], first):
                assert torch.equal(b.view(torch.int16), ref.view(torch.int16))


def test_chain_orders_layers_that_share_a_buffer(rk):
    """Two layers write the same output (the later one wins), and a third reads an input that an earlier one
    overwrites afterwards (it must read the old contents): the plan finds the hazards from the addresses and the
    layers run as launches in order."""
    S, m, n = 8, 1024, 2048
    cb = rand_half(2 << S, seed=8).cuda()
    c = [rand_codes(m * n // 16, seed=400 + i).cuda() for i in range(4)]
    x0, x1 = rand_half(n, seed=9).cuda(), rand_half(n, seed=10).cuda()
    shared = torch.zeros(m, dtype=torch.float16, device="cuda")
    a = torch.zeros(n, dtype=torch.float16, device="cuda")
    layers = [(c[0], x0, shared), (c[1], x1, shared)]
    chain = rk.MatvecChain(layers, cb)
    assert not chain.one_launch
    chain.run()
    y = torch.zeros(m, dtype=torch.float16, device="cuda")
    rk.decompress_matvec_16_8_1(c[1].reshape(1, m, 128), cb, x1, y)
    assert rel_l2(np_f16(shared), np_f16(y).astype(np.float64)) < REL_L2_TOL
    # write after read: layer 0 reads `a`, layer 1 overwrites `a` (square layers)
    m2 = n2 = 2048
    c2 = [rand_codes(m2 * n2 // 16, seed=500 + i).cuda() for i in range(2)]
    a.copy_(rand_half(n2, seed=11).cuda())
    a_before = a.clone()
    out0 = torch.zeros(m2, dtype=torch.float16, device="cuda")
    rk.MatvecChain([(c2[0], a, out0), (c2[1], x0, a)], cb).run()
    y0 = torch.zeros(m2, dtype=torch.float16, device="cuda")
    rk.decompress_matvec_16_8_1(c2[0].reshape(1, m2, 128), cb, a_before, y0)
    assert rel_l2(np_f16(out0), np_f16(y0).astype(np.float64)) < REL_L2_TOL
    y1 = torch.zeros(m2, dtype=torch.float16, device="cuda")
    rk.decompress_matvec_16_8_1(c2[1].reshape(1, m2, 128), cb, x0, y1)
    assert rel_l2(np_f16(a), np_f16(y1).astype(np.float64)) < REL_L2_TOL


def test_long_chain_at_the_headline_shape(rk):
    """200 independent 4096 x 11008 layers over 8 streams and 3 activation vectors (the two activation images and the
    two sets of partial sums of the loop go round many times); outputs of layers with equal inputs are equal bit for
    bit."""
    S = 8
    cb = rand_half(2 << S, seed=12).cuda()
    m, n = 4096, 11008
    comps = [rand_codes(m * n // 16, seed=600 + i).cuda() for i in range(8)]
    xs = [rand_half(n, seed=700 + i).cuda() for i in range(3)]
    outs = [torch.full((m,), float("nan"), dtype=torch.float16, device="cuda") for _ in range(200)]
    layers = [(comps[i % 8], xs[i % 3], outs[i]) for i in range(200)]
    chain = rk.MatvecChain(layers, cb)
    chain.run()
    assert chain.one_launch
    for i in range(24):
        check_layer(rk, comps[i % 8], cb, xs[i % 3], outs[i], S, 0)
    for i in range(24, 200):
        assert torch.equal(outs[i].view(torch.int16), outs[i % 24].view(torch.int16))


@pytest.mark.parametrize("count", [1, 2, 3])
def test_short_chains(rk, count):
    """One, two and three independent layers: the loop that serves such chains requests a layer ahead and sums the rows a
    layer behind, so its first and last iterations are special cases."""
    S = 8
    cb = rand_half(2 << S, seed=21).cuda()
    shapes = [(300, 4096 + 64), (64, 2048), (1024, 704)][:count]
    layers = []
    for i, (m, n) in enumerate(shapes):
        layers.append((rand_codes(m * n // 16, seed=900 + i).cuda(), rand_half(n, seed=910 + i).cuda(),
                       torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")))
    chain = rk.MatvecChain(layers, cb)
    for mode in (0, 1):
        chain.run(carry_mode=mode)
        assert chain.one_launch
        for comp, x, out in layers:
            assert not torch.isnan(out).any()
            check_layer(rk, comp, cb, x, out, S, mode)


def test_chain_with_four_elements_a_wave(rk):
    """8192 x 8192 layers: a workgroup has 64 stream elements of a layer, four a wave (the variant of the loop that holds
    four), and 12288 x 4096 beside it (three)."""
    S = 8
    cb = rand_half(2 << S, seed=22).cuda()
    layers = []
    for i, (m, n) in enumerate([(8192, 8192), (12288, 4096), (8192, 8192)]):
        layers.append((rand_codes(m * n // 16, seed=920 + i).cuda(), rand_half(n, seed=930 + i).cuda(),
                       torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")))
    chain = rk.MatvecChain(layers, cb)
    chain.run(carry_mode=1)
    assert chain.one_launch
    first = [out.clone() for _, _, out in layers]
    for comp, x, out in layers:
        check_layer(rk, comp, cb, x, out, S, 1)
    chain.run(carry_mode=1)
    for (_, _, out), ref in zip(layers, first):
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("seed", range(6))
def test_chain_of_random_shapes(rk, seed):
    """Eight independent layers of random shapes (any row count up to 3000, any multiple of 64 columns up to 12800: ragged
    slabs of every width, row blocks that end early, layers with fewer rows than workgroups), S and carry mode by seed."""
    rng = np.random.default_rng(1000 + seed)
    S, mode = (6, 8)[seed & 1], (seed >> 1) & 1
    cb = rand_half(2 << S, seed=40 + seed).cuda()
    layers = []
    for i in range(8):
        m, n = int(rng.integers(1, 3001)), 64 * int(rng.integers(1, 201))
        layers.append((rand_codes(m * n // 16, seed=1100 + 10 * seed + i).cuda(), rand_half(n, seed=1200 + 10 * seed + i).cuda(),
                       torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")))
    chain = rk.MatvecChain(layers, cb)
    chain.run(carry_mode=mode)
    assert chain.one_launch
    for comp, x, out in layers:
        assert not torch.isnan(out).any()
        check_layer(rk, comp, cb, x, out, S, mode)


def test_chain_rejects_bad_arguments(rk):
    lib = rk.library()
    cb = torch.zeros(512, dtype=torch.float16, device="cuda")
    ok = (torch.zeros(64 * 2048 // 16, dtype=torch.int32, device="cuda"), torch.zeros(2048, dtype=torch.float16, device="cuda"),
          torch.zeros(64, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError):
        rk.MatvecChain([], cb)
    chain = rk.MatvecChain([ok], cb)
    assert chain.one_launch
    assert lib.rptc_decompress_matvec_chain(None, cb.data_ptr(), 8, 0, None, None) == -1
    assert lib.rptc_decompress_matvec_chain(ctypes.byref(chain.plan), cb.data_ptr(), 7, 0, None, None) == -2
    assert lib.rptc_decompress_matvec_chain(ctypes.byref(chain.plan), cb.data_ptr(), 8, 3, None, None) == -4
    blank = rk.ChainPlan()
    assert lib.rptc_decompress_matvec_chain(ctypes.byref(blank), cb.data_ptr(), 8, 0, None, None) == -2
    assert lib.rptc_chain_desc_bytes(None, 1) == -1


def plan_status(rk, layers):
    arr = (rk.ChainLayer * len(layers))()
    for i, (c, x, out) in enumerate(layers):
        arr[i] = rk.ChainLayer(c.data_ptr(), x.data_ptr(), out.data_ptr(), out.numel(), x.numel())
    lib = rk.library()
    need = lib.rptc_chain_desc_bytes(arr, len(layers))
    assert need > 0
    desc = torch.zeros(need + 256, dtype=torch.uint8, device="cuda")
    plan = rk.ChainPlan()
    return lib.rptc_chain_plan(arr, len(layers), (desc.data_ptr() + 255) & ~255, need, ctypes.byref(plan), None)


def test_chain_plan_refuses_dependent_layers_and_layers_too_large(rk):
    """The C ABI itself: RPTC_EDEPEND (-8) when an output overlaps anything a layer of the chain reads or another layer
    writes, RPTC_ELIMIT (-5) when a layer does not fit the one-launch form; `MatvecChain` then launches per layer."""
    m = n = 2048
    comp = [torch.zeros(m * n // 16, dtype=torch.int32, device="cuda") for _ in range(2)]
    a, b, c = (torch.zeros(n, dtype=torch.float16, device="cuda") for _ in range(3))
    assert plan_status(rk, [(comp[0], a, b), (comp[1], a, c)]) == 0
    assert plan_status(rk, [(comp[0], a, b), (comp[1], b, c)]) == -8           # read after write
    assert plan_status(rk, [(comp[0], a, b), (comp[1], c, a)]) == -8           # write after read
    assert plan_status(rk, [(comp[0], a, b), (comp[1], c, b)]) == -8           # write after write
    assert plan_status(rk, [(comp[0], a, a)]) == -8                            # a layer's output is its own input
    assert plan_status(rk, [(comp[0], a, comp[1].view(torch.float16)[:m]), (comp[1], a, c)]) == -8    # output inside a stream
    half = b[:m // 2]
    assert plan_status(rk, [(comp[0][: m // 2 * n // 16], a, half), (comp[1][: m // 2 * n // 16], a, b[m // 4: m // 4 + m // 2])]) == -8
    # n too long for a thread's two activation registers; 16384 x 8192 has eight stream elements a wave
    long_n = (torch.zeros(4 * 16448 // 16, dtype=torch.int32, device="cuda"), torch.zeros(16448, dtype=torch.float16, device="cuda"),
              torch.zeros(4, dtype=torch.float16, device="cuda"))
    assert plan_status(rk, [long_n]) == -5
    big = (torch.zeros(16384 * 8192 // 16, dtype=torch.int32, device="cuda"), torch.zeros(8192, dtype=torch.float16, device="cuda"),
           torch.zeros(16384, dtype=torch.float16, device="cuda"))
    assert plan_status(rk, [big]) == -5


def test_chain_too_large_for_one_launch_runs_as_launches(rk):
    S, m, n = 8, 16384, 8192
    cb = rand_half(2 << S, seed=31).cuda()
    layers = [(rand_codes(m * n // 16, seed=940 + i).cuda(), rand_half(n, seed=950 + i).cuda(),
               torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")) for i in range(2)]
    chain = rk.MatvecChain(layers, cb)
    assert not chain.one_launch
    chain.run(carry_mode=1)
    for comp, x, out in layers:
        check_layer(rk, comp, cb, x, out, S, 1)

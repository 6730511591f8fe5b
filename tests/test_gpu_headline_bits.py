"""Decoded weights of the FUSED kernels at the headline geometry, bit for bit.

The dense export (a separate kernel) is held to the oracle at full size elsewhere; here the fused decode + mat-vec
itself is: with one-hot activations y[r] = W[r, p] exactly (one product 1.0 * w added to zeros in fp32), so every
launch reads one whole column of the matrix the kernel decodes, for all rows, at the shapes the benchmark runs
(4096 x 11008 and 11008 x 4096 on one workgroup per compute unit: two or three stream elements a wave, a ragged
last slab of 12 lanes).  The columns are chosen through the slot map of inference.cu:215-221,249 so that every slab,
the first and last lane of a row (full and ragged), both values of a pair and every shift group of the 32 steps are
hit.  The same columns go through one rptc_decompress_matvec_chain launch (its loop kernel) over the same stream.
"""
import numpy as np
import pytest
import torch

from util import np_f16, np_u32, rand_codes, rand_half

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


def column_of(n, slab, q, lane, b):
    """Column of value b of the pair that step-slot q of lane `lane` of slab `slab` multiplies (inference.cu:249)."""
    T, Lt, n8 = n // 2048, (n % 2048) // 64, n // 8
    P = 1024 * slab + 32 * q + lane if slab < T else 1024 * T + q * Lt + lane
    i, idx = divmod(P, n8)
    return 8 * idx + 2 * i + b


def probe_columns(n):
    T, Lt = n // 2048, (n % 2048) // 64
    cols = []
    for slab in range(T + (1 if Lt else 0)):
        lanes = 32 if slab < T else Lt
        for lane in sorted({0, 1, lanes // 2, lanes - 1}):
            # slots 0-3 / 28-31 are the steps that read the word in front of the element; the others spread over
            # the four shift groups and both halves of a window register
            for q, b in ((0, 0), (3, 1), (5, 0), (12, 1), (17, 0), (22, 1), (28, 0), (31, 1)):
                cols.append(column_of(n, slab, (q + 7 * slab + lane) % 32, lane, b))
    return sorted(set(cols))


def same_bits(got, want):
    g, w = np.asarray(got).view(np.uint16), np.asarray(want).view(np.uint16)
    nz = (w & 0x7FFF) != 0                      # -0.0 * 1.0 + 0.0 = +0.0 in the accumulator: zeros by value
    return np.array_equal(g[nz], w[nz]) and bool(np.all((g[~nz] & 0x7FFF) == 0))


@pytest.mark.parametrize("m,n,mode", [(4096, 11008, 0), (4096, 11008, 1), (11008, 4096, 0), (11008, 4096, 1)])
def test_fused_kernels_decode_the_headline_layers_bit_exactly(rk, oracle, m, n, mode):
    S = 8
    comp = rand_codes(m * n // 16, seed=42 + mode)
    cb = rand_half(2 << S, seed=43)
    want = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode)
    cols = probe_columns(n)
    assert len(cols) >= 64
    c, cbd = comp.cuda(), cb.cuda()
    c3 = c.reshape(n // 2048, m, 128) if n % 2048 == 0 else c
    prev_timing, prev_mode = rk.set_timing(False), rk.set_carry_mode(mode)
    try:
        # one launch of the drop-in op per column
        x = torch.zeros(n, dtype=torch.float16, device="cuda")
        out = torch.zeros(m, dtype=torch.float16, device="cuda")
        for p in cols:
            x.zero_()
            x[p] = 1.0
            out.fill_(float("nan"))
            rk.decompress_matvec_16_8_1(c3, cbd, x, out)
            assert same_bits(np_f16(out), want[:, p]), f"per-launch kernel, column {p}"
        # the same columns as the layers of one chain launch over the same stream
        xs = torch.zeros((len(cols), n), dtype=torch.float16, device="cuda")
        xs[torch.arange(len(cols)), torch.tensor(cols)] = 1.0
        outs = torch.full((len(cols), m), float("nan"), dtype=torch.float16, device="cuda")
        chain = rk.MatvecChain([(c, xs[i], outs[i]) for i in range(len(cols))], cbd)
        chain.run(carry_mode=mode)
        torch.cuda.synchronize()
        got = np_f16(outs)
        for i, p in enumerate(cols):
            assert same_bits(got[i], want[:, p]), f"chain, column {p}"
    finally:
        rk.set_timing(prev_timing)
        rk.set_carry_mode(prev_mode)

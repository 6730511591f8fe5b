"""The Viterbi search kernel against the CPU restatement of rptc.py:13-71 and against the host-side
search, bit for bit: the same path, the same fp32 cost, the same end state."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available()
    return rptc_kernels


def _case(seed, rows, steps, S, weighted):
    g = np.random.default_rng(seed)
    cb = g.standard_normal(2 << S).astype(np.float16)
    targets = (0.7 * g.standard_normal((rows, steps, 2))).astype(np.float32)
    weights = None
    if weighted == "shared":
        weights = g.uniform(0.25, 4.0, (steps, 2)).astype(np.float32)
    elif weighted == "rows":
        weights = g.uniform(0.25, 4.0, (rows, steps, 2)).astype(np.float32)
    return cb, targets, weights


@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("rows,steps,weighted", [(3, 1, None), (2, 33, None), (2, 64, "shared"), (3, 96, "rows"),
                                                 (1, 300, None)])
def test_viterbi_kernel_equals_the_oracle(rk, oracle, rows, steps, S, weighted):
    from rptc_kernels import quantize
    cb, targets, weights = _case(10 * steps + S, rows, steps, S, weighted)
    table = quantize.decode_table(torch.from_numpy(cb), S).numpy()
    sym, cost, end, ms = rk.viterbi_pairs(torch.from_numpy(targets).cuda(), torch.from_numpy(cb).cuda(),
                                          None if weights is None else torch.from_numpy(weights).cuda())
    assert ms > 0 and sym.dtype == torch.uint8 and sym.shape == (rows, steps)
    sym, cost, end = sym.cpu().numpy(), cost.cpu().numpy(), end.cpu().numpy()
    for r in range(rows):
        w = None if weights is None else (weights if weights.ndim == 2 else weights[r])
        osym, ocost, oend = oracle.viterbi(table, 4, targets[r], w)
        assert np.array_equal(sym[r].astype(np.int32), osym), f"row {r}"
        assert cost[r] == ocost and end[r] == oend


def test_viterbi_kernel_ties_take_the_first_index(rk, oracle):
    """Equal codebook pairs make many paths tie; the kernel resolves every tie as argmin does."""
    from rptc_kernels import quantize
    cb = np.zeros(512, dtype=np.float16)
    cb[::2], cb[1::2] = 0.5, -0.25          # every entry the same pair up to the hash's sign bit
    targets = np.zeros((2, 40, 2), dtype=np.float32)
    targets[1, :, 0] = -0.5                 # row 1 prefers the states whose hash sets the sign
    table = quantize.decode_table(torch.from_numpy(cb), 8).numpy()
    sym, cost, end, _ = rk.viterbi_pairs(torch.from_numpy(targets).cuda(), torch.from_numpy(cb).cuda())
    for r in range(2):
        osym, ocost, oend = oracle.viterbi(table, 4, targets[r])
        assert np.array_equal(sym[r].cpu().numpy().astype(np.int32), osym)
        assert float(cost[r]) == float(ocost) and int(end[r]) == oend


def test_quantize_matrix_on_the_gpu_uses_the_kernel_and_matches_the_host_search(rk, oracle):
    from rptc_kernels import packing, quantize
    g = np.random.default_rng(5)
    m, n, S = 8, 512, 8
    W = g.standard_normal((m, n)).astype(np.float32)
    cb = g.standard_normal(2 << S).astype(np.float16)
    imp = g.uniform(0.5, 2.0, n).astype(np.float32)
    for importance in (None, imp):
        sym_gpu, mse_gpu = quantize.quantize_matrix(torch.from_numpy(W).cuda(), torch.from_numpy(cb).cuda(), S,
                                                    importance=importance)
        sym_cpu, mse_cpu = quantize.quantize_matrix(torch.from_numpy(W), torch.from_numpy(cb), S, importance=importance)
        assert torch.equal(sym_gpu, sym_cpu) and abs(mse_gpu - mse_cpu) < 1e-6
    # and the symbols decode, through the packed stream and the mat-vec kernel's dense export, to the walk
    stream = torch.from_numpy(packing.pack_matvec(sym_gpu.numpy())).cuda()
    Wd = torch.empty((m, n), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(rk.CONTINUOUS)
    try:
        rk.matvec_dense(stream, torch.from_numpy(cb).cuda(), Wd, S)
    finally:
        rk.set_carry_mode(prev)
    walk = quantize.dequantize_symbols(sym_gpu, torch.from_numpy(cb), S)
    assert torch.equal(Wd.cpu().float(), walk)


def test_viterbi_rejects_bad_arguments(rk):
    cb = torch.zeros(512, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        rk.viterbi_pairs(torch.zeros((2, 8, 3), device="cuda"), cb)
    with pytest.raises(RuntimeError):
        rk.viterbi_pairs(torch.zeros((2, 8, 2), device="cuda"), cb[:100])
    with pytest.raises(RuntimeError):
        rk.viterbi_pairs(torch.zeros((2, 8, 2), device="cuda"), cb, torch.zeros((3, 8, 2), device="cuda"))


@pytest.mark.parametrize("L", [16, 14])
@pytest.mark.parametrize("rows,steps,weighted", [(2, 1, None), (2, 50, None), (2, 70, "shared"), (3, 40, "rows"),
                                                 (1, 257, None)])
def test_scalar_viterbi_kernel_equals_the_oracle(rk, oracle, rows, steps, L, weighted):
    """rptc.py:13-71 as it stands: 2 bits a step, one alphabet value a state."""
    g = np.random.default_rng(1000 * L + steps)
    alphabet = g.standard_normal(1 << L).astype(np.float16)
    targets = g.standard_normal((rows, steps)).astype(np.float32)
    weights = None
    if weighted == "shared":
        weights = g.uniform(0.25, 4.0, steps).astype(np.float32)
    elif weighted == "rows":
        weights = g.uniform(0.25, 4.0, (rows, steps)).astype(np.float32)
    sym, cost, end, ms = rk.viterbi_scalar(torch.from_numpy(targets).cuda(), torch.from_numpy(alphabet).cuda(),
                                           None if weights is None else torch.from_numpy(weights).cuda())
    assert ms > 0 and sym.shape == (rows, steps)
    sym, cost, end = sym.cpu().numpy(), cost.cpu().numpy(), end.cpu().numpy()
    table = alphabet.astype(np.float32)
    for r in range(rows):
        w = None if weights is None else (weights if weights.ndim == 1 else weights[r])
        osym, ocost, oend = oracle.viterbi(table, 2, targets[r], w)
        assert np.array_equal(sym[r].astype(np.int32), osym), f"row {r}"
        assert cost[r] == ocost and end[r] == oend


def test_scalar_viterbi_symbols_decode_through_decompress(rk, oracle):
    """Quantize rows for the scalar-LUT stream, pack them, decode with the decompress kernel in CONTINUOUS mode:
    the decoded values are the path's alphabet values (rptc.py:74-85) and their error is the reported cost."""
    from rptc_kernels import packing
    g = np.random.default_rng(3)
    m, n = 4, 2048
    alphabet = g.standard_normal(1 << 16).astype(np.float16)
    W = g.standard_normal((m, n)).astype(np.float32)
    sym, cost, _, _ = rk.viterbi_scalar(torch.from_numpy(W).cuda(), torch.from_numpy(alphabet).cuda())
    stream = torch.from_numpy(packing.pack_rowmajor(sym.cpu().numpy().astype(np.int64))).cuda()
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(rk.CONTINUOUS)
    try:
        rk.decompress(stream, torch.from_numpy(alphabet).cuda(), out)
    finally:
        rk.set_carry_mode(prev)
    What = out.cpu().numpy().astype(np.float64)
    for r in range(m):
        assert np.array_equal(out[r].cpu().numpy(), oracle.dequantize_h(alphabet, sym[r].cpu().numpy().astype(np.int32)))
        assert abs(((W[r] - What[r]) ** 2).sum() - float(cost[r])) < 1e-3 * float(cost[r])
    # 2 bits per weight on a Gaussian source with a random 65536-value alphabet: far below the 1-bit scalar
    # quantizer's 0.36 and above the rate-distortion bound 0.0625
    assert 0.0625 < float(cost.sum()) / (m * n) < 0.12


def test_quantize_matrix_scalar_on_the_gpu_matches_the_host_search(rk):
    from rptc_kernels import quantize
    g = np.random.default_rng(21)
    m, n = 3, 1024
    alphabet = g.standard_normal(1 << 14).astype(np.float16)
    W = g.standard_normal((m, n)).astype(np.float32)
    imp = g.uniform(0.5, 2.0, n).astype(np.float32)
    for importance in (None, imp):
        sym_gpu, mse_gpu = quantize.quantize_matrix_scalar(torch.from_numpy(W).cuda(), torch.from_numpy(alphabet).cuda(),
                                                           importance=importance)
        sym_cpu, mse_cpu = quantize.quantize_matrix_scalar(torch.from_numpy(W), torch.from_numpy(alphabet),
                                                           importance=importance)
        assert torch.equal(sym_gpu, sym_cpu) and abs(mse_gpu - mse_cpu) < 1e-6


def test_viterbi_kernels_on_a_full_length_row(rk, oracle):
    """One row of a 4096-column layer (2048 steps of the pair trellis, 4096 of the scalar one): path, cost and
    end state equal the oracle's after thousands of steps of accumulated fp32 sums."""
    from rptc_kernels import quantize
    g = np.random.default_rng(77)
    cb = g.standard_normal(512).astype(np.float16)
    targets = (0.7 * g.standard_normal((1, 2048, 2))).astype(np.float32)
    sym, cost, end, _ = rk.viterbi_pairs(torch.from_numpy(targets).cuda(), torch.from_numpy(cb).cuda())
    osym, ocost, oend = oracle.viterbi(quantize.decode_table(torch.from_numpy(cb), 8).numpy(), 4, targets[0])
    assert np.array_equal(sym[0].cpu().numpy().astype(np.int32), osym) and float(cost[0]) == float(ocost) and int(end[0]) == oend
    alphabet = g.standard_normal(1 << 16).astype(np.float16)
    row = g.standard_normal((1, 4096)).astype(np.float32)
    sym, cost, end, _ = rk.viterbi_scalar(torch.from_numpy(row).cuda(), torch.from_numpy(alphabet).cuda())
    osym, ocost, oend = oracle.viterbi(alphabet.astype(np.float32), 2, row[0])
    assert np.array_equal(sym[0].cpu().numpy().astype(np.int32), osym) and float(cost[0]) == float(ocost) and int(end[0]) == oend


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("S,rows,steps,weighted", [(8, 2, 1, None), (8, 2, 40, None), (6, 2, 33, "shared"), (8, 2, 25, "rows")])
def test_viterbi_kernel_at_3_and_4_bits_equals_the_oracle(rk, oracle, bits, S, rows, steps, weighted):
    """6 and 8 stream bits per step: 64 and 256 predecessors per state (a group's minimum spans four lanes at 8)."""
    from rptc_kernels import quantize
    cb, targets, weights = _case(100 * bits + steps + S, rows, steps, S, weighted)
    table = quantize.decode_table(torch.from_numpy(cb), S).numpy()
    sym, cost, end, _ = rk.viterbi_pairs(torch.from_numpy(targets).cuda(), torch.from_numpy(cb).cuda(),
                                         None if weights is None else torch.from_numpy(weights).cuda(), bits=bits)
    sym, cost, end = sym.cpu().numpy(), cost.cpu().numpy(), end.cpu().numpy()
    for r in range(rows):
        w = None if weights is None else (weights if weights.ndim == 2 else weights[r])
        osym, ocost, oend = oracle.viterbi(table, 2 * bits, targets[r], w)
        assert np.array_equal(sym[r].astype(np.int32), osym), f"row {r}"
        assert cost[r] == ocost and end[r] == oend


@pytest.mark.parametrize("bits", [3, 4])
def test_quantize_matrix_at_3_and_4_bits_on_the_gpu_matches_the_host_search(rk, bits):
    from rptc_kernels import quantize
    g = np.random.default_rng(40 + bits)
    m, n, S = 4, 256, 8
    W = g.standard_normal((m, n)).astype(np.float32)
    cb = g.standard_normal(2 << S).astype(np.float16)
    sym_gpu, mse_gpu = quantize.quantize_matrix(torch.from_numpy(W).cuda(), torch.from_numpy(cb).cuda(), S, bits=bits)
    sym_cpu, mse_cpu = quantize.quantize_matrix(torch.from_numpy(W), torch.from_numpy(cb), S, bits=bits)
    assert torch.equal(sym_gpu, sym_cpu) and abs(mse_gpu - mse_cpu) < 1e-6


def test_quantize_layer_feeds_the_scalar_lut_kernels(rk):
    """The reference's layer quantizer (quantize_hf.py:120-170) with the search kernel, then its symbols through
    the packers into the reference's two scalar-LUT kernels: decompress reproduces the rounded normalised
    weights bit for bit, decompress_matvec_t_16 their product with a vector."""
    from rptc_kernels import packing, quantize
    from util import rel_l2
    g = torch.Generator().manual_seed(9)
    out_f, in_f, banks = 64, 2048, 2
    W = torch.randn((out_f, in_f), generator=g) * (0.5 + torch.rand((out_f, 1), generator=g)) * 0.02
    h = 0.5 + torch.rand(in_f, generator=g)
    res = quantize.quantize_layer(W.cuda(), h.cuda(), L=16, banks=banks, seed=3)
    err = quantize.evaluate_layer(W.cuda(), res["recon"], h.cuda())
    assert err["frob_rel"] < 0.09 and err["proxy_diag"] < 0.09      # 2 bits/weight; rate-distortion bound 0.0625
    rows = out_f // banks
    x = torch.randn(in_f, generator=g).half().cuda()
    prev = rk.set_carry_mode(rk.CONTINUOUS)
    try:
        for b in range(banks):
            sym = res["symbols"][b * rows:(b + 1) * rows].numpy()
            alphabet = res["alphabets"][b].half().cuda()
            stream = torch.from_numpy(packing.pack_rowmajor(sym)).cuda()
            dec = torch.empty((rows, in_f), dtype=torch.float16, device="cuda")
            rk.decompress(stream, alphabet, dec)
            rounded = (res["recon"][b * rows:(b + 1) * rows] - res["biases_out"][b * rows:(b + 1) * rows] - res["biases_in"]) \
                / res["scales_out"][b * rows:(b + 1) * rows] / res["scales_in"]
            assert torch.allclose(dec.float(), rounded, atol=2e-3, rtol=1e-3)      # recon was put together in fp32
            y = torch.zeros(rows, dtype=torch.float16, device="cuda")
            rk.decompress_matvec_t_16(torch.from_numpy(packing.pack_transposed(sym)).cuda(), alphabet, x, y)
            want = dec.double() @ x.double()
            assert rel_l2(y.float().cpu().numpy(), want.cpu().numpy()) < 2e-3
    finally:
        rk.set_carry_mode(prev)

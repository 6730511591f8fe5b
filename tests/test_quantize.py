"""The Viterbi quantizer: optimal on a trellis small enough to enumerate, consistent with the decoder
the kernels implement, and better than chance on a real-size state space."""
import itertools

import numpy as np
import pytest
import torch

from rptc_kernels import packing, quantize


def test_viterbi_is_optimal_on_a_small_trellis():
    g = torch.Generator().manual_seed(0)
    state_bits, step_bits, steps, rows = 6, 2, 6, 3
    table = torch.randn((1 << state_bits, 2), generator=g)
    targets = torch.randn((rows, steps, 2), generator=g)
    sym, cost = quantize.viterbi_pairs(targets, table, state_bits=state_bits, step_bits=step_bits)
    for r in range(rows):
        best = None
        for seq in itertools.product(range(1 << step_bits), repeat=steps):
            state, c = 0, 0.0
            for t, s in enumerate(seq):
                state = ((state << step_bits) | s) & ((1 << state_bits) - 1)
                c += float(((targets[r, t] - table[state]) ** 2).sum())
            if best is None or c < best[0]:
                best = (c, seq)
        assert abs(best[0] - float(cost[r])) < 1e-4
        # the returned path has the reported cost (ties may pick another optimal path)
        state, c = 0, 0.0
        for t in range(steps):
            state = ((state << step_bits) | int(sym[r, t])) & ((1 << state_bits) - 1)
            c += float(((targets[r, t] - table[state]) ** 2).sum())
        assert abs(c - float(cost[r])) < 1e-4


def test_decode_table_matches_the_oracle_hash(oracle):
    cb = np.random.default_rng(1).standard_normal(512).astype(np.float16)
    table = quantize.decode_table(torch.from_numpy(cb), 8).numpy()
    for s in (0, 1, 0x00B5, 0x1234, 0xBEEF, 0xFFFF, 40000):
        _, e, sign = oracle.hash_window(s, 8)
        w0 = -abs(float(cb[2 * e])) if sign else abs(float(cb[2 * e]))
        assert table[s, 0] == np.float32(w0) and table[s, 1] == np.float32(cb[2 * e + 1])


def test_quantize_matrix_round_trip_through_the_packed_stream(oracle):
    g = np.random.default_rng(2)
    m, n, S = 4, 192, 8
    W = g.standard_normal((m, n)).astype(np.float32)
    cb = g.standard_normal(2 << S).astype(np.float16)
    symbols, mse = quantize.quantize_matrix(torch.from_numpy(W), torch.from_numpy(cb), S)
    assert symbols.shape == (m, n // 2) and int(symbols.max()) < 16
    # the decoder walk, the packed stream decoded by the oracle, and the reported error all agree
    What = quantize.dequantize_symbols(symbols, torch.from_numpy(cb), S).numpy()
    stream = packing.pack_matvec(symbols.numpy())
    Wor = oracle.matvec_dense(stream, cb, m, n, S, mode=oracle.CONTINUOUS).astype(np.float32)
    assert np.array_equal(What, Wor)
    assert abs(((W - What) ** 2).mean() - mse) < 1e-5
    # a 2-bit/weight trellis code with a 256-pair random codebook is far better than random symbols
    rand = quantize.dequantize_symbols(torch.from_numpy(g.integers(0, 16, (m, n // 2))), torch.from_numpy(cb), S).numpy()
    assert mse < 0.25 * ((W - rand) ** 2).mean()
    assert mse < 0.2          # unit-variance Gaussian at 2 bits/weight: rate-distortion bound 0.0625


def test_quantize_matrix_at_3_and_4_bits_round_trips_and_gets_better_with_the_rate(oracle):
    """More bits per step means more successors per state: the decoder walk, the packed stream decoded by the
    oracle and the reported error agree, and the error falls with the rate."""
    g = np.random.default_rng(5)
    m, n, S = 2, 128, 8
    W = g.standard_normal((m, n)).astype(np.float32)
    cb = g.standard_normal(2 << S).astype(np.float16)
    errors = {}
    for bits in (2, 3, 4):
        symbols, mse = quantize.quantize_matrix(torch.from_numpy(W), torch.from_numpy(cb), S, bits=bits)
        assert symbols.shape == (m, n // 2) and int(symbols.max()) < (1 << (2 * bits))
        What = quantize.dequantize_symbols(symbols, torch.from_numpy(cb), S, bits=bits).numpy()
        stream = packing.pack_matvec(symbols.numpy(), bits=bits)
        Wor = oracle.bits_dense(stream, cb, m, n, S, bits, mode=oracle.CONTINUOUS).astype(np.float32)
        assert np.array_equal(What, Wor)
        assert abs(((W - What) ** 2).mean() - mse) < 1e-5
        errors[bits] = mse
    assert errors[4] <= errors[3] <= errors[2]


def _walk_cost(table, step_bits, targets, weights, seq):
    """Cost of one symbol sequence by the decoder walk (rptc.py:74-85), in float64."""
    M = table.shape[0]
    state, c = 0, 0.0
    for t, s in enumerate(seq):
        state = ((state << step_bits) | int(s)) & (M - 1)
        d = targets[t].astype(np.float64) - table[state].astype(np.float64)
        w = np.ones_like(d) if weights is None else weights[t].astype(np.float64)
        c += float((w * d * d).sum())
    return c, state


@pytest.mark.parametrize("L,b,V,steps,weighted", [(4, 2, 1, 6, False), (6, 2, 1, 5, True), (6, 2, 2, 6, False),
                                                  (8, 4, 2, 3, True), (5, 1, 1, 9, False), (4, 4, 2, 3, False)])
def test_oracle_viterbi_is_optimal_by_enumeration(oracle, L, b, V, steps, weighted):
    """Every symbol sequence is tried: the oracle's cost is the smallest, and its path has that cost."""
    g = np.random.default_rng(100 * L + b)
    table = g.standard_normal((1 << L, V)).astype(np.float32)
    targets = g.standard_normal((steps, V)).astype(np.float32)
    weights = g.uniform(0.5, 2.0, (steps, V)).astype(np.float32) if weighted else None
    sym, cost, end = oracle.viterbi(table, b, targets, weights)
    best = min(_walk_cost(table, b, targets, weights, seq)[0] for seq in itertools.product(range(1 << b), repeat=steps))
    assert abs(best - float(cost)) < 1e-5 * max(1.0, best)
    c, state = _walk_cost(table, b, targets, weights, sym)
    assert abs(c - best) < 1e-5 * max(1.0, best) and state == end
    assert sym.min() >= 0 and sym.max() < (1 << b)


def test_oracle_viterbi_tie_rules(oracle):
    """A constant table makes every path cost the same: argmin's first index (rptc.py:27, 62) then picks
    end state 0 and, walking back, the predecessor with d = 0 at every step, i.e. all-zero symbols."""
    table = np.full((1 << 6, 1), 0.25, dtype=np.float32)
    targets = np.zeros((7, 1), dtype=np.float32)
    sym, cost, end = oracle.viterbi(table, 2, targets)
    assert end == 0 and not sym.any() and cost == np.float32(7 * 0.0625)
    # the trellis starts in state 0 (rptc.py:55-56): a table that makes state 0 expensive and state 1
    # free still pays for leaving through the shift register, never starting elsewhere
    table = np.ones((1 << 4, 1), dtype=np.float32)
    table[1] = 0.0
    sym, cost, end = oracle.viterbi(table, 2, np.zeros((1, 1), dtype=np.float32))
    assert list(sym) == [1] and end == 1 and cost == 0.0


def test_torch_viterbi_equals_the_oracle_bit_for_bit(oracle):
    """The host-side search and the C restatement choose the same path and report the same fp32 cost."""
    g = np.random.default_rng(7)
    for (L, b, steps, weighted) in ((8, 4, 12, False), (10, 2, 20, True), (16, 4, 10, True)):
        table = g.standard_normal((1 << L, 2)).astype(np.float32)
        targets = g.standard_normal((2, steps, 2)).astype(np.float32)
        weights = g.uniform(0.5, 2.0, (2, steps, 2)).astype(np.float32) if weighted else None
        sym, cost = quantize.viterbi_pairs(torch.from_numpy(targets), torch.from_numpy(table),
                                           None if weights is None else torch.from_numpy(weights), state_bits=L, step_bits=b)
        for r in range(2):
            osym, ocost, _ = oracle.viterbi(table, b, targets[r], None if weights is None else weights[r])
            assert np.array_equal(sym[r].numpy(), osym) and float(cost[r]) == float(ocost)


def test_scalar_quantizer_equals_the_oracle_and_decodes_through_the_packed_stream(oracle):
    """quantize_matrix_scalar on the CPU: the oracle's path bit for bit (weights 0 on the padding value add
    exact zeros), and the packed row-major stream decodes to the path's alphabet values."""
    g = np.random.default_rng(11)
    m, n, L = 2, 2048, 14
    alphabet = g.standard_normal(1 << L).astype(np.float16)
    W = g.standard_normal((m, n)).astype(np.float32)
    imp = g.uniform(0.5, 2.0, n).astype(np.float32)
    for importance in (None, imp):
        sym, mse = quantize.quantize_matrix_scalar(torch.from_numpy(W), torch.from_numpy(alphabet), importance=importance)
        for r in range(m):
            osym, ocost, _ = oracle.viterbi(alphabet.astype(np.float32), 2, W[r], importance)
            assert np.array_equal(sym[r].numpy(), osym)
    got = oracle.dequantize_h(alphabet, sym[0].numpy().astype(np.int32))
    assert got.shape == (n,)


def test_factorize_is_exact_and_balanced():
    """quantize_hf.py:77-117: the factors reproduce W exactly (that is how N is defined), N has unit row and
    column RMS and zero row and column means at the fixed point, and the balancing steps hold."""
    g = torch.Generator().manual_seed(3)
    out_f, in_f = 48, 80
    W = (torch.randn((out_f, in_f), generator=g) * (0.5 + torch.rand((out_f, 1), generator=g))
         * (0.5 + torch.rand((1, in_f), generator=g)) + 0.3 * torch.randn((out_f, 1), generator=g)
         + 0.2 * torch.randn((1, in_f), generator=g))
    b_out, b_in, s_out, s_in, N = quantize.factorize(W)
    assert torch.allclose(b_out + b_in + s_out * s_in * N, W, atol=1e-5)
    assert torch.allclose((N ** 2).mean(dim=0).sqrt(), torch.ones(in_f), atol=1e-3)
    assert torch.allclose((N ** 2).mean(dim=1).sqrt(), torch.ones(out_f), atol=2e-2)
    assert abs(float(b_out.mean() - b_in.mean())) < 1e-5
    assert abs(float(s_out.log().mean() - s_in.log().mean())) < 1e-4
    # and rows and columns of N are centred (the biases are the means of the scaled residual)
    assert float(N.mean(dim=1).abs().max()) < 2e-2 and float(N.mean(dim=0).abs().max()) < 2e-2


def test_quantile_alphabet_matches_numpy_interp():
    g = np.random.default_rng(4)
    vals = g.standard_normal(1000).astype(np.float32)
    L = 8
    got = np.sort(quantize.quantile_alphabet(torch.from_numpy(vals), L, seed=1).numpy())
    M = 1 << L
    want = np.interp((2 * np.arange(M) + 1) / 2 / M, (2 * np.arange(vals.size) + 1) / 2 / vals.size, np.sort(vals))
    assert np.allclose(got, want, atol=1e-6)


def test_quantize_layer_reconstructs_better_than_a_scalar_quantizer():
    """quantize_hf.py:160-170 end to end on a small layer (CPU search): the reconstruction's relative error at
    2 bits per weight is far below that of rounding to four levels."""
    g = torch.Generator().manual_seed(5)
    out_f, in_f = 16, 128
    W = torch.randn((out_f, in_f), generator=g) * (0.5 + torch.rand((out_f, 1), generator=g))
    h = 0.5 + torch.rand(in_f, generator=g)
    res = quantize.quantize_layer(W, h, L=10, banks=2, seed=1)
    err = quantize.evaluate_layer(W, res["recon"], h)
    assert res["symbols"].shape == (out_f, in_f) and int(res["symbols"].max()) <= 3
    assert err["frob_rel"] < 0.12 and err["proxy_diag"] < 0.12       # 2-bit Lloyd-Max scalar quantizer: 0.1175


def test_evaluate_layer_known_answer():
    """quantize_hf.py:172-185 by hand: W = [[3, 4]], recon = [[2, 2]] -> E = [[1, 2]];
    frob = (1 + 4) / sqrt(9 + 16) = 1 (the reference divides by the norm, not its square);
    proxy_diag with h = [2, 1]: (1*2 + 4*1) / (9*2 + 16*1) = 6 / 34."""
    W = torch.tensor([[3.0, 4.0]])
    recon = torch.tensor([[2.0, 2.0]])
    err = quantize.evaluate_layer(W, recon, torch.tensor([2.0, 1.0]))
    assert err["frob"] == pytest.approx(1.0)
    assert err["frob_rel"] == pytest.approx(5.0 / 25.0)
    assert err["proxy_diag"] == pytest.approx(6.0 / 34.0)


def test_sign_hadamard_rows_is_the_oracle_transform_and_orthogonal(oracle):
    g = np.random.default_rng(6)
    m, n = 3, 768                        # blocks of 256
    W = g.standard_normal((m, n)).astype(np.float16)
    signs = np.where(g.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    got = quantize.sign_hadamard_rows(torch.from_numpy(W.astype(np.float32)), torch.from_numpy(signs)).numpy()
    want = oracle.sign_hadamard(W, signs, 256)
    assert np.allclose(got, want, atol=1e-5)
    assert np.allclose((got ** 2).sum(axis=1), (W.astype(np.float64) ** 2).sum(axis=1), rtol=1e-5)

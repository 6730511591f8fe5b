"""The packers against the decoders' definitions: packed random symbols, decoded by the oracle in
CONTINUOUS mode, must equal a direct walk of the shift register over the symbols."""
import numpy as np
import pytest

from rptc_kernels import packing


def rng(seed):
    return np.random.default_rng(seed)


def test_pack_rowmajor_round_trip(oracle):
    g = rng(1)
    m, n = 3, 4096
    symbols = g.integers(0, 4, (m, n))
    cb = g.standard_normal(65536).astype(np.float16)
    stream = packing.pack_rowmajor(symbols)
    assert stream.shape == (m, n // 16) and stream.dtype == np.int32
    got = oracle.decompress(stream, cb, mode=oracle.CONTINUOUS)
    for r in range(m):
        assert np.array_equal(got[r].view(np.uint16), oracle.dequantize_h(cb, symbols[r]).view(np.uint16))


@pytest.mark.parametrize("L", [14, 16])
def test_pack_transposed_round_trip(oracle, L):
    g = rng(2)
    m, n = 5, 320
    symbols = g.integers(0, 4, (m, n))
    cb = g.standard_normal(1 << L).astype(np.float16)
    stream = packing.pack_transposed(symbols)
    assert stream.shape == (n // 64, m, 4)
    got = oracle.matvec_t_dense(stream, cb, m, n, L, mode=oracle.CONTINUOUS)
    for r in range(m):
        assert np.array_equal(got[r].view(np.uint16), oracle.dequantize_h(cb, symbols[r]).view(np.uint16))


@pytest.mark.parametrize("n", [2048, 4096, 2048 + 768, 704, 64])
@pytest.mark.parametrize("S", [6, 8])
def test_pack_matvec_round_trip(oracle, n, S):
    g = rng(n + S)
    m = 3
    symbols = g.integers(0, 16, (m, n // 2))
    cb = g.standard_normal(2 << S).astype(np.float16)
    stream = packing.pack_matvec(symbols)
    assert stream.shape == (m * n // 16,)
    got = oracle.matvec_dense(stream, cb, m, n, S, mode=oracle.CONTINUOUS).view(np.uint16)
    cols = packing.matvec_stream_columns(n)
    assert sorted(cols.tolist()) == list(range(0, n, 2))          # every pair of columns exactly once
    cbb = cb.view(np.uint16)
    for r in range(m):
        state = 0
        for p, sym in enumerate(symbols[r]):
            state = ((state << 4) | int(sym)) & 0xFFFF
            prod = state * (state + 1)
            e = (prod >> 8) & ((1 << S) - 1)
            w0 = (int(cbb[2 * e]) & 0x7FFF) | (prod & 0x8000)
            assert got[r, cols[p]] == w0 and got[r, cols[p] + 1] == cbb[2 * e + 1]


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("n", [2048, 2048 + 320, 64])
def test_pack_matvec_bits_round_trip(oracle, bits, n):
    """6- and 8-bit symbols (3 and 4 bits per weight): the packed stream decodes to the shift-register walk."""
    g = rng(n + bits)
    m, S = 2, 8
    sb = 2 * bits
    symbols = g.integers(0, 1 << sb, (m, n // 2))
    cb = g.standard_normal(2 << S).astype(np.float16)
    stream = packing.pack_matvec(symbols, bits=bits)
    assert stream.shape == (m * n * bits // 32,)
    got = oracle.bits_dense(stream, cb, m, n, S, bits, mode=oracle.CONTINUOUS).view(np.uint16)
    cols = packing.matvec_stream_columns(n)
    cbb = cb.view(np.uint16)
    for r in range(m):
        state = 0
        for p, sym in enumerate(symbols[r]):
            state = ((state << sb) | int(sym)) & 0xFFFF
            prod = state * (state + 1)
            e = (prod >> 8) & ((1 << S) - 1)
            w0 = (int(cbb[2 * e]) & 0x7FFF) | (prod & 0x8000)
            assert got[r, cols[p]] == w0 and got[r, cols[p] + 1] == cbb[2 * e + 1]

"""Host-side packers: trellis symbols -> the three packed streams the kernels read.

The reference has no packer: its quantizers return unpacked symbol arrays (rptc.py:68,
rptc_lite.py:57) and nothing writes the bitstreams its CUDA kernels consume.  The layouts below
are read off the decoders (inference.cu:42-96, 189-277; inference_t.cu:68-175): symbols are
consumed most-significant-bits first inside each 32-bit word, words in memory order.  All
functions are plain numpy and return int32 arrays ready for ``torch.from_numpy``.
"""
import numpy as np


def _words_from_symbols(symbols, bits):
    """[..., k] symbols of `bits` bits (32 % bits == 0) -> [..., k*bits/32] uint32, first symbol on top."""
    per = 32 // bits
    s = np.asarray(symbols, dtype=np.uint32)
    assert s.shape[-1] % per == 0 and (s < (1 << bits)).all()
    s = s.reshape(s.shape[:-1] + (s.shape[-1] // per, per))
    shifts = (32 - bits * (np.arange(per, dtype=np.uint32) + 1)).astype(np.uint32)
    return np.bitwise_or.reduce(s << shifts, axis=-1).astype(np.uint32)


def pack_rowmajor(symbols):
    """2-bit symbols [m, n] -> the stream of ``decompress``: int32 [m, n/16], n % 2048 == 0.

    Row r, output t is decoded from symbols t-7..t of the row (inference.cu:68-94)."""
    symbols = np.asarray(symbols)
    m, n = symbols.shape
    assert n % 2048 == 0, "decompress needs whole groups of 32 stream elements per row"
    return _words_from_symbols(symbols, 2).view(np.int32)


def pack_transposed(symbols):
    """2-bit symbols [m, n] -> the stream of ``decompress_matvec_t_*``: int32 [n/64, m, 4], n % 64 == 0.

    Element col of row r holds the row's symbols 64*col .. 64*col+63 (inference_t.cu:116)."""
    symbols = np.asarray(symbols)
    m, n = symbols.shape
    assert n % 64 == 0
    words = _words_from_symbols(symbols, 2).reshape(m, n // 64, 4)
    return np.ascontiguousarray(words.transpose(1, 0, 2)).view(np.int32)


def matvec_stream_columns(n):
    """Column of the FIRST weight of every step of a row of the hashed pair stream, in stream order.

    Returns int64 [n/2]: entry p is the column 8*idx + 2*i of the pair decoded by the p-th 4-bit
    symbol of a row, p = (slab*32 + lane)*32 + step for the full slabs and the ragged last slab
    appended (inference.cu:215-221,249; step s <-> (k, j): k = 7, 0, 4, 1, 5, 2, 6, 3 for
    s // 4 = 0..7, j = s % 4).  The second weight of the pair is the next column."""
    assert n % 64 == 0
    T, Lt, n8 = n // 2048, (n % 2048) // 64, n // 8
    k_of = np.array([7, 0, 4, 1, 5, 2, 6, 3])
    s = np.arange(32)
    q = 4 * k_of[s // 4] + s % 4                       # slot step index 4k + j
    cols = []
    for slab in range(T + (1 if Lt else 0)):
        lanes = 32 if slab < T else Lt
        lane = np.arange(lanes)[:, None]
        P = 1024 * slab + (32 * q[None, :] + lane if slab < T else q[None, :] * Lt + lane)
        i, idx = P // n8, P % n8
        cols.append((8 * idx + 2 * i).reshape(-1))
    return np.concatenate(cols).astype(np.int64)


def _element_words(symbols, step_bits):
    """[..., 32 k] symbols of `step_bits` bits -> [..., k * step_bits] uint32: every 32 symbols become one
    element of step_bits words, first symbol in the top bits of the first word."""
    s = np.asarray(symbols, dtype=np.uint32)
    assert s.shape[-1] % 32 == 0 and (s < (1 << step_bits)).all()
    shifts = np.arange(step_bits - 1, -1, -1, dtype=np.uint32)
    bits = ((s[..., None] >> shifts) & 1).astype(np.uint8).reshape(s.shape[:-1] + (s.shape[-1] * step_bits,))
    packed = np.packbits(bits, axis=-1, bitorder="big")
    return np.ascontiguousarray(packed).view(">u4").astype(np.uint32)


def pack_matvec(symbols, bits=2):
    """Symbols of 2*bits bits [m, n/2] in stream order -> the hashed pair stream: int32 [m*n*bits/32].

    bits == 2 is the stream of ``decompress_matvec_*`` (4-bit symbols); bits 3 and 4 (6- and 8-bit symbols) are
    this library's extension, elements of 2*bits words.

    Row r's p-th symbol is step p % 32 of lane (p // 32) % lanes of slab p // 1024; the flat result
    is [n/2048][m][32][4] followed by the ragged slab [m][Lt][4] (reshape to [n/2048, m, 128] when
    n % 2048 == 0).  In CONTINUOUS mode the decoder state before a step is the previous four
    symbols of the row."""
    symbols = np.asarray(symbols)
    m, half = symbols.shape
    n = 2 * half
    assert n % 64 == 0
    T, Lt = n // 2048, (n % 2048) // 64
    wpe = 2 * bits                                     # words per element
    words = _element_words(symbols, 2 * bits)          # [m, n/64 * wpe]: elements in stream order
    parts = []
    if T:
        full = words[:, :T * 32 * wpe].reshape(m, T, 32 * wpe)
        parts.append(np.ascontiguousarray(full.transpose(1, 0, 2)).reshape(-1))
    if Lt:
        parts.append(np.ascontiguousarray(words[:, T * 32 * wpe:]).reshape(-1))
    return np.concatenate(parts).view(np.int32)

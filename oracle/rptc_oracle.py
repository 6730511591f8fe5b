"""ctypes front end of the CPU oracle (oracle/rptc_oracle.c).

Test infrastructure only: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg, never by the rptc_kernels module.  Arrays are
numpy; fp16 values travel as uint16 bit patterns or numpy float16 views.
"""
import ctypes
import os

import numpy as np

from . import build as _build

AS_WRITTEN = 0
CONTINUOUS = 1

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_build.LIB):
            _build.build()
        _lib = ctypes.CDLL(_build.LIB)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        _lib.orc_dequantize.argtypes = [vp, i32, vp, i64, vp]
        _lib.orc_dequantize_h.argtypes = [vp, i32, vp, i64, vp]
        _lib.orc_decompress.argtypes = [vp, vp, vp, i64, i64, i32]
        _lib.orc_hash.argtypes = [ctypes.c_uint32, i32, vp, vp, vp]
        _lib.orc_matvec.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32]
        _lib.orc_matvec.restype = i32
        _lib.orc_matvec_dense.argtypes = [vp, vp, vp, i64, i64, i32, i32]
        _lib.orc_matvec_dense.restype = i32
        _lib.orc_matvec_t.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32]
        _lib.orc_matvec_t.restype = i32
        _lib.orc_matvec_t_dense.argtypes = [vp, vp, vp, i64, i64, i32, i32]
        _lib.orc_matvec_t_dense.restype = i32
        _lib.orc_lite_index_fn.argtypes = [ctypes.c_int32, i32, i32]
        _lib.orc_lite_index_fn.restype = ctypes.c_int32
        _lib.orc_lite_dequantize.argtypes = [vp, i32, i32, i32, i32, vp, i64, vp]
        _lib.orc_dense_matvec.argtypes = [vp, vp, vp, i64, i64, i64]
        _lib.orc_matvec_f32.argtypes = [vp, vp, vp, vp, i64, i64, i32, i32]
        _lib.orc_matvec_f32.restype = i32
        _lib.orc_half_to_float.argtypes = [vp, vp, i64]
        _lib.orc_float_to_half.argtypes = [vp, vp, i64]
        _lib.orc_bits_dense.argtypes = [vp, vp, vp, i64, i64, i32, i32, i32]
        _lib.orc_bits_dense.restype = i32
        _lib.orc_sign_hadamard.argtypes = [vp, vp, vp, i64, i64, i64, i32]
        _lib.orc_sign_hadamard.restype = i32
        _lib.orc_viterbi.argtypes = [vp, i32, i32, i32, vp, vp, i64, vp, vp, vp]
        _lib.orc_viterbi.restype = i32
        _lib.orc_num_threads.restype = i32
        _lib.orc_set_num_threads.argtypes = [i32]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _u32(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.int32:
        a = a.view(np.uint32)
    assert a.dtype == np.uint32, a.dtype
    return a


def _u16(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def dequantize(alphabet, symbols):
    """rptc.py:74-85 on a float32 alphabet of length 2^L and 2-bit symbols."""
    alphabet = np.ascontiguousarray(alphabet, dtype=np.float32)
    symbols = np.ascontiguousarray(symbols, dtype=np.int32)
    L = int(alphabet.shape[0]).bit_length() - 1
    assert alphabet.shape[0] == 1 << L
    out = np.empty(symbols.shape[0], dtype=np.float32)
    lib().orc_dequantize(_p(alphabet), L, _p(symbols), symbols.shape[0], _p(out))
    return out


def viterbi(table, step_bits, targets, weights=None):
    """rptc.py:13-71 (diag_only) on a trellis of table.shape[0] = 2^L states that takes step_bits per step and
    emits table.shape[1] values per state.  table float32 [2^L, V]; targets float32 [steps, V]; weights None
    or [steps, V].  Returns (symbols int32 [steps], cost float32, end_state int)."""
    table = np.ascontiguousarray(table, dtype=np.float32)
    targets = np.ascontiguousarray(targets, dtype=np.float32)
    if table.ndim == 1:
        table, targets = table[:, None], targets.reshape(-1, 1)
    M, V = table.shape
    L = int(M).bit_length() - 1
    assert M == 1 << L and targets.ndim == 2 and targets.shape[1] == V
    steps = targets.shape[0]
    w = None
    if weights is not None:
        w = np.ascontiguousarray(weights, dtype=np.float32).reshape(steps, V)
    symbols = np.empty(steps, dtype=np.int32)
    cost = np.zeros(1, dtype=np.float32)
    end = np.zeros(1, dtype=np.int32)
    rc = lib().orc_viterbi(_p(table), L, int(step_bits), V, _p(targets), _p(w) if w is not None else None, steps,
                           _p(symbols), _p(cost), _p(end))
    assert rc == 0, rc
    return symbols, cost[0], int(end[0])


def dequantize_h(alphabet, symbols):
    alphabet = _u16(alphabet)
    symbols = np.ascontiguousarray(symbols, dtype=np.int32)
    L = int(alphabet.shape[0]).bit_length() - 1
    out = np.empty(symbols.shape[0], dtype=np.uint16)
    lib().orc_dequantize_h(_p(alphabet), L, _p(symbols), symbols.shape[0], _p(out))
    return out.view(np.float16)


def decompress(compressed, codebook, mode=AS_WRITTEN):
    """inference.cu:42-96.  compressed int32 [m, 4*cn] -> float16 [m, 64*cn]."""
    c = _u32(compressed)
    cb = _u16(codebook)
    assert c.ndim == 2 and c.shape[1] % 4 == 0 and cb.shape == (65536,)
    m, cn = c.shape[0], c.shape[1] // 4
    out = np.empty((m, 64 * cn), dtype=np.uint16)
    lib().orc_decompress(_p(c), _p(cb), _p(out), m, cn, mode)
    return out.view(np.float16)


def hash_window(h, S):
    """(hash, entry, sign) of one window, inference.cu:250-262."""
    hv, e, s = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    lib().orc_hash(ctypes.c_uint32(h & 0xFFFFFFFF), S, ctypes.byref(hv), ctypes.byref(e), ctypes.byref(s))
    return hv.value, e.value, s.value


def matvec(compressed, codebook, x, m, S, mode=AS_WRITTEN):
    """inference.cu:189-277 with double accumulation.  x float16 [n] or [B, n];
    compressed is the flat stream (any shape, m*n/16 words).  Returns float64 [m] / [B, m]."""
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    xx = _u16(x)
    single = xx.ndim == 1
    xx = xx.reshape(-1, xx.shape[-1])
    B, n = xx.shape
    assert c.size * 16 == m * n, (c.size, m, n)
    assert cb.shape == (2 << S,)
    y = np.empty((B, m), dtype=np.float64)
    rc = lib().orc_matvec(_p(c), _p(cb), _p(xx), _p(y), m, n, B, S, mode)
    assert rc == 0, rc
    return y[0] if single else y


def matvec_dense(compressed, codebook, m, n, S, mode=AS_WRITTEN):
    """The dense float16 [m, n] matrix the hashed stream stands for."""
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    assert c.size * 16 == m * n and cb.shape == (2 << S,)
    W = np.empty((m, n), dtype=np.uint16)
    rc = lib().orc_matvec_dense(_p(c), _p(cb), _p(W), m, n, S, mode)
    assert rc == 0, rc
    return W.view(np.float16)


def matvec_t(compressed, codebook, x, m, L, mode=AS_WRITTEN):
    """inference_t.cu:68-175 with double accumulation; returns the sum to be added to out."""
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    xx = _u16(x)
    single = xx.ndim == 1
    xx = xx.reshape(-1, xx.shape[-1])
    B, n = xx.shape
    assert c.size * 16 >= m * n and cb.shape == (1 << L,)
    y = np.empty((B, m), dtype=np.float64)
    rc = lib().orc_matvec_t(_p(c), _p(cb), _p(xx), _p(y), m, n, B, L, mode)
    assert rc == 0, rc
    return y[0] if single else y


def matvec_t_dense(compressed, codebook, m, n, L, mode=AS_WRITTEN):
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    assert c.size * 16 >= m * n and cb.shape == (1 << L,)
    W = np.empty((m, n), dtype=np.uint16)
    rc = lib().orc_matvec_t_dense(_p(c), _p(cb), _p(W), m, n, L, mode)
    assert rc == 0, rc
    return W.view(np.float16)


def lite_index_fn(x, L, S):
    """rptc_lite.py:12-16 on int32 with wraparound."""
    x &= 0xFFFFFFFF
    if x >= 1 << 31:
        x -= 1 << 32
    return lib().orc_lite_index_fn(x, L, S)


def lite_dequantize(alphabet, L, S, R, symbols):
    """rptc_lite.py:63-73.  alphabet float32 [2^S, V]."""
    alphabet = np.ascontiguousarray(alphabet, dtype=np.float32)
    symbols = np.ascontiguousarray(symbols, dtype=np.int32)
    V = alphabet.shape[1]
    out = np.empty((symbols.shape[0], V), dtype=np.float32)
    lib().orc_lite_dequantize(_p(alphabet), L, S, R, V, _p(symbols), symbols.shape[0], _p(out))
    return out


def lite_quantize(alphabet, L, S, R, importance, samples):
    """rptc_lite.py:19-60: the search over the 2^L states whose values are alphabet[index_fn(state)] (the reference's
    `permuted_alphabet`, rptc_lite.py:27-29), R stream bits a step, cost sum_v importance * (samples - value)^2
    (rptc_lite.py:39); orc_viterbi is the same recursion and trace back (its tie rules are argmin's first index, as
    rptc_lite.py:34,52 use it).  alphabet float32 [2^S, V]; samples float32 [length, V]; importance the same shape or
    None (all ones).  Returns (quantized int32 [length], expected_loss float32)."""
    alphabet = np.ascontiguousarray(alphabet, dtype=np.float32)
    table = alphabet[[lite_index_fn(s, L, S) for s in range(1 << L)]]
    symbols, cost, _ = viterbi(table, R, samples, importance)
    return symbols, cost


def dense_matvec(W, x):
    """float64 y = W x from float16 W [m, n] and x [n] or [B, n]."""
    Wb = _u16(W)
    xx = _u16(x)
    single = xx.ndim == 1
    xx = xx.reshape(-1, xx.shape[-1])
    m, n = Wb.shape
    y = np.empty((xx.shape[0], m), dtype=np.float64)
    lib().orc_dense_matvec(_p(Wb), _p(xx), _p(y), m, n, xx.shape[0])
    return y[0] if single else y


def matvec_f32(compressed, codebook, x, m, S, mode=AS_WRITTEN):
    """The timed CPU leg: fused decode + mat-vec, float32 accumulation, threads over rows."""
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    xx = _u16(x)
    n = xx.shape[0]
    y = np.empty(m, dtype=np.float32)
    rc = lib().orc_matvec_f32(_p(c), _p(cb), _p(xx), _p(y), m, n, S, mode)
    assert rc == 0, rc
    return y


def bits_dense(compressed, codebook, m, n, S, bits, mode=AS_WRITTEN):
    """The dense float16 [m, n] matrix of a hashed pair stream at `bits` (2, 3, 4) bits per weight."""
    c = _u32(compressed).reshape(-1)
    cb = _u16(codebook)
    assert c.size * 32 == m * n * bits and cb.shape == (2 << S,)
    W = np.empty((m, n), dtype=np.uint16)
    rc = lib().orc_bits_dense(_p(c), _p(cb), _p(W), m, n, S, bits, mode)
    assert rc == 0, rc
    return W.view(np.float16)


def sign_hadamard(x, signs, block, inverse=False):
    """Blockwise sign-Hadamard transform in double of float16 x [n] or [batch, n]; returns float64."""
    xx = _u16(x)
    single = xx.ndim == 1
    xx = xx.reshape(-1, xx.shape[-1])
    ss = _u16(signs)
    batch, n = xx.shape
    y = np.empty((batch, n), dtype=np.float64)
    rc = lib().orc_sign_hadamard(_p(xx), _p(ss), _p(y), batch, n, block, 1 if inverse else 0)
    assert rc == 0, rc
    return y[0] if single else y


def half_to_float(h):
    h = _u16(h)
    f = np.empty(h.shape, dtype=np.float32)
    lib().orc_half_to_float(_p(h), _p(f), h.size)
    return f


def float_to_half(f):
    f = np.ascontiguousarray(f, dtype=np.float32)
    h = np.empty(f.shape, dtype=np.uint16)
    lib().orc_float_to_half(_p(f), _p(h), f.size)
    return h.view(np.float16)


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(t):
    lib().orc_set_num_threads(int(t))

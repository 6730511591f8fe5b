"""rptc_kernels for MI355X: the reference extension's seven ops over hand-written gfx950 kernels.

Drop-in for the reference's pybind11 module (rptc_kernels/csrc/rptc_kernels/wrapper.cpp:59-67):
the same seven callables, positional ``torch.Tensor`` arguments, outputs written in place into
tensors the caller allocates, elapsed milliseconds returned as a ``float``, argument errors
raised as ``RuntimeError`` (what ``TORCH_CHECK`` raises).  The work is done by
``librptc_hip.so`` through its C ABI (include/rptc_hip.h); this module only validates tensors
and passes raw device pointers plus the current HIP stream.  There is no CPU implementation:
without the library, or with CPU tensors, every op raises.

Differences from the reference, all deliberate:
* ``carry_mode`` (module-level, see ``set_carry_mode``) chooses between the CUDA source's literal
  arithmetic (``AS_WRITTEN``, the default) and one unbroken shift register per row
  (``CONTINUOUS``, the trellis of rptc.py:74-85).
* the returned milliseconds always time the op's own kernels on the stream they ran on (the
  reference's ``decompress_matvec_*`` times an idle stream, inference.cu:335-350).  Timing makes
  a call host-synchronous, as ``decompress`` and ``decompress_matvec_t_*`` are in the reference;
  ``set_timing(False)`` makes every op asynchronous and return 0.0.
* ``decompress_matvec_*`` accumulates in fp32 and accepts any row count and any ``n % 64 == 0``
  (a ragged last slab); ``decompress_matvec_t_*`` accepts any row count.

Beside the seven: ``matvec_dense`` / ``matvec_t_dense`` / ``matvec_bits_dense`` (the dense fp16 matrix
a stream stands for), ``decompress_matmul_16_{6,8}_1`` and ``decompress_matmul_bits`` (batch 1..32 on
the matrix cores), ``decompress_matvec_bits`` (2, 3, 4 bits per weight), ``decompress_matvec_silu`` and
``decompress_matvec_rmsnorm`` (the mat-vec with a decoder layer's element-wise step in its prologue),
``decompress_matvec_hadamard`` (with the sign-Hadamard transform of its activations in its prologue),
``decompress_matvec_affine`` / ``_silu_affine`` / ``_rmsnorm_affine`` (with the row/column scales and biases of
the reference's factorisation, quantize_hf.py:167, applied inside the kernel),
``sign_hadamard``, ``viterbi_pairs`` and ``viterbi_scalar`` (the quantizer's trellis search, rptc.py:13-71,
as kernels: for the hashed pair stream and for the reference's own scalar trellis), ``lite_dequantize`` and
``lite_quantize`` (rptc_lite.py's decoder and search).
Sub-modules: ``packing`` (symbols -> streams), ``quantize`` (the quantizer around that search),
``linear`` (``QuantizedLinear``, ``patch_model``), ``llama_decode`` (a Llama-shaped decode loop),
``eval_ppl`` (perplexity on a token file).
"""
import ctypes
import os

import torch

AS_WRITTEN = 0
CONTINUOUS = 1
# statuses of include/rptc_hip.h that callers may want to tell apart
ELIMIT = -5
EDEPEND = -8

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(os.path.dirname(_HERE), "librptc_hip.so")

_lib = None
_carry_mode = AS_WRITTEN
_timing = True

_VP, _I64, _INT = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
_FP = ctypes.POINTER(ctypes.c_float)



class ChainLayer(ctypes.Structure):
    """rptc_chain_layer of include/rptc_hip.h."""
    _fields_ = [("compressed", _VP), ("x", _VP), ("out", _VP), ("m", _I64), ("n", _I64)]


class ChainPlan(ctypes.Structure):
    """rptc_chain_t of include/rptc_hip.h (opaque)."""
    _fields_ = [("opaque", ctypes.c_uint64 * 10)]


_MATVEC_ARGS = [_VP, _VP, _VP, _VP, _I64, _I64, _INT, _VP, _FP]
_SIGNATURES = {
    "rptc_version": ([], _INT),
    "rptc_status_string": ([_INT], ctypes.c_char_p),
    "rptc_init": ([], _INT),
    "rptc_decompress": ([_VP, _VP, _VP, _I64, _I64, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_16_6_1": (_MATVEC_ARGS, _INT),
    "rptc_decompress_matvec_20_6_1": (_MATVEC_ARGS, _INT),
    "rptc_decompress_matvec_16_8_1": (_MATVEC_ARGS, _INT),
    "rptc_decompress_matvec_20_8_1": (_MATVEC_ARGS, _INT),
    "rptc_decompress_matvec_t_16": (_MATVEC_ARGS, _INT),
    "rptc_decompress_matvec_t_14": (_MATVEC_ARGS, _INT),
    "rptc_chain_desc_bytes": ([ctypes.POINTER(ChainLayer), _I64], _I64),
    "rptc_chain_plan": ([ctypes.POINTER(ChainLayer), _I64, _VP, _I64, ctypes.POINTER(ChainPlan), _VP], _INT),
    "rptc_decompress_matvec_chain": ([ctypes.POINTER(ChainPlan), _VP, _INT, _INT, _VP, _FP], _INT),
    "rptc_matvec_dense": ([_VP, _VP, _VP, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_matvec_t_dense": ([_VP, _VP, _VP, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matmul": ([_VP, _VP, _VP, _VP, _I64, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matmul_bits": ([_VP, _VP, _VP, _VP, _I64, _I64, _I64, _INT, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matmul_workspace_bytes": ([_I64, _I64, _I64, _INT], _I64),
    "rptc_decompress_matmul_ws": ([_VP, _VP, _VP, _VP, _I64, _I64, _I64, _INT, _INT, _INT, _VP, _I64, _VP, _FP], _INT),
    "rptc_scratch_check": ([_INT, ctypes.POINTER(ctypes.c_int), _VP], _INT),
    "rptc_viterbi_scratch_bytes": ([_I64, _I64], _I64),
    "rptc_viterbi_scalar_scratch_bytes": ([_I64, _I64], _I64),
    "rptc_viterbi_scalar": ([_VP, _VP, _I64, _VP, _INT, _VP, _VP, _VP, _VP, _I64, _I64, _VP, _FP], _INT),
    "rptc_viterbi_pairs": ([_VP, _VP, _I64, _VP, _VP, _VP, _VP, _VP, _I64, _I64, _INT, _VP, _FP], _INT),
    "rptc_lite_viterbi_scratch_bytes": ([_INT, _INT, _I64, _I64], _I64),
    "rptc_lite_viterbi": ([_VP, _VP, _I64, _VP, _INT, _INT, _INT, _INT, _VP, _VP, _VP, _VP, _I64, _I64, _VP, _FP], _INT),
    "rptc_viterbi_pairs_bits": ([_VP, _VP, _I64, _VP, _VP, _VP, _VP, _VP, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_lite_dequantize": ([_VP, _INT, _INT, _INT, _INT, _VP, _I64, _I64, _VP, _VP, _FP], _INT),
    "rptc_sign_hadamard": ([_VP, _VP, _VP, _I64, _I64, _I64, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_bits": ([_VP, _VP, _VP, _VP, _I64, _I64, _INT, _INT, _INT, _VP, _FP], _INT),
    "rptc_matvec_bits_dense": ([_VP, _VP, _VP, _I64, _I64, _INT, _INT, _INT, _VP, _FP], _INT),
    "rptc_add_rmsnorm": ([_VP, _VP, _VP, _VP, _VP, _I64, ctypes.c_float, _VP], _INT),
    "rptc_rope_cache": ([_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _I64, _I64, _VP], _INT),
    "rptc_attn_decode": ([_VP, _VP, _VP, _VP, _VP, _I64, _I64, _I64, _VP], _INT),
    "rptc_silu_mul": ([_VP, _VP, _I64, _VP], _INT),
    "rptc_greedy_next": ([_VP, _I64, _VP, _I64, _VP, _VP, _VP, _VP, _VP, _VP], _INT),
    "rptc_rope_attn_decode": ([_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _I64, _I64, _VP], _INT),
    "rptc_decompress_matvec_silu": ([_VP, _VP, _VP, _VP, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_hadamard": ([_VP, _VP, _VP, _VP, _VP, _I64, _I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_rmsnorm": ([_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _I64, ctypes.c_float, _INT, _INT,
                                        _VP, _FP], _INT),
    "rptc_decompress_matvec_affine": ([_VP] * 8 + [_I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_silu_affine": ([_VP] * 8 + [_I64, _I64, _INT, _INT, _VP, _FP], _INT),
    "rptc_decompress_matvec_rmsnorm_affine": ([_VP] * 11 + [_I64, _I64, ctypes.c_float, _INT, _INT, _VP, _FP], _INT),
}


def library_path():
    return _LIB_PATH


def exported_symbols():
    """Names the C header declares; used by the load test."""
    return sorted(_SIGNATURES)


def library():
    """The loaded C-ABI library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"rptc_kernels: {_LIB_PATH} is missing; build it with "
                "`python let-it-slide_amd/build.py` (hipcc, gfx950)")
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


def set_carry_mode(mode):
    """AS_WRITTEN (default) or CONTINUOUS; returns the previous mode."""
    global _carry_mode
    if mode not in (AS_WRITTEN, CONTINUOUS):
        raise ValueError("carry mode must be rptc_kernels.AS_WRITTEN or rptc_kernels.CONTINUOUS")
    prev, _carry_mode = _carry_mode, mode
    return prev


def get_carry_mode():
    return _carry_mode


def set_timing(enabled):
    """When False, ops launch asynchronously and return 0.0; returns the previous setting."""
    global _timing
    prev, _timing = _timing, bool(enabled)
    return prev


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_input(t, name):
    # CHECK_INPUT of the reference (inference.cu:26-28)
    _check(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
    _check(t.is_cuda, f"{name} must be a CUDA tensor")
    _check(t.is_contiguous(), f"{name} must be contiguous")


def _status(rc):
    if rc != 0:
        text = library().rptc_status_string(rc).decode()
        raise RuntimeError(f"rptc_kernels: {text} (status {rc})")


def _call(fn, tensors, *args, carry_mode=None, timed=None):
    """timed: None = the module-wide setting (``set_timing``); False = this call passes a NULL ``ms`` pointer and
    is asynchronous whatever the setting (what a layer inside a model wants: no global is touched)."""
    device = tensors[0].device
    for t in tensors[1:]:
        _check(t.device == device, "all tensors must be on the same device")
    ms = ctypes.c_float(0.0)
    mode = _carry_mode if carry_mode is None else carry_mode
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = fn(*[t.data_ptr() for t in tensors], *args, mode, ctypes.c_void_p(stream),
                ctypes.byref(ms) if (_timing if timed is None else timed) else None)
    _status(rc)
    return float(ms.value)


def decompress(compressed, codebook, out):
    """Decode the row-major stream: out[r, t] = codebook[16 stream bits ending at bit 2t+2].

    compressed int32 [m, 4c] with 4c % 128 == 0; codebook fp16 [65536]; out fp16 [m, 64c]
    (inference.cu:99-160).  Returns elapsed ms."""
    _check_input(compressed, "compressed")
    _check(compressed.dim() == 2, "compressed.dim() == 2")
    _check(compressed.size(1) % (4 * 32) == 0, "compressed.size(1) % (4 * 32) == 0")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    m = compressed.size(0)
    n = compressed.size(1) // 4 * 64
    _check(m >= 1 and compressed.size(1) >= 128, "compressed must not be empty")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1, "codebook.dim() == 1")
    _check(codebook.size(0) == 1 << 16, "codebook.size(0) == 1<<16")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 2, "out.dim() == 2")
    _check(out.size(0) == m, "out.size(0) == m")
    _check(out.size(1) == n, "out.size(1) == n")
    _check(out.dtype == torch.float16, "out.scalar_type() == torch::kFloat16")
    return _call(library().rptc_decompress, (compressed, codebook, out), m, compressed.size(1))


def _matvec(symbol, S, compressed, codebook, x, out):
    # checks of inference.cu:293-316, relaxed where the library accepts more
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(x, "x")
    _check(x.dim() == 1, "x.dim() == 1")
    _check(x.dtype == torch.float16, "x.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 1, "out.dim() == 1")
    _check(out.dtype == torch.float16, "out.scalar_type() == torch::kFloat16")
    n, m = x.size(0), out.size(0)
    if compressed.dim() == 3:
        # the reference layout [n/2048, m, 128]
        _check(compressed.size(2) == 32 * 4, "compressed.size(2) == 32 * 4")
        _check(compressed.size(1) == m, "out.size(0) == m")
        _check(compressed.size(0) * 32 * 4 * 16 == n, "x.size(0) == n")
    else:
        # flat stream with a ragged last slab (n % 2048 != 0)
        _check(compressed.dim() == 1, "compressed.dim() == 3 (or 1 for a ragged stream)")
        _check(n % 64 == 0, "x.size(0) % 64 == 0")
        _check(compressed.numel() * 16 == m * n, "compressed.numel() * 16 == m * n")
    _check(m >= 1 and n >= 64, "compressed must not be empty")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1, "codebook.dim() == 1")
    _check(codebook.size(0) == 1 << (S + 1), "codebook.size(0) == 1<<(S+V)")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    return _call(getattr(library(), symbol), (compressed, codebook, x, out), m, n)


def decompress_matvec_16_6_1(compressed, codebook, x, out):
    """out = W x for the hashed-codebook stream, 64 codebook pairs (inference.cu:358-362)."""
    return _matvec("rptc_decompress_matvec_16_6_1", 6, compressed, codebook, x, out)


def decompress_matvec_20_6_1(compressed, codebook, x, out):
    """Same function as decompress_matvec_16_6_1: the reference kernel ignores L (inference.cu:364-368)."""
    return _matvec("rptc_decompress_matvec_20_6_1", 6, compressed, codebook, x, out)


def decompress_matvec_16_8_1(compressed, codebook, x, out):
    """out = W x for the hashed-codebook stream, 256 codebook pairs (inference.cu:370-374)."""
    return _matvec("rptc_decompress_matvec_16_8_1", 8, compressed, codebook, x, out)


def decompress_matvec_20_8_1(compressed, codebook, x, out):
    """Same function as decompress_matvec_16_8_1 (inference.cu:376-380)."""
    return _matvec("rptc_decompress_matvec_20_8_1", 8, compressed, codebook, x, out)


def _matvec_t(symbol, L, compressed, codebook, x, out):
    # checks of inference_t.cu:188-221; m and n come from out and x as in the reference
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(out, "out")
    _check_input(x, "x")
    m, n = out.size(0), x.size(0)
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1, "codebook.dim() == 1")
    _check(codebook.size(0) == 1 << L, "codebook.size(0) == 1<<L")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    _check(x.dim() == 1, "x.dim() == 1")
    _check(x.size(0) % 8 == 0, "x.size(0) % 8 == 0")
    _check(x.dtype == torch.float16, "x.scalar_type() == torch::kFloat16")
    _check(n % 64 == 0 and n >= 64, "x.size(0) % 64 == 0 (the kernel reads whole uint4 elements)")
    _check(n <= 32768, "x must fit the 64 KiB activation buffer (n <= 32768)")
    _check(out.dim() == 1, "out.dim() == 1")
    _check(out.dtype == torch.float16, "out.scalar_type() == torch::kFloat16")
    _check(m >= 1, "out must not be empty")
    _check(compressed.numel() * 16 >= m * n, "compressed holds fewer than m*n/16 words")
    return _call(getattr(library(), symbol), (compressed, codebook, x, out), m, n)


def decompress_matvec_t_16(compressed, codebook, x, out):
    """out += W x for the column-interleaved stream, 2^16 scalar codebook (inference_t.cu:258-262)."""
    return _matvec_t("rptc_decompress_matvec_t_16", 16, compressed, codebook, x, out)


def decompress_matvec_t_14(compressed, codebook, x, out):
    """out += W x for the column-interleaved stream, 2^14 scalar codebook (inference_t.cu:264-268)."""
    return _matvec_t("rptc_decompress_matvec_t_14", 14, compressed, codebook, x, out)


# ---------------------------------------------------------------- additions to the reference API

def matvec_dense(compressed, codebook, out, S):
    """Write the dense fp16 [m, n] matrix a hashed-codebook stream stands for into ``out``."""
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(codebook, "codebook")
    _check(S in (6, 8), "S must be 6 or 8")
    _check(codebook.dim() == 1 and codebook.size(0) == 1 << (S + 1), "codebook.size(0) == 1<<(S+V)")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 2 and out.dtype == torch.float16, "out must be a 2-D fp16 tensor")
    m, n = out.shape
    _check(n % 64 == 0 and m >= 1 and n >= 64, "out.size(1) % 64 == 0")
    _check(compressed.numel() * 16 == m * n, "compressed.numel() * 16 == m * n")
    return _call(library().rptc_matvec_dense, (compressed, codebook, out), m, n, S)


def matvec_t_dense(compressed, codebook, out, L):
    """Write the dense fp16 [m, n] matrix a column-interleaved stream stands for into ``out``."""
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(codebook, "codebook")
    _check(L in (14, 16), "L must be 14 or 16")
    _check(codebook.dim() == 1 and codebook.size(0) == 1 << L, "codebook.size(0) == 1<<L")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 2 and out.dtype == torch.float16, "out must be a 2-D fp16 tensor")
    m, n = out.shape
    _check(n % 64 == 0 and m >= 1 and n >= 64, "out.size(1) % 64 == 0")
    _check(compressed.numel() * 16 >= m * n, "compressed holds fewer than m*n/16 words")
    return _call(library().rptc_matvec_t_dense, (compressed, codebook, out), m, n, L)


def _matmul(S, compressed, codebook, x, out, bits=2):
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(x, "x")
    _check(x.dim() == 2, "x.dim() == 2 ([batch, n])")
    _check(x.dtype == torch.float16, "x.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 2, "out.dim() == 2 ([batch, m])")
    _check(out.dtype == torch.float16, "out.scalar_type() == torch::kFloat16")
    batch, n = x.shape
    _check(out.size(0) == batch, "out.size(0) == x.size(0)")
    m = out.size(1)
    _check(1 <= batch <= 32, "1 <= batch <= 32")
    _check(n % 64 == 0 and n >= 64 and m >= 1, "x.size(1) % 64 == 0")
    _check(n <= 32768, "x.size(1) <= 32768")
    _check(bits in (2, 3, 4), "bits must be 2, 3 or 4")
    _check(compressed.numel() * 32 == m * n * bits, "compressed.numel() * 32 == m * n * bits")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1 and codebook.size(0) == 1 << (S + 1), "codebook.size(0) == 1<<(S+V)")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    return _call(library().rptc_decompress_matmul_bits, (compressed, codebook, x, out), m, n, batch, S, bits)


def decompress_matmul_16_6_1(compressed, codebook, x, out):
    """out[b] = W x[b] for batch 1..32 on the hashed-codebook stream with 64 pairs; x [batch, n], out [batch, m]."""
    return _matmul(6, compressed, codebook, x, out)


def decompress_matmul_16_8_1(compressed, codebook, x, out):
    """out[b] = W x[b] for batch 1..32 on the hashed-codebook stream with 256 pairs; x [batch, n], out [batch, m]."""
    return _matmul(8, compressed, codebook, x, out)


def decompress_matmul_bits(compressed, codebook, x, out, bits):
    """out[b] = W x[b] for batch 1..32 on the hashed pair stream at ``bits`` (2, 3, 4) bits per weight; S from the
    codebook length; x [batch, n], out [batch, m]."""
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1 and codebook.size(0) in (128, 512), "codebook.size(0) == 1<<(S+V), S in {6, 8}")
    return _matmul(6 if codebook.size(0) == 128 else 8, compressed, codebook, x, out, bits=bits)


def hadamard_block(n):
    """The default block length of the sign-Hadamard transform: the largest power of two dividing n (<= 32768)."""
    p = 1
    while n % (2 * p) == 0 and 2 * p <= 32768:
        p *= 2
    return p


def sign_hadamard(x, signs, out, block=0, inverse=False, timed=None):
    """Blockwise random-sign Hadamard transform of the rows of x ([n] or [batch, n], fp16).

    forward: out = H (signs * x) / sqrt(block); inverse: out = signs * (H x) / sqrt(block), per block of
    ``block`` elements (0 = the largest power of two dividing n).  ``out`` may be ``x``.  Returns elapsed ms."""
    _check_input(x, "x")
    _check_input(signs, "signs")
    _check_input(out, "out")
    _check(x.dtype == torch.float16 and signs.dtype == torch.float16 and out.dtype == torch.float16,
           "x, signs and out must be fp16")
    _check(x.dim() in (1, 2), "x.dim() in (1, 2)")
    _check(out.shape == x.shape, "out.shape == x.shape")
    n = x.size(-1)
    batch = x.size(0) if x.dim() == 2 else 1
    _check(signs.dim() == 1 and signs.size(0) == n, "signs.size(0) == n")
    p = block or hadamard_block(n)
    _check(p >= 2 and p & (p - 1) == 0 and n % p == 0 and p <= 32768, "block must be a power of two dividing n")
    device = x.device
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = library().rptc_sign_hadamard(x.data_ptr(), signs.data_ptr(), out.data_ptr(), batch, n, p,
                                          1 if inverse else 0, ctypes.c_void_p(stream),
                                          ctypes.byref(ms) if (_timing if timed is None else timed) else None)
    _status(rc)
    return float(ms.value)


def lite_dequantize(alphabet, L, S, R, quantized, timed=None):
    """``rptc_lite.dequantize(alphabet, L, S, R, quantized)`` (rptc_lite.py:63-73): the outputs of the general
    hashed-codebook trellis for a symbol sequence.

    alphabet: float32 [2^S, V]; quantized: int32 [length] or [rows, length] (every row a sequence of its own that
    starts from register 0).  Returns (dequantized float32 [length, V] or [rows, length, V], elapsed ms)."""
    _check_input(alphabet, "alphabet")
    _check_input(quantized, "quantized")
    _check(alphabet.dtype == torch.float32 and alphabet.dim() == 2, "alphabet must be float32 [2^S, V]")
    _check(quantized.dtype == torch.int32 and quantized.dim() in (1, 2), "quantized must be int32 [length] or [rows, length]")
    _check(1 <= R <= 16 and 1 <= S <= 16 and S <= L <= 31, "1 <= R <= 16, 1 <= S <= 16, S <= L <= 31")
    _check(alphabet.size(0) == 1 << S, "alphabet.size(0) == 1 << S")
    V = alphabet.size(1)
    _check(1 <= V <= 8, "1 <= V <= 8")
    rows = quantized.size(0) if quantized.dim() == 2 else 1
    length = quantized.size(-1)
    _check(rows >= 1 and length >= 1, "rows >= 1 and length >= 1")
    device = alphabet.device
    _check(quantized.device == device, "all tensors must be on the same device")
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(device):
        out = torch.empty(tuple(quantized.shape) + (V,), dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream().cuda_stream
        rc = library().rptc_lite_dequantize(alphabet.data_ptr(), L, S, R, V, quantized.data_ptr(), rows, length, out.data_ptr(),
                                            ctypes.c_void_p(stream), ctypes.byref(ms) if (_timing if timed is None else timed) else None)
    _status(rc)
    return out, float(ms.value)


def lite_quantize(alphabet, L, S, R, importance, samples):
    """``rptc_lite.quantize(alphabet, L, S, R, importance, samples)`` (rptc_lite.py:19-60): the symbol sequence whose
    ``lite_dequantize`` is closest to ``samples`` under the per-value ``importance``, by exact Viterbi search.

    alphabet: float32 [2^S, V]; samples, importance: float32 [length, V], or [rows, length, V] with every row a sequence
    of its own (importance may be None for all ones, or [length, V] for one set shared by all rows).  Takes
    S <= L <= 20, R <= 8, V <= 4; L = 16, R = 4, V = 2, S <= 9 (the parameters of the reference's own driver) run the
    fast kernel.  Returns (quantized int32 [length] or [rows, length], expected_loss float32 scalar or [rows])."""
    _check_input(alphabet, "alphabet")
    _check_input(samples, "samples")
    _check(alphabet.dtype == torch.float32 and alphabet.dim() == 2, "alphabet must be float32 [2^S, V]")
    _check(samples.dtype == torch.float32 and samples.dim() in (2, 3), "samples must be float32 [length, V] or [rows, length, V]")
    _check(1 <= S <= L and 1 <= R <= L, "1 <= S <= L and 1 <= R <= L")
    _check(alphabet.size(0) == 1 << S, "alphabet.size(0) == 1 << S")
    V = alphabet.size(1)
    _check(samples.size(-1) == V, "samples.size(-1) == alphabet.size(1)")
    single = samples.dim() == 2
    rows, steps = (1, samples.size(0)) if single else (samples.size(0), samples.size(1))
    _check(rows >= 1 and steps >= 1, "rows >= 1 and length >= 1")
    stride = 0
    if importance is not None:
        _check_input(importance, "importance")
        _check(importance.dtype == torch.float32, "importance must be float32")
        _check(tuple(importance.shape) in ((steps, V), (rows, steps, V)), "importance must have the shape of samples, or [length, V]")
        stride = 0 if importance.dim() == 2 else V * steps
    device = samples.device
    _check(alphabet.device == device, "all tensors must be on the same device")
    lib = library()
    with torch.cuda.device(device):
        scratch = torch.empty(max(lib.rptc_lite_viterbi_scratch_bytes(L, R, rows, steps), 16), dtype=torch.uint8, device=device)
        symbols = torch.empty((rows, steps), dtype=torch.uint8, device=device)
        end_state = torch.empty(rows, dtype=torch.int32, device=device)
        cost = torch.empty(rows, dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.rptc_lite_viterbi(samples.data_ptr(), importance.data_ptr() if importance is not None else None, stride,
                                   alphabet.data_ptr(), L, S, R, V, scratch.data_ptr(), symbols.data_ptr(), end_state.data_ptr(),
                                   cost.data_ptr(), rows, steps, ctypes.c_void_p(stream), None)
        _status(rc)
        torch.cuda.current_stream().synchronize()     # scratch is freed on return
    quantized = symbols.to(torch.int32)
    return (quantized[0], cost[0]) if single else (quantized, cost)


def viterbi_pairs(targets, codebook, weights=None, bits=2):
    """Exact Viterbi search on the trellis of ``decompress_matvec_16_{S}_1`` (65536 states, 4 stream bits
    and two weights per step; S from the codebook length), the search of rptc.py:13-71; ``bits`` = 3 or 4: the
    trellis of ``decompress_matvec_bits`` (6 or 8 stream bits per step, symbols up to 63 or 255).

    targets: float32 [rows, steps, 2] (weight pairs in stream order); weights: None, float32 [steps, 2]
    (one importance set for all rows) or [rows, steps, 2].  Returns (symbols uint8 [rows, steps],
    cost float32 [rows], end_state int32 [rows], elapsed ms).  Needs rows * steps * 2048 bytes of scratch."""
    _check_input(targets, "targets")
    _check_input(codebook, "codebook")
    _check(targets.dtype == torch.float32 and targets.dim() == 3 and targets.size(2) == 2,
           "targets must be float32 [rows, steps, 2]")
    _check(codebook.dtype == torch.float16 and codebook.numel() in (128, 512), "codebook must be fp16 of length 128 or 512")
    rows, steps = targets.size(0), targets.size(1)
    _check(rows >= 1 and steps >= 1, "rows >= 1 and steps >= 1")
    _check(bits in (2, 3, 4), "bits must be 2, 3 or 4")
    S = 6 if codebook.numel() == 128 else 8
    stride = 0
    if weights is not None:
        _check_input(weights, "weights")
        _check(weights.dtype == torch.float32, "weights must be float32")
        _check(tuple(weights.shape) in ((steps, 2), (rows, steps, 2)), "weights must be [steps, 2] or [rows, steps, 2]")
        stride = 0 if weights.dim() == 2 else 2 * steps
    device = targets.device
    lib = library()
    with torch.cuda.device(device):
        scratch = torch.empty(lib.rptc_viterbi_scratch_bytes(rows, steps), dtype=torch.uint8, device=device)
        symbols = torch.empty((rows, steps), dtype=torch.uint8, device=device)
        end_state = torch.empty(rows, dtype=torch.int32, device=device)
        cost = torch.empty(rows, dtype=torch.float32, device=device)
        ms = ctypes.c_float(0.0)
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.rptc_viterbi_pairs_bits(targets.data_ptr(), weights.data_ptr() if weights is not None else None, stride,
                                         codebook.data_ptr(), scratch.data_ptr(), symbols.data_ptr(), end_state.data_ptr(),
                                         cost.data_ptr(), rows, steps, S, bits, ctypes.c_void_p(stream),
                                         ctypes.byref(ms) if _timing else None)
        _status(rc)
        if not _timing:
            torch.cuda.current_stream().synchronize()     # scratch is freed on return
    return symbols, cost, end_state, float(ms.value)


def viterbi_scalar(targets, alphabet, weights=None):
    """The reference's trellis search as it stands (rptc.py:13-71, diag_only): 2^L states (L = 16 or 14 from the
    alphabet's length), 2 stream bits and one value per step, state s emitting alphabet[s]; the symbols are what
    ``decompress`` (L = 16) and ``decompress_matvec_t_{16,14}`` decode in CONTINUOUS mode.

    targets: float32 [rows, steps]; alphabet: fp16 [2^L]; weights: None, float32 [steps] or [rows, steps] (the
    reference's ``sum(corrections[index]**2)``).  Returns (symbols uint8 [rows, steps], cost float32 [rows],
    end_state int32 [rows], elapsed ms).  Needs rows * steps * 4096 bytes of scratch."""
    _check_input(targets, "targets")
    _check_input(alphabet, "alphabet")
    _check(targets.dtype == torch.float32 and targets.dim() == 2, "targets must be float32 [rows, steps]")
    _check(alphabet.dtype == torch.float16 and alphabet.numel() in (1 << 14, 1 << 16),
           "alphabet must be fp16 of length 2^14 or 2^16")
    rows, steps = targets.shape
    _check(rows >= 1 and steps >= 1, "rows >= 1 and steps >= 1")
    L = 14 if alphabet.numel() == 1 << 14 else 16
    stride = 0
    if weights is not None:
        _check_input(weights, "weights")
        _check(weights.dtype == torch.float32, "weights must be float32")
        _check(tuple(weights.shape) in ((steps,), (rows, steps)), "weights must be [steps] or [rows, steps]")
        stride = 0 if weights.dim() == 1 else steps
    device = targets.device
    lib = library()
    with torch.cuda.device(device):
        scratch = torch.empty(lib.rptc_viterbi_scalar_scratch_bytes(rows, steps), dtype=torch.uint8, device=device)
        symbols = torch.empty((rows, steps), dtype=torch.uint8, device=device)
        end_state = torch.empty(rows, dtype=torch.int32, device=device)
        cost = torch.empty(rows, dtype=torch.float32, device=device)
        ms = ctypes.c_float(0.0)
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.rptc_viterbi_scalar(targets.data_ptr(), weights.data_ptr() if weights is not None else None, stride,
                                     alphabet.data_ptr(), L, scratch.data_ptr(), symbols.data_ptr(), end_state.data_ptr(),
                                     cost.data_ptr(), rows, steps, ctypes.c_void_p(stream),
                                     ctypes.byref(ms) if _timing else None)
        _status(rc)
        if not _timing:
            torch.cuda.current_stream().synchronize()     # scratch is freed on return
    return symbols, cost, end_state, float(ms.value)


def decompress_matvec_bits(compressed, codebook, x, out, bits):
    """out = W x for the hashed pair stream at ``bits`` (2, 3, 4) bits per weight; S from the codebook length.

    compressed int32 with m*n*bits/32 words ([n/2048, m, 32, 2*bits] + ragged slab); bits == 2 is
    decompress_matvec_16_{S}_1."""
    _check(bits in (2, 3, 4), "bits must be 2, 3 or 4")
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1 and codebook.size(0) in (128, 512), "codebook.size(0) == 1<<(S+V), S in {6, 8}")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    S = 6 if codebook.size(0) == 128 else 8
    _check_input(x, "x")
    _check(x.dim() == 1 and x.dtype == torch.float16, "x must be a 1-D fp16 tensor")
    _check_input(out, "out")
    _check(out.dim() == 1 and out.dtype == torch.float16, "out must be a 1-D fp16 tensor")
    n, m = x.size(0), out.size(0)
    _check(n % 64 == 0 and n >= 64 and m >= 1, "x.size(0) % 64 == 0")
    _check(compressed.numel() * 32 == m * n * bits, "compressed.numel() * 32 == m * n * bits")
    return _call(library().rptc_decompress_matvec_bits, (compressed, codebook, x, out), m, n, S, bits)


def _fused_common(compressed, codebook, out, n):
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1 and codebook.size(0) in (128, 512), "codebook.size(0) == 1<<(S+V), S in {6, 8}")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    _check_input(out, "out")
    _check(out.dim() == 1 and out.dtype == torch.float16, "out must be a 1-D fp16 tensor")
    m = out.size(0)
    _check(n % 64 == 0 and n >= 64 and m >= 1, "x.size(0) % 64 == 0")
    _check(compressed.numel() * 16 == m * n, "compressed.numel() * 16 == m * n")
    return m, (6 if codebook.size(0) == 128 else 8)


def decompress_matvec_silu(compressed, codebook, gate_up, out):
    """out = W (silu(gate) * up) with gate_up = [gate | up] (fp16 [2n]): ``decompress_matvec_16_{S}_1`` with the
    gate of a Llama MLP computed inside the kernel.  Returns elapsed ms."""
    _check_input(gate_up, "gate_up")
    _check(gate_up.dim() == 1 and gate_up.dtype == torch.float16 and gate_up.size(0) % 2 == 0,
           "gate_up must be a 1-D fp16 tensor of even length")
    n = gate_up.size(0) // 2
    m, S = _fused_common(compressed, codebook, out, n)
    return _call(library().rptc_decompress_matvec_silu, (compressed, codebook, gate_up, out), m, n, S)


def decompress_matvec_hadamard(compressed, codebook, x, signs, out, block=0):
    """out = W (H (signs * x) / sqrt(block)): ``decompress_matvec_16_{S}_1`` with the forward ``sign_hadamard``
    of its activations computed inside the kernel (x and signs fp16 [n], n <= 15360; block = 0: the largest
    power of two dividing n).  Returns elapsed ms."""
    for t, name in ((x, "x"), (signs, "signs")):
        _check_input(t, name)
        _check(t.dim() == 1 and t.dtype == torch.float16 and t.size(0) == x.size(0), f"{name} must be fp16 [n]")
    n = x.size(0)
    m, S = _fused_common(compressed, codebook, out, n)
    return _call(library().rptc_decompress_matvec_hadamard, (compressed, codebook, x, signs, out), m, n, block, S)


def decompress_matvec_rmsnorm(compressed, codebook, x_in, delta, weight, x_out, out, eps=1e-5):
    """x_out = x_in + delta (delta may be None); out = W (rmsnorm(x_out) * weight): ``decompress_matvec_16_{S}_1``
    with the residual add and RMS norm of a decoder layer computed inside the kernel.  ``x_out`` must be a
    buffer of its own (not ``x_in``, not ``delta``).  Returns elapsed ms."""
    for t, name in ((x_in, "x_in"), (weight, "weight"), (x_out, "x_out")) + (((delta, "delta"),) if delta is not None else ()):
        _check_input(t, name)
        _check(t.dim() == 1 and t.dtype == torch.float16 and t.size(0) == x_in.size(0), f"{name} must be fp16 [n]")
    n = x_in.size(0)
    m, S = _fused_common(compressed, codebook, out, n)
    device = compressed.device
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = library().rptc_decompress_matvec_rmsnorm(
            compressed.data_ptr(), codebook.data_ptr(), x_in.data_ptr(), None if delta is None else delta.data_ptr(),
            weight.data_ptr(), x_out.data_ptr(), out.data_ptr(), m, n, float(eps), S, _carry_mode,
            ctypes.c_void_p(stream), ctypes.byref(ms) if _timing else None)
    _status(rc)
    return float(ms.value)


def _affine_ptrs(n, m, scales_in, biases_in, scales_out, biases_out):
    ptrs = []
    for t, name, length in ((scales_in, "scales_in", n), (biases_in, "biases_in", n),
                            (scales_out, "scales_out", m), (biases_out, "biases_out", m)):
        if t is None:
            ptrs.append(None)
            continue
        _check_input(t, name)
        _check(t.dim() == 1 and t.dtype == torch.float16 and t.size(0) == length, f"{name} must be fp16 [{length}]")
        ptrs.append(t.data_ptr())
    return ptrs


def _call_affine(fn, head, tail, device, carry_mode, timed=None):
    ms = ctypes.c_float(0.0)
    mode = _carry_mode if carry_mode is None else carry_mode
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = fn(*head, *tail, mode, ctypes.c_void_p(stream),
                ctypes.byref(ms) if (_timing if timed is None else timed) else None)
    _status(rc)
    return float(ms.value)


def decompress_matvec_affine(compressed, codebook, x, out, scales_in=None, biases_in=None, scales_out=None,
                             biases_out=None, carry_mode=None, timed=None):
    """out = scales_out * (W_hat (scales_in * x)) + biases_out * sum(x) + biases_in . x: the product with the
    matrix the reference's quantizer reconstructs, W = b_out + b_in + s_out * s_in * W_hat
    (quantize_hf.py:167), in one launch.  The four vectors are fp16 ([n], [n], [m], [m]) or None; n <= 16384.
    Returns elapsed ms."""
    _check_input(x, "x")
    _check(x.dim() == 1 and x.dtype == torch.float16, "x must be a 1-D fp16 tensor")
    n = x.size(0)
    m, S = _fused_common(compressed, codebook, out, n)
    aff = _affine_ptrs(n, m, scales_in, biases_in, scales_out, biases_out)
    return _call_affine(library().rptc_decompress_matvec_affine,
                        (compressed.data_ptr(), codebook.data_ptr(), x.data_ptr(), *aff, out.data_ptr()), (m, n, S),
                        compressed.device, carry_mode, timed)


def decompress_matvec_silu_affine(compressed, codebook, gate_up, out, scales_in=None, biases_in=None, scales_out=None,
                                  biases_out=None, carry_mode=None):
    """``decompress_matvec_affine`` on silu(gate) * up, gate_up = [gate | up] (fp16 [2n])."""
    _check_input(gate_up, "gate_up")
    _check(gate_up.dim() == 1 and gate_up.dtype == torch.float16 and gate_up.size(0) % 2 == 0,
           "gate_up must be a 1-D fp16 tensor of even length")
    n = gate_up.size(0) // 2
    m, S = _fused_common(compressed, codebook, out, n)
    aff = _affine_ptrs(n, m, scales_in, biases_in, scales_out, biases_out)
    return _call_affine(library().rptc_decompress_matvec_silu_affine,
                        (compressed.data_ptr(), codebook.data_ptr(), gate_up.data_ptr(), *aff, out.data_ptr()), (m, n, S),
                        compressed.device, carry_mode)


def decompress_matvec_rmsnorm_affine(compressed, codebook, x_in, delta, weight, x_out, out, eps=1e-5, scales_in=None,
                                     biases_in=None, scales_out=None, biases_out=None, carry_mode=None):
    """``decompress_matvec_affine`` on rmsnorm(x_in + delta) * weight; x_out = x_in + delta (see
    ``decompress_matvec_rmsnorm``)."""
    for t, name in ((x_in, "x_in"), (weight, "weight"), (x_out, "x_out")) + (((delta, "delta"),) if delta is not None else ()):
        _check_input(t, name)
        _check(t.dim() == 1 and t.dtype == torch.float16 and t.size(0) == x_in.size(0), f"{name} must be fp16 [n]")
    n = x_in.size(0)
    m, S = _fused_common(compressed, codebook, out, n)
    aff = _affine_ptrs(n, m, scales_in, biases_in, scales_out, biases_out)
    return _call_affine(library().rptc_decompress_matvec_rmsnorm_affine,
                        (compressed.data_ptr(), codebook.data_ptr(), x_in.data_ptr(),
                         None if delta is None else delta.data_ptr(), weight.data_ptr(), x_out.data_ptr(), *aff,
                         out.data_ptr()), (m, n, float(eps), S), compressed.device, carry_mode)


class MatvecChain:
    """A chain of ``decompress_matvec_16_{S}_1`` products (``rptc_decompress_matvec_chain``).

    ``layers`` is a sequence of ``(compressed, x, out)`` tensor triples (int32 stream, fp16 [n], fp16 [m]); the
    tensors are kept alive by the object and their addresses are fixed in the plan, their contents are read at
    run time.  One codebook and one carry mode serve the whole chain.

    Layers that do not depend on each other run in ONE launch.  When the library refuses the one-launch form - a
    layer reads or overwrites what another writes (``RPTC_EDEPEND``), or a layer is too large for it
    (``RPTC_ELIMIT``) - ``run`` makes one ``decompress_matvec_16_{S}_1`` launch per layer on the current stream,
    in order, which is what orders dependent layers; ``one_launch`` tells which of the two it is."""

    def __init__(self, layers, codebook):
        layers = list(layers)
        _check(len(layers) >= 1, "a chain needs at least one layer")
        _check_input(codebook, "codebook")
        _check(codebook.dim() == 1 and codebook.size(0) in (128, 512) and codebook.dtype == torch.float16,
               "codebook must be fp16 of length 128 or 512")
        self.S = 6 if codebook.size(0) == 128 else 8
        self.codebook = codebook
        self.layers = layers
        arr = (ChainLayer * len(layers))()
        for i, (c, x, out) in enumerate(layers):
            for t, name in ((c, "compressed"), (x, "x"), (out, "out")):
                _check_input(t, name)
                _check(t.device == codebook.device, "all tensors must be on the same device")
            _check(c.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
            _check(x.dim() == 1 and x.dtype == torch.float16, "x must be a 1-D fp16 tensor")
            _check(out.dim() == 1 and out.dtype == torch.float16, "out must be a 1-D fp16 tensor")
            n, m = x.size(0), out.size(0)
            _check(n % 64 == 0 and n >= 64 and m >= 1, "x.size(0) % 64 == 0")
            _check(c.numel() * 16 == m * n, "compressed.numel() * 16 == m * n")
            arr[i] = ChainLayer(c.data_ptr(), x.data_ptr(), out.data_ptr(), m, n)
        lib = library()
        need = lib.rptc_chain_desc_bytes(arr, len(layers))
        if need < 0:
            _status(int(need))
        with torch.cuda.device(codebook.device):
            self.desc = torch.zeros(need + 256, dtype=torch.uint8, device=codebook.device)
            base = (self.desc.data_ptr() + 255) & ~255
            self.plan = ChainPlan()
            stream = torch.cuda.current_stream().cuda_stream
            rc = lib.rptc_chain_plan(arr, len(layers), base, need, ctypes.byref(self.plan), ctypes.c_void_p(stream))
        self.one_launch = rc == 0
        if rc not in (0, EDEPEND, ELIMIT):
            _status(rc)

    def run(self, carry_mode=None, timed=None):
        """Runs the chain on the current stream; returns elapsed ms (0.0 when not timed)."""
        ms = ctypes.c_float(0.0)
        mode = _carry_mode if carry_mode is None else carry_mode
        want_ms = _timing if timed is None else timed
        lib = library()
        with torch.cuda.device(self.codebook.device):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            if self.one_launch:
                _status(lib.rptc_decompress_matvec_chain(ctypes.byref(self.plan), self.codebook.data_ptr(), self.S, mode,
                                                         stream, ctypes.byref(ms) if want_ms else None))
                return float(ms.value)
            fn = getattr(lib, f"rptc_decompress_matvec_16_{self.S}_1")
            total = 0.0
            for c, x, out in self.layers:
                _status(fn(c.data_ptr(), self.codebook.data_ptr(), x.data_ptr(), out.data_ptr(), out.size(0), x.size(0),
                           mode, stream, ctypes.byref(ms) if want_ms else None))
                total += float(ms.value)
        return total


def matvec_bits_dense(compressed, codebook, out, bits):
    """Write the dense fp16 [m, n] matrix of a hashed pair stream at ``bits`` bits per weight into ``out``."""
    _check(bits in (2, 3, 4), "bits must be 2, 3 or 4")
    _check_input(compressed, "compressed")
    _check(compressed.dtype == torch.int32, "compressed.scalar_type() == torch::kInt32")
    _check_input(codebook, "codebook")
    _check(codebook.dim() == 1 and codebook.size(0) in (128, 512), "codebook.size(0) == 1<<(S+V), S in {6, 8}")
    _check(codebook.dtype == torch.float16, "codebook.scalar_type() == torch::kFloat16")
    S = 6 if codebook.size(0) == 128 else 8
    _check_input(out, "out")
    _check(out.dim() == 2 and out.dtype == torch.float16, "out must be a 2-D fp16 tensor")
    m, n = out.shape
    _check(n % 64 == 0 and m >= 1 and n >= 64, "out.size(1) % 64 == 0")
    _check(compressed.numel() * 32 == m * n * bits, "compressed.numel() * 32 == m * n * bits")
    return _call(library().rptc_matvec_bits_dense, (compressed, codebook, out), m, n, S, bits)

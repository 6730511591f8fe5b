"""The C-ABI library loads without a GPU and exports every function include/rptc_hip.h declares;
the Python module validates arguments the way the reference's TORCH_CHECKs do."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rptc_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rptc_\w+)\s*\(", text)))


def test_header_declares_the_reference_surface():
    names = declared_functions()
    for op in ("decompress", "decompress_matvec_16_6_1", "decompress_matvec_20_6_1", "decompress_matvec_16_8_1",
               "decompress_matvec_20_8_1", "decompress_matvec_t_16", "decompress_matvec_t_14"):
        assert "rptc_" + op in names


def test_library_exports_every_declared_symbol():
    import rptc_kernels
    assert os.path.exists(rptc_kernels.library_path()), "build with python let-it-slide_amd/build.py"
    lib = ctypes.CDLL(rptc_kernels.library_path())
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert sorted(rptc_kernels.exported_symbols()) == declared_functions()
    assert rptc_kernels.library().rptc_version() >= 100
    assert b"NULL" in rptc_kernels.library().rptc_status_string(-1)


def test_python_module_has_the_reference_names():
    import rptc_kernels
    for op in ("decompress", "decompress_matvec_16_6_1", "decompress_matvec_20_6_1", "decompress_matvec_16_8_1",
               "decompress_matvec_20_8_1", "decompress_matvec_t_16", "decompress_matvec_t_14"):
        assert callable(getattr(rptc_kernels, op))


def test_cpu_tensors_are_rejected_not_computed():
    import rptc_kernels
    comp = torch.zeros((2, 128), dtype=torch.int32)
    cb = torch.zeros(65536, dtype=torch.float16)
    out = torch.zeros((2, 2048), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        rptc_kernels.decompress(comp, cb, out)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        rptc_kernels.decompress_matvec_16_8_1(torch.zeros((1, 32, 128), dtype=torch.int32),
                                              torch.zeros(512, dtype=torch.float16),
                                              torch.zeros(2048, dtype=torch.float16),
                                              torch.zeros(32, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        rptc_kernels.decompress_matvec_t_16(torch.zeros(256 * 64 // 16, dtype=torch.int32), cb,
                                            torch.zeros(64, dtype=torch.float16),
                                            torch.zeros(256, dtype=torch.float16))


def test_c_abi_rejects_bad_arguments_before_touching_a_device():
    import rptc_kernels
    lib = rptc_kernels.library()
    # NULL pointers and bad shapes are reported as negative statuses; no device is needed for these
    assert lib.rptc_decompress(None, None, None, 1, 128, 0, None, None) == -1
    assert lib.rptc_decompress(16, 16, 16, 1, 100, 0, None, None) == -2
    assert lib.rptc_decompress(16, 16, 16, 1, 128, 7, None, None) == -4
    assert lib.rptc_decompress(8, 16, 16, 1, 128, 0, None, None) == -3
    assert lib.rptc_decompress_matvec_16_8_1(16, 16, 16, 16, 32, 100, 0, None, None) == -2
    assert lib.rptc_decompress_matvec_t_16(16, 16, 16, 16, 256, 65536, 0, None, None) == -5
    assert lib.rptc_matvec_dense(16, 16, 16, 4, 64, 7, 0, None, None) == -2
    assert lib.rptc_matvec_t_dense(16, 16, 16, 4, 64, 15, 0, None, None) == -2
    # the entry points with no counterpart in the reference check before they launch, too
    assert lib.rptc_decompress_matmul(16, 16, 16, 16, 32, 2048, 33, 8, 0, None, None) == -5      # batch > 32
    assert lib.rptc_decompress_matmul_bits(16, 16, 16, 16, 32, 2048, 8, 8, 5, 0, None, None) == -2  # bits
    assert lib.rptc_decompress_matvec_bits(16, 16, 16, 16, 32, 2048, 7, 3, 0, None, None) == -2     # S
    assert lib.rptc_decompress_matvec_silu(None, 16, 16, 16, 32, 2048, 8, 0, None, None) == -1
    assert lib.rptc_decompress_matvec_rmsnorm(16, 16, 32, None, 48, 32, 64, 32, 2048, 1e-5, 8, 0, None, None) == -7   # x_out is x_in
    assert lib.rptc_decompress_matvec_rmsnorm(16, 16, 32, None, 48, 64, 80, 32, 32768, 1e-5, 8, 0, None, None) == -5  # n > 16384
    assert lib.rptc_decompress_matvec_affine(16, 16, 32, None, None, None, None, 64, 32, 32768, 8, 0, None, None) == -5  # n > 16384
    assert lib.rptc_decompress_matvec_affine(16, 16, 32, 8, None, None, None, 64, 32, 2048, 8, 0, None, None) == -3      # scales_in alignment
    assert lib.rptc_decompress_matvec_affine(16, 16, 32, None, None, None, None, 64, 32, 2048, 7, 0, None, None) == -2   # S
    assert lib.rptc_decompress_matvec_silu_affine(16, 16, None, None, None, None, None, 64, 32, 2048, 8, 0, None, None) == -1
    assert lib.rptc_decompress_matvec_rmsnorm_affine(16, 16, 32, None, 48, 32, None, None, None, None, 64, 32, 2048, 1e-5, 8, 0, None, None) == -7
    assert lib.rptc_greedy_next(16, 0, 16, 64, 16, 16, 16, 16, 16, None) == -2                   # empty vocabulary
    assert lib.rptc_greedy_next(16, 1000, None, 64, 16, 16, 16, 16, 16, None) == -1
    assert lib.rptc_sign_hadamard(16, 16, 16, 1, 4096, 48, 0, None, None) == -2                  # block not a power of two
    assert lib.rptc_decompress_matvec_hadamard(16, 16, 16, 16, 16, 32, 4096, 48, 8, 0, None, None) == -2   # block
    assert lib.rptc_decompress_matvec_hadamard(16, 16, 16, 16, 16, 32, 16384, 0, 8, 0, None, None) == -5   # n > 15360
    assert lib.rptc_rope_attn_decode(16, 16, 16, 16, 16, 16, 16, 4, 48, 128, None) == -2         # head_dim not a power of two
    assert lib.rptc_attn_decode(16, 16, 16, None, 16, 4, 64, 128, None) == -1
    assert lib.rptc_viterbi_pairs(16, None, 0, 16, 16, 16, 16, 16, 4, 64, 7, None, None) == -2    # S
    assert lib.rptc_viterbi_pairs(16, None, 0, 16, None, 16, 16, 16, 4, 64, 8, None, None) == -1  # no scratch
    assert lib.rptc_viterbi_pairs(16, 16, 100, 16, 16, 16, 16, 16, 4, 64, 8, None, None) == -2    # weight stride < 2 * steps
    assert lib.rptc_viterbi_scratch_bytes(4, 64) == 4 * 64 * 2048
    assert lib.rptc_viterbi_pairs_bits(16, None, 0, 16, 16, 16, 16, 16, 4, 64, 8, 5, None, None) == -2   # bits
    assert lib.rptc_viterbi_scalar(16, None, 0, 16, 15, 16, 16, 16, 16, 4, 64, None, None) == -2     # L
    assert lib.rptc_viterbi_scalar(16, None, 0, None, 16, 16, 16, 16, 16, 4, 64, None, None) == -1   # no alphabet
    assert lib.rptc_viterbi_scalar_scratch_bytes(4, 64) == 4 * 64 * 4096
    # the rptc_lite search: limits of both of its kernels, and the scratch each asks for
    assert lib.rptc_lite_viterbi(16, None, 0, 16, 16, 9, 4, 2, None, 16, 16, 16, 4, 64, None, None) == -1    # no scratch
    assert lib.rptc_lite_viterbi(16, None, 0, 16, 16, 17, 4, 2, 16, 16, 16, 16, 4, 64, None, None) == -2     # S > L
    assert lib.rptc_lite_viterbi(16, None, 0, 16, 21, 9, 4, 2, 16, 16, 16, 16, 4, 64, None, None) == -5      # L
    assert lib.rptc_lite_viterbi(16, None, 0, 16, 16, 9, 16, 2, 16, 16, 16, 16, 4, 64, None, None) == -5     # R
    assert lib.rptc_lite_viterbi(16, None, 0, 16, 16, 9, 4, 5, 16, 16, 16, 16, 4, 64, None, None) == -5      # V
    assert lib.rptc_lite_viterbi(16, 16, 100, 16, 12, 9, 4, 2, 16, 16, 16, 16, 4, 64, None, None) == -2      # importance stride < V * steps
    assert lib.rptc_lite_viterbi_scratch_bytes(16, 4, 4, 64) == 4 * 64 * 2048
    assert lib.rptc_lite_viterbi_scratch_bytes(12, 2, 3, 10) == (3 * (4096 + 1024) * 4 + 255) // 256 * 256 + 3 * 10 * 1024
    assert lib.rptc_lite_viterbi_scratch_bytes(21, 4, 1, 1) == 0 and lib.rptc_lite_viterbi_scratch_bytes(16, 16, 1, 1) == 0


def test_carry_mode_and_timing_switches():
    import rptc_kernels
    prev = rptc_kernels.set_carry_mode(rptc_kernels.CONTINUOUS)
    assert rptc_kernels.get_carry_mode() == rptc_kernels.CONTINUOUS
    rptc_kernels.set_carry_mode(prev)
    with pytest.raises(ValueError):
        rptc_kernels.set_carry_mode(3)
    prev = rptc_kernels.set_timing(False)
    rptc_kernels.set_timing(prev)


def test_bench_aids_library_exports_what_bench_binds():
    """`bench.py` binds the measurement aids by name when it starts: a missing symbol would end the benchmark before its
    first line.  (Loading the library and setting argument types touches no device.)"""
    import importlib.util
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = os.path.join(root, "bench_aids", "librptc_bench_aids.so")
    if not os.path.exists(path):
        pytest.skip("bench_aids/librptc_bench_aids.so is not built")
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    lib = bench.aids_library()
    for name in ("rptc_probe_empty", "rptc_probe_read", "rptc_probe_read_chain", "rptc_probe_lds", "rptc_probe_valu", "rptc_probe_decode"):
        assert hasattr(lib, name)

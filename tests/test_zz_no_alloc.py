"""The entry point that allocates nothing: rptc_decompress_matmul_bits keeps its scratch (packed activations,
partial tiles, arrival counters) in static device arrays, so it can be called where device memory cannot be
allocated.  Called through the C ABI twice in a row, the second time on a smaller input, it must give what
rptc_decompress_matmul_ws gives with the scratch in a caller's buffer: the same kernels, so bit for bit."""
import ctypes

import pytest
import torch

from util import rand_codes, rand_half

pytestmark = pytest.mark.gpu


def test_static_scratch_entry_point_equals_the_workspace_one_on_two_calls_in_a_row():
    import rptc_kernels
    lib = rptc_kernels.library()
    assert lib.rptc_init() == 0
    S, bits = 8, 2
    cb = rand_half(2 << S, seed=3).cuda()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the second call is smaller in every dimension: fewer row groups, fewer slabs, one plane of batch columns
    for call, (m, n, batch) in enumerate(((4096, 11008, 32), (1000, 4096 + 704, 5))):
        print(f"[case] call {call}: m={m} n={n} batch={batch}", flush=True)
        comp = rand_codes(m * n * bits // 32, seed=10 + call).cuda()
        x = rand_half(batch * n, seed=20 + call).reshape(batch, n).cuda()
        got = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
        want = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
        rc = lib.rptc_decompress_matmul_bits(comp.data_ptr(), cb.data_ptr(), x.data_ptr(), got.data_ptr(), m, n, batch, S, bits,
                                             0, stream, None)
        assert rc == 0, lib.rptc_status_string(rc)
        need = lib.rptc_decompress_matmul_workspace_bytes(m, n, batch, bits)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        rc = lib.rptc_decompress_matmul_ws(comp.data_ptr(), cb.data_ptr(), x.data_ptr(), want.data_ptr(), m, n, batch, S, bits,
                                           0, ws.data_ptr(), need, stream, None)
        assert rc == 0, lib.rptc_status_string(rc)
        torch.cuda.synchronize()
        assert not torch.isnan(got).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        # and it is the product: against the dense matrix the stream stands for
        W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
        rptc_kernels.matvec_bits_dense(comp, cb, W, bits)
        ref = x.double() @ W.double().t()
        assert float((got.double() - ref).norm() / ref.norm()) < 1e-3
    # beyond the static buffers' limits: refused, nothing launched
    big_n = 32768 + 64
    assert lib.rptc_decompress_matmul_bits(16, 16, 16, 16, 64, big_n, 8, S, bits, 0, None, None) == -5
    assert lib.rptc_decompress_matmul_bits(16, 16, 16, 16, 64, 4096, 33, S, bits, 0, None, None) == -5

"""GPU parity: the HIP kernels, called through the rptc_kernels module (ctypes -> C ABI), against
the CPU oracle on the same seeded inputs.  Decoded weights must match bit for bit; layer outputs
must be within rel-L2 1e-3 of the double-precision product of the decoded fp16 weights."""
import numpy as np
import pytest
import torch

from util import np_f16, np_u32, rand_codes, rand_half, rel_l2

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-3          # the tolerance the north star states for layer outputs (fp32 accumulate)
MODES = [0, 1]


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    rc = rptc_kernels.library().rptc_init()
    assert rc == 0, rptc_kernels.library().rptc_status_string(rc)
    return rptc_kernels


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def with_mode(rk, mode):
    class _Ctx:
        def __enter__(self):
            self.prev = rk.set_carry_mode(mode)

        def __exit__(self, *a):
            rk.set_carry_mode(self.prev)
    return _Ctx()


# ------------------------------------------------------------------ decompress (inference.cu:42-160)

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("m,cn", [(1, 32), (3, 96), (64, 64), (257, 32)])
def test_decompress_bit_exact(rk, oracle, mode, m, cn):
    comp = rand_codes(m * 4 * cn, seed=m + cn).reshape(m, 4 * cn)
    cb = rand_half(65536, seed=3)
    out = torch.full((m, 64 * cn), float("nan"), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        ms = rk.decompress(comp.cuda(), cb.cuda(), out)
    assert ms > 0
    want = oracle.decompress(np_u32(comp), np_f16(cb), mode=mode)
    assert np.array_equal(np_f16(out).view(np.uint16), want.view(np.uint16))


def test_decompress_state_sequence_with_bit_pattern_codebook(rk, oracle):
    # codebook[s] has raw bits s, so the output IS the decoder state: no float compare involved
    m, cn = 8, 64
    comp = rand_codes(m * 4 * cn, seed=99).reshape(m, 4 * cn)
    cb = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    out = torch.zeros((m, 64 * cn), dtype=torch.float16, device="cuda")
    for mode in MODES:
        with with_mode(rk, mode):
            rk.decompress(comp.cuda(), cb.cuda(), out)
        want = oracle.decompress(np_u32(comp), np_f16(cb), mode=mode)
        assert np.array_equal(np_f16(out).view(np.uint16), want.view(np.uint16))
    # hand-derived: first word of row 0 from state 0
    word = int(np_u32(comp)[0, 0])
    states = []
    s = 0
    for i in range(16):
        s = ((s << 2) | ((word >> (30 - 2 * i)) & 3)) & 0xFFFF
        states.append(s)
    assert np_f16(out).view(np.uint16)[0, :16].tolist() == states


def test_decompress_full_size_4096x4096(rk, oracle):
    m, cn = 4096, 64
    comp = rand_codes(m * 4 * cn, seed=42).reshape(m, 4 * cn)
    cb = rand_half(65536, seed=43)
    out = torch.zeros((m, 64 * cn), dtype=torch.float16, device="cuda")
    rk.decompress(comp.cuda(), cb.cuda(), out)
    want = oracle.decompress(np_u32(comp), np_f16(cb), mode=0)
    assert np.array_equal(np_f16(out).view(np.uint16), want.view(np.uint16))


def test_decompress_rejects_what_the_reference_rejects(rk):
    cb = torch.zeros(65536, dtype=torch.float16, device="cuda")
    good = torch.zeros((2, 128), dtype=torch.int32, device="cuda")
    out = torch.zeros((2, 2048), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        rk.decompress(torch.zeros((2, 64), dtype=torch.int32, device="cuda"), cb, out)      # size(1) % 128
    with pytest.raises(RuntimeError):
        rk.decompress(good.to(torch.int64), cb, out)                                         # dtype
    with pytest.raises(RuntimeError):
        rk.decompress(good, cb[:4096], out)                                                  # codebook size
    with pytest.raises(RuntimeError):
        rk.decompress(good, cb, out[:, :1024])                                               # out shape / contiguity
    with pytest.raises(RuntimeError):
        rk.decompress(good.t(), cb, out)                                                     # non-contiguous


# ------------------------------------------------------------------ decompress_matvec (inference.cu:189-380)

def matvec_fn(rk, L, S):
    return getattr(rk, f"decompress_matvec_{L}_{S}_1")


# (1540, 2048 + 192): on 256 compute units the last block of rows holds 4 of its 8 rows, so whole items of it are empty
MATVEC_SHAPES = [(32, 2048), (64, 4096), (33, 2048), (1, 64), (7, 704), (96, 4096 + 768), (512, 6144), (1540, 2048 + 192)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("m,n", MATVEC_SHAPES)
def test_matvec_dense_export_bit_exact(rk, oracle, mode, S, m, n):
    comp = rand_codes(m * n // 16, seed=m * 7 + n)
    cb = rand_half(2 << S, seed=S)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        rk.matvec_dense(comp.cuda(), cb.cuda(), W, S)
    want = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode)
    assert np.array_equal(np_f16(W).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("L,S", [(16, 6), (20, 6), (16, 8), (20, 8)])
@pytest.mark.parametrize("m,n", MATVEC_SHAPES)
def test_matvec_output_within_tolerance(rk, oracle, mode, L, S, m, n):
    comp = rand_codes(m * n // 16, seed=m + n)
    cb = rand_half(2 << S, seed=S + 10)
    x = rand_half(n, seed=5)
    out = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    c = comp.cuda().reshape(n // 2048, m, 128) if n % 2048 == 0 else comp.cuda()
    with with_mode(rk, mode):
        ms = matvec_fn(rk, L, S)(c, cb.cuda(), x.cuda(), out)
    assert ms > 0
    want = oracle.matvec(np_u32(comp), np_f16(cb), np_f16(x), m, S, mode=mode)
    got = np_f16(out).astype(np.float64)
    assert np.all(np.isfinite(got))
    # fp16 rounding of the result alone is 2^-11 relative per element
    assert rel_l2(got, want) < REL_L2_TOL


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("S", [6, 8])
def test_matvec_fused_kernel_decodes_bit_exactly(rk, oracle, mode, S):
    """One-hot activations: y[r] = W[r, p] exactly (a single product 1.0 * w, added to zeros in
    fp32), so the fused kernel's own decode and column map are checked bit for bit."""
    m, n = 64, 2048 + 192
    comp = rand_codes(m * n // 16, seed=123)
    cb = rand_half(2 << S, seed=S + 20)
    want = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode)
    c, cbd = comp.cuda(), cb.cuda()
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    x = torch.zeros(n, dtype=torch.float16, device="cuda")
    got = np.zeros((m, n), dtype=np.float16)
    prev_timing = rk.set_timing(False)
    try:
        with with_mode(rk, mode):
            cols = list(range(0, n, 7)) + list(range(n - 200, n)) + list(range(0, 64))
            for p in cols:
                x.zero_()
                x[p] = 1.0
                matvec_fn(rk, 16, S)(c, cbd, x, out)
                got[:, p] = np_f16(out)
    finally:
        rk.set_timing(prev_timing)
    cols = sorted(set(cols))
    g = got[:, cols].view(np.uint16)
    w = want[:, cols].view(np.uint16)
    # -0.0 * 1.0 + 0.0 = +0.0 in the accumulator: compare zeros by value
    nz = (w & 0x7FFF) != 0
    assert np.array_equal(g[nz], w[nz])
    assert np.all((g[~nz] & 0x7FFF) == 0)


@pytest.mark.parametrize("m,n", [(4096, 4096), (4096, 11008), (11008, 4096)])
def test_matvec_full_size(rk, oracle, m, n):
    S = 8
    comp = rand_codes(m * n // 16, seed=42)
    cb = rand_half(2 << S, seed=43)
    x = rand_half(n, seed=44)
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    c = comp.cuda().reshape(n // 2048, m, 128) if n % 2048 == 0 else comp.cuda()
    matvec_fn(rk, 16, S)(c, cb.cuda(), x.cuda(), out)
    want = oracle.matvec(np_u32(comp), np_f16(cb), np_f16(x), m, S, mode=0)
    assert rel_l2(np_f16(out), want) < REL_L2_TOL
    # decoded weights at full size, bit for bit
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    rk.matvec_dense(comp.cuda(), cb.cuda(), W, S)
    wantW = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=0)
    assert np.array_equal(np_f16(W).view(np.uint16), wantW.view(np.uint16))
    # size-independent properties: the fused product equals the dense product of the exported
    # matrix, and the op is linear in x
    y_dense = (W.double() @ x.cuda().double()).cpu().numpy()
    assert rel_l2(np_f16(out), y_dense) < REL_L2_TOL
    x2 = rand_half(n, seed=45)
    out2 = torch.zeros_like(out)
    out12 = torch.zeros_like(out)
    matvec_fn(rk, 16, S)(c, cb.cuda(), x2.cuda(), out2)
    xs = (x.float() + x2.float()).to(torch.float16)
    matvec_fn(rk, 16, S)(c, cb.cuda(), xs.cuda(), out12)
    lin = (W.double() @ xs.cuda().double()).cpu().numpy()
    assert rel_l2(np_f16(out12), lin) < REL_L2_TOL
    assert rel_l2(np_f16(out12).astype(np.float64), np_f16(out).astype(np.float64) + np_f16(out2).astype(np.float64)) < 5e-3


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("m,n", [(8192, 28672), (8192, 28672 + 192), (28672, 8192), (8192, 8192)])
def test_matvec_long_rows(rk, oracle, mode, m, n):
    """The Llama-3-70B layer shapes.  At n = 28672 the rows are so long that a CU's share of them needs the
    compact partial-sum layout (one sum per row and slab); the product must still match the double-precision
    product of the bit-exact dense matrix."""
    S = 8
    comp = rand_codes(m * n // 16, seed=52)
    cb = rand_half(2 << S, seed=53)
    x = rand_half(n, seed=54)
    out = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    c = comp.cuda().reshape(n // 2048, m, 128) if n % 2048 == 0 else comp.cuda()
    with with_mode(rk, mode):
        matvec_fn(rk, 16, S)(c, cb.cuda(), x.cuda(), out)
        W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
        rk.matvec_dense(comp.cuda(), cb.cuda(), W, S)
    y_dense = torch.cat([W[r0:r0 + 4096].double() @ x.cuda().double() for r0 in range(0, m, 4096)]).cpu().numpy()
    assert rel_l2(np_f16(out), y_dense) < REL_L2_TOL
    # the dense export is held to the oracle on the first rows (the whole matrix at this size takes the CPU a while)
    rows = 64
    idx = np_u32(comp).reshape(-1)
    T, Lt = n // 2048, (n % 2048) // 64
    parts = [idx[t * m * 128:(t * m + rows) * 128] for t in range(T)]
    if Lt:
        parts.append(idx[T * m * 128:T * m * 128 + rows * Lt * 4])
    wantW = oracle.matvec_dense(np.concatenate(parts), np_f16(cb), rows, n, S, mode=mode)
    assert np.array_equal(np_f16(W[:rows]).view(np.uint16), wantW.view(np.uint16))


def test_matvec_zero_stream_closed_form(rk):
    m, n, S = 64, 4096, 6
    cb = rand_half(2 << S, seed=3)
    x = rand_half(n, seed=4)
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    rk.decompress_matvec_16_6_1(torch.zeros((2, m, 128), dtype=torch.int32, device="cuda"), cb.cuda(), x.cuda(), out)
    xe = x.double()[0::2].sum().item()
    xo = x.double()[1::2].sum().item()
    want = abs(float(cb[0])) * xe + float(cb[1]) * xo
    assert np.allclose(np_f16(out).astype(np.float64), want, rtol=2e-3, atol=2e-2)


def test_matvec_rejects_what_the_reference_rejects(rk):
    cb = torch.zeros(512, dtype=torch.float16, device="cuda")
    comp = torch.zeros((1, 32, 128), dtype=torch.int32, device="cuda")
    x = torch.zeros(2048, dtype=torch.float16, device="cuda")
    out = torch.zeros(32, dtype=torch.float16, device="cuda")
    f = rk.decompress_matvec_16_8_1
    with pytest.raises(RuntimeError):
        f(torch.zeros((1, 32, 64), dtype=torch.int32, device="cuda"), cb, x, out)     # size(2) == 128
    with pytest.raises(RuntimeError):
        f(comp, cb[:128], x, out)                                                     # codebook size 2^(S+V)
    with pytest.raises(RuntimeError):
        f(comp, cb, x[:1024], out)                                                    # x.size(0) == n
    with pytest.raises(RuntimeError):
        f(comp, cb, x, out[:16])                                                      # out.size(0) == m
    with pytest.raises(RuntimeError):
        f(comp, cb, x.float(), out)                                                   # dtype
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_16_6_1(comp, cb, x, out)                                 # S=6 wants 128 values
    assert f(comp, cb, x, out) >= 0.0


# ------------------------------------------------------------------ decompress_matvec_t (inference_t.cu:68-268)

T_SHAPES = [(256, 64), (256, 1024), (300, 4096), (1, 128), (1024, 2048)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("L", [14, 16])
@pytest.mark.parametrize("m,n", T_SHAPES)
def test_matvec_t_dense_export_bit_exact(rk, oracle, mode, L, m, n):
    comp = rand_codes(m * n // 16, seed=m + n + L)
    cb = rand_half(1 << L, seed=L)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        rk.matvec_t_dense(comp.cuda(), cb.cuda(), W, L)
    want = oracle.matvec_t_dense(np_u32(comp), np_f16(cb), m, n, L, mode=mode)
    assert np.array_equal(np_f16(W).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("L", [14, 16])
@pytest.mark.parametrize("m,n", T_SHAPES)
def test_matvec_t_output_within_tolerance(rk, oracle, mode, L, m, n):
    comp = rand_codes(m * n // 16, seed=m + n + L)
    cb = rand_half(1 << L, seed=L)
    x = rand_half(n, seed=6)
    out0 = rand_half(m, seed=8)
    out = out0.cuda()
    with with_mode(rk, mode):
        ms = getattr(rk, f"decompress_matvec_t_{L}")(comp.cuda(), cb.cuda(), x.cuda(), out)
    assert ms > 0
    want = oracle.matvec_t(np_u32(comp), np_f16(cb), np_f16(x), m, L, mode=mode)
    want = want + np_f16(out0).astype(np.float64)         # the op accumulates into out
    assert rel_l2(np_f16(out), want) < REL_L2_TOL


@pytest.mark.parametrize("mode", MODES)
def test_matvec_t_fused_kernel_decodes_bit_exactly(rk, oracle, mode):
    L, m, n = 16, 128, 512
    comp = rand_codes(m * n // 16, seed=77)
    cb = rand_half(1 << L, seed=78)
    want = oracle.matvec_t_dense(np_u32(comp), np_f16(cb), m, n, L, mode=mode)
    c, cbd = comp.cuda(), cb.cuda()
    x = torch.zeros(n, dtype=torch.float16, device="cuda")
    got = np.zeros((m, n), dtype=np.float16)
    prev_timing = rk.set_timing(False)
    try:
        with with_mode(rk, mode):
            for p in range(n):
                x.zero_()
                x[p] = 1.0
                out = torch.zeros((m,), dtype=torch.float16, device="cuda")
                rk.decompress_matvec_t_16(c, cbd, x, out)
                got[:, p] = np_f16(out)
    finally:
        rk.set_timing(prev_timing)
    g, w = got.view(np.uint16), want.view(np.uint16)
    nz = (w & 0x7FFF) != 0
    assert np.array_equal(g[nz], w[nz])
    assert np.all((g[~nz] & 0x7FFF) == 0)


def test_matvec_t_full_size_4096(rk, oracle):
    L, m, n = 16, 4096, 4096
    comp = rand_codes(m * n // 16, seed=42)
    cb = rand_half(1 << L, seed=43)
    x = rand_half(n, seed=44)
    for mode in MODES:
        out = torch.zeros((m,), dtype=torch.float16, device="cuda")
        with with_mode(rk, mode):
            rk.decompress_matvec_t_16(comp.cuda(), cb.cuda(), x.cuda(), out)
        want = oracle.matvec_t(np_u32(comp), np_f16(cb), np_f16(x), m, L, mode=mode)
        assert rel_l2(np_f16(out), want) < REL_L2_TOL


def test_matvec_t_at_the_reference_activation_limit(rk, oracle):
    """n = 32768 is what the reference's 64 KiB of constant memory holds (inference_t.cu:49): accepted and right."""
    L, m, n = 16, 64, 32768
    comp = rand_codes(m * n // 16, seed=71)
    cb = rand_half(1 << L, seed=72)
    x = rand_half(n, seed=73)
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    rk.decompress_matvec_t_16(comp.cuda(), cb.cuda(), x.cuda(), out)
    want = oracle.matvec_t(np_u32(comp), np_f16(cb), np_f16(x), m, L, mode=0)
    assert rel_l2(np_f16(out), want) < REL_L2_TOL


def test_matvec_longest_row_and_beyond(rk, oracle):
    """The activation image, the table and two rows of partial sums must fit in 160 KiB of LDS: n = 32768 does,
    n = 65536 is refused with a status, not a fault."""
    S, m = 8, 32
    for n, ok in ((32768, True), (65536, False)):
        comp = rand_codes(m * n // 16, seed=81)
        cb = rand_half(2 << S, seed=82)
        x = rand_half(n, seed=83)
        out = torch.zeros((m,), dtype=torch.float16, device="cuda")
        c = comp.cuda().reshape(n // 2048, m, 128)
        if ok:
            rk.decompress_matvec_16_8_1(c, cb.cuda(), x.cuda(), out)
            want = oracle.matvec(np_u32(comp), np_f16(cb), np_f16(x), m, S, mode=0)
            assert rel_l2(np_f16(out), want) < REL_L2_TOL
        else:
            with pytest.raises(RuntimeError, match="exceeds"):
                rk.decompress_matvec_16_8_1(c, cb.cuda(), x.cuda(), out)


def test_matvec_t_rejects_bad_arguments(rk):
    cb = torch.zeros(65536, dtype=torch.float16, device="cuda")
    comp = torch.zeros(256 * 64 // 16, dtype=torch.int32, device="cuda")
    x = torch.zeros(64, dtype=torch.float16, device="cuda")
    out = torch.zeros(256, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_t_16(comp, cb[:16384], x, out)          # codebook.size(0) == 1<<L
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_t_14(comp, cb, x, out)
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_t_16(comp[:16], cb, x, out)             # stream too short
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_t_16(comp, cb, torch.zeros(40000, dtype=torch.float16, device="cuda"), out)
    assert rk.decompress_matvec_t_16(comp, cb, x, out) >= 0.0


# ------------------------------------------------------------------ decompress_matmul (batch 1..32, MFMA)

MATMUL_SHAPES = [(16, 2048), (64, 4096), (33, 2048), (5, 704), (96, 4096 + 768), (300, 6144)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("batch", [1, 8, 16, 17, 32])
@pytest.mark.parametrize("m,n", MATMUL_SHAPES)
def test_matmul_output_within_tolerance(rk, oracle, mode, S, batch, m, n):
    comp = rand_codes(m * n // 16, seed=m + n + batch)
    cb = rand_half(2 << S, seed=S + 30)
    x = rand_half(batch * n, seed=9).reshape(batch, n)
    out = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        ms = getattr(rk, f"decompress_matmul_16_{S}_1")(comp.cuda(), cb.cuda(), x.cuda(), out)
    assert ms > 0
    want = oracle.matvec(np_u32(comp), np_f16(cb), np_f16(x), m, S, mode=mode)      # [batch, m] in double
    got = np_f16(out).astype(np.float64)
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) < REL_L2_TOL
    for b in range(batch):
        assert rel_l2(got[b], want[b]) < 2 * REL_L2_TOL


@pytest.mark.parametrize("mode", MODES)
def test_matmul_identity_batch_recovers_weights_bit_exactly(rk, oracle, mode):
    """x = 32 one-hot rows at a time: out[b][r] = W[r][p_b] exactly, so the MFMA path's decode,
    operand layout and column map are checked bit for bit."""
    S, m, n = 8, 48, 2048 + 320
    comp = rand_codes(m * n // 16, seed=321)
    cb = rand_half(2 << S, seed=31)
    want = oracle.matvec_dense(np_u32(comp), np_f16(cb), m, n, S, mode=mode)
    c, cbd = comp.cuda(), cb.cuda()
    got = np.zeros((m, n), dtype=np.float16)
    out = torch.zeros((32, m), dtype=torch.float16, device="cuda")
    prev_timing = rk.set_timing(False)
    try:
        with with_mode(rk, mode):
            for p0 in range(0, n, 32):
                x = torch.zeros((32, n), dtype=torch.float16, device="cuda")
                x[torch.arange(32), torch.arange(p0, p0 + 32)] = 1.0
                rk.decompress_matmul_16_8_1(c, cbd, x, out)
                got[:, p0:p0 + 32] = np_f16(out).T
    finally:
        rk.set_timing(prev_timing)
    g, w = got.view(np.uint16), want.view(np.uint16)
    nz = (w & 0x7FFF) != 0
    assert np.array_equal(g[nz], w[nz])
    assert np.all((g[~nz] & 0x7FFF) == 0)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("batch", [1, 16, 19, 32])
@pytest.mark.parametrize("m,n", [(16, 2048), (33, 2048 + 704), (5, 704), (300, 6144)])
def test_matmul_bits_output_within_tolerance(rk, oracle, mode, bits, S, batch, m, n):
    """3 and 4 bits per weight on the matrix cores against the double-precision product of the oracle's dense matrix."""
    comp = rand_codes(m * n * bits // 32, seed=m + n + batch + bits)
    cb = rand_half(2 << S, seed=S + 60)
    x = rand_half(batch * n, seed=19).reshape(batch, n)
    out = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        ms = rk.decompress_matmul_bits(comp.cuda(), cb.cuda(), x.cuda(), out, bits)
    assert ms > 0
    W = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=mode)
    want = np_f16(x).astype(np.float64) @ W.astype(np.float64).T
    got = np_f16(out).astype(np.float64)
    assert np.all(np.isfinite(got))
    assert rel_l2(got, want) < REL_L2_TOL


@pytest.mark.parametrize("bits", [3, 4])
def test_matmul_bits_identity_batch_recovers_weights_bit_exactly(rk, oracle, bits):
    S, m, n, mode = 8, 40, 2048 + 128, 1
    comp = rand_codes(m * n * bits // 32, seed=654 + bits)
    cb = rand_half(2 << S, seed=61)
    want = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=mode)
    c, cbd = comp.cuda(), cb.cuda()
    got = np.zeros((m, n), dtype=np.float16)
    out = torch.zeros((32, m), dtype=torch.float16, device="cuda")
    prev_timing = rk.set_timing(False)
    try:
        with with_mode(rk, mode):
            for p0 in range(0, n, 32):
                x = torch.zeros((32, n), dtype=torch.float16, device="cuda")
                x[torch.arange(32), torch.arange(p0, p0 + 32)] = 1.0
                rk.decompress_matmul_bits(c, cbd, x, out, bits)
                got[:, p0:p0 + 32] = np_f16(out).T
    finally:
        rk.set_timing(prev_timing)
    g, w = got.view(np.uint16), want.view(np.uint16)
    nz = (w & 0x7FFF) != 0
    assert np.array_equal(g[nz], w[nz])
    assert np.all((g[~nz] & 0x7FFF) == 0)


@pytest.mark.parametrize("bits", [3, 4])
def test_matmul_bits_full_size_equals_the_mat_vec(rk, bits):
    """At the full layer size the batched product must agree, row by row, with the mat-vec kernel of the same stream."""
    S, m, n, batch = 8, 4096, 11008, 16
    comp = rand_codes(m * n * bits // 32, seed=42).cuda()
    cb = rand_half(2 << S, seed=43).cuda()
    x = rand_half(batch * n, seed=44).reshape(batch, n).cuda()
    out = torch.zeros((batch, m), dtype=torch.float16, device="cuda")
    rk.decompress_matmul_bits(comp, cb, x, out, bits)
    for b in (0, 7, 15):
        y = torch.zeros(m, dtype=torch.float16, device="cuda")
        rk.decompress_matvec_bits(comp, cb, x[b].contiguous(), y, bits)
        assert rel_l2(np_f16(out[b]), np_f16(y).astype(np.float64)) < REL_L2_TOL


@pytest.mark.parametrize("m,n", [(8192, 8192), (28672, 8192), (8192, 28672)])
def test_matmul_70b_shapes_batch_16(rk, m, n):
    """Batch 16 on the Llama-3-70B layer shapes (several row groups per slab, up to 14 slabs to merge) against
    the double-precision product of the exported dense matrix."""
    S, batch = 8, 16
    comp = rand_codes(m * n // 16, seed=91).cuda()
    cb = rand_half(2 << S, seed=92).cuda()
    x = rand_half(batch * n, seed=93).reshape(batch, n).cuda()
    out = torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda")
    rk.decompress_matmul_16_8_1(comp, cb, x, out)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    rk.matvec_dense(comp, cb, W, S)
    want = torch.cat([x.double() @ W[r0:r0 + 4096].double().t() for r0 in range(0, m, 4096)], dim=1)
    assert rel_l2(np_f16(out), want.cpu().numpy()) < REL_L2_TOL
    # twice in a row: the arrival counters must be back at zero after a call
    out2 = torch.full_like(out, float("nan"))
    rk.decompress_matmul_16_8_1(comp, cb, x, out2)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


@pytest.mark.parametrize("m,n", [(4096, 11008), (11008, 4096)])
@pytest.mark.parametrize("batch", [8, 16, 32])
def test_matmul_full_size_equals_decode_then_dense_gemm(rk, oracle, batch, m, n):
    S = 8
    comp = rand_codes(m * n // 16, seed=42)
    cb = rand_half(2 << S, seed=43)
    x = rand_half(batch * n, seed=44).reshape(batch, n)
    out = torch.zeros((batch, m), dtype=torch.float16, device="cuda")
    rk.decompress_matmul_16_8_1(comp.cuda(), cb.cuda(), x.cuda(), out)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    rk.matvec_dense(comp.cuda(), cb.cuda(), W, S)
    want = (x.cuda().double() @ W.double().t()).cpu().numpy()
    assert rel_l2(np_f16(out), want) < REL_L2_TOL
    # and the batch-1 kernel agrees with row 0
    y = torch.zeros((m,), dtype=torch.float16, device="cuda")
    rk.decompress_matvec_16_8_1(comp.cuda(), cb.cuda(), x[0].cuda().contiguous(), y)
    assert rel_l2(np_f16(y), want[0]) < REL_L2_TOL


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("batch", [8, 32])
def test_matmul_with_a_caller_workspace_is_bit_identical_and_reentrant(rk, bits, batch):
    """rptc_decompress_matmul_ws: the same kernels with the scratch in a buffer of the caller; two calls with two
    workspaces on two streams may overlap, and each equals the static-scratch entry point bit for bit."""
    import ctypes
    lib = rk.library()
    S, m, n = 8, 1024 + 48, 4096 + 768
    comp = rand_codes(m * n * bits // 32, seed=11).cuda()
    cb = rand_half(2 << S, seed=12).cuda()
    xs = [rand_half(batch * n, seed=13 + i).reshape(batch, n).cuda() for i in range(2)]
    want = [torch.zeros((batch, m), dtype=torch.float16, device="cuda") for _ in range(2)]
    for i in range(2):
        rk.decompress_matmul_bits(comp, cb, xs[i], want[i], bits)
    need = lib.rptc_decompress_matmul_workspace_bytes(m, n, batch, bits)
    assert need > 0
    ws = [torch.full((need,), 0xA5, dtype=torch.uint8, device="cuda") for _ in range(2)]      # garbage on purpose
    got = [torch.full((batch, m), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        for i in range(2):
            rc = lib.rptc_decompress_matmul_ws(comp.data_ptr(), cb.data_ptr(), xs[i].data_ptr(), got[i].data_ptr(), m, n, batch,
                                               S, bits, 0, ws[i].data_ptr(), need, ctypes.c_void_p(streams[i].cuda_stream), None)
            assert rc == 0, lib.rptc_status_string(rc)
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(got[i].view(torch.int16), want[i].view(torch.int16))
    # too small a workspace, a misaligned one, none at all
    assert lib.rptc_decompress_matmul_ws(comp.data_ptr(), cb.data_ptr(), xs[0].data_ptr(), got[0].data_ptr(), m, n, batch, S, bits,
                                         0, ws[0].data_ptr(), need - 256, None, None) == -5
    assert lib.rptc_decompress_matmul_ws(comp.data_ptr(), cb.data_ptr(), xs[0].data_ptr(), got[0].data_ptr(), m, n, batch, S, bits,
                                         0, ws[0].data_ptr() + 16, need, None, None) == -3
    assert lib.rptc_decompress_matmul_ws(comp.data_ptr(), cb.data_ptr(), xs[0].data_ptr(), got[0].data_ptr(), m, n, batch, S, bits,
                                         0, None, need, None, None) == -1


def test_arrival_counters_are_zero_after_the_split_ops(rk):
    """rptc_scratch_check: after ops that merge across workgroups (batched product, transposed mat-vec on a short
    matrix) every arrival counter is back at zero."""
    import ctypes
    lib = rk.library()
    S, m, n, batch = 8, 512, 4096, 8
    comp = rand_codes(m * n // 16, seed=21).cuda()
    out = torch.zeros((batch, m), dtype=torch.float16, device="cuda")
    rk.decompress_matmul_16_8_1(comp, rand_half(2 << S, seed=22).cuda(), rand_half(batch * n, seed=23).reshape(batch, n).cuda(), out)
    y = torch.zeros(m, dtype=torch.float16, device="cuda")
    rk.decompress_matvec_t_16(comp, rand_half(1 << 16, seed=24).cuda(), rand_half(n, seed=25).cuda(), y)
    nz = ctypes.c_int(-1)
    assert lib.rptc_scratch_check(0, ctypes.byref(nz), None) == 0
    assert nz.value == 0
    assert lib.rptc_scratch_check(1, None, None) == -1


def test_matmul_rejects_bad_arguments(rk):
    cb = torch.zeros(512, dtype=torch.float16, device="cuda")
    comp = torch.zeros(32 * 2048 // 16, dtype=torch.int32, device="cuda")
    x = torch.zeros((4, 2048), dtype=torch.float16, device="cuda")
    out = torch.zeros((4, 32), dtype=torch.float16, device="cuda")
    f = rk.decompress_matmul_16_8_1
    with pytest.raises(RuntimeError):
        f(comp, cb, x[0], out)                                  # x must be 2-D
    with pytest.raises(RuntimeError):
        f(comp, cb, x, out[:2])                                 # batch mismatch
    with pytest.raises(RuntimeError):
        f(comp, cb, torch.zeros((33, 2048), dtype=torch.float16, device="cuda"),
          torch.zeros((33, 32), dtype=torch.float16, device="cuda"))      # batch > 32
    with pytest.raises(RuntimeError):
        f(comp[:100], cb, x, out)                               # stream size
    assert f(comp, cb, x, out) >= 0.0


# ------------------------------------------------------------------ sign-Hadamard transform

@pytest.mark.parametrize("batch,n,block", [(1, 4096, 0), (3, 11008, 0), (2, 28672, 0), (1, 64, 0), (4, 8192, 256),
                                           (1, 32768, 0), (2, 704, 0)])
@pytest.mark.parametrize("inverse", [False, True])
def test_sign_hadamard_matches_oracle(rk, oracle, batch, n, block, inverse):
    x = rand_half(batch * n, seed=n).reshape(batch, n)
    signs = torch.where(torch.rand(n, generator=torch.Generator().manual_seed(n)) < 0.5, -1.0, 1.0).to(torch.float16)
    out = torch.zeros_like(x, device="cuda")
    ms = rk.sign_hadamard(x.cuda(), signs.cuda(), out, block=block, inverse=inverse)
    assert ms > 0
    P = block or rk.hadamard_block(n)
    want = oracle.sign_hadamard(np_f16(x), np_f16(signs), P, inverse=inverse)
    # fp32 butterflies, one fp16 rounding at the end: 2^-11 relative per element
    assert rel_l2(np_f16(out), want) < REL_L2_TOL


def test_sign_hadamard_round_trip_and_norm(rk):
    n = 11008
    x = rand_half(2 * n, seed=3).reshape(2, n).cuda()
    signs = torch.where(torch.rand(n, generator=torch.Generator().manual_seed(1)) < 0.5, -1.0, 1.0).to(torch.float16).cuda()
    y = torch.zeros_like(x)
    z = torch.zeros_like(x)
    rk.sign_hadamard(x, signs, y)
    rk.sign_hadamard(y, signs, z, inverse=True)
    assert rel_l2(z.cpu().numpy(), x.cpu().numpy()) < REL_L2_TOL
    assert abs(y.double().norm().item() / x.double().norm().item() - 1.0) < 1e-3
    # in place
    rk.sign_hadamard(y, signs, y, inverse=True)
    assert torch.equal(y, z)


# ------------------------------------------------------------------ 3 and 4 bits per weight (no reference counterpart)

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("m,n", [(32, 2048), (33, 4096 + 768), (7, 704), (512, 6144)])
def test_matvec_bits_dense_and_output(rk, oracle, mode, bits, S, m, n):
    comp = rand_codes(m * n * bits // 32, seed=m + n + bits)
    cb = rand_half(2 << S, seed=S + 40)
    x = rand_half(n, seed=11)
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    out = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    with with_mode(rk, mode):
        rk.matvec_bits_dense(comp.cuda(), cb.cuda(), W, bits)
        ms = rk.decompress_matvec_bits(comp.cuda(), cb.cuda(), x.cuda(), out, bits)
    assert ms > 0
    want = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=mode)
    assert np.array_equal(np_f16(W).view(np.uint16), want.view(np.uint16))
    y = oracle.dense_matvec(want, np_f16(x))
    assert rel_l2(np_f16(out), y) < REL_L2_TOL


@pytest.mark.parametrize("bits", [3, 4])
def test_matvec_bits_fused_kernel_decodes_bit_exactly(rk, oracle, bits):
    S, m, n = 8, 64, 2048 + 192
    comp = rand_codes(m * n * bits // 32, seed=55 + bits)
    cb = rand_half(2 << S, seed=56)
    want = oracle.bits_dense(np_u32(comp), np_f16(cb), m, n, S, bits, mode=1)
    c, cbd = comp.cuda(), cb.cuda()
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    x = torch.zeros(n, dtype=torch.float16, device="cuda")
    got = np.zeros((m, n), dtype=np.float16)
    prev_timing = rk.set_timing(False)
    cols = sorted(set(list(range(0, n, 5)) + list(range(n - 200, n))))
    try:
        with with_mode(rk, 1):
            for p in cols:
                x.zero_()
                x[p] = 1.0
                rk.decompress_matvec_bits(c, cbd, x, out, bits)
                got[:, p] = np_f16(out)
    finally:
        rk.set_timing(prev_timing)
    g, w = got[:, cols].view(np.uint16), want[:, cols].view(np.uint16)
    nz = (w & 0x7FFF) != 0
    assert np.array_equal(g[nz], w[nz])
    assert np.all((g[~nz] & 0x7FFF) == 0)


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("m,n", [(4096, 11008), (11008, 4096)])
def test_matvec_bits_full_size(rk, oracle, bits, m, n):
    S = 8
    comp = rand_codes(m * n * bits // 32, seed=42).cuda()
    cb = rand_half(2 << S, seed=43).cuda()
    x = rand_half(n, seed=44).cuda()
    out = torch.zeros((m,), dtype=torch.float16, device="cuda")
    W = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    rk.decompress_matvec_bits(comp, cb, x, out, bits)
    rk.matvec_bits_dense(comp, cb, W, bits)
    want = (W.double() @ x.double()).cpu().numpy()
    assert rel_l2(np_f16(out), want) < REL_L2_TOL
    # the dense export is held to the oracle on a subset of rows taken from all over the matrix (the whole matrix
    # at this size takes the CPU a while): a stream of just those rows has the same layout with m = rows
    rows = np.array(sorted({0, 1, 31, 32, 33, m // 2 - 1, m // 2, m - 64, m - 2, m - 1} | set(range(1000, 1032))))
    words = 2 * bits
    idx = np_u32(comp).reshape(-1)
    T, Lt = n // 2048, (n % 2048) // 64
    parts = [idx[t * m * 32 * words:(t + 1) * m * 32 * words].reshape(m, 32 * words)[rows].reshape(-1) for t in range(T)]
    if Lt:
        parts.append(idx[T * m * 32 * words:].reshape(m, Lt * words)[rows].reshape(-1))
    wantW = oracle.bits_dense(np.concatenate(parts), np_f16(cb), len(rows), n, S, bits, mode=0)
    assert np.array_equal(np_f16(W[torch.from_numpy(rows).cuda()]).view(np.uint16), wantW.view(np.uint16))

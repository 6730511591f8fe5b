"""The decode-only kernel, the per-launch mat-vec kernel, the chain's loop kernel, the transposed mat-vec kernel, the batched
kernel (matrix instructions, partial tiles handed over between workgroups), the sign-Hadamard transform and the general
trellis' dequantize kernels, as compiled, run on the CPU in a functional wave
model (`tests/wave_model.py`) against the oracle: every global access bounds-checked, loads completing late, registers and LDS full of garbage at the start, the
sixteen waves of a workgroup interleaved at random.  What the GPU tests cannot show: an access outside the buffers, or
a register used before its wait, is a test failure that names the instruction here and a dead process there.

Needs hipcc (cross-compiles without a GPU).  The descriptors are packed here as `matvec_loop_plan` packs them
(`csrc/matvec.hip`, `struct LoopLayer` in `csrc/matvec_loop.hpp`)."""
import importlib.util
import os
import shutil
import struct
import subprocess

import numpy as np
import pytest

import wave_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "let-it-slide_amd")
CUS = 256                        # the grid the planner makes on the target: one workgroup per compute unit


def compile_to_assembly(tmp_path_factory, name, extra=()):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not found")
    spec = importlib.util.spec_from_file_location("rptc_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = str(tmp_path_factory.mktemp("isa") / (name + ".s"))
    subprocess.run(["hipcc", *mod.FLAGS, *extra, "--cuda-device-only", "-S", os.path.join(PKG, "csrc", name + ".hip"), "-o", out],
                   check=True, capture_output=True)
    return out


@pytest.fixture(scope="module")
def matvec_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec")


@pytest.fixture(scope="module")
def lite_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "lite")


@pytest.fixture(scope="module")
def decompress_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "decompress")


@pytest.fixture(scope="module")
def matvec_t_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_t")


@pytest.fixture(scope="module")
def matmul_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matmul")


@pytest.fixture(scope="module")
def hadamard_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "hadamard")


def plan(shapes, addresses):
    """LoopLayer records and the launch's LDS geometry for layers of `shapes`, as the host planner computes them."""
    raw = bytearray()
    n_max = part_max = items_max = 0
    for i, ((m, n), (comp_at, x_at, out_at)) in enumerate(zip(shapes, addresses)):
        rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
        lt = (n & 2047) >> 6
        items_full = rpb // 2
        rw_tail = 64 // lt if lt else 1
        items_tail = (rpb + rw_tail - 1) // rw_tail if lt else 0
        magic = ((1 << 32) // items_full + 1) if items_full > 1 else 0
        same = 1 if i > 0 and shapes[i - 1] == (m, n) else 0
        raw += struct.pack("<QQQiiiiiIiiii", comp_at, x_at, out_at, m, n, rpb, rw_tail, items_tail, magic, same, 0, 0, 0)
        n_max, part_max = max(n_max, n), max(part_max, rpb * (n // 64))
        items_max = max(items_max, -(-((n >> 11) * items_full + items_tail) // 16))
    assert items_max <= 4
    lds_bytes = 65536 + 2 * (2 * n_max) + 2 * 4 * part_max
    assert lds_bytes <= 160 * 1024
    return np.frombuffer(bytes(raw), dtype=np.uint8).copy(), n_max // 2, part_max, lds_bytes, 3 if items_max <= 3 else 4


def run_chain(isa, oracle, shapes, S, mode, blocks, seed=7, burst=8, latency=(400, 60), shorten=None):
    rng = np.random.default_rng(seed)
    mem = wave_model.Memory()
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    cb_at = 0x7f5000003400
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    layers, addresses = [], []
    for i, (m, n) in enumerate(shapes):
        # one stream straddles a 4 GiB boundary (the carry into the high half of an address), the others sit at odd distances from one
        comp_at = 0x7f4100000000 + (i << 33) - (4096 if i % 3 == 1 else -0x23456700)
        x_at, out_at = 0x7f3ffff0fe00 + (i << 16), 0x7f2ffffe0100 + (i << 15)
        comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
        x = (rng.standard_normal(n) * 0.5).astype(np.float16).view(np.uint8).copy()
        out = np.full(2 * m, 0xEE, dtype=np.uint8)
        mem.add(comp_at, comp[:len(comp) - shorten] if shorten and i == len(shapes) - 1 else comp, f"stream {i}")
        mem.add(x_at, x, f"activations {i}")
        mem.add(out_at, out, f"output {i}")
        layers.append((comp, x, out, m, n))
        addresses.append((comp_at, x_at, out_at))
    desc, xslot_words, part_floats, lds_bytes, maxi = plan(shapes, addresses)
    desc_at = 0x7f6000001000
    mem.add(desc_at, desc, "descriptors")
    kernel = wave_model.Kernel(isa, "_ZN4rptc18matvec_loop_kernelILi%dELi%dELi%dE" % (S, mode, maxi))
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = latency
    kernel.launch(mem, (CUS,), 1024, [("ptr", desc_at), ("ptr", cb_at), ("i32", len(shapes)), ("i32", xslot_words), ("i32", part_floats)],
                  lds_bytes=lds_bytes, groups=[(b, 0, 0) for b in blocks], seed=seed, burst=burst)
    for i, (comp, x, out, m, n) in enumerate(layers):
        want = oracle.matvec(comp.view(np.uint32), cb, x.view(np.float16), m, S, mode=mode)
        got = out.view(np.float16).astype(np.float64)
        rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
        touched = np.zeros(m, dtype=bool)
        for b in blocks:
            r0, r1 = b * rpb, min(m, (b + 1) * rpb)
            if r0 >= r1:
                continue
            touched[r0:r1] = True
            err = np.abs(got[r0:r1] - want[r0:r1]).max() / (np.abs(want).max() + 1e-9)
            assert err < 2e-3, f"layer {i} ({m}x{n}), workgroup {b}: rows {r0}..{r1 - 1} differ by {err:.3g} of the layer's largest output"
        # rows of workgroups that did not run still hold the fill pattern
        assert (out.view(np.uint16)[~touched] == 0xEEEE).all(), f"layer {i}: a row outside the simulated workgroups was written"


RAGGED = [(33, 4096 + 768), (300, 64), (7, 704)]
MIXED = [(64, 2048), (33, 4096 + 768), (512, 6144), (1024, 2048 + 64), (2000, 1984), (2000, 1984)]


@pytest.mark.parametrize("S,mode", [(8, 0), (8, 1), (6, 0), (6, 1)])
def test_loop_kernel_matches_the_oracle(matvec_isa, oracle, S, mode):
    run_chain(matvec_isa, oracle, RAGGED, S, mode, blocks=[0, 1, 255])


def test_loop_kernel_on_mixed_shapes(matvec_isa, oracle):
    run_chain(matvec_isa, oracle, MIXED, 8, 1, blocks=[0, 16, 255])


def test_loop_kernel_where_a_wave_holds_an_empty_item_in_front_of_a_real_one(matvec_isa, oracle):
    """2546 rows are 254 blocks of ten and one of six: in that last block the items of rows 6 to 9 are empty, and the wave
    that holds slab 0's last item (empty) and slab 1's first (rows 0 and 1) must move its load cursor past the empty one."""
    run_chain(matvec_isa, oracle, [(2546, 7744)], 6, 0, blocks=[253, 254, 255])
    run_chain(matvec_isa, oracle, [(2546, 7744), (2546, 7744)], 8, 1, blocks=[254])
    # more of the kind (blocks of ten rows that end after 2, 7 and 8)
    for (m, n), mode in (((2472, 10304), 0), ((2187, 8128), 1), ((2258, 8128), 0)):
        run_chain(matvec_isa, oracle, [(m, n)], 8, mode, blocks=[(m - 1) // 10])


@pytest.mark.parametrize("seed", range(4))
def test_loop_kernel_on_random_shapes(matvec_isa, oracle, seed):
    """Four layers of random shapes; the first workgroup and, of every layer, the one that holds the end of its rows (where
    a row block is partial and items are empty)."""
    rng = np.random.default_rng(300 + seed)
    shapes = [(int(rng.integers(1, 3001)), 64 * int(rng.integers(1, 121))) for _ in range(4)]
    blocks = {0}
    for m, _ in shapes:
        blocks.add((m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS))))
    run_chain(matvec_isa, oracle, shapes, (6, 8)[seed & 1], (seed >> 1) & 1, blocks=sorted(blocks), seed=seed)


def test_loop_kernel_with_one_layer(matvec_isa, oracle):
    run_chain(matvec_isa, oracle, [(64, 2048)], 8, 0, blocks=[0, 31, 32])


@pytest.mark.parametrize("burst,latency", [(10 ** 6, (400, 60)), (8, (3000, 300)), (8, (40, 10))])
def test_loop_kernel_under_other_interleavings_and_latencies(matvec_isa, oracle, burst, latency):
    """Every wave running until it blocks; memory that answers very late; memory that answers at once."""
    run_chain(matvec_isa, oracle, RAGGED, 8, 1, blocks=[0, 255], seed=11, burst=burst, latency=latency)


def test_the_model_reports_an_access_outside_the_buffers(matvec_isa, oracle):
    """The last workgroup with rows reads the stream's last element: with the buffer 16 bytes short the model must say so."""
    with pytest.raises(wave_model.Fault, match="outside every region"):
        run_chain(matvec_isa, oracle, [(64, 2048)], 8, 0, blocks=[31], shorten=16)


@pytest.mark.parametrize("m,n,S,mode", [(64, 2048, 8, 0), (33, 4096 + 768, 8, 1), (300, 64, 6, 0), (1024, 2048 + 64, 6, 1),
                                        (2000, 1984, 8, 1), (7, 704, 8, 0), (5, 16384, 8, 1), (512, 6144, 6, 0)])
def test_per_launch_kernel_matches_the_oracle(matvec_isa, oracle, m, n, S, mode):
    """`matvec_kernel<S, MODE, 2, false>` (what `rptc_decompress_matvec_16_8_1` and its siblings launch), with the
    geometry of `plan_matvec` in `csrc/matvec.hip`; the first and the last workgroup and one in between."""
    rng = np.random.default_rng(m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    out = np.full(2 * m, 0xEE, dtype=np.uint8)
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100     # the stream straddles 4 GiB
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x.view(np.uint8).copy(), "activations")
    mem.add(o_at, out, "output")
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    lt = (n & 2047) >> 6
    rw_tail = 64 // lt if lt else 1
    items_full = rpb // 2
    items_tail = (rpb + rw_tail - 1) // rw_tail if lt else 0
    magic = ((1 << 32) // items_full + 1) if items_full > 1 else 0
    lds_bytes = 65536 + 2 * n + 4 * (n // 64) * rpb
    assert lds_bytes <= 160 * 1024
    grid = (m + rpb - 1) // rpb
    blocks = sorted({0, grid // 2, grid - 1})
    kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                       ("i32", items_tail), ("u32", magic), ("ptr", o_at)], lds_bytes=lds_bytes,
                  groups=[(b, 0, 0) for b in blocks], seed=m)
    want = oracle.matvec(comp.view(np.uint32), cb, x, m, S, mode=mode)
    got = out.view(np.float16).astype(np.float64)
    touched = np.zeros(m, dtype=bool)
    for b in blocks:
        r0, r1 = b * rpb, min(m, (b + 1) * rpb)
        touched[r0:r1] = True
        err = np.abs(got[r0:r1] - want[r0:r1]).max() / (np.abs(want).max() + 1e-9)
        assert err < 2e-3, f"workgroup {b}: rows {r0}..{r1 - 1} differ by {err:.3g} of the largest output"
    assert (out.view(np.uint16)[~touched] == 0xEEEE).all()


@pytest.mark.parametrize("L,S,R,V,rows,length", [(16, 9, 4, 2, 3, 1000), (16, 9, 4, 2, 3, 2048), (16, 9, 4, 2, 2, 1023),
                                                  (20, 13, 3, 2, 2, 515), (16, 8, 2, 3, 2, 300), (12, 6, 5, 1, 3, 77)])
def test_lite_dequantize_kernels_match_the_oracle(lite_isa, oracle, L, S, R, V, rows, length):
    """Both kernels of `csrc/lite.hip` (pairs with the alphabet in LDS and without, and the general one), launched as
    `rptc_lite_dequantize` launches them, with fewer workgroups than sequences so that the row loop strides, outputs
    at 8- and 16-byte alignments, and one symbol outside its range."""
    pairs = V == 2
    name = "_ZN4rptc28lite_dequantize_pairs_kernelILb%dE" % (1 if S <= 12 else 0) if pairs else "_ZN4rptc22lite_dequantize_kernelE"
    kernel = wave_model.Kernel(lite_isa, name)
    rng = np.random.default_rng(L * 1000 + length)
    alphabet = rng.standard_normal((1 << S, V)).astype(np.float32)
    symbols = rng.integers(0, 1 << R, (rows, length), dtype=np.int32)
    symbols[0, 17] = -5
    out = np.full((rows, length, V), np.nan, dtype=np.float32)
    out_bytes = out.view(np.uint8).reshape(-1)
    a_at, s_at, o_at = 0x7f0000100000, 0x7f0000300004, 0x7f0000500000 + (8 if length % 3 == 0 else 0)
    history = (32 + R - 1) // R - 1
    grid_y = min(rows, 2)
    for latency in ((400, 60), (30, 8)):
        mem = wave_model.Memory()
        mem.add(a_at, alphabet.view(np.uint8).reshape(-1), "alphabet")
        mem.add(s_at, symbols.view(np.uint8).reshape(-1), "symbols")
        mem.add(o_at, out_bytes, "output")
        out_bytes[:] = 0xFF
        wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = latency
        if pairs:
            lds = (32 + 512) * 4 + ((8 << S) if S <= 12 else 0)
            kernel.launch(mem, ((length + 511) // 512, grid_y), 256,
                          [("ptr", a_at), ("ptr", s_at), ("ptr", o_at), ("i64", length), ("i32", rows), ("i32", R), ("i32", history),
                           ("i32", L - S), ("u32", (1 << S) - 1)], lds_bytes=lds)
        else:
            chunks = (length + 7) // 8
            kernel.launch(mem, ((chunks + 255) // 256, grid_y), 256,
                          [("ptr", a_at), ("ptr", s_at), ("ptr", o_at), ("i64", length), ("i32", rows), ("u32", chunks), ("i32", R),
                           ("i32", history), ("i32", L - S), ("u32", (1 << S) - 1), ("i32", V)])
        want = np.stack([oracle.lite_dequantize(alphabet, L, S, R, symbols[r]) for r in range(rows)])
        assert np.array_equal(out.view(np.uint32), want.reshape(out.shape).view(np.uint32))


@pytest.mark.parametrize("m,words_per_row,mode,grid", [(3, 128, 0, 1), (5, 256, 1, 2), (2, 384, 1, 3)])
def test_decompress_kernel_matches_the_oracle(decompress_isa, oracle, m, words_per_row, mode, grid):
    """`decompress_kernel<MODE>` as `rptc_decompress` launches it, with fewer workgroups than the rows need (the
    kernel strides), bit for bit."""
    rng = np.random.default_rng(m * words_per_row)
    codebook = rng.integers(0, 65536, 65536, dtype=np.uint16)
    stream = rng.integers(0, 1 << 32, (m, words_per_row), dtype=np.uint64).astype(np.uint32)
    out = np.full((m, 16 * words_per_row), 0xEEEE, dtype=np.uint16)
    mem = wave_model.Memory()
    c_at, cb_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f2ffffe0100
    mem.add(c_at, stream.view(np.uint8).reshape(-1), "stream")
    mem.add(cb_at, codebook.view(np.uint8), "codebook")
    mem.add(o_at, out.view(np.uint8).reshape(-1), "output")
    groups = 2 * m * words_per_row
    kernel = wave_model.Kernel(decompress_isa, "_ZN4rptc17decompress_kernelILi%dE" % mode)
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", o_at), ("u32", words_per_row), ("u32", groups)],
                  lds_bytes=131072, seed=m)
    want = oracle.decompress(stream.view(np.int32), codebook, mode=mode).view(np.uint16)
    assert np.array_equal(out, want)


@pytest.mark.parametrize("m,n,L,mode,ksplit", [(100, 256, 16, 0, 1), (70, 512, 14, 1, 1), (64, 1024, 16, 1, 1), (64, 4096, 16, 1, 2),
                                               (130, 8192, 14, 0, 3), (5, 64, 14, 0, 1)])
def test_transposed_kernel_matches_the_oracle(matvec_t_isa, oracle, m, n, L, mode, ksplit):
    """`matvec_t_kernel<L, MODE>` as `launch_matvec_t` (`csrc/matvec_t.hip`) launches it: `out +=`, one workgroup per 64
    rows and, with `ksplit` > 1, several per row block that hand their partial sums over through memory (the model runs
    the workgroups one after the other, so the last one finds every arrival and adds the parts up)."""
    rng = np.random.default_rng(m + n + L)
    codebook = (rng.standard_normal(1 << L) * 0.1).astype(np.float16)
    cols = n // 64
    stream = rng.integers(0, 1 << 32, 4 * cols * m, dtype=np.uint64).astype(np.uint32)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    before = (rng.standard_normal(m) * 0.1).astype(np.float16)
    out = before.copy()
    parts, arrived = np.zeros(4096 * 64, dtype=np.float32), np.zeros(4096, dtype=np.uint32)
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at, p_at, a_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100, 0x7f6000000000, 0x7f6100000000
    mem.add(c_at, stream.view(np.uint8), "stream")
    mem.add(cb_at, codebook.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x.view(np.uint8).copy(), "activations")
    mem.add(o_at, out.view(np.uint8), "output")
    mem.add(p_at, parts.view(np.uint8), "partial sums")
    mem.add(a_at, arrived.view(np.uint8), "arrival counters")
    row_blocks = (m + 63) // 64
    lds_bytes = (2 << L) + 512 * 4 + (((cols + ksplit - 1) // ksplit) * 32 if mode == 0 else 0)
    kernel = wave_model.Kernel(matvec_t_isa, "_ZN4rptc15matvec_t_kernelILi%dELi%dEE" % (L, mode))
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel.launch(mem, (row_blocks * ksplit,), 512,
                  [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", cols), ("i32", ksplit), ("ptr", o_at), ("ptr", p_at),
                   ("ptr", a_at)], lds_bytes=lds_bytes, seed=m)
    want = before.astype(np.float64) + oracle.matvec_t(stream, codebook, x, m, L, mode=mode)
    err = np.abs(out.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-9)
    assert err < 3e-3
    assert not arrived.any(), "an arrival counter was left non-zero"


@pytest.mark.parametrize("m,n,batch,S,mode", [(40, 2048 + 128, 5, 8, 0), (16, 2048, 16, 6, 1), (100, 704, 20, 8, 1), (33, 4096, 2, 6, 0)])
def test_batched_kernel_matches_the_oracle(matmul_isa, oracle, m, n, batch, S, mode):
    """`pack_x_kernel` and `matmul_kernel<S, MODE, PLANES, 2>` as `run_matmul` (`csrc/matmul.hip`) launches them: the
    activations packed into the B operand's order, the arrival counters cleared whatever they held, one workgroup per
    (row group, slab), the last workgroup of a row group to arrive adding the slabs' tiles up (the model runs the workgroups
    one after the other).  One and two planes of 16 batch columns."""
    rng = np.random.default_rng(m + n + batch)
    codebook = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    stream = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal((batch, n)) * 0.5).astype(np.float16)
    out = np.full((batch, m), np.nan, dtype=np.float16)
    planes = 2 if batch > 16 else 1
    slabs = n // 2048 + (1 if n % 2048 else 0)
    total = (m + 15) // 16                                  # row blocks of 16 rows
    groups = max(1, min(2 * CUS // slabs, total))
    groups = max(groups, -(-total // (8 if planes == 1 else 6)))
    max_rb = -(-total // groups)
    xpack = np.zeros(planes * (n // 2) * 16, dtype=np.uint32)
    partial = np.zeros(groups * slabs * max_rb * planes * 256, dtype=np.float32)
    arrived = np.full(groups, 0xABCD, dtype=np.uint32)
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
    xp_at, p_at, a_at = 0x7f6000000000, 0x7f6100000000, 0x7f6200000000
    for at, data, name in ((c_at, stream, "stream"), (cb_at, codebook.view(np.uint8).copy(), "codebook"),
                           (x_at, x.view(np.uint8).reshape(-1).copy(), "activations"), (o_at, out.view(np.uint8).reshape(-1), "output"),
                           (xp_at, xpack.view(np.uint8), "packed activations"), (p_at, partial.view(np.uint8), "partial tiles"),
                           (a_at, arrived.view(np.uint8), "arrival counters")):
        mem.add(at, data, name)
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    pack = wave_model.Kernel(matmul_isa, "_ZN4rptc13pack_x_kernelE")
    threads = max(planes * (n // 8) * 16, groups)
    pack.launch(mem, ((threads + 255) // 256,), 256,
                [("ptr", x_at), ("ptr", xp_at), ("ptr", a_at), ("i32", groups), ("i32", n), ("i32", batch), ("i32", planes)], seed=m)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    kernel = wave_model.Kernel(matmul_isa, "_ZN4rptc13matmul_kernelILi%dELi%dELi%dELi2EE" % (S, mode, planes))
    kernel.launch(mem, (groups * slabs,), 512,
                  [("ptr", c_at), ("ptr", cb_at), ("ptr", xp_at), ("i32", m), ("i32", n), ("i32", total // groups), ("i32", total % groups),
                   ("i32", 0), ("i32", max_rb), ("ptr", p_at), ("ptr", a_at), ("ptr", o_at), ("i32", batch)],
                  lds_bytes=65536 + 8 * 2 * 256 * 4, seed=m)
    want = np.stack([oracle.matvec(stream.view(np.uint32), codebook, x[b], m, S, mode=mode) for b in range(batch)])
    err = np.abs(out.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-9)
    assert err < 2e-3


@pytest.mark.parametrize("m,n,batch,S,mode,tiles", [(16, 2048 + 768, 16, 8, 0, 1), (40, 4096 + 64 * 5, 5, 6, 1, 3), (30, 64 * 3, 16, 8, 1, 2),
                                                        (48, 2048 * 3, 9, 8, 0, 1), (20, 2048 + 64 * 30, 3, 6, 0, 2)])
def test_row_owner_batched_kernel_matches_the_oracle(matmul_isa, oracle, m, n, batch, S, mode, tiles):
    """`pack_x_tuples_kernel` and `matmul_rows_kernel<S, MODE, TILES>` (`csrc/matmul.hip`): the activations packed as the
    16-byte B operands of the MFMAs with a ragged slab padded by zeros, one workgroup per `tiles` blocks of 16 rows over
    the whole width, a wave's accumulators running over its (slab, four lanes-of-row) pairs.  Ragged widths that are and
    are not a multiple of four lanes-of-row, fewer pairs than waves, more than two pairs a wave, rows past m."""
    rng = np.random.default_rng(m + n + batch)
    codebook = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    stream = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal((batch, n)) * 0.5).astype(np.float16)
    out = np.full((batch, m), np.nan, dtype=np.float16)
    T, Lt = n // 2048, n % 2048 // 64
    xpack = np.full((32 * T + (Lt + 3) // 4 * 4) * 512, 0x7E007E00, dtype=np.uint32)        # NaNs wherever nothing is written
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at, xp_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100, 0x7f6000000000
    for at, data, name in ((c_at, stream, "stream"), (cb_at, codebook.view(np.uint8).copy(), "codebook"),
                           (x_at, x.view(np.uint8).reshape(-1).copy(), "activations"), (o_at, out.view(np.uint8).reshape(-1), "output"),
                           (xp_at, xpack.view(np.uint8), "packed activations")):
        mem.add(at, data, name)
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    pack = wave_model.Kernel(matmul_isa, "_ZN4rptc20pack_x_tuples_kernelE")
    pack.launch(mem, (((n // 8) * 16 + 384 + 255) // 256,), 256, [("ptr", x_at), ("ptr", xp_at), ("i32", n), ("i32", batch)], seed=m)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    kernel = wave_model.Kernel(matmul_isa, "_ZN4rptc18matmul_rows_kernelILi%dELi%dELi%dEE" % (S, mode, tiles))
    total = (m + 15) // 16
    kernel.launch(mem, (-(-total // tiles),), 1024,
                  [("ptr", c_at), ("ptr", cb_at), ("ptr", xp_at), ("ptr", o_at), ("i32", m), ("i32", n), ("i32", batch)],
                  lds_bytes=65536 + 16 * tiles * 1024, seed=m)
    want = np.stack([oracle.matvec(stream.view(np.uint32), codebook, x[b], m, S, mode=mode) for b in range(batch)])
    err = np.abs(out.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-9)
    assert err < 2e-3


@pytest.mark.parametrize("seed", range(3))
def test_row_owner_batched_kernel_on_random_shapes(matmul_isa, oracle, seed):
    import random
    rnd = random.Random(300 + seed)
    for _ in range(3):
        n = 64 * rnd.choice([1, 2, 3, 4, 5, 31, 32, 33, 35, 36, 47, 64, 65, 66, 96, 127, 128])
        m = rnd.choice([1, 2, 15, 16, 17, 31, 33, 48, 50, 64, 80])
        test_row_owner_batched_kernel_matches_the_oracle(matmul_isa, oracle, m, n, rnd.randint(1, 16), rnd.choice([6, 8]), rnd.choice([0, 1]),
                                                         rnd.choice([1, 2, 3]))


@pytest.mark.parametrize("batch,n,block,inverse,misalign", [(2, 512, 256, 0, 0), (1, 1024, 1024, 1, 0), (3, 192, 64, 0, 2), (1, 12, 4, 1, 0),
                                                            (1, 2048 + 512, 512, 0, 0)])
def test_sign_hadamard_kernel_matches_the_oracle(hadamard_isa, oracle, batch, n, block, inverse, misalign):
    """`sign_hadamard_kernel` as `rptc_sign_hadamard` launches it: one workgroup per block, 16-byte accesses where the
    block and the three addresses allow them, two-byte ones otherwise."""
    rng = np.random.default_rng(n + block)
    x = rng.standard_normal((batch, n)).astype(np.float16)
    signs = np.where(rng.integers(0, 2, n) == 1, 1.0, -1.0).astype(np.float16)
    out = np.full((batch, n), np.nan, dtype=np.float16)
    mem = wave_model.Memory()
    x_at, s_at, o_at = 0x7f3ffff0fe00 + misalign, 0x7f5000003400, 0x7f2ffffe0100
    mem.add(x_at, x.view(np.uint8).reshape(-1).copy(), "input")
    mem.add(s_at, signs.view(np.uint8).copy(), "signs")
    mem.add(o_at, out.view(np.uint8).reshape(-1), "output")
    wide = 1 if block % 8 == 0 and misalign % 16 == 0 else 0
    kernel = wave_model.Kernel(hadamard_isa, "_ZN4rptc20sign_hadamard_kernelE")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel.launch(mem, (batch * (n // block),), 256,
                  [("ptr", x_at), ("ptr", s_at), ("ptr", o_at), ("i32", n), ("i32", block), ("i32", block.bit_length() - 1),
                   ("i32", n // block), ("i32", inverse), ("i32", wide)], lds_bytes=(block + block // 32) * 4, seed=n)
    want = oracle.sign_hadamard(x, signs, block, inverse=bool(inverse))
    err = np.abs(out.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-9)
    assert err < 2e-3


# ---------------------------------------------------------------------------------------------------------------------
# matvec_steady_kernel: the chain of equal layers whose loop is one block of hand-written assembly (csrc/matvec_steady.hip)

@pytest.fixture(scope="module")
def steady_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_steady")


def run_steady(isa, oracle, m, n, count, S, mode, blocks, seed=7, burst=8, latency=(400, 60)):
    rng = np.random.default_rng(seed)
    mem = wave_model.Memory()
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    cb_at = 0x7f5000003400
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    layers, addresses = [], []
    for i in range(count):
        comp_at = 0x7f4100000000 + (i << 33) - (4096 if i % 3 == 1 else -0x23456700)
        x_at, out_at = 0x7f3ffff0fe00 + (i << 16), 0x7f2ffffe0100 + (i << 15)
        comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
        x = (rng.standard_normal(n) * 0.5).astype(np.float16).view(np.uint8).copy()
        out = np.full(2 * m, 0xEE, dtype=np.uint8)
        mem.add(comp_at, comp, f"stream {i}")
        mem.add(x_at, x, f"activations {i}")
        mem.add(out_at, out, f"output {i}")
        layers.append((comp, x, out))
        addresses.append((comp_at, x_at, out_at))
    desc, _, part_floats, _, maxi = plan([(m, n)] * count, addresses)
    assert part_floats * 4 <= 16384 and ((n >> 11) + (1 if n & 2047 else 0)) * 4096 <= 32768, "outside the steady kernel's layout"
    desc_at = 0x7f6000001000
    mem.add(desc_at, desc, "descriptors")
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    lt = (n & 2047) >> 6
    rw_tail = 64 // lt if lt else 1
    items_tail = (rpb + rw_tail - 1) // rw_tail if lt else 0
    items_full = rpb // 2
    magic = ((1 << 32) // items_full + 1) if items_full > 1 else 0
    kernel = wave_model.Kernel(isa, "_ZN4rptc20matvec_steady_kernelILi%dELi%dELi%dE" % (S, mode, maxi))
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = latency
    kernel.launch(mem, (CUS,), 1024, [("ptr", desc_at), ("ptr", cb_at), ("i32", count), ("i32", m), ("i32", n), ("i32", rpb),
                                      ("i32", rw_tail), ("i32", items_tail), ("u32", magic)],
                  lds_bytes=160 * 1024, groups=[(b, 0, 0) for b in blocks], seed=seed, burst=burst)
    for i, (comp, x, out) in enumerate(layers):
        want = oracle.matvec(comp.view(np.uint32), cb, x.view(np.float16), m, S, mode=mode)
        got = out.view(np.float16).astype(np.float64)
        touched = np.zeros(m, dtype=bool)
        for b in blocks:
            r0, r1 = b * rpb, min(m, (b + 1) * rpb)
            if r0 >= r1:
                continue
            touched[r0:r1] = True
            err = np.abs(got[r0:r1] - want[r0:r1]).max() / (np.abs(want).max() + 1e-9)
            assert err < 2e-3, f"layer {i} ({m}x{n}), workgroup {b}: rows {r0}..{r1 - 1} differ by {err:.3g} of the layer's largest output"
        assert (out.view(np.uint16)[~touched] == 0xEEEE).all(), f"layer {i}: a row outside the simulated workgroups was written"


@pytest.mark.parametrize("m,n,count,S,mode", [(33, 4096 + 768, 3, 8, 0), (33, 4096 + 768, 2, 8, 1), (300, 64, 4, 6, 0),
                                              (7, 704, 1, 6, 1), (512, 6144, 2, 8, 1), (1024, 2048 + 64, 5, 8, 0)])
def test_steady_kernel_matches_the_oracle(steady_isa, oracle, m, n, count, S, mode):
    run_steady(steady_isa, oracle, m, n, count, S, mode, blocks=sorted({0, 1, (m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS)))}))


def steady_fits(m, n):
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    lt = (n & 2047) >> 6
    rw_tail = 64 // lt if lt else 1
    total = (n >> 11) * (rpb // 2) + ((rpb + rw_tail - 1) // rw_tail if lt else 0)
    return (-(-total // 16) <= 4 and rpb * (n // 64) * 4 <= 16384 and ((n >> 11) + (1 if lt else 0)) * 4096 <= 32768 and n <= 16384)


@pytest.mark.parametrize("seed", range(6))
def test_steady_kernel_on_random_shapes(steady_isa, oracle, seed):
    """Chains of one random shape (any row count up to 3000, any multiple of 64 columns up to 12800 that the kernel's
    fixed LDS layout holds): the first workgroup, one in the middle and the one that holds the end of the rows, where a
    row block is partial and elements are empty; S and carry mode by seed."""
    rng = np.random.default_rng(700 + seed)
    while True:
        m, n = int(rng.integers(1, 3001)), 64 * int(rng.integers(1, 201))
        if steady_fits(m, n):
            break
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    last = (m - 1) // rpb
    run_steady(steady_isa, oracle, m, n, int(rng.integers(1, 5)), (6, 8)[seed & 1], (seed >> 1) & 1, blocks=sorted({0, last // 2, last}), seed=seed)


def test_steady_kernel_with_four_elements_a_wave_and_at_its_limits(steady_isa, oracle):
    """8192 x 8192: 64 elements a workgroup and layer, four a wave, the set of partial sums full (32 rows x 128);
    16384 columns: the activation image full; a single row; 64 columns."""
    run_steady(steady_isa, oracle, 8192, 8192, 2, 8, 1, blocks=[0, 255])
    run_steady(steady_isa, oracle, 5, 16384, 2, 8, 0, blocks=[0, 1, 2])
    run_steady(steady_isa, oracle, 1, 64, 3, 6, 1, blocks=[0])
    run_steady(steady_isa, oracle, 4096, 11008, 2, 8, 0, blocks=[0, 255])


@pytest.mark.parametrize("burst,latency", [(10 ** 6, (400, 60)), (8, (3000, 300)), (8, (40, 10))])
def test_steady_kernel_under_other_interleavings_and_latencies(steady_isa, oracle, burst, latency):
    """Every wave running until it blocks; memory that answers very late; memory that answers at once."""
    run_steady(steady_isa, oracle, 33, 4096 + 768, 3, 8, 1, blocks=[0, 16], seed=11, burst=burst, latency=latency)


@pytest.fixture(scope="module")
def steady_tuned_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_steady", extra=("-DST_TUNED",))


@pytest.mark.parametrize("m,n,count,S,mode", [(33, 4096 + 768, 3, 8, 0), (33, 4096 + 768, 2, 8, 1), (300, 64, 4, 6, 0), (7, 704, 1, 6, 1),
                                              (1024, 2048 + 64, 5, 8, 0), (8192, 8192, 2, 8, 0), (64, 16384, 2, 8, 1)])
def test_steady_kernel_with_the_untimed_changes(steady_tuned_isa, oracle, m, n, count, S, mode):
    """The -DST_TUNED build: the activation reload without a wait of its own, the rows added by the waves with the fewest
    elements, the next activations staged behind the first element, and a last layer that asks for nothing."""
    run_steady(steady_tuned_isa, oracle, m, n, count, S, mode, blocks=sorted({0, 1, (m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS)))}))


@pytest.mark.parametrize("burst,latency", [(1, (3000, 300)), (64, (5, 2)), (3, (40, 400))])
def test_steady_kernel_with_the_untimed_changes_under_other_interleavings(steady_tuned_isa, oracle, burst, latency):
    run_steady(steady_tuned_isa, oracle, 100, 4096 + 64 * 7, 3, 8, 1, blocks=[0, 1], burst=burst, latency=latency)


@pytest.fixture(scope="module")
def steady_mfma_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_steady", extra=("-DST_MFMA",))


@pytest.mark.parametrize("m,n,count,S,mode", [(33, 4096 + 768, 3, 8, 0), (300, 64, 2, 6, 1), (1024, 2048 + 64, 3, 8, 1), (8192, 8192, 2, 8, 0)])
def test_steady_kernel_with_the_products_on_the_matrix_unit(steady_mfma_isa, oracle, m, n, count, S, mode):
    """The -DST_MFMA build of the same kernel (v_mfma_f32_4x4x4_16b_f16 in place of the two-term dot products)."""
    run_steady(steady_mfma_isa, oracle, m, n, count, S, mode, blocks=sorted({0, (m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS)))}))


@pytest.fixture(scope="module")
def steady_roll_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_steady", extra=("-DST_ROLL",))


@pytest.mark.parametrize("m,n,count,S,mode", [(33, 4096 + 768, 3, 8, 0), (300, 64, 2, 6, 1), (1024, 2048 + 64, 3, 8, 1)])
def test_steady_kernel_with_the_decode_as_a_rolling_pipeline(steady_roll_isa, oracle, m, n, count, S, mode):
    """The -DST_ROLL build of the same kernel (sixteen gathers kept in flight, two products and two new gathers a step)."""
    run_steady(steady_roll_isa, oracle, m, n, count, S, mode, blocks=sorted({0, (m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS)))}))


@pytest.fixture(scope="module")
def viterbi_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "viterbi")


@pytest.mark.parametrize("S,steps,weighted", [(9, 3, False), (7, 2, True)])
def test_lite_search_kernel_matches_the_oracle(viterbi_isa, oracle, S, steps, weighted):
    """`viterbi_lite_kernel` and `viterbi_trace_kernel<4>` as `rptc_lite_viterbi` launches them (`csrc/viterbi.hip`): a few
    steps of the search over the 65536 states of rptc_lite.py's trellis at L = 16, R = 4, V = 2 against the oracle's
    `lite_quantize`: the same symbols, end state and cost to the bit (every sum is fp32 in the same order)."""
    rng = np.random.default_rng(S + steps)
    alphabet = rng.standard_normal((1 << S, 2)).astype(np.float32)
    samples = rng.standard_normal((steps, 2)).astype(np.float32)
    importance = (rng.random((steps, 2)) + 0.25).astype(np.float32) if weighted else None
    back = np.full(steps * 1024, 0xABCD, dtype=np.uint16)
    symbols = np.full(steps, 0xEE, dtype=np.uint8)
    end_state = np.full(1, -1, dtype=np.int32)
    cost = np.full(1, np.nan, dtype=np.float32)
    mem = wave_model.Memory()
    t_at, w_at, a_at, b_at, s_at, e_at, c_at = (0x7f4000000000, 0x7f4100000000, 0x7f4200000000, 0x7f4300000000, 0x7f4400000000,
                                                0x7f4500000000, 0x7f4600000000)
    mem.add(t_at, samples.view(np.uint8).reshape(-1).copy(), "samples")
    if weighted:
        mem.add(w_at, importance.view(np.uint8).reshape(-1).copy(), "importance")
    mem.add(a_at, alphabet.view(np.uint8).reshape(-1).copy(), "alphabet")
    mem.add(b_at, back.view(np.uint8), "back pointers")
    mem.add(s_at, symbols, "symbols")
    mem.add(e_at, end_state.view(np.uint8), "end state")
    mem.add(c_at, cost.view(np.uint8), "cost")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    search = wave_model.Kernel(viterbi_isa, "_ZN4rptc19viterbi_lite_kernelILb%dEE" % (1 if weighted else 0))
    search.launch(mem, (1,), 1024, [("ptr", t_at), ("ptr", w_at if weighted else 0), ("i64", 0), ("ptr", a_at), ("i32", S), ("ptr", b_at),
                                    ("ptr", e_at), ("ptr", c_at), ("i32", steps)], lds_bytes=(256 * 64 + 2 * 4096) * 4 + 2 * 1024 * 4, seed=S)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    trace = wave_model.Kernel(viterbi_isa, "_ZN4rptc20viterbi_trace_kernelILi4EE")
    trace.launch(mem, (1,), 64, [("ptr", b_at), ("ptr", e_at), ("ptr", s_at), ("i32", 1), ("i32", steps)], seed=S)
    want_symbols, want_cost = oracle.lite_quantize(alphabet, 16, S, 4, importance, samples)
    assert np.array_equal(symbols.astype(np.int32), want_symbols)
    assert cost.view(np.uint32)[0] == np.float32(want_cost).view(np.uint32)
    state = 0
    for v in want_symbols:
        state = ((state << 4) | int(v)) & 0xFFFF
    assert int(end_state[0]) == state


@pytest.mark.parametrize("L,S,R,V,rows,steps,weighted", [(8, 5, 2, 2, 2, 9, False), (6, 6, 1, 3, 1, 14, True), (12, 9, 4, 2, 1, 4, True),
                                                         (10, 4, 8, 1, 1, 3, False), (3, 2, 3, 4, 3, 5, True), (13, 7, 2, 2, 1, 2, False)])
def test_general_lite_search_kernel_matches_the_oracle(viterbi_isa, oracle, L, S, R, V, rows, steps, weighted):
    """`viterbi_lite_general_kernel` and its trace kernel as `rptc_lite_viterbi` launches them for parameters other than the
    reference driver's: path costs, group minima and back pointers in a scratch buffer of exactly the size
    `rptc_lite_viterbi_scratch_bytes` states (anything beyond it fails the model's bounds check); symbols and cost equal
    the oracle's `lite_quantize` to the bit, every row's importance set is its own.  The waves of the workgroup hand the
    path costs to each other through global memory across `__syncthreads()` (see `barrier_orders_memory`)."""
    rng = np.random.default_rng(100 * L + 10 * R + V)
    alphabet = rng.standard_normal((1 << S, V)).astype(np.float32)
    samples = rng.standard_normal((rows, steps, V)).astype(np.float32)
    importance = (rng.random((rows, steps, V)) + 0.25).astype(np.float32) if weighted else None
    states, groups = 1 << L, 1 << (L - R)
    back_offset = (rows * (states + groups) * 4 + 255) // 256 * 256
    scratch = np.full(back_offset + rows * steps * groups, 0xAB, dtype=np.uint8)
    symbols = np.full(rows * steps, 0xEE, dtype=np.uint8)
    end_state = np.full(rows, -1, dtype=np.int32)
    cost = np.full(rows, np.nan, dtype=np.float32)
    mem = wave_model.Memory()
    t_at, w_at, a_at, b_at, s_at, e_at, c_at = (0x7f4000000000, 0x7f4100000000, 0x7f4200000000, 0x7f4300000000, 0x7f4400000000,
                                                0x7f4500000000, 0x7f4600000000)
    mem.add(t_at, samples.view(np.uint8).reshape(-1).copy(), "samples")
    if weighted:
        mem.add(w_at, importance.view(np.uint8).reshape(-1).copy(), "importance")
    mem.add(a_at, alphabet.view(np.uint8).reshape(-1).copy(), "alphabet")
    mem.add(b_at, scratch, "scratch")
    mem.add(s_at, symbols, "symbols")
    mem.add(e_at, end_state.view(np.uint8), "end state")
    mem.add(c_at, cost.view(np.uint8), "cost")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    search = wave_model.Kernel(viterbi_isa, "_ZN4rptc27viterbi_lite_general_kernelILb%dEE" % (1 if weighted else 0))
    search.launch(mem, (rows,), 1024, [("ptr", t_at), ("ptr", w_at if weighted else 0), ("i64", V * steps if weighted else 0), ("ptr", a_at),
                                       ("i32", L), ("i32", S), ("i32", R), ("i32", V), ("ptr", b_at), ("ptr", b_at + back_offset),
                                       ("ptr", e_at), ("ptr", c_at), ("i32", steps)], lds_bytes=0, seed=L, barrier_orders_memory=True)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    trace = wave_model.Kernel(viterbi_isa, "_ZN4rptc33viterbi_lite_general_trace_kernelE")
    trace.launch(mem, (1,), 64, [("ptr", b_at + back_offset), ("ptr", e_at), ("ptr", s_at), ("i32", L), ("i32", R), ("i32", rows), ("i32", steps)],
                 seed=L)
    for r in range(rows):
        want_symbols, want_cost = oracle.lite_quantize(alphabet, L, S, R, importance[r] if weighted else None, samples[r])
        assert np.array_equal(symbols[r * steps:(r + 1) * steps].astype(np.int32), want_symbols), r
        assert cost.view(np.uint32)[r] == np.float32(want_cost).view(np.uint32), r
        state = 0
        for v in want_symbols:
            state = ((state << R) | int(v)) & (states - 1)
        assert int(end_state[r]) == state


@pytest.fixture(scope="module")
def steady_mfma_roll_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "matvec_steady", extra=("-DST_MFMA", "-DST_ROLL"))


@pytest.mark.parametrize("m,n,count,S,mode", [(33, 4096 + 768, 3, 8, 0), (300, 64, 2, 6, 1), (1024, 2048 + 64, 3, 8, 1)])
def test_steady_kernel_with_both_the_matrix_unit_and_the_rolling_pipeline(steady_mfma_roll_isa, oracle, m, n, count, S, mode):
    run_steady(steady_mfma_roll_isa, oracle, m, n, count, S, mode, blocks=sorted({0, (m - 1) // (2 * ((m + 2 * CUS - 1) // (2 * CUS)))}))


@pytest.mark.parametrize("S,bits,steps,weighted", [(8, 2, 3, False), (6, 2, 2, True), (8, 3, 2, False), (6, 3, 2, True)])
def test_pair_search_kernel_matches_the_oracle(viterbi_isa, oracle, S, bits, steps, weighted):
    """`viterbi_pairs_kernel<S, 2 bits, WEIGHTED>` and `viterbi_trace_kernel` (`csrc/viterbi.hip`) for a few steps of one
    row against `orc_viterbi` over the table of pairs the states decode to: symbols, end state and cost to the bit.  (The
    8-bits-a-step kernels keep a few registers in scratch memory, which the model does not have: they are GPU tests only.)"""
    import torch
    from rptc_kernels import quantize
    rng = np.random.default_rng(10 * S + bits)
    cb = rng.standard_normal(2 << S).astype(np.float16)
    targets = (0.7 * rng.standard_normal((steps, 2))).astype(np.float32)
    weights = rng.uniform(0.25, 4.0, (steps, 2)).astype(np.float32) if weighted else None
    table = quantize.decode_table(torch.from_numpy(cb), S).numpy()          # the same states at every width; a step shifts 2 * bits in
    back = np.full(steps * 1024, 0xABCD, dtype=np.uint16)
    symbols = np.full(steps, 0xEE, dtype=np.uint8)
    end_state = np.full(1, -1, dtype=np.int32)
    cost = np.full(1, np.nan, dtype=np.float32)
    mem = wave_model.Memory()
    t_at, w_at, a_at, b_at, s_at, e_at, c_at = (0x7f4000000000, 0x7f4100000000, 0x7f4200000000, 0x7f4300000000, 0x7f4400000000,
                                                0x7f4500000000, 0x7f4600000000)
    mem.add(t_at, targets.view(np.uint8).reshape(-1).copy(), "targets")
    if weighted:
        mem.add(w_at, weights.view(np.uint8).reshape(-1).copy(), "weights")
    mem.add(a_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(b_at, back.view(np.uint8), "back pointers")
    mem.add(s_at, symbols, "symbols")
    mem.add(e_at, end_state.view(np.uint8), "end state")
    mem.add(c_at, cost.view(np.uint8), "cost")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    search = wave_model.Kernel(viterbi_isa, "_ZN4rptc20viterbi_pairs_kernelILi%dELi%dELb%dEE" % (S, 2 * bits, 1 if weighted else 0))
    search.launch(mem, (1,), 1024, [("ptr", t_at), ("ptr", w_at if weighted else 0), ("i64", 0), ("ptr", a_at), ("ptr", b_at), ("ptr", e_at),
                                    ("ptr", c_at), ("i32", steps)], lds_bytes=(256 * 64 + 2 * 4096) * 4 + 2 * 1024 * 4, seed=S)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    trace = wave_model.Kernel(viterbi_isa, "_ZN4rptc20viterbi_trace_kernelILi%dEE" % (2 * bits))
    trace.launch(mem, (1,), 64, [("ptr", b_at), ("ptr", e_at), ("ptr", s_at), ("i32", 1), ("i32", steps)], seed=S)
    want_symbols, want_cost, want_end = oracle.viterbi(table, 2 * bits, targets, weights)
    assert np.array_equal(symbols.astype(np.int32), want_symbols)
    assert cost.view(np.uint32)[0] == np.float32(want_cost).view(np.uint32) and int(end_state[0]) == want_end


@pytest.fixture(scope="module")
def glue_isa(tmp_path_factory):
    return compile_to_assembly(tmp_path_factory, "decode_glue")


def _matvec_geometry(m, n):
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    lt = (n & 2047) >> 6
    rw_tail = 64 // lt if lt else 1
    items_full = rpb // 2
    items_tail = (rpb + rw_tail - 1) // rw_tail if lt else 0
    magic = ((1 << 32) // items_full + 1) if items_full > 1 else 0
    return rpb, rw_tail, items_tail, magic, 65536 + 2 * n + 4 * (n // 64) * rpb


@pytest.mark.parametrize("prologue,m,n,mode", [("silu", 40, 2048 + 320, 0), ("rmsnorm", 40, 2048 + 64, 1), ("rmsnorm", 33, 64 * 7, 0),
                                               ("rmsnorm", 40, 6144, 1), ("rmsnorm", 2, 11008, 1), ("silu", 2, 8192, 1)])
def test_fused_prologue_kernels_equal_the_separate_kernels(matvec_isa, glue_isa, prologue, m, n, mode):
    """`matvec_fused_kernel` with the SiLU gate or the residual add + RMS norm in its prologue (`csrc/matvec.hip`) against
    the stand-alone element-wise kernel (`csrc/decode_glue.hip`) followed by the plain mat-vec kernel, all three run in the
    model, and no access outside the buffers.  SiLU: the same output bits (the prologue repeats the stand-alone kernel's
    roundings).  Norm: the residual stream written back has the same bits; the sum of squares is added in another order
    (eight neighbours a thread and two-term dot products against one element a thread and step), so the scale can differ
    in its last fp32 bit, a few activations in their last fp16 bit and a few outputs with them (rarely: 511 x 6144 with these
    inputs is such a case, the ones here are not): outputs within fp16 rounding of each other."""
    S = 8
    rng = np.random.default_rng(m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    rpb, rw_tail, items_tail, magic, lds_plain = _matvec_geometry(m, n)
    grid = (m + rpb - 1) // rpb
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    c_at, cb_at, x_at, x2_at, w_at, xo_at, h_at, o_at, o2_at = (0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f3000000000, 0x7f3100000000,
                                                               0x7f3200000000, 0x7f3300000000, 0x7f2ffffe0100, 0x7f2e00000000)
    out_fused = np.full(2 * m, 0xEE, dtype=np.uint8)
    out_plain = np.full(2 * m, 0xEE, dtype=np.uint8)
    mem = wave_model.Memory()
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(o_at, out_fused, "output of the fused kernel")
    mem.add(o2_at, out_plain, "output of the plain kernel")
    common = [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail), ("i32", items_tail), ("u32", magic)]

    def forget_kernargs():
        mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    if prologue == "silu":
        gu = (rng.standard_normal(2 * n) * 1.5).astype(np.float16)
        h = np.full(2 * n, 0xEE, dtype=np.uint8)
        mem.add(x_at, gu.view(np.uint8).copy(), "gate and up")
        mem.add(h_at, h, "gated activations")
        wave_model.Kernel(glue_isa, "_ZN4rptc15silu_mul_kernelE").launch(mem, ((n + 255) // 256,), 256, [("ptr", x_at), ("ptr", h_at), ("i32", n)], seed=1)
        forget_kernargs()
        fused = wave_model.Kernel(matvec_isa, "_ZN4rptc19matvec_fused_kernelILi%dELi%dELi1ELb0EE" % (S, mode))
        fused.launch(mem, (grid,), 1024, common + [("ptr", 0), ("ptr", o_at), ("ptr", 0), ("ptr", 0), ("f32", 0.0), ("i32", 0)],
                     lds_bytes=lds_plain, seed=m)
    else:
        x_in = (rng.standard_normal(n) * 1.2).astype(np.float16)
        delta = (rng.standard_normal(n) * 0.3).astype(np.float16)
        weight = (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float16)
        res_a = np.full(2 * n, 0xEE, dtype=np.uint8)
        res_b = np.full(2 * n, 0xEE, dtype=np.uint8)
        h = np.full(2 * n, 0xEE, dtype=np.uint8)
        mem.add(x_at, x_in.view(np.uint8).copy(), "residual stream in")
        mem.add(x2_at, delta.view(np.uint8).copy(), "delta")
        mem.add(w_at, weight.view(np.uint8).copy(), "norm weight")
        mem.add(xo_at, res_a, "residual stream out (stand-alone)")
        mem.add(0x7f3400000000, res_b, "residual stream out (fused)")
        mem.add(h_at, h, "normed activations")
        eps = 1e-5
        wave_model.Kernel(glue_isa, "_ZN4rptc18add_rmsnorm_kernelE").launch(
            mem, (1,), 1024, [("ptr", x_at), ("ptr", x2_at), ("ptr", w_at), ("ptr", xo_at), ("ptr", h_at), ("i32", n), ("f32", eps)], seed=1)
        forget_kernargs()
        fused = wave_model.Kernel(matvec_isa, "_ZN4rptc19matvec_fused_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
        fused.launch(mem, (grid,), 1024, common + [("ptr", x2_at), ("ptr", o_at), ("ptr", w_at), ("ptr", 0x7f3400000000), ("f32", eps), ("i32", 0)],
                     lds_bytes=lds_plain + 48 * 4, seed=m)
        assert np.array_equal(res_a, res_b), "the residual stream written back differs"
    forget_kernargs()
    plain = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
    plain.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", h_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                      ("i32", items_tail), ("u32", magic), ("ptr", o2_at)], lds_bytes=lds_plain, seed=m)
    got, want = out_fused.view(np.float16).astype(np.float64), out_plain.view(np.float16).astype(np.float64)
    assert np.isfinite(got).all()
    if prologue == "silu":
        assert np.array_equal(out_fused, out_plain)
    else:
        assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max()


def _rope_reference(x, cos_row, sin_row):
    """The rotation of decode_glue.hip's rope_pair: products and sums in fp16, each rounded once."""
    a, b = x[0::2].astype(np.float16), x[1::2].astype(np.float16)
    c, s = cos_row.astype(np.float16), sin_row.astype(np.float16)
    out = np.empty_like(x)
    out[0::2] = (a * c).astype(np.float16) - (b * s).astype(np.float16)
    out[1::2] = (a * s).astype(np.float16) + (b * c).astype(np.float16)
    return out


@pytest.mark.parametrize("rope,heads,hd,max_len,pos,splits", [(False, 3, 64, 96, 50, 3), (True, 2, 128, 64, 37, 4), (False, 2, 32, 48, 0, 2),
                                                               (True, 1, 64, 32, 31, 2)])
def test_attention_kernel_matches_a_softmax_in_double(glue_isa, rope, heads, hd, max_len, pos, splits):
    """`attn_decode_kernel<ROPE>` (`csrc/decode_glue.hip`) as `rptc_attn_decode` / `rptc_rope_attn_decode` launch it: a head's
    keys cut into pieces, one workgroup each, the last to arrive merging them (the model runs the workgroups one after the
    other); with ROPE the rotation of q and k and the append to the caches happen inside.  Against softmax attention in
    double over positions 0..pos; the caches outside row pos untouched; the arrival counters left at zero."""
    rng = np.random.default_rng(heads * 1000 + pos)
    d = heads * hd
    k_cache = (rng.standard_normal((heads, max_len, hd)) * 0.5).astype(np.float16)
    v_cache = (rng.standard_normal((heads, max_len, hd)) * 0.5).astype(np.float16)
    cos_t = np.cos(rng.random((max_len, hd // 2)) * 6.28).astype(np.float16)
    sin_t = np.sin(rng.random((max_len, hd // 2)) * 6.28).astype(np.float16)
    qkv = (rng.standard_normal(3 * d) * 0.7).astype(np.float16)
    k_before, v_before = k_cache.copy(), v_cache.copy()
    if rope:
        q_eff = np.concatenate([_rope_reference(qkv[h * hd:(h + 1) * hd], cos_t[pos], sin_t[pos]) for h in range(heads)])
        for h in range(heads):
            k_before[h, pos] = _rope_reference(qkv[d + h * hd:d + (h + 1) * hd], cos_t[pos], sin_t[pos])
            v_before[h, pos] = qkv[2 * d + h * hd:2 * d + (h + 1) * hd]
        q_in = qkv
    else:
        q_eff = qkv[:d]
        q_in = qkv[:d].copy()
    out = np.full(d, np.nan, dtype=np.float16)
    parts = np.full(heads * splits * 258, np.nan, dtype=np.float32)
    arrived = np.zeros(heads, dtype=np.uint32)
    position = np.array([pos], dtype=np.int64)
    mem = wave_model.Memory()
    at = {name: 0x7f4000000000 + i * 0x100000000 for i, name in enumerate(("pos", "q", "k", "v", "cos", "sin", "out", "parts", "arrived"))}
    mem.add(at["pos"], position.view(np.uint8), "position")
    mem.add(at["q"], q_in.view(np.uint8).copy(), "query")
    mem.add(at["k"], k_cache.view(np.uint8).reshape(-1), "key cache")
    mem.add(at["v"], v_cache.view(np.uint8).reshape(-1), "value cache")
    mem.add(at["cos"], cos_t.view(np.uint8).reshape(-1).copy(), "cosines")
    mem.add(at["sin"], sin_t.view(np.uint8).reshape(-1).copy(), "sines")
    mem.add(at["out"], out.view(np.uint8), "output")
    mem.add(at["parts"], parts.view(np.uint8), "pieces")
    mem.add(at["arrived"], arrived.view(np.uint8), "arrival counters")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(glue_isa, "_ZN4rptc18attn_decode_kernelILb%dEE" % (1 if rope else 0))
    kernel.launch(mem, (heads * splits,), 256,
                  [("ptr", at["pos"]), ("ptr", at["q"]), ("ptr", at["k"]), ("ptr", at["v"]), ("i32", heads), ("i32", hd), ("i32", max_len),
                   ("i32", splits), ("ptr", at["cos"]), ("ptr", at["sin"]), ("ptr", at["out"]), ("ptr", at["parts"]), ("ptr", at["arrived"])],
                  lds_bytes=(16 + 2048) * 4 + hd * 6, seed=pos + 1)
    assert np.array_equal(k_cache.view(np.uint16), k_before.view(np.uint16)) and np.array_equal(v_cache.view(np.uint16), v_before.view(np.uint16))
    assert not arrived.any()
    for h in range(heads):
        q = q_eff[h * hd:(h + 1) * hd].astype(np.float64)
        keys, values = k_before[h, :pos + 1].astype(np.float64), v_before[h, :pos + 1].astype(np.float64)
        scores = keys @ q / np.sqrt(hd)
        w = np.exp(scores - scores.max())
        want = (w / w.sum()) @ values
        got = out[h * hd:(h + 1) * hd].astype(np.float64)
        assert np.abs(got - want).max() < 4e-3 * max(1.0, np.abs(want).max()), h


@pytest.mark.parametrize("vocab,d,ties", [(32000, 128, False), (1003, 64, True), (7, 8, False)])
def test_greedy_hand_over_kernel(glue_isa, vocab, d, ties):
    """`greedy_next_kernel` (`csrc/decode_glue.hip`): the first maximum of the logits (a vocabulary that is no multiple of
    eight included, and equal maxima), appended to the output list, its embedding row copied, index and position moved on."""
    rng = np.random.default_rng(vocab)
    logits = rng.standard_normal(vocab).astype(np.float16)
    if ties:
        top = np.float16(logits.astype(np.float32).max() + 1)
        logits[[900, 333, 1002]] = top
    embed = rng.standard_normal((vocab, d)).astype(np.float16)
    token = np.array([-1], dtype=np.int64)
    out_list = np.full(8, -1, dtype=np.int64)
    out_index = np.array([3], dtype=np.int64)
    pos = np.array([41], dtype=np.int64)
    x = np.full(d, np.nan, dtype=np.float16)
    mem = wave_model.Memory()
    at = {name: 0x7f4000000000 + i * 0x100000000 for i, name in enumerate(("logits", "embed", "token", "list", "index", "pos", "x"))}
    mem.add(at["logits"], logits.view(np.uint8).copy(), "logits")
    mem.add(at["embed"], embed.view(np.uint8).reshape(-1).copy(), "embedding")
    mem.add(at["token"], token.view(np.uint8), "token")
    mem.add(at["list"], out_list.view(np.uint8), "output list")
    mem.add(at["index"], out_index.view(np.uint8), "output index")
    mem.add(at["pos"], pos.view(np.uint8), "position")
    mem.add(at["x"], x.view(np.uint8), "next input")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(glue_isa, "_ZN4rptc18greedy_next_kernelE")
    kernel.launch(mem, (1,), 1024, [("ptr", at["logits"]), ("i32", vocab), ("ptr", at["embed"]), ("i32", d), ("ptr", at["token"]), ("ptr", at["list"]),
                                    ("ptr", at["index"]), ("ptr", at["pos"]), ("ptr", at["x"])], seed=vocab)
    want = int(np.argmax(logits.astype(np.float32)))
    assert int(token[0]) == want and int(out_list[3]) == want and int(out_index[0]) == 4 and int(pos[0]) == 42
    assert (out_list[[0, 1, 2, 4, 5, 6, 7]] == -1).all()
    assert np.array_equal(x.view(np.uint16), embed[want].view(np.uint16))


@pytest.mark.parametrize("heads,hd,max_len,pos", [(3, 64, 20, 7), (2, 128, 5, 4), (2, 32, 9, 9)])
def test_rope_and_cache_kernel(glue_isa, heads, hd, max_len, pos):
    """`rope_cache_kernel` (`csrc/decode_glue.hip`): q rotated, k rotated into its cache row, v copied into its, bit for bit
    against the same fp16 arithmetic; a position outside the caches writes nothing."""
    rng = np.random.default_rng(heads + pos)
    d = heads * hd
    qkv = (rng.standard_normal(3 * d) * 0.7).astype(np.float16)
    cos_t = np.cos(rng.random((max_len, hd // 2)) * 6.28).astype(np.float16)
    sin_t = np.sin(rng.random((max_len, hd // 2)) * 6.28).astype(np.float16)
    k_cache = rng.standard_normal((heads, max_len, hd)).astype(np.float16)
    v_cache = rng.standard_normal((heads, max_len, hd)).astype(np.float16)
    k_want, v_want = k_cache.copy(), v_cache.copy()
    q_out = np.full(d, np.nan, dtype=np.float16)
    q_want = q_out.copy()
    if pos < max_len:
        q_want = np.concatenate([_rope_reference(qkv[h * hd:(h + 1) * hd], cos_t[pos], sin_t[pos]) for h in range(heads)])
        for h in range(heads):
            k_want[h, pos] = _rope_reference(qkv[d + h * hd:d + (h + 1) * hd], cos_t[pos], sin_t[pos])
            v_want[h, pos] = qkv[2 * d + h * hd:2 * d + (h + 1) * hd]
    position = np.array([pos], dtype=np.int64)
    mem = wave_model.Memory()
    at = {name: 0x7f4000000000 + i * 0x100000000 for i, name in enumerate(("qkv", "cos", "sin", "pos", "q", "k", "v"))}
    mem.add(at["qkv"], qkv.view(np.uint8).copy(), "projection output")
    mem.add(at["cos"], cos_t.view(np.uint8).reshape(-1).copy(), "cosines")
    mem.add(at["sin"], sin_t.view(np.uint8).reshape(-1).copy(), "sines")
    mem.add(at["pos"], position.view(np.uint8), "position")
    mem.add(at["q"], q_out.view(np.uint8), "rotated query")
    mem.add(at["k"], k_cache.view(np.uint8).reshape(-1), "key cache")
    mem.add(at["v"], v_cache.view(np.uint8).reshape(-1), "value cache")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(glue_isa, "_ZN4rptc17rope_cache_kernelE")
    kernel.launch(mem, ((heads * hd // 2 + 255) // 256,), 256,
                  [("ptr", at["qkv"]), ("ptr", at["cos"]), ("ptr", at["sin"]), ("ptr", at["pos"]), ("ptr", at["q"]), ("ptr", at["k"]), ("ptr", at["v"]),
                   ("i32", heads), ("i32", hd), ("i32", max_len)], seed=pos)
    assert np.array_equal(q_out.view(np.uint16), q_want.view(np.uint16))
    assert np.array_equal(k_cache.view(np.uint16), k_want.view(np.uint16)) and np.array_equal(v_cache.view(np.uint16), v_want.view(np.uint16))


@pytest.mark.parametrize("m,n,mode,which", [(40, 2048 + 320, 0, "all"), (33, 64 * 7, 1, "none"), (20, 1024, 1, "out")])
def test_affine_kernel_applies_the_factorisation(matvec_isa, oracle, m, n, mode, which):
    """`matvec_affine_kernel<S, MODE, plain>` (`csrc/matvec.hip`): y = s_out * (W (s_in * a)) + b_out * sum(a) + b_in . a with
    the factorisation's four vectors (quantize_hf.py:167), any of them absent; against the same in double on the decoded
    matrix; with none of them the output bits are the plain kernel's."""
    S = 8
    rng = np.random.default_rng(m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    si = (rng.random(n) + 0.5).astype(np.float16) if which == "all" else None
    bi = (rng.standard_normal(n) * 0.02).astype(np.float16) if which == "all" else None
    so = (rng.random(m) + 0.5).astype(np.float16) if which in ("all", "out") else None
    bo = (rng.standard_normal(m) * 0.02).astype(np.float16) if which in ("all", "out") else None
    rpb, rw_tail, items_tail, magic, lds_plain = _matvec_geometry(m, n)
    grid = (m + rpb - 1) // rpb
    out = np.full(2 * m, 0xEE, dtype=np.uint8)
    mem = wave_model.Memory()
    at = {name: 0x7f4000000000 + i * 0x100000000 + 0x100 for i, name in enumerate(("comp", "cb", "x", "si", "bi", "so", "bo", "out", "plain"))}
    mem.add(at["comp"], comp, "stream")
    mem.add(at["cb"], cb.view(np.uint8).copy(), "codebook")
    mem.add(at["x"], x.view(np.uint8).copy(), "activations")
    for name, vec in (("si", si), ("bi", bi), ("so", so), ("bo", bo)):
        if vec is not None:
            mem.add(at[name], vec.view(np.uint8).copy(), name)
    mem.add(at["out"], out, "output")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    ptr = lambda name, vec: ("ptr", at[name] if vec is not None else 0)
    kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc20matvec_affine_kernelILi%dELi%dELi0EE" % (S, mode))
    kernel.launch(mem, (grid,), 1024,
                  [("ptr", at["comp"]), ("ptr", at["cb"]), ("ptr", at["x"]), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail), ("i32", items_tail),
                   ("u32", magic), ("ptr", 0), ("ptr", at["out"]), ("ptr", 0), ("ptr", 0), ("f32", 0.0), ptr("si", si), ptr("bi", bi), ptr("so", so),
                   ptr("bo", bo)], lds_bytes=lds_plain + 48 * 4, seed=m)
    W = oracle.matvec_dense(comp.view(np.uint32), cb, m, n, S, mode=mode).astype(np.float64)
    a64 = x.astype(np.float64)
    xs = (x * si).astype(np.float16).astype(np.float64) if si is not None else a64
    want = W @ xs
    if so is not None:
        want = want * so.astype(np.float64)
    if bo is not None:
        want = want + bo.astype(np.float64) * a64.sum()
    if bi is not None:
        want = want + (bi.astype(np.float64) * a64).sum()
    got = out.view(np.float16).astype(np.float64)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3
    if which == "none":
        plain_out = np.full(2 * m, 0xEE, dtype=np.uint8)
        mem.add(at["plain"], plain_out, "output of the plain kernel")
        mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
        plain = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
        plain.launch(mem, (grid,), 1024, [("ptr", at["comp"]), ("ptr", at["cb"]), ("ptr", at["x"]), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                          ("i32", items_tail), ("u32", magic), ("ptr", at["plain"])], lds_bytes=lds_plain, seed=m)
        assert np.array_equal(out, plain_out)


@pytest.mark.parametrize("bits,m,n,S,mode", [(3, 40, 2048 + 320, 8, 0), (4, 33, 4096, 6, 1), (3, 20, 64 * 5, 6, 1), (4, 70, 2048 + 64, 8, 0)])
def test_per_launch_kernel_at_3_and_4_bits(matvec_isa, oracle, bits, m, n, S, mode):
    """`matvec_kernel<S, MODE, BITS, false>` for the 3- and 4-bit streams (`rptc_decompress_matvec_bits`) against the dense
    matrix the oracle decodes from the same stream (`orc_bits_dense`) times the activations in double."""
    rng = np.random.default_rng(bits * 100 + m)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n * bits // 8, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    out = np.full(2 * m, 0xEE, dtype=np.uint8)
    rpb, rw_tail, items_tail, magic, lds_bytes = _matvec_geometry(m, n)
    grid = (m + rpb - 1) // rpb
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x.view(np.uint8).copy(), "activations")
    mem.add(o_at, out, "output")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi%dELb0EE" % (S, mode, bits))
    kernel.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                       ("i32", items_tail), ("u32", magic), ("ptr", o_at)], lds_bytes=lds_bytes, seed=m)
    W = oracle.bits_dense(comp.view(np.uint32), cb, m, n, S, bits, mode=mode).astype(np.float64)
    want = W @ x.astype(np.float64)
    got = out.view(np.float16).astype(np.float64)
    assert np.abs(got - want).max() / (np.abs(want).max() + 1e-9) < 2e-3


@pytest.mark.parametrize("bits,m,n,S,mode", [(2, 10, 2048 + 320, 8, 0), (2, 7, 64 * 3, 6, 1), (3, 9, 2048 + 64, 8, 1), (4, 5, 4096, 6, 0)])
def test_dense_export_kernels_are_bit_exact(matvec_isa, oracle, bits, m, n, S, mode):
    """`matvec_dense_kernel` / `bits_dense_kernel` (`csrc/matvec.hip`), one launch a slab as the library launches them:
    the fp16 matrix a stream stands for, bit for bit against the oracle's."""
    rng = np.random.default_rng(bits * 10 + m)
    cb = rng.standard_normal(2 << S).astype(np.float16)
    comp = rng.integers(0, 256, m * n * bits // 8, dtype=np.uint8)
    W = np.full(m * n, 0xEEEE, dtype=np.uint16)
    mem = wave_model.Memory()
    c_at, cb_at, w_at = 0x7f40fffff000, 0x7f5000003400, 0x7f2ffffe0100
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(w_at, W.view(np.uint8), "dense matrix")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    name = "_ZN4rptc19matvec_dense_kernelILi%dELi%dEE" % (S, mode) if bits == 2 else "_ZN4rptc17bits_dense_kernelILi%dELi%dELi%dEE" % (S, mode, bits)
    kernel = wave_model.Kernel(matvec_isa, name)
    T, lt = n >> 11, (n & 2047) >> 6
    for slab in range(T + (1 if lt else 0)):
        elems = m * (32 if slab < T else lt)
        kernel.launch(mem, ((elems + 255) // 256,), 256, [("ptr", c_at), ("ptr", cb_at), ("ptr", w_at), ("i32", m), ("i32", n), ("i32", slab),
                                                         ("i32", elems)], seed=slab + 1)
        mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    want = (oracle.matvec_dense(comp.view(np.uint32), cb, m, n, S, mode=mode) if bits == 2 else
            oracle.bits_dense(comp.view(np.uint32), cb, m, n, S, bits, mode=mode))
    assert np.array_equal(W.reshape(m, n), want.view(np.uint16))


@pytest.mark.parametrize("m,n,block,mode", [(40, 2048 + 256, 256, 0), (33, 1024, 1024, 1), (20, 64 * 6, 128, 0)])
def test_hadamard_prologue_kernel_equals_the_two_kernels(matvec_isa, hadamard_isa, m, n, block, mode):
    """`matvec_fused_kernel` with the sign-Hadamard transform of the activations in its prologue
    (`rptc_decompress_matvec_hadamard`) against `sign_hadamard_kernel` followed by the plain mat-vec kernel, all in the
    model: the same output bits."""
    S = 8
    rng = np.random.default_rng(m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = rng.standard_normal(n).astype(np.float16)
    signs = np.where(rng.integers(0, 2, n) == 1, 1.0, -1.0).astype(np.float16)
    rpb, rw_tail, items_tail, magic, lds_plain = _matvec_geometry(m, n)
    grid = (m + rpb - 1) // rpb
    h = np.full(2 * n, 0xEE, dtype=np.uint8)
    out_fused = np.full(2 * m, 0xEE, dtype=np.uint8)
    out_plain = np.full(2 * m, 0xEE, dtype=np.uint8)
    mem = wave_model.Memory()
    c_at, cb_at, x_at, s_at, h_at, o_at, o2_at = (0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f3000000000, 0x7f3300000000, 0x7f2ffffe0100,
                                                  0x7f2e00000000)
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x.view(np.uint8).copy(), "activations")
    mem.add(s_at, signs.view(np.uint8).copy(), "signs")
    mem.add(h_at, h, "transformed activations")
    mem.add(o_at, out_fused, "output of the fused kernel")
    mem.add(o2_at, out_plain, "output of the plain kernel")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    log_p = block.bit_length() - 1
    wave_model.Kernel(hadamard_isa, "_ZN4rptc20sign_hadamard_kernelE").launch(
        mem, (n // block,), 256, [("ptr", x_at), ("ptr", s_at), ("ptr", h_at), ("i32", n), ("i32", block), ("i32", log_p), ("i32", n // block),
                                  ("i32", 0), ("i32", 1 if block % 8 == 0 else 0)], lds_bytes=(block + block // 32) * 4, seed=n)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    common = [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail), ("i32", items_tail), ("u32", magic)]
    fused = wave_model.Kernel(matvec_isa, "_ZN4rptc19matvec_fused_kernelILi%dELi%dELi3ELb0EE" % (S, mode))
    fused.launch(mem, (grid,), 1024, common + [("ptr", s_at), ("ptr", o_at), ("ptr", 0), ("ptr", 0), ("f32", 0.0), ("i32", log_p)],
                 lds_bytes=lds_plain + (n + n // 32 + 1) * 4, seed=m)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    plain = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
    plain.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", h_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                      ("i32", items_tail), ("u32", magic), ("ptr", o2_at)], lds_bytes=lds_plain, seed=m)
    assert np.array_equal(out_fused, out_plain)


def test_per_launch_kernel_with_compact_sums_on_long_rows(matvec_isa, oracle):
    """`matvec_kernel<S, MODE, 2, true>`: rows so long (n = 28672) that one partial sum per row and 64 columns does not fit
    beside the table and the activations; the lanes of a full slab are added first and a row keeps one sum per slab."""
    m, n, S, mode = 8192, 28672, 8, 0
    rng = np.random.default_rng(5)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    out = np.full(2 * m, 0xEE, dtype=np.uint8)
    rpb, rw_tail, items_tail, magic, lds_wide = _matvec_geometry(m, n)
    assert lds_wide > 160 * 1024                                    # which is why the library picks the compact form here
    lds_bytes = 65536 + 2 * n + 4 * ((n >> 11) + ((n & 2047) >> 6)) * rpb
    grid = (m + rpb - 1) // rpb
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x.view(np.uint8).copy(), "activations")
    mem.add(o_at, out, "output")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    blocks = [0, grid - 1]
    kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb1EE" % (S, mode))
    kernel.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                       ("i32", items_tail), ("u32", magic), ("ptr", o_at)], lds_bytes=lds_bytes,
                  groups=[(b, 0, 0) for b in blocks], seed=3)
    want = oracle.matvec(comp.view(np.uint32), cb, x, m, S, mode=mode)
    got = out.view(np.float16).astype(np.float64)
    for b in blocks:
        r0, r1 = b * rpb, min(m, (b + 1) * rpb)
        assert np.abs(got[r0:r1] - want[r0:r1]).max() / (np.abs(want).max() + 1e-9) < 2e-3


@pytest.mark.parametrize("m,n,L,mode", [(70, 192, 16, 0), (300, 128, 14, 1), (5, 64, 16, 1)])
def test_transposed_dense_export_is_bit_exact(matvec_t_isa, oracle, m, n, L, mode):
    """`matvec_t_dense_kernel<L, MODE>` (`csrc/matvec_t.hip`), a two-dimensional grid (row blocks x columns of 64)."""
    rng = np.random.default_rng(m + n + L)
    cb = rng.standard_normal(1 << L).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    W = np.full(m * n, 0xEEEE, dtype=np.uint16)
    mem = wave_model.Memory()
    c_at, cb_at, w_at = 0x7f40fffff000, 0x7f5000003400, 0x7f2ffffe0100
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(w_at, W.view(np.uint8), "dense matrix")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(matvec_t_isa, "_ZN4rptc21matvec_t_dense_kernelILi%dELi%dEE" % (L, mode))
    kernel.launch(mem, ((m + 255) // 256, n // 64), 256, [("ptr", c_at), ("ptr", cb_at), ("ptr", w_at), ("i32", m), ("i32", n // 64)], seed=m)
    want = oracle.matvec_t_dense(comp.view(np.uint32), cb, m, n, L, mode=mode)
    assert np.array_equal(W.reshape(m, n), want.view(np.uint16))


@pytest.mark.parametrize("L,steps,weighted", [(14, 3, False), (16, 2, True)])
def test_scalar_search_kernel_matches_the_oracle(viterbi_isa, oracle, L, steps, weighted):
    """`viterbi_scalar_kernel<L, WEIGHTED>` and its trace kernel (`csrc/viterbi.hip`): the reference's own trellis (2 bits and
    one alphabet value a step) for a few steps against `orc_viterbi`, to the bit."""
    rng = np.random.default_rng(L + steps)
    alphabet = rng.standard_normal(1 << L).astype(np.float16)
    targets = (0.7 * rng.standard_normal(steps)).astype(np.float32)
    weights = rng.uniform(0.25, 4.0, steps).astype(np.float32) if weighted else None
    back = np.full(steps * 1024, 0xABCDABCD, dtype=np.uint32)
    symbols = np.full(steps, 0xEE, dtype=np.uint8)
    end_state = np.full(1, -1, dtype=np.int32)
    cost = np.full(1, np.nan, dtype=np.float32)
    mem = wave_model.Memory()
    t_at, w_at, a_at, b_at, s_at, e_at, c_at = (0x7f4000000000, 0x7f4100000000, 0x7f4200000000, 0x7f4300000000, 0x7f4400000000,
                                                0x7f4500000000, 0x7f4600000000)
    mem.add(t_at, targets.view(np.uint8).copy(), "targets")
    if weighted:
        mem.add(w_at, weights.view(np.uint8).copy(), "weights")
    mem.add(a_at, alphabet.view(np.uint8).copy(), "alphabet")
    mem.add(b_at, back.view(np.uint8), "back pointers")
    mem.add(s_at, symbols, "symbols")
    mem.add(e_at, end_state.view(np.uint8), "end state")
    mem.add(c_at, cost.view(np.uint8), "cost")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    search = wave_model.Kernel(viterbi_isa, "_ZN4rptc21viterbi_scalar_kernelILi%dELb%dEE" % (L, 1 if weighted else 0))
    search.launch(mem, (1,), 1024, [("ptr", t_at), ("ptr", w_at if weighted else 0), ("i64", 0), ("ptr", a_at), ("ptr", b_at), ("ptr", e_at),
                                    ("ptr", c_at), ("i32", steps)], lds_bytes=2 * ((1 << L) // 4) * 4 + 2 * 1024 * 4, seed=L)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    trace = wave_model.Kernel(viterbi_isa, "_ZN4rptc27viterbi_scalar_trace_kernelILi%dEE" % L)
    trace.launch(mem, (1,), 64, [("ptr", b_at), ("ptr", e_at), ("ptr", s_at), ("i32", 1), ("i32", steps)], seed=L)
    want_symbols, want_cost, want_end = oracle.viterbi(alphabet.astype(np.float32), 2, targets, weights)
    assert np.array_equal(symbols.astype(np.int32), want_symbols)
    assert cost.view(np.uint32)[0] == np.float32(want_cost).view(np.uint32) and int(end_state[0]) == want_end


@pytest.mark.parametrize("bits,m,n,batch,S,mode", [(3, 40, 2048 + 128, 5, 8, 0), (4, 100, 704, 20, 6, 1), (4, 16, 2048, 16, 8, 1), (3, 33, 4096, 18, 6, 0)])
def test_batched_kernel_at_3_and_4_bits(matmul_isa, oracle, bits, m, n, batch, S, mode):
    """`matmul_kernel<S, MODE, PLANES, BITS>` for the 3- and 4-bit streams (an element is 2 * BITS words; fewer row blocks a
    workgroup) behind `pack_x_kernel`, against the dense matrix the oracle decodes times the activations."""
    rng = np.random.default_rng(m + n + batch + bits)
    codebook = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    stream = rng.integers(0, 256, m * n * bits // 8, dtype=np.uint8)
    x = (rng.standard_normal((batch, n)) * 0.5).astype(np.float16)
    out = np.full((batch, m), np.nan, dtype=np.float16)
    planes = 2 if batch > 16 else 1
    slabs = n // 2048 + (1 if n % 2048 else 0)
    total = (m + 15) // 16
    groups = max(1, min(2 * CUS // slabs, total))
    groups = max(groups, -(-total // (6 if planes == 1 else 3)))
    max_rb = -(-total // groups)
    xpack = np.zeros(planes * (n // 2) * 16 + 1536, dtype=np.uint32)
    partial = np.zeros(groups * slabs * max_rb * planes * 256, dtype=np.float32)
    arrived = np.full(groups, 0xABCD, dtype=np.uint32)
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
    xp_at, p_at, a_at = 0x7f6000000000, 0x7f6100000000, 0x7f6200000000
    for at, data, name in ((c_at, stream, "stream"), (cb_at, codebook.view(np.uint8).copy(), "codebook"),
                           (x_at, x.view(np.uint8).reshape(-1).copy(), "activations"), (o_at, out.view(np.uint8).reshape(-1), "output"),
                           (xp_at, xpack.view(np.uint8), "packed activations"), (p_at, partial.view(np.uint8), "partial tiles"),
                           (a_at, arrived.view(np.uint8), "arrival counters")):
        mem.add(at, data, name)
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    pack = wave_model.Kernel(matmul_isa, "_ZN4rptc13pack_x_kernelE")
    threads = max(planes * (n // 8) * 16, groups)
    pack.launch(mem, ((threads + 255) // 256,), 256,
                [("ptr", x_at), ("ptr", xp_at), ("ptr", a_at), ("i32", groups), ("i32", n), ("i32", batch), ("i32", planes)], seed=m)
    mem.regions = [r for r in mem.regions if r[2] != "kernarg"]
    kernel = wave_model.Kernel(matmul_isa, "_ZN4rptc13matmul_kernelILi%dELi%dELi%dELi%dEE" % (S, mode, planes, bits))
    kernel.launch(mem, (groups * slabs,), 512,
                  [("ptr", c_at), ("ptr", cb_at), ("ptr", xp_at), ("i32", m), ("i32", n), ("i32", total // groups), ("i32", total % groups),
                   ("i32", 0), ("i32", max_rb), ("ptr", p_at), ("ptr", a_at), ("ptr", o_at), ("i32", batch)],
                  lds_bytes=65536 + 8 * 2 * 256 * 4, seed=m)
    W = oracle.bits_dense(stream.view(np.uint32), codebook, m, n, S, bits, mode=mode).astype(np.float64)
    want = x.astype(np.float64) @ W.T
    assert np.abs(out.astype(np.float64) - want).max() / (np.abs(want).max() + 1e-9) < 2e-3
    assert not arrived.any()


def run_one_layer(isa, oracle, m, n, S, mode, blocks, seed=7, burst=8, latency=(400, 60), silu=False):
    """`matvec_one_kernel<S, MODE, MAXI>` (`csrc/matvec_steady.hip`) as `matvec_one_launch` launches it: the per-launch op's
    arguments plus the reciprocal of the ragged row's length, the chain kernel's fixed LDS layout."""
    rng = np.random.default_rng(seed + m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    x_in = x
    if silu:
        # [gate | up]: the activations are silu(gate) * up, the gate rounded to fp16 before the product (csrc/rptc_common.hpp)
        gate, up = (rng.standard_normal(n) * 1.5).astype(np.float16), (rng.standard_normal(n) * 0.5).astype(np.float16)
        g32 = gate.astype(np.float32)
        x = ((g32 / (1.0 + np.exp(-g32))).astype(np.float16) * up).astype(np.float16)
        x_in = np.concatenate([gate, up])
    out = np.full(2 * m, 0xEE, dtype=np.uint8)
    rpb, rw_tail, items_tail, magic, _ = _matvec_geometry(m, n)
    T, lt = n >> 11, (n & 2047) >> 6
    total = T * (rpb // 2) + items_tail
    per_wave = -(-total // 16)
    assert (T + (1 if lt else 0)) * 4096 <= 32768 and rpb * (n // 64) * 4 <= 65536 and per_wave <= 6
    tail_magic = 65536 // lt + 1 if lt else 0
    grid = (m + rpb - 1) // rpb
    mem = wave_model.Memory()
    c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
    mem.add(c_at, comp, "stream")
    mem.add(cb_at, cb.view(np.uint8).copy(), "codebook")
    mem.add(x_at, x_in.view(np.uint8).copy(), "activations")
    mem.add(o_at, out, "output")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = latency
    kernel = wave_model.Kernel(isa, "_ZN4rptc17matvec_one_kernelILi%dELi%dELi%dELi%dEE" % (S, mode, 3 if per_wave <= 3 else 4 if per_wave <= 4 else 6, 1 if silu else 0))
    blocks = sorted({b for b in blocks if b < grid})
    kernel.launch(mem, (grid,), 1024, [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail),
                                       ("i32", items_tail), ("u32", magic), ("u32", tail_magic), ("ptr", o_at), ("ptr", 0), ("ptr", 0),
                                       ("ptr", 0), ("f32", 0.0)], lds_bytes=160 * 1024,
                  groups=[(b, 0, 0) for b in blocks], seed=seed, burst=burst)
    want = oracle.matvec(comp.view(np.uint32), cb, x, m, S, mode=mode)
    got = out.view(np.float16).astype(np.float64)
    touched = np.zeros(m, dtype=bool)
    for b in blocks:
        r0, r1 = b * rpb, min(m, (b + 1) * rpb)
        touched[r0:r1] = True
        err = np.abs(got[r0:r1] - want[r0:r1]).max() / (np.abs(want).max() + 1e-9)
        assert err < 2e-3, f"workgroup {b}: rows {r0}..{r1 - 1} differ by {err:.3g} of the largest output"
    assert (out.view(np.uint16)[~touched] == 0xEEEE).all()


@pytest.mark.parametrize("m,n,S,mode", [(33, 4096 + 768, 8, 0), (33, 4096 + 768, 6, 1), (300, 64, 6, 0), (7, 704, 8, 1), (4096, 11008, 8, 0),
                                        (11008, 4096, 8, 1), (8192, 8192, 8, 0), (64, 16384, 6, 1), (1000, 2048 + 64 * 31, 8, 1),
                                        (22016, 4096, 8, 0), (22016, 4096, 6, 1), (12288, 4096, 8, 1), (40000, 2048 + 192, 8, 1)])
def test_one_layer_kernel_matches_the_oracle(steady_isa, oracle, m, n, S, mode):
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    run_one_layer(steady_isa, oracle, m, n, S, mode, blocks=[0, 1, (m - 1) // rpb])


@pytest.mark.parametrize("seed", range(4))
def test_one_layer_kernel_on_random_shapes(steady_isa, oracle, seed):
    """Shapes drawn from ragged and full widths and from row counts around the grid's multiples, whatever fits the
    kernel's LDS layout and six elements a wave; first, last and one other workgroup; S, carry mode, the SiLU form, the
    interleaving and the memory latency by seed."""
    import random
    rnd = random.Random(900 + seed)
    done = 0
    while done < 3:
        n = 64 * rnd.choice([1, 2, 5, 31, 32, 33, 47, 64, 65, 96, 127, 128, 160, 172, 200, 255, 256])
        m = rnd.choice([1, 2, 3, 17, 100, 511, 512, 513, 1000, 4096, 5000, 11008, 12288, 22016, 30000, 44000])
        rpb, rw_tail, items_tail, magic, _ = _matvec_geometry(m, n)
        T, lt = n >> 11, (n & 2047) >> 6
        per_wave = -(-(T * (rpb // 2) + items_tail) // 16)
        if not ((T + (1 if lt else 0)) * 4096 <= 32768 and rpb * (n // 64) * 4 <= 65536 and per_wave <= 6):
            continue
        grid = (m + rpb - 1) // rpb
        run_one_layer(steady_isa, oracle, m, n, rnd.choice([6, 8]), rnd.choice([0, 1]), blocks=sorted({0, grid - 1, rnd.randrange(grid)}),
                      seed=rnd.randrange(1000), burst=rnd.choice([1, 8, 64]), latency=rnd.choice([(400, 60), (3000, 300), (5, 2)]),
                      silu=rnd.random() < 0.3)
        done += 1


@pytest.mark.parametrize("burst,latency", [(1, (3000, 300)), (64, (5, 2))])
def test_one_layer_kernel_under_other_interleavings(steady_isa, oracle, burst, latency):
    run_one_layer(steady_isa, oracle, 100, 4096 + 64 * 7, 8, 1, blocks=[0, 3], burst=burst, latency=latency)


@pytest.mark.parametrize("m,n,S,mode", [(40, 2048 + 320, 8, 0), (4096, 11008, 8, 1), (300, 64, 6, 0)])
def test_one_layer_kernel_with_the_silu_gate_in_front(steady_isa, oracle, m, n, S, mode):
    rpb = 2 * ((m + 2 * CUS - 1) // (2 * CUS))
    run_one_layer(steady_isa, oracle, m, n, S, mode, blocks=[0, (m - 1) // rpb], silu=True)


@pytest.mark.parametrize("m,n,S,mode", [(4096, 11008, 8, 0), (33, 4096 + 768, 6, 1), (22016, 4096, 8, 1)])
def test_one_layer_kernel_has_the_per_launch_kernels_bits(matvec_isa, steady_isa, m, n, S, mode):
    """Both kernels add an element's four sums, a row's partial sums and the lanes of the row's wave in the same order, so
    routing the op through the other kernel changes no output bit."""
    rng = np.random.default_rng(3)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    rpb, rw_tail, items_tail, magic, lds_plain = _matvec_geometry(m, n)
    lt = (n & 2047) >> 6
    per_wave = -(-((n >> 11) * (rpb // 2) + items_tail) // 16)
    grid = (m + rpb - 1) // rpb
    outs = []
    for one in (True, False):
        out = np.full(2 * m, 0xEE, dtype=np.uint8)
        mem = wave_model.Memory()
        c_at, cb_at, x_at, o_at = 0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f2ffffe0100
        for at, data, name in ((c_at, comp, "stream"), (cb_at, cb.view(np.uint8).copy(), "codebook"), (x_at, x.view(np.uint8).copy(), "activations"),
                               (o_at, out, "output")):
            mem.add(at, data, name)
        wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
        head = [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail), ("i32", items_tail), ("u32", magic)]
        if one:
            kernel = wave_model.Kernel(steady_isa, "_ZN4rptc17matvec_one_kernelILi%dELi%dELi%dELi0EE" % (S, mode, 3 if per_wave <= 3 else 4 if per_wave <= 4 else 6))
            kernel.launch(mem, (grid,), 1024, head + [("u32", 65536 // lt + 1 if lt else 0), ("ptr", o_at), ("ptr", 0), ("ptr", 0), ("ptr", 0), ("f32", 0.0)],
                          lds_bytes=160 * 1024, groups=[(0, 0, 0)], seed=1)
        else:
            kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc13matvec_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
            kernel.launch(mem, (grid,), 1024, head + [("ptr", o_at)], lds_bytes=lds_plain, groups=[(0, 0, 0)], seed=1)
        outs.append(out)
    assert np.array_equal(outs[0], outs[1]) and (outs[0][:2 * min(rpb, m)] != 0xEE).any()


@pytest.mark.parametrize("m,n,S,mode,with_delta", [(40, 2048 + 320, 8, 0, True), (12288, 4096, 8, 1, True), (33, 64 * 7, 6, 0, False),
                                                   (22016, 4096, 8, 1, True)])
def test_one_layer_kernel_with_the_norm_in_front_has_the_fused_kernels_bits(matvec_isa, steady_isa, m, n, S, mode, with_delta):
    """The XMODE 2 form (residual add + RMS norm in the prologue) against `matvec_fused_kernel` with the same prologue:
    the same output bits and the same residual stream written back."""
    rng = np.random.default_rng(m + n)
    cb = (rng.standard_normal(2 << S) * 0.1).astype(np.float16)
    comp = rng.integers(0, 256, m * n // 4, dtype=np.uint8)
    x_in = (rng.standard_normal(n) * 1.2).astype(np.float16)
    delta = (rng.standard_normal(n) * 0.3).astype(np.float16)
    weight = (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float16)
    rpb, rw_tail, items_tail, magic, lds_plain = _matvec_geometry(m, n)
    lt = (n & 2047) >> 6
    per_wave = -(-((n >> 11) * (rpb // 2) + items_tail) // 16)
    grid = (m + rpb - 1) // rpb
    results = []
    for one in (True, False):
        out = np.full(2 * m, 0xEE, dtype=np.uint8)
        res = np.full(2 * n, 0xEE, dtype=np.uint8)
        mem = wave_model.Memory()
        c_at, cb_at, x_at, d_at, w_at, r_at, o_at = (0x7f40fffff000, 0x7f5000003400, 0x7f3ffff0fe00, 0x7f3000000000, 0x7f3100000000, 0x7f3200000000,
                                                     0x7f2ffffe0100)
        for at, data, name in ((c_at, comp, "stream"), (cb_at, cb.view(np.uint8).copy(), "codebook"), (x_at, x_in.view(np.uint8).copy(), "residual in"),
                               (d_at, delta.view(np.uint8).copy(), "delta"), (w_at, weight.view(np.uint8).copy(), "norm weight"),
                               (r_at, res, "residual out"), (o_at, out, "output")):
            mem.add(at, data, name)
        wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
        head = [("ptr", c_at), ("ptr", cb_at), ("ptr", x_at), ("i32", m), ("i32", n), ("i32", rpb), ("i32", rw_tail), ("i32", items_tail), ("u32", magic)]
        dptr = ("ptr", d_at if with_delta else 0)
        if one:
            kernel = wave_model.Kernel(steady_isa, "_ZN4rptc17matvec_one_kernelILi%dELi%dELi%dELi2EE" % (S, mode, 3 if per_wave <= 3 else 4 if per_wave <= 4 else 6))
            kernel.launch(mem, (grid,), 1024, head + [("u32", 65536 // lt + 1 if lt else 0), ("ptr", o_at), dptr, ("ptr", w_at), ("ptr", r_at), ("f32", 1e-5)],
                          lds_bytes=160 * 1024, groups=[(0, 0, 0)], seed=1)
        else:
            kernel = wave_model.Kernel(matvec_isa, "_ZN4rptc19matvec_fused_kernelILi%dELi%dELi2ELb0EE" % (S, mode))
            kernel.launch(mem, (grid,), 1024, head + [dptr, ("ptr", o_at), ("ptr", w_at), ("ptr", r_at), ("f32", 1e-5), ("i32", 0)],
                          lds_bytes=lds_plain + 48 * 4, groups=[(0, 0, 0)], seed=1)
        results.append((out, res))
    assert np.array_equal(results[0][0], results[1][0]) and np.array_equal(results[0][1], results[1][1])
    assert (results[0][1] != 0xEE).any() and (results[0][0][:2 * min(rpb, m)] != 0xEE).any()


# ------------------------------------------------------------------------------------------------
# bench_aids/probe.hip: the read-only kernels whose times bench.py prints as the memory floor

@pytest.fixture(scope="module")
def probe_isa(tmp_path_factory):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not found")
    out = str(tmp_path_factory.mktemp("isa") / "probe.s")
    subprocess.run(["hipcc", "-O3", "-std=c++17", "--offload-arch=gfx950", "-I", os.path.join(PKG, "csrc"), "--cuda-device-only", "-S",
                    os.path.join(os.path.dirname(PKG), "bench_aids", "probe.hip"), "-o", out], check=True, capture_output=True)
    return out


@pytest.mark.parametrize("copies,layers,per_group16,grid", [(3, 5, 2752, 4), (1, 1, 7, 3), (2, 4, 3072, 2)])
def test_read_only_chain_probe_stays_inside_its_layers(probe_isa, copies, layers, per_group16, grid):
    """`probe_read_chain_kernel` reads workgroup b's share of every layer and nothing else: the buffers have no slack, so a
    request one element past a layer or the pointer table fails the model's bounds check; nothing is stored."""
    rng = np.random.default_rng(copies + layers)
    mem = wave_model.Memory()
    ptrs = np.zeros(copies, dtype=np.uint64)
    for c in range(copies):
        at = 0x7f4100000000 + (c << 32) + 0x100 * c
        ptrs[c] = at
        mem.add(at, rng.integers(0, 256, 16 * per_group16 * grid, dtype=np.uint8), f"layer {c}")
    p_at = 0x7f2000000000
    mem.add(p_at, ptrs.view(np.uint8).copy(), "layer pointers")
    wave_model.Wave.vm_latency, wave_model.Wave.lgkm_latency = 400, 60
    kernel = wave_model.Kernel(probe_isa, "_ZN12_GLOBAL__N_123probe_read_chain_kernelEPKmiiiPj")
    kernel.launch(mem, (grid,), 1024, [("ptr", p_at), ("i32", copies), ("i32", layers), ("i32", per_group16), ("ptr", 0)],
                  lds_bytes=0, groups=[(0, 0, 0), (grid - 1, 0, 0)], seed=2)


def test_read_only_probe_stays_inside_its_buffer(probe_isa):
    total16 = 2 * 3072 + 1000
    mem = wave_model.Memory()
    at = 0x7f4100000000
    mem.add(at, np.arange(16 * total16, dtype=np.uint32).astype(np.uint8), "stream")
    kernel = wave_model.Kernel(probe_isa, "_ZN12_GLOBAL__N_117probe_read_kernelEPKjPjm")
    kernel.launch(mem, (3,), 1024, [("ptr", at), ("ptr", 0), ("u64", total16)], lds_bytes=0, groups=[(0, 0, 0), (2, 0, 0)], seed=2)

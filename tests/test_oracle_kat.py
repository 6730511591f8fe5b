"""Pins the CPU oracle against evidence that does not come from the oracle: hand-derived known
answers, exhaustive integer closed forms, bit-string brute force and thread-level simulations of
the CUDA kernels on tiny inputs.  Runs without a GPU."""
import json
import os

import numpy as np
import pytest

import sim

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat.json")))


def rng(seed=42):
    return np.random.default_rng(seed)


def rand_words(shape, seed=42):
    return rng(seed).integers(0, 1 << 32, size=shape, dtype=np.uint64).astype(np.uint32)


def rand_half(n, seed=7):
    return rng(seed).standard_normal(n).astype(np.float16)


IDENT16 = np.arange(65536, dtype=np.uint16)          # codebook[s] has the raw bits s


# ------------------------------------------------------------------ fp16 conversions

def test_half_to_float_all_patterns(oracle):
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.half_to_float(h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_float_to_half_matches_numpy_rne(oracle):
    g = rng(3)
    f = np.concatenate([
        (g.standard_normal(200000) * 10.0 ** g.integers(-9, 6, 200000)).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 2.0 ** -14 * (1 - 2.0 ** -11), 5.9604645e-08 * 1.5, np.inf, -np.inf], dtype=np.float32),
        # every half value plus/minus tiny offsets exercises ties
        (np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)),
    ])
    # exact midpoints between consecutive halves
    hv = np.arange(0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    hn = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((hv + hn) / 2).astype(np.float32)
    f = np.concatenate([f, mids, -mids]).astype(np.float32)
    assert f.dtype == np.float32
    with np.errstate(over="ignore"):
        want = f.astype(np.float16)
    got = oracle.float_to_half(f)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------ rptc.py:74-85

def test_dequantize_hand_derived_states(oracle):
    # symbols of 0xDEADBEEF, MSB first; identity alphabet returns the state itself
    word = 0xDEADBEEF
    symbols = [(word >> (30 - 2 * i)) & 3 for i in range(16)]
    alphabet = np.arange(65536, dtype=np.float32)
    got = oracle.dequantize(alphabet, symbols).astype(np.int64)
    want = [int(s, 16) for s in KAT["shift_register_states_of_word_0xDEADBEEF"]]
    # re-derive the table: the state is the last 8 symbols written in base 4
    rederived = []
    for t in range(16):
        last = symbols[max(0, t - 7):t + 1]
        rederived.append(int("".join(format(s, "02b") for s in last), 2))
    assert rederived == want
    assert got.tolist() == want


@pytest.mark.parametrize("L", [4, 10, 14, 16])
def test_dequantize_is_sliding_window(oracle, L):
    g = rng(L)
    symbols = g.integers(0, 4, 300)
    alphabet = g.standard_normal(1 << L).astype(np.float32)
    got = oracle.dequantize(alphabet, symbols)
    bits = "".join(format(int(s), "02b") for s in symbols)
    want = np.array([alphabet[sim.window(bits, 2 * (t + 1), L)] for t in range(300)], dtype=np.float32)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ inference.cu:42-96

@pytest.mark.parametrize("continuous", [False, True])
def test_decompress_vs_bitstring_bruteforce(oracle, continuous):
    comp = rand_words((3, 4 * 96), seed=11)          # 96 elements: crosses two 32-element boundaries
    got = oracle.decompress(comp, IDENT16, mode=int(continuous)).view(np.uint16)
    want = sim.decompress_bruteforce(comp, IDENT16, continuous)
    assert np.array_equal(got, want)


def test_decompress_modes_differ_only_after_every_32nd_element(oracle):
    comp = rand_words((2, 4 * 64), seed=5)
    a = oracle.decompress(comp, IDENT16, mode=oracle.AS_WRITTEN).view(np.uint16)
    c = oracle.decompress(comp, IDENT16, mode=oracle.CONTINUOUS).view(np.uint16)
    diff = np.argwhere(a != c)
    assert len(diff) > 0
    # only the first 7 outputs of element 32 can see the history bits
    assert set(diff[:, 1].tolist()) <= set(range(64 * 32, 64 * 32 + 7))
    # and there the as-written history is the high half of the previous w
    r = 0
    prev_w = int(comp[r, 4 * 31 + 3])
    first = int(comp[r, 4 * 32]) >> 30
    assert a[r, 64 * 32] == (((prev_w >> 16) << 2) | first) & 0xFFFF
    assert c[r, 64 * 32] == (((prev_w & 0xFFFF) << 2) | first) & 0xFFFF


def test_decompress_continuous_equals_rptc_dequantize(oracle):
    g = rng(9)
    symbols = g.integers(0, 4, 64 * 64)              # one row, 64 elements
    words = sim.pack_symbols_msb_first(symbols).reshape(1, -1)
    cb = g.standard_normal(65536).astype(np.float16)
    got = oracle.decompress(words, cb, mode=oracle.CONTINUOUS)[0]
    want = oracle.dequantize_h(cb, symbols)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    want32 = oracle.dequantize(cb.astype(np.float32), symbols)
    assert np.array_equal(got.astype(np.float32), want32)


def test_decompress_constant_streams(oracle):
    cb = rand_half(65536)
    zeros = np.zeros((2, 4 * 32), dtype=np.uint32)
    out = oracle.decompress(zeros, cb)
    assert np.all(out.view(np.uint16) == cb.view(np.uint16)[0])
    ones = np.full((1, 4 * 32), 0xFFFFFFFF, dtype=np.uint32)
    out = oracle.decompress(ones, IDENT16).view(np.uint16)[0]
    assert out[:8].tolist() == [(1 << (2 * (i + 1))) - 1 for i in range(8)]
    assert np.all(out[7:] == 0xFFFF)


# ------------------------------------------------------------------ inference.cu:250-262 hash

def test_hash_known_answers(oracle):
    for row in KAT["matvec_hash"]:
        h = int(row["h"], 16)
        assert (h * (h + 1)) & 0xFFFFFFFF == int(row["hash"], 16)      # the table itself
        for S, key in ((8, "e8"), (6, "e6")):
            hv, e, s = oracle.hash_window(h, S)
            assert hv == int(row["hash"], 16)
            assert e == row[key]
            assert s == row["sign"]


@pytest.mark.parametrize("S", [6, 8])
def test_hash_exhaustive(oracle, S):
    for h in range(0, 65536, 1):
        prod = h * (h + 1)                            # exact Python integer
        hv, e, s = oracle.hash_window(h, S)
        assert hv == prod & 0xFFFFFFFF
        assert e == (prod >> 8) % (1 << S)
        assert s == (prod >> 15) & 1
    # bits above 16 in h do not reach the entry or the sign
    for h in (0x12345678, 0xFFFFBEEF, 0x8000FFFF):
        assert oracle.hash_window(h, S)[1:] == oracle.hash_window(h & 0xFFFF, S)[1:]


# ------------------------------------------------------------------ inference.cu:189-277

@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("continuous", [False, True])
def test_matvec_vs_thread_level_simulation(oracle, S, continuous):
    T, m = 2, 3
    comp = rand_words((T, m, 128), seed=20 + S)
    cb = rand_half(2 << S, seed=S)
    x = rand_half(2048 * T, seed=1)
    got = oracle.matvec(comp, cb, x, m, S, mode=int(continuous))
    want = sim.matvec_cuda_sim(comp, cb.view(np.uint16), x, S, continuous)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("n", [2048, 4096, 2048 + 64, 4096 + 768, 64, 704])
@pytest.mark.parametrize("mode", [0, 1])
def test_matvec_one_hot_recovers_dense(oracle, n, mode):
    """x = e_p gives y[r] = W[r, p]: pins the (slab, k, j, lane) -> column map of the dense export
    against the literal kernel loop, ragged last slab included."""
    m, S = 2, 8
    comp = rand_words(m * n // 16, seed=n)
    cb = rand_half(2 << S, seed=2)
    W = oracle.matvec_dense(comp, cb, m, n, S, mode=mode)
    eye = np.eye(n, dtype=np.float16)
    Y = oracle.matvec(comp, cb, eye, m, S, mode=mode)        # [n, m]
    assert np.array_equal(Y.T, W.astype(np.float64))
    # every column was written exactly once: the map is a bijection
    cb1 = np.ones(2 << S, dtype=np.float16)
    W1 = oracle.matvec_dense(comp, cb1, m, n, S, mode=mode)
    assert np.all(np.abs(W1.astype(np.float32)) == 1.0)


def test_matvec_zero_stream_closed_form(oracle):
    # all-zero stream: every window is 0 -> hash 0 -> entry 0, sign 0
    m, n, S = 4, 4096, 6
    comp = np.zeros(m * n // 16, dtype=np.uint32)
    cb = rand_half(2 << S, seed=3)
    x = rand_half(n, seed=4)
    y = oracle.matvec(comp, cb, x, m, S)
    xe = x.astype(np.float64)[0::2].sum()
    xo = x.astype(np.float64)[1::2].sum()
    want = abs(float(cb[0])) * xe + float(cb[1]) * xo
    assert np.allclose(y, want, rtol=1e-12)


def test_matvec_sign_is_replaced_not_toggled(oracle):
    # window 0x00B5 -> hash 0x80AE: sign bit 1, entry 0 (S=6).  Put it in the last 16 bits of x.
    m, n, S = 1, 2048, 6
    comp = np.zeros(m * n // 16, dtype=np.uint32)
    comp[0] = 0x00B5                                   # lane 0, word x: step (k=0, j=3) sees lo16(x)
    for neg in (False, True):
        cb = np.ones(2 << S, dtype=np.float16) * 2
        if neg:
            cb[0] = -2.0
        W = oracle.matvec_dense(comp, cb, m, n, S)
        # step k=0, j=3 of lane 0, slab 0: P = (0*4+3)*32 = 96 -> i = 0, idx = 96 -> columns 768, 769
        assert float(W[0, 768]) == -2.0 and float(W[0, 769]) == 2.0
        # entry 0 elsewhere (window 0) keeps magnitude with sign bit 0
        assert float(W[0, 0]) == 2.0


def test_matvec_lane0_carry_rule(oracle):
    """Two-element example where the modes differ: lane 0's first four steps see its own w as
    history when read as written, the previous slab's lane 31 (or 0) when continuous."""
    m, n, S = 1, 4096, 8
    comp = np.zeros((2, m, 128), dtype=np.uint32)
    comp[0, 0, 3] = 0x00001234                         # slab 0 lane 0 .w
    comp[0, 0, 4 * 31 + 3] = 0x0000BEEF                # slab 0 lane 31 .w
    comp[1, 0, 3] = 0x00005678                         # slab 1 lane 0 .w
    cb = np.arange(2 << S).astype(np.float16)
    Wa = oracle.matvec_dense(comp, cb, m, n, S, mode=oracle.AS_WRITTEN)
    Wc = oracle.matvec_dense(comp, cb, m, n, S, mode=oracle.CONTINUOUS)

    def pair(h):
        prod = h * (h + 1)
        e = (prod >> 8) & 0xFF
        w0 = np.array([(int(cb.view(np.uint16)[2 * e]) & 0x7FFF) | (prod & 0x8000)], dtype=np.uint16).view(np.float16)[0]
        return float(w0), float(cb[2 * e + 1])

    # slab t, lane 0, step (k=7, j): P = ((8t+7)*4+j)*32, window = (carry16 << 4(j+1)) & 0xFFFF (x word is 0)
    for t, own, prev in ((0, 0x1234, 0x0000), (1, 0x5678, 0xBEEF)):
        for j in range(4):
            P = ((8 * t + 7) * 4 + j) * 32
            i, idx = divmod(P, n // 8)
            col = 8 * idx + 2 * i
            wa = pair((own << (4 * (j + 1))) & 0xFFFF)
            wc = pair((prev << (4 * (j + 1))) & 0xFFFF)
            assert (float(Wa[0, col]), float(Wa[0, col + 1])) == wa
            assert (float(Wc[0, col]), float(Wc[0, col + 1])) == wc


def test_matvec_f32_leg_agrees(oracle):
    m, n, S = 64, 4096 + 768, 8
    comp = rand_words(m * n // 16, seed=77)
    cb = rand_half(2 << S, seed=5)
    x = rand_half(n, seed=6)
    y64 = oracle.matvec(comp, cb, x, m, S)
    y32 = oracle.matvec_f32(comp, cb, x, m, S)
    assert np.linalg.norm(y32 - y64) / np.linalg.norm(y64) < 1e-5
    W = oracle.matvec_dense(comp, cb, m, n, S)
    assert np.allclose(oracle.dense_matvec(W, x), y64, rtol=1e-10, atol=1e-9)


# ------------------------------------------------------------------ inference_t.cu:68-175

@pytest.mark.parametrize("L", [14, 16])
@pytest.mark.parametrize("continuous", [False, True])
def test_matvec_t_vs_thread_level_simulation(oracle, L, continuous):
    m, n = 5, 256
    comp = rand_words(m * n // 16, seed=30 + L)
    cb = rand_half(1 << L, seed=L)
    x = rand_half(n, seed=8)
    got = oracle.matvec_t(comp, cb, x, m, L, mode=int(continuous))
    want = sim.matvec_t_cuda_sim(comp, cb.view(np.uint16), x, m, L, continuous)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    W = oracle.matvec_t_dense(comp, cb, m, n, L, mode=int(continuous))
    assert np.allclose(oracle.dense_matvec(W, x), got, rtol=1e-10, atol=1e-9)


@pytest.mark.parametrize("L", [14, 16])
def test_matvec_t_as_written_is_top_nibbles(oracle, L):
    """As written the word never advances: after word i the state is the top nibbles of the last
    words, newest lowest; the even column of all eight steps uses the half-advanced state."""
    m, n = 2, 256
    comp = rand_words(m * n // 16, seed=44)
    ident = np.arange(1 << L, dtype=np.uint16)
    W = oracle.matvec_t_dense(comp, ident, m, n, L, mode=oracle.AS_WRITTEN).view(np.uint16)
    mask = (1 << L) - 1
    for r in range(m):
        words = [int(comp[(col * m + r) * 4 + k]) for col in range(n // 64) for k in range(4)]
        nib = [w >> 28 for w in words]
        for wi in range(len(words)):
            hist = 0
            for q in range(max(0, wi - 4), wi):
                hist = (hist << 4) | nib[q]
            s4 = ((hist << 4) | nib[wi]) & mask
            s2 = (((hist & mask) << 2) | (words[wi] >> 30)) & mask
            cols = W[r, 16 * wi:16 * wi + 16]
            assert np.all(cols[0::2] == s2)
            assert np.all(cols[1::2] == s4)


@pytest.mark.parametrize("L", [14, 16])
def test_matvec_t_continuous_is_rptc_dequantize(oracle, L):
    g = rng(L + 100)
    m, n = 3, 192
    symbols = g.integers(0, 4, (m, n))
    cb = g.standard_normal(1 << L).astype(np.float16)
    comp = np.zeros(m * n // 16, dtype=np.uint32).reshape(n // 64, m, 4)
    for r in range(m):
        comp[:, r, :] = sim.pack_symbols_msb_first(symbols[r]).reshape(n // 64, 4)
    W = oracle.matvec_t_dense(comp, cb, m, n, L, mode=oracle.CONTINUOUS)
    for r in range(m):
        want = oracle.dequantize_h(cb, symbols[r])
        assert np.array_equal(W[r].view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------ rptc_lite.py:12-16

def _index_fn_python(x, L, S):
    x &= 0xFFFFFFFF
    x = (x * (2 * x + 1)) & 0xFFFFFFFF
    sx = x - (1 << 32) if x >= 1 << 31 else x         # int32 view
    sx ^= sx >> (L - S)                               # Python >> on negatives is arithmetic
    return sx & ((1 << S) - 1)


def test_lite_index_fn_known_answers(oracle):
    for x, want in KAT["lite_index_fn_L16_S9"]:
        assert _index_fn_python(x, 16, 9) == want
        assert oracle.lite_index_fn(x, 16, 9) == want
    g = rng(1)
    for x in g.integers(0, 1 << 32, 2000):
        assert oracle.lite_index_fn(int(x), 16, 9) == _index_fn_python(int(x), 16, 9)


def _index_fn_numpy_int32(x, L, S):
    """rptc_lite.py:12-16 evaluated the way the reference evaluates it: element-wise on int32 arrays, where the
    product wraps around and >> is an arithmetic shift (jax's default integer type is int32; numpy's int32 arrays
    have the same two properties).  Independent of the C restatement's unsigned arithmetic and casts."""
    x = np.asarray(x).astype(np.int32)
    with np.errstate(over="ignore"):
        x = x * (np.int32(2) * x + np.int32(1))
    x = x ^ (x >> np.int32(L - S))
    return x & np.int32((1 << S) - 1)


@pytest.mark.parametrize("L,S", [(16, 9), (16, 8), (12, 6), (20, 10), (16, 16)])
def test_lite_index_fn_exhaustive_against_int32_arrays(oracle, L, S):
    """Every state of the shift register (all 2^L values, L <= 16: 65536 of them; a 2^16 sample otherwise), every
    16-bit pattern shifted to the top of the word (negative int32 values: the arithmetic shift matters there),
    and a random sample of the whole int32 range."""
    states = np.arange(1 << min(L, 16), dtype=np.int64)
    if L > 16:
        states = rng(L).integers(0, 1 << L, 1 << 16)
    high = (np.arange(1 << 16, dtype=np.int64) << 16) - (1 << 31)
    anywhere = rng(S).integers(-(1 << 31), 1 << 31, 1 << 16)
    for xs in (states, high, anywhere):
        want = _index_fn_numpy_int32(xs, L, S)
        got = np.array([oracle.lite_index_fn(int(x) & 0xFFFFFFFF, L, S) for x in xs], dtype=np.int32)
        assert np.array_equal(got, want)
        assert want.min() >= 0 and want.max() < (1 << S)


def test_lite_index_fn_depends_on_the_low_L_bits_only(oracle):
    """x (2x + 1) mod 2^L depends on x mod 2^L only, and the index reads bits [0, S) and [L-S, L) of the product:
    bits of x above L never reach it.  This is why the reference's unmasked register (rptc_lite.py:65) is a
    window of L bits."""
    L, S = 16, 9
    g = rng(7)
    low = g.integers(0, 1 << L, 4096)
    high = g.integers(0, 1 << (32 - L), 4096)
    for lo, hi in zip(low, high):
        assert oracle.lite_index_fn(int((hi << L) | lo), L, S) == oracle.lite_index_fn(int(lo), L, S)


@pytest.mark.parametrize("L,S,R,V", [(16, 9, 4, 2), (16, 8, 2, 1), (12, 6, 3, 4), (16, 9, 8, 2)])
def test_lite_dequantize_is_a_window_of_L_bits(oracle, L, S, R, V):
    """rptc_lite.py:63-73 on sequences long enough for the int32 register to wrap many times: the output at step t
    is alphabet[index_fn(last L stream bits)], the index taken with the int32-array evaluation above on a register
    MASKED to L bits (which the reference never does; the property above says it changes nothing)."""
    g = rng(L * 100 + R)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    symbols = g.integers(0, 1 << R, 300)
    got = oracle.lite_dequantize(alphabet, L, S, R, symbols)
    state, want_idx = 0, []
    for s in symbols:
        state = ((state << R) | int(s)) & ((1 << L) - 1)
        want_idx.append(state)
    want = alphabet[_index_fn_numpy_int32(np.array(want_idx), L, S)]
    assert np.array_equal(got, want)
    # the first steps, by hand: state = s0, then (s0 << R) | s1
    s0, s1 = int(symbols[0]), int(symbols[1])
    assert np.array_equal(got[0], alphabet[int(_index_fn_numpy_int32([s0], L, S)[0])])
    assert np.array_equal(got[1], alphabet[int(_index_fn_numpy_int32([(s0 << R) | s1], L, S)[0])])


def test_lite_dequantize_window(oracle):
    L, S, R, V = 16, 9, 4, 2
    g = rng(2)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    symbols = g.integers(0, 1 << R, 40)
    got = oracle.lite_dequantize(alphabet, L, S, R, symbols)
    state = 0
    for t, s in enumerate(symbols):
        state = ((state << R) | int(s)) & 0xFFFFFFFF
        assert np.array_equal(got[t], alphabet[_index_fn_python(state, L, S)])


# ------------------------------------------------------------------ rptc_lite.py:19-60 (the search)

@pytest.mark.parametrize("L,S,R,V,steps,weighted", [(6, 3, 2, 2, 5, False), (6, 4, 3, 2, 4, True), (4, 2, 1, 1, 9, True), (8, 5, 4, 2, 3, False),
                                                     (5, 5, 2, 3, 5, True)])
def test_lite_quantize_finds_the_cheapest_sequence(oracle, L, S, R, V, steps, weighted):
    """Every symbol sequence of a small trellis, decoded by the decoder's own restatement (rptc_lite.py:63-73) and priced
    as rptc_lite.py:39 prices a step: none is cheaper than what the search returns, the returned sequence has that price,
    and among the cheapest sequences it is the one the recursion's first-index tie rule picks whenever the optimum is
    unique (random floats: it is)."""
    import itertools
    g = rng(100 * L + steps)
    alphabet = g.standard_normal((1 << S, V)).astype(np.float32)
    samples = g.standard_normal((steps, V)).astype(np.float32)
    importance = (g.random((steps, V)) + 0.25).astype(np.float32) if weighted else None
    got, cost = oracle.lite_quantize(alphabet, L, S, R, importance, samples)
    w = importance if weighted else np.ones((steps, V), dtype=np.float32)

    def price(seq):
        out = oracle.lite_dequantize(alphabet, L, S, R, np.array(seq, dtype=np.int32))
        return float((w.astype(np.float64) * (samples.astype(np.float64) - out) ** 2).sum())
    prices = {seq: price(seq) for seq in itertools.product(range(1 << R), repeat=steps)}
    best = min(prices, key=prices.get)
    assert abs(prices[best] - float(cost)) <= 1e-5 * max(1.0, prices[best])
    assert abs(price(tuple(int(v) for v in got)) - float(cost)) <= 1e-5 * max(1.0, float(cost))
    ranked = sorted(prices.values())
    if ranked[1] - ranked[0] > 1e-4:
        assert tuple(int(v) for v in got) == best


def test_lite_quantize_starts_from_state_zero_and_breaks_ties_low(oracle):
    """rho[0] = 0 and infinity elsewhere at the start (rptc_lite.py:42-43): the first symbols shift into a zero register.
    With an alphabet of equal rows every sequence costs the same; argmin's first index (rptc_lite.py:34 for a step,
    :52 for the end state) then gives the all-zero sequence."""
    L, S, R, V = 6, 3, 2, 2
    alphabet = np.full((1 << S, V), 0.5, dtype=np.float32)
    samples = rng(5).standard_normal((7, V)).astype(np.float32)
    got, cost = oracle.lite_quantize(alphabet, L, S, R, None, samples)
    assert not got.any()
    assert abs(float(cost) - float(((samples - 0.5) ** 2).sum())) < 1e-4


# ------------------------------------------------------------------ sign-Hadamard transform (no reference counterpart)

@pytest.mark.parametrize("P", [2, 64, 256, 1024])
def test_sign_hadamard_equals_dense_sylvester_product(oracle, P):
    from scipy.linalg import hadamard
    g = rng(P)
    n = 3 * P
    x = g.standard_normal((2, n)).astype(np.float16)
    s = np.where(g.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    H = hadamard(P).astype(np.float64)
    xs = x.astype(np.float64) * s.astype(np.float64)
    fwd = np.concatenate([(xs[:, b * P:(b + 1) * P] @ H.T) / np.sqrt(P) for b in range(3)], axis=1)
    assert np.allclose(oracle.sign_hadamard(x, s, P), fwd, rtol=1e-12, atol=1e-12)
    xd = x.astype(np.float64)
    inv = np.concatenate([(xd[:, b * P:(b + 1) * P] @ H.T) / np.sqrt(P) for b in range(3)], axis=1) * s.astype(np.float64)
    assert np.allclose(oracle.sign_hadamard(x, s, P, inverse=True), inv, rtol=1e-12, atol=1e-12)


def test_sign_hadamard_is_orthogonal(oracle):
    g = rng(5)
    n, P = 11008, 256
    x = g.standard_normal(n).astype(np.float16)
    s = np.where(g.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    y = oracle.sign_hadamard(x, s, P)
    assert np.isclose(np.linalg.norm(y), np.linalg.norm(x.astype(np.float64)), rtol=1e-12)

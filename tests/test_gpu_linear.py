"""QuantizedLinear and the model patcher on the GPU, against dense reconstructions."""
import numpy as np
import pytest
import torch

from util import rand_codes, rand_half, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available()
    return rptc_kernels


@pytest.mark.parametrize("batch", [1, 5, 32, 70])
def test_quantized_linear_matches_dense_reconstruction(rk, batch):
    from rptc_kernels.linear import QuantizedLinear
    n, m = 4096 + 768, 1024
    layer = QuantizedLinear.from_random(n, m, S=8, seed=1)
    g = torch.Generator(device="cuda").manual_seed(2)
    so = (torch.rand(m, generator=g, device="cuda") + 0.5).half()
    si = (torch.rand(n, generator=g, device="cuda") + 0.5).half()
    bo = (torch.randn(m, generator=g, device="cuda") * 0.01).half()
    bi = (torch.randn(n, generator=g, device="cuda") * 0.01).half()
    layer.set_affine(so, si, bo, bi)
    x = torch.randn((batch, n), generator=g, device="cuda").half()
    y = layer(x)
    assert y.shape == (batch, m) and y.dtype == torch.float16
    # quantize_hf.py:167: W = b_out + b_in + s_out * s_in * W_hat
    W = bo.double()[:, None] + bi.double()[None, :] + so.double()[:, None] * si.double()[None, :] * layer.decoded_weight().double()
    want = x.double() @ W.t()
    assert rel_l2(y.cpu().numpy(), want.cpu().numpy()) < 2e-3      # several fp16 roundings in the epilogue


def test_quantized_linear_with_sign_hadamard(rk):
    from rptc_kernels.linear import QuantizedLinear
    n, m = 11008, 256
    layer = QuantizedLinear.from_random(n, m, S=6, seed=3)
    signs = torch.where(torch.rand(n, device="cuda") < 0.5, -1.0, 1.0).half()
    layer.set_signs(signs)
    x = torch.randn((3, 2, n), device="cuda").half()
    y = layer(x)
    assert y.shape == (3, 2, m)
    t = torch.empty((6, n), dtype=torch.float16, device="cuda")
    rk.sign_hadamard(x.reshape(6, n).contiguous(), signs, t)
    want = t.double() @ layer.decoded_weight().double().t()
    assert rel_l2(y.reshape(6, m).cpu().numpy(), want.cpu().numpy()) < 1e-3


def test_from_weight_in_the_sign_hadamard_basis_spreads_outliers(rk):
    """A weight with a few large columns: quantized as it is, the outliers cost most of the error; in the
    sign-Hadamard basis they are spread over their block, and the layer (which transforms its input) is closer
    to the dense product."""
    from rptc_kernels.linear import QuantizedLinear
    g = torch.Generator().manual_seed(12)
    m, n = 64, 1024
    W = torch.randn((m, n), generator=g) * 0.02
    W[:, ::97] *= 12.0
    signs = torch.where(torch.rand(n, generator=g) < 0.5, -1.0, 1.0)
    x = torch.randn((4, n), generator=g).half().cuda()
    want = x.double() @ W.double().cuda().t()
    errs = []
    for sg in (None, signs):
        layer = QuantizedLinear.from_weight(W, S=8, seed=5, signs=sg)
        errs.append(rel_l2(layer(x).float().cpu().numpy(), want.cpu().numpy()))
    assert errs[1] < 0.6 * errs[0] and errs[1] < 0.4


def test_from_symbols_decodes_the_trellis_path(rk):
    from rptc_kernels.linear import QuantizedLinear
    from rptc_kernels import packing
    g = np.random.default_rng(4)
    m, n, S = 32, 2048 + 128, 8
    symbols = g.integers(0, 16, (m, n // 2))
    cb = g.standard_normal(2 << S).astype(np.float16)
    layer = QuantizedLinear.from_symbols(symbols, cb, m, S=S)
    W = layer.decoded_weight().cpu().numpy().view(np.uint16)
    cols = packing.matvec_stream_columns(n)
    cbb = cb.view(np.uint16)
    for r in (0, 17, 31):
        state = 0
        for p, sym in enumerate(symbols[r]):
            state = ((state << 4) | int(sym)) & 0xFFFF
            prod = state * (state + 1)
            e = (prod >> 8) & 0xFF
            assert W[r, cols[p]] == (int(cbb[2 * e]) & 0x7FFF) | (prod & 0x8000)
            assert W[r, cols[p] + 1] == cbb[2 * e + 1]


def test_patch_model_replaces_the_reference_module_list(rk):
    from rptc_kernels.linear import QuantizedLinear, patch_model

    class Attn(torch.nn.Module):
        def __init__(self, d):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj, self.o_proj = (torch.nn.Linear(d, d, bias=False) for _ in range(4))

    class Mlp(torch.nn.Module):
        def __init__(self, d, f):
            super().__init__()
            self.gate_proj, self.up_proj = torch.nn.Linear(d, f, bias=False), torch.nn.Linear(d, f, bias=False)
            self.down_proj = torch.nn.Linear(f, d, bias=False)

        def forward(self, x):
            return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))

    class Layer(torch.nn.Module):
        def __init__(self, d, f):
            super().__init__()
            self.self_attn, self.mlp = Attn(d), Mlp(d, f)

    class Inner(torch.nn.Module):
        def __init__(self, d, f):
            super().__init__()
            self.layers = torch.nn.ModuleList([Layer(d, f) for _ in range(2)])

    class Model(torch.nn.Module):
        def __init__(self, d=256, f=704):
            super().__init__()
            self.model = Inner(d, f)
            self.lm_head = torch.nn.Linear(d, 100, bias=False)

    model = Model().half().cuda()
    names = patch_model(model)
    assert len(names) == 14 and "lm_head" not in names        # 7 projections per layer, quantize_hf.py:189
    assert isinstance(model.model.layers[1].mlp.down_proj, QuantizedLinear)
    assert isinstance(model.lm_head, torch.nn.Linear)
    mlp = model.model.layers[0].mlp
    x = torch.randn((1, 256), device="cuda").half()
    y = mlp(x)
    Wg, Wu, Wd = (l.decoded_weight().float() for l in (mlp.gate_proj, mlp.up_proj, mlp.down_proj))
    h = (torch.nn.functional.silu(x.float() @ Wg.t()).half().float() * (x.float() @ Wu.t()).half().float()).half().float()
    want = h @ Wd.t()
    assert rel_l2(y.float().cpu().numpy(), want.cpu().numpy()) < 5e-3


def test_from_weight_quantizes_and_runs(rk):
    """A real (small) weight through the Viterbi quantizer, the packer and the fused kernel: the layer
    output equals the dense product of what the symbols decode to, and the quantization error is the
    2-bit trellis code's, not a random matrix's."""
    from rptc_kernels.linear import QuantizedLinear
    from rptc_kernels import quantize
    g = torch.Generator().manual_seed(5)
    m, n = 16, 256
    W = torch.randn((m, n), generator=g) * 0.02
    layer = QuantizedLinear.from_weight(W, S=8)
    What = layer.decoded_weight().float().cpu()
    rel = ((W - What).norm() / W.norm()).item()
    assert rel < 0.45, rel                    # ~0.3 for a 2 bit/weight trellis code on Gaussian data
    x = torch.randn((1, n), generator=g).half().cuda()
    y = layer(x)
    want = x.double().cpu() @ What.double().t()
    assert rel_l2(y.cpu().numpy(), want.numpy()) < 1e-3


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("batch", [1, 20])
def test_quantized_linear_at_3_and_4_bits(rk, bits, batch):
    from rptc_kernels.linear import QuantizedLinear
    n, m = 2048 + 192, 96
    layer = QuantizedLinear.from_random(n, m, S=8, seed=3, bits=bits)
    assert layer.compressed.numel() * 32 == m * n * bits
    x = torch.randn((batch, n), generator=torch.Generator().manual_seed(4)).half().cuda()
    y = layer(x)
    W = layer.decoded_weight()
    want = x.double() @ W.double().t()
    assert rel_l2(y.cpu().numpy(), want.cpu().numpy()) < 1e-3


def test_from_weight_at_3_bits_beats_2_bits(rk):
    from rptc_kernels.linear import QuantizedLinear
    g = torch.Generator().manual_seed(6)
    W = torch.randn((8, 256), generator=g) * 0.05
    l2 = QuantizedLinear.from_weight(W, S=8, bits=2)
    l3 = QuantizedLinear.from_weight(W, S=8, bits=3)
    assert l3.quantization_mse <= l2.quantization_mse
    x = torch.randn((1, 256), generator=g).half().cuda()
    want = x.double().cpu() @ l3.decoded_weight().double().cpu().t()
    assert rel_l2(l3(x).cpu().numpy(), want.numpy()) < 1e-3


def test_llama_decode_paths_agree(rk):
    """A 2-layer Llama-shaped model on streams: the fused one-token step matches the torch path's logits,
    graph replay reproduces direct launches token for token, and the logits match the same network run on
    the decoded dense weights."""
    from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama, greedy_decode
    from rptc_kernels.linear import QuantizedLinear
    shape = LlamaShape(layers=2, d_model=256, heads=4, d_ff=704, vocab=1000, max_len=128)
    model = QuantizedLlama(shape, S=8, seed=7)
    prompt = torch.randint(0, shape.vocab, (40,), generator=torch.Generator().manual_seed(1))
    runs = {}
    for mode in ("fused_graph", "fused", "glue_graph", "glue", "torch_graph", "torch"):
        model.k_cache.zero_(); model.v_cache.zero_()
        runs[mode], _ = greedy_decode(model, prompt, 12, mode=mode)
    assert runs["fused_graph"] == runs["fused"]
    assert runs["glue_graph"] == runs["glue"]
    assert runs["torch_graph"] == runs["torch"]

    # one decode step after the same prefill: fused glue vs torch glue
    pos = torch.arange(40, device="cuda")
    with torch.no_grad():
        model.k_cache.zero_(); model.v_cache.zero_()
        for p0 in (0, 32):
            model.forward_tokens(prompt[p0:p0 + 32].cuda(), pos[p0:p0 + 32])
        tok = torch.tensor([5], device="cuda")
        p40 = torch.tensor([40], device="cuda")
        kc, vc = model.k_cache.clone(), model.v_cache.clone()
        lt = model.forward_tokens(tok, p40)
        kt = model.k_cache.clone()
        model.k_cache.copy_(kc); model.v_cache.copy_(vc)
        lf = model.decode_step(tok, p40)
        assert rel_l2(lf.cpu().numpy(), lt.cpu().numpy()) < 1e-2
        assert rel_l2(model.k_cache.float().cpu().numpy(), kt.float().cpu().numpy()) < 1e-2
        # nine launches per layer against five: the same roundings, so nearly the same logits
        kf = model.k_cache.clone()
        model.k_cache.copy_(kc); model.v_cache.copy_(vc)
        lg = model.decode_step(tok, p40, fuse=False)
        assert rel_l2(lf.cpu().numpy(), lg.cpu().numpy()) < 2e-3
        assert rel_l2(model.k_cache.float().cpu().numpy(), kf.float().cpu().numpy()) < 2e-3

    # dense reference: swap every QuantizedLinear for a matmul with its decoded weight
    class Dense(torch.nn.Module):
        def __init__(self, w):
            super().__init__()
            self.w = w

        def forward(self, x):
            return (x.float() @ self.w.float().t()).half()

    with torch.no_grad():
        model.k_cache.zero_(); model.v_cache.zero_()
        logits_q = model.forward_tokens(prompt[:32].cuda(), pos[:32])
        for blk in model.blocks:
            for name, child in list(blk.named_children()):
                if isinstance(child, QuantizedLinear):
                    setattr(blk, name, Dense(child.decoded_weight()))
        model.k_cache.zero_(); model.v_cache.zero_()
        logits_d = model.forward_tokens(prompt[:32].cuda(), pos[:32])
    assert rel_l2(logits_q.cpu().numpy(), logits_d.cpu().numpy()) < 2e-2


def test_llama_built_from_dense_weights_through_the_reference_procedure(rk):
    """Random-init dense projections, factorised and searched (quantize_hf.py:77-170's flow on the hashed pair
    stream): every decode path agrees, and the logits are those of the same network on the matrices the layers
    reconstruct (quantize_hf.py:167)."""
    from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama, greedy_decode
    from rptc_kernels.linear import QuantizedLinear
    shape = LlamaShape(layers=2, d_model=256, heads=4, d_ff=704, vocab=1000, max_len=128)
    model = QuantizedLlama(shape, S=8, seed=11, quantize_init=True)
    blk = model.blocks[0]
    for name in ("qkv_proj", "o_proj", "gate_up_proj", "down_proj"):
        layer = getattr(blk, name)
        assert all(v is not None for v in (layer.scales_in, layer.scales_out, layer.biases_in, layer.biases_out))
        # the search did its work: 2 bits per weight on a Gaussian matrix lands well under the variance
        assert layer.quantization_mse < 0.12
    prompt = torch.randint(0, shape.vocab, (40,), generator=torch.Generator().manual_seed(2))
    runs = {}
    for mode in ("fused_graph", "fused", "glue", "torch"):
        model.k_cache.zero_(); model.v_cache.zero_()
        runs[mode], _ = greedy_decode(model, prompt, 10, mode=mode)
    assert runs["fused_graph"] == runs["fused"]

    pos = torch.arange(40, device="cuda")
    with torch.no_grad():
        model.k_cache.zero_(); model.v_cache.zero_()
        for p0 in (0, 32):
            model.forward_tokens(prompt[p0:p0 + 32].cuda(), pos[p0:p0 + 32])
        tok = torch.tensor([5], device="cuda")
        p40 = torch.tensor([40], device="cuda")
        kc, vc = model.k_cache.clone(), model.v_cache.clone()
        lf = model.decode_step(tok, p40)
        model.k_cache.copy_(kc); model.v_cache.copy_(vc)
        lg = model.decode_step(tok, p40, fuse=False)
        assert rel_l2(lf.cpu().numpy(), lg.cpu().numpy()) < 5e-3

        # dense reference on the reconstructed matrices, float32 products
        class Dense(torch.nn.Module):
            def __init__(self, w):
                super().__init__()
                self.w = w

            def forward(self, x):
                return (x.float() @ self.w.t()).half()

        for b in model.blocks:
            for name, child in list(b.named_children()):
                if isinstance(child, QuantizedLinear):
                    setattr(b, name, Dense(child.reconstructed_weight()))
        model.k_cache.copy_(kc); model.v_cache.copy_(vc)
        ld = model.forward_tokens(tok, p40)
    assert rel_l2(lf.cpu().numpy(), ld.cpu().numpy()) < 2e-2


@pytest.mark.parametrize("vocab,d", [(32000, 4096), (1000, 256), (5, 64), (70001, 128)])
def test_greedy_next_is_argmax_plus_bookkeeping(rk, vocab, d):
    import ctypes
    lib = rk.library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(vocab)
    embed = torch.randn((vocab, d), generator=g).half().cuda()
    out_list = torch.full((8,), -1, dtype=torch.long, device="cuda")
    idx = torch.tensor([2], dtype=torch.long, device="cuda")
    pos = torch.tensor([40], dtype=torch.long, device="cuda")
    tok = torch.tensor([7], dtype=torch.long, device="cuda")
    x = torch.zeros(d, dtype=torch.float16, device="cuda")
    for case in range(3):
        logits = torch.randn(vocab, generator=g).half().cuda()
        if case == 1:                               # equal maxima: the first one wins, as torch.argmax
            top = logits.max()
            logits[vocab // 2] = top
            logits[vocab - 1] = top
        if case == 2:
            logits[:] = 0.0                         # all equal: index 0
        want = int(logits.argmax())
        assert lib.rptc_greedy_next(logits.data_ptr(), vocab, embed.data_ptr(), d, tok.data_ptr(), out_list.data_ptr(),
                                    idx.data_ptr(), pos.data_ptr(), x.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert int(tok) == want and int(out_list[2 + case]) == want
        assert int(idx) == 3 + case and int(pos) == 41 + case
        assert torch.equal(x.view(torch.int16), embed[want].view(torch.int16))


# ------------------------------------------------------------------ projections with a fused element-wise prologue

def _stream(m, n, S=8, seed=0):
    comp = rand_codes(m * n // 16, seed=seed + m + n).cuda()
    cb = rand_half(2 << S, seed=seed + S).cuda()
    return comp, cb


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("S", [6, 8])
@pytest.mark.parametrize("m,n", [(64, 2048), (33, 704), (96, 4096 + 768), (32, 28672)])
def test_matvec_silu_equals_silu_then_matvec(rk, mode, S, m, n):
    """The gate is computed with the roundings of the stand-alone kernel, so the fused call is bit-identical."""
    import ctypes
    comp, cb = _stream(m, n, S, seed=3)
    gu = rand_half(2 * n, seed=21).cuda()
    act = torch.empty(n, dtype=torch.float16, device="cuda")
    rc = rk.library().rptc_silu_mul(gu.data_ptr(), act.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    want = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        getattr(rk, f"decompress_matvec_16_{S}_1")(comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp, cb, act, want)
        ms = rk.decompress_matvec_silu(comp, cb, gu, got)
    finally:
        rk.set_carry_mode(prev)
    assert ms > 0
    g, u = gu[:n].float(), gu[n:].float()
    assert rel_l2(act.float().cpu().numpy(), (torch.nn.functional.silu(g) * u).cpu().numpy()) < 1e-3
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("with_delta", [False, True])
@pytest.mark.parametrize("m,n", [(64, 2048), (40, 256), (96, 4096), (32, 16384)])
def test_matvec_rmsnorm_equals_norm_then_matvec(rk, mode, with_delta, m, n):
    import ctypes
    S = 8
    comp, cb = _stream(m, n, S, seed=5)
    x = rand_half(n, seed=31).cuda()
    delta = rand_half(n, seed=32, scale=0.5).cuda() if with_delta else None
    w = (1.0 + 0.1 * rand_half(n, seed=33).float()).half().cuda()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x_ref, h_ref = torch.empty_like(x), torch.empty_like(x)
    rc = rk.library().rptc_add_rmsnorm(x.data_ptr(), None if delta is None else delta.data_ptr(), w.data_ptr(),
                                       x_ref.data_ptr(), h_ref.data_ptr(), n, 1e-5, stream)
    assert rc == 0
    want = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    x_out = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        getattr(rk, f"decompress_matvec_16_{S}_1")(comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp, cb, h_ref, want)
        rk.decompress_matvec_rmsnorm(comp, cb, x, delta, w, x_out, got, eps=1e-5)
    finally:
        rk.set_carry_mode(prev)
    assert torch.equal(x_out.view(torch.int16), x_ref.view(torch.int16))       # the residual stream is exact
    # the norm: against float64 from the definition
    r = x_ref.double()
    h64 = r * torch.rsqrt((r * r).mean() + 1e-5) * w.double()
    assert rel_l2(h_ref.float().cpu().numpy(), h64.cpu().numpy()) < 1e-3
    # the sum of squares is added in another order, so the activations may differ in the last fp16 bit
    assert rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) < 1e-3


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("m,n,block", [(64, 4096, 0), (33, 11008, 0), (40, 2048 + 192, 0), (32, 8192, 0), (24, 14336, 0), (64, 4096, 256),
                                       (16, 64, 0)])
def test_matvec_hadamard_equals_transform_then_matvec(rk, mode, m, n, block):
    """The butterflies are the stand-alone kernel's, in the same order, so the fused call is bit-identical."""
    S = 8
    comp, cb = _stream(m, n, S, seed=7)
    x = rand_half(n, seed=51).cuda()
    signs = torch.where(torch.rand(n, generator=torch.Generator().manual_seed(52)) < 0.5, -1.0, 1.0).half().cuda()
    t = torch.empty_like(x)
    rk.sign_hadamard(x, signs, t, block=block)
    want = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        getattr(rk, f"decompress_matvec_16_{S}_1")(comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp, cb, t, want)
        ms = rk.decompress_matvec_hadamard(comp, cb, x, signs, got, block=block)
    finally:
        rk.set_carry_mode(prev)
    assert ms > 0
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_hadamard(comp, cb, x, signs, got, block=48)


def test_matvec_hadamard_refuses_vectors_that_do_not_fit_in_lds(rk):
    m, n = 32, 16384
    comp, cb = _stream(m, n, 8, seed=11)
    x = rand_half(n, seed=3).cuda()
    out = torch.empty(m, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds"):
        rk.decompress_matvec_hadamard(comp, cb, x, torch.ones_like(x), out)


def test_matvec_rmsnorm_rejects_aliases_and_long_vectors(rk):
    m, n = 32, 2048
    comp, cb = _stream(m, n, 8, seed=9)
    x, w = rand_half(n, seed=1).cuda(), rand_half(n, seed=2).cuda()
    out = torch.empty(m, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="aliases"):
        rk.decompress_matvec_rmsnorm(comp, cb, x, None, w, x, out)
    with pytest.raises(RuntimeError, match="aliases"):
        rk.decompress_matvec_rmsnorm(comp, cb, x, w, w, w, out)
    n2 = 16384 + 2048
    comp2, _ = _stream(m, n2, 8, seed=10)
    x2 = rand_half(n2, seed=3).cuda()
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_rmsnorm(comp2, cb, x2, None, x2.clone(), torch.empty_like(x2), out)


def _affine_vectors(m, n, which, seed):
    g = torch.Generator().manual_seed(seed)
    si = (torch.rand(n, generator=g) + 0.5).half().cuda() if "si" in which else None
    bi = (torch.randn(n, generator=g) * 0.02).half().cuda() if "bi" in which else None
    so = (torch.rand(m, generator=g) + 0.5).half().cuda() if "so" in which else None
    bo = (torch.randn(m, generator=g) * 0.02).half().cuda() if "bo" in which else None
    return si, bi, so, bo


def _affine_truth(W, a, si, bi, so, bo):
    """quantize_hf.py:167 in float64 on the decoded matrix W and the fp16 activations a (s_in * a rounded to
    fp16, as every path of this library stages it)."""
    a64 = a.double()
    xs = (a * si).double() if si is not None else a64            # fp16 product, rounded
    y = W.double() @ xs
    if so is not None:
        y = y * so.double()
    if bo is not None:
        y = y + bo.double() * a64.sum()
    if bi is not None:
        y = y + (bi.double() * a64).sum()
    return y


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("which", [(), ("si",), ("bi",), ("so",), ("bo",), ("si", "bi", "so", "bo")])
@pytest.mark.parametrize("S,m,n", [(8, 64, 2048), (6, 33, 704), (8, 96, 4096 + 768), (8, 600, 4096), (8, 32, 16384), (8, 2, 64)])
def test_matvec_affine_applies_the_factorisation(rk, mode, which, S, m, n):
    comp, cb = _stream(m, n, S, seed=13)
    x = rand_half(n, seed=61).cuda()
    si, bi, so, bo = _affine_vectors(m, n, which, seed=62)
    W = torch.empty((m, n), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        rk.matvec_dense(comp, cb, W, S)
        ms = rk.decompress_matvec_affine(comp, cb, x, got, si, bi, so, bo)
        if not which:
            plain = torch.empty_like(got)
            getattr(rk, f"decompress_matvec_16_{S}_1")(comp.reshape(n // 2048, m, 128) if n % 2048 == 0 else comp, cb, x, plain)
            assert torch.equal(got.view(torch.int16), plain.view(torch.int16))
    finally:
        rk.set_carry_mode(prev)
    assert ms > 0
    want = _affine_truth(W, x, si, bi, so, bo)
    assert rel_l2(got.float().cpu().numpy(), want.cpu().numpy()) < 1e-3


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("m,n", [(64, 2048), (96, 4096 + 768), (40, 11008)])
def test_matvec_silu_affine(rk, mode, m, n):
    import ctypes
    S = 8
    comp, cb = _stream(m, n, S, seed=15)
    gu = rand_half(2 * n, seed=71).cuda()
    act = torch.empty(n, dtype=torch.float16, device="cuda")
    assert rk.library().rptc_silu_mul(gu.data_ptr(), act.data_ptr(), n, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    si, bi, so, bo = _affine_vectors(m, n, ("si", "bi", "so", "bo"), seed=72)
    W = torch.empty((m, n), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        rk.matvec_dense(comp, cb, W, S)
        rk.decompress_matvec_silu_affine(comp, cb, gu, got, si, bi, so, bo)
    finally:
        rk.set_carry_mode(prev)
    assert rel_l2(got.float().cpu().numpy(), _affine_truth(W, act, si, bi, so, bo).cpu().numpy()) < 1e-3


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("with_delta", [False, True])
@pytest.mark.parametrize("m,n", [(64, 2048), (40, 256), (96, 4096), (32, 16384)])
def test_matvec_rmsnorm_affine(rk, mode, with_delta, m, n):
    import ctypes
    S = 8
    comp, cb = _stream(m, n, S, seed=17)
    x = rand_half(n, seed=81).cuda()
    delta = rand_half(n, seed=82, scale=0.5).cuda() if with_delta else None
    w = (1.0 + 0.1 * rand_half(n, seed=83).float()).half().cuda()
    x_ref, h_ref = torch.empty_like(x), torch.empty_like(x)
    assert rk.library().rptc_add_rmsnorm(x.data_ptr(), None if delta is None else delta.data_ptr(), w.data_ptr(),
                                         x_ref.data_ptr(), h_ref.data_ptr(), n, 1e-5,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    si, bi, so, bo = _affine_vectors(m, n, ("si", "bi", "so", "bo"), seed=84)
    W = torch.empty((m, n), dtype=torch.float16, device="cuda")
    got = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
    x_out = torch.full((n,), float("nan"), dtype=torch.float16, device="cuda")
    prev = rk.set_carry_mode(mode)
    try:
        rk.matvec_dense(comp, cb, W, S)
        rk.decompress_matvec_rmsnorm_affine(comp, cb, x, delta, w, x_out, got, 1e-5, si, bi, so, bo)
    finally:
        rk.set_carry_mode(prev)
    assert torch.equal(x_out.view(torch.int16), x_ref.view(torch.int16))
    # the normed activations may differ from the stand-alone kernel's in the last fp16 bit (order of the sum of squares)
    assert rel_l2(got.float().cpu().numpy(), _affine_truth(W, h_ref, si, bi, so, bo).cpu().numpy()) < 1e-3


def test_matvec_affine_refuses_long_vectors_and_checks_lengths(rk):
    m, n = 32, 16384 + 2048
    comp, cb = _stream(m, n, 8, seed=19)
    x = rand_half(n, seed=3).cuda()
    out = torch.empty(m, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds"):
        rk.decompress_matvec_affine(comp, cb, x, out, scales_in=torch.ones_like(x))
    m, n = 32, 2048
    comp, cb = _stream(m, n, 8, seed=20)
    x = rand_half(n, seed=4).cuda()
    with pytest.raises(RuntimeError):
        rk.decompress_matvec_affine(comp, cb, x, out, scales_out=torch.ones(n, dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("heads,hd,max_len,pos", [(4, 64, 128, 0), (4, 64, 128, 77), (32, 128, 1024, 640), (2, 16, 64, 63),
                                                 (256, 16, 32, 20), (64, 128, 2048, 2047), (3, 256, 48, 5)])
def test_rope_attn_decode_equals_rope_then_attention(rk, heads, hd, max_len, pos):
    import ctypes
    lib = rk.library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    d = heads * hd
    g = torch.Generator().manual_seed(pos + heads)
    qkv = torch.randn(3 * d, generator=g).half().cuda()
    kc = torch.randn((heads, max_len, hd), generator=g).half().cuda()
    vc = torch.randn((heads, max_len, hd), generator=g).half().cuda()
    # positions the context has not reached hold whatever an allocator left there: not-a-numbers here,
    # which must not leak into the result (the kernels may read such rows, and mask them)
    kc[:, pos:] = float("nan")
    vc[:, pos:] = float("nan")
    ang = torch.arange(max_len).float()[:, None] / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))[None, :]
    cos, sin = ang.cos().half().cuda().contiguous(), ang.sin().half().cuda().contiguous()
    p = torch.tensor([pos], dtype=torch.long, device="cuda")
    k1, v1, k2, v2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    q = torch.empty(d, dtype=torch.float16, device="cuda")
    o1 = torch.empty(d, dtype=torch.float16, device="cuda")
    o2 = torch.full((d,), float("nan"), dtype=torch.float16, device="cuda")
    assert lib.rptc_rope_cache(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), p.data_ptr(), q.data_ptr(), k1.data_ptr(),
                               v1.data_ptr(), heads, hd, max_len, stream) == 0
    assert lib.rptc_attn_decode(q.data_ptr(), k1.data_ptr(), v1.data_ptr(), p.data_ptr(), o1.data_ptr(), heads, hd, max_len,
                                stream) == 0
    assert lib.rptc_rope_attn_decode(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), p.data_ptr(), k2.data_ptr(),
                                     v2.data_ptr(), o2.data_ptr(), heads, hd, max_len, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(k1.view(torch.int16), k2.view(torch.int16)) and torch.equal(v1.view(torch.int16), v2.view(torch.int16))
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
    assert torch.isfinite(o2.float()).all()
    # and against the definition in float64
    kk, vv = k1[:, :pos + 1].double(), v1[:, :pos + 1].double()
    sc = torch.einsum("hd,hsd->hs", q.view(heads, hd).double(), kk) / hd ** 0.5
    want = torch.einsum("hs,hsd->hd", torch.softmax(sc, dim=-1), vv).reshape(-1)
    assert rel_l2(o2.float().cpu().numpy(), want.cpu().numpy()) < 2e-3


@pytest.mark.parametrize("quantize_init", [False, True])
def test_llama_2_7b_shaped_layer_at_position_600(rk, quantize_init):
    """One decoder layer at the Llama-2-7B shape (d 4096, 32 heads x 128, MLP 11008, vocabulary 32000), one token at
    position 600 over a cache of 600 seeded rows: the five-launch fused step (12288x4096 and 22016x4096 with the
    add + RMS norm prologue, rotation + cache append + 32-head attention, 4096x4096, 4096x11008 with the SiLU
    prologue) against the same arithmetic in framework ops on the decoded (or reconstructed) dense weights.
    Each projection is held to rel-L2 1e-3 on the input the fused step itself fed it; the logits to 2e-2."""
    from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama
    shape = LlamaShape(layers=1, d_model=4096, heads=32, d_ff=11008, vocab=32000, max_len=1024)
    model = QuantizedLlama(shape, S=8, seed=5, quantize_init=quantize_init)
    blk = model.blocks[0]
    d, f, pos_i = shape.d_model, shape.d_ff, 600
    g = torch.Generator(device="cuda").manual_seed(17)
    blk.norm1.copy_((1 + 0.1 * torch.randn(d, generator=g, device="cuda")).half())
    blk.norm2.copy_((1 + 0.1 * torch.randn(d, generator=g, device="cuda")).half())
    model.k_cache[:, :, :pos_i].copy_((torch.randn((1, shape.heads, pos_i, shape.head_dim), generator=g, device="cuda") * 0.5).half())
    model.v_cache[:, :, :pos_i].copy_((torch.randn((1, shape.heads, pos_i, shape.head_dim), generator=g, device="cuda") * 0.5).half())
    kc, vc = model.k_cache.clone(), model.v_cache.clone()
    tok = torch.tensor([1234], device="cuda")
    pos = torch.tensor([pos_i], device="cuda")

    def dense(layer):
        return (layer.reconstructed_weight() if quantize_init else layer.decoded_weight()).double()

    with torch.no_grad():
        logits_f = model.decode_step(tok, pos)
        torch.cuda.synchronize()
        x0 = model.embed[tok].reshape(-1)
        # q, k, v: the norm of the embedding row through the fused 12288 x 4096 projection
        h1 = model._rms(x0[None], blk.norm1)[0]
        want = dense(blk.qkv_proj) @ h1.double()
        assert rel_l2(model._qkv.double().cpu().numpy(), want.cpu().numpy()) < 1e-3
        # rotation + cache append + attention, from the projection's own output
        q, k, v = model._qkv.split(d)
        qr = model._rope(q.reshape(1, shape.heads, shape.head_dim), pos)
        kr = model._rope(k.reshape(1, shape.heads, shape.head_dim), pos)
        assert torch.equal(model.k_cache[0, :, pos_i], kr[0]) and torch.equal(model.v_cache[0, :, pos_i], v.reshape(shape.heads, -1))
        assert torch.equal(model.k_cache[0, :, :pos_i], kc[0, :, :pos_i]) and torch.equal(model.k_cache[0, :, pos_i + 1:], kc[0, :, pos_i + 1:])
        K, V = model.k_cache[0, :, :pos_i + 1].double(), model.v_cache[0, :, :pos_i + 1].double()
        att = torch.softmax(torch.einsum("hd,hsd->hs", qr[0].double(), K) / shape.head_dim ** 0.5, dim=-1)
        want = torch.einsum("hs,hsd->hd", att, V).reshape(-1)
        assert rel_l2(model._att.double().cpu().numpy(), want.cpu().numpy()) < 2e-3
        # o projection on the attention output the step produced
        want = dense(blk.o_proj) @ model._att.double()
        assert rel_l2(model._o.double().cpu().numpy(), want.cpu().numpy()) < 1e-3
        # gate / up: residual add + norm prologue of the 22016 x 4096 projection
        x1 = x0 + model._o
        h2 = model._rms(x1[None], blk.norm2)[0]
        want = dense(blk.gate_up_proj) @ h2.double()
        assert rel_l2(model._gu.double().cpu().numpy(), want.cpu().numpy()) < 1e-3
        # down: SiLU prologue of the 4096 x 11008 projection
        act = torch.nn.functional.silu(model._gu[:f].float()).half() * model._gu[f:]
        want = dense(blk.down_proj) @ act.double()
        assert rel_l2(model._down.double().cpu().numpy(), want.cpu().numpy()) < 2e-3

        # the whole step against framework ops on the dense matrices
        class Dense(torch.nn.Module):
            def __init__(self, w):
                super().__init__()
                self.w = w.float()

            def forward(self, x):
                return (x.float() @ self.w.t()).half()

        for name in ("qkv_proj", "o_proj", "gate_up_proj", "down_proj"):
            setattr(blk, name, Dense(dense(getattr(blk, name))))
        model.k_cache.copy_(kc); model.v_cache.copy_(vc)
        logits_d = model.forward_tokens(tok, pos)
    assert rel_l2(logits_f.cpu().numpy(), logits_d.cpu().numpy()) < 2e-2

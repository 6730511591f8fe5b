"""The whole Llama-2-7B-shaped decoder on the GPU: 32 layers (d 4096, 32 heads, MLP 11008, vocabulary 32000) on seeded
random 2-bit streams, a prompt of 512 seeded token ids, 128 greedy tokens, batch 1.

The reference generates with transformers on dense weights (quantize_hf.py:229-236); here every projection
(quantize_hf.py:189) runs on its packed stream.  Checked: the replayed HIP graph reproduces the direct launches token for
token over all 128 positions (KV-cache indexing across 32 layers, the position and token hand-over inside the graph, the
arg-max over 32000 logits), cache rows past the last written position stay untouched, and at sampled (layer, position)
pairs of the full-depth model every projection is within rel-L2 1e-3 of the double-precision product of its decoded
dense matrix with the input the step itself fed it.
"""
import pytest
import torch

from util import rel_l2

pytestmark = pytest.mark.gpu

PROMPT, NEW = 512, 128


@pytest.fixture(scope="module")
def rk():
    import rptc_kernels
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    assert rptc_kernels.library().rptc_init() == 0
    return rptc_kernels


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def test_llama_2_7b_shape_prompt_512_then_128_greedy_tokens(rk):
    from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama, greedy_decode
    shape = LlamaShape()                      # 32 layers, d 4096, 32 heads, MLP 11008, vocabulary 32000, 1024 positions
    assert (shape.layers, shape.d_model, shape.heads, shape.d_ff, shape.vocab) == (32, 4096, 32, 11008, 32000)
    model = QuantizedLlama(shape, S=8, seed=42)
    g = torch.Generator(device="cuda").manual_seed(9)
    for blk in model.blocks:                  # norms that are not all ones, so a skipped or doubled norm shows
        blk.norm1.copy_((1 + 0.1 * torch.randn(shape.d_model, generator=g, device="cuda")).half())
        blk.norm2.copy_((1 + 0.1 * torch.randn(shape.d_model, generator=g, device="cuda")).half())
    prompt = torch.randint(0, shape.vocab, (PROMPT,), generator=torch.Generator().manual_seed(42))
    last_written = PROMPT + NEW - 2           # the last token generated is never fed back
    sentinel = 123.0

    runs = {}
    for mode in ("fused_graph", "fused"):
        model.k_cache.fill_(sentinel)
        model.v_cache.fill_(sentinel)
        print(f"[step] greedy decode, {mode}", flush=True)
        runs[mode], seconds = greedy_decode(model, prompt, NEW, mode=mode)
        print(f"[step] {mode}: {(NEW - 1) / seconds:.1f} tok/s", flush=True)
        assert len(runs[mode]) == NEW and all(0 <= t < shape.vocab for t in runs[mode])
        # rows the context has not reached are untouched, in every layer; the rows it has reached are written
        assert bool((model.k_cache[:, :, last_written + 1:] == sentinel).all())
        assert bool((model.v_cache[:, :, last_written + 1:] == sentinel).all())
        assert not bool((model.k_cache[:, :, :last_written + 1] == sentinel).all(dim=-1).any())
        assert not bool((model.v_cache[:, :, :last_written + 1] == sentinel).all(dim=-1).any())
    assert runs["fused_graph"] == runs["fused"]
    assert len(set(runs["fused"])) > 1        # not stuck on one token

    # Sampled (layer, position) pairs of the full-depth model: one more step at two positions of the context just
    # built, the work buffers snapshotted behind the sampled layers.
    d, f = shape.d_model, shape.d_ff
    for pos_i, sampled in ((600, (0, 17)), (last_written, (9, 31))):
        snaps = {}

        def after_layer(i):
            if i in sampled:
                torch.cuda.synchronize()
                snaps[i] = {name: getattr(model, name).clone() for name in ("_x", "_x2", "_qkv", "_att", "_o", "_gu", "_down")}
                snaps[i]["k"] = model.k_cache[i, :, :pos_i + 1].clone()
                snaps[i]["v"] = model.v_cache[i, :, :pos_i + 1].clone()

        tok = torch.tensor([runs["fused"][pos_i - PROMPT]], device="cuda")
        pos = torch.tensor([pos_i], device="cuda")
        print(f"[step] one step at position {pos_i}, layers {sampled}", flush=True)
        with torch.no_grad():
            logits = model.decode_step(tok, pos, after_layer=after_layer)
            torch.cuda.synchronize()
            assert bool(torch.isfinite(logits).all())
            for i in sampled:
                s, blk = snaps[i], model.blocks[i]
                # q, k, v: add + RMS norm prologue of the 12288 x 4096 projection, on the residual stream it wrote
                h1 = model._rms(s["_x2"][None], blk.norm1)[0]
                want = blk.qkv_proj.decoded_weight().double() @ h1.double()
                assert rel_l2(s["_qkv"].double().cpu().numpy(), want.cpu().numpy()) < 1e-3, (i, pos_i, "qkv")
                # rotation, cache append at this position and attention over positions 0..pos
                q, k, v = s["_qkv"].split(d)
                qr = model._rope(q.reshape(1, shape.heads, shape.head_dim), pos)
                kr = model._rope(k.reshape(1, shape.heads, shape.head_dim), pos)
                assert torch.equal(s["k"][:, pos_i], kr[0]) and torch.equal(s["v"][:, pos_i], v.reshape(shape.heads, -1))
                att = torch.softmax(torch.einsum("hd,hsd->hs", qr[0].double(), s["k"].double()) / shape.head_dim ** 0.5, dim=-1)
                want = torch.einsum("hs,hsd->hd", att, s["v"].double()).reshape(-1)
                assert rel_l2(s["_att"].double().cpu().numpy(), want.cpu().numpy()) < 2e-3, (i, pos_i, "attention")
                # o projection
                want = blk.o_proj.decoded_weight().double() @ s["_att"].double()
                assert rel_l2(s["_o"].double().cpu().numpy(), want.cpu().numpy()) < 1e-3, (i, pos_i, "o")
                # gate / up: the residual stream after attention is what the prologue wrote
                assert torch.equal(s["_x"], (s["_x2"].float() + s["_o"].float()).half())
                h2 = model._rms(s["_x"][None], blk.norm2)[0]
                want = blk.gate_up_proj.decoded_weight().double() @ h2.double()
                assert rel_l2(s["_gu"].double().cpu().numpy(), want.cpu().numpy()) < 1e-3, (i, pos_i, "gate_up")
                # down: SiLU prologue of the 4096 x 11008 projection
                act = torch.nn.functional.silu(s["_gu"][:f].float()).half() * s["_gu"][f:]
                want = blk.down_proj.decoded_weight().double() @ act.double()
                assert rel_l2(s["_down"].double().cpu().numpy(), want.cpu().numpy()) < 2e-3, (i, pos_i, "down")

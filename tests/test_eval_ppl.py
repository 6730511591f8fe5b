"""The perplexity harness (the measure of the reference's contrib/eval_ppl.py:13-45)."""
import math
import os

import numpy as np
import pytest
import torch

from rptc_kernels import eval_ppl


def test_uniform_logits_give_the_vocabulary_size():
    vocab, seqlen = 50, 16
    tokens = eval_ppl.synthetic_tokens(5 * seqlen + 3, vocab)          # the 3 left-over tokens are dropped
    ppl, loss, n = eval_ppl.perplexity(lambda w: torch.zeros(w.numel(), vocab), tokens, seqlen)
    assert n == 5
    assert abs(ppl - vocab) < 1e-6 * vocab and abs(loss - math.log(vocab)) < 1e-6


def test_a_model_that_knows_the_next_token_has_perplexity_one():
    vocab, seqlen = 20, 8
    tokens = eval_ppl.synthetic_tokens(3 * seqlen, vocab, seed=1)

    def oracle_logits(w):
        lg = torch.full((w.numel(), vocab), -50.0)
        lg[torch.arange(w.numel() - 1), w[1:]] = 50.0                   # position t predicts token t+1
        return lg
    ppl, _, _ = eval_ppl.perplexity(oracle_logits, tokens, seqlen)
    assert abs(ppl - 1.0) < 1e-6


def test_matches_a_float64_restatement_and_the_window_mean():
    # mean over windows of (mean over the T-1 predicted positions), then exp: eval_ppl.py:35-45
    vocab, seqlen, nw = 11, 6, 4
    g = torch.Generator().manual_seed(3)
    table = torch.randn(vocab, vocab, generator=g)                      # logits depend on the current token
    tokens = eval_ppl.synthetic_tokens(nw * seqlen, vocab, seed=2)
    ppl, loss, n = eval_ppl.perplexity(lambda w: table[w], tokens, seqlen)
    t = tokens.numpy().reshape(nw, seqlen)
    tb = table.numpy().astype(np.float64)
    losses = []
    for w in t:
        acc = 0.0
        for a, b in zip(w[:-1], w[1:]):
            acc += math.log(np.exp(tb[a]).sum()) - tb[a, b]
        losses.append(acc / (seqlen - 1))
    assert n == nw and abs(loss - np.mean(losses)) < 1e-5 and abs(ppl - math.exp(np.mean(losses))) < 1e-4 * ppl


def test_token_files_round_trip(tmp_path):
    ids = np.array([5, 0, 31999, 17, 4], dtype=np.int64)
    np.save(tmp_path / "t.npy", ids.astype(np.int32))
    ids.astype("<u2").tofile(tmp_path / "t.u16")
    ids.astype("<i4").tofile(tmp_path / "t.i32")
    (tmp_path / "t.txt").write_text(" ".join(str(int(i)) for i in ids))
    torch.save(torch.from_numpy(ids), tmp_path / "t.pt")
    for name in ("t.npy", "t.u16", "t.i32", "t.txt", "t.pt"):
        got = eval_ppl.load_tokens(os.fspath(tmp_path / name))
        assert got.dtype == torch.int64 and got.tolist() == ids.tolist(), name
    with pytest.raises(ValueError):
        eval_ppl.load_tokens("tokens.pkl")
    with pytest.raises(ValueError):
        eval_ppl.perplexity(lambda w: None, ids[:3], 8)


@pytest.mark.gpu
def test_perplexity_of_a_stream_model_matches_its_dense_twin():
    """A 2-layer Llama-shaped model on packed streams against the same model with every projection
    replaced by a dense fp16 matmul over the decoded weights: same perplexity to 1 %."""
    print("\n[case] perplexity: streams vs decoded dense weights", flush=True)
    from rptc_kernels.llama_decode import LlamaShape, QuantizedLlama
    shape = LlamaShape(layers=2, d_model=256, heads=4, d_ff=704, vocab=1000, max_len=64)
    model = QuantizedLlama(shape, S=8, seed=11)
    tokens = eval_ppl.synthetic_tokens(3 * 64, shape.vocab, seed=5)
    ppl_q, loss_q, n = eval_ppl.perplexity(eval_ppl.llama_logits_fn(model), tokens, 64)
    assert n == 3 and math.isfinite(ppl_q)

    class Dense(torch.nn.Module):
        def __init__(self, q):
            super().__init__()
            self.w = q.decoded_weight()

        def forward(self, x):
            return (x.float() @ self.w.float().t()).half()
    for blk in model.blocks:
        for name in ("qkv_proj", "o_proj", "gate_up_proj", "down_proj"):
            setattr(blk, name, Dense(getattr(blk, name)))
    ppl_d, loss_d, _ = eval_ppl.perplexity(eval_ppl.llama_logits_fn(model), tokens, 64)
    assert abs(loss_q - loss_d) < 1e-2 * abs(loss_d), (ppl_q, ppl_d)

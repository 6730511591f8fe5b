"""Perplexity of a causal language model on a local token file.

Same measure as the reference's contrib/eval_ppl.py:13-45: the token stream is cut into
``numel // seqlen`` windows of ``seqlen`` tokens (eval_ppl.py:22-24), each window goes through the
model on its own, the loss of a window is the mean cross entropy of logits[:-1] against tokens[1:]
(eval_ppl.py:35-39), and the perplexity is exp of the mean window loss (eval_ppl.py:43-45).  What
differs is where the tokens come from: the reference tokenizes wikitext2 / c4 with a downloaded
tokenizer (gptq_data_utils.py:12-73); here they are read from a file of token ids, or drawn from a
seeded generator when there is none, because nothing can be downloaded.
"""
import argparse
import json
import math

import numpy as np
import torch


def load_tokens(path):
    """1-D int64 tensor of token ids from ``.npy`` (no pickles), ``.pt`` (tensor only), ``.txt``
    (whitespace-separated integers) or a raw little-endian file (``.u16`` / ``.i32``)."""
    if path.endswith(".npy"):
        arr = np.load(path, allow_pickle=False)
    elif path.endswith(".pt"):
        arr = torch.load(path, weights_only=True).cpu().numpy()
    elif path.endswith(".txt"):
        with open(path) as f:
            arr = np.array([int(t) for t in f.read().split()], dtype=np.int64)
    elif path.endswith(".u16"):
        arr = np.fromfile(path, dtype="<u2")
    elif path.endswith(".i32"):
        arr = np.fromfile(path, dtype="<i4")
    else:
        raise ValueError(f"unknown token file type: {path}")
    return torch.from_numpy(np.ascontiguousarray(arr).astype(np.int64).reshape(-1))


def synthetic_tokens(count, vocab, seed=42):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g, dtype=torch.int64)


def window_loss(logits, tokens):
    """Mean cross entropy (nats) of logits[:-1] against tokens[1:]; logits [T, vocab], tokens [T]."""
    logp = torch.log_softmax(logits[:-1].float(), dim=-1)
    return float(-logp.gather(1, tokens[1:].reshape(-1, 1).to(logp.device)).mean())


def perplexity(logits_fn, tokens, seqlen, progress=None):
    """``logits_fn(window)`` maps a 1-D window of ``seqlen`` token ids to logits [seqlen, vocab].
    Returns (perplexity, mean loss, number of windows)."""
    tokens = torch.as_tensor(tokens, dtype=torch.int64).reshape(-1)
    nsamples = tokens.numel() // seqlen
    if nsamples < 1:
        raise ValueError(f"{tokens.numel()} tokens do not fill one window of {seqlen}")
    windows = tokens[:nsamples * seqlen].view(nsamples, seqlen)
    acc = 0.0
    with torch.no_grad():
        for i in range(nsamples):
            acc += window_loss(logits_fn(windows[i]), windows[i])
            if progress is not None:
                progress(i + 1, nsamples, acc / (i + 1))
    avg = acc / nsamples
    return math.exp(avg), avg, nsamples


def llama_logits_fn(model, chunk=32):
    """Logits of every position of a window from a ``llama_decode.QuantizedLlama``: the window is fed in
    chunks of ``chunk`` tokens (the batch the fused mat-mat kernel takes) through the KV cache, which is
    simply overwritten from position 0 for every window."""
    dev = model.embed.device

    def fn(window):
        T = window.numel()
        if T > model.shape.max_len:
            raise ValueError(f"window of {T} tokens exceeds the model's max_len {model.shape.max_len}")
        w = window.to(dev)
        out = []
        for p0 in range(0, T, chunk):
            part = w[p0:p0 + chunk]
            out.append(model.forward_tokens(part, torch.arange(p0, p0 + part.numel(), device=dev), all_logits=True))
        return torch.cat(out, dim=0)
    return fn


def main(argv=None):
    from .llama_decode import LlamaShape, QuantizedLlama
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--tokens", help="token id file (.npy, .pt, .txt, .u16, .i32); default: seeded random ids")
    ap.add_argument("--seqlen", type=int, default=512)
    ap.add_argument("--windows", type=int, default=4, help="windows of synthetic tokens when no file is given")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--d-model", type=int, default=4096)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--d-ff", type=int, default=11008)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--seed", type=int, default=42)
    a = ap.parse_args(argv)
    shape = LlamaShape(layers=a.layers, d_model=a.d_model, heads=a.heads, d_ff=a.d_ff, vocab=a.vocab, max_len=a.seqlen)
    model = QuantizedLlama(shape, seed=a.seed)
    tokens = load_tokens(a.tokens) if a.tokens else synthetic_tokens(a.windows * a.seqlen, a.vocab, a.seed)
    if int(tokens.max()) >= a.vocab or int(tokens.min()) < 0:
        raise ValueError("token ids outside the model's vocabulary")
    ppl, loss, n = perplexity(llama_logits_fn(model), tokens, a.seqlen)
    print(json.dumps({"perplexity": ppl, "avg_loss": loss, "windows": n, "seqlen": a.seqlen,
                      "tokens": a.tokens or "synthetic", "model": "random-init Llama shape on 2-bit streams"}))


if __name__ == "__main__":
    main()

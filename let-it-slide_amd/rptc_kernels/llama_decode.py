"""A Llama-architecture decoder whose seven projections per layer are QuantizedLinear streams.

The reference quantizes ``model.layers.N.{self_attn.{q,k,v,o}_proj, mlp.{gate,up,down}_proj}`` of a
HuggingFace Llama-2-7B (quantize_hf.py:189) but writes dense weights back and generates with
``transformers`` (quantize_hf.py:229-236).  Here the same module list runs on the packed streams.
The model is built from its shape only (random-init norms, embeddings and lm_head; seeded random
streams for the projections): nothing is downloaded.  Greedy decode of one sequence; the whole
per-token step is captured in one HIP graph so that host launch overhead does not set the rate.
"""
import torch

from .linear import QuantizedLinear


class LlamaShape:
    def __init__(self, layers=32, d_model=4096, heads=32, d_ff=11008, vocab=32000, max_len=1024, rope_theta=10000.0):
        self.layers, self.d_model, self.heads, self.d_ff = layers, d_model, heads, d_ff
        self.vocab, self.max_len, self.rope_theta = vocab, max_len, rope_theta
        self.head_dim = d_model // heads


class QuantizedLlama(torch.nn.Module):
    def __init__(self, shape, S=8, seed=42, device="cuda"):
        super().__init__()
        self.shape = shape
        g = torch.Generator(device=device)
        g.manual_seed(seed)
        d, f = shape.d_model, shape.d_ff
        self.embed = (torch.randn((shape.vocab, d), generator=g, device=device) * 0.02).half()
        self.lm_head = (torch.randn((shape.vocab, d), generator=g, device=device) * d ** -0.5).half()
        self.final_norm = torch.ones(d, dtype=torch.float16, device=device)
        self.blocks = torch.nn.ModuleList()
        for i in range(shape.layers):
            blk = torch.nn.Module()
            for j, (name, n_in, n_out) in enumerate((("q_proj", d, d), ("k_proj", d, d), ("v_proj", d, d), ("o_proj", d, d),
                                                     ("gate_proj", d, f), ("up_proj", d, f), ("down_proj", f, d))):
                setattr(blk, name, QuantizedLinear.from_random(n_in, n_out, S=S, seed=seed + 16 * i + j, device=device))
            blk.norm1 = torch.ones(d, dtype=torch.float16, device=device)
            blk.norm2 = torch.ones(d, dtype=torch.float16, device=device)
            self.blocks.append(blk)
        hd = shape.head_dim
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, hd, 2, device=device).float() / hd))
        ang = torch.arange(shape.max_len, device=device).float()[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().half(), ang.sin().half()                       # [max_len, hd/2]
        self.k_cache = torch.zeros((shape.layers, shape.heads, shape.max_len, hd), dtype=torch.float16, device=device)
        self.v_cache = torch.zeros_like(self.k_cache)

    @staticmethod
    def _rms(x, w):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * w

    def _rope(self, t, pos):
        # t [T, heads, hd]; pos [T] (long)
        c, s = self.cos[pos][:, None, :], self.sin[pos][:, None, :]
        a, b = t[..., 0::2], t[..., 1::2]
        return torch.stack([a * c - b * s, a * s + b * c], dim=-1).flatten(-2)

    def forward_tokens(self, tokens, pos):
        """tokens [T] long, pos [T] long (their positions, contiguous); writes the KV cache at pos and
        returns the logits of the last token.  Attention looks at cache positions <= the token's own."""
        sh = self.shape
        T = tokens.numel()
        x = self.embed[tokens]                                                     # [T, d]
        key_pos = torch.arange(sh.max_len, device=x.device)
        mask = key_pos[None, :] <= pos[:, None]                                    # [T, max_len]
        for i, blk in enumerate(self.blocks):
            h = self._rms(x, blk.norm1)
            q = self._rope(blk.q_proj(h).view(T, sh.heads, sh.head_dim), pos)
            k = self._rope(blk.k_proj(h).view(T, sh.heads, sh.head_dim), pos)
            v = blk.v_proj(h).view(T, sh.heads, sh.head_dim)
            self.k_cache[i].index_copy_(1, pos, k.transpose(0, 1))
            self.v_cache[i].index_copy_(1, pos, v.transpose(0, 1))
            o = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), self.k_cache[i], self.v_cache[i],
                                                                 attn_mask=mask[None])      # [heads, T, hd]
            o = o.transpose(0, 1).reshape(T, sh.d_model)
            x = x + blk.o_proj(o)
            h = self._rms(x, blk.norm2)
            x = x + blk.down_proj(torch.nn.functional.silu(blk.gate_proj(h)) * blk.up_proj(h))
        h = self._rms(x[-1:], self.final_norm)
        return (h @ self.lm_head.t()).float()                                      # [1, vocab]


def greedy_decode(model, prompt, new_tokens, use_graph=True):
    """Prefill the prompt (in chunks of 32 tokens: the batch the fused mat-mat kernel takes), then decode
    ``new_tokens`` greedily one at a time.  Returns (token list, seconds spent in the decode loop)."""
    import time
    dev = model.embed.device
    prompt = torch.as_tensor(prompt, dtype=torch.long, device=dev)
    P = prompt.numel()
    with torch.no_grad():
        logits = None
        for p0 in range(0, P, 32):
            chunk = prompt[p0:p0 + 32]
            logits = model.forward_tokens(chunk, torch.arange(p0, p0 + chunk.numel(), device=dev))
        tok = logits.argmax(-1)                                                    # [1]
        out = [int(tok)]
        s_tok = tok.clone()
        s_pos = torch.tensor([P], dtype=torch.long, device=dev)
        if use_graph:
            # warm up on a side stream, then capture one decode step with static token/position tensors
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                model.forward_tokens(s_tok, s_pos)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                s_next = model.forward_tokens(s_tok, s_pos).argmax(-1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(new_tokens - 1):
            if use_graph:
                graph.replay()
                nxt = s_next
            else:
                nxt = model.forward_tokens(s_tok, s_pos).argmax(-1)
            s_tok.copy_(nxt)
            s_pos.add_(1)
            out.append(nxt.clone())
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    return [int(t) for t in out], dt

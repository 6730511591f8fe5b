"""A Llama-architecture decoder whose projections are QuantizedLinear streams.

The reference quantizes ``model.layers.N.{self_attn.{q,k,v,o}_proj, mlp.{gate,up,down}_proj}`` of a
HuggingFace Llama-2-7B (quantize_hf.py:189) but writes dense weights back and generates with
``transformers`` (quantize_hf.py:229-236).  Here the same projections run on the packed streams,
grouped the way the reference groups them for its Hessians (quantize_hf.py:14-22: q, k, v -> one
"qkv" matrix, gate and up -> one "up" matrix), which is one kernel launch per group.  The model is
built from its shape only (random-init norms, embeddings and lm_head; for the projections seeded random
streams, or random-init dense weights quantized with the reference's procedure): nothing is downloaded.

Two ways through a token: ``forward_tokens`` (torch ops between the projections; used for the
prompt, any number of tokens) and ``decode_step`` (this library's fused glue kernels, one token).
Greedy decoding captures one ``decode_step`` in a HIP graph and replays it per token.
"""
import ctypes
import time

import torch

import rptc_kernels as rk
from .linear import QuantizedLinear


class LlamaShape:
    def __init__(self, layers=32, d_model=4096, heads=32, d_ff=11008, vocab=32000, max_len=1024, rope_theta=10000.0):
        self.layers, self.d_model, self.heads, self.d_ff = layers, d_model, heads, d_ff
        self.vocab, self.max_len, self.rope_theta = vocab, max_len, rope_theta
        self.head_dim = d_model // heads


class QuantizedLlama(torch.nn.Module):
    EPS = 1e-5

    def __init__(self, shape, S=8, seed=42, device="cuda", quantize_init=False, init_std=0.02):
        """quantize_init=False: seeded random streams (decode cost does not depend on the data).
        quantize_init=True: every projection is a random-init dense weight (normal, ``init_std``: the
        initialisation of the reference's model class) put through the reference's procedure - row/column
        factorisation (quantize_hf.py:77-117), then the trellis search on the normalised matrix - and run
        with its four vectors applied inside the mat-vec kernels."""
        super().__init__()
        self.shape = shape
        g = torch.Generator(device=device)
        g.manual_seed(seed)
        d, f = shape.d_model, shape.d_ff
        self.embed = (torch.randn((shape.vocab, d), generator=g, device=device) * 0.02).half()
        self.lm_head = (torch.randn((shape.vocab, d), generator=g, device=device) * d ** -0.5).half()
        self.final_norm = torch.ones(d, dtype=torch.float16, device=device)
        self.blocks = torch.nn.ModuleList()
        codebook = None
        if quantize_init:
            # the normalised matrices have unit RMS: one unit-variance codebook serves every projection
            codebook = torch.randn(2 << S, generator=torch.Generator().manual_seed(seed)).to(torch.float16)
        for i in range(shape.layers):
            blk = torch.nn.Module()
            for j, (name, n_in, n_out) in enumerate((("qkv_proj", d, 3 * d), ("o_proj", d, d),
                                                     ("gate_up_proj", d, 2 * f), ("down_proj", f, d))):
                if quantize_init:
                    W = torch.randn((n_out, n_in), generator=g, device=device) * init_std
                    layer = QuantizedLinear.from_weight(W, codebook=codebook, S=S, device=device, factorize=True)
                    del W
                else:
                    layer = QuantizedLinear.from_random(n_in, n_out, S=S, seed=seed + 16 * i + j, device=device)
                setattr(blk, name, layer)
            blk.norm1 = torch.ones(d, dtype=torch.float16, device=device)
            blk.norm2 = torch.ones(d, dtype=torch.float16, device=device)
            self.blocks.append(blk)
        hd = shape.head_dim
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, hd, 2, device=device).float() / hd))
        ang = torch.arange(shape.max_len, device=device).float()[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().half().contiguous(), ang.sin().half().contiguous()    # [max_len, hd/2]
        self.k_cache = torch.zeros((shape.layers, shape.heads, shape.max_len, hd), dtype=torch.float16, device=device)
        self.v_cache = torch.zeros_like(self.k_cache)
        # work buffers of the one-token path
        z = lambda k: torch.zeros(k, dtype=torch.float16, device=device)
        self._x, self._x2, self._h, self._qkv, self._q, self._att = z(d), z(d), z(d), z(3 * d), z(d), z(d)
        self._o, self._gu, self._act, self._down = z(d), z(2 * f), z(f), z(d)

    # ---------------------------------------------------------------- torch path (any number of tokens)

    @classmethod
    def _rms(cls, x, w):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + cls.EPS)).half() * w

    def _rope(self, t, pos):
        # t [T, heads, hd]; pos [T] (long): rotate the (2i, 2i+1) pairs
        c, s = self.cos[pos][:, None, :], self.sin[pos][:, None, :]
        a, b = t[..., 0::2], t[..., 1::2]
        return torch.stack([a * c - b * s, a * s + b * c], dim=-1).flatten(-2)

    def forward_tokens(self, tokens, pos, all_logits=False):
        """tokens [T] long, pos [T] long (their positions, contiguous); writes the KV cache at pos and
        returns the logits of the last token ([1, vocab]), or of every token ([T, vocab]) with
        ``all_logits``.  Attention looks at cache positions <= the token's own."""
        sh = self.shape
        T, d, f = tokens.numel(), sh.d_model, sh.d_ff
        x = self.embed[tokens]                                                     # [T, d]
        key_pos = torch.arange(sh.max_len, device=x.device)
        mask = key_pos[None, :] <= pos[:, None]                                    # [T, max_len]
        for i, blk in enumerate(self.blocks):
            h = self._rms(x, blk.norm1)
            q, k, v = blk.qkv_proj(h).split(d, dim=-1)
            q = self._rope(q.reshape(T, sh.heads, sh.head_dim), pos)
            k = self._rope(k.reshape(T, sh.heads, sh.head_dim), pos)
            v = v.reshape(T, sh.heads, sh.head_dim)
            self.k_cache[i].index_copy_(1, pos, k.transpose(0, 1))
            self.v_cache[i].index_copy_(1, pos, v.transpose(0, 1))
            o = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), self.k_cache[i], self.v_cache[i],
                                                                 attn_mask=mask[None])      # [heads, T, hd]
            x = x + blk.o_proj(o.transpose(0, 1).reshape(T, d))
            h = self._rms(x, blk.norm2)
            g, u = blk.gate_up_proj(h).split(f, dim=-1)
            x = x + blk.down_proj(torch.nn.functional.silu(g) * u)
        h = self._rms(x if all_logits else x[-1:], self.final_norm)
        return (h @ self.lm_head.t()).float()                                      # [T or 1, vocab]

    # ---------------------------------------------------------------- fused one-token path

    def decode_step(self, token, pos, fuse=True, half_logits=False, input_ready=False, after_layer=None):
        """token [1] long, pos [1] long, both on the device (read by the kernels, so a captured graph can be
        replayed with new values).  Returns the logits [1, vocab] (float; fp16 as the lm_head product leaves
        them with ``half_logits``).  ``input_ready``: the token's embedding row is already in the decoder's
        input buffer (``rptc_greedy_next`` put it there), so it is not gathered again.

        The position must be below ``shape.max_len``: it lives on the device, so it is not checked here
        (``greedy_decode`` checks its whole range up front; the kernels skip a position outside the caches).

        ``after_layer``: called as ``after_layer(i)`` when layer i's launches have been queued (fused form only;
        not inside a graph capture): the work buffers then hold, once the stream has been waited for, what that
        layer's projections read and wrote (``_x2`` the residual stream it started from, ``_qkv``, ``_att``, ``_o``,
        ``_x`` the residual stream after attention, ``_gu``, ``_down``).

        ``fuse`` (default): five launches per layer - the qkv and gate/up projections do the residual add and
        RMS norm in their prologue, the down projection the SiLU gate, and one kernel rotates q and k, appends
        to the cache and attends.  ``fuse=False``: the same arithmetic as nine launches per layer."""
        sh = self.shape
        lib = rk.library()
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        d, f = sh.d_model, sh.d_ff

        def ok(rc):
            if rc:
                raise RuntimeError(lib.rptc_status_string(rc).decode())

        def affine(layer):
            # the four vectors of the reference's factorisation as pointers, or None when the layer has none
            vs = (layer.scales_in, layer.biases_in, layer.scales_out, layer.biases_out)
            if all(v is None for v in vs):
                return None
            return [None if v is None else v.data_ptr() for v in vs]

        def gemv(layer, x, out):
            aff = affine(layer)
            if aff is not None and layer.in_features > 16384:
                out.copy_(layer(x.unsqueeze(0))[0])        # too long for the fused form: framework ops around the plain call
                return
            if aff is not None:
                ok(lib.rptc_decompress_matvec_affine(layer.compressed.data_ptr(), layer.codebook.data_ptr(), x.data_ptr(), *aff,
                                                     out.data_ptr(), layer.out_features, layer.in_features, layer.S,
                                                     layer.carry_mode, stream, None))
                return
            fn = getattr(lib, f"rptc_decompress_matvec_16_{layer.S}_1")
            ok(fn(layer.compressed.data_ptr(), layer.codebook.data_ptr(), x.data_ptr(), out.data_ptr(),
                  layer.out_features, layer.in_features, layer.carry_mode, stream, None))

        def gemv_norm(layer, x_in, delta, weight, x_out, out):
            aff = affine(layer)
            if aff is not None:
                ok(lib.rptc_decompress_matvec_rmsnorm_affine(layer.compressed.data_ptr(), layer.codebook.data_ptr(),
                                                             x_in.data_ptr(), delta, weight.data_ptr(), x_out.data_ptr(), *aff,
                                                             out.data_ptr(), layer.out_features, layer.in_features, self.EPS,
                                                             layer.S, layer.carry_mode, stream, None))
                return
            ok(lib.rptc_decompress_matvec_rmsnorm(layer.compressed.data_ptr(), layer.codebook.data_ptr(), x_in.data_ptr(),
                                                  delta, weight.data_ptr(), x_out.data_ptr(), out.data_ptr(),
                                                  layer.out_features, layer.in_features, self.EPS, layer.S,
                                                  layer.carry_mode, stream, None))

        def gemv_silu(layer, gate_up, out):
            aff = affine(layer)
            if aff is not None and layer.in_features > 16384:
                ok(lib.rptc_silu_mul(gate_up.data_ptr(), self._act.data_ptr(), layer.in_features, stream))
                gemv(layer, self._act, out)
                return
            if aff is not None:
                ok(lib.rptc_decompress_matvec_silu_affine(layer.compressed.data_ptr(), layer.codebook.data_ptr(),
                                                          gate_up.data_ptr(), *aff, out.data_ptr(), layer.out_features,
                                                          layer.in_features, layer.S, layer.carry_mode, stream, None))
                return
            ok(lib.rptc_decompress_matvec_silu(layer.compressed.data_ptr(), layer.codebook.data_ptr(), gate_up.data_ptr(),
                                               out.data_ptr(), layer.out_features, layer.in_features, layer.S,
                                               layer.carry_mode, stream, None))

        if not input_ready:
            self._x.copy_(self.embed[token].reshape(-1))
        delta = None
        if fuse:
            xa, xb = self._x, self._x2          # the residual stream alternates between two buffers
            for i, blk in enumerate(self.blocks):
                gemv_norm(blk.qkv_proj, xa, delta, blk.norm1, xb, self._qkv)
                ok(lib.rptc_rope_attn_decode(self._qkv.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(), pos.data_ptr(),
                                             self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr(), self._att.data_ptr(),
                                             sh.heads, sh.head_dim, sh.max_len, stream))
                gemv(blk.o_proj, self._att, self._o)
                gemv_norm(blk.gate_up_proj, xb, self._o.data_ptr(), blk.norm2, xa, self._gu)
                gemv_silu(blk.down_proj, self._gu, self._down)
                delta = self._down.data_ptr()
                if after_layer is not None:
                    after_layer(i)
            ok(lib.rptc_add_rmsnorm(xa.data_ptr(), delta, self.final_norm.data_ptr(), xb.data_ptr(), self._h.data_ptr(), d,
                                    self.EPS, stream))
            logits = self._h.unsqueeze(0) @ self.lm_head.t()
            return logits if half_logits else logits.float()
        for i, blk in enumerate(self.blocks):
            ok(lib.rptc_add_rmsnorm(self._x.data_ptr(), delta, blk.norm1.data_ptr(), self._x.data_ptr(),
                                    self._h.data_ptr(), d, self.EPS, stream))
            gemv(blk.qkv_proj, self._h, self._qkv)
            ok(lib.rptc_rope_cache(self._qkv.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(), pos.data_ptr(),
                                   self._q.data_ptr(), self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr(),
                                   sh.heads, sh.head_dim, sh.max_len, stream))
            ok(lib.rptc_attn_decode(self._q.data_ptr(), self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr(),
                                    pos.data_ptr(), self._att.data_ptr(), sh.heads, sh.head_dim, sh.max_len, stream))
            gemv(blk.o_proj, self._att, self._o)
            ok(lib.rptc_add_rmsnorm(self._x.data_ptr(), self._o.data_ptr(), blk.norm2.data_ptr(), self._x.data_ptr(),
                                    self._h.data_ptr(), d, self.EPS, stream))
            gemv(blk.gate_up_proj, self._h, self._gu)
            ok(lib.rptc_silu_mul(self._gu.data_ptr(), self._act.data_ptr(), f, stream))
            gemv(blk.down_proj, self._act, self._down)
            delta = self._down.data_ptr()
        ok(lib.rptc_add_rmsnorm(self._x.data_ptr(), delta, self.final_norm.data_ptr(), self._x.data_ptr(),
                                self._h.data_ptr(), d, self.EPS, stream))
        logits = self._h.unsqueeze(0) @ self.lm_head.t()
        return logits if half_logits else logits.float()


def check_context(shape, prompt_len, new_tokens):
    """The caches and the rotary tables hold ``shape.max_len`` positions; the last token generated is never fed
    back, so positions 0 .. prompt_len + new_tokens - 2 are written.  Raises ValueError when they do not fit
    (the kernels themselves skip a position outside the caches rather than write out of bounds)."""
    if prompt_len < 1 or new_tokens < 1:
        raise ValueError("the prompt and the number of new tokens must be at least 1")
    if prompt_len + new_tokens - 1 > shape.max_len:
        raise ValueError(f"prompt of {prompt_len} tokens + {new_tokens} new tokens needs {prompt_len + new_tokens - 1} "
                         f"cache positions, the model was built with max_len = {shape.max_len}")


def greedy_decode(model, prompt, new_tokens, mode="fused_graph"):
    """Prefill the prompt (in chunks of 32 tokens: the batch the fused mat-mat kernel takes), then decode
    ``new_tokens`` greedily one at a time.  mode: "fused_graph" (five launches per layer, one HIP graph per
    token), "fused" (the same, direct launches), "glue_graph" / "glue" (nine launches per layer: the
    element-wise steps as kernels of their own), "torch_graph" / "torch" (framework ops between the projections).
    Returns (token list, seconds spent in the decode loop)."""
    dev = model.embed.device
    prompt = torch.as_tensor(prompt, dtype=torch.long, device=dev)
    P = prompt.numel()
    check_context(model.shape, P, new_tokens)
    if mode.startswith("fused"):
        step = model.decode_step
    elif mode.startswith("glue"):
        step = lambda t, p: model.decode_step(t, p, fuse=False)
    else:
        step = model.forward_tokens
    with torch.no_grad():
        logits = None
        for p0 in range(0, P, 32):
            chunk = prompt[p0:p0 + 32]
            logits = model.forward_tokens(chunk, torch.arange(p0, p0 + chunk.numel(), device=dev))
        tok = logits.argmax(-1)                                                    # [1]
        out = [tok.clone()]
        s_tok = tok.clone()
        s_pos = torch.tensor([P], dtype=torch.long, device=dev)
        graph = None
        if mode.endswith("graph"):
            # warm up on a side stream, then capture one step with static token/position tensors
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step(s_tok, s_pos)
            torch.cuda.current_stream().wait_stream(side)
            # the token hand-over is part of the graph: the new token becomes the next input, is appended
            # to the output buffer, and position and output index move on, so a token is one replay
            s_idx = torch.zeros(1, dtype=torch.long, device=dev)
            s_out = torch.zeros(max(new_tokens - 1, 1), dtype=torch.long, device=dev)
            graph = torch.cuda.CUDAGraph()
            if mode.startswith("fused"):
                # the hand-over is one kernel of the library: arg-max, output list, next embedding row, counters
                lib = rk.library()
                model._x.copy_(model.embed[s_tok].reshape(-1))
                with torch.cuda.graph(graph):
                    logits16 = model.decode_step(s_tok, s_pos, half_logits=True, input_ready=True)
                    rc = lib.rptc_greedy_next(logits16.data_ptr(), model.shape.vocab, model.embed.data_ptr(), model.shape.d_model,
                                              s_tok.data_ptr(), s_out.data_ptr(), s_idx.data_ptr(), s_pos.data_ptr(),
                                              model._x.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
                    if rc:
                        raise RuntimeError(lib.rptc_status_string(rc).decode())
            else:
                with torch.cuda.graph(graph):
                    s_next = step(s_tok, s_pos).argmax(-1)
                    s_out.index_copy_(0, s_idx, s_next)
                    s_tok.copy_(s_next)
                    s_pos.add_(1)
                    s_idx.add_(1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if graph is not None:
            for _ in range(new_tokens - 1):
                graph.replay()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            return [int(out[0])] + [int(t) for t in s_out[:new_tokens - 1]], dt
        for _ in range(new_tokens - 1):
            nxt = step(s_tok, s_pos).argmax(-1)
            s_tok.copy_(nxt)
            s_pos.add_(1)
            out.append(nxt.clone())
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    return [int(t) for t in out], dt

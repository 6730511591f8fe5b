"""QuantizedLinear: a linear layer whose weight lives as a packed trellis stream.

The reference never builds such a module: ``quantize_hf.py:215`` writes the de-quantized matrix
back into a dense ``nn.Linear`` (``module.weight.copy_(recon)``).  This module keeps the stream and
runs the fused kernels instead.  It follows the reference's reconstruction formula
(``quantize_hf.py:167``)

    W = b_out + b_in + s_out * s_in * W_hat            (b_out, s_out per row; b_in, s_in per column)

so  y = s_out * (W_hat (s_in * x)) + b_out * sum(x) + (b_in . x),  with W_hat the matrix the stream
decodes to, and its list of quantized modules (``quantize_hf.py:189``).
"""
import re

import torch

import rptc_kernels as rk

# the modules quantize_hf.py:189 quantizes
REFERENCE_PATTERN = r"model\.layers\.(\d+)\.(self_attn\.(\w+)_proj|mlp\.(\w+)_proj)"


class QuantizedLinear(torch.nn.Module):
    """y = W x with W held as a hashed-pair trellis stream (2 bits/weight, the reference's format, or 3 or
    4) plus the optional row/column scales and biases of the reference's factorisation and an optional
    sign-Hadamard transform of the input."""

    def __init__(self, in_features, out_features, S=8, carry_mode=rk.CONTINUOUS, device="cuda", bits=2):
        super().__init__()
        if in_features % 64 != 0:
            raise ValueError("in_features must be a multiple of 64 (whole stream elements per row)")
        if S not in (6, 8):
            raise ValueError("S must be 6 or 8")
        if bits not in (2, 3, 4):
            raise ValueError("bits must be 2, 3 or 4")
        self.in_features, self.out_features, self.S, self.carry_mode = in_features, out_features, S, carry_mode
        self.bits = bits
        words = out_features * in_features * bits // 32
        self.register_buffer("compressed", torch.zeros(words, dtype=torch.int32, device=device))
        self.register_buffer("codebook", torch.zeros(2 << S, dtype=torch.float16, device=device))
        # Optional vectors: registered as None, so ``state_dict`` only holds the ones that are set, and
        # ``load_state_dict`` into a fresh layer restores them only if the layer first gets buffers of the right
        # shape (``set_affine`` / ``set_signs`` with placeholders); ``from_*`` constructors are the usual way.
        for name in ("scales_out", "scales_in", "biases_out", "biases_in", "signs"):
            self.register_buffer(name, None)

    # ---------------------------------------------------------------- construction

    @classmethod
    def from_random(cls, in_features, out_features, S=8, seed=42, weight_std=None, device="cuda", **kw):
        """Seeded random stream and codebook: decode cost does not depend on the data, so this is
        what the synthetic benchmarks use.  The codebook is scaled so that W has std weight_std
        (default 1/sqrt(in_features))."""
        layer = cls(in_features, out_features, S=S, device=device, **kw)
        g = torch.Generator(device=device)
        g.manual_seed(seed)
        layer.compressed.copy_(torch.randint(-(1 << 31), 1 << 31, layer.compressed.shape, generator=g,
                                             dtype=torch.int64, device=device).to(torch.int32))
        std = weight_std if weight_std is not None else in_features ** -0.5
        layer.codebook.copy_((torch.randn(2 << S, generator=g, device=device) * std).to(torch.float16))
        return layer

    @classmethod
    def from_symbols(cls, symbols, codebook, out_features, S=8, device="cuda", **kw):
        """symbols: trellis symbols of 2*bits bits [out_features, in_features/2] in stream order (numpy or tensor)."""
        from rptc_kernels import packing
        import numpy as np
        sym = symbols.cpu().numpy() if isinstance(symbols, torch.Tensor) else np.asarray(symbols)
        layer = cls(2 * sym.shape[1], out_features, S=S, device=device, **kw)
        layer.compressed.copy_(torch.from_numpy(packing.pack_matvec(sym, bits=layer.bits)).to(device))
        layer.codebook.copy_(torch.as_tensor(codebook, dtype=torch.float16).to(device))
        return layer

    @classmethod
    def from_weight(cls, weight, codebook=None, S=8, importance=None, seed=42, device="cuda", bits=2, signs=None,
                    factorize=False):
        """Quantize a dense weight [out, in] with the Viterbi search of ``rptc_kernels.quantize`` (run on
        ``device``) and pack the result.  codebook: fp16 [2^(S+1)] or None for a seeded Gaussian one
        scaled to the weight's standard deviation.  signs: +-1 per input feature; the layer then stores
        the weight in the sign-Hadamard basis (outliers spread over a block) and transforms its input.
        factorize: take the reference's row/column scales and biases out first (quantize_hf.py:77-117), search
        on the normalised matrix with column i weighted by importance_i * s_in_i^2 (the reference hands
        diag(H) * s_in to a search that squares it, quantize_hf.py:139 and rptc.py:32; here ``importance`` is
        the loss weight itself) and keep the four vectors on the layer (``set_affine``)."""
        from rptc_kernels import quantize
        W = torch.as_tensor(weight).to(device=device, dtype=torch.float32)
        if factorize:
            if signs is not None:
                raise ValueError("factorize and signs are two ways to condition a weight: use one")
            b_out, b_in, s_out, s_in, N = quantize.factorize(W)
            imp = None
            if importance is not None:
                imp = torch.as_tensor(importance, dtype=torch.float32, device=device).reshape(-1) * s_in.reshape(-1) ** 2
            layer = cls.from_weight(N, codebook=codebook, S=S, importance=imp, seed=seed, device=device, bits=bits)
            return layer.set_affine(s_out.reshape(-1), s_in.reshape(-1), b_out.reshape(-1), b_in.reshape(-1))
        if signs is not None:
            W = quantize.sign_hadamard_rows(W, signs)
        if codebook is None:
            g = torch.Generator().manual_seed(seed)
            codebook = (torch.randn(2 << S, generator=g) * W.std().item()).to(torch.float16)
        codebook = torch.as_tensor(codebook, dtype=torch.float16)
        symbols, mse = quantize.quantize_matrix(W, codebook.to(device), S, importance=importance, bits=bits)
        layer = cls.from_symbols(symbols, codebook, W.size(0), S=S, device=device, bits=bits)
        layer.quantization_mse = mse
        if signs is not None:
            layer.set_signs(signs)
        return layer

    def set_affine(self, scales_out=None, scales_in=None, biases_out=None, biases_in=None):
        """The reference's row/column factorisation (quantize_hf.py:77-117,167); any may be None."""
        def prep(v, n):
            if v is None:
                return None
            v = torch.as_tensor(v, dtype=torch.float16, device=self.compressed.device).reshape(-1).contiguous()
            if v.numel() != n:
                raise ValueError("wrong length")
            return v
        self.scales_out = prep(scales_out, self.out_features)
        self.biases_out = prep(biases_out, self.out_features)
        self.scales_in = prep(scales_in, self.in_features)
        self.biases_in = prep(biases_in, self.in_features)
        return self

    def set_signs(self, signs):
        """+-1 per input feature: the input goes through the sign-Hadamard transform first, i.e. the
        stream encodes W_hat in the transformed basis."""
        self.signs = None if signs is None else torch.as_tensor(
            signs, dtype=torch.float16, device=self.compressed.device).reshape(-1).contiguous()
        return self

    # ---------------------------------------------------------------- forward

    def _product(self, x2):
        """x2 fp16 [batch, n] contiguous -> fp16 [batch, m] = W_hat x, through the fused kernels."""
        batch = x2.size(0)
        out = torch.empty((batch, self.out_features), dtype=torch.float16, device=x2.device)
        lib = rk.library()
        if batch == 1:
            rk._call(lib.rptc_decompress_matvec_bits, (self.compressed, self.codebook, x2, out), self.out_features,
                     self.in_features, self.S, self.bits, carry_mode=self.carry_mode, timed=False)
            return out
        for b0 in range(0, batch, 32):
            xb = x2[b0:b0 + 32]
            ob = out[b0:b0 + 32]
            rk._call(lib.rptc_decompress_matmul_bits, (self.compressed, self.codebook, xb, ob), self.out_features,
                     self.in_features, xb.size(0), self.S, self.bits, carry_mode=self.carry_mode, timed=False)
        return out

    def forward(self, x):
        if x.dtype != torch.float16 or not x.is_cuda:
            raise RuntimeError("QuantizedLinear runs on fp16 CUDA tensors only (there is no CPU path)")
        shape = x.shape
        x2 = x.reshape(-1, self.in_features).contiguous()
        affine = (self.scales_in, self.biases_in, self.scales_out, self.biases_out)
        if (x2.size(0) == 1 and self.bits == 2 and self.signs is None and self.in_features <= 16384
                and self.out_features <= 1024 * torch.cuda.get_device_properties(x2.device).multi_processor_count
                and any(v is not None for v in affine)):
            # one token: scales and biases are applied inside the mat-vec
            y = torch.empty((1, self.out_features), dtype=torch.float16, device=x2.device)
            rk.decompress_matvec_affine(self.compressed, self.codebook, x2[0], y[0], *affine, carry_mode=self.carry_mode,
                                        timed=False)
            return y.reshape(shape[:-1] + (self.out_features,))
        xs = x2 * self.scales_in if self.scales_in is not None else x2
        if self.signs is not None and xs.size(0) == 1 and self.bits == 2 and self.in_features <= 15360:
            # one token: the transform runs in the prologue of the mat-vec
            y = torch.empty((1, self.out_features), dtype=torch.float16, device=xs.device)
            rk._call(rk.library().rptc_decompress_matvec_hadamard, (self.compressed, self.codebook, xs, self.signs, y),
                     self.out_features, self.in_features, 0, self.S, carry_mode=self.carry_mode, timed=False)
            return self._epilogue(y, x2, shape)
        if self.signs is not None:
            t = torch.empty_like(xs)
            rk.sign_hadamard(xs, self.signs, t, timed=False)
            xs = t
        y = self._product(xs)
        return self._epilogue(y, x2, shape)

    def _epilogue(self, y, x2, shape):
        if self.scales_out is not None:
            y = y * self.scales_out
        if self.biases_out is not None:
            y = y + self.biases_out * x2.float().sum(dim=1, keepdim=True).to(torch.float16)
        if self.biases_in is not None:
            y = y + (x2.float() @ self.biases_in.float()).to(torch.float16).unsqueeze(1)
        return y.reshape(shape[:-1] + (self.out_features,))

    # ---------------------------------------------------------------- inspection

    def decoded_weight(self):
        """W_hat, fp16 [m, n], bit-exact decode of the stream."""
        W = torch.empty((self.out_features, self.in_features), dtype=torch.float16, device=self.compressed.device)
        rk._call(rk.library().rptc_matvec_bits_dense, (self.compressed, self.codebook, W), self.out_features,
                 self.in_features, self.S, self.bits, carry_mode=self.carry_mode, timed=False)
        return W

    def reconstructed_weight(self):
        """The dense matrix this layer multiplies by, float32 [m, n]: b_out + b_in + s_out * s_in * W_hat
        (quantize_hf.py:167) with the vectors that are set; without signs."""
        if self.signs is not None:
            raise RuntimeError("a layer with a sign-Hadamard transform has no dense matrix in the input's own basis here")
        W = self.decoded_weight().float()
        if self.scales_in is not None:
            W = W * self.scales_in.float()[None, :]
        if self.scales_out is not None:
            W = W * self.scales_out.float()[:, None]
        if self.biases_out is not None:
            W = W + self.biases_out.float()[:, None]
        if self.biases_in is not None:
            W = W + self.biases_in.float()[None, :]
        return W

    def compressed_bytes(self):
        return self.compressed.numel() * 4

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, S={self.S}, bits_per_weight={self.bits}"


def patch_model(model, pattern=REFERENCE_PATTERN, S=8, seed=42, make_layer=None):
    """Replace every ``nn.Linear`` whose qualified name matches ``pattern`` (default: the modules
    quantize_hf.py:189 quantizes) by a QuantizedLinear.  ``make_layer(name, linear)`` may build the
    replacement; by default a seeded random stream of the same shape is used (synthetic weights).
    Returns the list of replaced names."""
    rx = re.compile(pattern)
    replaced = []
    for i, (name, module) in enumerate(list(model.named_modules())):
        if not isinstance(module, torch.nn.Linear) or re.fullmatch(rx, name) is None:
            continue
        if make_layer is not None:
            new = make_layer(name, module)
        else:
            new = QuantizedLinear.from_random(module.in_features, module.out_features, S=S, seed=seed + i,
                                              device=module.weight.device)
        parent = model
        parts = name.split(".")
        for p in parts[:-1]:
            parent = getattr(parent, p)
        setattr(parent, parts[-1], new)
        replaced.append(name)
    return replaced

"""Viterbi trellis quantizer for the hashed pair stream (torch, runs on CPU or GPU).

Semantics follow the reference's quantizer (rptc.py:13-71, diag_only path): the trellis starts in
state 0 (``rho[0] = 0``, rptc.py:55-56), a step shifts new symbol bits into the state
(rptc.py:77-79), the path cost is the sum of per-step squared errors, and the best final state is
traced back (rptc.py:60-65).  What differs is the decoder the path is optimised for: the one the
inference kernels implement (inference.cu:250-262) — a 16-bit state, 4 bits per step, two weights
per step looked up through ``hash = s*(s+1)`` — so that the symbols can be packed
(``packing.pack_matvec``) and run by ``decompress_matvec_*`` in CONTINUOUS mode.  The reference
itself never connects its quantizer to its kernels.

The search is exact (full Viterbi over all 65 536 states); ties are broken by ``torch.min``'s first
index, which need not match ``jnp.argmin`` of the reference bit for bit.
"""
import torch

from . import packing

STATE_BITS = 16
STEP_BITS = 4


def decode_table(codebook, S):
    """[65536, 2] float32: the weight pair state s decodes to (inference.cu:250-262)."""
    cb = torch.as_tensor(codebook).to(torch.float32).reshape(-1)
    assert cb.numel() == 2 << S
    s = torch.arange(1 << STATE_BITS, dtype=torch.int64, device=cb.device)
    prod = s * (s + 1)
    e = (prod >> 8) & ((1 << S) - 1)
    sign = ((prod >> 15) & 1).to(torch.float32)
    w0 = cb[2 * e].abs() * (1.0 - 2.0 * sign)      # the hash bit replaces the sign of the first value
    w1 = cb[2 * e + 1]
    return torch.stack([w0, w1], dim=1)


def viterbi_pairs(targets, table, weights=None, state_bits=STATE_BITS, step_bits=STEP_BITS):
    """Exact trellis search.  targets [rows, steps, 2] float; table [2^state_bits, 2]; weights None or
    [rows, steps, 2] (per-weight importance, the diagonal of rptc.py's ``corrections``).
    Returns (symbols int64 [rows, steps], cost float [rows])."""
    rows, steps, _ = targets.shape
    M, R = 1 << state_bits, 1 << step_bits
    dev = targets.device
    table = table.to(dev)
    rho = torch.full((rows, M), float("inf"), device=dev)
    rho[:, 0] = 0.0
    back = torch.empty((steps, rows, M >> step_bits), dtype=torch.uint8, device=dev)
    t0, t1 = table[:, 0].unsqueeze(0), table[:, 1].unsqueeze(0)
    for t in range(steps):
        # state s' = ((s << step_bits) | sym) & (M-1): its predecessors share the low bits s' >> step_bits
        best, arg = rho.view(rows, R, M >> step_bits).min(dim=1)
        back[t] = arg.to(torch.uint8)
        d0 = targets[:, t, 0:1] - t0
        d1 = targets[:, t, 1:2] - t1
        if weights is None:
            loss = d0 * d0 + d1 * d1
        else:
            loss = weights[:, t, 0:1] * (d0 * d0) + weights[:, t, 1:2] * (d1 * d1)     # rptc.py:32: c * (x - a)**2
        rho = best.repeat_interleave(R, dim=1) + loss
    cost, state = rho.min(dim=1)
    symbols = torch.empty((rows, steps), dtype=torch.int64, device=dev)
    r = torch.arange(rows, device=dev)
    for t in range(steps - 1, -1, -1):
        symbols[:, t] = state & (R - 1)
        low = state >> step_bits
        top = back[t, r, low].to(torch.int64)
        state = (top << (state_bits - step_bits)) | low
    return symbols, cost


def viterbi_scalar(targets, alphabet, weights=None):
    """The reference's search as it stands (rptc.py:13-71, diag_only): 2 bits a step, state s emits alphabet[s].
    targets [rows, steps] float; alphabet [2^L]; weights None or [rows, steps].  Returns (symbols int64
    [rows, steps], cost float [rows])."""
    alphabet = alphabet.to(torch.float32).reshape(-1)
    L = alphabet.numel().bit_length() - 1
    w = None if weights is None else torch.stack([weights, torch.zeros_like(weights)], dim=2)
    table = torch.stack([alphabet, torch.zeros_like(alphabet)], dim=1)       # second value: always 0 error
    tg = torch.stack([targets, torch.zeros_like(targets)], dim=2)
    return viterbi_pairs(tg, table, w, state_bits=L, step_bits=2)


def quantize_matrix_scalar(W, alphabet, importance=None, rows_per_batch=None):
    """Quantize W [m, n] to 2-bit symbols [m, n] for the scalar-LUT streams (``packing.pack_rowmajor`` ->
    ``decompress``, ``packing.pack_transposed`` -> ``decompress_matvec_t_*``, CONTINUOUS mode): the reference's
    quantizer (rptc.py:13-71) row by row.  alphabet: [2^16] or [2^14]; importance: optional [n] per-column weight.
    Returns (symbols int64 [m, n] on the CPU, mse float).  A matrix on the GPU is searched by the HIP kernel
    (``rptc_kernels.viterbi_scalar``)."""
    W = torch.as_tensor(W)
    m, n = W.shape
    dev = W.device
    Wf = W.to(torch.float32).contiguous()
    imp = None if importance is None else torch.as_tensor(importance, dtype=torch.float32, device=dev).contiguous()
    out = torch.empty((m, n), dtype=torch.int64)
    total = 0.0
    if W.is_cuda:
        import rptc_kernels as rk
        ab16 = torch.as_tensor(alphabet).to(dev).to(torch.float16).contiguous()
        rows_per_batch = rows_per_batch or max(1, min(m, (1 << 30) // (4096 * n)))
    else:
        rows_per_batch = rows_per_batch or 16
    for r0 in range(0, m, rows_per_batch):
        tg = Wf[r0:r0 + rows_per_batch]
        if W.is_cuda:
            sym, cost, _, _ = rk.viterbi_scalar(tg, ab16, imp)
        else:
            sym, cost = viterbi_scalar(tg, torch.as_tensor(alphabet), None if imp is None else imp.expand(tg.size(0), -1))
        out[r0:r0 + rows_per_batch] = sym.cpu()
        total += cost.sum().item()
    return out, total / (m * n)


def quantize_matrix(W, codebook, S=8, importance=None, rows_per_batch=64, bits=2):
    """Quantize W [m, n] (n % 64 == 0) to symbols of 2*bits bits [m, n/2] in stream order, for the decoder
    of ``decompress_matvec_*`` (bits == 2) or ``decompress_matvec_bits`` in CONTINUOUS mode.  importance:
    optional [n] per-column weight (e.g. the Hessian diagonal, quantize_hf.py:164).  Returns (symbols int64
    [m, n/2] on the CPU, mse float).  A matrix on the GPU is searched by the HIP kernel
    (``rptc_kernels.viterbi_pairs``), which chooses the same path as ``viterbi_pairs`` here bit for bit."""
    W = torch.as_tensor(W)
    m, n = W.shape
    dev = W.device
    table = decode_table(torch.as_tensor(codebook).to(dev), S)
    cols = torch.from_numpy(packing.matvec_stream_columns(n)).to(dev)     # first column of every step
    Wf = W.to(torch.float32)
    targets = torch.stack([Wf[:, cols], Wf[:, cols + 1]], dim=2)          # [m, n/2, 2] in stream order
    wts = None
    if importance is not None:
        imp = torch.as_tensor(importance, dtype=torch.float32, device=dev)
        wts = torch.stack([imp[cols], imp[cols + 1]], dim=1).unsqueeze(0)
    out = torch.empty((m, n // 2), dtype=torch.int64)
    total = 0.0
    on_gpu = W.is_cuda
    if on_gpu:
        # the search kernel: one workgroup per row, 2048 bytes of back pointers per row and step
        import rptc_kernels as rk
        cb16 = torch.as_tensor(codebook).to(dev).to(torch.float16).contiguous()
        shared = None if wts is None else wts[0].contiguous()
        rows_per_batch = max(1, min(m, (1 << 30) // (1024 * n)))
    for r0 in range(0, m, rows_per_batch):
        tg = targets[r0:r0 + rows_per_batch]
        if on_gpu:
            sym, cost, _, _ = rk.viterbi_pairs(tg.contiguous(), cb16, shared, bits=bits)
        else:
            w = None if wts is None else wts.expand(tg.size(0), -1, -1)
            sym, cost = viterbi_pairs(tg, table, w, step_bits=2 * bits)
        out[r0:r0 + rows_per_batch] = sym.cpu()
        total += cost.sum().item()
    return out, total / (m * n)


def dequantize_symbols(symbols, codebook, S=8, bits=2):
    """The dense matrix [m, n] a symbol array (stream order) decodes to, by walking the shift register
    (rptc.py:74-85 with 4-bit steps and the hashed pair lookup): the definition the kernels are held to."""
    symbols = torch.as_tensor(symbols, dtype=torch.int64)
    m, half = symbols.shape
    n = 2 * half
    table = decode_table(torch.as_tensor(codebook), S)
    cols = torch.from_numpy(packing.matvec_stream_columns(n))
    state = torch.zeros(m, dtype=torch.int64)
    W = torch.empty((m, n), dtype=torch.float32)
    for p in range(half):
        state = ((state << (2 * bits)) | symbols[:, p]) & ((1 << STATE_BITS) - 1)
        W[:, cols[p]] = table[state, 0]
        W[:, cols[p] + 1] = table[state, 1]
    return W


def factorize(W, iterations=64):
    """Row/column conditioning of a weight in front of the search: W = b_out + b_in + s_out * s_in * N with N close to
    zero mean and unit RMS along every row and every column (the model the reference's quantizer fits,
    quantize_hf.py:77-117, and reconstructs with at quantize_hf.py:167).

    It is a fixed point of four conditions, imposed in turn (``iterations`` rounds, as many as the reference runs):
      * every row of (W - b_out - b_in) / s_in sums to zero        -> b_out is the 1/s_in-weighted row mean of W - b_in
      * every column of (W - b_out - b_in) / s_out sums to zero    -> b_in likewise, over rows, with weights 1/s_out
      * every row of (W - b_out - b_in) / s_in has mean square s_out^2, every column of (W - b_out - b_in) / s_out
        has mean square s_in^2
    and two gauges that the model leaves free: a constant can move between b_out and b_in (fixed by giving them equal
    means) and a factor between s_out and s_in (fixed by giving them equal geometric means).
    W float [out, in] on any device.  Returns (b_out [out, 1], b_in [1, in], s_out [out, 1], s_in [1, in], N [out, in])."""
    W = torch.as_tensor(W).to(torch.float32)
    rows, cols = W.shape
    bias = [W.new_zeros((rows, 1)), W.new_zeros((1, cols))]          # [per row, per column]
    scale = [W.new_ones((rows, 1)), W.new_ones((1, cols))]

    def weighted_mean(A, w, dim):
        # sum(A * w) / sum(w) along dim, w broadcast along the other axis
        return (A * w).mean(dim=dim, keepdim=True) / w.mean()

    def root_mean_square(A, dim):
        return A.square().mean(dim=dim, keepdim=True).sqrt()

    for _ in range(iterations):
        # biases: rows against the current column side, then columns against the new rows; then the gauge
        bias[0] = weighted_mean(W - bias[1], 1 / scale[1], dim=1)
        bias[1] = weighted_mean(W - bias[0], 1 / scale[0], dim=0)
        shift = (bias[1].mean() - bias[0].mean()) / 2
        bias[0], bias[1] = bias[0] + shift, bias[1] - shift
        # scales on the residual of the new biases, rows first; then the gauge
        R = W - bias[0] - bias[1]
        scale[0] = root_mean_square(R / scale[1], dim=1)
        scale[1] = root_mean_square(R / scale[0], dim=0)
        ratio = torch.exp((scale[1].log().mean() - scale[0].log().mean()) / 2)
        scale[0], scale[1] = scale[0] * ratio, scale[1] / ratio
    N = (W - bias[0] - bias[1]) / scale[0] / scale[1]
    return bias[0], bias[1], scale[0], scale[1], N


def quantile_alphabet(values, L=16, seed=0):
    """The reference's per-bank alphabet (quantize_hf.py:137-141): 2^L values read off the sorted sample at the
    mid-point quantiles (linear interpolation), then shuffled.  The shuffle is seeded with torch, not with
    jax.random.permutation."""
    fp = torch.sort(values.reshape(-1).to(torch.float32)).values
    M, K = 1 << L, fp.numel()
    x = (2 * torch.arange(M, dtype=torch.float64, device=fp.device) + 1) / 2 / M
    pos = (x * K - 0.5).clamp(0, K - 1)                 # xp[k] = (2k + 1) / 2K  ->  k = x K - 1/2
    lo = pos.floor().long()
    hi = (lo + 1).clamp(max=K - 1)
    frac = (pos - lo.to(torch.float64)).to(torch.float32)
    alphabet = fp[lo] * (1 - frac) + fp[hi] * frac
    g = torch.Generator().manual_seed(seed)
    return alphabet[torch.randperm(M, generator=g).to(fp.device)]


def quantize_layer(W, hessian_diag=None, L=16, banks=32, seed=0):
    """quantize_hf.py:120-170 for one layer: factorise, weigh column i by (H_ii * s_in_i)^2 (the reference
    passes diag(H) * s_in as ``corrections`` and the search squares it, rptc.py:32), cut the rows into
    ``banks`` groups with one shuffled quantile alphabet each, search every row on the scalar trellis
    (``viterbi_scalar``: the HIP kernel for a matrix on the GPU), and put the layer back together.
    Returns a dict with the reconstruction ``recon`` [out, in], the 2-bit ``symbols`` [out, in], the
    ``alphabets`` [banks, 2^L] (fp16 values as float32) and the factors; out % banks == 0."""
    W = torch.as_tensor(W).to(torch.float32)
    out_features, in_features = W.shape
    if out_features % banks != 0:
        raise ValueError("the row count must be a multiple of the number of banks")
    b_out, b_in, s_out, s_in, N = factorize(W)
    imp = None
    if hessian_diag is not None:
        h = torch.as_tensor(hessian_diag, dtype=torch.float32, device=W.device).reshape(-1)
        imp = (h * s_in.reshape(-1)) ** 2
    rows_per_bank = out_features // banks
    symbols = torch.empty((out_features, in_features), dtype=torch.int64)
    rounded = torch.empty_like(N)
    alphabets = []
    for b in range(banks):
        rows = slice(b * rows_per_bank, (b + 1) * rows_per_bank)
        alphabet = quantile_alphabet(N[rows], L, seed + b).to(torch.float16)      # the kernels' table is fp16
        sym, _ = quantize_matrix_scalar(N[rows], alphabet, importance=imp)
        symbols[rows] = sym
        state = torch.zeros(rows_per_bank, dtype=torch.int64)
        af = alphabet.to(torch.float32).cpu()
        vals = torch.empty((rows_per_bank, in_features), dtype=torch.float32)
        for t in range(in_features):                                              # rptc.py:74-85
            state = ((state << 2) | sym[:, t]) & ((1 << L) - 1)
            vals[:, t] = af[state]
        rounded[rows] = vals.to(W.device)
        alphabets.append(af)
    recon = b_out + b_in + s_out * s_in * rounded
    return {"recon": recon, "symbols": symbols, "alphabets": torch.stack(alphabets), "biases_out": b_out, "biases_in": b_in,
            "scales_out": s_out, "scales_in": s_in, "normalized": N}


def evaluate_layer(W, recon, hessian_diag=None):
    """Errors of a reconstruction as the reference reports them (quantize_hf.py:172-185): ``frob`` =
    sum(E^2) / sqrt(sum(W^2)) (the reference divides the squared error by the NORM of W, not by its square,
    so the figure scales with ||W||), and ``proxy_diag`` = sum(E^2 h) / sum(W^2 h) with h the Hessian
    diagonal when one is given.  ``frob_rel`` = sum(E^2) / sum(W^2) is this library's addition (scale-free)."""
    W = torch.as_tensor(W).to(torch.float32)
    E = W - recon.to(W.device)
    res = {"frob": float((E ** 2).sum() / (W ** 2).sum().sqrt()), "frob_rel": float((E ** 2).sum() / (W ** 2).sum())}
    if hessian_diag is not None:
        h = torch.as_tensor(hessian_diag, dtype=torch.float32, device=W.device).reshape(1, -1)
        res["proxy_diag"] = float(((E * h) * E).sum() / ((W * h) * W).sum())
    return res


def sign_hadamard_rows(W, signs, block=0):
    """Every row of W [m, n] through the forward sign-Hadamard transform of ``rptc_kernels.sign_hadamard``
    (y = H_P (signs * x) / sqrt(P) per block of P columns; block 0: the largest power of two dividing n), in
    float32.  With T that (orthogonal) map, W x = (W T^t)(T x) and row r of W T^t is T applied to row r of W:
    the weights a layer stores when its input goes through the transform first."""
    W = torch.as_tensor(W).to(torch.float32)
    m, n = W.shape
    P = block
    if P == 0:
        P = 1
        while n % (2 * P) == 0 and 2 * P <= 32768:
            P *= 2
    if P < 2 or P & (P - 1) or n % P:
        raise ValueError("block must be a power of two dividing n")
    y = (W * torch.as_tensor(signs).to(W.device, torch.float32).reshape(1, n)).reshape(m, n // P, P)
    h = 1
    while h < P:                                         # Sylvester order: butterflies over strides 1, 2, 4, ...
        y = y.reshape(m, n // P, P // (2 * h), 2, h)
        a, b = y[:, :, :, 0, :], y[:, :, :, 1, :]
        y = torch.stack([a + b, a - b], dim=3)
        h *= 2
    return (y.reshape(m, n) / P ** 0.5)

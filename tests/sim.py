"""Slow, independent Python restatements used only to pin the C oracle on tiny inputs.

Two styles are used on purpose:
* bit-string brute force (the textbook sliding window over the row's bits), which shares no
  arithmetic with the oracle's shift/mask code;
* thread-level simulations of the CUDA kernels (32-lane warps, shuffles emulated on lists),
  which re-read the lane-0 carry behaviour from the shuffle semantics instead of from the
  oracle's derived rule.
"""
import numpy as np

U32 = 0xFFFFFFFF


def bits_of_words(words):
    """MSB-first bit string of a sequence of uint32 words in memory order."""
    return "".join(format(int(w) & U32, "032b") for w in words)


def window(bitstr, end, width=16):
    """The `width` bits ending at position `end` (exclusive), zero-extended on the left."""
    start = end - width
    if start < 0:
        s = "0" * (-start) + bitstr[:end]
    else:
        s = bitstr[start:end]
    return int(s, 2) if s else 0


def decompress_bruteforce(compressed, codebook_bits, continuous):
    """inference.cu:42-96 by bit strings.  compressed uint32 [m, 4cn]; returns uint16 [m, 64cn]."""
    m, words = compressed.shape
    cn = words // 4
    out = np.zeros((m, 64 * cn), dtype=np.uint16)
    for r in range(m):
        row = bits_of_words(compressed[r])
        for c in range(cn):
            base = 128 * c
            if c == 0:
                hist = "0" * 16
            elif continuous or c % 32 != 0:
                hist = row[base - 16:base]          # low half of the previous w
            else:
                hist = row[base - 32:base - 16]      # the uint16 below the element in memory = high half of w
            s = hist + row[base:base + 128]
            for i in range(64):
                st = int(s[2 * (i + 1):2 * (i + 1) + 16], 2)
                out[r, 64 * c + i] = codebook_bits[st]
    return out


def fsl(lo, hi, s):
    """__funnelshift_l(lo, hi, s): upper 32 bits of (hi:lo) << s, s in [0, 31]."""
    return (((hi << 32) | lo) << s >> 32) & U32


def matvec_cuda_sim(compressed, codebook_bits, x, S, continuous=False):
    """Thread-level simulation of decompress_matvec_kernel (inference.cu:189-277), one warp per
    row, with double accumulation.  compressed uint32 [T, m, 128]; x float16 [n]."""
    T, m, _ = compressed.shape
    n = 2048 * T
    xf = x.astype(np.float64)
    # smem_x (inference.cu:215-221): half2 slots
    smem_x = np.zeros((n // 2, 2))
    for idx in range(n // 8):
        for i in range(4):
            smem_x[idx + i * (n // 2 // 4)] = xf[8 * idx + 2 * i:8 * idx + 2 * i + 2]
    cb = codebook_bits.view(np.float16).astype(np.float64)
    y = np.zeros(m)
    for r in range(m):
        inner = [np.zeros(2) for _ in range(32)]
        carry = [0] * 32
        for it in range(T):
            elem = [[int(v) & U32 for v in compressed[it, r, 4 * l:4 * l + 4]] for l in range(32)]
            w = [e[3] for e in elem]
            # __shfl_up_sync(FULL_MASK, elem.w, 1): lane 0 keeps its own value
            shfl_up = [w[l - 1] if l >= 1 else w[l] for l in range(32)]
            # __shfl_down_sync(FULL_MASK, elem.w, 31): lane 0 reads lane 31, the rest keep theirs
            shfl_down = [w[l + 31] if l + 31 < 32 else w[l] for l in range(32)]
            if continuous:
                prev = carry[:]            # what `carry = next_carry` of the last iteration left
                new_carry = [shfl_up[l] if l >= 1 else prev[0] for l in range(32)]
            else:
                new_carry = shfl_up        # the assignment overwrites every lane, lane 0 included
            for l in range(32):
                ex, ey, ez, ew = elem[l]
                reg_c = [ex, ey, ez, ew,
                         fsl(ey, ex, 16), fsl(ez, ey, 16), fsl(ew, ez, 16), fsl(ex, new_carry[l], 16)]
                for k in range(8):
                    for j in range(4):
                        reg_a = smem_x[((it * 8 + k) * 4 + j) * 32 + l]
                        h = reg_c[k] >> (16 - 4 - 4 * j)
                        h = (h * (h + 1)) & U32
                        idx = h >> 1
                        mask = ((1 << S) - 1) << 7
                        entry = (idx & mask) >> 7      # lop3 0xCA splices idx under mask into the address
                        w0 = int(codebook_bits[2 * entry])
                        w1 = int(codebook_bits[2 * entry + 1])
                        w0 = (0x8000 & h) | (~0x8000 & w0 & 0xFFFF)   # lop3 0xCA with toggle
                        f0 = float(np.array([w0], dtype=np.uint16).view(np.float16)[0])
                        f1 = cb[2 * entry + 1]
                        inner[l] = inner[l] + np.array([f0, f1]) * reg_a
            carry = shfl_down
        y[r] = sum(v[0] + v[1] for v in inner)
    return y


def matvec_t_cuda_sim(compressed, codebook_bits, x, m, L, continuous=False):
    """Thread-level simulation of decompress_matvec_t_kernel (inference_t.cu:68-175)."""
    n = x.shape[0]
    c = compressed.reshape(-1).astype(np.uint64)
    cb = codebook_bits.view(np.float16).astype(np.float64)
    xf = x.astype(np.float64)
    mask = (1 << L) - 1
    y = np.zeros(m)
    for row in range(m):
        carry = 0
        acc = np.zeros(2)
        for col in range(n // 16 // 4):
            base = (row + col * m) * 4
            reg_c = [int(c[base + q]) for q in range(4)]
            for k in range(4):
                sft2, sft4 = [0] * 8, [0] * 8
                word = reg_c[k]
                if not continuous:
                    for j in range(8):
                        sft2[j] = mask & fsl(word, carry, 2)
                        sft4[j] = mask & fsl(word, carry, 4)
                else:
                    cc = carry
                    for j in range(8):
                        sft2[j] = mask & fsl(word, cc, 2)
                        sft4[j] = mask & fsl(word, cc, 4)
                        cc = sft4[j]
                        word = (word << 4) & U32
                for j in range(8):
                    carry = sft4[j]
                    p = col * 32 + k * 8 + j
                    acc = acc + np.array([cb[sft2[j]], cb[sft4[j]]]) * xf[2 * p:2 * p + 2]
        y[row] = acc[0] + acc[1]
    return y


def pack_symbols_msb_first(symbols):
    """2-bit symbols -> uint32 words, first symbol in the top bits."""
    symbols = np.asarray(symbols, dtype=np.uint32).reshape(-1, 16)
    words = np.zeros(symbols.shape[0], dtype=np.uint32)
    for i in range(16):
        words |= symbols[:, i] << np.uint32(30 - 2 * i)
    return words

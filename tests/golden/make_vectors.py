"""Writes tests/golden/vectors_small.npz: small seeded inputs with the outputs the CPU oracle gives
for them, one case per op and carry mode.

Run it only after tests/test_oracle_kat.py passes (the oracle is then held to the hand-derived
known answers and the thread-level simulations of the reference kernels).  The file freezes those
outputs, so that a later change to the oracle or to a kernel is measured against committed data
and not only against a live oracle call.  Nothing from the reference runs here.

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import rptc_oracle as orc      # noqa: E402
from util import np_f16, np_u32, rand_codes, rand_half     # noqa: E402

# name -> (op, keyword arguments); sizes keep the file at a few hundred KiB
CASES = {
    "decompress": dict(m=3, cn=32),
    "matvec_s6": dict(m=8, n=2048, S=6),
    "matvec_s8_ragged": dict(m=5, n=2048 + 192, S=8),
    "matvec_t_16": dict(m=64, n=128, L=16),
    "matvec_t_14": dict(m=64, n=128, L=14),
    "bits3": dict(m=4, n=2048 + 64, S=8, bits=3),
    "bits4": dict(m=4, n=2048 + 64, S=6, bits=4),
    "hadamard": dict(batch=2, n=11008, block=256),
}


def build():
    out = {}
    c = CASES["decompress"]
    comp = np_u32(rand_codes(c["m"] * 4 * c["cn"], seed=1001)).reshape(c["m"], 4 * c["cn"])
    cb = np_f16(rand_half(65536, seed=1002))
    out["decompress.comp"], out["decompress.codebook"] = comp, cb.view(np.uint16)
    for mode in (0, 1):
        out[f"decompress.out.mode{mode}"] = orc.decompress(comp, cb, mode=mode).view(np.uint16)

    for name in ("matvec_s6", "matvec_s8_ragged"):
        c = CASES[name]
        m, n, S = c["m"], c["n"], c["S"]
        comp = np_u32(rand_codes(m * n // 16, seed=1010 + S))
        cb = np_f16(rand_half(2 << S, seed=1020 + S))
        x = np_f16(rand_half(n, seed=1030 + S))
        out[f"{name}.comp"], out[f"{name}.codebook"], out[f"{name}.x"] = comp, cb.view(np.uint16), x.view(np.uint16)
        for mode in (0, 1):
            out[f"{name}.W.mode{mode}"] = orc.matvec_dense(comp, cb, m, n, S, mode=mode).view(np.uint16)
            out[f"{name}.y.mode{mode}"] = orc.matvec(comp, cb, x, m, S, mode=mode)

    for name in ("matvec_t_16", "matvec_t_14"):
        c = CASES[name]
        m, n, L = c["m"], c["n"], c["L"]
        comp = np_u32(rand_codes(m * n // 16, seed=1040 + L))
        cb = np_f16(rand_half(1 << L, seed=1050 + L))
        x = np_f16(rand_half(n, seed=1060 + L))
        out[f"{name}.comp"], out[f"{name}.codebook"], out[f"{name}.x"] = comp, cb.view(np.uint16), x.view(np.uint16)
        for mode in (0, 1):
            out[f"{name}.W.mode{mode}"] = orc.matvec_t_dense(comp, cb, m, n, L, mode=mode).view(np.uint16)
            out[f"{name}.y.mode{mode}"] = orc.matvec_t(comp, cb, x, m, L, mode=mode)

    for name in ("bits3", "bits4"):
        c = CASES[name]
        m, n, S, bits = c["m"], c["n"], c["S"], c["bits"]
        comp = np_u32(rand_codes(m * n * bits // 32, seed=1070 + bits))
        cb = np_f16(rand_half(2 << S, seed=1080 + bits))
        x = np_f16(rand_half(n, seed=1090 + bits))
        out[f"{name}.comp"], out[f"{name}.codebook"], out[f"{name}.x"] = comp, cb.view(np.uint16), x.view(np.uint16)
        for mode in (0, 1):
            W = orc.bits_dense(comp, cb, m, n, S, bits, mode=mode)
            out[f"{name}.W.mode{mode}"] = W.view(np.uint16)
            out[f"{name}.y.mode{mode}"] = orc.dense_matvec(W, x)

    c = CASES["hadamard"]
    x = np_f16(rand_half(c["batch"] * c["n"], seed=1100)).reshape(c["batch"], c["n"])
    signs = np.where(np.random.default_rng(1101).integers(0, 2, c["n"]) == 1, 1.0, -1.0).astype(np.float16)
    out["hadamard.x"], out["hadamard.signs"] = x.view(np.uint16), signs.view(np.uint16)
    out["hadamard.y"] = np.asarray(orc.sign_hadamard(x, signs, c["block"], inverse=False))
    return out


if __name__ == "__main__":
    arrays = build()
    path = os.path.join(HERE, "vectors_small.npz")
    np.savez_compressed(path, **arrays)
    print(path, os.path.getsize(path), "bytes,", len(arrays), "arrays")

#!/usr/bin/env python3
"""Writes tests/golden/codegen_vectors.npz: float32 weights and the (shift, sign) that the reference's
get_shift_and_sign (deepshift/utils.py:23-29) gives for them on the CPU,

    sign = torch.sign(w);  shift = torch.round(torch.log(torch.abs(w)) / np.log(2))

evaluated here with plain torch CPU ops (the reference package is not imported).  The inputs are the
cases where the result depends on how the float32 logarithm and division round: the floats nearest to
2^(n + 1/2) and their neighbours up to 3 ulps on both sides for n = -40 .. 8, the exact powers of two
and their neighbours, denormals, zeros, infinities, and 4096 seeded random weights.

    python tests/golden/make_codegen_vectors.py
"""
import os

import numpy as np
import torch


def main():
    bits = []
    for n in range(-40, 9):
        for centre in (np.float32(2.0 ** (n + 0.5)), np.float32(2.0 ** n)):
            u = int(centre.view(np.uint32))
            bits += [u + d for d in range(-3, 4)]
    w = np.array(bits, np.uint32).view(np.float32)
    rng = np.random.default_rng(2024)
    rand = (rng.standard_normal(4096) * np.exp(rng.uniform(-12, 2, 4096))).astype(np.float32)
    special = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-40, 3e-39, np.inf, -np.inf, 0.75, 0.7, 0.35, -0.1,
                        1.0, -1.0, 3.4028235e38], np.float32)
    w = np.concatenate([w, -w[::3], rand, special]).astype(np.float32)
    t = torch.from_numpy(w)
    shift = torch.round(torch.log(torch.abs(t)) / np.log(2))
    sign = torch.sign(t)
    here = os.path.dirname(os.path.abspath(__file__))
    np.savez_compressed(os.path.join(here, "codegen_vectors.npz"), w=w, shift=shift.numpy(), sign=sign.numpy())
    ties = int((torch.log(torch.abs(t)) / np.log(2) % 1 == 0.5).sum())
    print("%d weights, %d of them exact float32 ties of log2" % (w.size, ties))


if __name__ == "__main__":
    main()

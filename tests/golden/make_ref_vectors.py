"""Writes tests/golden/ref_cpu_vectors.npz: seeded inputs and the outputs that the reference's own
CPU shift kernel (kernels/cpu/shift_cpu.cpp, compiled by oracle/Makefile into oracle/_ref) returns
for them.  Run where the reference checkout is present:

    make -C oracle && python tests/golden/make_ref_vectors.py

The fixture is data only (inputs + expected outputs); it lets the oracle and the GPU library be
checked against the real reference where oracle/_ref cannot be built.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import shift_oracle as so  # noqa: E402


def main():
    ref = so.load_reference_cpu_kernel()
    if ref is None:
        raise SystemExit("oracle/_ref is not built")
    rng = np.random.default_rng(20240607)

    M, K, N = 37, 101, 19
    lin_x = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(M, K), dtype=np.int64).astype(np.int32)
    lin_x[0, :4] = [2147418112, -2 ** 31, -1, 65536]
    lin_shift = -rng.integers(0, 32, size=(N, K)).astype(np.int8)
    lin_sign = rng.choice(np.array([-1, 0, 1], np.int32), size=(N, K), p=[0.45, 0.1, 0.45])
    lin_bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    lin_y = np.array(ref.linear_kernel(lin_x.tolist(), lin_shift.tolist(), lin_sign.tolist(),
                                       lin_bias.tolist()), np.int64).astype(np.int32)

    Nb, C, Hp, Wp, O, FH, FW = 3, 5, 11, 12, 7, 3, 3
    stride = (2, 1)
    conv_x = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(Nb, C, Hp, Wp), dtype=np.int64).astype(np.int32)
    conv_shift = -rng.integers(0, 16, size=(O, C, FH, FW)).astype(np.int8)
    conv_sign = rng.choice(np.array([-1, 1], np.int32), size=(O, C, FH, FW))
    conv_bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    conv_y = np.array(ref.convolution_kernel(conv_x.tolist(), conv_shift.tolist(), conv_sign.tolist(),
                                             conv_bias.tolist(), list(stride), [0, 0]),
                      np.int64).astype(np.int32)

    out = os.path.join(HERE, "ref_cpu_vectors.npz")
    np.savez_compressed(out, lin_x=lin_x, lin_shift=lin_shift, lin_sign=lin_sign, lin_bias=lin_bias,
                        lin_y=lin_y, conv_x=conv_x, conv_shift=conv_shift, conv_sign=conv_sign,
                        conv_bias=conv_bias, conv_y=conv_y, conv_stride=np.array(stride, np.int32))
    print(out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()

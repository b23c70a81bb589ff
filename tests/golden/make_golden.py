"""Writes the golden fixtures of this directory.

The reference holds no stored vectors for the MXFP4 GEMM path (its tests
regenerate inputs and compare with its torch oracle on a GPU), so the fixtures
are produced by this repository's own exact oracle (oracle/mxfp4_oracle.py,
``scaled_gemm_exact``: per-32-group integer dot products scaled by exact powers
of two and summed in f64), which the CPU test-suite pins against exact-rational
brute force.  Each fixture is data only: packed inputs and the expected C.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import mxfp4_oracle as orc  # noqa: E402

CASES = [
    # name, m, n, k, seed, scale range
    ("g_32x32x128", 32, 32, 128, 11, (124, 130)),
    ("g_64x48x256", 64, 48, 256, 12, (124, 130)),
    ("g_37x80x512_wide", 37, 80, 512, 13, (100, 154)),
    ("g_1x64x1024", 1, 64, 1024, 14, (120, 134)),
    ("g_48x32x160_ktail", 48, 32, 160, 15, (124, 130)),
]


def main():
    for name, m, n, k, seed, (lo, hi) in CASES:
        x, xs, w_t, ws = orc.make_inputs(m, n, k, seed, lo, hi)
        c = orc.scaled_gemm_exact(x, w_t, xs, ws)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, x_scales=xs, w_t=w_t, w_scales=ws,
                            c_exact=c, x_scales_shuffled=orc.e8m0_shuffle_padded(xs),
                            w_scales_shuffled=orc.e8m0_shuffle_padded(ws),
                            w_t_preshuffled=orc.b_preshuffle(w_t) if n % 16 == 0 and k % 64 == 0
                            else np.zeros((0, 0), np.uint8))
        print(name, c.shape, float(np.abs(c).max()))

    # decode tables: every byte value through both decoders
    b = np.arange(256, dtype=np.uint8).reshape(1, 256)
    np.savez_compressed(os.path.join(HERE, "g_decode_all_bytes.npz"), bytes=b,
                        e2m1_f32_bits=orc.mxfp4_to_f32(b).view(np.uint32),
                        e8m0_f32_bits=orc.e8m0_to_f32(b.reshape(-1)).view(np.uint32))


if __name__ == "__main__":
    main()

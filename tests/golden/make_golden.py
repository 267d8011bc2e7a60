"""Writes tests/golden/naive_ref_vectors.npz: inputs and the outputs the
reference's OWN naive convolution layers produce for them.

Run in the container that holds the reference checkout:
    python tests/golden/make_golden.py
It compiles the two reference headers through oracle/Makefile (target `ref`)
and calls them; nothing of the reference is copied, the file holds only input
and output numbers.  The inputs come from the seeded generator in oracle/, so
the file can be regenerated bit for bit.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

# name -> (N, C, H, W, K, kh, kw, sh, sw, pt, pb, pl, pr, which reference header)
CASES = {
    "fixed3x3_c3_7x9": (1, 3, 7, 9, 4, 3, 3, 1, 1, 1, 1, 1, 1, "fixed"),
    "fixed3x3_c5_13x13_pad0": (1, 5, 13, 13, 6, 3, 3, 1, 1, 0, 0, 0, 0, "fixed"),
    "fixed3x3_c8_14x14_batch2": (2, 8, 14, 14, 5, 3, 3, 1, 1, 1, 1, 1, 1, "fixed"),
    "general3x3_c8_14x14": (1, 8, 14, 14, 5, 3, 3, 1, 1, 1, 1, 1, 1, "general"),
    "general3x3_s2_c6_15x15": (1, 6, 15, 15, 7, 3, 3, 2, 2, 1, 1, 1, 1, "general"),
    "general1x1_c16_7x7": (1, 16, 7, 7, 9, 1, 1, 1, 1, 0, 0, 0, 0, "general"),
    "general1x1_s2_c8_8x8": (1, 8, 8, 8, 4, 1, 1, 2, 2, 0, 0, 0, 0, "general"),
    "general7x7_s2_c3_17x17": (1, 3, 17, 17, 4, 7, 7, 2, 2, 3, 3, 3, 3, "general"),
    "general5x3_s1x2_asym": (2, 4, 11, 12, 3, 5, 3, 1, 2, 0, 1, 2, 1, "general"),
    "general3x3_bias_c4_9x9": (1, 4, 9, 9, 3, 3, 3, 1, 1, 1, 1, 1, 1, "general_bias"),
}


def main():
    O.build(force=True)
    if O.ref_lib() is None:
        raise SystemExit("oracle/_ref was not built: the reference checkout is needed")
    out = {}
    for i, (name, c) in enumerate(sorted(CASES.items())):
        s = O.Shape(*c[:13])
        x, w = O.make_inputs(s, seed=100 + i)
        out[name + "/shape"] = np.array(c[:13], np.int32)
        out[name + "/x"] = x
        out[name + "/w"] = w
        if c[13] == "fixed":
            y = O.ref_naive_3x3s1(s, x, w)
        elif c[13] == "general":
            y = O.ref_naive_general(s, x, w)
        else:
            oh, ow = O.out_hw(s)
            b = O.rng_uniform(7000 + i, (s.K, oh, ow))
            out[name + "/bias_elems"] = b
            y = O.ref_naive_general(s, x, w, b)
        out[name + "/y"] = y
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "naive_ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(CASES), "cases")


if __name__ == "__main__":
    main()

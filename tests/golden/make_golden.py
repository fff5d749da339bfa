"""Writes the golden fixtures in this directory.

Every expected output is produced by the REFERENCE library's own CPU lowering
of the composed pipeline (oracle/_ref/, built by oracle/build_ref.sh from the
reference tree), on small seeded inputs.  Run in the development container
only: the fixtures, not the reference, travel to the GPU box.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as o  # noqa: E402
from oracle import ref  # noqa: E402


def main():
    if not ref.available():
        raise SystemExit("oracle/_ref is not built: run `bash oracle/build_ref.sh` first")
    fx = {}
    # blur, uniform[0,1)
    img = o.uniform((38, 44), 11)
    fx["blur_xy_in"] = img
    fx["blur_xy_out"] = ref.blur_chain(img, "xy", 12, 14)
    img = o.uniform((26, 52), 12)
    fx["blur_xyx_in"] = img
    fx["blur_xyx_out"] = ref.blur_chain(img, "xyx", 8, 16)
    # a wider one that spans more than one 252-column wave strip
    img = o.uniform((14, 600), 13)
    fx["blur_xyx_wide_in"] = img
    fx["blur_xyx_wide_out"] = ref.blur_chain(img, "xyx", 4, 149)
    # blur, ascending (the reference's own blur check input)
    img = o.ascending(34, 40)
    fx["blur_xy_asc_in"] = img
    fx["blur_xy_asc_out"] = ref.blur_chain(img, "xy", 8, 19)
    # softmax, N(0, 2^2)
    x = o.normal((8, 64), 21, 0.0, 2.0)
    fx["softmax64_in"] = x
    fx["softmax64_out"] = ref.softmax_rows(x, 2)
    x = o.normal((4, 1000), 22, 0.0, 2.0)
    fx["softmax1000_in"] = x
    fx["softmax1000_out"] = ref.softmax_rows(x, 1)
    x = o.normal((2, 4096), 23, 0.0, 2.0)
    fx["softmax4096_in"] = x
    fx["softmax4096_out"] = ref.softmax_rows(x, 1)
    # GEMM, uniform[-1,1), one k tile (sequential-k sums)
    A = o.uniform((16, 24), 31, -1.0, 1.0)
    B = o.uniform((24, 8), 32, -1.0, 1.0)
    fx["gemm_A"] = A
    fx["gemm_B"] = B
    fx["gemm_C"] = ref.gemm(A, B, 4, 4, 24)
    # the reference's known-answer shape: ascending 10x10 (test/test-cpu-mm.cpp:13-85)
    A = o.ascending(10, 10)
    fx["gemm_asc_A"] = A
    fx["gemm_asc_C"] = ref.gemm(A, A, 5, 5, 10)
    np.savez_compressed(os.path.join(HERE, "reference_vectors.npz"), **fx)
    print("wrote", os.path.join(HERE, "reference_vectors.npz"), {k: v.shape for k, v in fx.items()})


if __name__ == "__main__":
    main()

"""Generate ``tests/golden/chamfer_found_cases.npz``: inputs on which a chamfer kernel of
this library once returned a result that differs from the reference's rule, with the
expected outputs.

Case "zero_extent_frame" (5 x 93 queries against 5 x 207 keys): in one batch element the
keys sit within one unit in the last place of each other at coordinates near 900 and 180
of the 207 are identical. A frame trimmed to a few mean deviations then has no extent, the
power-of-two scale of the fp16 terms stays 1 and the other keys' offsets of 6e-5 have no
precision left in those terms, so an equal-distance tie went to key 144 instead of key 0
(the reference keeps the lowest index: strict '<' over ascending j,
torkit3d/csrc/cuda/chamfer_distance_kernel.cu:60-78). The clouds are kept exactly as the
random differential run produced them.

The expected outputs come from the exact-rational fp32 restatement of ``make_golden.py``
(no code shared with ``oracle/`` or the kernels).

Run:  python tests/golden/make_chamfer_cases.py            (recomputes the outputs from
      the inputs the fixture already holds)
      python tests/golden/make_chamfer_cases.py x.npz      (first creation: x.npz holds
      arrays x1, x2)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from make_golden import chamfer_one_direction  # noqa: E402

OUT = os.path.join(HERE, "chamfer_found_cases.npz")


def main():
    src = np.load(sys.argv[1] if len(sys.argv) > 1 else OUT)
    if len(sys.argv) > 1:
        x1, x2 = src["x1"], src["x2"]
    else:
        x1, x2 = src["zero_extent_frame_xyz1"], src["zero_extent_frame_xyz2"]
    x1 = np.ascontiguousarray(x1, np.float32)
    x2 = np.ascontiguousarray(x2, np.float32)
    d1, i1 = chamfer_one_direction(x1, x2)
    d2, i2 = chamfer_one_direction(x2, x1)
    np.savez_compressed(OUT, zero_extent_frame_xyz1=x1, zero_extent_frame_xyz2=x2,
                        zero_extent_frame_dist1=d1, zero_extent_frame_idx1=i1,
                        zero_extent_frame_dist2=d2, zero_extent_frame_idx2=i2)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()

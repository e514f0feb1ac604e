"""Writes tests/golden/reference_shape_grid.json: the 81 forward and 81 backward (B, S, D, I)
cases that the reference's test module parametrizes over (fused_swiglu/test_swiglu.py:58-67 and
:81-90).  They are a pure function of numpy's legacy generator seeded with 0 (test_swiglu.py:11),
drawn in the nesting order of the two list comprehensions, so this script needs neither the
reference nor a GPU.  Run:  python tests/golden/make_shape_grid.py"""
import json
import os

import numpy as np

NUM_TEST = 3  # the reference's default (test_swiglu.py:13-16)


def draw(rs):
    return [
        [int(b), int(sq), int(dm), int(di)]
        for b in rs.randint(1, 4, size=NUM_TEST)
        for sq in 64 * rs.randint(1, 32, size=NUM_TEST)
        for dm in 64 * rs.randint(1, 128, size=NUM_TEST)
        for di in 64 * rs.randint(1, 128, size=NUM_TEST)
    ]


if __name__ == "__main__":
    rs = np.random.RandomState(0)
    fwd = draw(rs)
    bwd = draw(rs)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_shape_grid.json")
    with open(out, "w") as f:
        json.dump({"num_test": NUM_TEST, "fwd": fwd, "bwd": bwd}, f)
    print(out, len(fwd), len(bwd), fwd[0], bwd[0])

"""Writes the committed fixtures ``tests/golden/*.npz``: seeded inputs and the float64 oracle's outputs.

The reference tree holds no golden tensors for this path and cannot be imported here (it needs jax), so these
vectors come from the oracle, after the oracle itself was pinned by ``tests/test_oracle_*.py``.  They freeze the
expected values so that a later change of the oracle or of the input generators is noticed.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import wkv4 as o4, wkv6 as o6, wkv7 as o7  # noqa: E402
from tests.inputs import wkv4_inputs, wkv6_inputs, wkv7_inputs  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    x = wkv7_inputs(2, 24, 1, 64, seed=101, p_reset=0.1, min_len_frac=0.4)
    x["new_starts"][1, int(x["length"][1]) % 24] = True
    args = (x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    out = {}
    for compat in (0, 1):
        s, y = o7.wkv7_base(*args, compat=bool(compat))
        g = o7.wkv7_bwd(*args, x["dy"], x["ds"], compat=bool(compat))
        out.update({f"new_s_c{compat}": s, f"y_c{compat}": y})
        out.update({f"g{n}_c{compat}": v for n, v in zip("rwkvabs", g)})
    np.savez_compressed(os.path.join(HERE, "wkv7_small.npz"), **x, **out)

    x = wkv6_inputs(2, 24, 1, 64, seed=102, p_reset=0.1)
    args = (x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"])
    out = {}
    for compat in (0, 1):
        s, y = o6.wkv6_base(*args, compat=bool(compat))
        g = o6.wkv6_bwd(*args, x["dy"], x["ds"], compat=bool(compat))
        out.update({f"new_s_c{compat}": s, f"y_c{compat}": y})
        out.update({f"g{n}_c{compat}": v for n, v in zip("rkvwus", g)})
    np.savez_compressed(os.path.join(HERE, "wkv6_small.npz"), **x, **out)

    x = wkv4_inputs(2, 30, 64, seed=103, p_reset=0.08)
    out = {}
    for compat in (0, 1):
        s, y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=bool(compat))
        out.update({f"new_s_c{compat}": s, f"y_c{compat}": y})
    np.savez_compressed(os.path.join(HERE, "wkv4_small.npz"), **x, **out)


if __name__ == "__main__":
    main()

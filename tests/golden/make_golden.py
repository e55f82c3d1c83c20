"""Writes tests/golden/config0.npz: outputs of the float64 token recurrence on benchmark configuration 0.

The reference ships no golden vectors (all of its tests draw unseeded random inputs), and its files are not
imported here; the fixture pins this repository's own oracle and seeded input generator against drift.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "hdla-impl_amd"))

from hdla_hip.synthetic import make_config  # noqa: E402
from oracle import hrdplr_oracle as O  # noqa: E402

if __name__ == "__main__":
    inp = make_config(0)
    o, h = O.recurrence(inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, 1.0, None)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "config0.npz"),
                        o_every8=o.float().numpy()[:, ::8], final_state=h.float().numpy(),
                        q_sum=np.float64(inp.q.double().sum().item()), gk_sum=np.float64(inp.gk.double().sum().item()))
    print("wrote config0.npz")

"""Writes tests/golden/config0.npz: outputs of the float64 token recurrence on benchmark configuration 0, and
tests/golden/layer0.npz: outputs of the float64 normalisation and layer oracles on small seeded inputs.

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
from oracle import layer_oracle as LO  # noqa: E402
from oracle import normalize_oracle as NO  # noqa: E402


def layer_case():
    """Seeded inputs of the layer fixture: a state_dict with the reference's parameter names (embed_dim 32, 4 heads)
    and x [2, 10, 32]."""
    import torch
    g = torch.Generator().manual_seed(2024)
    d, H, D = 32, 4, 8
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * (2.0 / s[-1] ** 0.5)
    sd = {"q_proj.weight": r(d, d), "k_proj.weight": r(d, d), "v_proj.weight": r(d, d), "f_proj.0.weight": r(D, d),
          "f_proj.1.weight": r(d, D), "bet_proj.weight": r(H, d), "o_proj.weight": r(d, d), "norm.weight": 1 + 0.1 * r(d),
          "output_gate.0.weight": r(D, d), "output_gate.1.weight": r(d, D)}
    x = torch.randn(2, 10, d, generator=g, dtype=torch.float64)
    gate = torch.randn(2, 10, d, generator=g, dtype=torch.float64)
    return sd, x, gate, H

if __name__ == "__main__":
    inp = make_config(0)
    o, h = O.recurrence(inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, 1.0, None)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "config0.npz"),
                        o_every8=o.float().numpy()[:, ::8], final_state=h.float().numpy(),
                        q_sum=np.float64(inp.q.double().sum().item()), gk_sum=np.float64(inp.gk.double().sum().item()))
    print("wrote config0.npz")
    sd, x, gate, H = layer_case()
    out, S = LO.hdla_layer(sd, x, H)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "layer0.npz"),
                        layer_out=out.numpy(), layer_state=S.numpy(),
                        rms_gate_pre=NO.rms_norm_fused_gate(x, gate, sd["norm.weight"], eps=1e-5).numpy(),
                        group_post=NO.normalize(x, sd["norm.weight"], gate, "sigmoid", "post", c=8 ** 0.5, eps=1e-3,
                                                num_groups=4).numpy(),
                        l2=NO.l2_norm(x.reshape(2, 10, 4, 8)).numpy())
    print("wrote layer0.npz")

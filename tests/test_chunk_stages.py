"""The hand-written forward/backward algebra of the 16-token chunk pipeline (oracle/chunk_stages.py), which is
what the HIP kernels implement stage by stage, against autograd through the token recurrence."""
import pytest
import torch

from hdla_hip.synthetic import make_inputs
from oracle import chunk_stages as CS
from oracle import hrdplr_oracle as O


@pytest.mark.parametrize("T,gk_div", [(16, 1.0), (40, 1.0), (96, 16.0), (7, 1.0)])
def test_stages_match_autograd(T, gk_div):
    x = make_inputs(21, 2, T, 2, 16, 8, gk_div=gk_div)
    leaves = [t.double().requires_grad_() for t in (x.q, x.k, x.v, x.a, x.b, x.gk, x.h0)]
    o, ht = O.recurrence(*leaves[:6], 0.6, leaves[6])
    do, dht = x.do.double(), x.dht.double()
    ref = torch.autograd.grad([o, ht], leaves, [do, dht])
    o2, ht2, g, _ = CS.forward_backward(*[t.detach() for t in leaves[:6]], 0.6, leaves[6].detach(), do, dht)
    assert O.rel_l2(o2, o) < 1e-12 and O.rel_l2(ht2, ht) < 1e-12
    for name, r in zip(["dq", "dk", "dv", "da", "db", "dgk", "dh0"], ref):
        assert O.rel_l2(g[name], r) < 1e-11, name


def test_stages_without_initial_state_or_final_gradient():
    x = make_inputs(22, 1, 33, 2, 16, 16)
    leaves = [t.double().requires_grad_() for t in (x.q, x.k, x.v, x.a, x.b, x.gk)]
    o, _ = O.recurrence(*leaves, 1.0, None)
    do = x.do.double()
    ref = torch.autograd.grad([o], leaves, [do])
    _, _, g, _ = CS.forward_backward(*[t.detach() for t in leaves], 1.0, None, do, None)
    for name, r in zip(["dq", "dk", "dv", "da", "db", "dgk"], ref):
        assert O.rel_l2(g[name], r) < 1e-11, name

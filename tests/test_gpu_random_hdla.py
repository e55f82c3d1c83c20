"""Seeded sweep over shapes and options of the operators with a, b formed in the kernels (chunked forward + backward,
token-serial forward) against the float64 recurrence on oracle.parameterize_a_b; tolerances of test_gpu_hdla.py."""
import random

import pytest
import torch

from hdla_hip import chunk_hdla_delta_rule, fused_recurrent_hdla_delta_rule
from oracle import hrdplr_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
NAMES = ["dq", "dk", "dv", "dbeta", "dlog_f", "dh0"]


@pytest.mark.parametrize("seed", range(4))
def test_parameterised_operators_sweep(seed):
    rnd = random.Random(300 + seed)
    for case in range(8):
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float32])
        K, V, H = rnd.choice([64, 128, 48]), rnd.choice([64, 128, 96]), rnd.choice([1, 2, 3, 5, 17])
        varlen = rnd.random() < 0.4
        if varlen:
            cuts = sorted(rnd.sample(range(1, 150), rnd.choice([1, 2, 4])))
            cu = torch.tensor([0] + cuts + [cuts[-1] + rnd.choice([0, 1, 33])])
            B, T, N = 1, int(cu[-1]), len(cu) - 1
        else:
            cu, B, T = None, rnd.choice([1, 2, 3]), rnd.choice([1, 15, 16, 17, 50, 130])
            N = B
        gk_div, scale = rnd.choice([1.0, 4.0, 16.0]), rnd.choice([1.0, 0.125])
        g = torch.Generator().manual_seed(seed * 100 + case)
        rn = lambda *s: torch.randn(*s, generator=g)
        q = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1)
        k = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1)
        v, beta = rn(B, T, H, V), 2.0 * torch.rand(B, T, H, 1, generator=g)
        log_f = torch.nn.functional.logsigmoid(rn(B, T, H, K)) / gk_div
        h0, do, dht = rn(N, H, K, V), rn(B, T, H, V), rn(N, H, K, V)
        lo = [t.to(dtype).double().requires_grad_() for t in (q, k, v, beta, log_f)] + [h0.double().requires_grad_()]
        a, b = O.parameterize_a_b(lo[3], lo[1], lo[4])
        ro, rht = O.recurrence(lo[0], lo[1], lo[2], a, b, lo[4], scale, lo[5], cu_seqlens=cu)
        rg = torch.autograd.grad([ro, rht], lo, [do.to(dtype).double(), dht.double()])
        ld = [t.to(dtype).to(DEV).requires_grad_() for t in (q, k, v, beta, log_f)] + [h0.to(DEV).requires_grad_()]
        o, ht = chunk_hdla_delta_rule(*ld[:5], scale=scale, initial_state=ld[5], output_final_state=True,
                                      cu_seqlens=None if cu is None else cu.to(DEV))
        gg = torch.autograd.grad([o, ht], ld, [do.to(dtype).to(DEV), dht.to(DEV)])
        tol_o, tol_g = (5e-3, 1e-2) if dtype == torch.bfloat16 else (1e-5, 1e-5)
        what = (dtype, B, T, H, K, V, None if cu is None else cu.tolist(), gk_div, scale)
        assert O.rel_l2(o, ro) <= tol_o and O.rel_l2(ht, rht) <= tol_o, what
        for n, x, y in zip(NAMES, gg, rg):
            assert O.rel_l2(x, y) <= tol_g, (n, what)
        if cu is None and T <= 20:                          # the token-serial operator on the same inputs
            with torch.no_grad():
                o2, ht2 = fused_recurrent_hdla_delta_rule(*[t.detach() for t in ld[:5]], scale=scale,
                                                          initial_state=ld[5].detach(), output_final_state=True)
            assert O.rel_l2(o2, ro) <= tol_o and O.rel_l2(ht2, rht) <= tol_o, what

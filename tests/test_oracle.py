"""Pins the CPU oracle (oracle/hrdplr_oracle.py) without the reference being importable: closed forms, special
cases that reduce to textbook recurrences, invariants and finite differences.  Each check is chosen so that a
plausible mistake (wrong row order of a/b, decay applied before the rank terms, output read before the update,
a dropped term, a transposed operand) breaks at least one of them."""
import os

import numpy as np
import pytest
import torch

from hdla_hip.synthetic import make_inputs, make_config
from oracle import hrdplr_oracle as O

D = torch.float64


def _inp(seed, B=2, T=24, H=2, K=8, V=6, gk_div=1.0):
    x = make_inputs(seed, B, T, H, K, V, gk_div=gk_div)
    return [t.to(D) for t in (x.q, x.k, x.v, x.a, x.b, x.gk, x.h0)]


def test_single_token_closed_form():
    # recurrent.py:93-104 for one token: both rank terms read S0, the decay multiplies S0, o reads S1
    q, k, v, a, b, g, S0 = _inp(1, B=3, T=1, H=2, K=5, V=4)
    o, S1 = O.recurrence(q, k, v, a, b, g, 0.5, S0)
    a0, a1, b0, b1 = a[:, 0], a[:, 1], b[:, 0], b[:, 1]                      # rows t*R + r
    exp = torch.exp(g[:, 0])[..., None] * S0 \
        + b0[..., None] * torch.einsum('bhk,bhkv->bhv', a0, S0)[:, :, None] \
        + b1[..., None] * torch.einsum('bhk,bhkv->bhv', a1, S0)[:, :, None] \
        + k[:, 0][..., None] * v[:, 0][:, :, None]
    assert torch.allclose(S1, exp, atol=1e-12)
    assert torch.allclose(o[:, 0], 0.5 * torch.einsum('bhk,bhkv->bhv', q[:, 0], exp), atol=1e-12)


def test_two_tokens_row_order_of_ab():
    # token 1 must use rows 2 and 3 of a/b (rank fastest); explicit matrix form S1 = (Diag + sum b a^T) S0 + k v^T
    q, k, v, a, b, g, S0 = _inp(2, B=1, T=2, H=1, K=4, V=3)
    o, S2 = O.recurrence(q, k, v, a, b, g, 1.0, S0)
    S = S0[0, 0]
    for t in range(2):
        P = torch.diag(torch.exp(g[0, t, 0]))
        for r in range(2):
            P = P + torch.outer(b[0, 2 * t + r, 0], a[0, 2 * t + r, 0])
        S = P @ S + torch.outer(k[0, t, 0], v[0, t, 0])
        assert torch.allclose(o[0, t, 0], S.T @ q[0, t, 0], atol=1e-12)
    assert torch.allclose(S2[0, 0], S, atol=1e-12)


def test_zero_ab_is_gated_linear_attention():
    q, k, v, a, b, g, S0 = _inp(3)
    z = torch.zeros_like(a)
    o, ST = O.recurrence(q, k, v, z, z, g, 1.0, S0)
    G = g.cumsum(1)                                                          # [B,T,H,K]
    T = q.shape[1]
    for t in (0, 5, T - 1):
        dec = torch.exp(G[:, t:t + 1] - G[:, :t + 1])                        # [B,t+1,H,K]
        att = torch.einsum('bhk,bjhk,bjhk->bjh', q[:, t], dec, k[:, :t + 1])
        exp = torch.einsum('bjh,bjhv->bhv', att, v[:, :t + 1]) \
            + torch.einsum('bhk,bhkv->bhv', q[:, t] * torch.exp(G[:, t]), S0)
        assert torch.allclose(o[:, t], exp, atol=1e-10)


def test_deltanet_special_case():
    # g = 0, second rank zero, a = -beta*b: S_t = (I - beta b b^T) S_{t-1} + k v^T
    q, k, v, a, b, g, S0 = _inp(4, B=1, T=12, H=1, K=6, V=5)
    g = torch.zeros_like(g)
    a = a.clone(); b = b.clone()
    a[:, 1::2] = 0; b[:, 1::2] = 0
    o, ST = O.recurrence(q, k, v, a, b, g, 1.0, S0)
    S = S0[0, 0]
    for t in range(12):
        bb, aa = b[0, 2 * t, 0], a[0, 2 * t, 0]
        beta = -(aa @ bb) / (bb @ bb)
        S = (torch.eye(6, dtype=D) - beta * torch.outer(bb, bb)) @ S + torch.outer(k[0, t, 0], v[0, t, 0])
        assert torch.allclose(o[0, t, 0], S.T @ q[0, t, 0], atol=1e-11)


def test_linear_in_v_and_initial_state():
    q, k, v, a, b, g, S0 = _inp(5)
    x = make_inputs(55, 2, 24, 2, 8, 6)
    v2, S2 = x.v.to(D), x.h0.to(D)
    o1, h1 = O.recurrence(q, k, v, a, b, g, 1.0, S0)
    o2, h2 = O.recurrence(q, k, v2, a, b, g, 1.0, S2)
    o3, h3 = O.recurrence(q, k, 2 * v - 3 * v2, a, b, g, 1.0, 2 * S0 - 3 * S2)
    assert torch.allclose(o3, 2 * o1 - 3 * o2, atol=1e-10) and torch.allclose(h3, 2 * h1 - 3 * h2, atol=1e-10)


@pytest.mark.parametrize("C", [16, 32, 64])
def test_chunk_form_equals_recurrence(C):
    q, k, v, a, b, g, S0 = _inp(6, B=2, T=128, H=2, K=16, V=8)
    o1, h1 = O.recurrence(q, k, v, a, b, g, 0.3, S0)
    o2, h2 = O.chunk_naive(q, k, v, a, b, g, 0.3, S0, chunk_size=C, dtype=D)
    assert O.rel_l2(o2, o1) < 1e-12 and O.rel_l2(h2, h1) < 1e-12


def test_chunk_form_fp32_close_to_fp64():
    q, k, v, a, b, g, S0 = _inp(7, B=1, T=256, H=2, K=16, V=16, gk_div=16.0)
    o1, h1 = O.recurrence(q, k, v, a, b, g, 1.0, S0)
    o2, h2 = O.chunk_naive(q, k, v, a, b, g, 1.0, S0, chunk_size=16, dtype=torch.float32)
    assert O.rel_l2(o2, o1) < 1e-5 and O.rel_l2(h2, h1) < 1e-5


def test_split_sequence_hand_off():
    q, k, v, a, b, g, S0 = _inp(8, T=40)
    o, h = O.recurrence(q, k, v, a, b, g, 1.0, S0)
    s = 17
    o1, hm = O.recurrence(q[:, :s], k[:, :s], v[:, :s], a[:, :2 * s], b[:, :2 * s], g[:, :s], 1.0, S0)
    o2, h2 = O.recurrence(q[:, s:], k[:, s:], v[:, s:], a[:, 2 * s:], b[:, 2 * s:], g[:, s:], 1.0, hm)
    assert torch.allclose(torch.cat([o1, o2], 1), o, atol=1e-12) and torch.allclose(h2, h, atol=1e-12)


def test_reverse_is_time_flip():
    q, k, v, a, b, g, S0 = _inp(9)
    o, h = O.recurrence(q, k, v, a, b, g, 1.0, S0, reverse=True)
    B, T, H, K = q.shape
    fl = lambda x: x.flip(1)
    flab = lambda x: x.reshape(B, T, 2, H, K).flip(1).reshape(B, 2 * T, H, K)     # flip tokens, keep rank order
    o2, h2 = O.recurrence(fl(q), fl(k), fl(v), flab(a), flab(b), fl(g), 1.0, S0)
    assert torch.allclose(o, o2.flip(1), atol=1e-12) and torch.allclose(h, h2, atol=1e-12)


def test_varlen_equals_per_sequence():
    q, k, v, a, b, g, _ = _inp(10, B=1, T=50)
    S0 = make_inputs(77, 3, 1, 2, 8, 6).h0.to(D)
    cu = torch.tensor([0, 7, 30, 50])
    o, h = O.recurrence(q, k, v, a, b, g, 1.0, S0, cu_seqlens=cu)
    for n in range(3):
        s, e = int(cu[n]), int(cu[n + 1])
        on, hn = O.recurrence(q[:, s:e], k[:, s:e], v[:, s:e], a[:, 2 * s:2 * e], b[:, 2 * s:2 * e], g[:, s:e], 1.0,
                              S0[n:n + 1])
        assert torch.allclose(o[:, s:e], on, atol=1e-12) and torch.allclose(h[n:n + 1], hn, atol=1e-12)


def test_scale_is_a_prescale_of_q():
    q, k, v, a, b, g, S0 = _inp(11)
    o1, _ = O.recurrence(q, k, v, a, b, g, 0.37, S0)
    o2, _ = O.recurrence(0.37 * q, k, v, a, b, g, 1.0, S0)
    assert torch.allclose(o1, o2, atol=1e-12)


def test_gradients_by_finite_differences():
    q, k, v, a, b, g, S0 = _inp(12, B=1, T=5, H=1, K=3, V=2)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, a, b, g, S0)]

    def f(*xs):
        o, h = O.recurrence(*xs[:6], 0.8, xs[6])
        return o, h
    assert torch.autograd.gradcheck(f, leaves, eps=1e-6, atol=1e-6)


def test_golden_fixture_config0():
    """Seeded fixture of benchmark configuration 0 (B1 T256 H2 K=V=64): guards the oracle and the input generator
    against drift.  The reference holds no golden vectors of its own; this one was written by
    tests/golden/make_golden.py from the float64 recurrence."""
    path = os.path.join(os.path.dirname(__file__), "golden", "config0.npz")
    gold = np.load(path)
    inp = make_config(0)
    o, h = O.recurrence(inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, 1.0, None)
    assert np.allclose(o.float().numpy()[:, ::8], gold["o_every8"], rtol=1e-5, atol=1e-6)
    assert np.allclose(h.float().numpy(), gold["final_state"], rtol=1e-5, atol=1e-6)
    assert abs(float(inp.q.double().sum()) - float(gold["q_sum"])) < 1e-6
    assert abs(float(inp.gk.double().sum()) - float(gold["gk_sum"])) < 1e-5
    o2, h2 = O.chunk_naive(inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, 1.0, None, chunk_size=16, dtype=torch.float32)
    assert O.rel_l2(o2, o) < 1e-5 and O.rel_l2(h2, h) < 1e-5


def test_parameterize_a_b_gives_the_two_sided_householder_decay():
    # hdla_custom.py:270-288: with a, b = parameterize_a_b(beta, k, log_f) one step of the recurrence without input
    # (k v^T = 0) multiplies the state by (I - beta k k^T) Diag(f) (I - beta k k^T); recurrence() applies
    # Diag(f) + sum_r b_r a_r^T, so the two must agree for any state (row order r = 0, 1 of a/b included)
    g = torch.Generator().manual_seed(5)
    B, T, H, K, V = 2, 1, 3, 7, 4
    k = torch.randn(B, T, H, K, generator=g, dtype=D)
    k = k / k.norm(dim=-1, keepdim=True)
    beta = 2 * torch.rand(B, T, H, 1, generator=g, dtype=D)
    log_f = -torch.rand(B, T, H, K, generator=g, dtype=D)
    S0 = torch.randn(B, H, K, V, generator=g, dtype=D)
    a, b = O.parameterize_a_b(beta, k, log_f)
    assert a.shape == (B, 2 * T, H, K) and b.shape == a.shape
    zero = torch.zeros(B, T, H, V, dtype=D)
    _, S1 = O.recurrence(torch.zeros_like(k), k, zero, a, b, log_f, 1.0, S0)
    kk = k[:, 0]
    P = torch.eye(K, dtype=D) - beta[:, 0, :, :, None] * kk[..., :, None] * kk[..., None, :]     # I - beta k k^T
    Hm = P @ torch.diag_embed(torch.exp(log_f[:, 0])) @ P
    assert torch.allclose(S1, Hm @ S0, atol=1e-12)
    # [B,T,H] beta is accepted as well, and the two ranks are not interchangeable
    a3, b3 = O.parameterize_a_b(beta[..., 0], k, log_f)
    assert torch.equal(a3, a) and torch.equal(b3, b)
    assert not torch.allclose(a[:, 0], a[:, 1]) and torch.equal(b[:, 1], k[:, 0])


def test_hrdplr_naive_shim_has_the_reference_signature_and_ignores_scale():
    """hrdplr_naive(q, k, v, a, b, gk, scale, initial_state, output_final_state, RANK_AB, head_first, chunk_size)
    (naive.py:76-90): equals the recurrence at scale 1 whatever `scale` is passed (naive.py:83 is never read)."""
    import inspect
    from hdla_hip.synthetic import make_inputs
    assert list(inspect.signature(O.hrdplr_naive).parameters) == [
        "q", "k", "v", "a", "b", "gk", "scale", "initial_state", "output_final_state", "RANK_AB", "head_first", "chunk_size"]
    inp = make_inputs(41, 2, 64, 2, 32, 16, gk_div=1.0)
    t = [x.double() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    o_r, s_r = O.recurrence(*t, 1.0, inp.h0.double())
    for scale in (1.0, 0.25):
        o, s = O.hrdplr_naive(*t, scale, inp.h0.double(), True, 2, False, chunk_size=16)
        assert o.dtype == torch.float64 and O.rel_l2(o, o_r) < 1e-12 and O.rel_l2(s, s_r) < 1e-12
    o, s = O.hrdplr_naive(*t, 1.0, None, False, 2, False, 32)
    assert s is None and o.shape == inp.v.shape

"""The operators under HIP graph capture: the library only launches kernels on the caller's stream (no allocation, no
memset, no synchronisation), so a captured call must replay to exactly what the eager call gives.  Every graph is
replayed several times on fresh input contents, with eager work and synchronisations in between, and every replay is
compared bit for bit with the eager result on the same inputs."""
import pytest
import torch

from hdla_hip import chunk_hdla_delta_rule, chunk_hrdplr_delta_rule, fused_recurrent_hdla_delta_rule, normalize_fn
from hdla_hip.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _capture(fn, warmup=2):
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


def _replay_and_compare(g, static_in, static_out, eager, fresh, n=4):
    for i in range(n):
        new = fresh(i)
        for s, t in zip(static_in, new):
            s.copy_(t)
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        ref = eager(*new)                                     # eager work between replays
        torch.cuda.synchronize()
        for a, b in zip(got, ref):
            assert torch.equal(a, b), f"replay {i} differs from the eager call"


def test_chunked_forward_and_backward_replay():
    B, T, H, K, V = 2, 200, 3, 64, 64
    def fresh(i):
        x = make_inputs(100 + i, B, T, H, K, V)
        return [t.bfloat16().to(DEV) for t in (x.q, x.k, x.v, x.a, x.b, x.gk)] + [x.h0.to(DEV), x.do.bfloat16().to(DEV), x.dht.to(DEV)]

    def run(q, k, v, a, b, gk, h0, do, dht):
        leaves = [t.detach().requires_grad_() for t in (q, k, v, a, b, gk, h0)]
        o, ht = chunk_hrdplr_delta_rule(*leaves[:6], 2, scale=1.0, initial_state=leaves[6], output_final_state=True)
        return [o.detach(), ht.detach()] + list(torch.autograd.grad([o, ht], leaves, [do, dht]))

    static_in = fresh(99)
    g, static_out = _capture(lambda: run(*static_in))
    _replay_and_compare(g, static_in, static_out, run, fresh)


def test_parameterised_operator_and_norm_replay():
    B, T, H, K, V = 1, 130, 4, 128, 128
    def fresh(i):
        x = make_inputs(200 + i, B, T, H, K, V)
        beta = 2 * torch.rand(B, T, H, 1, generator=torch.Generator().manual_seed(i))
        return [t.bfloat16().to(DEV) for t in (x.q, x.k, x.v, beta, x.gk, x.do)]

    w = torch.ones(H * V, device=DEV)

    def run(q, k, v, beta, lf, do):
        leaves = [t.detach().requires_grad_() for t in (q, k, v, beta, lf)]
        wl = w.detach().requires_grad_()
        o, _ = chunk_hdla_delta_rule(*leaves, scale=1.0)
        y = normalize_fn(o.flatten(2), wl, gate=leaves[2].flatten(2), c=(H * V) ** 0.5, eps=1e-5)
        return [y.detach()] + list(torch.autograd.grad(y, leaves + [wl], do.flatten(2)))

    static_in = fresh(99)
    g, static_out = _capture(lambda: run(*static_in))
    _replay_and_compare(g, static_in, static_out, run, fresh)


def test_decode_step_replay_carries_the_state():
    B, H, K, V = 8, 4, 128, 128
    def fresh(i):
        x = make_inputs(300 + i, B, 1, H, K, V)
        beta = 2 * torch.rand(B, 1, H, 1, generator=torch.Generator().manual_seed(i))
        return [t.bfloat16().to(DEV) for t in (x.q, x.k, x.v, beta, x.gk)]

    S = torch.zeros(B, H, K, V, device=DEV)                   # the graph updates its state in place

    def step(q, k, v, beta, lf):
        o, S_new = fused_recurrent_hdla_delta_rule(q, k, v, beta, lf, scale=1.0, initial_state=S, output_final_state=True)
        S.copy_(S_new)
        return [o]

    static_in = fresh(99)
    g, static_out = _capture(lambda: step(*static_in), warmup=1)
    S.zero_()
    S_ref = torch.zeros_like(S)
    for i in range(5):
        new = fresh(i)
        for s, t in zip(static_in, new):
            s.copy_(t)
        g.replay()
        torch.cuda.synchronize()
        o_ref, S_ref = fused_recurrent_hdla_delta_rule(*new, scale=1.0, initial_state=S_ref, output_final_state=True)
        assert torch.equal(static_out[0], o_ref) and torch.equal(S, S_ref), f"decode replay {i}"

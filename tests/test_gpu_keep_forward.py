"""keep_forward=True: the forward pass leaves its per-chunk intermediates for the backward pass (hdla_chunk_fwd_keep /
hdla_chunk_bwd_kept) instead of the backward pass recomputing them from the inputs.  Checked against the float64 oracle
to the same tolerances as the default route, against the classic launch plan without keeping (outputs and every gradient
must be the same bits: the same kernels work on the same bytes, whether the backward pass recomputes them or reads what the
forward pass kept), and through the C ABI for its argument errors."""
import contextlib
import ctypes
import os

import pytest
import torch

from hdla_hip import _lib, chunk_hdla_delta_rule, chunk_hrdplr_delta_rule
from hdla_hip.synthetic import make_config, make_inputs
from oracle import hrdplr_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.bfloat16: (5e-3, 1e-2), torch.float32: (1e-5, 1e-5)}
GRADS = ["dq", "dk", "dv", "da", "db", "dgk", "dh0"]


@contextlib.contextmanager
def _classic_route():
    """The launch plan whose kernels the kept route shares (the default plan may be the fused one)."""
    old = os.environ.get("HDLA_HIP_ROUTE")
    os.environ["HDLA_HIP_ROUTE"] = "classic"
    try:
        yield
    finally:
        if old is None:
            del os.environ["HDLA_HIP_ROUTE"]
        else:
            os.environ["HDLA_HIP_ROUTE"] = old


def _run(inp, dtype, scale, keep, cu=None, use_h0=True):
    leaves = [t.to(dtype).to(DEV).requires_grad_() for t in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    h0 = inp.h0.to(DEV).requires_grad_() if use_h0 else None
    o, ht = chunk_hrdplr_delta_rule(*leaves, 2, scale=scale, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                                    keep_forward=keep)
    g = torch.autograd.grad([o, ht], leaves + ([h0] if use_h0 else []), [inp.do.to(dtype).to(DEV), inp.dht.to(DEV)])
    return o.detach(), ht.detach(), dict(zip(GRADS, g))


def _oracle(inp, dtype, scale, cu=None, use_h0=True):
    leaves = [t.to(dtype).double().requires_grad_() for t in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    h0 = inp.h0.double().requires_grad_() if use_h0 else None
    o, ht = O.recurrence(*leaves, scale, h0, cu_seqlens=cu)
    g = torch.autograd.grad([o, ht], leaves + ([h0] if use_h0 else []), [inp.do.to(dtype).double(), inp.dht.double()])
    return o.detach(), ht.detach(), dict(zip(GRADS, g))


def _check(got, ref, dtype, what):
    tol_o, tol_g = TOL[dtype]
    errs = {"o": O.rel_l2(got[0], ref[0]), "ht": O.rel_l2(got[1], ref[1])}
    errs.update({n: O.rel_l2(got[2][n], ref[2][n]) for n in ref[2]})
    print(what, {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    assert errs["o"] <= tol_o and errs["ht"] <= tol_o, errs
    assert all(errs[n] <= tol_g for n in ref[2]), errs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,H,K,V", [(2, 100, 2, 64, 64), (1, 70, 3, 128, 128), (1, 48, 2, 64, 128), (2, 33, 2, 128, 64)])
def test_kept_route_against_the_oracle_and_the_recomputing_route(dtype, B, T, H, K, V):
    inp = make_inputs(500 + T, B, T, H, K, V, gk_div=2.0)
    kept = _run(inp, dtype, 0.7, True)
    with _classic_route():
        plain = _run(inp, dtype, 0.7, False)
    _check(kept, _oracle(inp, dtype, 0.7), dtype, f"kept {dtype} T{T} K{K} V{V}")
    assert torch.equal(kept[0], plain[0]) and torch.equal(kept[1], plain[1])
    for n in GRADS:
        assert torch.equal(kept[2][n], plain[2][n]), n


def test_kept_route_packed_sequences_strong_decay_and_no_state():
    inp = make_inputs(601, 1, 150, 2, 64, 64, gk_div=1.0, n_states=4)
    inp.gk[..., 7] = -15.0                                       # takes the strong-decay route in every chunk
    cu = torch.tensor([0, 17, 17, 90, 150])
    for dtype in (torch.bfloat16, torch.float32):
        _check(_run(inp, dtype, 1.0, True, cu=cu), _oracle(inp, dtype, 1.0, cu=cu), dtype, f"kept, packed, strong {dtype}")
    inp = make_inputs(602, 2, 40, 2, 64, 64)
    _check(_run(inp, torch.float32, 1.0, True, use_h0=False), _oracle(inp, torch.float32, 1.0, use_h0=False),
           torch.float32, "kept, no initial state")


def test_kept_workspace_serves_repeated_backward_passes_and_is_skipped_without_gradients():
    inp = make_inputs(603, 1, 64, 2, 64, 64)
    leaves = [t.bfloat16().to(DEV).requires_grad_() for t in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    o, _ = chunk_hrdplr_delta_rule(*leaves, 2, scale=1.0, keep_forward=True)
    do = inp.do.bfloat16().to(DEV)
    g1 = torch.autograd.grad(o, leaves, do, retain_graph=True)
    g2 = torch.autograd.grad(o, leaves, do)
    assert all(torch.equal(a, b) for a, b in zip(g1, g2))
    assert o.grad_fn.kept is not None
    with torch.no_grad():
        o2, _ = chunk_hrdplr_delta_rule(*leaves, 2, scale=1.0, keep_forward=True)
    assert torch.equal(o, o2) and o2.grad_fn is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_parameterised_operator_kept_route(dtype):
    g = torch.Generator().manual_seed(9)
    B, T, H, K, V = 2, 90, 2, 64, 128
    q = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=g), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=g), dim=-1)
    v, beta = torch.randn(B, T, H, V, generator=g), 2 * torch.rand(B, T, H, 1, generator=g)
    lf = torch.nn.functional.logsigmoid(torch.randn(B, T, H, K, generator=g)) / 2
    h0, do, dht = torch.randn(B, H, K, V, generator=g), torch.randn(B, T, H, V, generator=g), torch.randn(B, H, K, V, generator=g)
    res = []
    for keep in (True, False):
        leaves = [t.to(dtype).to(DEV).requires_grad_() for t in (q, k, v, beta, lf)] + [h0.to(DEV).requires_grad_()]
        o, ht = chunk_hdla_delta_rule(*leaves[:5], scale=1.0, initial_state=leaves[5], output_final_state=True, keep_forward=keep)
        res.append((o.detach(), ht.detach(), torch.autograd.grad([o, ht], leaves, [do.to(dtype).to(DEV), dht.to(DEV)])))
    ref = [t.to(dtype).double().requires_grad_() for t in (q, k, v, beta, lf)] + [h0.double().requires_grad_()]
    a, b = O.parameterize_a_b(ref[3], ref[1], ref[4])
    o_r, ht_r = O.recurrence(ref[0], ref[1], ref[2], a, b, ref[4], 1.0, ref[5])
    g_r = torch.autograd.grad([o_r, ht_r], ref, [do.to(dtype).double(), dht.double()])
    tol_o, tol_g = TOL[dtype]
    assert O.rel_l2(res[0][0], o_r) <= tol_o and O.rel_l2(res[0][1], ht_r) <= tol_o
    errs = [O.rel_l2(x, y) for x, y in zip(res[0][2], g_r)]
    print("parameterised, kept", dtype, [f"{e:.2e}" for e in errs], flush=True)
    assert max(errs) <= tol_g
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])


def test_config2_full_size_kept_route_matches_the_recomputing_route():
    inp = make_config(2)
    kept = _run(inp, torch.bfloat16, 1.0, True)
    with _classic_route():
        plain = _run(inp, torch.bfloat16, 1.0, False)
    assert torch.equal(kept[0], plain[0]) and torch.equal(kept[1], plain[1])
    assert all(torch.equal(kept[2][n], plain[2][n]) for n in GRADS)


def test_c_abi_rejects_a_short_kept_buffer_and_reports_sizes():
    lib = _lib.load()
    dims = _lib.make_dims(1, 64, 2, 64, 64, 2, 1, torch.bfloat16, torch.bfloat16, 1.0, None, route=_lib.ROUTE_CLASSIC)
    sizes = [lib.hdla_workspace_bytes(ctypes.byref(dims), p) for p in range(5)]
    assert all(s > 0 for s in sizes[:4]) and sizes[4] == 0
    assert sizes[_lib.PASS_FWD_KEEP] > sizes[_lib.PASS_FWD] and sizes[_lib.PASS_BWD_KEPT] < sizes[_lib.PASS_BWD]
    t = [torch.zeros(1, 64 * r, 2, 64, dtype=torch.bfloat16, device=DEV) for r in (1, 1, 1, 2, 2, 1)]
    o = torch.empty_like(t[2])
    small = torch.empty(sizes[_lib.PASS_FWD_KEEP] - 256, dtype=torch.uint8, device=DEV)
    P = _lib.ptr
    rc = lib.hdla_chunk_fwd_keep(ctypes.byref(dims), P(t[0]), P(t[1]), P(t[2]), P(t[3]), P(t[4]), None, P(t[5]), None, P(o),
                                 None, P(small), small.numel(), _lib.current_stream(torch.device(DEV)))
    assert rc == -5

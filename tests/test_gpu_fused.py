"""The fused route of the chunked operator (preparation inside the scan kernels, sequences cut into time segments)
through the C ABI: against the classic route (same bits where there is one segment, to rounding otherwise), against the
float64 recurrence, and the workspace's error word (no wave ever ran out of its bounded wait)."""
import ctypes

import pytest
import torch

from hdla_hip import _lib
from hdla_hip.synthetic import make_inputs
from oracle import hrdplr_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
NAMES = ("q", "k", "v", "a", "b", "gk")


def _dev(inp, gk_dtype=torch.bfloat16):
    x = {n: getattr(inp, n).bfloat16().to(DEV).contiguous() for n in NAMES}
    x["gk"] = getattr(inp, "gk").to(gk_dtype).to(DEV).contiguous()
    x["h0"], x["dht"] = inp.h0.float().to(DEV).contiguous(), inp.dht.float().to(DEV).contiguous()
    x["do"] = inp.do.bfloat16().to(DEV).contiguous()
    return x


def _check_err(ws, dims, pass_):
    off = _lib.workspace_layout(dims, pass_)["ERR"]
    if off >= 0:
        torch.cuda.synchronize()
        word = int(ws[off:off + 4].view(torch.int32).item())
        assert word & ~3 != 0x48444c00, "a wave of the fused kernels ran out of its bounded wait"


def forward(x, route, segments, cu=None, h0=True, boundary=False, scale=0.7):
    lib = _lib.load()
    B, T, H, K = x["q"].shape
    V = x["v"].shape[-1]
    N = B if cu is None else cu.numel() - 1
    dims = _lib.make_dims(B, T, H, K, V, 2, N, torch.bfloat16, x["gk"].dtype, scale, cu, route=route, segments=segments)
    ws = _lib.workspace(dims, 0, DEV)
    o = torch.zeros_like(x["v"])
    ht = torch.empty(N, H, K, V, dtype=torch.float32, device=DEV)
    bnd = _lib.boundary(dims, DEV) if boundary else None
    P = _lib.ptr
    rc = lib.hdla_chunk_fwd_b(ctypes.byref(dims), P(x["q"]), P(x["k"]), P(x["v"]), P(x["a"]), P(x["b"]), None, P(x["gk"]),
                              P(x["h0"]) if h0 else None, P(o), P(ht), P(bnd), 0 if bnd is None else bnd.numel(),
                              P(ws), ws.numel(), _lib.current_stream(torch.device(DEV)))
    _lib.check(rc, "hdla_chunk_fwd_b")
    _check_err(ws, dims, 0)
    return o, ht, bnd


def backward(x, route, segments, cu=None, h0=True, bnd=None, scale=0.7):
    lib = _lib.load()
    B, T, H, K = x["q"].shape
    V = x["v"].shape[-1]
    N = B if cu is None else cu.numel() - 1
    dims = _lib.make_dims(B, T, H, K, V, 2, N, torch.bfloat16, x["gk"].dtype, scale, cu, route=route, segments=segments)
    ws = _lib.workspace(dims, 1, DEV)
    g = {n: torch.zeros_like(x[n]) for n in NAMES}
    dh0 = torch.empty(N, H, K, V, dtype=torch.float32, device=DEV)
    P = _lib.ptr
    rc = lib.hdla_chunk_bwd_b(ctypes.byref(dims), P(x["q"]), P(x["k"]), P(x["v"]), P(x["a"]), P(x["b"]), None, P(x["gk"]),
                              P(x["h0"]) if h0 else None, P(x["do"]), P(x["dht"]), P(g["q"]), P(g["k"]), P(g["v"]),
                              P(g["a"]), P(g["b"]), None, P(g["gk"]), P(dh0), P(bnd), 0 if bnd is None else bnd.numel(),
                              P(ws), ws.numel(), _lib.current_stream(torch.device(DEV)))
    _lib.check(rc, "hdla_chunk_bwd_b")
    _check_err(ws, dims, 1)
    g["h0"] = dh0
    return g


SHAPES = [(2, 200, 3), (1, 16, 1), (1, 5, 2), (3, 1000, 2), (1, 129, 4)]


@pytest.mark.parametrize("B,T,H", SHAPES)
def test_forward_one_segment_against_classic_route(B, T, H):
    x = _dev(make_inputs(21, B, T, H, 64, 64, gk_div=2.0))
    o_c, ht_c, _ = forward(x, _lib.ROUTE_CLASSIC, 0)
    o_f, ht_f, _ = forward(x, _lib.ROUTE_FUSED, 1)
    # (not bit for bit: the fused producers add the two halves of a score tile's sum over channels in another order)
    assert O.rel_l2(o_f, o_c) <= 5e-4 and O.rel_l2(ht_f, ht_c) <= 5e-4


@pytest.mark.parametrize("segments", [2, 3, 4, 8])
@pytest.mark.parametrize("B,T,H", [(2, 200, 3), (1, 1000, 2), (1, 40, 2)])
def test_forward_segments_against_classic_route_and_recurrence(B, T, H, segments):
    inp = make_inputs(22, B, T, H, 64, 64, gk_div=8.0)
    x = _dev(inp)
    o_c, ht_c, _ = forward(x, _lib.ROUTE_CLASSIC, 0)
    o_f, ht_f, bnd = forward(x, _lib.ROUTE_FUSED, segments, boundary=True)
    e_o, e_h = O.rel_l2(o_f, o_c), O.rel_l2(ht_f, ht_c)
    cpu = [getattr(inp, n).bfloat16().double() for n in NAMES]
    o_r, ht_r = O.recurrence(*cpu, 0.7, inp.h0.double())
    r_o, r_h = O.rel_l2(o_f, o_r), O.rel_l2(ht_f, ht_r)
    print(f"segments {segments}: vs classic o {e_o:.2e} ht {e_h:.2e}; vs recurrence o {r_o:.2e} ht {r_h:.2e}", flush=True)
    assert e_o <= 3e-3 and e_h <= 3e-3
    assert r_o <= 5e-3 and r_h <= 5e-3


@pytest.mark.parametrize("segments", [16, 37, 64])
def test_many_segments_forward_and_backward(segments):
    """Long sequences of few heads are cut into up to 64 segments (here: 2 x 3 (sequence, head) pairs, 125 chunks, so
    that 64 segments hold one or two chunks each): both passes against the classic route, with the boundary record and
    without."""
    x = _dev(make_inputs(27, 2, 2000, 3, 64, 64, gk_div=8.0))
    o_c, ht_c, _ = forward(x, _lib.ROUTE_CLASSIC, 0)
    o_f, ht_f, bnd = forward(x, _lib.ROUTE_FUSED, segments, boundary=True)
    assert O.rel_l2(o_f, o_c) <= 3e-3 and O.rel_l2(ht_f, ht_c) <= 3e-3
    g_c = backward(x, _lib.ROUTE_CLASSIC, 0)
    for b in (bnd, None):
        g_f = backward(x, _lib.ROUTE_FUSED, segments, bnd=b)
        errs = {n: O.rel_l2(g_f[n], g_c[n]) for n in g_c}
        print(f"segments {segments} kept {b is not None}:", {k: f"{v:.1e}" for k, v in errs.items()}, flush=True)
        assert all(e <= 6e-3 for e in errs.values()), errs


def test_forward_packed_sequences_and_no_initial_state():
    cu = torch.tensor([0, 37, 37, 500, 516, 1200], dtype=torch.int64)
    inp = make_inputs(23, 1, 1200, 2, 64, 64, gk_div=4.0, n_states=5)
    x = _dev(inp)
    cud = cu.to(DEV)
    for h0 in (True, False):
        o_c, ht_c, _ = forward(x, _lib.ROUTE_CLASSIC, 0, cu=cud, h0=h0)
        o_1, ht_1, _ = forward(x, _lib.ROUTE_FUSED, 1, cu=cud, h0=h0)
        assert O.rel_l2(o_1, o_c) <= 5e-4 and O.rel_l2(ht_1, ht_c) <= 5e-4
        o_f, ht_f, _ = forward(x, _lib.ROUTE_FUSED, 4, cu=cud, h0=h0)
        assert O.rel_l2(o_f, o_c) <= 3e-3 and O.rel_l2(ht_f, ht_c) <= 3e-3


@pytest.mark.parametrize("B,T,H", SHAPES)
def test_backward_one_segment_against_classic_route(B, T, H):
    x = _dev(make_inputs(24, B, T, H, 64, 64, gk_div=2.0))
    g_c = backward(x, _lib.ROUTE_CLASSIC, 0)
    g_f = backward(x, _lib.ROUTE_FUSED, 1)
    for n in g_c:
        assert O.rel_l2(g_f[n], g_c[n]) <= 1e-3, n


@pytest.mark.parametrize("kept", [True, False])
@pytest.mark.parametrize("segments", [2, 4, 8])
@pytest.mark.parametrize("B,T,H", [(2, 200, 3), (1, 1000, 2)])
def test_backward_segments_against_classic_route(B, T, H, segments, kept):
    x = _dev(make_inputs(25, B, T, H, 64, 64, gk_div=8.0))
    g_c = backward(x, _lib.ROUTE_CLASSIC, 0)
    bnd = forward(x, _lib.ROUTE_FUSED, segments, boundary=True)[2] if kept else None
    g_f = backward(x, _lib.ROUTE_FUSED, segments, bnd=bnd)
    errs = {n: O.rel_l2(g_f[n], g_c[n]) for n in g_c}
    print(f"segments {segments} kept {kept}:", {k: f"{v:.1e}" for k, v in errs.items()}, flush=True)
    assert all(e <= 6e-3 for e in errs.values()), errs


def test_backward_packed_sequences_fp32_decay():
    cu = torch.tensor([0, 37, 37, 500, 516, 1200], dtype=torch.int64).to(DEV)
    x = _dev(make_inputs(26, 1, 1200, 2, 64, 64, gk_div=4.0, n_states=5), gk_dtype=torch.float32)
    g_c = backward(x, _lib.ROUTE_CLASSIC, 0, cu=cu)
    g_1 = backward(x, _lib.ROUTE_FUSED, 1, cu=cu)
    for n in g_c:
        assert O.rel_l2(g_1[n], g_c[n]) <= 1e-3, n
    g_f = backward(x, _lib.ROUTE_FUSED, 4, cu=cu)
    errs = {n: O.rel_l2(g_f[n], g_c[n]) for n in g_c}
    assert all(e <= 6e-3 for e in errs.values()), errs


def test_config2_full_size_against_classic_route():
    inp = make_inputs(2, 4, 2048, 16, 64, 64)
    x = _dev(inp)
    o_c, ht_c, _ = forward(x, _lib.ROUTE_CLASSIC, 0, scale=1.0)
    o_f, ht_f, bnd = forward(x, _lib.ROUTE_FUSED, 0, boundary=True, scale=1.0)
    print(f"config 2 forward, fused vs classic: o {O.rel_l2(o_f, o_c):.2e} ht {O.rel_l2(ht_f, ht_c):.2e}", flush=True)
    assert O.rel_l2(o_f, o_c) <= 3e-3 and O.rel_l2(ht_f, ht_c) <= 3e-3
    g_c = backward(x, _lib.ROUTE_CLASSIC, 0, scale=1.0)
    for b in (bnd, None):
        g_f = backward(x, _lib.ROUTE_FUSED, 0, bnd=b, scale=1.0)
        errs = {n: O.rel_l2(g_f[n], g_c[n]) for n in g_c}
        print("config 2 backward, fused vs classic:", {k: f"{v:.1e}" for k, v in errs.items()}, flush=True)
        assert all(e <= 6e-3 for e in errs.values()), errs


@pytest.mark.parametrize("segments", [1, 4])
def test_stage_wise_launches_reproduce_the_single_calls(segments):
    """hdla_chunk_stages on the fused route (what bench.py times kernel by kernel): the stages launched one at a time
    leave the same bits as hdla_chunk_fwd / hdla_chunk_bwd."""
    lib = _lib.load()
    x = _dev(make_inputs(28, 2, 520, 3, 64, 64, gk_div=8.0))
    B, T, H, K = x["q"].shape
    dims = _lib.make_dims(B, T, H, K, 64, 2, B, torch.bfloat16, torch.bfloat16, 0.7, None, route=_lib.ROUTE_FUSED, segments=segments)
    P, stream = _lib.ptr, _lib.current_stream(torch.device(DEV))
    o_1, ht_1, _ = forward(x, _lib.ROUTE_FUSED, segments)
    g_1 = backward(x, _lib.ROUTE_FUSED, segments)                    # no boundary record: the summary pass runs first
    ws = _lib.workspace(dims, 0, DEV)
    o = torch.zeros_like(x["v"])
    ht = torch.empty(B, H, K, 64, dtype=torch.float32, device=DEV)
    g = {n: torch.zeros_like(x[n]) for n in NAMES}
    dh0 = torch.empty(B, H, K, 64, dtype=torch.float32, device=DEV)

    def stage(pass_, mask, w):
        rc = lib.hdla_chunk_stages(ctypes.byref(dims), pass_, mask, P(x["q"]), P(x["k"]), P(x["v"]), P(x["a"]), P(x["b"]), P(x["gk"]),
                                   P(x["h0"]), P(o), P(ht), P(x["do"]), P(x["dht"]), P(g["q"]), P(g["k"]), P(g["v"]), P(g["a"]),
                                   P(g["b"]), P(g["gk"]), P(dh0), P(w), w.numel(), stream)
        _lib.check(rc, "hdla_chunk_stages")
    for mask in ([2, 16] if segments > 1 else [2]):
        stage(0, mask, ws)
    assert torch.equal(o, o_1) and torch.equal(ht, ht_1)
    wb = _lib.workspace(dims, 1, DEV)
    for mask in (([16] if segments > 1 else []) + [2, 4, 8]):
        stage(1, mask, wb)
    _check_err(wb, dims, 1)
    g["h0"] = dh0
    for n in g_1:
        assert torch.equal(g[n], g_1[n]), n

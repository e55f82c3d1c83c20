"""Every intermediate buffer the kernels leave in the workspace, against the stage-by-stage CPU restatement.
With fp32 inputs a wrong index or mask shows as an O(1) error, not as rounding; the bf16 runs cover the code
paths only that type takes (paired 16x16x32 products, packed conversions) at bf16 tolerance."""
import ctypes

import pytest
import torch

import gpu_util as G
from hdla_hip import _lib
from hdla_hip import chunk as CK
from hdla_hip.synthetic import make_inputs
from oracle import chunk_stages as CS
from oracle import hrdplr_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


TOL = {torch.float32: 5e-6, torch.bfloat16: 1e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,H,K,V", [(2, 40, 2, 64, 64), (1, 64, 2, 128, 128), (1, 35, 2, 128, 64), (1, 20, 2, 64, 128)])
def test_workspace_buffers_backward_pass(B, T, H, K, V, dtype, monkeypatch):
    monkeypatch.setenv("HDLA_HIP_ROUTE", "classic")       # the buffers below are those of the four-kernel launch plan
    _backward_buffers(B, T, H, K, V, dtype, None)


@pytest.mark.parametrize("segments", [1, 2, 3])
@pytest.mark.parametrize("B,T,H", [(2, 40, 2), (1, 150, 3)])
def test_workspace_buffers_backward_pass_fused_route(B, T, H, segments, monkeypatch):
    """What the fused kernels leave for chunk_grad: (I - A_ab)^-1, the states and state gradients entering the chunks and
    dv_new, in the same tile formats as the classic route (with several time segments the states are the true ones: the
    checkpoint kernel starts every segment from the chained state).  u is not among them: chunk_grad rebuilds it."""
    monkeypatch.setenv("HDLA_HIP_ROUTE", "fused")
    monkeypatch.setenv("HDLA_HIP_SEGMENTS", str(segments))
    _backward_buffers(B, T, H, 64, 64, torch.bfloat16, ("TM", "HC", "DHC", "DVN"))


def _backward_buffers(B, T, H, K, V, dtype, only):
    scale = 0.7
    inp = make_inputs(11, B, T, H, K, V, gk_div=1.0)
    q, k, v, a, b, gk, do = (x.to(dtype).double() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, inp.do))
    h0, dht = inp.h0.double(), inp.dht.double()
    _, _, _, st = CS.forward_backward(q, k, v, a, b, gk, scale, h0, do, dht)
    d = lambda x: x.to(dtype).to(DEV).contiguous()
    f32 = lambda x: x.float().to(DEV).contiguous()
    out = CK.chunk_hrdplr_bwd(d(q), d(k), d(v), d(a), d(b), d(gk), scale, f32(h0), d(do), f32(dht), keep_workspace=True)
    ws, dims = out[-2], out[-1]
    torch.cuda.synchronize()
    L = _lib.workspace_layout(dims, 1)
    nch, KT, VT = L["nch"], K // 16, V // 16
    SA, SB = L["SA_STRIDE"], L["SB_STRIDE"]
    p, f, r = st["p"], st["f"], st["r"]
    NT = p["q"].shape[2]
    assert nch == B * NT

    def bh(x):                                            # [B,H,NT,...] -> [H, B*NT, ...]
        return x.permute(1, 0, 2, *range(3, x.dim())).reshape(H, B * NT, *x.shape[3:])

    def state(off):
        """Checkpoints of the scans: tiles of the transposed state (rows value, inner channel), pairs along the
        channel tiles, [K/32][V/16][pair] -> [H, nch, K, V]."""
        t = G.pair_tiles(ws, off, dtype, H, nch, KT // 2, VT, 2)          # [.., kp, vt, which, v, k]
        return t.permute(0, 1, 2, 4, 6, 3, 5).reshape(H, nch, K, V)

    def vnew(off):
        """dv_new: tiles of the transposed matrices (rows value, inner token), the two ranks paired,
        [V/16][pair] -> [H, nch, 2, 16, V]."""
        t = G.pair_tiles(ws, off, dtype, H, nch, VT, 2)                   # [.., vt, s, v, token]
        return t.permute(0, 1, 3, 5, 2, 4).reshape(H, nch, 2, 16, V)

    got = {
        "W": lambda: (G.cat_tiles(G.pair_tiles(ws, L["W"], dtype, H, nch, 2, KT, stride=SA), 3), bh(p["w"])),
        "UT": lambda: (G.cat_tiles(G.pair_tiles(ws, L["UT"], dtype, H, nch, VT, 2).transpose(2, 3), 3, transpose=True), bh(p["u"])),
        "KGT": lambda: (G.cat_tiles(G.pair_tiles(ws, L["KGT"], dtype, H, nch, KT, stride=SA), 2, transpose=True), bh(p["kg"])),
        "BGT": lambda: (G.cat_tiles(G.pair_tiles(ws, L["BGT"], dtype, H, nch, 2, KT, stride=SA), 3, transpose=True), bh(p["bg"])),
        "VTT": lambda: (G.cat_tiles(G.tiles(ws, L["VTT"], dtype, H, nch, VT), 2, transpose=True), bh(p["v"])),
        "EGL": lambda: (G.rows(ws, L["EGL"], torch.float32, H, nch, K, stride=SA), bh(torch.exp(p["gl"]))[..., 0, :]),
        "AQBT": lambda: (G.pair_tiles(ws, L["AQBT"], dtype, H, nch, 2, stride=SB), bh(p["Aqb"]).transpose(-1, -2)),
        "QGT": lambda: (G.cat_tiles(G.pair_tiles(ws, L["QGT"], dtype, H, nch, KT, stride=SB), 2, transpose=True), bh(p["qg"])),
        "TM": lambda: (G.pair_tiles(ws, L["TM"], dtype, H, nch, 2, 2), bh(p["Tm"]).transpose(-1, -2)),   # tiles hold the blocks transposed
        "HC": lambda: (state(L["HC"]), bh(f["h"])),
        "DHC": lambda: (state(L["DHC"]), bh(r["dh"])),
        "DVN": lambda: (vnew(L["DVN"]), bh(r["dvn"])),
    }
    errs = {n: O.rel_l2(*xy()) for n, xy in got.items() if only is None or n in only}
    print(dtype, {k: f"{v:.1e}" for k, v in errs.items()}, flush=True)
    assert all(e <= TOL[dtype] for e in errs.values()), errs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,V", [(64, 64), (128, 128)])
def test_workspace_buffers_forward_pass(K, V, dtype):
    scale, B, T, H = 0.7, 1, 48, 2
    inp = make_inputs(12, B, T, H, K, V, gk_div=1.0)
    q, k, v, a, b, gk = (x.to(dtype).double() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk))
    _, _, p, f = CS.forward(q, k, v, a, b, gk, scale, inp.h0.double())
    d = lambda x: x.to(dtype).to(DEV).contiguous()
    lib = _lib.load()
    dims = _lib.make_dims(B, T, H, K, V, 2, B, dtype, dtype, scale, None, route=_lib.ROUTE_CLASSIC)
    ws = _lib.workspace(dims, 0, DEV)
    t = [d(x) for x in (q, k, v, a, b, gk)] + [inp.h0.float().to(DEV).contiguous()]
    o = torch.empty_like(t[2])
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=DEV)
    rc = lib.hdla_chunk_fwd(ctypes.byref(dims), *[_lib.ptr(x) for x in t], _lib.ptr(o), _lib.ptr(ht), _lib.ptr(ws),
                            ws.numel(), _lib.current_stream(DEV))
    torch.cuda.synchronize()
    assert rc == 0
    L = _lib.workspace_layout(dims, 0)
    nch, KT, SA = L["nch"], K // 16, L["SA_STRIDE"]
    NT = p["q"].shape[2]
    bh = lambda x: x.permute(1, 0, 2, *range(3, x.dim())).reshape(H, B * NT, *x.shape[3:])
    errs = {
        "QG": O.rel_l2(G.cat_tiles(G.pair_tiles(ws, L["QG"], dtype, H, nch, KT, stride=SA), 2), bh(p["qg"])),
        "AQK": O.rel_l2(G.tiles(ws, L["AQK"], dtype, H, nch, stride=SA), bh(p["Aqk"])),
        "AQB": O.rel_l2(G.pair_tiles(ws, L["AQB"], dtype, H, nch, 2, stride=SA), bh(p["Aqb"])),
        "o": O.rel_l2(o, CS._unchunk(f["o"], T)),
        "ht": O.rel_l2(ht, f["ht"]),
    }
    print(dtype, {k: f"{v:.1e}" for k, v in errs.items()}, flush=True)
    assert all(e <= TOL[dtype] for e in errs.values()), errs

"""Host side without a GPU: the C-ABI library loads and exports every symbol include/hdla_hip.h declares, its
argument checks return the documented codes before any launch, and the Python operators raise like the reference's."""
import ctypes
import os
import re

import pytest
import torch

import hdla_hip
from hdla_hip import _lib, chunk_hrdplr_delta_rule, fused_recurrent_dplr_delta_rule
from hdla_hip.synthetic import make_inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _dims(**kw):
    d = dict(B=2, T=64, H=2, K=64, V=64, R=2, N=2, in_dtype=torch.bfloat16, gk_dtype=torch.bfloat16, scale=1.0,
             cu_seqlens=None, route=_lib.ROUTE_AUTO, segments=0)
    d.update(kw)
    dims = _lib.make_dims(d["B"], d["T"], d["H"], d["K"], d["V"], d["R"], d["N"], d["in_dtype"], d["gk_dtype"],
                          d["scale"], None, route=d["route"], segments=d["segments"])
    if d["cu_seqlens"] is not None:
        dims.cu_seqlens = d["cu_seqlens"]
    return dims


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "hdla_hip.h")).read()
    names = set(re.findall(r"\b(hdla_[a-z_]+)\s*\(", header))
    assert {"hdla_version", "hdla_strerror", "hdla_workspace_bytes", "hdla_workspace_layout", "hdla_chunk_fwd",
            "hdla_chunk_bwd", "hdla_chunk_stages", "hdla_recurrent_fwd", "hdla_param_chunk_fwd", "hdla_param_chunk_bwd",
            "hdla_param_recurrent_fwd", "hdla_calib_stream", "hdla_normalize_fwd", "hdla_normalize_bwd",
            "hdla_normalize_workspace_bytes", "hdla_layer_pre_fwd", "hdla_layer_pre_bwd", "hdla_logsigmoid_fwd",
            "hdla_logsigmoid_bwd", "hdla_skinny_wgrad", "hdla_skinny_wgrad_workspace_bytes", "hdla_boundary_bytes",
            "hdla_chunk_fwd_b", "hdla_chunk_bwd_b"} <= names
    for n in names:
        assert hasattr(lib, n), n
    assert lib.hdla_version() == _lib.HDLA_VERSION == int(re.search(r"#define HDLA_VERSION (\d+)", header).group(1))
    assert lib.hdla_strerror(0) == b"success"


def test_workspace_size_and_layout():
    lib = _lib.load()
    d = _dims(route=_lib.ROUTE_CLASSIC)
    fwd, bwd = lib.hdla_workspace_bytes(ctypes.byref(d), 0), lib.hdla_workspace_bytes(ctypes.byref(d), 1)
    assert 0 < fwd < bwd
    L = _lib.workspace_layout(d, 1)
    assert L["nch"] == 2 * 4 and L["total"] == bwd
    # the two scan operand blocks come first in each slot order; every buffer starts on a 256-byte boundary
    offs = [L[k] for k in ("W", "BGT", "KGT", "EGL", "UT", "VTT", "QGT", "AQBT", "TM", "HC", "DHC", "DVN")]
    assert offs == sorted(offs) and len(set(offs)) == len(offs) and all(o % 256 == 0 for o in offs)
    K = d.K
    assert L["SA_STRIDE"] % 1024 == 0 and L["SA_STRIDE"] >= 5 * (K // 16) * 512 + 4 * K       # bf16 tiles + fp32 decay
    assert L["SB_STRIDE"] % 1024 == 0 and L["SB_STRIDE"] >= (K // 16 + 2) * 512
    assert L["UT"] - L["W"] >= d.H * L["nch"] * L["SA_STRIDE"] and L["TM"] - L["QGT"] >= d.H * L["nch"] * L["SB_STRIDE"]
    Lf = _lib.workspace_layout(d, 0)
    # the forward block: the backward pass's block as a prefix (same offsets of W, BGT, KGT, EGL), then the output's parts
    assert all(Lf[k] - Lf["W"] == L[k] - L["W"] for k in ("BGT", "KGT", "EGL"))
    assert Lf["EGL"] < Lf["AQK"] < Lf["QG"] < Lf["AQB"] < Lf["W"] + Lf["SA_STRIDE"] and Lf["SB_STRIDE"] == 0
    assert Lf["SA_STRIDE"] > L["SA_STRIDE"]
    # ragged T and packed sequences reserve one extra chunk per sequence
    assert _lib.workspace_layout(_dims(T=65, route=_lib.ROUTE_CLASSIC), 0)["nch"] == 2 * 5
    assert _lib.workspace_layout(_dims(B=1, N=3, T=64, cu_seqlens=256, route=_lib.ROUTE_CLASSIC), 0)["nch"] == 4 + 3
    # a forward pass that keeps its intermediates for the backward pass, and the scratch of that backward pass
    keep, kept = lib.hdla_workspace_bytes(ctypes.byref(d), 2), lib.hdla_workspace_bytes(ctypes.byref(d), 3)
    assert fwd < keep and 0 < kept < bwd and keep + kept > bwd
    Lk, Ls = _lib.workspace_layout(d, 2), _lib.workspace_layout(d, 3)
    assert Lk["SA_STRIDE"] == Lf["SA_STRIDE"] and Lk["TM"] > Lk["AQBT"] > Lk["QGT"] > Lk["VTT"] and Lk["STRONG"] > Lk["TM"]
    assert Ls["HC"] == 0 and Ls["HC"] < Ls["DHC"] < Ls["DVN"] < Ls["total"] == kept
    assert lib.hdla_workspace_bytes(ctypes.byref(d), 4) == 0 and lib.hdla_workspace_bytes(ctypes.byref(d), -1) == 0


def test_routes_workspaces_and_boundary_records():
    lib = _lib.load()
    B = lambda d: lib.hdla_boundary_bytes(ctypes.byref(d))
    W = lambda d, p: lib.hdla_workspace_bytes(ctypes.byref(d), p)
    # bf16 with K = V = 64 takes the fused route unless told otherwise: its scratch holds no scan operands
    big = dict(B=4, N=4, T=2048, H=16)
    auto, classic, fused = _dims(**big), _dims(route=_lib.ROUTE_CLASSIC, **big), _dims(route=_lib.ROUTE_FUSED, **big)
    assert W(auto, 0) == W(fused, 0) < W(classic, 0) / 2 and W(auto, 1) == W(fused, 1) < W(classic, 1)
    L = _lib.workspace_layout(fused, 1)
    assert L["ERR"] >= 0 and L["total"] == W(fused, 1) and L["KGT"] == 0 and 0 < L["HC"] < L["DHC"] < L["DVN"]
    assert _lib.workspace_layout(classic, 1)["ERR"] == -1
    # other shapes have the classic route only
    assert W(_dims(K=128, V=128), 0) == W(_dims(K=128, V=128, route=_lib.ROUTE_CLASSIC), 0) > 0
    assert W(_dims(K=128, V=128, route=_lib.ROUTE_FUSED), 0) == 0
    assert W(_dims(in_dtype=torch.float32, gk_dtype=torch.float32, route=_lib.ROUTE_FUSED), 1) == 0
    assert W(_dims(route=3), 0) == 0 and W(_dims(segments=-1), 0) == 0
    ok = ctypes.c_void_p(4096)
    assert lib.hdla_chunk_fwd(ctypes.byref(_dims(route=7)), ok, ok, ok, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -9
    assert lib.hdla_chunk_fwd(ctypes.byref(_dims(K=128, V=128, route=_lib.ROUTE_FUSED)), ok, ok, ok, ok, ok, ok, None, ok,
                              None, ok, 1 << 40, None) == -9
    # boundary record: one fp32 K x V state per (sequence, head, segment); none for one segment or the classic route
    assert B(classic) == 0 and B(_dims(segments=1)) == 0
    assert B(_dims(segments=4)) == 2 * 2 * 4 * 64 * 64 * 4
    assert B(_dims(segments=100)) == 2 * 2 * 64 * 64 * 64 * 4                    # capped at 64 segments
    # chosen by the library: enough segments to give every compute unit a workgroup, never segments of a few chunks
    assert B(_dims(B=4, N=4, T=2048, H=16)) == 4 * 16 * 4 * 64 * 64 * 4
    assert B(_dims(B=64, N=64, T=2048, H=16)) == 0 and B(_dims(T=64)) == 0
    # a boundary record that is too small or misaligned is refused
    f = lib.hdla_chunk_fwd_b
    d4 = _dims(segments=4)
    assert f(ctypes.byref(d4), ok, ok, ok, ok, ok, None, ok, None, ok, None, ok, 16, ok, 1 << 40, None) == -5
    assert f(ctypes.byref(d4), ok, ok, ok, ok, ok, None, ok, None, ok, None, ctypes.c_void_p(4096 + 8), 1 << 30, ok, 1 << 40, None) == -5


@pytest.mark.parametrize("kw,code", [
    (dict(K=96), -2), (dict(V=32), -2), (dict(R=1), -3), (dict(R=3), -3), (dict(H=0), -2), (dict(T=-1), -2),
    (dict(in_dtype=torch.float32, gk_dtype=torch.bfloat16), -4), (dict(N=3), -7), (dict(B=2, cu_seqlens=256), -7),
])
def test_bad_dims_are_rejected_before_launch(kw, code):
    lib = _lib.load()
    d = _dims(**kw)
    assert lib.hdla_workspace_bytes(ctypes.byref(d), 0) == 0
    one = ctypes.c_void_p(256)
    rc = lib.hdla_chunk_fwd(ctypes.byref(d), one, one, one, one, one, one, None, one, None, one, 1 << 40, None)
    assert rc == code
    assert lib.hdla_recurrent_fwd(ctypes.byref(d), one, one, one, one, one, one, 0, None, one, None, None) == code
    assert len(lib.hdla_strerror(rc)) > 8


def test_null_misaligned_and_small_workspace():
    lib = _lib.load()
    d = _dims()
    ok = ctypes.c_void_p(4096)
    assert lib.hdla_chunk_fwd(ctypes.byref(d), None, ok, ok, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -1
    bad = ctypes.c_void_p(4096 + 8)
    assert lib.hdla_chunk_fwd(ctypes.byref(d), bad, ok, ok, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -6
    assert lib.hdla_chunk_fwd(ctypes.byref(d), ok, ok, ok, ok, ok, ok, None, ok, None, ok, 1024, None) == -5
    assert lib.hdla_chunk_fwd(ctypes.byref(d), ok, ok, ok, ok, ok, ok, None, ok, None, None, 1 << 40, None) == -5
    assert lib.hdla_chunk_fwd(ctypes.byref(d), ok, ok, ok, ok, ok, ok, None, ok, None, ctypes.c_void_p(4096 + 16), 1 << 40, None) == -5
    assert lib.hdla_chunk_bwd(ctypes.byref(d), ok, ok, ok, ok, ok, ok, None, None, None, ok, ok, ok, ok, ok, ok, None,
                              ok, 1 << 40, None) == -1
    assert lib.hdla_workspace_layout(ctypes.byref(d), 0, None) == -1


def test_parameterised_entry_points_check_their_arguments():
    lib = _lib.load()
    d = _dims()
    ok, bad = ctypes.c_void_p(4096), ctypes.c_void_p(4096 + 8)
    f = lib.hdla_param_chunk_fwd
    assert f(ctypes.byref(d), ok, ok, ok, None, ok, None, ok, None, ok, 1 << 40, None) == -1      # beta is required
    assert f(ctypes.byref(d), ok, None, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -1
    assert f(ctypes.byref(d), ok, bad, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -6
    assert f(ctypes.byref(d), ok, ok, ok, ok, ok, None, ok, None, ok, 1024, None) == -5
    assert f(ctypes.byref(_dims(K=96)), ok, ok, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -2
    g = lib.hdla_param_chunk_bwd
    assert g(ctypes.byref(d), ok, ok, ok, ok, ok, None, ok, None, ok, ok, ok, None, ok, None, ok, 1 << 40, None) == -1   # dbeta
    assert g(ctypes.byref(d), ok, ok, ok, ok, ok, None, ok, None, ok, ok, ok, ok, ok, None, None, 1 << 40, None) == -5
    r = lib.hdla_param_recurrent_fwd
    assert r(ctypes.byref(d), ok, ok, ok, None, ok, 0, None, ok, None, None) == -1                    # beta is required
    assert r(ctypes.byref(d), ok, ok, ok, ok, None, 0, None, ok, None, None) == -1
    assert r(ctypes.byref(d), ok, ok, ok, ok, ok, 0, bad, ok, None, None) == -6
    assert r(ctypes.byref(_dims(V=96)), ok, ok, ok, ok, ok, 0, None, ok, None, None) == -2


def test_normalize_entry_points_check_their_arguments():
    lib = _lib.load()
    ok, bad = ctypes.c_void_p(4096), ctypes.c_void_p(4096 + 8)
    nd = lambda **kw: _lib.HdlaNormDims(**{**dict(rows=8, G=1, E=1024, dtype=0, weight_dtype=1, gate_pos=1, c=32.0,
                                                  eps=1e-5), **kw})
    f, b, wsb = lib.hdla_normalize_fwd, lib.hdla_normalize_bwd, lib.hdla_normalize_workspace_bytes
    assert f(ctypes.byref(nd()), None, ok, ok, ok, None) == -1
    assert f(ctypes.byref(nd()), ok, ok, None, ok, None) == -1                       # gate_pos 1 needs a gate
    assert f(ctypes.byref(nd()), ok, ok, bad, ok, None) == -6
    assert f(ctypes.byref(nd(E=1020)), ok, ok, ok, ok, None) == -2                   # groups must start on 16 bytes
    assert f(ctypes.byref(nd(E=32768)), ok, ok, ok, ok, None) == -2                  # longer than one workgroup holds
    assert f(ctypes.byref(nd(dtype=3)), ok, ok, ok, ok, None) == -4
    assert f(ctypes.byref(nd(gate_pos=3)), ok, ok, ok, ok, None) == -2
    assert f(ctypes.byref(nd(rows=0)), None, None, None, None, None) == 0            # nothing to do
    need = wsb(ctypes.byref(nd()))
    assert need > 0 and need % (1024 * 4) == 0 and wsb(ctypes.byref(nd(E=1020))) == 0
    assert wsb(ctypes.byref(nd(rows=1 << 20))) <= 8192 * 4 * 1024 * 4                # bounded however many rows
    assert b(ctypes.byref(nd()), ok, ok, ok, ok, ok, ok, None, ok, need, None) == -1           # weight without dw
    assert b(ctypes.byref(nd()), ok, ok, ok, ok, ok, None, ok, ok, need, None) == -1           # gate without dgate
    assert b(ctypes.byref(nd()), ok, ok, ok, ok, ok, ok, ok, ok, need - 1, None) == -5
    assert b(ctypes.byref(nd()), ok, ok, ok, ok, ok, ok, ok, None, need, None) == -5


def test_layer_pre_entry_points_check_their_arguments():
    lib = _lib.load()
    ok, bad = ctypes.c_void_p(4096), ctypes.c_void_p(4096 + 8)
    pd = lambda **kw: _lib.HdlaPreDims(**{**dict(rows=8, H=16, D=64, dtype=0, ldy=3216, col_q=0, col_k=1024, col_v=2048,
                                                 col_beta=3072, norm_q=0, norm_k=1, norm_v=0, beta_scale=2.0, eps=1e-5),
                                          **kw})
    f, b = lib.hdla_layer_pre_fwd, lib.hdla_layer_pre_bwd
    assert f(ctypes.byref(pd()), None, ok, ok, ok, ok, None) == -1
    assert f(ctypes.byref(pd()), ok, ok, ok, ok, None, None) == -1                   # beta columns given, no beta output
    assert f(ctypes.byref(pd(col_beta=-1)), ok, ok, bad, ok, None, None) == -6
    assert f(ctypes.byref(pd(D=48)), ok, ok, ok, ok, ok, None) == -2                 # 6 lanes a head: not a power of two
    assert f(ctypes.byref(pd(D=1024, H=1)), ok, ok, ok, ok, ok, None) == -2          # more than one wavefront a head
    assert f(ctypes.byref(pd(ldy=3210)), ok, ok, ok, ok, ok, None) == -6             # rows off 16-byte boundaries
    assert f(ctypes.byref(pd(col_k=1028)), ok, ok, ok, ok, ok, None) == -6
    assert f(ctypes.byref(pd(col_v=2200)), ok, ok, ok, ok, ok, None) == -2           # range runs past the row
    assert f(ctypes.byref(pd(col_beta=3208)), ok, ok, ok, ok, ok, None) == -2
    assert f(ctypes.byref(pd(dtype=7)), ok, ok, ok, ok, ok, None) == -4
    assert f(ctypes.byref(pd(rows=0)), None, None, None, None, None, None) == 0
    assert b(ctypes.byref(pd()), ok, ok, ok, ok, None, ok, None) == -1               # dbeta missing
    assert b(ctypes.byref(pd()), ok, ok, ok, ok, ok, None, None) == -1
    lf, lb = lib.hdla_logsigmoid_fwd, lib.hdla_logsigmoid_bwd
    assert lf(0, 12, ok, ok, None) == -2
    assert lf(0, 16, None, ok, None) == -1 and lf(5, 16, ok, ok, None) == -4 and lf(0, 0, None, None, None) == 0
    assert lb(0, 16, ok, None, ok, None) == -1 and lb(0, 16, ok, bad, ok, None) == -6
    sg, sw = lib.hdla_skinny_wgrad, lib.hdla_skinny_wgrad_workspace_bytes
    need = sw(0, 8192, 64, 1024)
    assert need == 8 * 1024 * 64 * 4 and sw(1, 8192, 64, 1024) == 0 and sw(0, 8192, 48, 1024) == 0
    assert sw(0, 5, 128, 64) == 1 * 64 * 128 * 4                                    # fewer rows than one tile: one range
    assert sg(0, 8192, 64, 1024, None, 1024, ok, 64, ok, ok, need, None) == -1
    assert sg(1, 8192, 64, 1024, ok, 1024, ok, 64, ok, ok, need, None) == -4         # bf16 only
    assert sg(0, 8192, 48, 1024, ok, 1024, ok, 48, ok, ok, need, None) == -2
    assert sg(0, 8192, 64, 1000, ok, 1000, ok, 64, ok, ok, need, None) == -2
    assert sg(0, 8192, 64, 1024, ok, 512, ok, 64, ok, ok, need, None) == -2          # row stride shorter than a row
    assert sg(0, 8192, 64, 1024, ok, 1028, ok, 64, ok, ok, need, None) == -6
    assert sg(0, 8192, 64, 1024, ok, 1024, ok, 64, bad, ok, need, None) == -6
    assert sg(0, 8192, 64, 1024, ok, 1024, ok, 64, ok, ok, need - 1, None) == -5
    assert sg(0, 8192, 64, 1024, ok, 1024, ok, 64, ok, None, need, None) == -5


def test_normalize_python_entry_validates_and_needs_a_gpu():
    from hdla_hip import normalize as NZ
    x = torch.randn(4, 64)
    with pytest.raises(NotImplementedError):
        NZ.normalize_fn(x, use_mean=True)
    with pytest.raises(NotImplementedError):
        NZ.normalize_fn(x, bias=torch.zeros(64))
    with pytest.raises(NotImplementedError):
        NZ.normalize_fn(x, gate=x, gate_act="silu")
    with pytest.raises(ValueError):
        NZ.normalize_fn(x, gate=x[:2])
    with pytest.raises(AssertionError):
        NZ.normalize_fn(x, num_groups=3)
    with pytest.raises(_lib.HdlaError):
        NZ.l2_norm(x)                                                   # CPU tensor: no fallback
    assert isinstance(NZ.get_norm_fn("rmsnorm_fused_gate")(64, bias=False, num_groups=2), NZ.RMSNormFusedGate)


def test_parameterised_python_entry_validates_and_needs_a_gpu():
    from hdla_hip import chunk_hdla_delta_rule, fused_recurrent_hdla_delta_rule, parameterize_a_b
    x = make_inputs(3, 2, 32, 2, 64, 64)
    q, k, v, gk = [t.bfloat16() for t in (x.q, x.k, x.v, x.gk)]
    beta = torch.rand(2, 32, 2, 1).bfloat16()
    with pytest.raises(ValueError):
        chunk_hdla_delta_rule(q, k, v, beta[:, :5], gk)
    with pytest.raises(ValueError):
        chunk_hdla_delta_rule(q, k[:, :5], v, beta, gk)
    with pytest.raises(_lib.HdlaError):
        chunk_hdla_delta_rule(q, k, v, beta, gk)                      # CPU tensors: no fallback
    with pytest.raises(ValueError):
        fused_recurrent_hdla_delta_rule(q, k, v, beta[:, :5], gk)
    with pytest.raises(ValueError, match="batch size is expected to be 1"):
        fused_recurrent_hdla_delta_rule(q, k, v, beta, gk, cu_seqlens=torch.tensor([0, 16, 32]))
    with pytest.raises(_lib.HdlaError):
        fused_recurrent_hdla_delta_rule(q, k, v, beta, gk)
    a, b = parameterize_a_b(beta.float(), k.float(), gk.float())       # the reference's helper, with its return
    assert a.shape == (2, 64, 2, 64) and b.shape == a.shape
    assert torch.equal(b[:, 1::2], k.float()) and torch.allclose(a[:, 0::2], -beta.float() * k.float())


def _cpu_args(T=32, K=64, V=64, R=2, B=2):
    x = make_inputs(3, B, T, 2, K, V, R=R)
    return [t.bfloat16() for t in (x.q, x.k, x.v, x.a, x.b, x.gk)], x


def test_python_entry_points_validate_like_the_reference():
    (q, k, v, a, b, gk), x = _cpu_args()
    with pytest.raises(AssertionError):
        chunk_hrdplr_delta_rule(q, k, v, a, b, gk, 2, head_first=True)
    with pytest.raises(AssertionError):
        chunk_hrdplr_delta_rule(q, k.float(), v, a, b, gk, 2)
    with pytest.raises(ValueError):
        chunk_hrdplr_delta_rule(q, k, v, a[:, :-1], b, gk, 2)
    with pytest.raises(ValueError, match="batch size is expected to be 1"):
        chunk_hrdplr_delta_rule(q, k, v, a, b, gk, 2, cu_seqlens=torch.tensor([0, 16, 32]))
    with pytest.raises(ValueError, match="number of initial states"):
        chunk_hrdplr_delta_rule(q[:1], k[:1], v[:1], a[:1], b[:1], gk[:1], 2, initial_state=x.h0,
                                cu_seqlens=torch.tensor([0, 8, 16, 32]))
    with pytest.raises(AssertionError):
        fused_recurrent_dplr_delta_rule(q, k, v, a, b, gk, 2, head_first=True)
    with pytest.raises(ValueError, match="batch size is expected to be 1"):
        fused_recurrent_dplr_delta_rule(q, k, v, a, b, gk, 2, cu_seqlens=torch.tensor([0, 16, 32]))
    with pytest.raises(ValueError, match="a must have 4 dimensions"):
        fused_recurrent_dplr_delta_rule(q, k, v, a[0], b, gk, 2)
    with pytest.raises(AssertionError, match="must be divisible"):
        fused_recurrent_dplr_delta_rule(q, k, v, a[:, :-1], b[:, :-1], gk, 2)
    with pytest.raises(NotImplementedError):
        chunk_hrdplr_delta_rule(q, k, v, torch.cat([a, a[:, :32]], 1), torch.cat([b, b[:, :32]], 1), gk, 3)


def test_chunked_operators_name_the_token_serial_ones_for_head_dimensions_beyond_128():
    from hdla_hip import chunk_hdla_delta_rule
    x = make_inputs(4, 1, 16, 1, 256, 64)
    t = [y.bfloat16() for y in (x.q, x.k, x.v, x.a, x.b, x.gk)]
    with pytest.raises(ValueError, match="maximum 128.*fused_recurrent_dplr_delta_rule"):
        chunk_hrdplr_delta_rule(*t, 2)
    with pytest.raises(ValueError, match="maximum 128"):
        chunk_hdla_delta_rule(t[0], t[1], t[2], torch.ones(1, 16, 1, 1).bfloat16(), t[5])
    x = make_inputs(4, 1, 16, 1, 64, 200)
    t = [y.bfloat16() for y in (x.q, x.k, x.v, x.a, x.b, x.gk)]
    with pytest.raises(ValueError, match="head dimension 200 is not supported.*fused_recurrent_hdla_delta_rule"):
        chunk_hrdplr_delta_rule(*t, 2)


def test_no_cpu_fallback():
    (q, k, v, a, b, gk), _ = _cpu_args()
    with pytest.raises(_lib.HdlaError, match="GPU only"):
        chunk_hrdplr_delta_rule(q, k, v, a, b, gk, 2)
    with pytest.raises(_lib.HdlaError, match="GPU only"):
        fused_recurrent_dplr_delta_rule(q, k, v, a, b, gk, 2)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("HDLA_HIP_LIB", "/nonexistent/libhdla_hip.so")
    with pytest.raises(_lib.HdlaError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_product_code_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "hdla-impl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cuh")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("no CPU or PyTorch fallback", ""), os.path.join(dirpath, f)


def test_recurrent_backward_is_not_implemented():
    class Ctx:
        _fwd_used_autocast = False
        _dtype = torch.float32
    with pytest.raises(NotImplementedError, match="only for inference"):
        hdla_hip.FusedRecurrentDPLRDeltaRuleFunction.backward(Ctx(), None, None)


def test_package_exports_resolve():
    import types
    import hdla_hip
    for name in hdla_hip.__all__:
        assert hasattr(hdla_hip, name), name
    assert isinstance(hdla_hip.layer_pre, types.ModuleType) and callable(hdla_hip.layer_pre.layer_pre)


def test_cu_seqlens_on_the_cpu_is_validated_before_any_launch():
    import torch
    from hdla_hip import _lib
    _lib.check_cu_seqlens(torch.tensor([0, 3, 3, 10]), 10)
    for bad in ([1, 5, 10], [0, 5, 9], [0, 7, 5, 10], [0, 5, 12], [-2, 10]):
        with pytest.raises(ValueError):
            _lib.check_cu_seqlens(torch.tensor(bad), 10)
    with pytest.raises(ValueError):
        _lib.check_cu_seqlens(torch.tensor([[0, 10]]), 10)
    with pytest.raises(ValueError):
        _lib.check_cu_seqlens(torch.tensor([0]), 0)

"""hdla_hip.normalize_fn (HIP kernels through the C ABI) against oracle/normalize_oracle.py in float64 with autograd:
relative L2 <= 1e-5 for fp32 tensors; for bf16 tensors <= 5e-3 on outputs and <= 1e-2 on gradients (the bf16 rounding
of the stored result is 2^-9 relative per element)."""
import pytest
import torch

from hdla_hip import normalize as NZ
from oracle import hrdplr_oracle as O
from oracle import normalize_oracle as NO

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.bfloat16: (5e-3, 1e-2), torch.float32: (1e-5, 1e-5)}


def _rand(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def _run(dtype, shape, G, use_w, gate_pos, c, eps, seed, w_dtype=torch.float32):
    D = shape[-1]
    x, gate, w, do = _rand(seed, *shape), _rand(seed + 1, *shape), 1.0 + 0.3 * _rand(seed + 2, D), _rand(seed + 3, *shape)
    xs = x.to(dtype)
    gs = gate.to(dtype) if gate_pos else None
    ws = w.to(w_dtype) if use_w else None
    # oracle on the rounded inputs
    leaves = [t.double().requires_grad_() for t in (xs, gs, ws) if t is not None]
    it = iter(leaves)
    xo = next(it)
    go = next(it) if gs is not None else None
    wo = next(it) if ws is not None else None
    ro = NO.normalize(xo, wo, go, "sigmoid", gate_pos or "pre", c=c, eps=eps, num_groups=G)
    rg = torch.autograd.grad(ro, leaves, do.to(dtype).double())
    # HIP
    dl = [t.to(DEV).requires_grad_() for t in (xs, gs, ws) if t is not None]
    it = iter(dl)
    xd = next(it)
    gd = next(it) if gs is not None else None
    wd = next(it) if ws is not None else None
    o = NZ.normalize_fn(xd, wd, gate=gd, gate_pos=gate_pos or "pre", c=c, eps=eps, num_groups=G)
    assert o.dtype == dtype and o.shape == xs.shape
    g = torch.autograd.grad(o, dl, do.to(dtype).to(DEV))
    names = ["dx"] + (["dgate"] if gs is not None else []) + (["dw"] if ws is not None else [])
    errs = {"o": O.rel_l2(o, ro)}
    errs.update({n: O.rel_l2(a, b) for n, a, b in zip(names, g, rg)})
    for a, l in zip(g, dl):
        assert a.dtype == l.dtype and a.shape == l.shape
    return errs


CASES = [
    # dtype, shape, G, weight, gate_pos, c, eps
    (torch.bfloat16, (4, 64, 1024), 1, True, "pre", 32.0, 1e-5),       # the layer's gated RMS norm, 16 heads x 64
    (torch.bfloat16, (2, 33, 2048), 1, True, "post", 2048 ** 0.5, 1e-5),
    (torch.bfloat16, (3, 17, 4096), 1, True, "pre", 64.0, 1e-5),       # largest row one wavefront holds
    (torch.bfloat16, (2, 9, 8192), 1, True, "pre", 8192 ** 0.5, 1e-5),  # a workgroup per row, four pieces a lane
    (torch.bfloat16, (11, 16384), 1, True, "post", 128.0, 1e-5),       # largest bf16 row
    (torch.bfloat16, (6, 10240), 2, True, "pre", 5120 ** 0.5, 1e-5),   # two long groups a row, ragged over 256 lanes
    (torch.bfloat16, (2, 50, 16, 64), 1, False, None, 1.0, 1e-5),      # l2_norm of a [B,T,H,K] tensor
    (torch.bfloat16, (2, 50, 3, 128), 1, False, None, 1.0, 1e-5),
    (torch.bfloat16, (1, 77, 768), 12, True, "pre", 8.0, 1e-5),        # group rms norm, 12 groups of 64
    (torch.bfloat16, (5, 1, 96), 1, True, None, 96 ** 0.5, 1e-6),      # 12 pieces over 16 lanes
    (torch.bfloat16, (9, 1000), 5, True, "post", 200 ** 0.5, 1e-5),    # 25 pieces over 32 lanes, groups not a power of two
    (torch.float32, (4, 31, 1024), 1, True, "pre", 32.0, 1e-5),
    (torch.float32, (2, 10, 2048), 1, True, "post", 2048 ** 0.5, 1e-6),
    (torch.float32, (3, 40, 4, 64), 1, False, None, 1.0, 1e-5),
    (torch.float32, (2, 19, 512), 8, True, "pre", 8.0, 1e-5),
    (torch.float32, (7, 36), 3, True, None, 12 ** 0.5, 1e-5),
    (torch.float32, (5, 3, 4096), 1, True, "pre", 64.0, 1e-5),
    (torch.float32, (4, 8192), 1, False, None, 1.0, 1e-5),
]


@pytest.mark.parametrize("dtype,shape,G,use_w,gate_pos,c,eps", CASES)
def test_against_the_oracle(dtype, shape, G, use_w, gate_pos, c, eps):
    errs = _run(dtype, shape, G, use_w, gate_pos, c, eps, seed=sum(shape))
    print(dtype, shape, G, use_w, gate_pos, {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    tol_o, tol_g = TOL[dtype]
    assert errs.pop("o") <= tol_o
    for n, e in errs.items():
        assert e <= tol_g, (n, e)


def test_weight_in_bf16_and_many_rows():
    errs = _run(torch.bfloat16, (8192, 1024), 1, True, "pre", 32.0, 1e-5, seed=5, w_dtype=torch.bfloat16)
    print("8192 x 1024, bf16 weight", {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    assert errs["o"] <= 5e-3 and errs["dx"] <= 1e-2 and errs["dgate"] <= 1e-2
    assert errs["dw"] <= 1e-2          # returned in the weight's dtype


def test_empty_and_single_row():
    x = torch.empty(0, 64, device=DEV, dtype=torch.bfloat16)
    assert NZ.l2_norm(x).shape == (0, 64)
    w = torch.ones(64, device=DEV, requires_grad=True)
    xe = torch.empty(0, 64, device=DEV, requires_grad=True)
    NZ.normalize_fn(xe, w, c=8.0).sum().backward()
    assert torch.equal(w.grad, torch.zeros_like(w.grad))
    errs = _run(torch.float32, (1, 64), 1, True, "pre", 8.0, 1e-5, seed=9)
    assert max(errs.values()) <= 1e-5


def test_modules_match_their_formula():
    x, g = _rand(1, 2, 24, 512).to(DEV), _rand(2, 2, 24, 512).to(DEV)
    m = NZ.get_norm_fn("rmsnorm_fused_gate")(512, bias=False, gate_act="sigmoid", gate_pos="pre", num_groups=8).to(DEV)
    with torch.no_grad():
        m.weight.copy_(1.0 + 0.1 * _rand(3, 512))
    ref = NO.rms_norm_fused_gate(x.cpu(), g.cpu(), m.weight.detach().cpu(), eps=1e-5)
    assert O.rel_l2(m(x, g), ref) <= 1e-5
    gm = NZ.get_norm_fn("grouprmsnorm_fused_gate")(512, bias=False, gate_act="sigmoid", gate_pos="post", num_groups=8).to(DEV)
    ref = NO.normalize(x.cpu(), gm.weight.detach().cpu(), g.cpu(), "sigmoid", "post", c=8.0, eps=1e-5, num_groups=8)
    assert O.rel_l2(gm(x, g), ref) <= 1e-5
    assert O.rel_l2(NZ.RMSNorm(512).to(DEV)(x), NO.normalize(x.cpu(), c=512 ** 0.5, eps=1e-5)) <= 1e-5
    assert O.rel_l2(NZ.l2_norm(x.half()), NO.l2_norm(x.half().cpu(), eps=1.6e-5)) <= 1e-3
    with pytest.raises(NotImplementedError):
        NZ.get_norm_fn("layernorm")

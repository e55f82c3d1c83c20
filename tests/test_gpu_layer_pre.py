"""hdla_hip.layer_pre (the layer's elementwise stage as HIP kernels, through the C ABI) against the same steps in float64
torch (silu, sigmoid and logsigmoid are the library's; the l2 normalisation is oracle/normalize_oracle.py) with autograd:
relative L2 <= 1e-5 in fp32, <= 5e-3 (outputs) / 1e-2 (gradients) in bf16."""
import pytest
import torch
import torch.nn.functional as F

from hdla_hip import layer_pre as LP
from oracle import hrdplr_oracle as O
from oracle import normalize_oracle as NO

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.bfloat16: (5e-3, 1e-2), torch.float32: (1e-5, 1e-5)}


def _ref(y, H, D, cq, ck, cv, cb, ct, nq, nk, nv, scale):
    rows = y.shape[0]
    take = lambda c: F.silu(y[:, c:c + H * D]).reshape(rows, H, D)
    q, k, v = take(cq), take(ck), take(cv)
    q = NO.l2_norm(q) if nq else q
    k = NO.l2_norm(k) if nk else k
    v = NO.l2_norm(v) if nv else v
    beta = scale * torch.sigmoid(y[:, cb:cb + H]).unsqueeze(-1) if cb >= 0 else None
    tail = y[:, ct:] if ct < y.shape[1] else None
    return q, k, v, beta, tail


@pytest.mark.parametrize("dtype,rows,H,D,layout,flags", [
    (torch.bfloat16, 300, 16, 64, "layer", (False, True, False)),        # the layer's default: q | k | v | beta | tail
    (torch.bfloat16, 77, 4, 128, "layer", (True, True, True)),
    (torch.bfloat16, 50, 3, 32, "gaps", (False, True, False)),           # permuted ranges with unused columns between
    (torch.bfloat16, 1, 2, 512, "nobeta", (True, False, True)),          # widest head: 64 lanes
    (torch.float32, 123, 8, 64, "layer", (False, True, False)),
    (torch.float32, 40, 2, 128, "gaps", (True, True, False)),
    (torch.float32, 9, 5, 16, "nobeta", (False, True, True)),
])
def test_layer_pre_against_torch(dtype, rows, H, D, layout, flags):
    hd = H * D
    if layout == "layer":
        cq, ck, cv, cb, ct = 0, hd, 2 * hd, 3 * hd, 3 * hd + H
        ldy = ct + 2 * D + (-(ct + 2 * D)) % 8
    elif layout == "gaps":
        cv, cq, ck = 8, hd + 24, 2 * hd + 40
        cb, ct = 3 * hd + 48, 3 * hd + 48 + H + 5
        ldy = ct + 19 + (-(ct + 19)) % 8
    else:
        cq, ck, cv, cb = 0, hd, 2 * hd, -1
        ct = ldy = 3 * hd
    g = torch.Generator().manual_seed(rows + H)
    y = (2.0 * torch.randn(rows, ldy, generator=g)).to(dtype)
    nq, nk, nv = flags
    yo = y.double().requires_grad_()
    ref = _ref(yo, H, D, cq, ck, cv, cb, ct, nq, nk, nv, 2.0)
    yd = y.to(DEV).requires_grad_()
    got = LP.layer_pre(yd, H, D, cq, ck, cv, cb, ct, (ldy - ct,) if ct < ldy else (), nq, nk, nv, 2.0)
    got = tuple(got) + (None,) * (5 - len(got))
    cot = [torch.randn(t.shape, generator=g).to(dtype) if t is not None else None for t in ref]
    live = [i for i, t in enumerate(ref) if t is not None]
    (dref,) = torch.autograd.grad([ref[i] for i in live], yo, [cot[i].double() for i in live])
    (dgot,) = torch.autograd.grad([got[i] for i in live], yd, [cot[i].to(DEV) for i in live])
    tol_o, tol_g = TOL[dtype]
    for i, name in enumerate(["q", "k", "v", "beta", "tail"]):
        if ref[i] is None:
            assert got[i] is None
            continue
        assert got[i].dtype == dtype and got[i].shape == ref[i].shape and got[i].is_contiguous()
        e = O.rel_l2(got[i], ref[i])
        assert e <= tol_o, (name, e)
    e = O.rel_l2(dgot, dref)
    print(dtype, rows, H, D, layout, f"dy {e:.2e}", flush=True)
    assert e <= tol_g
    if layout == "gaps":                                   # columns no range covers get a zero gradient
        used = torch.zeros(ldy, dtype=torch.bool)
        for c in (cq, ck, cv):
            used[c:c + hd] = True
        used[cb:cb + H] = True
        used[ct:] = True
        assert float(dgot[:, ~used.to(DEV)].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_logsigmoid(dtype):
    g = torch.Generator().manual_seed(0)
    x = torch.cat([6 * torch.randn(4000, generator=g), torch.tensor([-200.0, -90.0, -30.0, 0.0, 30.0, 90.0, 200.0, 1e-3])]).to(dtype)
    x = x.reshape(3, -1)
    do = torch.randn(x.shape, generator=g).to(dtype)
    xo = x.double().requires_grad_()
    ro = F.logsigmoid(xo)
    (rg,) = torch.autograd.grad(ro, xo, do.double())
    xd = x.to(DEV).requires_grad_()
    o = LP.logsigmoid(xd)
    (gd,) = torch.autograd.grad(o, xd, do.to(DEV))
    assert o.dtype == dtype and torch.isfinite(o).all() and torch.isfinite(gd).all()
    tol_o, tol_g = TOL[dtype]
    assert O.rel_l2(o, ro) <= tol_o and O.rel_l2(gd, rg) <= tol_g
    # the decay it feeds: exp(log_f) = sigmoid(x) to the same tolerance where it matters (|x| moderate)
    small = x.abs() <= 30
    assert O.rel_l2(torch.exp(o.double().cpu())[small], torch.sigmoid(x.double())[small]) <= tol_o


def test_empty_input():
    y = torch.empty(0, 3 * 128 + 8, device=DEV, dtype=torch.bfloat16)
    q, k, v, beta, t0, t1 = LP.layer_pre(y, 2, 64, 0, 128, 256, 384, 386, (2, 4), False, True, False, 2.0)
    assert q.shape == (0, 2, 64) and beta.shape == (0, 2, 1) and t0.shape == (0, 2) and t1.shape == (0, 4)
    assert LP.logsigmoid(torch.empty(0, 8, device=DEV)).shape == (0, 8)


@pytest.mark.parametrize("M,N,K,strided", [(8192, 64, 1024, True), (100, 64, 128, False), (33, 128, 512, True),
                                              (1, 128, 4096, False), (4097, 64, 2048, False), (70000, 64, 64, False)])
def test_low_rank_up_weight_gradient_against_float64_matmul(M, N, K, strided):
    """hdla_skinny_wgrad through LowRankUpFunction's backward: dW = dY^T @ X0 against the float64 product of the same
    bf16 operands; the result is rounded to bf16 once (2^-9 relative per element)."""
    g = torch.Generator().manual_seed(M + N)
    dy = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(K, N, generator=g) / K ** 0.5).bfloat16()
    x0 = torch.randn(M, N, generator=g).bfloat16()
    wd = w.to(DEV).requires_grad_()
    if strided:                                             # the layer's case: x0 is a column range of a wider tensor
        wide = torch.cat([x0, x0 + 1], dim=1).to(DEV).requires_grad_()
        xd = wide[:, :N]
    else:
        xd = x0.to(DEV).requires_grad_()
    y = LP.low_rank_up(xd, wd)
    assert torch.equal(y, F.linear(xd, wd))
    gx, gw = torch.autograd.grad(y, [xd, wd], dy.to(DEV))
    rx, rw = dy.double() @ w.double(), dy.double().T @ x0.double()
    ex, ew = O.rel_l2(gx, rx), O.rel_l2(gw, rw)
    print(M, N, K, f"dx0 {ex:.2e} dw {ew:.2e}", flush=True)
    assert gw.dtype == torch.bfloat16 and gw.shape == (K, N) and gx.shape == (M, N)
    assert ex <= 3e-3 and ew <= 3e-3
    # exactness on small integers: every partial and final sum is an integer that fp32 and bf16 hold exactly
    picked = torch.arange(0, M, max(1, M // 7))[:7]          # at most seven non-zero rows spread over the row ranges
    a = torch.zeros(M, K)
    a[picked] = torch.randint(-2, 3, (len(picked), K), generator=g).float()
    b = torch.randint(-2, 3, (M, N), generator=g).float()
    yi = LP.low_rank_up(b.bfloat16().to(DEV), wd)
    (gi,) = torch.autograd.grad(yi, wd, a.bfloat16().to(DEV))
    assert torch.equal(gi.float().cpu(), a.T @ b)

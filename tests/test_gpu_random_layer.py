"""Seeded sweep over shapes and options of the kernels around the operator (normalisation, the layer's pre kernels, the
weight-gradient kernel) against their float64 references; same tolerances as the fixed cases in test_gpu_normalize.py
and test_gpu_layer_pre.py."""
import random

import pytest
import torch
import torch.nn.functional as F

from hdla_hip import layer_pre as LP
from hdla_hip import normalize as NZ
from oracle import hrdplr_oracle as O
from oracle import normalize_oracle as NO

pytestmark = pytest.mark.gpu
DEV = "cuda"
E_UNITS = [1, 2, 3, 5, 8, 13, 16, 31, 64, 100, 128, 129, 255, 256, 257, 511, 512, 513, 700, 1024, 1025, 2047, 2048]


@pytest.mark.parametrize("seed", range(4))
def test_normalize_sweep(seed):
    rnd = random.Random(seed)
    done = 0
    while done < 12:
        dtype = rnd.choice([torch.bfloat16, torch.float32])
        n = 8 if dtype == torch.bfloat16 else 4
        G, E = rnd.choice([1, 1, 1, 2, 3, 4, 6, 7, 12, 16, 20]), n * rnd.choice(E_UNITS)
        if E > (16384 if dtype == torch.bfloat16 else 8192) or G * E > 40000:
            continue
        rows = min(rnd.choice([1, 2, 3, 7, 17, 64, 100, 333, 1000, 4097]), max(1, int(3e6 // (G * E))))
        use_w, gp = rnd.random() < 0.7, rnd.choice([None, "pre", "post"])
        g = torch.Generator().manual_seed(seed * 1000 + done)
        x, gate, do = (torch.randn(rows, G * E, generator=g).to(dtype) for _ in range(3))
        w = 1 + 0.3 * torch.randn(G * E, generator=g)
        pick = lambda f: [f(x)] + ([f(gate)] if gp else []) + ([f(w)] if use_w else [])
        lo, ld = pick(lambda t: t.double().requires_grad_()), pick(lambda t: t.to(DEV).requires_grad_())
        ro = NO.normalize(lo[0], lo[-1] if use_w else None, lo[1] if gp else None, "sigmoid", gp or "pre", c=E ** 0.5,
                          eps=1e-5, num_groups=G)
        o = NZ.normalize_fn(ld[0], ld[-1] if use_w else None, gate=ld[1] if gp else None, gate_pos=gp or "pre",
                            c=E ** 0.5, eps=1e-5, num_groups=G)
        rg, gg = torch.autograd.grad(ro, lo, do.double()), torch.autograd.grad(o, ld, do.to(DEV))
        errs = [O.rel_l2(o, ro)] + [O.rel_l2(a, b) for a, b in zip(gg, rg)]
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
        assert max(errs) <= tol, (dtype, rows, G, E, use_w, gp, errs)
        done += 1


@pytest.mark.parametrize("seed", range(3))
def test_layer_pre_sweep(seed):
    rnd = random.Random(100 + seed)
    for case in range(10):
        dtype = rnd.choice([torch.bfloat16, torch.float32])
        n = 8 if dtype == torch.bfloat16 else 4
        D, H = n * rnd.choice([1, 2, 4, 8, 16, 32, 64]), rnd.choice([1, 2, 3, 5, 16, 33])
        hd = H * D
        rows = min(rnd.choice([1, 2, 5, 63, 64, 65, 500, 3000]), max(1, int(2e6 // hd)))
        use_b = rnd.random() < 0.7
        tw = rnd.choice([(), (n,), (3, 5), (D, D)])
        ct = 3 * hd + (H if use_b else 0)
        ldy = ct + sum(tw)
        if ldy % n:
            tw, ldy = tw + ((-ldy) % n,), ldy + (-ldy) % n
        flags = [rnd.random() < 0.5 for _ in range(3)]
        g = torch.Generator().manual_seed(seed * 1000 + case)
        y = (2 * torch.randn(rows, ldy, generator=g)).to(dtype)
        yo, yd = y.double().requires_grad_(), y.to(DEV).requires_grad_()
        ref = [F.silu(yo[:, c:c + hd]).reshape(rows, H, D) for c in (0, hd, 2 * hd)]
        ref = [NO.l2_norm(t) if f else t for t, f in zip(ref, flags)]
        if use_b:
            ref.append(torch.sigmoid(yo[:, 3 * hd:3 * hd + H]).unsqueeze(-1))
        c = ct
        for wd in tw:
            ref.append(yo[:, c:c + wd])
            c += wd
        got = [t for t in LP.layer_pre(yd, H, D, 0, hd, 2 * hd, 3 * hd if use_b else -1, ct, tw, *flags, 1.0)
               if t is not None]
        assert len(got) == len(ref)
        cot = [torch.randn(t.shape, generator=g).to(dtype) for t in ref]
        (dr,) = torch.autograd.grad(ref, yo, [t.double() for t in cot])
        (dg,) = torch.autograd.grad(got, yd, [t.to(DEV) for t in cot])
        errs = [O.rel_l2(a, b) for a, b in zip(got, ref)] + [O.rel_l2(dg, dr)]
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
        assert max(errs) <= tol, (dtype, rows, H, D, use_b, tw, flags, errs)


def test_weight_gradient_sweep():
    rnd = random.Random(7)
    for case in range(16):
        M, N = rnd.choice([1, 15, 16, 17, 100, 1000, 4096, 9999, 30000]), rnd.choice([64, 128])
        K = 64 * rnd.choice([1, 2, 3, 8, 16, 33, 64])
        M = min(M, int(2e7 // K))
        g = torch.Generator().manual_seed(2000 + case)
        dy, x0, w = (torch.randn(*s, generator=g).bfloat16() for s in ((M, K), (M, N), (K, N)))
        wd = w.to(DEV).requires_grad_()
        (gw,) = torch.autograd.grad(LP.low_rank_up(x0.to(DEV), wd), wd, dy.to(DEV))
        assert O.rel_l2(gw, dy.double().T @ x0.double()) <= 3e-3, (M, N, K)

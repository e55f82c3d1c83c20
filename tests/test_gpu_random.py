"""A seeded sweep over shapes and options of the chunked operator (packed and ragged batches, with and without
initial state and final-state gradient, weak to strong decay, both input types), each case against the float64
recurrence with the stated tolerances.  The fixed cases elsewhere pin particular code paths; this one looks for the
combination nobody thought of."""
import random

import pytest
import torch

from hdla_hip.synthetic import make_inputs
from test_gpu_chunk import _compare, _gpu, _oracle

pytestmark = pytest.mark.gpu


def _case(rng):
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    K, V = rng.choice([64, 128]), rng.choice([64, 128])
    H = rng.choice([1, 2, 3, 5, 16, 17, 33, 40, 70])
    if rng.random() < 0.4:
        lens = [rng.choice([0, 1, 5, 16, 17, 31, 48, 100]) for _ in range(rng.randint(1, 5))]
        if sum(lens) == 0:
            lens[0] = 7
        B, T, N = 1, sum(lens), len(lens)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int64)
    else:
        B, T, cu = rng.randint(1, 3), rng.choice([1, 2, 15, 16, 17, 47, 96, 97, 130, 200]), None
        N = B
    return dict(dtype=dtype, B=B, T=T, H=H, K=K, V=V, N=N, cu=cu, use_h0=rng.random() < 0.7, use_dht=rng.random() < 0.7,
                gk_div=rng.choice([1.0, 2.0, 16.0]), scale=rng.choice([1.0, 0.5, K ** -0.5]))


@pytest.mark.parametrize("seed", range(4))
def test_random_cases(seed):
    rng = random.Random(1000 + seed)
    for it in range(10):
        c = _case(rng)
        inp = make_inputs(10000 + 100 * seed + it, c["B"], c["T"], c["H"], c["K"], c["V"], gk_div=c["gk_div"], n_states=c["N"])
        heads = sorted({0, c["H"] // 2, c["H"] - 1})
        what = (f"seed {seed} case {it}: {c['dtype']} B{c['B']} T{c['T']} H{c['H']} K{c['K']} V{c['V']} "
                f"cu={None if c['cu'] is None else c['cu'].tolist()} h0={c['use_h0']} dht={c['use_dht']} gk/{c['gk_div']}")
        got = _gpu(inp, c["dtype"], c["scale"], use_h0=c["use_h0"], use_dht=c["use_dht"], cu=c["cu"])
        ref = _oracle(inp, c["dtype"], c["scale"], heads=heads, use_h0=c["use_h0"], use_dht=c["use_dht"], cu=c["cu"])
        _compare(got, ref, c["dtype"], heads=heads, what=what)


@pytest.mark.parametrize("seed", range(3))
def test_random_packed_batches_strong_decay_and_kept_forward(seed, monkeypatch):
    """Packed batches of up to 40 sequences (some empty, no particular order), a share of the log-decays strong enough
    for the strong-decay route, table on the CPU or on the GPU: the default launch plan against the float64 recurrence,
    and the route that keeps the forward pass's intermediates bit for bit the same as the classic launch plan that
    recomputes them."""
    from hdla_hip import chunk_hrdplr_delta_rule
    from oracle import hrdplr_oracle as O
    rng = random.Random(2000 + seed)
    for it in range(8):
        dtype = rng.choice([torch.bfloat16, torch.float32])
        K, V, H = rng.choice([64, 128]), rng.choice([64, 128]), rng.choice([1, 2, 3])
        N = rng.choice([2, 3, 5, 9, 20, 40])
        lens = [rng.choice([0, 1, 5, 15, 16, 17, 31, 33, 48]) for _ in range(N)]
        if sum(lens) == 0:
            lens[0] = 7
        T = sum(lens)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int64)
        inp = make_inputs(20000 + 100 * seed + it, 1, T, H, K, V, gk_div=rng.choice([16.0, 4.0, 1.0]), n_states=N)
        gk = inp.gk
        if rng.random() < 0.5:
            g = torch.Generator().manual_seed(it)
            gk = torch.where(torch.rand(1, T, H, K, generator=g) < 0.08, -60 * torch.rand(1, T, H, K, generator=g), gk)
        use_h0, use_dht, scale = rng.random() < 0.7, rng.random() < 0.7, rng.choice([1.0, 0.5])
        cu_arg = cu.to("cuda") if rng.random() < 0.5 else cu

        def run(keep):
            leaves = [x.to(dtype).to("cuda").requires_grad_() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, gk)]
            h0 = inp.h0.to("cuda").requires_grad_() if use_h0 else None
            o, ht = chunk_hrdplr_delta_rule(*leaves, 2, scale=scale, initial_state=h0, output_final_state=True,
                                            cu_seqlens=cu_arg, keep_forward=keep)
            outs, gos = [o], [inp.do.to(dtype).to("cuda")]
            if use_dht:
                outs.append(ht); gos.append(inp.dht.to("cuda"))
            return [o, ht] + list(torch.autograd.grad(outs, leaves + ([h0] if use_h0 else []), gos))

        got, kept = run(False), run(True)
        what = f"seed {seed} case {it}: {dtype} H{H} K{K} V{V} lens={lens} h0={use_h0} dht={use_dht}"
        # the kept route shares its kernels with the classic launch plan (the default plan may be the fused one)
        monkeypatch.setenv("HDLA_HIP_ROUTE", "classic")
        classic = run(False)
        monkeypatch.delenv("HDLA_HIP_ROUTE")
        assert all(torch.equal(a, b) for a, b in zip(classic, kept)), what
        lv = [x.to(dtype).double().requires_grad_() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, gk)]
        h0r = inp.h0.double().requires_grad_() if use_h0 else None
        o_r, ht_r = O.recurrence(*lv, scale, h0r, cu_seqlens=cu)
        outs, gos = [o_r], [inp.do.to(dtype).double()]
        if use_dht:
            outs.append(ht_r); gos.append(inp.dht.double())
        ref = [o_r, ht_r] + list(torch.autograd.grad(outs, lv + ([h0r] if use_h0 else []), gos))
        tol_o, tol_g = (5e-3, 1e-2) if dtype == torch.bfloat16 else (1e-5, 1e-5)
        for i, (a, b) in enumerate(zip(got, ref)):
            assert torch.isfinite(a.float()).all(), what
            e = O.rel_l2(a, b)
            assert e <= (tol_o if i < 2 else tol_g), f"{what}: output {i} error {e:.2e}"

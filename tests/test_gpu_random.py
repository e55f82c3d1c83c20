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

"""Seeded synthetic inputs for the five benchmark configurations of the HDLA hot path.

One CPU generator seeded ``1000 + cfg`` draws, in fp32 and in this fixed order, q, k, v, b_0, beta_0, b_1, beta_1,
gk, h0, do, dht, so that a CPU checker and the GPU path see identical values.  q and k are L2-normalised over K,
each b_r is a unit vector and a_r = -beta_r * b_r with beta_r ~ U(0, 2) (the Householder-style parameterisation
of HRDPLR/hdla_custom.py:270-288), a/b are interleaved rank-fastest to [B, 2T, H, K] (HRDPLR/hdla_custom.py:39-43)
and gk = logsigmoid(N(0,1)) / 16.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

# (B, T, H, K, V) of the five configurations; config 3 is a packed batch of four sequences,
# config 4 is one decode step (1024 of them are timed).
CONFIG_SHAPES = {
    0: (1, 256, 2, 64, 64),
    1: (4, 2048, 16, 64, 64),
    2: (4, 2048, 16, 64, 64),
    3: (1, 16384, 16, 128, 128),
    4: (256, 1, 32, 128, 128),
}
CONFIG3_CU_SEQLENS = (0, 2048, 6144, 10240, 16384)


@dataclass
class Inputs:
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    a: torch.Tensor
    b: torch.Tensor
    gk: torch.Tensor
    h0: torch.Tensor
    do: torch.Tensor
    dht: torch.Tensor
    cu_seqlens: Optional[torch.Tensor] = None

    def to(self, device=None, dtype=None) -> "Inputs":
        """Move to ``device``; cast q,k,v,a,b,gk,do to ``dtype`` (states and their gradients stay fp32)."""
        def mv(x, cast):
            if x is None:
                return None
            if cast and dtype is not None:
                x = x.to(dtype)
            return x.to(device) if device is not None else x
        return Inputs(mv(self.q, True), mv(self.k, True), mv(self.v, True), mv(self.a, True), mv(self.b, True),
                      mv(self.gk, True), mv(self.h0, False), mv(self.do, True), mv(self.dht, False),
                      mv(self.cu_seqlens, False))


def make_inputs(seed: int, B: int, T: int, H: int, K: int, V: int, R: int = 2, n_states: Optional[int] = None,
                h0_std: float = 1.0, gk_div: float = 16.0) -> Inputs:
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    q = F.normalize(rn(B, T, H, K), dim=-1)
    k = F.normalize(rn(B, T, H, K), dim=-1)
    v = rn(B, T, H, V)
    a_r, b_r = [], []
    for _ in range(R):
        bb = F.normalize(rn(B, T, H, K), dim=-1)
        beta = 2.0 * torch.rand(B, T, H, 1, generator=g, dtype=torch.float32)
        b_r.append(bb)
        a_r.append(-beta * bb)
    a = torch.stack(a_r, dim=2).reshape(B, T * R, H, K)
    b = torch.stack(b_r, dim=2).reshape(B, T * R, H, K)
    gk = F.logsigmoid(rn(B, T, H, K)) / gk_div
    N = B if n_states is None else n_states
    h0 = rn(N, H, K, V) * h0_std
    do = rn(B, T, H, V)
    dht = rn(N, H, K, V)
    return Inputs(q, k, v, a, b, gk, h0, do, dht)


def make_config(cfg: int, shape: Optional[Tuple[int, int, int, int, int]] = None) -> Inputs:
    """Inputs of benchmark configuration ``cfg`` (0-4); ``shape`` overrides (B,T,H,K,V) for reduced-size parity runs."""
    B, T, H, K, V = shape if shape is not None else CONFIG_SHAPES[cfg]
    if cfg == 3:
        cu = torch.tensor(CONFIG3_CU_SEQLENS, dtype=torch.int64)
        if shape is not None:
            cu = (cu * T) // CONFIG3_CU_SEQLENS[-1]
        inp = make_inputs(1000 + cfg, B, T, H, K, V, n_states=len(cu) - 1)
        inp.cu_seqlens = cu
        return inp
    if cfg == 4:
        return make_inputs(1000 + cfg, B, T, H, K, V, h0_std=0.1)
    return make_inputs(1000 + cfg, B, T, H, K, V)

"""CPU restatement of the reference's fused normalisation (TEST INFRASTRUCTURE ONLY: imported by tests/ and by
bench.py's cpu_baseline leg, never by the product path).

It follows the Triton kernel the HDLA layer actually runs, ``_normalize_fwd``
(HRDPLR/normalizations/normalize/normalize/normalize_triton.py:21-125), reached through ``NormOp``
(HRDPLR/normalizations/utils.py:9-74), ``RMSNormFusedGate`` (HRDPLR/normalizations/rms_norm.py:48-90) and ``l2_norm``
(HRDPLR/normalizations/l2_norm.py:4-14):

    x' = x * act(gate)                        (gate given, gate_pos == "pre";   normalize_triton.py:84-89)
    sigma = sqrt(sum_e x'^2 / E + eps)        per (row, group) of E = D / num_groups channels   (:103)
    o = (c / sqrt(E)) * x' / sigma * weight   (:104-109)
    o = o * act(gate)                         (gate_pos == "post";  :116-117)

Note that the file beside it, ``normalize_torch.py:76-77``, puts eps elsewhere (sqrt(sum x^2 + eps)); the layer imports
the Triton one (``normalize/__init__.py:9``), so that is what is restated.  Only what the HDLA layer can reach is
covered: no mean subtraction, bias or residual; gate activation "sigmoid" (the activation table lives in the ``xopes``
package, a dependency that is not part of the reference tree).

Gradients come from autograd through this float64 code.  Pins (tests/test_oracle_normalize.py): with c = sqrt(E) the
ungated form is the library's ``torch.nn.functional.rms_norm``; ``l2_norm`` tends to ``F.normalize`` as eps -> 0 and
equals x / sqrt(|x|^2 + E eps) exactly; grouping equals the ungrouped call on a reshaped tensor; a large eps separates
the two eps placements.
"""
from typing import Optional

import torch


def normalize(x: torch.Tensor, weight: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
              gate_act: str = "sigmoid", gate_pos: str = "pre", c: float = 1.0, eps: float = 1e-6,
              num_groups: int = 1, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """normalize_triton.py:21-125 for use_mean = False, no bias, no residual; result in ``dtype``."""
    assert gate_act == "sigmoid" and gate_pos in ("pre", "post")
    D = x.shape[-1]
    assert D % num_groups == 0
    E = D // num_groups
    x = x.to(dtype)
    g = None if gate is None else torch.sigmoid(gate.to(dtype))
    if g is not None and gate_pos == "pre":
        x = x * g
    xg = x.reshape(*x.shape[:-1], num_groups, E)
    sigma = torch.sqrt((xg * xg).sum(-1, keepdim=True) / E + eps)
    o = (c / E ** 0.5) * xg / sigma
    if weight is not None:
        o = o * weight.to(dtype).reshape(num_groups, E)
    o = o.reshape(x.shape)
    if g is not None and gate_pos == "post":
        o = o * g
    return o


def l2_norm(x: torch.Tensor, eps: float = 1e-5, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """HRDPLR/normalizations/l2_norm.py:4-14: c = 1, one group over the last dimension."""
    return normalize(x, c=1.0, eps=eps, dtype=dtype)


def rms_norm_fused_gate(x: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5,
                        gate_act: str = "sigmoid", gate_pos: str = "pre", dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """RMSNormFusedGate.forward, HRDPLR/normalizations/rms_norm.py:74-88: NormOp("rmsnorm") sets c = sqrt(dim) and
    one group (normalizations/utils.py:35-39)."""
    return normalize(x, weight, gate, gate_act, gate_pos, c=x.shape[-1] ** 0.5, eps=eps, dtype=dtype)

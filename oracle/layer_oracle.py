"""CPU restatement of the HDLA layer's forward pass (TEST INFRASTRUCTURE ONLY: imported by tests/, never by the
product path).  Follows ``HDLA_Custom.forward``, HRDPLR/hdla_custom.py:191-350, line by line in float64 torch, on a
``state_dict`` with the reference's parameter names; the recurrence, the parameterisation and the normalisations are the
oracles of the neighbouring files (each pinned by its own tests), so what this file adds is the wiring: projections,
activations, head and block rearrangements, the left-padding mask, the state hand-over and the output path.

Pins of the wiring (tests/test_oracle_layer.py): causality and the chunk-free definition (the output at token t equals a
fresh run on the prefix); a split run that carries the state equals one run; ``num_blocks = 1`` with one head reduces
to the plain single-head formula written out in the test; masked tokens leave the state untouched.
"""
from typing import Callable, Dict, Optional, Tuple

import torch
import torch.nn.functional as F

from . import hrdplr_oracle as O
from . import normalize_oracle as NO


def _linear(sd: Dict[str, torch.Tensor], name: str, x: torch.Tensor) -> torch.Tensor:
    y = x @ sd[name + ".weight"].double().T
    if name + ".bias" in sd:
        y = y + sd[name + ".bias"].double()
    return y


def hdla_layer(sd: Dict[str, torch.Tensor], x: torch.Tensor, num_heads: int, *, num_blocks: int = 1,
               use_output_gate: bool = True, beta_activation: str = "neg", norm_q: bool = False, norm_v: bool = False,
               gate_pos: str = "pre", attention_mask: Optional[torch.Tensor] = None, q_offset: int = 0,
               initial_state: Optional[torch.Tensor] = None, act=F.silu, eps: float = 1e-5,
               rounding: Optional[Callable[[torch.Tensor, str], torch.Tensor]] = None
               ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (output [b, n, d], final state [b, H, K, V]) in float64.  ``sd``: q_proj, k_proj, v_proj, f_proj.0/1,
    bet_proj (absent: beta = 2), o_proj, norm.weight, output_gate.0/1, offset (optional).

    ``rounding(t, stage)`` (optional) is applied to what each stage of a module hands to the next -- stage "proj": the
    outputs of the projections; "pre": q, k, v, beta, log_f as the operator receives them; "op": the operator's output;
    "norm": the gated norm's output; "out": the layer's output -- so that a test can measure what storing these in a
    narrow type costs by itself, stage by stage (the default rounds nothing)."""
    rnd = (lambda t, stage: t) if rounding is None else rounding

    def _lin(sd_, name, x_):                                 # projections hand over rounded results
        return rnd(_linear(sd_, name, x_), "proj")
    x = x.double()
    b, n, d = x.shape
    D = d // num_heads
    q, k, v = _lin(sd, "q_proj", x), _lin(sd, "k_proj", x), _lin(sd, "v_proj", x)          # hdla_custom.py:206-208
    f = _lin(sd, "f_proj.1", _lin(sd, "f_proj.0", x))                                      # :209-212
    if "offset" in sd:
        f = f + sd["offset"].double()
    log_f = rnd(F.logsigmoid(f), "pre")                                                     # :219
    if "bet_proj.weight" in sd:
        beta = torch.sigmoid(_lin(sd, "bet_proj", x)).unsqueeze(-1)                         # :221-224
        if beta_activation == "neg":
            beta = beta * 2
        beta = rnd(beta, "pre")
    else:
        beta = torch.full((b, n, num_heads, 1), 2.0, dtype=torch.float64)                   # :226
    q, k, v = act(q), act(k), act(v)                                                        # :228-230
    q, k, v, log_f = (t.reshape(b, n, num_heads, D) for t in (q, k, v, log_f))             # :233-236
    if num_blocks > 1:                                                                      # :238-245
        nb = num_blocks
        q, k, log_f = (t.reshape(b, n, num_heads * nb, D // nb) for t in (q, k, log_f))
        v = v.repeat_interleave(nb, dim=2)
        beta = beta.repeat_interleave(nb, dim=2)
    if norm_q:
        q = NO.l2_norm(q)                                                                   # :247-251
    k = NO.l2_norm(k)
    if norm_v:
        v = NO.l2_norm(v)
    q, k, v = rnd(q, "pre"), rnd(k, "pre"), rnd(v, "pre")
    if attention_mask is not None and not bool(attention_mask.all()) and n > 1:            # :259-267
        keep = (attention_mask[:, q_offset:] != 0).unsqueeze(-1).unsqueeze(-1)
        k = torch.where(keep, k, torch.zeros_like(k))
        log_f = torch.where(keep, log_f, torch.zeros_like(log_f))
    a, bb = O.parameterize_a_b(beta, k, log_f)                                              # :290
    h0 = None if initial_state is None else initial_state.double()
    o, S = O.recurrence(q, k, v, a, bb, log_f, 1.0, h0)                                     # :296-323, scale = 1
    o = rnd(o, "op")
    if num_blocks > 1:
        o = o.reshape(b, n, num_heads, num_blocks, -1).sum(-2)                              # :326-329
    o = o.reshape(b, n, d)                                                                  # :340
    w = sd["norm.weight"].double()
    if use_output_gate:                                                                     # :341-345
        gate = _lin(sd, "output_gate.1", _lin(sd, "output_gate.0", x))
        o = NO.rms_norm_fused_gate(o, gate, w, eps=eps, gate_pos=gate_pos)
    else:
        o = NO.normalize(o, w, c=d ** 0.5, eps=eps)
    o = rnd(o, "norm")
    return rnd(_linear(sd, "o_proj", o), "out"), S                                       # :348

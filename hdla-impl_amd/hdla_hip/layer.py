"""The HDLA token mixer built on this library's operators: the drop-in for ``HDLA_Custom``, HRDPLR/hdla_custom.py:45-350.

Same constructor arguments, parameter names (so a reference ``state_dict`` loads), forward signature and return value
``(output, past_key_values)``.  What runs on the GPU:

* projections: the BLAS library through torch, as in the reference (hdla_custom.py:206-213), but with everything
  that multiplies x gathered into one GEMM
* activations, head split, per-head l2 normalisation of q, k, v, beta and the log decay: two kernels each way
  (``hdla_hip.layer_pre``; hdla_custom.py:214-251) in the default configuration (silu activations, one block);
  otherwise, or with ``fuse_pre=False``, torch's elementwise operators and ``hdla_hip.normalize.l2_norm``
* the gated RMS norm after the operator: ``hdla_hip.normalize`` (hdla_custom.py:341-345)
* the recurrence: ``chunk_hdla_delta_rule`` / ``fused_recurrent_hdla_delta_rule``, which form a and b from
  (beta, k, log_f) inside the kernels; the reference calls ``parameterize_a_b`` first (hdla_custom.py:290, a function
  that as shipped returns nothing) and hands a, b to the plain operators (:296-323).  ``fuse_ab=False`` takes that
  route with the working helper.

Which operator runs: the reference uses the chunked one when training or when ``use_cache`` is set and the token-serial
one otherwise (hdla_custom.py:295,310); ``dispatch="reference"`` keeps that.  The default ``dispatch="auto"`` uses the
chunked operator when gradients are needed or the call carries more than 8 tokens and the token-serial one for shorter
calls (decode steps, short bursts), which is where each is the faster (at 8 tokens they take the same time from
B=1, H=16 to B=256, H=32; at 1 token the token-serial one is 1.5-2.3x faster, at 64 tokens the chunked one 3x); both
compute the same function.

``past_key_values`` is duck-typed on the three calls the reference makes (hdla_custom.py:254-257, 332-337):
``len(cache)``, ``cache[layer_idx]["recurrent_state"][0]``, ``cache.get_seq_length(layer_idx)`` and
``cache.update(recurrent_state=[S], layer_idx=i, offset=n)``; ``RecurrentCache`` below is a minimal one.
"""
import math
from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .chunk import chunk_hrdplr_delta_rule
from . import layer_pre as _pre
from .hdla import chunk_hdla_delta_rule, fused_recurrent_hdla_delta_rule, parameterize_a_b
from .normalize import get_norm_fn, l2_norm
from .recurrent import fused_recurrent_dplr_delta_rule

EMBED_DIM_BASE = 256                 # HRDPLR/normalizations/normalization_utils.py:14
RECURRENT_BELOW = 9                  # dispatch="auto": calls shorter than this run token by token (measured crossover: 8)


def get_activation_fn(activation: str) -> Callable[[torch.Tensor], torch.Tensor]:
    """HRDPLR/activations.py:10-58."""
    table = {
        "gelu": F.gelu, "relu": F.relu, "elu": F.elu, "sigmoid": torch.sigmoid, "exp": torch.exp, "leak": F.leaky_relu,
        "relu2": lambda x: F.relu(x) ** 2, "1+elu": lambda x: 1 + F.elu(x), "2+elu": lambda x: 2 + F.elu(x),
        "swish": F.silu, "silu": F.silu, "softmax_1": lambda x: F.softmax(x, dim=-1),
        "softmax_2": lambda x: F.softmax(x, dim=-2),
    }
    return table.get(activation, lambda x: x)


class RecurrentCache:
    """The part of fla's ``Cache`` the layer touches: one state list and a token count per layer."""

    def __init__(self):
        self.states, self.seen = [], []

    def __len__(self):
        return len(self.states)

    def __getitem__(self, layer_idx):
        return self.states[layer_idx]

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self.seen[layer_idx] if layer_idx < len(self.seen) else 0

    def update(self, recurrent_state=None, layer_idx: int = 0, offset: int = 1, **kwargs):
        while len(self.states) <= layer_idx:
            self.states.append({"recurrent_state": [None]})
            self.seen.append(0)
        self.states[layer_idx] = {"recurrent_state": recurrent_state}
        self.seen[layer_idx] += offset
        return self.states[layer_idx]


class HDLA_Custom(nn.Module):
    """S[t] = (I - beta k k^T) Diag(f) (I - beta k k^T) S[t-1] + k v^T,  o[t] = S[t]^T q[t]   (hdla_custom.py:46-62,270-288)."""

    def __init__(
        self,
        embed_dim: int,
        num_heads: int,
        bias: bool = False,
        layer_idx: int = 0,
        use_output_gate: bool = True,
        token_mixer_norm_type: str = "rmsnorm",
        q_activation: str = "silu",
        k_activation: str = "silu",
        v_activation: str = "silu",
        use_beta: bool = True,
        beta_activation: str = "neg",
        qkv_norm_type: int = 2,
        norm_q: bool = False,
        norm_v: bool = False,
        causal: bool = True,
        max_position_embeddings: int = 1024,
        token_mixer_init_type: int = 4,
        rescale_type: int = 2,
        num_hidden_layers: int = 12,
        init_std: float = 0.02,
        gain: float = 0.01,
        gate_act: str = "sigmoid",
        gate_pos: str = "pre",
        threshold: float = 0.99,
        use_offset: bool = False,
        num_blocks: int = 1,
        fuse_ab: bool = True,
        dispatch: str = "auto",
        fuse_pre: bool = True,
        **kwargs,
    ):
        super().__init__()
        assert causal, f"Only causal={causal} is supported"
        assert dispatch in ("auto", "reference")
        self.layer_idx, self.causal, self.use_output_gate = layer_idx, causal, use_output_gate
        self.q_proj = nn.Linear(embed_dim, embed_dim, bias=bias)
        self.k_proj = nn.Linear(embed_dim, embed_dim, bias=bias)
        self.v_proj = nn.Linear(embed_dim, embed_dim, bias=bias)
        self.head_dim = embed_dim // num_heads
        self.f_proj = nn.Sequential(nn.Linear(embed_dim, self.head_dim, bias=bias),
                                    nn.Linear(self.head_dim, embed_dim, bias=bias))
        self.use_beta = use_beta
        if use_beta:
            self.bet_proj = nn.Linear(embed_dim, num_heads, bias=bias)
        self.o_proj = nn.Linear(embed_dim, embed_dim, bias=bias)
        self.q_act, self.k_act, self.v_act = (get_activation_fn(a) for a in (q_activation, k_activation, v_activation))
        self.beta_activation = beta_activation
        norm_type = f"{token_mixer_norm_type}_fused_gate" if use_output_gate else token_mixer_norm_type
        self.norm = get_norm_fn(norm_type)(embed_dim, bias=bias, gate_act=gate_act, gate_pos=gate_pos,
                                           num_groups=num_heads)
        if use_output_gate:
            self.output_gate = nn.Sequential(nn.Linear(embed_dim, self.head_dim, bias=bias),
                                             nn.Linear(self.head_dim, embed_dim, bias=bias))
        self.embed_dim, self.num_heads = embed_dim, num_heads
        self.use_offset, self.threshold = use_offset, threshold
        self.qkv_norm_type, self.norm_q, self.norm_v = qkv_norm_type, norm_q, norm_v
        self.token_mixer_init_type, self.rescale_type = token_mixer_init_type, rescale_type
        self.num_hidden_layers, self.init_std, self.gain = num_hidden_layers, init_std, gain
        self.num_blocks = num_blocks
        self.fuse_ab, self.dispatch, self.fuse_pre = fuse_ab, dispatch, fuse_pre
        self._all_silu = all(a in ("silu", "swish") for a in (q_activation, k_activation, v_activation))
        self._init_weights()

    # ---- initialisation: hdla_custom.py:159-187 and normalization_utils.py:115-211 (the branches a module of this
    # layer can reach: Linear weights, the decay offset, the rescaling of o_proj) ------------------------------------
    def _init_weights(self):
        self.setup_decay()
        self.apply(self._initialize_weights)

    def setup_decay(self):
        if not self.use_offset:
            return
        a = self.threshold                                   # sigmoid(offset) = threshold at f_proj(x) = 0
        offset = torch.ones(self.embed_dim) * math.log(a / (1 - a))
        if hasattr(self, "offset"):
            self.offset.data.copy_(offset)
        else:
            self.offset = nn.Parameter(offset, requires_grad=True)

    def _initialize_weights(self, module):
        if getattr(module, "_is_hf_initialized", False):
            return
        if self.token_mixer_init_type in (1, 2, 3, 4):
            gain = {1: 2 ** -2.5, 2: 2 ** -0.5, 3: self.init_std / ((self.embed_dim / EMBED_DIM_BASE) ** 0.5),
                    4: self.gain}[self.token_mixer_init_type]
            if isinstance(module, nn.Linear):
                nn.init.xavier_uniform_(module.weight, gain=gain)
                if module.bias is not None:
                    nn.init.zeros_(module.bias)
        for name, p in module.named_parameters():
            if name in ("o_proj.weight", "out_proj.weight"):
                with torch.no_grad():
                    if self.rescale_type == 1:
                        p /= math.sqrt(2 * self.num_hidden_layers)
                    elif self.rescale_type == 2:
                        p *= 0
        module._is_hf_initialized = True

    def extra_repr(self):
        return (f"embed_dim={self.embed_dim}, num_heads={self.num_heads}, num_blocks={self.num_blocks}, "
                f"fuse_ab={self.fuse_ab}, dispatch={self.dispatch}")

    def _gathered(self, heads):
        """Weights (and biases) of the projections of x, concatenated.  With gradients, or in training mode, the
        concatenation is rebuilt per call (and is part of the graph).  In evaluation mode without gradients it is built
        once and reused: it is rebuilt when a parameter is replaced or modified in place (tracked by its version
        counter), on ``.train()`` / ``.eval()``, ``.to()`` and ``load_state_dict``, and by ``reset_cache()`` -- which
        is what code that writes through ``param.data`` (untracked) has to call."""
        ps = [m.weight for m in heads] + ([m.bias for m in heads] if heads[0].bias is not None else [])
        if self.training or (torch.is_grad_enabled() and any(p.requires_grad for p in ps)):
            w = torch.cat([m.weight for m in heads], dim=0)
            return w, (torch.cat([m.bias for m in heads], dim=0) if heads[0].bias is not None else None)
        key = tuple((p.data_ptr(), p._version, p.dtype, p.device) for p in ps)
        if getattr(self, "_gathered_key", None) != key:
            with torch.no_grad():
                w = torch.cat([m.weight for m in heads], dim=0)
                b = torch.cat([m.bias for m in heads], dim=0) if heads[0].bias is not None else None
            self._gathered_key, self._gathered_val = key, (w, b)
        return self._gathered_val

    def reset_cache(self):
        """Forget the concatenated projection weight of evaluation mode."""
        self._gathered_key = self._gathered_val = None

    def train(self, mode: bool = True):
        self.reset_cache()
        return super().train(mode)

    def _apply(self, fn, *args, **kwargs):
        self.reset_cache()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self.reset_cache()
        return super()._load_from_state_dict(*args, **kwargs)

    def _up(self, lin: nn.Linear, x0: torch.Tensor) -> torch.Tensor:
        """Second half of a low-rank projection (head_dim -> embed_dim)."""
        if self.fuse_pre and lin.bias is None and x0.is_cuda and x0.dtype == torch.bfloat16 == lin.weight.dtype:
            return _pre.low_rank_up(x0, lin.weight)
        return lin(x0)

    # ---- the part of forward() before the recurrence (hdla_custom.py:202-267) --------------------------------------
    def project(self, x, attention_mask=None, q_offset=0, lower_bound=None):
        """x [b, n, d] -> q, k, v [b, n, H, D], beta [b, n, H, 1], log_f [b, n, H, D] with H = num_heads * num_blocks,
        and the inner activations of the output gate [b, n, head_dim] (None without a gate)."""
        b, n, d = x.shape
        # every projection of x in one GEMM (q, k, v, beta, the first halves of the decay and gate projections): one
        # read of x forward, one GEMM each for dx and dW backward instead of six and their sums
        heads = [self.q_proj, self.k_proj, self.v_proj]
        if self.use_beta:
            heads.append(self.bet_proj)
        heads.append(self.f_proj[0])
        if self.use_output_gate:
            heads.append(self.output_gate[0])
        w, bias = self._gathered(heads)
        y = F.linear(x, w, bias)
        ldy, hd = y.shape[-1], self.head_dim
        if (self.fuse_pre and self._all_silu and self.num_blocks == 1 and lower_bound is None and x.is_cuda
                and _pre.supported(y.dtype, hd, ldy, (d, 2 * d, 3 * d))):
            # activations, head split, l2 normalisation and beta in one kernel each way; its backward pass writes the
            # gradient of y in place
            col_tail = 3 * d + (self.num_heads if self.use_beta else 0)
            q, k, v, beta, f0, *rest = _pre.layer_pre(
                y.reshape(b * n, ldy), self.num_heads, hd, 0, d, 2 * d, 3 * d if self.use_beta else -1, col_tail,
                (hd, hd) if self.use_output_gate else (hd,), self.norm_q, True, self.norm_v,
                2.0 if self.beta_activation == "neg" else 1.0)
            q, k, v = (t.view(b, n, self.num_heads, hd) for t in (q, k, v))
            beta = beta.view(b, n, self.num_heads, 1) if self.use_beta else x.new_full((b, n, self.num_heads, 1), 2.0)
            f = self._up(self.f_proj[1], f0).view(b, n, d)
            if self.use_offset:
                f = f + self.offset
            log_f = _pre.logsigmoid(f).view(b, n, self.num_heads, hd)
            gate0 = rest[0].view(b, n, hd) if self.use_output_gate else None
            if attention_mask is not None and not attention_mask.all() and n > 1:        # left padding
                keep = attention_mask[:, q_offset:].unsqueeze(-1).unsqueeze(-1) != 0
                k = k.masked_fill(~keep, 0)
                log_f = log_f.masked_fill(~keep, 0)
            return q, k, v, beta, log_f, gate0
        parts = dict(zip([id(m) for m in heads], y.split([m.out_features for m in heads], dim=-1)))
        q, k, v, f0 = (parts[id(m)] for m in (self.q_proj, self.k_proj, self.v_proj, self.f_proj[0]))
        gate0 = parts[id(self.output_gate[0])] if self.use_output_gate else None
        f = self.f_proj[1](f0)
        if self.use_offset:
            f = f + self.offset
        if lower_bound is not None:
            log_f = torch.log(lower_bound + (1 - lower_bound) * torch.sigmoid(f))
        else:
            log_f = F.logsigmoid(f)
        if self.use_beta:
            beta = torch.sigmoid(parts[id(self.bet_proj)]).unsqueeze(-1)
            if self.beta_activation == "neg":
                beta = beta * 2
        else:
            beta = x.new_full((b, n, self.num_heads, 1), 2.0)
        q, k, v = self.q_act(q), self.k_act(k), self.v_act(v)
        q, k, v, log_f = (t.unflatten(-1, (-1, self.head_dim)) for t in (q, k, v, log_f))
        if self.num_blocks > 1:
            nb = self.num_blocks
            q, k, log_f = (t.unflatten(-1, (nb, -1)).flatten(2, 3) for t in (q, k, log_f))     # b n (h k) d
            v = v.repeat_interleave(nb, dim=2)
            beta = beta.repeat_interleave(nb, dim=2)
        if self.norm_q:
            q = l2_norm(q)
        k = l2_norm(k)
        if self.norm_v:
            v = l2_norm(v)
        if attention_mask is not None and not attention_mask.all() and n > 1:        # left padding
            keep = attention_mask[:, q_offset:].unsqueeze(-1).unsqueeze(-1) != 0
            k = k.masked_fill(~keep, 0)
            log_f = log_f.masked_fill(~keep, 0)
        return q, k, v, beta, log_f, gate0

    def forward(self, x, attention_mask: Optional[torch.Tensor] = None, past_key_values=None,
                use_cache: Optional[bool] = False, lower_bound: Optional[torch.Tensor] = None, **kwargs):
        b, n, d = x.shape
        recurrent_state, q_offset = None, 0
        if past_key_values is not None and len(past_key_values) > self.layer_idx:
            recurrent_state = past_key_values[self.layer_idx]["recurrent_state"][0]
            q_offset = past_key_values.get_seq_length(self.layer_idx)
        q, k, v, beta, log_f, gate0 = self.project(x, attention_mask, q_offset, lower_bound)
        dtype = q.dtype
        k, v, beta, log_f = k.to(dtype), v.to(dtype), beta.to(dtype), log_f.to(dtype)

        if self.dispatch == "reference":
            chunked = bool(self.training or use_cache)
        else:
            chunked = (torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v, beta, log_f))) \
                or n >= RECURRENT_BELOW
        # output_final_state: the reference asks for it iff use_cache (hdla_custom.py:306,320)
        if self.fuse_ab:
            op = chunk_hdla_delta_rule if chunked else fused_recurrent_hdla_delta_rule
            output, recurrent_state = op(q, k, v, beta, log_f, scale=1.0, initial_state=recurrent_state,
                                         output_final_state=bool(use_cache))
        else:
            a, bb = parameterize_a_b(beta=beta.float(), k=k.float(), log_f=log_f.float())
            if chunked:
                output, recurrent_state = chunk_hrdplr_delta_rule(
                    q=q, k=k, v=v, a=a.to(dtype), b=bb.to(dtype), gk=log_f, RANK_AB=2, initial_state=recurrent_state,
                    output_final_state=bool(use_cache), scale=1.0, head_first=False, chunk_size=16)
            else:
                output, recurrent_state = fused_recurrent_dplr_delta_rule(
                    q=q, k=k, v=v, a=a.to(dtype), b=bb.to(dtype), gk=log_f, rank_ab=2, initial_state=recurrent_state,
                    output_final_state=bool(use_cache), scale=1.0, head_first=False)

        if self.num_blocks > 1:
            output = output.unflatten(2, (-1, self.num_blocks)).sum(dim=-2)
        if past_key_values is not None:
            past_key_values.update(recurrent_state=[recurrent_state], layer_idx=self.layer_idx, offset=n)
        output = output.flatten(2, 3)
        if self.use_output_gate:
            output = self.norm(output, self._up(self.output_gate[1], gate0))
        else:
            output = self.norm(output)
        return self.o_proj(output), past_key_values

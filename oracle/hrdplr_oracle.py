"""CPU oracle for the rank-R DPLR delta-rule linear attention of HDLA.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it is the checker for the HIP path, used by
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``.

It restates, in plain differentiable torch on the CPU, the algorithm of the reference:

* :func:`recurrence` follows the fused-recurrent kernel body ``HRDPLR/recurrent.py:81-104`` token by token
  (both rank terms read the pre-update, pre-decay state ``:93-98``; the decay is applied at ``:100``;
  the output uses the post-update state ``:104``), its ``REVERSE`` walk ``:63,108-115`` and its packed
  variable-length addressing ``:54-58``.
* :func:`chunk_naive` follows the chunk form of ``HRDPLR/naive.py:76-263`` (cumulative decays ``:107-108``,
  the four masked score matrices ``:136-184``, the forward-substitution inverse ``:189-192``, the WY pair
  ``:195-196`` and the chunk loop ``:232-255``).  Like the reference it ignores ``scale`` unless asked
  (``naive.py:83`` is never read), so callers pre-scale ``q``; here ``scale`` multiplies ``q`` explicitly so
  both oracles share one convention.

Parity of the oracle itself is pinned without importing the reference (``tests/test_oracle.py``):
closed forms (T = 1; a = b = 0 gives gated linear attention; g = 0 with one rank gives DeltaNet),
linearity in (v, S0), chunk-size independence, chunk form == recurrence, split-sequence state hand-off,
reverse == time flip, variable-length == per-sequence calls, and gradients by central finite differences.

* :func:`parameterize_a_b` follows ``HRDPLR/hdla_custom.py:19-43`` (the build of a, b from beta, k, log_f that the
  layer runs right before the operator, ``:290``), with the ``return`` the reference's function lacks.  It is
  pinned by the identity its own comment states (``hdla_custom.py:270-288``): the one-step transition
  ``Diag(f) + b_1 a_1^T + b_2 a_2^T`` equals ``(I - beta k k^T) Diag(f) (I - beta k k^T)``.
"""
from typing import Optional, Tuple

import torch


def _check_shapes(q, k, v, a, b, gk, rank_ab):
    B, T, H, K = q.shape
    V = v.shape[-1]
    assert k.shape == (B, T, H, K) and gk.shape == (B, T, H, K)
    assert v.shape == (B, T, H, V)
    assert a.shape == (B, T * rank_ab, H, K) and b.shape == a.shape
    return B, T, H, K, V


def recurrence(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, b: torch.Tensor, gk: torch.Tensor,
    scale: float = 1.0,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = True,
    rank_ab: int = 2,
    reverse: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    dtype: torch.dtype = torch.float64,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Token-serial recurrence (HRDPLR/recurrent.py:81-104).

        S_t = Diag(exp(g_t)) S_{t-1} + sum_r b_t^r (a_t^r . S_{t-1}) + k_t v_t^T ,   o_t = scale * S_t^T q_t

    ``a`` and ``b`` hold row ``t*R + r`` for rank ``r`` of token ``t`` (recurrent.py:66-67,96-97).
    Returns ``o`` [B,T,H,V] and the final state [N,H,K,V] (N = number of sequences), both in ``dtype``.
    """
    B, T, H, K, V = _check_shapes(q, k, v, a, b, gk, rank_ab)
    R = rank_ab
    q, k, v, a, b, gk = (x.to(dtype) for x in (q, k, v, a, b, gk))
    if cu_seqlens is None:
        bounds = [(n, 0, T) for n in range(B)]
    else:
        assert B == 1
        cu = [int(x) for x in cu_seqlens]
        bounds = [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]
    N = len(bounds)
    o_rows = [[None] * T for _ in range(B)]
    finals = []
    for n, (bi, bos, eos) in enumerate(bounds):
        if initial_state is not None:
            S = initial_state[n].to(dtype)
        else:
            S = q.new_zeros(H, K, V)
        steps = range(eos - 1, bos - 1, -1) if reverse else range(bos, eos)
        for t in steps:
            q_t, k_t, v_t, g_t = q[bi, t], k[bi, t], v[bi, t], gk[bi, t]          # [H,K] / [H,V]
            contrib = 0
            for r in range(R):
                a_r, b_r = a[bi, t * R + r], b[bi, t * R + r]                        # [H,K]
                contrib = contrib + b_r[:, :, None] * torch.einsum('hk,hkv->hv', a_r, S)[:, None, :]
            S = torch.exp(g_t)[:, :, None] * S + contrib + k_t[:, :, None] * v_t[:, None, :]
            o_rows[bi][t] = scale * torch.einsum('hk,hkv->hv', q_t, S)
        finals.append(S)
    o = torch.stack([torch.stack(rows, 0) if rows else q.new_zeros(0, H, V) for rows in o_rows], 0)
    ht = torch.stack(finals, 0) if output_final_state else None
    return o, ht


def chunk_naive(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, b: torch.Tensor, gk: torch.Tensor,
    scale: float = 1.0,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = True,
    rank_ab: int = 2,
    chunk_size: int = 16,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Chunk form of HRDPLR/naive.py:76-263, written without in-place autograd hazards.

    Rows of a/b inside a chunk keep the reference's ``(token, rank)`` order with rank fastest
    (naive.py:102-105,168).  Requires ``T % chunk_size == 0`` like the reference (naive.py:98-105).
    """
    B, T, H, K, V = _check_shapes(q, k, v, a, b, gk, rank_ab)
    R, C = rank_ab, chunk_size
    assert T % C == 0, "the chunk form needs T to be a multiple of chunk_size (naive.py:98)"
    NT = T // C
    q, k, v, a, b, gk = (x.to(dtype) for x in (q, k, v, a, b, gk))
    q = q * scale

    def split(x, rows):                      # [B, NT*rows, H, D] -> [B, H, NT, rows, D]
        return x.reshape(B, NT, rows, H, x.shape[-1]).permute(0, 3, 1, 2, 4)

    q, k, v, gk = (split(x, C) for x in (q, k, v, gk))
    a, b = split(a, C * R), split(b, C * R)
    gi = gk.cumsum(-2)                                                   # naive.py:107
    ge = gi - gk                                                         # naive.py:108
    gi_ab = gi.repeat_interleave(R, dim=-2)                              # naive.py:110
    ge_ab = ge.repeat_interleave(R, dim=-2)                              # naive.py:111
    tok = torch.arange(C)
    tok_ab = tok.repeat_interleave(R)

    def scores(x, gx, y, gy, mask):
        # sum_k x_i[k] y_j[k] exp(gx_i[k] - gy_j[k]) restricted to mask (naive.py:149-184); the exponent is
        # clamped to <= 0 on the masked-out side so it cannot overflow there.
        d = gx[..., :, None, :] - gy[..., None, :, :]
        d = torch.where(mask[:, :, None], d, torch.zeros_like(d))
        return ((x[..., :, None, :] * y[..., None, :, :]) * torch.exp(d)).sum(-1) * mask

    A_qk = scores(q, gi, k, gi, tok[:, None] >= tok[None, :])            # naive.py:141,149
    A_qb = scores(q, gi, b, gi_ab, tok[:, None] >= tok_ab[None, :])      # naive.py:142,158
    A_ak = scores(a, ge_ab, k, gi, tok_ab[:, None] > tok[None, :])       # naive.py:144,169
    A_ab = scores(a, ge_ab, b, gi_ab, tok_ab[:, None] > tok_ab[None, :])  # naive.py:145,177

    eye = torch.eye(C * R, dtype=dtype)
    # (I - A_ab)^-1 : the row recurrence of naive.py:189-192 is forward substitution on a unit lower
    # triangular matrix, i.e. a triangular solve.
    Tm = torch.linalg.solve_triangular(eye - A_ab, eye.expand_as(A_ab), upper=False)
    w = Tm @ (a * torch.exp(ge_ab))                                      # naive.py:195
    u = Tm @ (A_ak @ v)                                                  # naive.py:196
    decay_to_end = torch.exp(gi[..., -1:, :] - gi)                       # naive.py:207-209
    kg = k * decay_to_end                                                # naive.py:214
    bg = b * decay_to_end.repeat_interleave(R, dim=-2)                   # naive.py:215
    qg = q * torch.exp(gi)                                               # naive.py:240

    S = initial_state.to(dtype) if initial_state is not None else q.new_zeros(B, H, K, V)
    outs = []
    for n in range(NT):                                                  # naive.py:232-255
        v2 = w[:, :, n] @ S + u[:, :, n]
        outs.append(A_qk[:, :, n] @ v[:, :, n] + A_qb[:, :, n] @ v2 + qg[:, :, n] @ S)
        S = S * torch.exp(gi[:, :, n, -1, :, None]) + kg[:, :, n].transpose(-1, -2) @ v[:, :, n] \
            + bg[:, :, n].transpose(-1, -2) @ v2
    o = torch.stack(outs, 2)                                             # [B,H,NT,C,V]
    o = o.permute(0, 2, 3, 1, 4).reshape(B, T, H, V)                     # naive.py:263
    return o, (S if output_final_state else None)


def hrdplr_naive(q, k, v, a, b, gk, scale, initial_state, output_final_state, RANK_AB, head_first, chunk_size):
    """The reference's oracle under its own name and positional signature (HRDPLR/naive.py:76-90, exported at
    HRDPLR/__init__.py:3), so that its test call pattern ``hrdplr_naive(q, k, v, a, b, gk, 1.0, initial_state, True,
    RANK_AB, False, chunk_size=BT)`` (test_integrated.py:72-74) can be replayed.  Like the reference it never reads
    ``scale`` (naive.py:83: the output is ``(q * exp(gi)) @ S`` without it, :240), works in the dtype of ``q``, needs
    ``T % chunk_size == 0`` (:98-105) and returns ``(o, final_state or None)`` (:263)."""
    assert not head_first, "only head_first=False is supported (naive.py:98-105 rearranges [B, T, H, D])"
    del scale
    return chunk_naive(q, k, v, a, b, gk, 1.0, initial_state, output_final_state, rank_ab=RANK_AB,
                       chunk_size=chunk_size, dtype=q.dtype)


def parameterize_a_b(beta: torch.Tensor, k: torch.Tensor, log_f: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """HRDPLR/hdla_custom.py:19-43: beta [B,T,H,1] (or [B,T,H]), k and log_f [B,T,H,K] -> a, b [B,2T,H,K]."""
    if beta.dim() == 3:
        beta = beta.unsqueeze(-1)
    f = torch.exp(log_f)
    a_t1 = -beta * k                                                   # :24
    a_t2 = -beta * f * k                                               # :25
    b_t1, b_t2 = k, k                                                  # :27-28
    a_1 = a_t1                                                         # :30
    a_2 = a_t2 + a_t1 * torch.sum(b_t1 * a_t2, dim=-1, keepdim=True)   # :31-33
    b_1 = f * b_t1                                                     # :35
    b_2 = b_t2                                                         # :36
    B, T, H, K = k.shape
    a = torch.stack([a_1, a_2], dim=2).reshape(B, 2 * T, H, K)         # :38-41: rank-minor rows
    b = torch.stack([b_1, b_2], dim=2).reshape(B, 2 * T, H, K)
    return a, b


def rel_l2(x: torch.Tensor, ref: torch.Tensor) -> float:
    """Relative L2 error ||x - ref|| / ||ref|| in float64 (the metric of every parity tolerance here)."""
    x, ref = x.detach().double().cpu(), ref.detach().double().cpu()
    den = ref.norm().item()
    num = (x - ref).norm().item()
    return num / den if den > 0 else num

"""Fused recurrent (decode) entry point: the drop-in for HRDPLR/recurrent.py.

* ``fused_recurrent_dplr_delta_rule``          <- HRDPLR/recurrent.py:227-319
* ``FusedRecurrentDPLRDeltaRuleFunction``      <- HRDPLR/recurrent.py:180-224 (forward only; backward raises)
* ``fused_recurrent_dplr_delta_rule_fwd``      <- HRDPLR/recurrent.py:121-177, now one call of ``hdla_recurrent_fwd``
"""
import ctypes
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from .chunk import _native_dim, _pad_last, _rank2, _require_gpu
from .utils import autocast_custom_bwd, autocast_custom_fwd, contiguous

_RECURRENT_D = (64, 128, 256)     # head sizes the token-serial kernel is built for (smaller ones are zero-padded)


def fused_recurrent_dplr_delta_rule_fwd(q, k, v, a, b, gk, rank_ab, scale=1.0, initial_state=None,
                                        output_final_state=False, reverse=False, cu_seqlens=None):
    """Launch of the token-serial kernel on native shapes (rank 2, K and V in {64, 128})."""
    B, TR, H, K = a.shape
    T = TR // rank_ab
    assert TR == T * rank_ab, f"Merged dimension TR={TR} must be divisible by rank_ab={rank_ab}"
    assert b.shape == (B, TR, H, K), f"b shape {b.shape} doesn't match a shape {a.shape}"
    assert k.shape == (B, T, H, K), f"k shape {k.shape} should be (B, T, H, K)"
    assert v.shape == (B, T, H, v.shape[-1]), f"v shape {v.shape} should be (B, T, H, V)"
    assert q.shape == (B, T, H, K), f"q shape {q.shape} should be (B, T, H, K)"
    assert gk.shape == (B, T, H, K), f"gk shape {gk.shape} should be (B, T, H, K)"
    lib = _lib.load()
    V = v.shape[-1]
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    with torch.cuda.device(q.device):
        dims = _lib.make_dims(B, T, H, K, V, 2, N, q.dtype, gk.dtype, scale, cu_seqlens)
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        ht = q.new_empty(N, H, K, V, dtype=torch.float32) if output_final_state else None
        o = torch.zeros_like(v) if cu_seqlens is not None else torch.empty_like(v)     # rows of no sequence stay zero
        rc = lib.hdla_recurrent_fwd(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                    _lib.ptr(gk), int(bool(reverse)), _lib.ptr(h0), _lib.ptr(o), _lib.ptr(ht),
                                    _lib.current_stream(q.device))
        _lib.check(rc, "hdla_recurrent_fwd")
    return o, ht


class FusedRecurrentDPLRDeltaRuleFunction(torch.autograd.Function):

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, a, b, gk, rank_ab, scale=None, initial_state=None, output_final_state=False,
                reverse=False, cu_seqlens=None):
        return fused_recurrent_dplr_delta_rule_fwd(q, k, v, a, b, gk, rank_ab, scale, initial_state,
                                                   output_final_state, reverse, cu_seqlens)

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        raise NotImplementedError(
            "Backward pass for fused_recurrent_dplr_delta_rule is not implemented and will not be supported. "
            "This kernel is only for inference. "
            "For training, please use `chunk_hrdplr_delta_rule`."
        )


def fused_recurrent_dplr_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    a: torch.Tensor,
    b: torch.Tensor,
    gk: torch.Tensor,
    rank_ab: int = 1,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    reverse: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
    head_first: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Token-serial evaluation of S_t = Diag(exp(gk_t)) S_{t-1} + sum_r b_t^r (a_t^r . S_{t-1}) + k_t v_t^T.

    Signature, argument meaning and error behaviour of HRDPLR/recurrent.py:227-319: ``a``/``b`` are
    ``[B, T*rank_ab, H, K]`` with the rank index fastest, ``gk`` is a log-space decay, ``initial_state`` is
    ``[N, H, K, V]``, ``cu_seqlens`` packs N sequences into a batch of one; returns ``(o, final_state)`` with
    ``o`` in ``v``'s dtype and ``final_state`` fp32 or ``None``.
    """
    assert head_first == False, ""                                                          # recurrent.py:276
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f"The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`."
                f"Please flatten variable-length inputs before processing."
            )
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f"The number of initial states is expected to be equal to the number of input sequences, "
                f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}."
            )
    if len(a.shape) != 4:
        raise ValueError(f"a must have 4 dimensions [B, T*RANK_AB, H, K], got {len(a.shape)}")
    if len(b.shape) != 4:
        raise ValueError(f"b must have 4 dimensions [B, T*RANK_AB, H, K], got {len(b.shape)}")
    B, TR, _, _ = a.shape
    T_expected = TR // rank_ab
    assert TR == T_expected * rank_ab, f"Merged dimension TR={TR} must be divisible by rank_ab={rank_ab}"
    assert q.shape[1] == T_expected, f"q time dimension {q.shape[1]} must match T={T_expected} from merged dimension"
    if scale is None:
        scale = q.shape[-1] ** -0.5                                                          # recurrent.py:302-303
    if rank_ab not in (1, 2):
        raise NotImplementedError(f"rank_ab = {rank_ab} is not supported (1 or 2)")
    _require_gpu(q, k, v, a, b, gk, initial_state)
    if cu_seqlens is not None:
        _lib.check_cu_seqlens(cu_seqlens, q.shape[1])
        cu_seqlens = cu_seqlens.to(device=q.device, dtype=torch.int64).contiguous()

    K, V = q.shape[-1], v.shape[-1]
    out_dtype = v.dtype
    if q.dtype == torch.float16:
        q, k, v, a, b, gk = (x.float() for x in (q, k, v, a, b, gk))
    elif q.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported dtype {q.dtype}")
    k, v, a, b = k.to(q.dtype), v.to(q.dtype), a.to(q.dtype), b.to(q.dtype)
    if gk.dtype != torch.float32 and gk.dtype != q.dtype:
        gk = gk.float()
    Kn, Vn = _native_dim(K, _RECURRENT_D), _native_dim(V, _RECURRENT_D)
    h0 = initial_state
    if h0 is not None and (Kn != K or Vn != V):
        h0 = F.pad(h0, (0, Vn - V, 0, Kn - K))
    o, final_state = FusedRecurrentDPLRDeltaRuleFunction.apply(
        _pad_last(q, Kn), _pad_last(k, Kn), _pad_last(v, Vn), _pad_last(_rank2(a, rank_ab), Kn),
        _pad_last(_rank2(b, rank_ab), Kn), _pad_last(gk, Kn), 2, scale, h0, output_final_state, reverse, cu_seqlens)
    if Vn != V:
        o = o[..., :V]
    if final_state is not None and (Kn != K or Vn != V):
        final_state = final_state[:, :, :K, :V]
    return o.to(out_dtype), final_state

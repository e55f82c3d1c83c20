"""The operator as the HDLA layer uses it: with a and b given by (beta, k, log_f).

* ``parameterize_a_b``        <- HRDPLR/hdla_custom.py:19-43, with the ``return`` the reference's function lacks (as
  shipped, ``a, b = parameterize_a_b(...)`` at ``hdla_custom.py:290`` unpacks ``None``)
* ``chunk_hdla_delta_rule``   <- the call sequence ``hdla_custom.py:290-309``: ``parameterize_a_b`` followed by
  ``chunk_hrdplr_delta_rule`` on ``a.to(dtype), b.to(dtype), gk=log_f``, in one operator that never materialises a and
  b: the kernels form them from (beta, k, log_f) where they are used, and the backward pass returns the gradients of
  (q, k, v, beta, log_f) directly (C ABI: ``hdla_param_chunk_fwd`` / ``hdla_param_chunk_bwd``).

* ``fused_recurrent_hdla_delta_rule`` <- the same pair for the token-serial operator (``parameterize_a_b`` +
  ``fused_recurrent_dplr_delta_rule``, HRDPLR/recurrent.py:227-319), forward only, for decode steps that carry the
  state a chunked prefill returned (C ABI: ``hdla_param_recurrent_fwd``).

a and b are half of the operator's input bytes and da, db half of its gradient bytes; the layer also saves the
elementwise kernels (and their backward) that would build them.
"""
import ctypes
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from .chunk import (_dims, _native_dim, _pad_last, _require_gpu, chunk_hrdplr_bwd, chunk_hrdplr_bwd_kept,
                    chunk_hrdplr_fwd)
from .utils import autocast_custom_bwd, autocast_custom_fwd, contiguous


def parameterize_a_b(beta: torch.Tensor, k: torch.Tensor, log_f: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """beta [B,T,H,1], k and log_f [B,T,H,K] -> a, b [B,2T,H,K] (rows t*2 + r), HRDPLR/hdla_custom.py:19-43.

    The decay they describe is (I - beta k k^T) Diag(exp(log_f)) (I - beta k k^T) (hdla_custom.py:270-288)."""
    f = torch.exp(log_f)
    a_t1 = -beta * k
    a_t2 = -beta * f * k
    a_2 = a_t2 + a_t1 * torch.sum(k * a_t2, dim=-1, keepdim=True)
    B, T, H, K = k.shape
    a = torch.stack([a_t1, a_2], dim=2).reshape(B, 2 * T, H, K)
    b = torch.stack([f * k, k], dim=2).reshape(B, 2 * T, H, K)
    return a, b


def _fwd(q, k, v, beta, gk, scale, initial_state, output_final_state, cu_seqlens, want_boundary=False):
    return chunk_hrdplr_fwd(q, k, v, None, None, gk, scale, initial_state, output_final_state, cu_seqlens, beta=beta,
                            want_boundary=want_boundary)


def _bwd(q, k, v, beta, gk, scale, initial_state, do, dht, cu_seqlens, want_dh0, boundary=None):
    return chunk_hrdplr_bwd(q, k, v, None, None, gk, scale, initial_state, do, dht, cu_seqlens, want_dh0=want_dh0,
                            beta=beta, boundary=boundary)


class ChunkHDLAFunction(torch.autograd.Function):
    """Same contract as ChunkDPLRDeltaRuleFunction: the forward pass saves only its inputs, the backward pass
    recomputes (HRDPLR/hrdplr.py:137,154)."""

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, beta, gk, scale, initial_state, output_final_state, cu_seqlens=None, keep_forward=False):
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        ctx.kept = None
        boundary = None
        if keep_forward and any(ctx.needs_input_grad):     # see ChunkDPLRDeltaRuleFunction.forward
            o, final_state, ctx.kept = chunk_hrdplr_fwd(q, k, v, None, None, gk, scale, h0, output_final_state, cu_seqlens,
                                                        keep=True, beta=beta)
        elif any(ctx.needs_input_grad) and _lib.keep_boundaries_default():
            o, final_state, boundary = _fwd(q, k, v, beta, gk, scale, h0, output_final_state, cu_seqlens, want_boundary=True)
        else:
            o, final_state = _fwd(q, k, v, beta, gk, scale, h0, output_final_state, cu_seqlens)
        ctx.save_for_backward(q, k, v, beta, gk, initial_state, cu_seqlens, boundary)
        ctx.scale = scale
        return o.to(q.dtype), final_state

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        q, k, v, beta, gk, initial_state, cu_seqlens, boundary = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(v)
        do = do.to(v.dtype).contiguous()
        if dht is not None:
            dht = dht.to(torch.float32).contiguous()
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        if ctx.kept is not None:
            dq, dk, dv, dbeta, dgk, dh0 = chunk_hrdplr_bwd_kept(q, k, v, None, None, gk, ctx.scale, h0, do, dht, ctx.kept,
                                                                cu_seqlens, want_dh0=initial_state is not None, beta=beta)
        else:
            dq, dk, dv, dbeta, dgk, dh0 = _bwd(q, k, v, beta, gk, ctx.scale, h0, do, dht, cu_seqlens,
                                               want_dh0=initial_state is not None, boundary=boundary)
        if dh0 is not None:
            dh0 = dh0.to(initial_state.dtype)
        return dq.to(q), dk.to(k), dv.to(v), dbeta.to(beta), dgk.to(gk), None, dh0, None, None, None


@torch.compiler.disable
def chunk_hdla_delta_rule(
    q: torch.Tensor,                 # [B, T, H, K]
    k: torch.Tensor,                 # [B, T, H, K]
    v: torch.Tensor,                 # [B, T, H, V]
    beta: torch.Tensor,              # [B, T, H, 1] or [B, T, H]
    log_f: torch.Tensor,             # [B, T, H, K], log-space decay
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,    # [N, H, K, V]
    output_final_state: bool = False,
    *,
    cu_seqlens: Optional[torch.Tensor] = None,
    keep_forward: Optional[bool] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``chunk_hrdplr_delta_rule(q, k, v, *parameterize_a_b(beta, k, log_f), gk=log_f, RANK_AB=2, ...)`` with a and
    b (rounded to q's dtype, as ``hdla_custom.py:301-304`` does) formed inside the kernels.  Returns ``(o, final_state)``
    like the plain operator; gradients flow to q, k, v, beta, log_f and initial_state.  ``keep_forward``: as for
    ``chunk_hrdplr_delta_rule``."""
    assert q.dtype == k.dtype == v.dtype
    if q.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be 4-dimensional [B, T, H, D]")
    B, T, H, K = q.shape
    V = v.shape[-1]
    if k.shape != q.shape or log_f.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} log_f {tuple(log_f.shape)}")
    if beta.shape not in ((B, T, H, 1), (B, T, H)):
        raise ValueError(f"beta must be [B, T, H, 1] or [B, T, H], got {tuple(beta.shape)}")
    _native_dim(K), _native_dim(V)                   # raises for head dimensions beyond the chunked kernels' 128
    if cu_seqlens is not None:
        if B != 1:
            raise ValueError(f"The batch size is expected to be 1 rather than {B} when using `cu_seqlens`."
                             f"Please flatten variable-length inputs before processing.")
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(f"The number of initial states is expected to be equal to the number of input sequences, "
                             f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.")
        _lib.check_cu_seqlens(cu_seqlens, q.shape[1])
        cu_seqlens = cu_seqlens.to(device=q.device, dtype=torch.int64).contiguous()
    elif initial_state is not None and initial_state.shape[0] != B:
        raise ValueError(f"initial_state must hold one state per sequence ({B}), got {initial_state.shape[0]}")
    _require_gpu(q, k, v, beta, log_f, initial_state)
    scale = K ** -0.5 if scale is None else scale

    out_dtype, beta_shape = q.dtype, beta.shape
    if q.dtype == torch.float16:
        q, k, v, beta, log_f = (x.float() for x in (q, k, v, beta, log_f))
    elif q.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported dtype {q.dtype}")
    beta = beta.to(q.dtype).reshape(B, T, H)
    gk = log_f
    if gk.dtype != torch.float32 and gk.dtype != q.dtype:
        gk = gk.float()
    Kn, Vn = _native_dim(K), _native_dim(V)       # zero channels of k add nothing to s and give zero a, b
    h0 = initial_state
    if h0 is not None and (Kn != K or Vn != V):
        h0 = F.pad(h0, (0, Vn - V, 0, Kn - K))
    o, final_state = ChunkHDLAFunction.apply(_pad_last(q, Kn), _pad_last(k, Kn), _pad_last(v, Vn), beta,
                                             _pad_last(gk, Kn), scale, h0, output_final_state, cu_seqlens,
                                             _lib.keep_forward_default() if keep_forward is None else bool(keep_forward))
    if Vn != V:
        o = o[..., :V]
    if final_state is not None and (Kn != K or Vn != V):
        final_state = final_state[:, :, :K, :V]
    return o.to(out_dtype), final_state


@torch.compiler.disable
def fused_recurrent_hdla_delta_rule(
    q: torch.Tensor,                 # [B, T, H, K]
    k: torch.Tensor,                 # [B, T, H, K]
    v: torch.Tensor,                 # [B, T, H, V]
    beta: torch.Tensor,              # [B, T, H, 1] or [B, T, H]
    log_f: torch.Tensor,             # [B, T, H, K], log-space decay
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,    # [N, H, K, V]
    output_final_state: bool = False,
    reverse: bool = False,
    cu_seqlens: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``fused_recurrent_dplr_delta_rule(q, k, v, *parameterize_a_b(beta, k, log_f), gk=log_f, rank_ab=2, ...)``
    with a and b (rounded to q's dtype) formed per token inside the kernel.  Inference only: no gradients, like
    the plain recurrent operator (HRDPLR/recurrent.py:219-224)."""
    assert q.dtype == k.dtype == v.dtype
    if q.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be 4-dimensional [B, T, H, D]")
    B, T, H, K = q.shape
    V = v.shape[-1]
    if k.shape != q.shape or log_f.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} log_f {tuple(log_f.shape)}")
    if beta.shape not in ((B, T, H, 1), (B, T, H)):
        raise ValueError(f"beta must be [B, T, H, 1] or [B, T, H], got {tuple(beta.shape)}")
    if cu_seqlens is not None:
        if B != 1:
            raise ValueError(f"The batch size is expected to be 1 rather than {B} when using `cu_seqlens`."
                             f"Please flatten variable-length inputs before processing.")
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(f"The number of initial states is expected to be equal to the number of input sequences, "
                             f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.")
        _lib.check_cu_seqlens(cu_seqlens, q.shape[1])
        cu_seqlens = cu_seqlens.to(device=q.device, dtype=torch.int64).contiguous()
    elif initial_state is not None and initial_state.shape[0] != B:
        raise ValueError(f"initial_state must hold one state per sequence ({B}), got {initial_state.shape[0]}")
    if any(x.requires_grad for x in (q, k, v, beta, log_f)) and torch.is_grad_enabled():
        raise NotImplementedError("fused_recurrent_hdla_delta_rule is only for inference. "
                                  "For training, please use `chunk_hdla_delta_rule`.")
    _require_gpu(q, k, v, beta, log_f, initial_state)
    scale = K ** -0.5 if scale is None else scale

    out_dtype = v.dtype
    if q.dtype == torch.float16:
        q, k, v, beta, log_f = (x.float() for x in (q, k, v, beta, log_f))
    elif q.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported dtype {q.dtype}")
    beta = beta.to(q.dtype).reshape(B, T, H).contiguous()
    gk = log_f
    if gk.dtype != torch.float32 and gk.dtype != q.dtype:
        gk = gk.float()
    Kn, Vn = _native_dim(K, (64, 128, 256)), _native_dim(V, (64, 128, 256))
    h0 = None if initial_state is None else initial_state.to(torch.float32)
    if h0 is not None and (Kn != K or Vn != V):
        h0 = F.pad(h0, (0, Vn - V, 0, Kn - K))
    q, k, v, gk = (_pad_last(x, n).contiguous() for x, n in ((q, Kn), (k, Kn), (v, Vn), (gk, Kn)))
    N = B if cu_seqlens is None else cu_seqlens.numel() - 1
    lib = _lib.load()
    with torch.cuda.device(q.device):
        dims = _dims(q, v, gk, scale, cu_seqlens, N)
        h0 = None if h0 is None else h0.contiguous()
        ht = torch.empty(N, H, Kn, Vn, dtype=torch.float32, device=q.device) if output_final_state else None
        o = torch.zeros_like(v) if cu_seqlens is not None else torch.empty_like(v)     # rows of no sequence stay zero
        rc = lib.hdla_param_recurrent_fwd(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(beta),
                                          _lib.ptr(gk), int(bool(reverse)), _lib.ptr(h0), _lib.ptr(o), _lib.ptr(ht),
                                          _lib.current_stream(q.device))
        _lib.check(rc, "hdla_param_recurrent_fwd")
    if Vn != V:
        o = o[..., :V]
    if ht is not None and (Kn != K or Vn != V):
        ht = ht[:, :, :K, :V]
    return o.to(out_dtype), ht

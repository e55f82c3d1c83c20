"""Chunked (training) entry point of the rank-2 DPLR delta rule: the drop-in for HRDPLR/hrdplr.py.

Same call signature, return values and autograd contract as the reference:

* ``chunk_hrdplr_delta_rule``            <- HRDPLR/hrdplr.py:286-318
* ``ChunkDPLRDeltaRuleFunction``         <- HRDPLR/hrdplr.py:101-284 (forward saves only the inputs, backward
  recomputes; 12 positional arguments, one gradient slot each; here a 13th, ``cu_seqlens``, is appended)

The stage launchers of HRDPLR/fwd_func.py and HRDPLR/bwd_func.py are replaced by two calls into the C ABI of
libhdla_hip.so (``hdla_chunk_fwd`` / ``hdla_chunk_bwd``).  Differences a caller can observe:

* ``chunk_size`` is a hint; the kernels always work on 16-token chunks (results do not depend on it, and 16 is
  the only size the reference's backward handles, HRDPLR/bwd_func.py:299);
* ``cu_seqlens`` (keyword-only) packs variable-length sequences on the T axis, as in the recurrent entry
  (HRDPLR/recurrent.py:278-288);
* head dimensions other than 64/128 (up to 128) and ``RANK_AB = 1`` run through exact zero padding;
* float16 inputs are computed in fp32.
"""
import ctypes
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from .utils import autocast_custom_bwd, autocast_custom_fwd, contiguous

_NATIVE_D = (64, 128)


def _require_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _lib.HdlaError("the HDLA HIP operators run on a GPU only (got a tensor on "
                                 f"{t.device}); there is no CPU fallback")


def _native_dim(d: int, sizes=_NATIVE_D) -> int:
    for n in sizes:
        if d <= n:
            return n
    hint = ""
    if sizes[-1] < 256:
        hint = ("; the chunked operators hold a head's state tile by tile in registers and stop there: for head dimensions "
                "up to 256 use the token-serial operators fused_recurrent_dplr_delta_rule / "
                "fused_recurrent_hdla_delta_rule (forward only)")
    raise ValueError(f"head dimension {d} is not supported (maximum {sizes[-1]}){hint}")


def _pad_last(x: Optional[torch.Tensor], d: int) -> Optional[torch.Tensor]:
    if x is None or x.shape[-1] == d:
        return x
    return F.pad(x, (0, d - x.shape[-1]))


def _rank2(x: torch.Tensor, rank: int) -> torch.Tensor:
    """[B, T*rank, H, K] with rank 1 -> rank 2 by interleaving zero rows (a zero rank term changes nothing)."""
    if rank == 2:
        return x
    if rank != 1:
        raise NotImplementedError(f"RANK_AB = {rank} is not supported (1 or 2)")
    B, T, H, K = x.shape
    return torch.stack([x, torch.zeros_like(x)], dim=2).reshape(B, 2 * T, H, K)


def _dims(q, v, gk, scale, cu_seqlens, n_seq):
    B, T, H, K = q.shape
    return _lib.make_dims(B, T, H, K, v.shape[-1], 2, n_seq, q.dtype, gk.dtype, scale, cu_seqlens)


def chunk_hrdplr_fwd(q, k, v, a, b, gk, scale, initial_state, output_final_state, cu_seqlens=None, keep=False,
                     beta=None, want_boundary=False):
    """Forward launch sequence (HRDPLR/hrdplr.py:25-99) on native shapes: returns (o, final_state), with ``keep`` also
    the workspace the backward pass can run on instead of recomputing it (``hdla_chunk_fwd_keep``), with
    ``want_boundary`` also the record of the states at the time-segment boundaries (None where the route has none).
    With ``beta`` a and b are formed in the kernels (they may be None)."""
    lib = _lib.load()
    B, T, H, K = q.shape
    V = v.shape[-1]
    N = B if cu_seqlens is None else cu_seqlens.numel() - 1
    with torch.cuda.device(q.device):
        dims = _dims(q, v, gk, scale, cu_seqlens, N)
        # with a packed-sequence table that was not validated on the host, rows outside every sequence stay unwritten
        o = torch.zeros_like(v) if cu_seqlens is not None else torch.empty_like(v)
        ht = torch.empty(N, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
        if keep:
            ws = _lib.workspace(dims, _lib.PASS_FWD_KEEP, q.device)
            rc = lib.hdla_chunk_fwd_keep(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a),
                                         _lib.ptr(b), _lib.ptr(beta), _lib.ptr(gk), _lib.ptr(initial_state), _lib.ptr(o),
                                         _lib.ptr(ht), _lib.ptr(ws), ws.numel(), _lib.current_stream(q.device))
            _lib.check(rc, "hdla_chunk_fwd_keep")
            return o, ht, ws
        ws = _lib.workspace(dims, _lib.PASS_FWD, q.device)
        bnd = _lib.boundary(dims, q.device) if want_boundary else None
        rc = lib.hdla_chunk_fwd_b(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                  _lib.ptr(beta), _lib.ptr(gk), _lib.ptr(initial_state), _lib.ptr(o), _lib.ptr(ht),
                                  _lib.ptr(bnd), 0 if bnd is None else bnd.numel(),
                                  _lib.ptr(ws), ws.numel(), _lib.current_stream(q.device))
        _lib.check(rc, "hdla_chunk_fwd_b")
    if want_boundary:
        return o, ht, bnd
    return o, ht


def chunk_hrdplr_bwd_kept(q, k, v, a, b, gk, scale, initial_state, do, dht, kept, cu_seqlens=None, want_dh0=True,
                          beta=None):
    """Backward launch sequence on the workspace a forward pass kept (``hdla_chunk_bwd_kept``): the per-chunk
    intermediates are read there, not recomputed.  Returns (dq, dk, dv, da, db, dgk, dh0), or with ``beta``
    (dq, dk, dv, dbeta, dgk, dh0)."""
    lib = _lib.load()
    B, T, H, K = q.shape
    V = v.shape[-1]
    N = B if cu_seqlens is None else cu_seqlens.numel() - 1
    with torch.cuda.device(q.device):
        dims = _dims(q, v, gk, scale, cu_seqlens, N)
        ws = _lib.workspace(dims, _lib.PASS_BWD_KEPT, q.device)
        # rows outside every sequence of a packed batch stay unwritten: they must not carry garbage upstream
        new = torch.zeros_like if cu_seqlens is not None else torch.empty_like
        dq, dk, dv, dgk = new(q), new(k), new(v), new(gk)
        da = db = dbeta = None
        if beta is None:
            da, db = new(a), new(b)
        else:
            dbeta = new(beta)
        dh0 = torch.empty(N, H, K, V, dtype=torch.float32, device=q.device) if want_dh0 else None
        rc = lib.hdla_chunk_bwd_kept(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                     _lib.ptr(beta), _lib.ptr(gk), _lib.ptr(initial_state), _lib.ptr(do), _lib.ptr(dht),
                                     _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(da), _lib.ptr(db), _lib.ptr(dbeta),
                                     _lib.ptr(dgk), _lib.ptr(dh0), _lib.ptr(kept), kept.numel(), _lib.ptr(ws), ws.numel(),
                                     _lib.current_stream(q.device))
        _lib.check(rc, "hdla_chunk_bwd_kept")
    if beta is None:
        return dq, dk, dv, da, db, dgk, dh0
    return dq, dk, dv, dbeta, dgk, dh0


def chunk_hrdplr_bwd(q, k, v, a, b, gk, scale, initial_state, do, dht, cu_seqlens=None, want_dh0=True,
                     keep_workspace=False, beta=None, boundary=None):
    """Backward launch sequence (HRDPLR/hrdplr.py:149-284) on native shapes.  Returns (dq, dk, dv, da, db, dgk, dh0), or
    with ``beta`` (dq, dk, dv, dbeta, dgk, dh0).  ``boundary``: the record a forward pass left (see chunk_hrdplr_fwd)."""
    lib = _lib.load()
    B, T, H, K = q.shape
    V = v.shape[-1]
    N = B if cu_seqlens is None else cu_seqlens.numel() - 1
    # rows outside every sequence of a packed batch stay unwritten: they must not carry garbage upstream
    new = torch.zeros_like if cu_seqlens is not None else torch.empty_like
    with torch.cuda.device(q.device):
        dims = _dims(q, v, gk, scale, cu_seqlens, N)
        ws = _lib.workspace(dims, 1, q.device)
        dq, dk, dv, dgk = new(q), new(k), new(v), new(gk)
        da = db = dbeta = None
        if beta is None:
            da, db = new(a), new(b)
        else:
            dbeta = new(beta)
        dh0 = torch.empty(N, H, K, V, dtype=torch.float32, device=q.device) if want_dh0 else None
        rc = lib.hdla_chunk_bwd_b(ctypes.byref(dims), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                  _lib.ptr(beta), _lib.ptr(gk), _lib.ptr(initial_state), _lib.ptr(do), _lib.ptr(dht),
                                  _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(da), _lib.ptr(db), _lib.ptr(dbeta),
                                  _lib.ptr(dgk), _lib.ptr(dh0), _lib.ptr(boundary),
                                  0 if boundary is None else boundary.numel(),
                                  _lib.ptr(ws), ws.numel(), _lib.current_stream(q.device))
        _lib.check(rc, "hdla_chunk_bwd_b")
    if beta is not None:
        return dq, dk, dv, dbeta, dgk, dh0
    if keep_workspace:
        return dq, dk, dv, da, db, dgk, dh0, ws, dims
    return dq, dk, dv, da, db, dgk, dh0


class ChunkDPLRDeltaRuleFunction(torch.autograd.Function):
    """Autograd contract of HRDPLR/hrdplr.py:101-284."""

    @staticmethod
    @contiguous
    @autocast_custom_fwd
    def forward(ctx, q, k, v, a, b, gk, scale, initial_state, output_final_state, RANK_AB, head_first, chunk_size,
                cu_seqlens=None, keep_forward=False):
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        # keep_forward (off unless asked for): the per-chunk intermediates of this pass stay alive on ctx until the
        # backward pass, which then does not recompute them; only when a gradient can be asked for at all
        ctx.kept = None
        boundary = None
        if keep_forward and any(ctx.needs_input_grad):
            o, final_state, ctx.kept = chunk_hrdplr_fwd(q, k, v, a, b, gk, scale, h0, output_final_state, cu_seqlens, keep=True)
        elif any(ctx.needs_input_grad) and _lib.keep_boundaries_default():
            o, final_state, boundary = chunk_hrdplr_fwd(q, k, v, a, b, gk, scale, h0, output_final_state, cu_seqlens,
                                                        want_boundary=True)
        else:
            o, final_state = chunk_hrdplr_fwd(q, k, v, a, b, gk, scale, h0, output_final_state, cu_seqlens)
        # the inputs (hrdplr.py:137) and, where the route cuts sequences into time segments, the states at the segment
        # boundaries (64 KiB per sequence, head and segment; HDLA_HIP_INPUTS_ONLY=1: not even those)
        ctx.save_for_backward(q, k, v, a, b, gk, initial_state, cu_seqlens, boundary)
        ctx.scale = scale
        ctx.chunk_size = chunk_size
        ctx.output_final_state = output_final_state
        ctx.RANK_AB = RANK_AB
        ctx.head_first = head_first
        return o.to(q.dtype), final_state

    @staticmethod
    @contiguous
    @autocast_custom_bwd
    def backward(ctx, do, dht):
        q, k, v, a, b, gk, initial_state, cu_seqlens, boundary = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(v)
        do = do.to(v.dtype).contiguous()
        if dht is not None:
            dht = dht.to(torch.float32).contiguous()
        h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
        if ctx.kept is not None:
            dq, dk, dv, da, db, dgk, dh0 = chunk_hrdplr_bwd_kept(q, k, v, a, b, gk, ctx.scale, h0, do, dht, ctx.kept,
                                                                 cu_seqlens, want_dh0=initial_state is not None)
        else:
            dq, dk, dv, da, db, dgk, dh0 = chunk_hrdplr_bwd(q, k, v, a, b, gk, ctx.scale, h0, do, dht, cu_seqlens,
                                                            want_dh0=initial_state is not None, boundary=boundary)
        if dh0 is not None:
            dh0 = dh0.to(initial_state.dtype)
        # one slot per forward argument (hrdplr.py:284), plus one each for cu_seqlens and keep_forward
        return dq.to(q), dk.to(k), dv.to(v), da.to(a), db.to(b), dgk.to(gk), None, dh0, None, None, None, None, None, None


@torch.compiler.disable
def chunk_hrdplr_delta_rule(
    q: torch.Tensor,                 # [B, T, H, K]
    k: torch.Tensor,                 # [B, T, H, K]
    v: torch.Tensor,                 # [B, T, H, V]
    a: torch.Tensor,                 # [B, T * RANK_AB, H, K]
    b: torch.Tensor,                 # [B, T * RANK_AB, H, K]
    gk: torch.Tensor,                # [B, T, H, K], log-space decay
    RANK_AB: int,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,    # [N, H, K, V]
    output_final_state: bool = False,
    head_first: bool = False,
    chunk_size: int = 32,
    *,
    cu_seqlens: Optional[torch.Tensor] = None,
    keep_forward: Optional[bool] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """S_t = Diag(exp(gk_t)) S_{t-1} + sum_r b_t^r (a_t^r . S_{t-1}) + k_t v_t^T,  o_t = scale * S_t^T q_t.

    Signature and semantics of HRDPLR/hrdplr.py:286-318; returns ``(o [B,T,H,V] in q.dtype, final_state
    [N,H,K,V] fp32 or None)``.

    ``keep_forward`` (keyword-only, not in the reference): True keeps the forward pass's per-chunk intermediates alive
    until the backward pass (about 1.6 times the bytes of q, k, v, a, b, gk together), which then skips recomputing
    them; False (and None without HDLA_HIP_KEEP_FORWARD=1 in the environment) is the reference's behaviour: only the
    inputs are kept (hrdplr.py:137) and the backward pass recomputes (:161-198).  Results agree to rounding.
    """
    assert head_first is False or head_first == 0, "only head_first=False is supported (HRDPLR/fwd_func.py:28)"
    assert q.dtype == k.dtype == v.dtype                                                   # hrdplr.py:301
    if RANK_AB not in (1, 2):
        raise NotImplementedError(f"RANK_AB = {RANK_AB} is not supported (1 or 2)")
    if q.dim() != 4 or v.dim() != 4 or a.dim() != 4 or b.dim() != 4:
        raise ValueError("q, k, v, a, b must be 4-dimensional [B, T, H, D]")
    B, T, H, K = q.shape
    V = v.shape[-1]
    if k.shape != q.shape or gk.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} gk {tuple(gk.shape)}")
    if a.shape != (B, T * RANK_AB, H, K) or b.shape != a.shape:
        raise ValueError(f"a and b must be [B, T*RANK_AB, H, K] = {(B, T * RANK_AB, H, K)}, "
                         f"got {tuple(a.shape)} and {tuple(b.shape)}")
    if int(chunk_size) < 1:
        raise ValueError("chunk_size must be positive")
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
    _require_gpu(q, k, v, a, b, gk, initial_state)
    scale = K ** -0.5 if scale is None else scale                                           # hrdplr.py:302

    out_dtype = q.dtype
    if q.dtype == torch.float16:
        q, k, v, a, b, gk = (x.float() for x in (q, k, v, a, b, gk))
    elif q.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported dtype {q.dtype}")
    a, b = a.to(q.dtype), b.to(q.dtype)
    if gk.dtype != torch.float32 and gk.dtype != q.dtype:
        gk = gk.float()
    Kn, Vn = _native_dim(K), _native_dim(V)
    a2, b2 = _rank2(a, RANK_AB), _rank2(b, RANK_AB)
    h0 = initial_state
    if h0 is not None and (Kn != K or Vn != V):
        h0 = F.pad(h0, (0, Vn - V, 0, Kn - K))
    o, final_state = ChunkDPLRDeltaRuleFunction.apply(
        _pad_last(q, Kn), _pad_last(k, Kn), _pad_last(v, Vn), _pad_last(a2, Kn), _pad_last(b2, Kn), _pad_last(gk, Kn),
        scale, h0, output_final_state, 2, head_first, chunk_size, cu_seqlens,
        _lib.keep_forward_default() if keep_forward is None else bool(keep_forward))
    if Vn != V:
        o = o[..., :V]
    if final_state is not None and (Kn != K or Vn != V):
        final_state = final_state[:, :, :K, :V]
    return o.to(out_dtype), final_state

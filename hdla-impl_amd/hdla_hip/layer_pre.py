"""The elementwise stage of the HDLA layer between its projections and the operator, as two fused operators.

* ``layer_pre``   : (y, ...) -> q, k, v, beta, tails.  ``y [rows, ldy]`` is the output of the layer's one projection
  GEMM; q, k, v are ``silu`` of three of its column ranges, split into heads and l2-normalised where asked
  (HRDPLR/hdla_custom.py:228-251), beta is ``beta_scale * sigmoid`` of a fourth (:221-224), and the tails are
  contiguous copies of the column ranges from ``col_tail`` on (the inner activations of the low-rank decay and gate
  projections).  Its backward pass writes the gradient of all of y once (C ABI ``hdla_layer_pre_fwd/_bwd``).
* ``logsigmoid``  : HRDPLR/hdla_custom.py:219 (C ABI ``hdla_logsigmoid_fwd/_bwd``).
* ``low_rank_up`` : ``F.linear(x0, W)`` for the second half of a low-rank projection (head_dim -> embed_dim,
  hdla_custom.py:117-121,151-155) whose weight gradient ``dY^T @ x0`` — a tiny output contracted over all rows, for
  which a BLAS kernel tiled over the output has 16 workgroups — runs in a kernel of this library that also splits the
  rows (C ABI ``hdla_skinny_wgrad``); forward and input gradient stay BLAS calls.
"""
import ctypes

import torch
import torch.nn.functional as F

from . import _lib
from .chunk import _require_gpu


def supported(dtype: torch.dtype, D: int, ldy: int, cols) -> bool:
    """Shapes the kernels take: a head is 16 bytes times a power of two (<= 64) of lanes, rows and column ranges
    start on 16-byte boundaries."""
    if dtype not in (torch.bfloat16, torch.float32):
        return False
    n = 8 if dtype == torch.bfloat16 else 4
    if D % n:
        return False
    lanes = D // n
    return lanes <= 64 and lanes & (lanes - 1) == 0 and ldy % n == 0 and all(c % n == 0 for c in cols)


class LayerPreFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, y, H, D, col_q, col_k, col_v, col_beta, col_tail, tail_widths, norm_q, norm_k, norm_v, beta_scale,
                eps):
        assert y.dim() == 2 and y.is_contiguous()
        lib = _lib.load()
        rows, ldy = y.shape
        assert col_tail + sum(tail_widths) == ldy
        dims = _lib.HdlaPreDims(rows, H, D, _lib.dtype_code(y.dtype), ldy, col_q, col_k, col_v, col_beta,
                                int(norm_q), int(norm_k), int(norm_v), float(beta_scale), float(eps))
        with torch.cuda.device(y.device):
            q, k, v = (torch.empty(rows, H, D, dtype=y.dtype, device=y.device) for _ in range(3))
            beta = torch.empty(rows, H, 1, dtype=y.dtype, device=y.device) if col_beta >= 0 else None
            rc = lib.hdla_layer_pre_fwd(ctypes.byref(dims), _lib.ptr(y), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v),
                                        _lib.ptr(beta), _lib.current_stream(y.device))
            _lib.check(rc, "hdla_layer_pre_fwd")
            tails, c = [], col_tail
            for wdt in tail_widths:
                tails.append(y[:, c:c + wdt].contiguous())
                c += wdt
        ctx.save_for_backward(y)
        ctx.dims, ctx.col_tail, ctx.tail_widths = dims, col_tail, tuple(tail_widths)
        return (q, k, v, beta) + tuple(tails)

    @staticmethod
    def backward(ctx, dq, dk, dv, dbeta, *dtails):
        (y,) = ctx.saved_tensors
        dims, col_tail = ctx.dims, ctx.col_tail
        lib = _lib.load()
        rows, ldy = y.shape
        H, D = dims.H, dims.D
        z = lambda g, *shape: (torch.zeros(*shape, dtype=y.dtype, device=y.device) if g is None
                               else g.to(y.dtype).contiguous())
        dq, dk, dv = z(dq, rows, H, D), z(dk, rows, H, D), z(dv, rows, H, D)
        if dims.col_beta >= 0:
            dbeta = z(dbeta, rows, H, 1)
        with torch.cuda.device(y.device):
            covered = 3 * H * D + (H if dims.col_beta >= 0 else 0) + (ldy - col_tail)
            dy = torch.empty_like(y) if covered == ldy else torch.zeros_like(y)      # gaps between the ranges stay zero
            rc = lib.hdla_layer_pre_bwd(ctypes.byref(dims), _lib.ptr(y), _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv),
                                        _lib.ptr(dbeta) if dims.col_beta >= 0 else None, _lib.ptr(dy),
                                        _lib.current_stream(y.device))
            _lib.check(rc, "hdla_layer_pre_bwd")
            c = col_tail
            for wdt, g in zip(ctx.tail_widths, dtails):
                if g is None:
                    dy[:, c:c + wdt].zero_()
                else:
                    dy[:, c:c + wdt].copy_(g)
                c += wdt
        return (dy,) + (None,) * 13


@torch.compiler.disable
def layer_pre(y, H, D, col_q, col_k, col_v, col_beta, col_tail, tail_widths, norm_q, norm_k, norm_v, beta_scale,
              eps=1e-5):
    """y [rows, ldy] -> q, k, v [rows, H, D], beta [rows, H, 1] (None when col_beta < 0), then one contiguous copy per
    entry of ``tail_widths`` of consecutive column ranges starting at ``col_tail`` (together they must reach ldy).
    The column ranges must not overlap."""
    _require_gpu(y)
    return LayerPreFunction.apply(y, H, D, col_q, col_k, col_v, col_beta, col_tail, tuple(tail_widths), norm_q, norm_k,
                                  norm_v, beta_scale, eps)


class LogSigmoidFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x):
        x = x.contiguous()
        lib = _lib.load()
        with torch.cuda.device(x.device):
            y = torch.empty_like(x)
            rc = lib.hdla_logsigmoid_fwd(_lib.dtype_code(x.dtype), x.numel(), _lib.ptr(x), _lib.ptr(y),
                                         _lib.current_stream(x.device))
            _lib.check(rc, "hdla_logsigmoid_fwd")
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        dy = dy.to(x.dtype).contiguous()
        lib = _lib.load()
        with torch.cuda.device(x.device):
            dx = torch.empty_like(x)
            rc = lib.hdla_logsigmoid_bwd(_lib.dtype_code(x.dtype), x.numel(), _lib.ptr(x), _lib.ptr(dy), _lib.ptr(dx),
                                         _lib.current_stream(x.device))
            _lib.check(rc, "hdla_logsigmoid_bwd")
        return dx


@torch.compiler.disable
def logsigmoid(x: torch.Tensor) -> torch.Tensor:
    """log(sigmoid(x)) elementwise; the element count must be a multiple of 16 bytes' worth."""
    _require_gpu(x)
    return LogSigmoidFunction.apply(x)


def skinny_ok(dy: torch.Tensor, n_cols: int) -> bool:
    return (dy.is_cuda and dy.dtype == torch.bfloat16 and n_cols in (64, 128) and dy.shape[-1] % 64 == 0
            and dy.shape[0] > 0)


class LowRankUpFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x0, weight):
        ctx.save_for_backward(x0, weight)
        return F.linear(x0, weight)

    @staticmethod
    def backward(ctx, dy):
        x0, weight = ctx.saved_tensors
        K, N = weight.shape                                   # embed_dim, head_dim
        dy2 = dy.reshape(-1, K)
        dx0 = dw = None
        if ctx.needs_input_grad[0]:
            dx0 = (dy2 @ weight).reshape(x0.shape)
        if ctx.needs_input_grad[1]:
            x2 = x0.reshape(-1, N)
            if (skinny_ok(dy2, N) and weight.dtype == x2.dtype == torch.bfloat16 and dy2.stride(1) == 1 and x2.stride(1) == 1
                    and dy2.stride(0) % 8 == 0 and x2.stride(0) % 8 == 0 and dy2.data_ptr() % 16 == 0 and x2.data_ptr() % 16 == 0):
                lib = _lib.load()
                M = dy2.shape[0]
                with torch.cuda.device(dy2.device):
                    nws = lib.hdla_skinny_wgrad_workspace_bytes(_lib.HDLA_BF16, M, N, K)
                    ws = torch.empty(nws, dtype=torch.uint8, device=dy2.device)
                    dw = torch.empty(K, N, dtype=torch.bfloat16, device=dy2.device)
                    rc = lib.hdla_skinny_wgrad(_lib.HDLA_BF16, M, N, K, _lib.ptr(dy2), dy2.stride(0), _lib.ptr(x2),
                                               x2.stride(0), _lib.ptr(dw), _lib.ptr(ws), nws,
                                               _lib.current_stream(dy2.device))
                    _lib.check(rc, "hdla_skinny_wgrad")
            else:
                dw = dy2.t() @ x2
        return dx0, dw


@torch.compiler.disable
def low_rank_up(x0: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x0 [..., head_dim] @ weight[embed_dim, head_dim]^T`` with this library's kernel for the weight gradient."""
    return LowRankUpFunction.apply(x0, weight)

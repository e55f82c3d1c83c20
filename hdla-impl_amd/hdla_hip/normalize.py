"""Fused normalisation with an optional gate: the drop-in for the reference's ``normalize_fn`` and what sits on it.

* ``normalize_fn``            <- ``normalize_triton``, HRDPLR/normalizations/normalize/normalize/normalize_triton.py:452-499
  (same argument names, order and defaults), one call of ``hdla_normalize_fwd`` / ``hdla_normalize_bwd``
* ``NormalizeFunction``       <- ``NormalizeTriton``, normalize_triton.py:255-449 (saves its inputs; sigma is recomputed
  in the backward kernel instead of being stored)
* ``l2_norm``                 <- HRDPLR/normalizations/l2_norm.py:4-14
* ``RMSNorm``, ``RMSNormFusedGate``, ``SRMSNorm``, ``GroupRMSNorm``, ``GroupRMSNormFusedGate``, ``get_norm_fn``
  <- HRDPLR/normalizations/rms_norm.py:11-90, srms_norm.py, group_rms_norm.py:12-140, __init__.py:15-39, through the
  dispatch of ``NormOp`` (HRDPLR/normalizations/utils.py:9-74)

Covered: what the HDLA layer reaches (no mean subtraction, bias or residual; gate activation "sigmoid", before or
after the norm).  Anything else raises ``NotImplementedError``; tensors must live on the GPU.
"""
import ctypes
from typing import Optional

import torch
import torch.nn as nn

from . import _lib
from .chunk import _require_gpu
from .utils import contiguous

_GATE_POS = {"pre": 1, "post": 2}


def _norm_dims(x, weight, gate_pos, c, eps, num_groups):
    D = x.shape[-1]
    rows = x.numel() // D if D else 0
    return _lib.HdlaNormDims(rows, num_groups, D // num_groups, _lib.dtype_code(x.dtype),
                             _lib.dtype_code(weight.dtype) if weight is not None else _lib.HDLA_FP32,
                             gate_pos, float(c), float(eps))


class NormalizeFunction(torch.autograd.Function):

    @staticmethod
    @contiguous
    def forward(ctx, x, weight, gate, gate_pos, c, eps, num_groups):
        lib = _lib.load()
        with torch.cuda.device(x.device):
            dims = _norm_dims(x, weight, gate_pos, c, eps, num_groups)
            o = torch.empty_like(x)
            rc = lib.hdla_normalize_fwd(ctypes.byref(dims), _lib.ptr(x), _lib.ptr(weight), _lib.ptr(gate), _lib.ptr(o),
                                        _lib.current_stream(x.device))
            _lib.check(rc, "hdla_normalize_fwd")
        ctx.save_for_backward(x, weight, gate)
        ctx.cfg = (gate_pos, c, eps, num_groups)
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        x, weight, gate = ctx.saved_tensors
        gate_pos, c, eps, num_groups = ctx.cfg
        lib = _lib.load()
        do = do.to(x.dtype)
        with torch.cuda.device(x.device):
            dims = _norm_dims(x, weight, gate_pos, c, eps, num_groups)
            dx = torch.empty_like(x)
            dgate = torch.empty_like(x) if gate is not None else None
            dw = ws = None
            nws = 0
            if weight is not None:
                dw = torch.empty(x.shape[-1], dtype=torch.float32, device=x.device)
                nws = lib.hdla_normalize_workspace_bytes(ctypes.byref(dims))
                ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=x.device)
            rc = lib.hdla_normalize_bwd(ctypes.byref(dims), _lib.ptr(x), _lib.ptr(weight), _lib.ptr(gate), _lib.ptr(do),
                                        _lib.ptr(dx), _lib.ptr(dgate), _lib.ptr(dw), _lib.ptr(ws), nws,
                                        _lib.current_stream(x.device))
            _lib.check(rc, "hdla_normalize_bwd")
        if dw is not None:
            dw = dw.to(weight.dtype).reshape(weight.shape)
        return dx, dw, dgate, None, None, None, None


@torch.compiler.disable
def normalize_fn(
    x: torch.Tensor,
    weight: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    residual: Optional[torch.Tensor] = None,
    gate: Optional[torch.Tensor] = None,
    gate_act: str = "sigmoid",
    gate_pos: str = "pre",
    c: float = 1.0,
    eps: float = 1e-6,
    use_mean: bool = False,
    num_groups: int = 1,
    return_residual: bool = False,
) -> torch.Tensor:
    """``o = c / sqrt(E) * x' / sqrt(mean_E(x'^2) + eps) * weight`` per group of ``E = D / num_groups`` channels of the
    last dimension, with ``x' = x * sigmoid(gate)`` (``gate_pos == "pre"``) or ``o * sigmoid(gate)`` afterwards
    (``"post"``).  Signature of normalize_triton.py:452-465; ``o`` has ``x``'s dtype and shape."""
    assert x.shape[-1] % num_groups == 0, "The last dimension of x must be divisible by num_groups"
    if bias is not None or residual is not None or return_residual or use_mean:
        raise NotImplementedError("hdla_hip.normalize_fn covers the forms the HDLA layer uses: no bias, no residual, "
                                  "no mean subtraction")
    if gate is not None:
        if gate_act != "sigmoid":
            raise NotImplementedError(f"gate_act = {gate_act!r}: only 'sigmoid' is built")
        if gate_pos not in _GATE_POS:
            raise ValueError(f"gate_pos must be 'pre' or 'post', got {gate_pos!r}")
        if gate.shape != x.shape:
            raise ValueError(f"gate {tuple(gate.shape)} must have the shape of x {tuple(x.shape)}")
    if weight is not None and weight.numel() != x.shape[-1]:
        raise ValueError(f"weight must hold {x.shape[-1]} elements, got {tuple(weight.shape)}")
    _require_gpu(x, weight, gate)
    out_dtype = x.dtype
    if x.dtype == torch.float16:
        eps = max(eps, 1.6e-5)                                          # normalize_triton.py:281-282
        x = x.float()
    elif x.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported dtype {x.dtype}")
    if gate is not None:
        gate = gate.to(x.dtype)
    if weight is not None and weight.dtype not in (torch.bfloat16, torch.float32):
        weight = weight.float()
    o = NormalizeFunction.apply(x, weight, gate, _GATE_POS[gate_pos] if gate is not None else 0, c, eps, num_groups)
    return o.to(out_dtype)


def l2_norm(x: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """x / sqrt(|x|^2 + E eps) over the last dimension (HRDPLR/normalizations/l2_norm.py:4-14)."""
    return normalize_fn(x=x, weight=None, bias=None, residual=None, c=1, eps=eps, use_mean=False, num_groups=1)


class RMSNorm(nn.Module):
    """HRDPLR/normalizations/rms_norm.py:11-45 (without the residual arguments)."""

    def __init__(self, dim: int, eps: float = 1e-5, **kwargs):
        super().__init__()
        self.eps, self.dim = eps, dim
        self.weight = nn.Parameter(torch.ones(dim))

    def extra_repr(self) -> str:
        return f"dim={self.dim}, eps={self.eps}"

    def forward(self, x, residual=None, return_residual=False):
        return normalize_fn(x, self.weight, None, residual, c=self.dim ** 0.5, eps=self.eps,
                            return_residual=return_residual)


class SRMSNorm(nn.Module):
    """RMS norm without a weight (HRDPLR/normalizations/srms_norm.py)."""

    def __init__(self, dim: int, eps: float = 1e-5, **kwargs):
        super().__init__()
        self.eps, self.dim = eps, dim

    def extra_repr(self) -> str:
        return f"dim={self.dim}, eps={self.eps}"

    def forward(self, x, residual=None, return_residual=False):
        return normalize_fn(x, None, None, residual, c=self.dim ** 0.5, eps=self.eps, return_residual=return_residual)


class RMSNormFusedGate(nn.Module):
    """HRDPLR/normalizations/rms_norm.py:48-90: RMS norm over the whole last dimension of ``x * sigmoid(gate)``
    ("pre") or followed by ``* sigmoid(gate)`` ("post")."""

    def __init__(self, dim: int, eps: float = 1e-5, gate_act="sigmoid", gate_pos="pre", **kwargs):
        super().__init__()
        self.eps, self.dim, self.gate_act, self.gate_pos = eps, dim, gate_act, gate_pos
        self.weight = nn.Parameter(torch.ones(dim))

    def extra_repr(self) -> str:
        return f"dim={self.dim}, eps={self.eps}, gate_act={self.gate_act}, gate_pos={self.gate_pos}"

    def forward(self, x, gate):
        return normalize_fn(x, self.weight, gate=gate, gate_act=self.gate_act, gate_pos=self.gate_pos,
                            c=self.dim ** 0.5, eps=self.eps)


class GroupRMSNorm(nn.Module):
    """HRDPLR/normalizations/group_rms_norm.py:12-70: RMS norm per group of ``num_channels / num_groups`` channels.
    The reference's module creates a bias parameter but always passes ``None`` for it (group_rms_norm.py:56-58), so
    none is created here."""

    def __init__(self, num_channels: int, num_groups: int, eps: float = 1e-5, affine: bool = True, **kwargs):
        super().__init__()
        if num_channels % num_groups != 0:
            raise ValueError("num_channels must be divisible by num_groups")
        self.num_groups, self.num_channels, self.eps, self.affine = num_groups, num_channels, eps, affine
        if affine:
            self.weight = nn.Parameter(torch.ones(num_channels))
        else:
            self.register_parameter("weight", None)

    def extra_repr(self) -> str:
        return f"num_groups={self.num_groups}, num_channels={self.num_channels}, eps={self.eps}, affine={self.affine}"

    def forward(self, x):
        return normalize_fn(x, self.weight, c=(self.num_channels // self.num_groups) ** 0.5, eps=self.eps,
                            num_groups=self.num_groups)


class GroupRMSNormFusedGate(GroupRMSNorm):
    """HRDPLR/normalizations/group_rms_norm.py:73-140."""

    def __init__(self, num_channels: int, num_groups: int, eps: float = 1e-5, affine: bool = True,
                 gate_act="sigmoid", gate_pos="pre", **kwargs):
        super().__init__(num_channels, num_groups, eps, affine)
        self.gate_act, self.gate_pos = gate_act, gate_pos

    def forward(self, x, gate):
        return normalize_fn(x, self.weight, gate=gate, gate_act=self.gate_act, gate_pos=self.gate_pos,
                            c=(self.num_channels // self.num_groups) ** 0.5, eps=self.eps, num_groups=self.num_groups)


def get_norm_fn(norm_type: str):
    """The RMS family of HRDPLR/normalizations/__init__.py:15-39; the other types are not part of this library."""
    table = {"rmsnorm": RMSNorm, "rmsnorm_fused_gate": RMSNormFusedGate, "srmsnorm": SRMSNorm,
             "grouprmsnorm": GroupRMSNorm, "grouprmsnorm_fused_gate": GroupRMSNormFusedGate}
    if norm_type not in table:
        raise NotImplementedError(f"norm type {norm_type!r} is not built (available: {sorted(table)})")
    return table[norm_type]

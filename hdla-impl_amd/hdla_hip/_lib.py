"""ctypes binding of libhdla_hip.so (the C ABI declared in include/hdla_hip.h).

The library is the only compute path: if it cannot be loaded every operator raises, there is no fallback.
"""
import ctypes
import os
from typing import Optional

import torch

HDLA_BF16, HDLA_FP32 = 0, 1
HDLA_VERSION = 200          # the header this binding was written against (struct layouts, entry points)
ROUTE_AUTO, ROUTE_CLASSIC, ROUTE_FUSED = 0, 1, 2
_ROUTES = {"": ROUTE_AUTO, "auto": ROUTE_AUTO, "classic": ROUTE_CLASSIC, "fused": ROUTE_FUSED}
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libhdla_hip.so"
_lib = None


class HdlaDims(ctypes.Structure):
    _fields_ = [
        ("B", ctypes.c_int32), ("T", ctypes.c_int32), ("H", ctypes.c_int32), ("K", ctypes.c_int32),
        ("V", ctypes.c_int32), ("R", ctypes.c_int32), ("N", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32), ("gk_dtype", ctypes.c_int32), ("scale", ctypes.c_float),
        ("cu_seqlens", ctypes.c_void_p), ("route", ctypes.c_int32), ("segments", ctypes.c_int32),
    ]


class HdlaWsLayout(ctypes.Structure):
    _names = ["nch", "W", "UT", "KGT", "BGT", "VTT", "EGL", "QG", "AQK", "AQB", "AQBT", "QGT", "TM",
              "HC", "DHC", "DVN", "STRONG", "SA_STRIDE", "SB_STRIDE", "CHUNK_OFF", "CHUNK_SEQ", "total", "ERR"]
    _fields_ = [(n, ctypes.c_int64) for n in _names]


class HdlaNormDims(ctypes.Structure):
    """struct hdla_norm_dims of include/hdla_hip.h."""
    _fields_ = [("rows", ctypes.c_int64), ("G", ctypes.c_int32), ("E", ctypes.c_int32), ("dtype", ctypes.c_int32),
                ("weight_dtype", ctypes.c_int32), ("gate_pos", ctypes.c_int32), ("c", ctypes.c_float),
                ("eps", ctypes.c_float)]


class HdlaPreDims(ctypes.Structure):
    """struct hdla_pre_dims of include/hdla_hip.h."""
    _fields_ = [("rows", ctypes.c_int64)] + [(n, ctypes.c_int32) for n in (
        "H", "D", "dtype", "ldy", "col_q", "col_k", "col_v", "col_beta", "norm_q", "norm_k", "norm_v")] + [
        ("beta_scale", ctypes.c_float), ("eps", ctypes.c_float)]


class HdlaError(RuntimeError):
    pass


def lib_path() -> str:
    return os.environ.get("HDLA_HIP_LIB", os.path.join(_HERE, _LIB_NAME))


def load():
    """Load the shared library once; raise if it is missing (build it with __graft_entry__.build() or
    `make -C hdla-impl_amd/csrc`)."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise HdlaError(f"{path} not found: build the HIP library first (make -C hdla-impl_amd/csrc); "
                        "there is no CPU or PyTorch fallback for these operators")
    lib = ctypes.CDLL(path)
    P, F = ctypes.c_void_p, ctypes.POINTER(HdlaDims)
    lib.hdla_version.restype = ctypes.c_int
    lib.hdla_version.argtypes = []
    if lib.hdla_version() != HDLA_VERSION:
        raise HdlaError(f"{path} is version {lib.hdla_version()} of the C ABI, this binding needs {HDLA_VERSION}: "
                        "rebuild the library (make -C hdla-impl_amd/csrc)")
    lib.hdla_strerror.restype = ctypes.c_char_p
    lib.hdla_strerror.argtypes = [ctypes.c_int]
    lib.hdla_workspace_bytes.restype = ctypes.c_size_t
    lib.hdla_workspace_bytes.argtypes = [F, ctypes.c_int]
    lib.hdla_workspace_layout.restype = ctypes.c_int
    lib.hdla_workspace_layout.argtypes = [F, ctypes.c_int, ctypes.POINTER(HdlaWsLayout)]
    lib.hdla_chunk_fwd.restype = ctypes.c_int
    lib.hdla_chunk_fwd.argtypes = [F] + [P] * 9 + [P, ctypes.c_size_t, P]
    lib.hdla_chunk_fwd_static.restype = ctypes.c_int
    lib.hdla_chunk_fwd_static.argtypes = [F] + [P] * 9 + [P]
    lib.hdla_chunk_bwd.restype = ctypes.c_int
    lib.hdla_chunk_bwd.argtypes = [F] + [P] * 16 + [P, ctypes.c_size_t, P]
    lib.hdla_param_chunk_fwd.restype = ctypes.c_int
    lib.hdla_param_chunk_fwd.argtypes = [F] + [P] * 8 + [P, ctypes.c_size_t, P]
    lib.hdla_param_chunk_bwd.restype = ctypes.c_int
    lib.hdla_param_chunk_bwd.argtypes = [F] + [P] * 14 + [P, ctypes.c_size_t, P]
    lib.hdla_boundary_bytes.restype = ctypes.c_size_t
    lib.hdla_boundary_bytes.argtypes = [F]
    lib.hdla_chunk_fwd_b.restype = ctypes.c_int
    lib.hdla_chunk_fwd_b.argtypes = [F] + [P] * 10 + [P, ctypes.c_size_t, P, ctypes.c_size_t, P]
    lib.hdla_chunk_bwd_b.restype = ctypes.c_int
    lib.hdla_chunk_bwd_b.argtypes = [F] + [P] * 18 + [P, ctypes.c_size_t, P, ctypes.c_size_t, P]
    lib.hdla_chunk_fwd_keep.restype = ctypes.c_int
    lib.hdla_chunk_fwd_keep.argtypes = [F] + [P] * 10 + [P, ctypes.c_size_t, P]
    lib.hdla_chunk_bwd_kept.restype = ctypes.c_int
    lib.hdla_chunk_bwd_kept.argtypes = [F] + [P] * 18 + [P, ctypes.c_size_t, P, ctypes.c_size_t, P]
    lib.hdla_chunk_stages.restype = ctypes.c_int
    lib.hdla_chunk_stages.argtypes = [F, ctypes.c_int, ctypes.c_int] + [P] * 18 + [P, ctypes.c_size_t, P]
    lib.hdla_calib_stream.restype = ctypes.c_int
    lib.hdla_calib_stream.argtypes = [ctypes.POINTER(P), ctypes.c_int, ctypes.POINTER(P), ctypes.c_int, ctypes.c_size_t, P]
    lib.hdla_recurrent_fwd.restype = ctypes.c_int
    lib.hdla_recurrent_fwd.argtypes = [F] + [P] * 6 + [ctypes.c_int] + [P] * 4
    lib.hdla_param_recurrent_fwd.restype = ctypes.c_int
    lib.hdla_param_recurrent_fwd.argtypes = [F] + [P] * 5 + [ctypes.c_int] + [P] * 4
    NF = ctypes.POINTER(HdlaNormDims)
    lib.hdla_normalize_workspace_bytes.restype = ctypes.c_size_t
    lib.hdla_normalize_workspace_bytes.argtypes = [NF]
    lib.hdla_normalize_fwd.restype = ctypes.c_int
    lib.hdla_normalize_fwd.argtypes = [NF] + [P] * 5
    lib.hdla_normalize_bwd.restype = ctypes.c_int
    lib.hdla_normalize_bwd.argtypes = [NF] + [P] * 8 + [ctypes.c_size_t, P]
    PF = ctypes.POINTER(HdlaPreDims)
    lib.hdla_layer_pre_fwd.restype = ctypes.c_int
    lib.hdla_layer_pre_fwd.argtypes = [PF] + [P] * 6
    lib.hdla_layer_pre_bwd.restype = ctypes.c_int
    lib.hdla_layer_pre_bwd.argtypes = [PF] + [P] * 7
    lib.hdla_logsigmoid_fwd.restype = ctypes.c_int
    lib.hdla_logsigmoid_fwd.argtypes = [ctypes.c_int, ctypes.c_int64, P, P, P]
    lib.hdla_logsigmoid_bwd.restype = ctypes.c_int
    lib.hdla_logsigmoid_bwd.argtypes = [ctypes.c_int, ctypes.c_int64, P, P, P, P]
    lib.hdla_skinny_wgrad.restype = ctypes.c_int
    lib.hdla_skinny_wgrad.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, P, ctypes.c_int64, P,
                                      ctypes.c_int64, P, P, ctypes.c_size_t, P]
    lib.hdla_skinny_wgrad_workspace_bytes.restype = ctypes.c_size_t
    lib.hdla_skinny_wgrad_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().hdla_strerror(rc).decode()
        raise HdlaError(f"{what} failed with code {rc}: {msg}")


def ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return HDLA_BF16
    if dt == torch.float32:
        return HDLA_FP32
    raise HdlaError(f"unsupported dtype {dt}")


def default_route() -> int:
    """Launch plan of the chunked operators when the caller does not say: environment variable HDLA_HIP_ROUTE =
    auto (the library chooses: the fused kernels where they are built), classic or fused."""
    name = os.environ.get("HDLA_HIP_ROUTE", "auto").lower()
    if name not in _ROUTES:
        raise HdlaError(f"HDLA_HIP_ROUTE must be one of auto, classic, fused (got {name!r})")
    return _ROUTES[name]


def default_segments() -> int:
    """Time segments per sequence on the fused route: environment variable HDLA_HIP_SEGMENTS, 0 = the library chooses."""
    return int(os.environ.get("HDLA_HIP_SEGMENTS", "0"))


def make_dims(B, T, H, K, V, R, N, in_dtype, gk_dtype, scale, cu_seqlens: Optional[torch.Tensor],
              route: Optional[int] = None, segments: Optional[int] = None) -> HdlaDims:
    return HdlaDims(B, T, H, K, V, R, N, dtype_code(in_dtype), dtype_code(gk_dtype), float(scale),
                    None if cu_seqlens is None else cu_seqlens.data_ptr(),
                    default_route() if route is None else route, default_segments() if segments is None else segments)


def keep_boundaries_default() -> bool:
    """Whether the forward pass of the chunked operators hands the states at the time-segment boundaries (fused route:
    64 KiB per sequence, head and segment) to the backward pass, which otherwise re-derives them from the inputs with
    one more pass.  On by default; HDLA_HIP_INPUTS_ONLY=1 keeps strictly the inputs between the passes."""
    return os.environ.get("HDLA_HIP_INPUTS_ONLY", "0") in ("", "0", "false", "False")


def boundary(dims: HdlaDims, device) -> Optional[torch.Tensor]:
    """An empty boundary record for these dimensions, or None where the route has none."""
    n = load().hdla_boundary_bytes(ctypes.byref(dims))
    return torch.empty(n, dtype=torch.uint8, device=device) if n else None


def check_cu_seqlens(cu_seqlens: torch.Tensor, T: int) -> None:
    """Validate a packed-sequence table that is still on the CPU (free: no device synchronisation): it must start at
    0, end at T and never decrease.  A table that already lives on the GPU is not read back; the kernels force its
    entries into [0, T], so a bad one cannot cause an access outside the tensors, but rows that belong to no sequence
    are then left unwritten in the outputs."""
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
        raise ValueError(f"cu_seqlens must be a 1-d tensor of N+1 >= 2 entries, got shape {tuple(cu_seqlens.shape)}")
    if cu_seqlens.is_cuda:
        return
    cu = cu_seqlens.to(torch.int64)
    if int(cu[0]) != 0 or int(cu[-1]) != T or bool((cu[1:] < cu[:-1]).any()):
        raise ValueError(f"cu_seqlens must start at 0, end at the number of tokens ({T}) and never decrease, "
                         f"got {cu.tolist()}")


PASS_FWD, PASS_BWD, PASS_FWD_KEEP, PASS_BWD_KEPT = 0, 1, 2, 3


def keep_forward_default() -> bool:
    """Whether the chunked operators keep the forward pass's per-chunk intermediates for the backward pass when the
    caller does not say (``keep_forward=None``): environment variable HDLA_HIP_KEEP_FORWARD=1.  Off by default: the
    reference keeps only the inputs between the passes (HRDPLR/hrdplr.py:137) and so does this library unless asked."""
    return os.environ.get("HDLA_HIP_KEEP_FORWARD", "0") not in ("", "0", "false", "False")


def current_stream(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def workspace(dims: HdlaDims, pass_: int, device) -> torch.Tensor:
    n = load().hdla_workspace_bytes(ctypes.byref(dims), pass_)
    if n == 0:
        raise HdlaError("hdla_workspace_bytes rejected the dimensions "
                        f"(B={dims.B},T={dims.T},H={dims.H},K={dims.K},V={dims.V},R={dims.R},N={dims.N})")
    return torch.empty(n, dtype=torch.uint8, device=device)


def workspace_layout(dims: HdlaDims, pass_: int) -> dict:
    out = HdlaWsLayout()
    check(load().hdla_workspace_layout(ctypes.byref(dims), pass_, ctypes.byref(out)), "hdla_workspace_layout")
    return {n: getattr(out, n) for n in HdlaWsLayout._names}

"""hdla_chunk_fwd_static (the entry point that allocates nothing) against hdla_chunk_fwd, through the C ABI.

Both run the same kernels, the first on the library's built-in scratch array, the second on a caller-owned workspace,
so the results must be equal bit for bit.  Two calls in a row share the array; the second is smaller, so whatever the
first left behind lies beyond (and inside) what the second uses."""
import ctypes

import pytest
import torch

from hdla_hip import _lib
from hdla_hip.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
STATIC_BYTES = 64 << 20


def _call(fn_static, dims, t, h0, with_ws):
    lib = _lib.load()
    o = torch.full_like(t[2], float("nan"))
    ht = torch.full((dims.N, dims.H, dims.K, dims.V), float("nan"), dtype=torch.float32, device=DEV)
    args = [ctypes.byref(dims)] + [_lib.ptr(x) for x in t] + [_lib.ptr(h0), _lib.ptr(o), _lib.ptr(ht)]
    if with_ws:
        ws = _lib.workspace(dims, 0, DEV)
        rc = lib.hdla_chunk_fwd(*args, _lib.ptr(ws), ws.numel(), _lib.current_stream(DEV))
    else:
        rc = lib.hdla_chunk_fwd_static(*args, _lib.current_stream(DEV))
    torch.cuda.synchronize()
    return rc, o, ht


def _case(seed, B, T, H, K, V, dtype, cu=None):
    inp = make_inputs(seed, B, T, H, K, V, gk_div=2.0, n_states=None if cu is None else len(cu) - 1)
    t = [x.to(dtype).to(DEV).contiguous() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    h0 = inp.h0.float().to(DEV).contiguous()
    cu_t = None if cu is None else torch.tensor(cu, dtype=torch.int64, device=DEV)
    N = B if cu is None else len(cu) - 1
    dims = _lib.make_dims(B, T, H, K, V, 2, N, dtype, dtype, 0.5, cu_t)
    return dims, t, h0, cu_t


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_two_calls_in_a_row_match_the_workspace_entry_point(dtype):
    # first call: a large shape (most of the array for bf16); second: a smaller one, other head size, packed sequences
    big = _case(31, 2, 1000, 8, 64, 64, dtype)
    small = _case(32, 1, 150, 3, 128, 64, dtype, cu=[0, 40, 41, 150])
    for dims, t, h0, _cu in (big, small):
        print("static call", dims.B, dims.T, dims.H, dims.K, dims.V, dtype, flush=True)
        need = _lib.load().hdla_workspace_bytes(ctypes.byref(dims), 0)
        assert 0 < need <= STATIC_BYTES
        rc_s, o_s, ht_s = _call(True, dims, t, h0, with_ws=False)
        rc_w, o_w, ht_w = _call(False, dims, t, h0, with_ws=True)
        assert rc_s == 0 and rc_w == 0
        assert torch.isfinite(o_w.float()).all() and torch.isfinite(ht_w).all()
        assert torch.equal(o_s, o_w) and torch.equal(ht_s, ht_w)


def test_size_limit_and_argument_errors():
    lib = _lib.load()
    dims, t, h0, _ = _case(33, 8, 2048, 16, 64, 64, torch.bfloat16)      # 117 MB of workspace or more: beyond the array
    assert lib.hdla_workspace_bytes(ctypes.byref(dims), 0) > STATIC_BYTES
    rc, _, _ = _call(True, dims, t, h0, with_ws=False)
    assert rc == -8 and b"HDLA_STATIC_WORKSPACE_BYTES" in lib.hdla_strerror(rc)
    bad = _lib.make_dims(1, 32, 2, 48, 64, 2, 1, torch.bfloat16, torch.bfloat16, 1.0, None)   # unsupported K
    assert lib.hdla_chunk_fwd_static(ctypes.byref(bad), *([None] * 9), None) == -2

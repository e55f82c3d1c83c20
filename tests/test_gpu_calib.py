"""The streaming kernel behind `bench.py --workload copy`: every mix it offers writes exactly what it read, over the
whole of the buffers and not beyond, and unsupported arguments are refused."""
import ctypes

import pytest
import torch

from hdla_hip import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _call(lib, reads, writes, nbytes):
    rd = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in reads], *([None] * (3 - len(reads))))
    wr = (ctypes.c_void_p * 2)(*[t.data_ptr() for t in writes], *([None] * (2 - len(writes))))
    return lib.hdla_calib_stream(rd, len(reads), wr, len(writes), nbytes, _lib.current_stream(torch.device(DEV)))


@pytest.mark.parametrize("nr,nw", [(1, 0), (0, 1), (1, 1), (2, 1), (3, 1), (1, 2)])
@pytest.mark.parametrize("n", [16, 4096 * 256 * 16 * 2 + 48, 5 * 1024 * 1024 + 16])
def test_every_mix_copies_sums(nr, nw, n):
    lib = _lib.load()
    words = n // 4
    g = torch.Generator().manual_seed(n + nr)
    reads = [torch.randint(-1000, 1000, (words + 8,), dtype=torch.int32, generator=g).to(DEV) for _ in range(nr)]
    writes = [torch.full((words + 8,), 77, dtype=torch.int32, device=DEV) for _ in range(nw)]
    before = [r.clone() for r in reads]
    assert _call(lib, reads, writes, n) == 0
    torch.cuda.synchronize()
    want = torch.tensor([1, 2, 3, 4], dtype=torch.int32, device=DEV).repeat(words // 4)
    for r in reads:
        want = want + r[:words]
    for w_ in writes:
        assert torch.equal(w_[:words], want)
        assert bool((w_[words:] == 77).all())            # nothing past the end
    for r, b in zip(reads, before):
        assert torch.equal(r, b)


def test_refusals():
    lib = _lib.load()
    x = torch.zeros(64, dtype=torch.int32, device=DEV)
    y = torch.zeros(64, dtype=torch.int32, device=DEV)
    assert _call(lib, [x], [y], 40) == -2                 # not a multiple of 16
    assert _call(lib, [x], [y], 0) == -2
    assert _call(lib, [x, x, x], [y, y], 64) == -2        # mix not offered
    assert _call(lib, [], [], 64) == -2
    assert _call(lib, [x[1:]], [y], 64) == -6             # misaligned
    rd = (ctypes.c_void_p * 3)(None, None, None)
    wr = (ctypes.c_void_p * 2)(y.data_ptr(), None)
    assert lib.hdla_calib_stream(rd, 1, wr, 1, 64, None) == -1

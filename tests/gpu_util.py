"""Helpers shared by the GPU parity tests: decoding of workspace buffers written by the HIP kernels."""
import torch


def _raw(ws: torch.Tensor, off: int, count: int, dtype: torch.dtype, stride: int = 0, slots: int = 1) -> torch.Tensor:
    """`count` elements at byte offset `off`; with `stride`, they are `slots` equal pieces `stride` bytes apart
    (the parts of the scan operand blocks, one block per (head, chunk) slot)."""
    nbytes = count * torch.empty((), dtype=dtype).element_size()
    if not stride:
        return ws[off:off + nbytes].view(dtype)
    assert nbytes % slots == 0 and nbytes // slots <= stride
    return torch.as_strided(ws, (slots, nbytes // slots), (stride, 1), off).contiguous().view(-1).view(dtype)


def tiles(ws, off, dtype, H, nch, *lead, stride=0):
    """Buffer of 16x16 tiles in fragment order -> float64 tensor [H, nch, *lead, 16 (row), 16 (inner)].

    Element 4*lane + i of a tile is row lane % 16, inner index 4*(lane // 16) + i."""
    n = 1
    for x in lead:
        n *= x
    t = _raw(ws, off, H * nch * n * 256, dtype, stride, H * nch).double().reshape(H, nch, *lead, 4, 16, 4)   # [g][c][i]
    nd = t.dim()
    t = t.transpose(nd - 3, nd - 2)                                                          # [c][g][i]
    return t.reshape(H, nch, *lead, 16, 16).cpu()


def pair_tiles(ws, off, dtype, H, nch, *lead, stride=0):
    """Like tiles(), for buffers whose tiles are stored interleaved in pairs along the last lead dimension:
    element 8*lane + 4*which + i of a 512-element pair block belongs to tile `which` of the pair."""
    n = 1
    for x in lead:
        n *= x
    assert lead[-1] % 2 == 0
    t = _raw(ws, off, H * nch * n * 256, dtype, stride, H * nch).double()
    t = t.reshape(H, nch, *lead[:-1], lead[-1] // 2, 64, 2, 4)
    nd = t.dim()
    t = t.transpose(nd - 3, nd - 2)                                   # [npairs, 2, 64, 4]
    t = t.reshape(H, nch, *lead, 4, 16, 4)
    nd = t.dim()
    t = t.transpose(nd - 3, nd - 2)
    return t.reshape(H, nch, *lead, 16, 16).cpu()


def rows(ws, off, dtype, H, nch, *shape, stride=0):
    n = 1
    for x in shape:
        n *= x
    return _raw(ws, off, H * nch * n, dtype, stride, H * nch).double().reshape(H, nch, *shape).cpu()


def cat_tiles(t, dim_tiles, transpose=False):
    """[..., nt, 16, 16] -> rows x (nt*16) (or its transpose view when the tiles hold the transposed matrix).

    With transpose=False the tile index runs along the inner dimension: result [..., 16, nt*16].
    With transpose=True each tile is (rows = tiled dimension, inner = other): result [..., 16 (inner), nt*16]."""
    assert dim_tiles == t.dim() - 3
    if not transpose:
        return torch.cat([t[..., i, :, :] for i in range(t.shape[-3])], dim=-1)
    return torch.cat([t[..., i, :, :].transpose(-1, -2) for i in range(t.shape[-3])], dim=-1)

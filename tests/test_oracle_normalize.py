"""Pins of oracle/normalize_oracle.py (CPU): the restated formula against library routines and closed forms, chosen so
that a misplaced eps, a wrong constant, a wrong group reshape or a gate on the wrong side fails one of them."""
import pytest
import torch
import torch.nn.functional as F

from oracle import normalize_oracle as NO


def _x(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_rms_form_is_the_library_rms_norm():
    # c = sqrt(E): o = x / sqrt(mean(x^2) + eps) * w, which is torch.nn.functional.rms_norm; eps = 0.5 is large
    # enough to tell sqrt(mean + eps) from sqrt(sum + eps) or sqrt(mean) + eps
    x, w = _x(0, 3, 5, 96), _x(1, 96)
    ref = F.rms_norm(x, (96,), w, eps=0.5)
    assert torch.allclose(NO.normalize(x, w, c=96 ** 0.5, eps=0.5), ref, rtol=1e-12, atol=1e-12)
    other = 96 ** 0.5 * x / torch.sqrt((x * x).sum(-1, keepdim=True) + 0.5) * w        # normalize_torch.py:76-77
    assert not torch.allclose(other, ref, rtol=1e-3, atol=1e-3)


def test_l2_norm_closed_form_and_limit():
    x = _x(2, 4, 7, 64)
    got = NO.l2_norm(x, eps=1e-5)
    assert torch.allclose(got, x / torch.sqrt((x * x).sum(-1, keepdim=True) + 64 * 1e-5), rtol=1e-12, atol=1e-12)
    assert torch.allclose(NO.l2_norm(x, eps=0.0), F.normalize(x, dim=-1), rtol=1e-12, atol=1e-12)
    assert torch.allclose(NO.l2_norm(x, eps=0.0).norm(dim=-1), torch.ones(4, 7, dtype=torch.float64))


def test_groups_are_independent_rows():
    x, w = _x(3, 6, 128), _x(4, 128)
    got = NO.normalize(x, w, c=32 ** 0.5, eps=1e-3, num_groups=4)
    ref = F.rms_norm(x.reshape(6, 4, 32), (32,), None, eps=1e-3).reshape(6, 128) * w
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-12)


def test_gate_before_and_after():
    x, g, w = _x(5, 2, 9, 64), _x(6, 2, 9, 64), _x(7, 64)
    s = torch.sigmoid(g)
    pre = NO.rms_norm_fused_gate(x, g, w, eps=1e-2, gate_pos="pre")
    post = NO.rms_norm_fused_gate(x, g, w, eps=1e-2, gate_pos="post")
    assert torch.allclose(pre, F.rms_norm(x * s, (64,), w, eps=1e-2), rtol=1e-12, atol=1e-12)
    assert torch.allclose(post, F.rms_norm(x, (64,), w, eps=1e-2) * s, rtol=1e-12, atol=1e-12)
    assert not torch.allclose(pre, post, rtol=1e-2, atol=1e-2)


def test_scale_invariance_and_output_rms():
    # without eps the result does not depend on the scale of x, and its rms over a group is c / sqrt(E)
    x = _x(8, 5, 48)
    a, b = NO.normalize(x, c=3.0, eps=0.0), NO.normalize(7.5 * x, c=3.0, eps=0.0)
    assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)
    assert torch.allclose((a * a).mean(-1).sqrt(), torch.full((5,), 3.0 / 48 ** 0.5, dtype=torch.float64))

"""Pins oracle/conv_oracle.py (CPU only) with checks that do not retype its formula."""
import math

import torch
import torch.nn.functional as F

from oracle.conv_oracle import conv1d_silu


def _rand(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64)


def test_matches_the_library_convolution_the_reference_calls():
    for width in (1, 3, 7, 9):
        x, w, b = _rand(3, 29, 10), _rand(10, 1, width, seed=1), _rand(10, seed=2)
        ref = F.silu(F.conv1d(x.transpose(1, 2), w, b, padding=width // 2, groups=10)).transpose(1, 2)
        torch.testing.assert_close(conv1d_silu(x, w, b), ref, rtol=1e-12, atol=1e-12)
        ref = F.silu(F.conv1d(x.transpose(1, 2), w, None, padding=width // 2, groups=10)).transpose(1, 2)
        torch.testing.assert_close(conv1d_silu(x, w), ref, rtol=1e-12, atol=1e-12)


def test_scalar_loop_on_a_tiny_case():
    x, w, b = _rand(2, 5, 3), _rand(3, 3, seed=1), _rand(3, seed=2)
    got = conv1d_silu(x, w, b)
    for bb in range(2):
        for l in range(5):
            for c in range(3):
                pre = b[c].item()
                for k in range(3):
                    j = l + k - 1
                    if 0 <= j < 5:
                        pre += w[c, k].item() * x[bb, j, c].item()
                assert abs(got[bb, l, c].item() - pre / (1.0 + math.exp(-pre))) < 1e-12


def test_identity_filter_is_plain_silu():
    x = _rand(2, 11, 4)
    w = torch.zeros(4, 7, dtype=torch.float64)
    w[:, 3] = 1.0
    torch.testing.assert_close(conv1d_silu(x, w), F.silu(x), rtol=1e-12, atol=1e-12)


def test_gradcheck():
    x, w, b = _rand(1, 9, 3).requires_grad_(), _rand(3, 5, seed=1).requires_grad_(), _rand(3, seed=2).requires_grad_()
    assert torch.autograd.gradcheck(conv1d_silu, (x, w, b), eps=1e-6, atol=1e-6)

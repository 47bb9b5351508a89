"""Pins oracle/rmsnorm_oracle.py (CPU only) with checks that do not retype its formula."""
import math

import torch
import torch.nn.functional as F

from oracle.rmsnorm_oracle import rms_norm_gated


def _rand(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64)


def test_plain_norm_matches_torch_rms_norm():
    x, w = _rand(5, 48), _rand(48, seed=1)
    ref = F.rms_norm(x, (48,), weight=w, eps=1e-5)
    torch.testing.assert_close(rms_norm_gated(x, w, eps=1e-5), ref, rtol=1e-12, atol=1e-12)


def test_scalar_loop_on_a_tiny_case():
    x, w, b, z = _rand(2, 6), _rand(6, seed=1), _rand(6, seed=2), _rand(2, 6, seed=3)
    for before in (True, False):
        got = rms_norm_gated(x, w, b, z, eps=1e-3, group_size=3, norm_before_gate=before)
        for r in range(2):
            for g in range(2):
                vals = []
                for j in range(3):
                    v = x[r, 3 * g + j].item()
                    zz = z[r, 3 * g + j].item()
                    if not before:
                        v = v * zz / (1.0 + math.exp(-zz))
                    vals.append(v)
                rstd = 1.0 / math.sqrt(sum(v * v for v in vals) / 3 + 1e-3)
                for j in range(3):
                    zz = z[r, 3 * g + j].item()
                    y = vals[j] * rstd * w[3 * g + j].item() + b[3 * g + j].item()
                    if before:
                        y = y * zz / (1.0 + math.exp(-zz))
                    assert abs(got[r, 3 * g + j].item() - y) < 1e-12


def test_gate_orders_by_their_definitions():
    x, w, z = _rand(4, 32), _rand(32, seed=1), _rand(4, 32, seed=2)
    plain = lambda t: rms_norm_gated(t, w, eps=1e-6)   # noqa: E731
    torch.testing.assert_close(rms_norm_gated(x, w, z=z, norm_before_gate=True), plain(x) * F.silu(z), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(rms_norm_gated(x, w, z=z, norm_before_gate=False), plain(x * F.silu(z)), rtol=1e-12, atol=1e-12)


def test_groups_are_independent_rows():
    x, w = _rand(3, 24), _rand(24, seed=1)
    got = rms_norm_gated(x, w, group_size=8, eps=1e-6)
    ones = torch.ones(8, dtype=torch.float64)
    ref = rms_norm_gated(x.reshape(9, 8), ones, eps=1e-6).reshape(3, 24) * w
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)


def test_scale_invariance_without_eps():
    x, w = _rand(3, 16), _rand(16, seed=1)
    torch.testing.assert_close(rms_norm_gated(7.5 * x, w, eps=0.0), rms_norm_gated(x, w, eps=0.0), rtol=1e-12, atol=1e-12)


def test_gradcheck():
    x, w, b, z = (t.requires_grad_(True) for t in (_rand(2, 8), _rand(8, seed=1), _rand(8, seed=2), _rand(2, 8, seed=3)))
    for before in (True, False):
        assert torch.autograd.gradcheck(lambda a, c, d, e: rms_norm_gated(a, c, d, e, 1e-5, 4, before), (x, w, b, z))


# ---- the LayerNorm of the same reference kernels (is_rms_norm=False) ----
def test_layer_norm_matches_torch_layer_norm_and_group_norm():
    x, w, b = _rand(5, 48), _rand(48, seed=1), _rand(48, seed=2)
    ref = F.layer_norm(x, (48,), weight=w, bias=b, eps=1e-5)
    torch.testing.assert_close(rms_norm_gated(x, w, b, eps=1e-5, is_rms_norm=False), ref, rtol=1e-12, atol=1e-12)
    # groups of 12 columns = torch's group norm with 4 groups over the channel axis
    refg = F.group_norm(x, 4, weight=w, bias=b, eps=1e-5)
    torch.testing.assert_close(rms_norm_gated(x, w, b, eps=1e-5, group_size=12, is_rms_norm=False), refg, rtol=1e-12, atol=1e-12)


def test_layer_norm_is_shift_invariant_and_gates_by_definition():
    x, w, z = _rand(4, 32), _rand(32, seed=1), _rand(4, 32, seed=2)
    ln = lambda t: rms_norm_gated(t, w, eps=1e-6, is_rms_norm=False)   # noqa: E731
    torch.testing.assert_close(ln(x + 3.25), ln(x), rtol=1e-10, atol=1e-10)          # the RMS norm is not: see below
    assert (rms_norm_gated(x + 3.25, w, eps=1e-6) - rms_norm_gated(x, w, eps=1e-6)).abs().max() > 0.1
    torch.testing.assert_close(rms_norm_gated(x, w, z=z, norm_before_gate=True, is_rms_norm=False), ln(x) * F.silu(z), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(rms_norm_gated(x, w, z=z, norm_before_gate=False, is_rms_norm=False), ln(x * F.silu(z)), rtol=1e-12, atol=1e-12)

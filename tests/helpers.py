"""Shared helpers of the test-suite: seeded inputs, tolerances, comparison."""
import math
import os

import torch

from oracle import bimamba2_oracle as O

# tolerances of the parity contract: float32 rtol = atol = 1e-4; bfloat16 / float16 rtol = atol = 2e-2
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def make_case(batch, seqlen, nheads, headdim, ngroups, dstate, dtype=torch.float32, seed=0, with_z=False,
              with_D=True, D_has_hdim=False, with_bias=True, ref_style=False):
    """Inputs on the CPU.  x, B, C, z are rounded to `dtype` (so the oracle sees exactly what the kernels see).
    ref_style=True uses the distributions of the reference's tests (tests/fixtures/fwd.py:14-28 there):
    A = -0.5|N(0,1)|, dt_bias = 0.5 N(0,1)."""
    inp = O.make_inputs(batch, seqlen, nheads, headdim, ngroups, dstate, seed=seed, dtype=dtype, with_z=with_z,
                        with_D=with_D, D_has_hdim=D_has_hdim)
    if ref_style:
        g = torch.Generator().manual_seed(seed + 1)
        inp["A"] = -0.5 * torch.randn(nheads, generator=g).abs()
        inp["dt_bias"] = 0.5 * torch.randn(nheads, generator=g)
    if not with_bias:
        inp["dt_bias"] = None
    return inp


def to64(inp):
    return {k: (v.double() if torch.is_tensor(v) else v) for k, v in inp.items()}


def to_dev(inp, device="cuda"):
    return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in inp.items()}


# Every comparison leaves a record here; tests/conftest.py writes them out at the end of the session when the
# environment variable BIMAMBA2_PARITY_MARGINS names a file.  `strict` is max |err| / (tol * (1 + |ref|)), the
# plain rtol = atol = tol criterion; `scaled` the same with atol in units of max(1, RMS(ref)).
MARGINS = []

# For 16-bit inputs, the gradients that are sums of rounded terms over heads x headdim (dB, dC), over headdim / dstate and a
# chunk (ddt), or over the whole batch and sequence (dA, dD, ddt_bias), and the gradients of the initial states (sums over
# the sequence), take their absolute tolerance in units of the tensor's RMS (assert_close(scaled=True)).  Everything else
# - out, out_x, final states, dx, dz, every forward intermediate, and every tensor of a float32 case - is held to the
# plain criterion.
REDUCED = frozenset(("ddt", "dA", "dD", "ddt_bias", "dB", "dC", "dinitial_f", "dinitial_b"))


def is_reduced(name, dtype):
    return dtype != torch.float32 and name in REDUCED


def _record(name, dtype, tol, strict, scaled, mode, n):
    MARGINS.append({"test": os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], "tensor": name,
                    "dtype": str(dtype).replace("torch.", ""), "tol": tol, "strict": strict, "scaled": scaled,
                    "mode": mode, "numel": n})


def assert_close(got, ref, dtype, name="", scale=1.0, scaled=False):
    """Default (strict): |got - ref| <= tol + tol * |ref| for EVERY element, tol = 1e-4 (float32) or 2e-2 (16-bit):
    plain rtol = atol = tol.
    scaled=True: |got - ref| <= tol * (s + |ref|) with s = max(1, RMS(ref)), i.e. the absolute tolerance in units of
    the tensor's own magnitude, and for 16-bit types up to 0.1 % of the elements may exceed the bound by at most 4x.
    It is for tensors that are long sums of rounded terms (the rounding error of a sum scales with the size of its
    terms, not with the possibly cancelling result): gradients summed over heads, positions or the batch whose
    magnitude is far from 1.  Which tensors use it, and by how much the strict bound is missed there, is recorded
    in MARGINS."""
    tol = TOL[dtype] * scale
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - ref).abs()
    s = max(1.0, ref.square().mean().sqrt().item())
    r_strict = (err / (tol * (1.0 + ref.abs()))).max().item() if err.numel() else 0.0
    r_scaled = (err / (tol * (s + ref.abs()))).max().item() if err.numel() else 0.0
    _record(name, dtype, tol, r_strict, r_scaled, "scaled" if scaled else "strict", err.numel())
    bound = tol * (s if scaled else 1.0) + tol * ref.abs()
    bad = err > bound
    if scaled and dtype != torch.float32 and bad.any():
        # 16-bit operands: rounding noise has tails
        if bad.double().mean().item() <= 1e-3 and not (err > 4 * bound).any():
            return
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        raise AssertionError(
            f"{name}: {int(bad.sum())}/{bad.numel()} outside tol {tol:g} ({'scaled' if scaled else 'strict'}); max err "
            f"{err.max().item():.3e} = {r_strict:.2f} x strict bound, {r_scaled:.2f} x scaled bound "
            f"(ref max {ref.abs().max().item():.3e}, rms scale {s:.3e}); first at {idx}: got {got[tuple(idx)].item():.6e} "
            f"ref {ref[tuple(idx)].item():.6e}")

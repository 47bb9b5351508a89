"""Shared helpers of the test-suite: seeded inputs, tolerances, comparison."""
import math

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


def assert_close(got, ref, dtype, name="", scale=1.0):
    """|got - ref| <= tol * (s + |ref|) elementwise: rtol = tol and atol = tol * s, where s = max(1, RMS(ref))
    expresses the absolute tolerance in units of the tensor's own magnitude (for tensors of unit scale or
    smaller this is plain rtol = atol = tol).  Rounding errors of a sum are proportional to the size of its
    terms, not of the (possibly cancelling) result, hence the tensor-level scale."""
    tol = TOL[dtype] * scale
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - ref).abs()
    s = max(1.0, ref.square().mean().sqrt().item())
    bound = tol * s + tol * ref.abs()
    bad = err > bound
    if dtype != torch.float32 and bad.any():
        # 16-bit operands: rounding noise has tails.  Up to 0.1 % of the elements may exceed the bound, none
        # by more than a factor 4; everything else must be inside it.
        if bad.double().mean().item() <= 1e-3 and not (err > 4 * bound).any():
            return
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        raise AssertionError(
            f"{name}: {int(bad.sum())}/{bad.numel()} outside tol {tol:g}; max err {err.max().item():.3e} "
            f"(ref max {ref.abs().max().item():.3e}, rms scale {s:.3e}); first at {idx}: got {got[tuple(idx)].item():.6e} "
            f"ref {ref[tuple(idx)].item():.6e}")

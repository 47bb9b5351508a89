"""The HIP path's 16-bit error beside the error of the reference's own rounding points.

For bf16 inputs the parity contract (rtol = atol = 2e-2 against the exact math) is met element by element for the
outputs, but the gradients that are long sums of rounded terms (ddt, ddt_bias, dB, dC, dA, dD) exceed a plain absolute
2e-2 in ANY 16-bit implementation.  oracle/rounding_emulation.py restates the reference's algorithm with the reference's
rounding points; here both it and the HIP path are compared with the float64 math on the same inputs, tensor by tensor:
 (i)  the HIP path's error is of the size of the emulation's (at most RATIO_CAP times its ratio to the plain bound, or
      inside the plain bound outright);
 (ii) every element of the HIP result lies within the plain bound widened by the emulation's own largest error of that
      tensor (the "envelope").
dD is the documented exception to (i): the reference forms it in float32 from dout * silu(z) before that product is
rounded (its dz kernel reads x as well, src/ssd/bi/ssd_chunk_scan.py:428-440 there), the HIP path from the 16-bit
dout * silu(z) that its dx kernel holds anyway; its error is held to 2e-2 of the tensor's RMS instead."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from oracle.rounding_emulation import reference_rounded
from tests import helpers
from tests.helpers import TOL, make_case, to64, to_dev

pytestmark = pytest.mark.gpu
NAMES = ("out", "dx", "dz", "dB", "dC", "ddt", "dA", "dD", "ddt_bias")
RATIO_CAP = 2.0

CASES = [
    # batch, seqlen, H, P, G, N, chunk         (z gate, D per head, dt_bias + softplus throughout)
    (2, 200, 4, 32, 2, 16, 64),                # generic kernels (smoke shape)
    (1, 300, 2, 64, 1, 64, 256),               # 16-bit fast path (smoke shape)
    (1, 4096, 32, 64, 8, 64, 256),             # one batch row of the training configuration with 8 groups
]


def _ratio(got, ref, tol):
    return ((got - ref).abs() / (tol * (1.0 + ref.abs()))).max().item()


@pytest.mark.parametrize("case", CASES)
def test_hip_error_against_the_reference_rounding_envelope(case):
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q = case
    dtype, tol = torch.bfloat16, TOL[torch.bfloat16]
    inp = make_case(b, L, H, P, G, N, dtype, with_z=True)
    dout = torch.randn(b, L, H, P, generator=torch.Generator().manual_seed(1)).to(dtype)
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    out.backward(dout.cuda())
    hip = {"out": out, **{"d" + k: leaves[k].grad for k in ("x", "z", "B", "C", "dt", "A", "D", "dt_bias")}}
    hip = {k: v.detach().double().cpu() for k, v in hip.items()}
    r = to64(inp)
    kw = dict(D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True)
    emu = reference_rounded(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], Q, dtype=dtype, **kw)
    exact = reference_rounded(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], Q, dtype=None, **kw)
    report = {}
    for k in NAMES:
        r_hip, r_emu = _ratio(hip[k], exact[k], tol), _ratio(emu[k], exact[k], tol)
        rms = max(1.0, exact[k].square().mean().sqrt().item())
        report[k] = (round(r_hip, 2), round(r_emu, 2))
        helpers._record(k + " (HIP / exact)", dtype, tol, r_hip, r_hip / rms, "envelope", hip[k].numel())
        helpers._record(k + " (reference rounding / exact)", dtype, tol, r_emu, r_emu / rms, "envelope", hip[k].numel())
    print(f"\n{case}: plain-bound ratios (HIP, reference rounding): {report}")
    for k in NAMES:
        r_hip, r_emu = report[k]
        err = (hip[k] - exact[k]).abs()
        if k == "dD":
            rms = max(1.0, exact[k].square().mean().sqrt().item())
            assert (err <= tol * (rms + exact[k].abs())).all(), f"dD: {r_hip} x the plain bound, RMS {rms:.1f}"
            continue
        # (i) same size as the reference's own rounding error
        assert r_hip <= max(1.0, RATIO_CAP * r_emu), f"{k}: HIP {r_hip} x the plain bound, reference rounding {r_emu} x"
        # (ii) inside the plain bound widened by the emulation's largest error of this tensor
        env = (emu[k] - exact[k]).abs().max()
        assert (err <= tol * (1.0 + exact[k].abs()) + env).all(), f"{k}: outside the envelope"

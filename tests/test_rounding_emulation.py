"""The stage-by-stage restatement with the reference's rounding points (oracle/rounding_emulation.py).

1. With rounding switched off it is exact: output and every gradient equal torch.autograd through the oracle's closed form.
   This pins the hand-written backward formulas (they are not a retyping of the closed form: the closed form has no chunks,
   no states, no per-stage terms).
2. With bf16 rounding at the reference's places, its error against the exact math is what a faithful 16-bit implementation of
   the reference's algorithm leaves per tensor.  The sizes are recorded (and bounded from above, loosely) so that the GPU
   test can put the HIP path's errors beside them."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from oracle.rounding_emulation import reference_rounded
from tests.helpers import TOL, make_case, to64

NAMES = ("out", "dx", "dz", "dB", "dC", "ddt", "dA", "dD", "ddt_bias")

CASES = [
    # batch, seqlen, H, P, G, N, chunk, z, D per column, softplus, dt_limit
    (2, 50, 4, 8, 2, 4, 16, True, False, True, (0.0, float("inf"))),
    (1, 37, 2, 4, 1, 8, 16, False, True, True, (0.01, 0.2)),
    (2, 64, 2, 8, 2, 4, 32, True, True, False, (0.0, float("inf"))),
]


def strict_ratio(got, ref, tol):
    return ((got - ref).abs() / (tol * (1.0 + ref.abs()))).max().item()


@pytest.mark.parametrize("case", CASES)
def test_without_rounding_it_is_the_exact_math(case):
    b, L, H, P, G, N, Q, z, Dhp, sp, lim = case
    inp = to64(make_case(b, L, H, P, G, N, torch.float32, with_z=z, D_has_hdim=Dhp))
    dout = torch.randn(b, L, H, P, generator=torch.Generator().manual_seed(3)).double()
    kw = dict(D=inp["D"], z=inp["z"], dt_bias=inp["dt_bias"], dt_softplus=sp, dt_limit=lim)
    ref = O.bimamba2_grads(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], **kw)
    got = reference_rounded(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], Q, dtype=None, **kw)
    for k in NAMES:
        if ref[k] is None:
            assert got[k] is None
            continue
        scale = max(1.0, ref[k].abs().max().item())
        assert (got[k] - ref[k]).abs().max().item() <= 1e-9 * scale, k


def test_error_of_the_reference_rounding_points_in_bf16():
    """The smoke shape of the 16-bit fast path (headdim 64, dstate 64, chunk 256, ragged): how far a bf16 run of the
    reference's algorithm lands from the exact math, per tensor, in units of the plain bound 2e-2 * (1 + |ref|)."""
    b, L, H, P, G, N, Q = 1, 300, 2, 64, 1, 64, 256
    inp = to64(make_case(b, L, H, P, G, N, torch.bfloat16, with_z=True))
    dout = torch.randn(b, L, H, P, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).double()
    kw = dict(D=inp["D"], z=inp["z"], dt_bias=inp["dt_bias"], dt_softplus=True)
    ref = O.bimamba2_grads(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], **kw)
    emu = reference_rounded(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], Q, dtype=torch.bfloat16, **kw)
    ratios = {k: strict_ratio(emu[k], ref[k], TOL[torch.bfloat16]) for k in NAMES}
    print("strict ratios of the bf16 emulation:", {k: round(v, 2) for k, v in ratios.items()})
    # rounding is on: nothing is exact any more ...
    assert all(v > 0 for v in ratios.values())
    # ... the elementwise outputs stay near the plain bound, and the summed gradients are the ones that pass it
    assert ratios["out"] < 1.5 and ratios["dx"] < 1.5 and ratios["dz"] < 1.5
    assert max(ratios.values()) < 20

"""bimamba2_fwd_static, the forward entry point that allocates nothing: its intermediates live in a buffer that is part
of the library's device image instead of a caller-supplied workspace.  Called through the C ABI and compared bit for bit
with bimamba2_fwd on two calls in a row, the second on a smaller problem (the buffer keeps the first call's contents).
Collected last: a failure here must not hide the other tests behind `pytest -x`."""
import ctypes

import pytest
import torch

from tests.helpers import make_case, to_dev

pytestmark = pytest.mark.gpu


def _forward(ops, d, Q, entry):
    """out, out_x, final_f, final_b of one forward through `entry`; the caller-owned tensors are the inputs and outputs only."""
    c = ops._problem(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, d["D"], d["z"], d["dt_bias"], True, (0.0, float("inf")))
    x = d["x"]
    out = c.new("out", x.shape, x.dtype)
    out_x = c.new("out_x", x.shape, x.dtype)
    fs = (x.shape[0], x.shape[2], x.shape[3], d["B"].shape[3])
    ff, fb = c.new("final_f", fs), c.new("final_b", fs)
    for t in (out, out_x, ff, fb):
        t.fill_(float("nan"))
    if entry == "bimamba2_fwd":
        c.workspace(False)
    c.run(entry)
    torch.cuda.synchronize()
    return out, out_x, ff, fb


# (batch, seqlen, H, P, G, N, chunk, dtype): first call, then a smaller second call
CASES = [
    ((2, 1024, 8, 64, 1, 64, 256, torch.bfloat16), (1, 300, 4, 64, 1, 64, 256, torch.bfloat16)),   # 16-bit kernels
    ((2, 200, 4, 32, 2, 16, 64, torch.float32), (1, 70, 2, 32, 1, 16, 64, torch.float32)),          # generic kernels
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_forward_matches_the_workspace_forward_twice(first, second):
    from bi_mamba2_amd import ops
    for seed, shape in enumerate((first, second)):
        b, L, H, P, G, N, Q, dtype = shape
        d = to_dev(make_case(b, L, H, P, G, N, dtype, seed=seed, with_z=True))
        ref = _forward(ops, d, Q, "bimamba2_fwd")
        got = _forward(ops, d, Q, "bimamba2_fwd_static")
        for g, r, name in zip(got, ref, ("out", "out_x", "final_f", "final_b")):
            assert torch.isfinite(g.float()).all(), name
            assert torch.equal(g, r), f"{name} differs on call {seed + 1} ({shape})"


def test_static_forward_refuses_what_does_not_fit():
    from bi_mamba2_amd import _lib, ops
    lib = _lib.load()
    # batch 8 x 4096 x 64 heads: float32 chunk states alone are far beyond the buffer
    b, L, H, P, G, N, Q = 8, 4096, 64, 64, 1, 64, 256
    x = torch.empty(b, L, H, P, device="cuda", dtype=torch.bfloat16)
    dt = torch.empty(b, L, H, device="cuda")
    A = torch.empty(H, device="cuda")
    B = torch.empty(b, L, G, N, device="cuda", dtype=torch.bfloat16)
    c = ops._problem(x, dt, A, B, B, Q, None, None, None, False, (0.0, float("inf")))
    c.new("out", x.shape, x.dtype)
    assert lib.bimamba2_workspace_bytes(ctypes.byref(c.p), 0) > (64 << 20)
    with pytest.raises(ValueError, match="static scratch"):
        c.run("bimamba2_fwd_static")

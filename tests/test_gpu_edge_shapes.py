"""GPU parity on the smallest and most ragged shapes: one position, a sequence shorter than a chunk on the fast-path
kernels (one partly filled chunk), a last chunk of one position, forward and backward."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, make_case, to64, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z
    (1, 1, 2, 16, 1, 8, 32, torch.float32, False),
    (2, 7, 2, 32, 2, 16, 64, torch.float32, True),
    (1, 1, 2, 64, 1, 64, 256, torch.bfloat16, True),          # fast-path kernels, one position
    (2, 40, 4, 64, 1, 64, 256, torch.bfloat16, True),         # fast-path kernels, 40 of 256 positions
    (1, 257, 2, 64, 1, 64, 256, torch.bfloat16, False),       # last chunk holds one position
    (1, 65, 2, 128, 2, 64, 64, torch.float16, True),          # two headdim tiles, last chunk of one position
]


@pytest.mark.parametrize("case", CASES)
def test_tiny_and_ragged_shapes(case):
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q, dtype, z = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z)
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    out.backward(dout.cuda())
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True)
    assert_close(out, ref["out"], dtype, "out")
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if ref["d" + k] is not None:
            assert_close(leaves[k].grad, ref["d" + k], dtype, "d" + k)

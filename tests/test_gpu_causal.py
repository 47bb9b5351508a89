"""GPU parity of the single-direction (causal) comparator, forward and backward, against the oracle's causal operator
in float64, through the C ABI; and its refusal of shapes it has no kernels for."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, is_reduced, make_case, to64, to_dev

pytestmark = pytest.mark.gpu
INF = float("inf")


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


CASES = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z, D
    (2, 512, 8, 64, 1, 64, 256, torch.bfloat16, True, "h"),
    (1, 700, 4, 64, 2, 64, 256, torch.bfloat16, False, "hp"),     # ragged last chunk (188 valid rows), grouped heads
    (2, 256, 4, 128, 4, 64, 128, torch.float16, True, "h"),       # two headdim tiles, one 16-row tile per wave
    (1, 192, 2, 64, 1, 64, 64, torch.bfloat16, True, "none"),
]


@pytest.mark.parametrize("case", CASES)
def test_causal_forward_and_backward(ops, case):
    b, L, H, P, G, N, Q, dtype, z, Dk = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"))
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.causal_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                         z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    out.backward(dout.to(out.device))
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True, form="causal", chunk_size=Q)
    assert_close(out, ref["out"], dtype, "out")
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if ref["d" + k] is not None:
            assert_close(leaves[k].grad, ref["d" + k], dtype, "d" + k, scaled=is_reduced("d" + k, dtype))


def test_causal_refuses_shapes_without_kernels(ops):
    inp = to_dev(make_case(1, 128, 2, 32, 1, 16, torch.float32))
    with pytest.raises(ValueError):
        ops.causal_chunk_scan_combined(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], 64, D=inp["D"],
                                       dt_bias=inp["dt_bias"], dt_softplus=True)

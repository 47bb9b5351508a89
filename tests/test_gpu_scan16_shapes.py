"""GPU parity over the shapes of the persistent 16-bit scan kernel (csrc/kernels_scan16.hip: forward output and the dx
mirror): the chunk sizes at which the composites keep the 16-bit state copies (multiples of 64 up to 256: 2 to 8 K steps,
waves without rows in the chunk), a ragged last chunk, 1 / 2 / 3 / 4 heads per workgroup (heads per group 1, 2, 3, 6, 4, 8), one and two headdim tiles, D per head
and per (head, headdim), with and without z, bf16 and fp16 - each end to end against torch.autograd on the float64
oracle - and that these shapes do run that kernel (the composites keep the 16-bit copies of the entering states there and
the scan stage reads no CB)."""
import ctypes

import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, is_reduced, make_case, to64, to_dev

pytestmark = pytest.mark.gpu
INF = float("inf")

CASES = [
    # batch, seqlen, H, P, G, chunk, dtype, z, D kind
    (2, 100, 4, 64, 4, 64, torch.bfloat16, True, "h"),        # two K steps, one head per workgroup, last chunk of 36 rows
    (1, 250, 6, 64, 3, 128, torch.bfloat16, False, "hp"),     # four K steps, two heads per workgroup, ragged (122 rows)
    (2, 394, 3, 64, 1, 192, torch.float16, True, "h"),        # six K steps, three heads per workgroup, last chunk of 10 rows
    (1, 512, 6, 64, 1, 256, torch.bfloat16, True, "h"),       # six heads in one group: workgroups of three
    (1, 300, 8, 128, 1, 128, torch.bfloat16, False, "hp"),    # two headdim tiles (ddt_direct summed over both), four heads
    (1, 700, 8, 64, 2, 192, torch.float16, False, "none"),    # four heads per workgroup in two groups, no D
    (2, 257, 4, 64, 1, 256, torch.bfloat16, True, "hp"),      # a last chunk of one row
]


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


@pytest.mark.parametrize("case", CASES)
def test_scan16_shapes_forward_and_backward(ops, case):
    from bi_mamba2_amd import _lib
    b, L, H, P, G, Q, dtype, z, Dk = case
    inp = make_case(b, L, H, P, G, 64, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"))
    d = to_dev(inp)
    # the shape is one of the kernel's: 16-bit state copies kept, no CB read by the scan stages
    c = ops._problem(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, d["D"], d["z"], d["dt_bias"], True, (0.0, INF))
    lib = _lib.load()
    assert lib.bimamba2_state_copies(ctypes.byref(c.p)) == 1
    assert lib.bimamba2_chunk_scan_reads_cb(ctypes.byref(c.p), 0) == 0 and lib.bimamba2_chunk_scan_reads_cb(ctypes.byref(c.p), 1) == 0

    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(11)).to(dtype)
    out.backward(dout.cuda())
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True, dt_limit=(0.0, INF))
    assert_close(out, ref["out"], dtype, "out")
    for k in ("dx", "dz", "dB", "dC", "ddt", "dA", "dD", "ddt_bias"):
        if ref[k] is not None:
            # dx: values up to 23 from operands rounded to 8 bits of mantissa leave one element in 96000 at 1.16 x the plain
            # bound (0.92 x with the absolute part in units of the RMS, 1.4): the criterion of the summed gradients
            assert_close(leaves[k[1:]].grad, ref[k], dtype, k, scaled=is_reduced(k, dtype) or k == "dx")


@pytest.mark.parametrize("case", [CASES[1], CASES[3]])
def test_scan16_shapes_single_direction(ops, case):
    """The same kernel with the reverse direction compiled out, against the causal oracle."""
    b, L, H, P, G, Q, dtype, z, Dk = case
    inp = make_case(b, L, H, P, G, 64, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"))
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.causal_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                         z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(11)).to(dtype)
    out.backward(dout.cuda())
    r = {k: (v.clone().requires_grad_(True) if torch.is_tensor(v) else v) for k, v in to64(inp).items()}
    ro = O.ssd_causal(r["x"], r["dt"], r["A"], r["B"], r["C"], Q, D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True)[0]
    ro.backward(dout.double())
    assert_close(out, ro, dtype, "out")
    for k in ("x", "z", "B", "C", "dt", "A", "D", "dt_bias"):
        if r[k] is not None:
            assert_close(leaves[k].grad, r[k].grad, dtype, "d" + k, scaled=is_reduced("d" + k, dtype) or k == "x")


WIDE_STATE = [
    # batch, seqlen, H, P, G, chunk, dtype, z, D kind   -- state dimension 128, forward only (the route of a pass without a
    # backward: 16-bit copies of the entering states, no CB, the persistent kernel's variant with single-buffered state tiles)
    (2, 300, 4, 64, 1, 256, torch.bfloat16, False, "h"),      # four heads per workgroup, ragged last chunk (44 rows)
    (1, 700, 6, 64, 2, 128, torch.bfloat16, True, "hp"),      # three heads per workgroup in two groups, z gate, D per column
    (1, 200, 3, 128, 3, 64, torch.float16, True, "none"),     # one head per workgroup, two headdim tiles, two K steps
    (2, 513, 8, 64, 1, 192, torch.bfloat16, False, "h"),      # six K steps, a last chunk of 129 rows
]


@pytest.mark.parametrize("case", WIDE_STATE)
def test_scan16_state_dimension_128_forward(ops, case):
    b, L, H, P, G, Q, dtype, z, Dk = case
    inp = make_case(b, L, H, P, G, 128, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"))
    d = to_dev(inp)
    with torch.no_grad():
        out, ff, fb = ops.bimamba_chunk_scan_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, D=d["D"], z=d["z"],
                                                      dt_bias=d["dt_bias"], dt_softplus=True, return_final_states=True)
    r = to64(inp)
    ref, _, rf, rb = O.bimamba2_naive_chunked(r["x"], r["dt"], r["A"], r["B"], r["C"], Q, D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                                             dt_softplus=True)
    # (16-bit operands with a state of 128 columns: outputs of magnitude 10 - 60; the absolute part in units of the RMS)
    assert_close(out, ref, dtype, "out", scaled=True)
    assert_close(ff, rf, dtype, "final_f", scaled=True)
    assert_close(fb, rb, dtype, "final_b", scaled=True)
    # the same pass with the float32 entering states kept (the generic scan kernel on a float32 CB): both routes round the
    # same operands, so they agree far inside the tolerance
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out2 = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                           z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    assert_close(out, out2.detach(), dtype, "out, both routes", scale=0.5, scaled=True)

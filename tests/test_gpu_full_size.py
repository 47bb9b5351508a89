"""The operator at the baseline's full shapes: size-independent properties (flip equivariance, linearity) of outputs and
gradients, and float64 oracle comparisons on one batch row."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, make_case, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


FULL = [
    # the baseline's configurations 1 (forward bench) and 3 (forward + backward, 8 groups), bf16
    dict(batch=4, seqlen=2048, nheads=32, headdim=64, ngroups=1, dstate=64, chunk=256),
    dict(batch=4, seqlen=4096, nheads=32, headdim=64, ngroups=8, dstate=64, chunk=256),
]


@pytest.mark.parametrize("cfg", FULL)
def test_full_size_flip_equivariance_and_linearity(ops, cfg):
    """f(flip(inputs)) = flip(f(inputs)) and f(2x) = 2 f(x), forward and backward, at full size in bf16."""
    inp = make_case(cfg["batch"], cfg["seqlen"], cfg["nheads"], cfg["headdim"], cfg["ngroups"], cfg["dstate"],
                    torch.bfloat16, with_z=True)
    d = to_dev(inp)
    dout = torch.randn(inp["x"].shape, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).cuda()

    def run(x, dt, B, C, z, g):
        leaves = [t.clone().requires_grad_(True) for t in (x, dt, B, C, z)]
        par = [d[k].clone().requires_grad_(True) for k in ("A", "D", "dt_bias")]
        out = ops.bimamba_chunk_scan_combined(leaves[0], leaves[1], par[0], leaves[2], leaves[3], cfg["chunk"], D=par[1],
                                              z=leaves[4], dt_bias=par[2], dt_softplus=True)
        grads = torch.autograd.grad(out, leaves + par, g)
        return out, grads

    out, gr = run(d["x"], d["dt"], d["B"], d["C"], d["z"], dout)
    assert torch.isfinite(out.float()).all()
    fo, fg = run(d["x"].flip(1), d["dt"].flip(1), d["B"].flip(1), d["C"].flip(1), d["z"].flip(1), dout.flip(1))
    # both sides carry bf16 rounding of a different summation order
    assert_close(fo.flip(1), out.float(), torch.bfloat16, "flip: out")
    for name, a, b_ in zip(("dx", "ddt", "dB", "dC", "dz"), fg[:5], gr[:5]):
        assert_close(a.flip(1), b_.float(), torch.bfloat16, "flip: " + name)
    for name, a, b_ in zip(("dA", "dD", "ddt_bias"), fg[5:], gr[5:]):
        assert_close(a, b_.float(), torch.bfloat16, "flip: " + name, scaled=True)
    o2, _ = run(2 * d["x"], d["dt"], d["B"], d["C"], d["z"], dout)
    assert_close(o2, 2 * out.float(), torch.bfloat16, "linearity in x")


@pytest.mark.parametrize("cfg", FULL)
def test_full_size_one_batch_row_against_the_oracle(ops, cfg):
    """Forward and every gradient at the baseline's full shapes against float64 autograd through the oracle's chunked
    flip-and-sum path on one batch row (all heads, all groups).  out, dx, dz, ddt, dB, dC of that row are taken from
    the full-size run; dA, dD and ddt_bias are sums over the batch, so for them the device path runs on that row alone
    (rows do not interact: every kernel's work units are per batch row)."""
    dtype, Q, row = torch.bfloat16, cfg["chunk"], 1
    inp = make_case(cfg["batch"], cfg["seqlen"], cfg["nheads"], cfg["headdim"], cfg["ngroups"], cfg["dstate"], dtype, with_z=True)
    d = to_dev(inp)
    dout = torch.randn(inp["x"].shape, generator=torch.Generator().manual_seed(3)).to(dtype)
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")
    per_row = ("x", "dt", "B", "C", "z")

    def device_grads(sel):
        leaves = {k: (d[k][sel] if k in per_row else d[k]).clone().requires_grad_(True) for k in names}
        out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                              z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
        grads = torch.autograd.grad(out, [leaves[k] for k in names], dout[sel].cuda())
        return out, dict(zip(names, grads))

    out_full, g_full = device_grads(slice(None))
    out_row, g_row = device_grads(slice(row, row + 1))

    r = {k: (inp[k][row:row + 1] if k in per_row else inp[k]).double().requires_grad_(True) for k in names}
    ref = O.bimamba2_naive_chunked(r["x"], r["dt"], r["A"], r["B"], r["C"], Q, D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                                   dt_softplus=True)[0]
    ref.backward(dout[row:row + 1].double())
    # outputs reach 40-60 here while 16-bit operands carry 8 bits of mantissa: a handful of the 4-8 million elements miss
    # the plain bound (by up to 1.4x: the recorded margins), hence the tail allowance of the scaled form for out
    assert_close(out_full[row:row + 1], ref, dtype, "out", scaled=True)
    assert torch.equal(out_full[row:row + 1], out_row), "a batch row must not depend on the others"
    for k in per_row:      # dx, dz: a handful of elements in millions beyond the plain bound, as for out
        assert_close(g_full[k][row:row + 1], r[k].grad, dtype, "d" + k, scaled=True)
    for k in ("A", "D", "dt_bias"):
        assert_close(g_row[k], r[k].grad, dtype, "d" + k, scaled=True)


def test_long_sequence_forward_against_chunked_oracle_sample(ops):
    """Baseline configuration 2 (seqlen 16384, 64 chunks, dstate 128), bf16 forward: one batch row and a few heads
    are checked against the oracle's chunked float64 path."""
    inp = make_case(2, 16384, 48, 64, 1, 128, torch.bfloat16, with_z=False)
    d = to_dev(inp)
    out = ops.bimamba_chunk_scan_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], 256, D=d["D"], dt_bias=d["dt_bias"], dt_softplus=True)
    hs = [0, 17, 47]
    r = {k: (v.double() if v is not None else None) for k, v in inp.items()}
    ref = O.bimamba2_naive_chunked(r["x"][:1, :, hs], r["dt"][:1, :, hs], r["A"][hs], r["B"][:1], r["C"][:1], 256,
                                   D=r["D"][hs], dt_bias=r["dt_bias"][hs], dt_softplus=True)[0]
    # 3 million outputs of magnitude up to 25 from operands with 8 bits of mantissa: the largest error sits at 0.9 - 1.05 x the
    # plain bound depending on the kernel's summation order (one element at 1.03 x with the persistent kernel, none with the
    # generic one), hence the form with the absolute part in units of the RMS (1.06 here) and its tail allowance, as for the
    # other full-size outputs
    assert_close(out[:1, :, hs], ref, torch.bfloat16, "long forward", scaled=True)

"""GPU parity of the backward path against torch.autograd on the float64 oracle, through the C ABI."""
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


def _run_bwd(ops, inp, Q, sp, lim, seed=5):
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=sp, dt_limit=lim)
    g = torch.Generator().manual_seed(seed)
    dout = torch.randn(out.shape, generator=g).to(out.dtype)
    out.backward(dout.to(out.device))
    grads = {"d" + k: (v.grad if v is not None else None) for k, v in leaves.items()}
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=sp, dt_limit=lim)
    return out, grads, ref


def _check(out, grads, ref, dtype, big=False):
    """big: the case's outputs are far from unit scale (raw dt without softplus: steps of size 1), so the absolute
    tolerance of every tensor is taken in units of its RMS; otherwise only the summed gradients (helpers.REDUCED) are."""
    assert_close(out, ref["out"], dtype, "out", scaled=big)
    for k in ("dx", "dB", "dC", "dz"):
        if ref[k] is not None:
            assert grads[k].dtype == dtype
            assert_close(grads[k], ref[k], dtype, k, scaled=big or is_reduced(k, dtype))
    for k in ("ddt", "dA", "dD", "ddt_bias"):
        if ref[k] is not None:
            assert_close(grads[k], ref[k], dtype, k, scaled=big or is_reduced(k, dtype))


# the reference's own end-to-end backward grid (tests/test_bwd_scan.py:8-16 there)
REF_BWD_GRID = [(b, L, 1, P, 1, N, 32) for b in (1, 2) for L in (32, 64, 128) for P in (1, 4) for N in (1, 4)]


@pytest.mark.parametrize("shape", REF_BWD_GRID)
def test_backward_reference_grid(ops, shape):
    b, L, H, P, G, N, Q = shape
    inp = make_case(b, L, H, P, G, N, torch.float32, with_D=False, ref_style=True)
    out, grads, ref = _run_bwd(ops, inp, Q, True, (0.0, INF))
    _check(out, grads, ref, torch.float32)


E2E = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z, D, bias, softplus, limit
    (2, 256, 4, 32, 1, 16, 64, torch.float32, False, "h", True, True, (0.0, INF)),
    (2, 250, 4, 32, 2, 16, 64, torch.float32, True, "hp", True, True, (0.0, INF)),
    (1, 130, 2, 64, 1, 64, 128, torch.float32, True, "h", False, False, (0.0, INF)),
    (2, 200, 4, 16, 4, 8, 32, torch.float32, False, "none", True, True, (0.01, 0.2)),
    (1, 100, 2, 128, 1, 128, 48, torch.float32, True, "hp", True, True, (0.0, INF)),
    (2, 512, 8, 64, 1, 64, 256, torch.bfloat16, True, "h", True, True, (0.0, INF)),
    (1, 700, 4, 64, 2, 128, 256, torch.bfloat16, False, "h", True, True, (0.0, INF)),
    (2, 256, 4, 64, 4, 64, 128, torch.float16, True, "h", True, True, (0.0, INF)),
    # shapes whose scan kernels rebuild CB themselves, with a ragged last chunk (44 valid rows), grouped heads,
    # resp. two headdim tiles
    (2, 300, 4, 64, 2, 64, 256, torch.bfloat16, False, "hp", True, True, (0.0, INF)),
    (1, 200, 2, 128, 1, 64, 128, torch.float16, True, "h", True, True, (0.0, INF)),
]


@pytest.mark.parametrize("case", E2E)
def test_backward_end_to_end(ops, case):
    b, L, H, P, G, N, Q, dtype, z, Dk, bias, sp, lim = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"), with_bias=bias)
    out, grads, ref = _run_bwd(ops, inp, Q, sp, lim)
    _check(out, grads, ref, dtype, big=not sp)


@pytest.mark.parametrize("case", [E2E[1], E2E[5]])
def test_backward_with_recomputation(ops, case, monkeypatch):
    """The backward pass recomputes the forward intermediates (as the reference does) instead of reading the
    ones the forward kept."""
    monkeypatch.setattr(ops, "KEEP_FORWARD_INTERMEDIATES", False)
    b, L, H, P, G, N, Q, dtype, z, Dk, bias, sp, lim = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"), with_bias=bias)
    out, grads, ref = _run_bwd(ops, inp, Q, sp, lim)
    _check(out, grads, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sixteen_bit_state_copies_against_float32_states(ops, dtype):
    """Where the kernels can, the composites keep the states entering the chunks (and their gradients) in copies of the
    input's 16-bit type instead of float32, and the scan kernels that know the copies run.  Every kernel that reads the
    entering states rounds them to that type for its MFMA anyway, so both ways must agree within the tolerance of the type
    (different kernels with different rounding points: not bit for bit).  The float32 side: forward with the states returned as tensors, which switches
    the copies off."""
    import ctypes
    from bi_mamba2_amd import _lib
    Q = 256
    inp = make_case(2, 700, 4, 64, 2, 64, dtype, with_z=True)
    d = to_dev(inp)
    args = (d["x"], d["dt"], d["A"], d["B"], d["C"], Q)
    kw = dict(D=d["D"], z=d["z"], dt_bias=d["dt_bias"], dt_softplus=True)
    dout = torch.randn(d["x"].shape, generator=torch.Generator().manual_seed(7)).to(dtype).cuda()

    c = ops._problem(*args, d["D"], d["z"], d["dt_bias"], True, (0.0, INF))
    assert _lib.load().bimamba2_state_copies(ctypes.byref(c.p)) == 1
    c32 = ops._problem(d["x"].float(), d["dt"], d["A"], d["B"].float(), d["C"].float(), Q, d["D"], d["z"].float(), d["dt_bias"], True, (0.0, INF))
    assert _lib.load().bimamba2_state_copies(ctypes.byref(c32.p)) == 0

    res_c = ops._mamba_chunk_scan_combined_fwd(*args, **kw, return_intermediates=False, keep_for_bwd=True)
    assert res_c[9][2][3] == ops._BLOB_FIELDS_COPIES
    res_f = ops._mamba_chunk_scan_combined_fwd(*args, **kw, return_intermediates=True, keep_for_bwd=True)
    # (two 16-bit results against each other, each with its own rounding: absolute tolerance in units of the RMS)
    assert_close(res_c[0], res_f[0].double(), dtype, "out", scaled=True)
    assert_close(res_c[1], res_f[1].double(), dtype, "out_x", scaled=True)
    g_c = ops._mamba_chunk_scan_combined_bwd(dout, *args[:5], res_c[1], Q, **kw, saved=res_c[9])
    g_f = ops._mamba_chunk_scan_combined_bwd(dout, *args[:5], res_f[1], Q, **kw, saved=res_f[9])
    names = ("dx", "ddt", "dA", "dB", "dC", "dD", "dz", "ddt_bias")
    for name, a, b in zip(names, g_c, g_f):
        assert_close(a, b.double(), dtype, name, scaled=True)


def test_backward_takes_a_misaligned_gradient_view(ops):
    """The gradient arrives as a view that is neither 16-byte aligned nor has strides that are multiples of 8 elements
    (a slice of a wider tensor at an odd column), at a shape where the forward kept only the 16-bit copies of the entering
    states: the backward pass must give what it gives for the contiguous copy of the same values."""
    b, L, H, P, G, N, Q, dtype = 2, 512, 4, 64, 1, 64, 256, torch.bfloat16
    d = to_dev(make_case(b, L, H, P, G, N, dtype, with_z=False))
    wide = torch.randn(b, L, H, P + 3, generator=torch.Generator().manual_seed(3)).to(dtype).cuda()
    view = wide[..., 1:P + 1]
    assert view.data_ptr() % 16 and view.stride(2) % 8
    res = []
    for g in (view, view.contiguous()):
        leaves = {k: d[k].clone().requires_grad_(True) for k in ("x", "dt", "A", "B", "C", "D", "dt_bias")}
        out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                              dt_bias=leaves["dt_bias"], dt_softplus=True)
        out.backward(g)
        res.append({k: v.grad for k, v in leaves.items()})
    for k in res[0]:
        assert torch.equal(res[0][k], res[1][k]), k

"""GPU parity of the forward path: every stage kernel and the whole operator against the float64 oracle,
through the C ABI (bi_mamba2_amd.ops calls libbimamba2_hip.so via ctypes)."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, make_case, to64, to_dev

pytestmark = pytest.mark.gpu

INF = float("inf")

# batch, seqlen, H, P, G, N, chunk
STAGE_SHAPES = [
    (2, 200, 4, 32, 2, 16, 64),     # partial last chunk, grouped heads
    (1, 512, 2, 64, 1, 64, 256),    # the benchmark's tile sizes
    (2, 96, 4, 16, 4, 4, 32),       # small dims (padding inside the MFMA tiles)
    (1, 100, 2, 128, 1, 128, 48),   # two headdim / dstate tiles, chunk not a multiple of 64
]


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


@pytest.mark.parametrize("shape", STAGE_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_stages(ops, shape, dtype):
    b, L, H, P, G, N, Q = shape
    inp = make_case(b, L, H, P, G, N, dtype, with_z=True, D_has_hdim=(P == 32))
    r = to64(inp)
    d = to_dev(inp)
    # stage 1: cumsum
    dt_ref, csf_ref, csb_ref = O.stage_chunk_cumsum(r["dt"], r["A"], Q, r["dt_bias"], True)
    csf, csb, dt_out = ops._chunk_cumsum_fwd(d["dt"], d["A"], Q, dt_bias=d["dt_bias"], dt_softplus=True)
    assert_close(dt_out, dt_ref, torch.float32, "dt_out")
    assert_close(csf, csf_ref, torch.float32, "cs_f")
    assert_close(csb, csb_ref, torch.float32, "cs_b")
    # later stages take the device cumsums as input; the oracle takes the same values in float64
    csf64, csb64, dt64 = csf.double().cpu(), csb.double().cpu(), dt_out.double().cpu()
    # stage 2: CB
    CB = ops._bmm_chunk_fwd(d["C"], d["B"], Q)
    CB_ref = O.stage_bmm_chunk(r["C"], r["B"], Q)
    assert_close(CB, CB_ref, dtype, "CB")
    # stage 3: chunk states
    sf, sb = ops._chunk_state_fwd(d["B"], d["x"], dt_out, csf, csb)
    sf_ref, sb_ref = O.stage_chunk_state(r["B"], r["x"], dt64, csf64, csb64)
    assert_close(sf, sf_ref, dtype, "states_f")
    assert_close(sb, sb_ref, dtype, "states_b")
    # stage 4: inter-chunk scan (float32 arithmetic on float32 inputs)
    pf, pb, ff, fb = ops._state_passing_fwd(sf, sb, csf, csb)
    pf_ref, pb_ref, ff_ref, fb_ref = O.stage_state_passing(sf.double().cpu(), sb.double().cpu(), csf64, csb64)
    for got, ref, name in ((pf, pf_ref, "prev_f"), (pb, pb_ref, "prev_b"), (ff, ff_ref, "final_f"), (fb, fb_ref, "final_b")):
        assert_close(got, ref, torch.float32, name)
    # stage 5: chunk scan
    out, out_x = ops._chunk_scan_fwd(CB, d["x"], dt_out, csf, csb, d["C"], pf, pb, D=d["D"], z=d["z"])
    out_ref, outx_ref = O.stage_chunk_scan(CB.double().cpu(), r["x"], dt64, csf64, csb64, r["C"], pf.double().cpu(),
                                           pb.double().cpu(), r["D"], r["z"])
    big = N > 64      # dot products over 128 state columns of 16-bit operands: outputs of RMS ~ 10
    assert_close(out_x, outx_ref, dtype, "out_x", scaled=big)
    assert_close(out, out_ref, dtype, "out", scaled=big)


# the reference's own end-to-end forward grid (tests/test_fwd_scan.py:8-16 there): z = None, D = None
REF_FWD_GRID = [(b, L, 4, P, 4, N, 32) for b in (1, 2) for L in (32, 64, 128) for P in (4, 16) for N in (4, 16)]


@pytest.mark.parametrize("shape", REF_FWD_GRID)
def test_forward_reference_grid(ops, shape):
    b, L, H, P, G, N, Q = shape
    inp = make_case(b, L, H, P, G, N, torch.float32, with_D=False, ref_style=True)
    r, d = to64(inp), to_dev(inp)
    out = ops.bimamba_chunk_scan_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, dt_bias=d["dt_bias"], dt_softplus=True)
    ref = O.bimamba2_quadratic(r["x"], r["dt"], r["A"], r["B"], r["C"], dt_bias=r["dt_bias"], dt_softplus=True)[0]
    assert_close(out, ref, torch.float32, "out")


E2E = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z, D ('none'|'h'|'hp'), bias, softplus, limit
    (2, 256, 4, 32, 1, 16, 64, torch.float32, False, "h", True, True, (0.0, INF)),       # the reference’s own CPU-runnable benchmark shape
    (2, 250, 4, 32, 2, 16, 64, torch.float32, True, "hp", True, True, (0.0, INF)),
    (1, 130, 2, 64, 1, 64, 128, torch.float32, True, "h", False, False, (0.0, INF)),
    (2, 200, 4, 16, 4, 8, 32, torch.float32, False, "none", True, True, (0.01, 0.2)),
    (2, 512, 8, 64, 1, 64, 256, torch.bfloat16, True, "h", True, True, (0.0, INF)),
    (1, 700, 4, 64, 2, 128, 256, torch.bfloat16, False, "h", True, True, (0.0, INF)),
    (1, 300, 2, 128, 1, 32, 64, torch.bfloat16, True, "hp", True, True, (0.0, INF)),
    (2, 256, 4, 64, 4, 64, 128, torch.float16, True, "h", True, True, (0.0, INF)),
]


@pytest.mark.parametrize("case", E2E)
def test_forward_end_to_end(ops, case):
    b, L, H, P, G, N, Q, dtype, z, Dk, bias, sp, lim = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z, with_D=(Dk != "none"), D_has_hdim=(Dk == "hp"), with_bias=bias)
    r, d = to64(inp), to_dev(inp)
    out, ff, fb = ops.bimamba_chunk_scan_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, D=d["D"], z=d["z"],
                                                  dt_bias=d["dt_bias"], dt_softplus=sp, dt_limit=lim,
                                                  return_final_states=True)
    ref = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                                dt_softplus=sp, dt_limit=lim)
    assert out.dtype == dtype and ff.dtype == torch.float32
    assert_close(out, ref[0], dtype, "out", scaled=not sp)      # raw dt without softplus: outputs far from unit scale
    assert_close(ff, ref[2], dtype, "final_f")
    assert_close(fb, ref[3], dtype, "final_b")


def test_forward_strided_inputs(ops):
    """x, B, C carved out of one projection output (as the BiMamba2 layer does): strided views, no copies."""
    b, L, H, P, G, N, Q = 2, 192, 4, 32, 1, 16, 64
    inp = make_case(b, L, H, P, G, N, torch.float32)
    r, d = to64(inp), to_dev(inp)
    packed = torch.cat([d["x"].flatten(2), d["B"].flatten(2), d["C"].flatten(2)], -1)
    x, B, C = torch.split(packed, [H * P, G * N, G * N], -1)
    out = ops.bimamba_chunk_scan_combined(x.unflatten(-1, (H, P)), d["dt"], d["A"], B.unflatten(-1, (G, N)),
                                          C.unflatten(-1, (G, N)), Q, D=d["D"], dt_bias=d["dt_bias"], dt_softplus=True)
    ref = O.bimamba2_quadratic(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], dt_bias=r["dt_bias"], dt_softplus=True)[0]
    assert_close(out, ref, torch.float32, "out")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_stages_rebuild_cb_when_it_is_not_given(ops, dtype):
    """The scan, dx and dCB stages called without CB (the way the composites call them at such shapes) agree with the
    same stages reading the CB of the bmm stage.  Ragged last chunk (44 rows), two head groups."""
    b, L, H, P, G, N, Q = 2, 300, 4, 64, 2, 64, 256
    inp = make_case(b, L, H, P, G, N, dtype, with_z=True)
    d = to_dev(inp)
    csf, csb, dt_out = ops._chunk_cumsum_fwd(d["dt"], d["A"], Q, dt_bias=d["dt_bias"], dt_softplus=True)
    CB = ops._bmm_chunk_fwd(d["C"], d["B"], Q)
    sf, sb = ops._chunk_state_fwd(d["B"], d["x"], dt_out, csf, csb)
    pf, pb, _, _ = ops._state_passing_fwd(sf, sb, csf, csb)
    out1, outx1 = ops._chunk_scan_fwd(CB, d["x"], dt_out, csf, csb, d["C"], pf, pb, D=d["D"], z=d["z"])
    out2, outx2 = ops._chunk_scan_fwd(None, d["x"], dt_out, csf, csb, d["C"], pf, pb, D=d["D"], z=d["z"], B=d["B"])
    assert_close(outx2, outx1.double().cpu(), dtype, "out_x without CB")
    assert_close(out2, out1.double().cpu(), dtype, "out without CB")
    g = torch.Generator().manual_seed(11)
    dout = torch.randn(d["x"].shape, generator=g).to(dtype).cuda()
    dsf = torch.randn(pf.shape, generator=g).cuda() * 0.1
    dsb = torch.randn(pf.shape, generator=g).cuda() * 0.1
    dx1, ddt1, dD1 = ops._chunk_scan_chunk_state_bwd_dx(d["x"], dt_out, csf, csb, d["B"], CB, dout, dsf, dsb, D=d["D"])
    dx2, ddt2, dD2 = ops._chunk_scan_chunk_state_bwd_dx(d["x"], dt_out, csf, csb, d["B"], None, dout, dsf, dsb, D=d["D"], C=d["C"])
    assert_close(dx2, dx1.double().cpu(), dtype, "dx without CB")
    # positions past the end of the sequence are not written by either path
    valid = (torch.arange(ddt1.shape[2])[:, None] * Q + torch.arange(Q)[None, :] < L).to(ddt1.device)
    assert_close(torch.where(valid, ddt2, 0.0), torch.where(valid, ddt1, 0.0).double().cpu(), dtype, "ddt_direct without CB", scaled=True)
    assert_close(dD2, dD1.double().cpu(), dtype, "dD without CB", scaled=True)
    dCB1, da1 = ops._chunk_scan_bwd_dcb(d["x"], dt_out, csf, csb, dout, CB, ngroups=G)
    dCB2, da2 = ops._chunk_scan_bwd_dcb(d["x"], dt_out, csf, csb, dout, None, ngroups=G, B=d["B"], C=d["C"])
    assert_close(dCB2, dCB1.double().cpu(), dtype, "dCB without CB", scaled=True)
    assert_close(da2, da1.double().cpu(), dtype, "da_intra without CB", scaled=True)
    # shapes whose kernels cannot rebuild CB refuse a missing CB instead of reading a null pointer
    with pytest.raises(ValueError):
        ops._chunk_scan_fwd(None, d["x"].float(), dt_out, csf, csb, d["C"].float(), pf, pb, B=d["B"].float())

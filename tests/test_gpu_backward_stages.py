"""GPU parity of every backward stage on its own (the reference tests its backward kernels one by one as well:
tests/test_bwd_chunk_scan.py, tests/test_bwd_chunk_state.py, tests/test_bwd_state_passing.py there), through the stage
wrappers of bi_mamba2_amd.ops and the C ABI.

The expected value of a backward stage is torch.autograd through the oracle's restatement of the matching FORWARD stage
(oracle.bimamba2_oracle.stage_*, pinned on the CPU by "the stages composed equal the closed form"), in float64, fed with
the device's own inputs to that stage - so an error is attributed to the stage that made it, and no backward formula is
written down a second time."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, make_case, to64, to_dev

pytestmark = pytest.mark.gpu

# batch, seqlen, H, P, G, N, chunk
SHAPES = [
    (2, 200, 4, 32, 2, 16, 64),     # partial last chunk, grouped heads
    (1, 512, 2, 64, 1, 64, 256),    # the benchmark's tile sizes
    (2, 96, 4, 16, 4, 4, 32),       # small dims (padding inside the MFMA tiles)
    (1, 100, 2, 128, 1, 128, 48),   # two headdim / dstate tiles, chunk not a multiple of 64
    (1, 300, 32, 64, 1, 64, 256),   # 32 heads in one group: four head slices of partial dB / dC sums
    (1, 128, 32, 16, 2, 16, 64),    # 16 heads per group: two slices
]


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


def _leaf(t):
    return t.detach().double().cpu().requires_grad_(True)


def _c(t):
    return t.detach().double().cpu()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_stages(ops, shape, dtype):
    b, L, H, P, G, N, Q = shape
    inp = make_case(b, L, H, P, G, N, dtype, with_z=True, D_has_hdim=(P == 32))
    r, d = to64(inp), to_dev(inp)
    big = dtype != torch.float32      # 16-bit: summed gradients in units of their RMS (see tests/helpers.py)
    dout = torch.randn(inp["x"].shape, generator=torch.Generator().manual_seed(9)).to(dtype)
    nc = (L + Q - 1) // Q
    valid = (torch.arange(nc)[:, None] * Q + torch.arange(Q)[None, :] < L)      # (nc, Q): positions inside the sequence

    # ---- forward intermediates on the device (each checked on its own in test_gpu_forward.py)
    csf, csb, dt_out = ops._chunk_cumsum_fwd(d["dt"], d["A"], Q, dt_bias=d["dt_bias"], dt_softplus=True)
    CB = ops._bmm_chunk_fwd(d["C"], d["B"], Q)
    sf, sb = ops._chunk_state_fwd(d["B"], d["x"], dt_out, csf, csb)
    pf, pb, _, _ = ops._state_passing_fwd(sf, sb, csf, csb)
    out, out_x = ops._chunk_scan_fwd(CB, d["x"], dt_out, csf, csb, d["C"], pf, pb, D=d["D"], z=d["z"])
    csf64, csb64, dt64, CB64 = _c(csf), _c(csb), _c(dt_out), _c(CB)

    # ---- dz, dout * silu(z)   (a8)
    dz, dout_x = ops._chunk_scan_bwd_dz(d["x"], d["z"], out_x, dout.cuda(), Q)
    z64 = _leaf(inp["z"])
    (_c(out_x) * F.silu(z64)).backward(dout.double())
    assert_close(dz, z64.grad, dtype, "dz")
    assert_close(dout_x, dout.double() * F.silu(r["z"]), dtype, "dout_x")
    dy64 = _c(dout_x)

    def scan(CBv, x, dtv, cf, cb_, C, prf, prb, D):
        return O.stage_chunk_scan(CBv, x, dtv, cf, cb_, C, prf, prb, D, None)[0]

    # ---- gradient with respect to the states entering the chunks   (a9)
    dpf, dpb = ops._chunk_scan_bwd_dstates(d["C"], csf, csb, dout_x)
    prf, prb = _leaf(pf), _leaf(pb)
    scan(CB64, r["x"], dt64, csf64, csb64, r["C"], prf, prb, r["D"]).backward(dy64)
    assert_close(dpf, prf.grad, dtype, "dprev_f", scaled=big)
    assert_close(dpb, prb.grad, dtype, "dprev_b", scaled=big)

    # ---- the two stages above as one launch, where that kernel exists: the same bits
    if dtype != torch.float32 and N == 64 and P % 64 == 0 and Q % 32 == 0:
        dz1, dox1, dpf1, dpb1 = ops._chunk_scan_bwd_dz_dstates(d["z"], out_x, dout.cuda(), d["C"], csf, csb)
        assert torch.equal(dz1, dz) and torch.equal(dox1, dout_x), "dz / dout_x of the merged launch"
        assert torch.equal(dpf1, dpf) and torch.equal(dpb1, dpb), "dstates of the merged launch"

    # ---- adjoint of the two inter-chunk recurrences + gradient of the chunk totals   (a10)
    dSf, dSb, ddAcf, ddAcb = ops._state_passing_bwd(pf, pb, csf, csb, dpf, dpb)
    Sf, Sb, cf, cb_ = _leaf(sf), _leaf(sb), _leaf(csf), _leaf(csb)
    opf, opb, _, _ = O.stage_state_passing(Sf, Sb, cf, cb_)
    torch.autograd.backward([opf, opb], [_c(dpf), _c(dpb)])
    assert_close(dSf, Sf.grad, torch.float32, "dstates_f")          # float32 arithmetic on float32 inputs
    assert_close(dSb, Sb.grad, torch.float32, "dstates_b")
    assert_close(ddAcf, cf.grad[..., -1], torch.float32, "ddA_chunk_f", scaled=True)
    assert_close(ddAcb, cb_.grad[..., 0], torch.float32, "ddA_chunk_b", scaled=True)

    # ---- dx, ddt_direct, dD   (a11): the scan's x path and the chunk states' x path
    dx, ddt_direct, dD = ops._chunk_scan_chunk_state_bwd_dx(d["x"], dt_out, csf, csb, d["B"], CB, dout_x, dSf, dSb, D=d["D"])
    x64, dtl, D64 = _leaf(inp["x"]), _leaf(dt_out), _leaf(inp["D"])
    y = scan(CB64, x64, dtl, csf64, csb64, r["C"], _c(pf), _c(pb), D64)
    S2f, S2b = O.stage_chunk_state(r["B"], x64, dtl, csf64, csb64)
    torch.autograd.backward([y, S2f, S2b], [dy64, _c(dSf), _c(dSb)])
    assert_close(dx, x64.grad, dtype, "dx")
    m = valid.to(ddt_direct.device)
    # sums over headdim of products of size 100 and more (RMS 176, maximum 1546 at the 32-head shape): in units of the RMS
    assert_close(torch.where(m, ddt_direct, 0.0), dtl.grad, dtype, "ddt_direct", scaled=True)
    assert_close(dD, D64.grad, dtype, "dD", scaled=big)

    # ---- dB through the chunk states + its decay terms   (a12)
    dBs, vf, vb = ops._chunk_state_bwd_db(d["x"], dt_out, csf, csb, dSf, dSb, B=d["B"], ngroups=G)
    assert dBs.shape[0] == (H // G + 7) // 8
    B64, cf, cb_ = _leaf(inp["B"]), _leaf(csf), _leaf(csb)
    S3f, S3b = O.stage_chunk_state(B64, r["x"], dt64, cf, cb_)
    torch.autograd.backward([S3f, S3b], [_c(dSf), _c(dSb)])
    assert_close(dBs.sum(0), B64.grad, dtype, "dB (state part)", scaled=big)
    # S_f = sum_k e^{cs_f[Q-1] - cs_f[k]} (...): v_f[k] = -dL/dcs_f[k] for k < Q-1; S_b likewise with cs_b[0], k > 0
    assert_close(torch.where(m, vf, 0.0)[..., :-1], -cf.grad[..., :-1], dtype, "v_f", scaled=big)
    assert_close(torch.where(m, vb, 0.0)[..., 1:], -cb_.grad[..., 1:], dtype, "v_b", scaled=big)

    # ---- dC through the entering states + its decay terms   (a13): the scan without its within-chunk part
    dCs, uf, ub = ops._chunk_scan_bwd_dC(pf, pb, csf, csb, dout_x, C=d["C"], ngroups=G)
    C64, cf, cb_ = _leaf(inp["C"]), _leaf(csf), _leaf(csb)
    scan(torch.zeros_like(CB64), r["x"], dt64, cf, cb_, C64, _c(pf), _c(pb), None).backward(dy64)
    assert_close(dCs.sum(0), C64.grad, dtype, "dC (state part)", scaled=big)
    assert_close(torch.where(m, uf, 0.0), cf.grad, dtype, "u_f", scaled=big)
    assert_close(torch.where(m, ub, 0.0), cb_.grad, dtype, "u_b", scaled=big)

    # ---- dCB   (a14)
    dCB, da = ops._chunk_scan_bwd_dcb(d["x"], dt_out, csf, csb, dout_x, CB, ngroups=G)
    CBl = _leaf(CB)
    scan(CBl, r["x"], dt64, csf64, csb64, r["C"], _c(pf), _c(pb), None).backward(dy64)
    lim = min(Q, L - (nc - 1) * Q)     # the last chunk's rows and columns past the sequence end are not part of the contract
    got, ref = _c(dCB).clone(), CBl.grad.clone()
    got[:, -1, :, lim:, :] = 0; got[:, -1, :, :, lim:] = 0
    ref[:, -1, :, lim:, :] = 0; ref[:, -1, :, :, lim:] = 0
    assert_close(got, ref, dtype, "dCB", scaled=big)

    # ---- dB, dC: partial sums + the two products with dCB   (a15)
    dB, dC = ops._bmm_chunk_bwd(d["B"], d["C"], dCB, dBs, dCs)
    B64, C64 = _leaf(inp["B"]), _leaf(inp["C"])
    O.stage_bmm_chunk(C64, B64, Q).backward(ref)
    assert_close(dB, B64.grad + _c(dBs).sum(0), dtype, "dB", scaled=big)
    assert_close(dC, C64.grad + _c(dCs).sum(0), dtype, "dC", scaled=big)

    # ---- ddt, dA, ddt_bias   (a16 + a17): everything that reaches dt * A, against autograd of the whole staged forward
    ddt, dA, ddt_bias = ops._chunk_cumsum_bwd(da, uf, ub, vf, vb, ddAcf, ddAcb, ddt_direct, d["dt"], d["A"],
                                              dt_bias=d["dt_bias"], dt_softplus=True)
    dt_l, A_l, bias_l = _leaf(inp["dt"]), _leaf(inp["A"]), _leaf(inp["dt_bias"])
    O.bimamba2_staged(r["x"], dt_l, A_l, r["B"], r["C"], Q, D=r["D"], dt_bias=bias_l, dt_softplus=True)[0].backward(dy64)
    assert_close(ddt, dt_l.grad, dtype, "ddt", scaled=big)
    assert_close(dA, A_l.grad, dtype, "dA", scaled=big)
    assert_close(ddt_bias, bias_l.grad, dtype, "ddt_bias", scaled=big)


# batch, seqlen, H, P, G, N, chunk, dtype: one K step, a last chunk of one position, two channel tiles, grouped heads, fp16
MERGED = [
    (2, 64, 2, 64, 1, 64, 32, torch.bfloat16),
    (1, 257, 4, 64, 2, 64, 256, torch.bfloat16),
    (1, 200, 2, 128, 2, 64, 96, torch.bfloat16),
    (2, 300, 4, 64, 4, 64, 128, torch.float16),
]


@pytest.mark.parametrize("case", MERGED)
def test_dz_and_dstates_in_one_launch(ops, case):
    """bimamba2_chunk_scan_bwd_dz_dstates against the two separate entry points (themselves held to the oracle above), on
    strided z / dout views as the layer passes them, and its refusal of what it does not cover."""
    b, L, H, P, G, N, Q, dtype = case
    gen = torch.Generator().manual_seed(5)
    wide = torch.randn(b, L, 2 * H * P + 8, generator=gen).to(dtype).cuda()
    z = wide[..., :H * P].view(b, L, H, P)                      # row stride 2 H P + 8: a slice of a wider projection
    dout = wide[..., H * P + 8:].view(b, L, H, P)
    out_x = torch.randn(b, L, H, P, generator=gen).to(dtype).cuda()
    C = torch.randn(b, L, G, N, generator=gen).to(dtype).cuda()
    dt = torch.rand(b, L, H, generator=gen).cuda() * 0.1
    A = -torch.rand(H, generator=gen).cuda() - 0.5
    csf, csb, _ = ops._chunk_cumsum_fwd(dt, A, Q)
    dz, dox = ops._chunk_scan_bwd_dz(out_x, z, out_x, dout, Q)
    dz1, dox1, dpf1, dpb1 = ops._chunk_scan_bwd_dz_dstates(z, out_x, dout, C, csf, csb)
    if dtype == torch.bfloat16:
        assert torch.equal(dz1, dz) and torch.equal(dox1, dox)
    else:
        # float16: the compiler rounds the products to 16 bits in one step in one kernel and in two in the other, which
        # moves one value in 10 000 by one unit in the last place
        for got, want in ((dz1, dz), (dox1, dox)):
            torch.testing.assert_close(got.float(), want.float(), rtol=2.0 ** -10, atol=2.0 ** -24)
            assert int((got != want).sum()) <= got.numel() // 2000
    dpf, dpb = ops._chunk_scan_bwd_dstates(C, csf, csb, dox1)    # from the merged launch's own dout_x: the same bits
    assert torch.equal(dpf1, dpf) and torch.equal(dpb1, dpb)
    with pytest.raises(ValueError):                             # float32: the two separate kernels only (unsupported)
        ops._chunk_scan_bwd_dz_dstates(z.float(), out_x.float(), dout.float(), C.float(), csf, csb)

"""GPU tests of the BiMamba2 layer around the operator, and size-independent properties of the operator at the
baseline's full shapes (where the float64 oracle would take too long)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, make_case, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


def _layer_reference(m, u):
    """The layer's forward with the SSD replaced by the CPU oracle (float64)."""
    sd = {k: v.detach().double().cpu() for k, v in m.state_dict().items()}
    u = u.detach().double().cpu()
    zxbcdt = u @ sd["in_proj.weight"].T
    bc = m.ngroups * m.d_state
    z, xBC, dt = torch.split(zxbcdt, [m.d_inner, m.d_inner + 2 * bc, m.nheads], -1)
    dt = F.softplus(dt + sd["dt_bias"])
    xBC = F.silu(F.conv1d(xBC.transpose(1, 2), sd["conv1d.weight"], sd["conv1d.bias"], padding=m.d_conv // 2,
                          groups=xBC.shape[-1]).transpose(1, 2))
    x, B, C = torch.split(xBC, [m.d_inner, bc, bc], -1)
    y = O.bimamba2_quadratic(x.unflatten(-1, (m.nheads, m.headdim)), dt, -torch.exp(sd["A_log"]),
                             B.unflatten(-1, (m.ngroups, m.d_state)), C.unflatten(-1, (m.ngroups, m.d_state)), D=sd["D"])[0]
    y = y.flatten(-2)
    y = y * torch.rsqrt(y.square().mean(-1, keepdim=True) + 1e-5) * sd["norm.weight"] * F.silu(z)
    return y @ sd["out_proj.weight"].T


def test_bimamba2_layer_forward_backward():
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(0)
    m = BiMamba2(d_model=64, d_state=16, headdim=16, ngroups=1, chunk_size=64).cuda()
    with torch.no_grad():
        m.A_log.copy_(torch.log(torch.rand(m.nheads) * 4 + 0.5))
    u = torch.randn(2, 200, 64, device="cuda", requires_grad=True)
    out = m(u)
    ref = _layer_reference(m, u)
    assert_close(out, ref, torch.float32, "layer output", scale=10)   # float32 GEMMs / conv around the operator
    out.square().mean().backward()
    assert u.grad is not None and torch.isfinite(u.grad).all()
    for name, p in m.named_parameters():
        if name not in ("fc_D.weight",):
            assert p.grad is not None and torch.isfinite(p.grad).all(), name
    # the operator's parameter gradients against autograd through the reference composition
    m2 = BiMamba2(d_model=64, d_state=16, headdim=16, ngroups=1, chunk_size=64).double()
    m2.load_state_dict({k: v.double().cpu() for k, v in m.state_dict().items()})
    assert set(m2.state_dict()) == set(m.state_dict())


def test_bimamba2_layer_bf16_runs():
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(0)
    m = BiMamba2(d_model=128, d_state=64, headdim=64, chunk_size=256).cuda().to(torch.bfloat16)
    u = torch.randn(2, 512, 128, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    out = m(u)
    assert out.shape == u.shape and out.dtype == torch.bfloat16
    out.float().square().mean().backward()
    assert torch.isfinite(u.grad.float()).all()


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
        A = d["A"].clone().requires_grad_(True)
        out = ops.bimamba_chunk_scan_combined(leaves[0], leaves[1], A, leaves[2], leaves[3], cfg["chunk"], D=d["D"],
                                              z=leaves[4], dt_bias=d["dt_bias"], dt_softplus=True)
        grads = torch.autograd.grad(out, leaves + [A], g)
        return out, grads

    out, gr = run(d["x"], d["dt"], d["B"], d["C"], d["z"], dout)
    assert torch.isfinite(out.float()).all()
    fo, fg = run(d["x"].flip(1), d["dt"].flip(1), d["B"].flip(1), d["C"].flip(1), d["z"].flip(1), dout.flip(1))
    # both sides carry bf16 rounding of a different summation order
    assert_close(fo.flip(1), out.float(), torch.bfloat16, "flip: out")
    for name, a, b_ in zip(("dx", "ddt", "dB", "dC", "dz"), fg[:5], gr[:5]):
        assert_close(a.flip(1), b_.float(), torch.bfloat16, "flip: " + name)
    assert_close(fg[5], gr[5].float(), torch.bfloat16, "flip: dA")
    o2, _ = run(2 * d["x"], d["dt"], d["B"], d["C"], d["z"], dout)
    assert_close(o2, 2 * out.float(), torch.bfloat16, "linearity in x")


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
    assert_close(out[:1, :, hs], ref, torch.bfloat16, "long forward")

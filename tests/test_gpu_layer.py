"""GPU tests of the BiMamba2 layer around the operator (reference src/ssd/modules.py:118-187): output, input gradient and
every parameter gradient against float64 autograd through the same composition with the SSD replaced by the CPU oracle,
at a small float32 size and at the baseline's layer configuration (batch 16 x seqlen 1024, d_model 768, bf16)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

# fc_D is created by the reference's constructor and never used by its forward (modules.py:110 there)
UNUSED = ("fc_D.weight",)


def _layer_reference(m, params, u, chunked):
    """The layer's forward in the dtype of `params` / `u` (float64 tensors on the CPU), SSD by the oracle."""
    zxbcdt = u @ params["in_proj.weight"].T
    bc = m.ngroups * m.d_state
    z, xBC, dt = torch.split(zxbcdt, [m.d_inner, m.d_inner + 2 * bc, m.nheads], -1)
    dt = F.softplus(dt + params["dt_bias"])
    xBC = F.silu(F.conv1d(xBC.transpose(1, 2), params["conv1d.weight"], params["conv1d.bias"], padding=m.d_conv // 2,
                          groups=xBC.shape[-1]).transpose(1, 2))
    x, B, C = torch.split(xBC, [m.d_inner, bc, bc], -1)
    args = (x.unflatten(-1, (m.nheads, m.headdim)), dt, -torch.exp(params["A_log"]),
            B.unflatten(-1, (m.ngroups, m.d_state)), C.unflatten(-1, (m.ngroups, m.d_state)))
    if chunked:
        y = O.bimamba2_naive_chunked(*args, m.chunk_size, D=params["D"])[0]
    else:
        y = O.bimamba2_quadratic(*args, D=params["D"])[0]
    y = y.flatten(-2)
    y = y * torch.rsqrt(y.square().mean(-1, keepdim=True) + 1e-5) * params["norm.weight"] * F.silu(z)
    return y @ params["out_proj.weight"].T


def _reference_grads(m, u, dy, chunked):
    params = {k: v.detach().double().cpu().requires_grad_(True) for k, v in m.state_dict().items() if k not in UNUSED}
    u64 = u.detach().double().cpu().requires_grad_(True)
    out = _layer_reference(m, params, u64, chunked)
    out.backward(dy.detach().double().cpu())
    return out.detach(), u64.grad, {k: v.grad for k, v in params.items()}


def test_bimamba2_layer_forward_backward(monkeypatch):
    from bi_mamba2_amd.modules import BiMamba2, _GradPieces
    copies_log = []              # which pieces' gradients each split's backward had to copy into its buffer
    monkeypatch.setattr(_GradPieces, "on_copied", staticmethod(copies_log.append))
    torch.manual_seed(0)
    m = BiMamba2(d_model=64, d_state=16, headdim=16, ngroups=1, chunk_size=64).cuda()
    with torch.no_grad():
        m.A_log.copy_(torch.log(torch.rand(m.nheads) * 4 + 0.5))
    u = torch.randn(2, 200, 64, device="cuda", requires_grad=True)
    dy = torch.randn(2, 200, 64, generator=torch.Generator().manual_seed(1)).cuda()
    out = m(u)
    out.backward(dy)
    ref, du_ref, dp_ref = _reference_grads(m, u, dy, chunked=False)
    # plain float32 tolerance throughout, although float32 GEMMs (torch) and the conv / norm kernels stand between the
    # operator and what is compared
    assert_close(out, ref, torch.float32, "layer output")
    assert_close(u.grad, du_ref, torch.float32, "layer du")
    for name, p in m.named_parameters():
        if name in UNUSED:
            continue
        assert p.grad is not None, name
        assert_close(p.grad, dp_ref[name], torch.float32, "layer d" + name)
    assert set(dp_ref) | set(UNUSED) == set(m.state_dict())
    # the gradients of z (norm) and xBC (convolution) were written in place into the projection output's gradient; only the
    # small dt piece was copied there
    # (the same class serves the split of the convolution's output into x, B, C, whose backward runs first: its three
    # gradients - the operator's dx, dB, dC - arrive in place as well)
    assert copies_log[-2:] == [(), (2,)]


def test_bimamba2_layer_with_a_state_wider_than_the_kernels():
    """d_state 320: the operator sums over pieces of the state dimension, and the layer lets autograd put the gradients
    of x, B, C together (the in-place route is for what the kernels take in one piece)."""
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(3)
    m = BiMamba2(d_model=32, d_state=320, headdim=32, ngroups=1, chunk_size=64).cuda()
    with torch.no_grad():
        m.A_log.copy_(torch.log(torch.rand(m.nheads) * 4 + 0.5))
    u = torch.randn(1, 150, 32, device="cuda", requires_grad=True)
    dy = torch.randn(1, 150, 32, generator=torch.Generator().manual_seed(1)).cuda()
    out = m(u)
    out.backward(dy)
    ref, du_ref, dp_ref = _reference_grads(m, u, dy, chunked=False)
    assert_close(out, ref, torch.float32, "layer output")
    assert_close(u.grad, du_ref, torch.float32, "layer du")
    for name, p in m.named_parameters():
        if name not in UNUSED:
            assert_close(p.grad, dp_ref[name], torch.float32, "layer d" + name)


def test_bimamba2_layer_without_input_gradient_and_twice():
    """Frozen input (only the parameters take gradients) and two backward passes through two forwards that share the
    layer: the buffer of the split's gradients belongs to one forward call."""
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(0)
    m = BiMamba2(d_model=64, d_state=16, headdim=16, ngroups=1, chunk_size=64).cuda()
    u1 = torch.randn(2, 100, 64, device="cuda")
    u2 = torch.randn(2, 100, 64, device="cuda", requires_grad=True)
    o1, o2 = m(u1), m(u2)
    (o1.sum() + 2 * o2.sum()).backward()
    g_both = {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}
    du2 = u2.grad.clone()
    m.zero_grad()
    u2.grad = None
    m(u1).sum().backward()
    g1 = {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}
    m.zero_grad()
    (2 * m(u2).sum()).backward()
    for n, p in m.named_parameters():
        if p.grad is not None:
            assert_close(g_both[n], (g1[n] + p.grad).double(), torch.float32, "sum of two passes, d" + n, scaled=True)
    assert torch.equal(du2, u2.grad)


def test_parameter_maps_in_one_launch():
    """_ParamsAsFloat32 (bimamba2_cast_many behind it): A = -exp(A_log) and float32 copies of 16-bit parameters, and their
    gradients back in the parameters' types, against the torch ops they replace; a missing bias and a parameter without
    gradient included."""
    from bi_mamba2_amd.modules import _ParamsAsFloat32
    g = torch.Generator().manual_seed(4)
    mk = lambda *shape, dt: torch.randn(*shape, generator=g).to(dt).cuda().requires_grad_(True)
    A_log, D, dtb = mk(24, dt=torch.bfloat16), mk(24, dt=torch.float32), mk(24, dt=torch.float16)
    cw, nw = mk(300, 1, 7, dt=torch.bfloat16), mk(1536, dt=torch.bfloat16)
    nw.requires_grad_(False)
    outs = _ParamsAsFloat32.apply(A_log, D, dtb, cw, None, nw)
    assert outs[4] is None and all(o.dtype == torch.float32 for o in outs if o is not None)
    refs = (-torch.exp(A_log.float()), D.float(), dtb.float(), cw.float(), None, nw.float())
    for o, r in zip(outs, refs):
        if o is not None:
            assert o.shape == r.shape
            # exp of a 16-bit value in float32: the library's and torch's exp may differ in the last bit
            assert torch.allclose(o, r.detach(), rtol=1e-6, atol=0)
    assert not outs[5].requires_grad
    gs = [torch.randn(o.shape, generator=g).cuda() for o in outs[:4]]
    loss = sum((o * w).sum() for o, w in zip(outs[:4], gs))
    loss.backward()
    want = {"A_log": (gs[0] * refs[0].detach()).to(torch.bfloat16), "D": gs[1], "dt_bias": gs[2].to(torch.float16),
            "conv": gs[3].to(torch.bfloat16)}
    got = {"A_log": A_log.grad, "D": D.grad, "dt_bias": dtb.grad, "conv": cw.grad}
    for k in want:
        assert got[k].dtype == want[k].dtype and got[k].shape == want[k].shape, k
        assert torch.allclose(got[k].float(), want[k].float(), rtol=1e-2 if k == "A_log" else 0, atol=0), k
    assert nw.grad is None


def test_bimamba2_layer_bf16_runs():
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(0)
    m = BiMamba2(d_model=128, d_state=64, headdim=64, chunk_size=256).cuda().to(torch.bfloat16)
    u = torch.randn(2, 512, 128, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    out = m(u)
    assert out.shape == u.shape and out.dtype == torch.bfloat16
    out.float().square().mean().backward()
    assert torch.isfinite(u.grad.float()).all()


def test_bimamba2_layer_baseline_configuration():
    """The baseline's layer configuration: d_model 768, d_state 64, d_conv 7, expand 2, headdim 64 (24 heads), one group,
    chunk 256, batch 16 x seqlen 1024, bf16, weights as the constructor draws them.  The full batch runs forward and
    backward; output and input gradient of two batch rows are compared with the float64 composition, and the parameter
    gradients with those of the same two rows run as a batch of their own (they are sums over the batch)."""
    from bi_mamba2_amd.modules import BiMamba2
    torch.manual_seed(0)
    dt16 = torch.bfloat16
    m = BiMamba2(d_model=768, d_state=64, d_conv=7, expand=2, headdim=64, ngroups=1, chunk_size=256).cuda().to(dt16)
    assert m.nheads == 24 and m.d_inner == 1536
    g = torch.Generator().manual_seed(2)
    u = torch.randn(16, 1024, 768, generator=g).to(dt16).cuda().requires_grad_(True)
    dy = torch.randn(16, 1024, 768, generator=g).to(dt16).cuda()
    out = m(u)
    out.backward(dy)
    assert out.shape == u.shape and out.dtype == dt16
    assert torch.isfinite(out.float()).all() and torch.isfinite(u.grad.float()).all()
    full_grads = {k: p.grad.clone() for k, p in m.named_parameters() if k not in UNUSED}

    rows = [0, 11]
    ref, du_ref, dp_ref = _reference_grads(m, u[rows], dy[rows], chunked=True)
    # bf16 GEMM outputs, conv output, SSD output and norm output are each rounded to bf16 on the device and not in
    # the float64 composition; output and input gradient still meet the plain bf16 bound, the parameter gradients (sums
    # over 2048 positions) are compared in units of their RMS
    assert_close(out[rows], ref, dt16, "layer output (rows of the full batch)")
    assert_close(u.grad[rows], du_ref, dt16, "layer du (rows of the full batch)")

    m.zero_grad(set_to_none=True)
    u2 = u.detach()[rows].clone().requires_grad_(True)
    out2 = m(u2)
    out2.backward(dy[rows])
    assert_close(out2, ref, dt16, "layer output")
    assert_close(u2.grad, du_ref, dt16, "layer du")
    for name, p in m.named_parameters():
        if name in UNUSED:
            continue
        assert_close(p.grad, dp_ref[name], dt16, "layer d" + name, scaled=True)
        # the full batch's parameter gradients: finite and of the size eight such pairs of rows would give
        fg = full_grads[name].float()
        assert torch.isfinite(fg).all(), name
        assert fg.norm() <= 16 * max(p.grad.float().norm(), 1e-3), name

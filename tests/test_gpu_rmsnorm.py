"""GPU parity of the gated RMS norm and of the gated LayerNorm (forward and backward, through the C ABI) against the
float64 oracle."""
import pytest
import torch

from oracle.rmsnorm_oracle import rms_norm_gated
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

CASES = [
    # shape, group_size, z, bias, norm_before_gate, dtype
    ((2, 37, 256), None, True, False, True, torch.float32),      # the BiMamba2 layer's configuration
    ((2, 37, 256), None, True, False, False, torch.float32),
    ((3, 5, 192), 64, True, True, True, torch.float32),          # groups + bias
    ((3, 5, 192), 64, False, False, True, torch.float32),        # no gate
    ((4, 100), None, True, False, True, torch.float32),          # width not a multiple of 8: scalar accesses
    ((2, 64, 2048), None, True, False, True, torch.bfloat16),    # the benchmark layer's width
    ((2, 64, 2048), 512, True, True, False, torch.bfloat16),
    ((5, 37, 1536), None, True, False, True, torch.bfloat16),    # 3 x 512 columns: the baseline layer's width (d_model 768)
    ((8, 4096), None, True, False, True, torch.float16),
    ((3, 8192), None, False, False, True, torch.bfloat16),       # the widest group one wave holds
    ((600, 2, 128), None, True, True, True, torch.float32),      # more rows than partial-sum slots
    ((5, 16384), None, True, False, True, torch.bfloat16),       # beyond 8192 columns: one workgroup per (row, group)
    ((3, 2, 24576), 12288, True, True, False, torch.float16),    # two wide groups, bias, gate first
    ((4, 9000), None, False, True, True, torch.float32),         # wide, no gate, width not a multiple of 512
    ((2, 32768), None, True, False, True, torch.bfloat16),       # the widest group (64 KB of a 16-bit row, as the reference)
]


@pytest.mark.parametrize("rms", [True, False], ids=["rmsnorm", "layernorm"])
@pytest.mark.parametrize("case", CASES)
def test_rmsnorm_gated_forward_backward(case, rms):
    from bi_mamba2_amd.layernorm_gated import layernorm_fn
    shape, gs, with_z, with_b, before, dtype = case
    g = torch.Generator().manual_seed(3)
    n = shape[-1]
    x = torch.randn(shape, generator=g)
    if not rms:
        x = x + 0.75                     # a mean worth subtracting
    x = x.to(dtype)
    z = torch.randn(shape, generator=g).to(dtype) if with_z else None
    w = (1.0 + 0.3 * torch.randn(n, generator=g)).float()
    b = (0.2 * torch.randn(n, generator=g)).float() if with_b else None
    dy = torch.randn(shape, generator=g).to(dtype)
    leaves = [t.cuda().requires_grad_(True) if t is not None else None for t in (x, w, b, z)]
    out = layernorm_fn(leaves[0], leaves[1], leaves[2], z=leaves[3], eps=1e-5, group_size=gs, norm_before_gate=before, is_rms_norm=rms)
    assert out.dtype == dtype and out.shape == tuple(shape)
    out.backward(dy.cuda())
    ref_leaves = [t.double().requires_grad_(True) if t is not None else None for t in (x, w, b, z)]
    ref = rms_norm_gated(ref_leaves[0], ref_leaves[1], ref_leaves[2], ref_leaves[3], eps=1e-5, group_size=gs, norm_before_gate=before,
                         is_rms_norm=rms)
    ref.backward(dy.double())
    assert_close(out, ref.detach(), dtype, "out")
    for got, r, name in zip(leaves, ref_leaves, ("dx", "dweight", "dbias", "dz")):
        if r is not None:
            assert_close(got.grad, r.grad, dtype, name)


def test_rmsnorm_strided_rows_and_module():
    """Rows that are views into a wider projection output (as in the layer), and the module with its parameter."""
    from bi_mamba2_amd.layernorm_gated import RMSNorm
    g = torch.Generator().manual_seed(5)
    wide = torch.randn(2, 33, 3 * 128, generator=g).cuda()
    x, z = wide[..., :128], wide[..., 256:]
    m = RMSNorm(128, eps=1e-5, norm_before_gate=True, device="cuda")
    with torch.no_grad():
        m.weight.copy_(1.0 + 0.1 * torch.randn(128, generator=g))
    out = m(x, z)
    ref = rms_norm_gated(x.double().cpu(), m.weight.detach().double().cpu(), None, z.double().cpu(), eps=1e-5)
    assert_close(out, ref, torch.float32, "out (strided)")


def test_rmsnorm_gate_gradient_into_a_slice():
    """dz_place: the gradient of z lands in a slice of a wider buffer (the layer's use), bit for bit what the plain call
    returns."""
    from bi_mamba2_amd.layernorm_gated import rmsnorm_fn
    g = torch.Generator().manual_seed(8)
    x = torch.randn(3, 21, 128, generator=g).to(torch.bfloat16).cuda()
    z = torch.randn(3, 21, 128, generator=g).to(torch.bfloat16).cuda()
    w = (1.0 + 0.1 * torch.randn(128, generator=g)).cuda()
    dy = torch.randn(3, 21, 128, generator=g).to(torch.bfloat16).cuda()
    za = z.clone().requires_grad_(True)
    rmsnorm_fn(x, w, None, z=za, eps=1e-5).backward(dy)
    wide = torch.full((3, 21, 128 + 40), 3.0, dtype=torch.bfloat16, device="cuda")
    zb = z.clone().requires_grad_(True)
    rmsnorm_fn(x, w, None, z=zb, eps=1e-5, dz_place=lambda: wide[..., 16:16 + 128]).backward(dy)
    assert torch.equal(zb.grad, za.grad) and torch.equal(wide[..., 16:16 + 128], za.grad)
    assert (wide[..., :16] == 3.0).all() and (wide[..., 16 + 128:] == 3.0).all()


def test_layernorm_module():
    """The LayerNorm module (weight and bias parameters), gated, against the oracle."""
    from bi_mamba2_amd.layernorm_gated import LayerNorm
    g = torch.Generator().manual_seed(6)
    x, z = (torch.randn(3, 20, 96, generator=g) + 1.5).cuda(), torch.randn(3, 20, 96, generator=g).cuda()
    m = LayerNorm(96, eps=1e-5, group_size=32, norm_before_gate=False, device="cuda")
    with torch.no_grad():
        m.weight.copy_(1.0 + 0.1 * torch.randn(96, generator=g))
        m.bias.copy_(0.1 * torch.randn(96, generator=g))
    x.requires_grad_(True)
    out = m(x, z)
    out.sum().backward()
    xr = x.detach().double().cpu().requires_grad_(True)
    wr, br = m.weight.detach().double().cpu().requires_grad_(True), m.bias.detach().double().cpu().requires_grad_(True)
    ref = rms_norm_gated(xr, wr, br, z.double().cpu(), eps=1e-5, group_size=32, norm_before_gate=False, is_rms_norm=False)
    ref.sum().backward()
    assert_close(out, ref.detach(), torch.float32, "out")
    assert_close(x.grad, xr.grad, torch.float32, "dx")
    assert_close(m.weight.grad, wr.grad, torch.float32, "dweight")
    assert_close(m.bias.grad, br.grad, torch.float32, "dbias")


def test_rmsnorm_refuses_cpu_tensors_and_bad_groups():
    from bi_mamba2_amd.layernorm_gated import rmsnorm_fn
    with pytest.raises(RuntimeError):
        rmsnorm_fn(torch.randn(4, 64), torch.ones(64), None)
    with pytest.raises((ValueError, AssertionError)):
        rmsnorm_fn(torch.randn(4, 64).cuda(), torch.ones(64).cuda(), None, group_size=48)

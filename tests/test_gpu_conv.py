"""GPU parity of the depthwise conv1d + SiLU kernels (forward and backward) against the float64 oracle, through the
C ABI, on contiguous inputs and on strided views like the layer's."""
import pytest
import torch

from oracle.conv_oracle import conv1d_silu
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

CASES = [
    # batch, seqlen, channels, width, dtype, bias, view
    (2, 100, 64, 7, torch.float32, True, False),
    (3, 57, 24, 3, torch.float32, False, True),
    (1, 5, 8, 9, torch.float32, True, False),          # sequence shorter than the filter
    (2, 300, 1664, 7, torch.bfloat16, True, True),     # the layer's conv channels, a view of the projection output
    (2, 129, 96, 5, torch.float16, True, False),
    (2, 64, 30, 7, torch.bfloat16, True, False),       # channels not a multiple of 4: one channel per thread
    (1, 40, 16, 1, torch.float32, True, False),
]


@pytest.mark.parametrize("case", CASES)
def test_conv1d_silu_forward_and_backward(case):
    from bi_mamba2_amd.conv1d import conv1d_silu_fn
    b, L, C, W, dtype, has_bias, view = case
    g = torch.Generator().manual_seed(0)
    extra = 40 if view else 0
    big = torch.randn(b, L, C + extra, generator=g).to(dtype)
    x = big[..., 8:8 + C] if view else big
    w = (torch.randn(C, 1, W, generator=g) * 0.4)
    bias = torch.randn(C, generator=g) * 0.2 if has_bias else None
    dout = torch.randn(b, L, C, generator=g).to(dtype)

    xd = x.cuda() if not view else big.cuda()[..., 8:8 + C]
    xd = xd.detach().requires_grad_(True)
    wd = w.cuda().requires_grad_(True)
    bd = bias.cuda().requires_grad_(True) if has_bias else None
    out = conv1d_silu_fn(xd, wd, bd)
    assert out.shape == (b, L, C) and out.dtype == dtype and out.is_contiguous()
    out.backward(dout.cuda())

    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    b64 = bias.double().requires_grad_(True) if has_bias else None
    ref = conv1d_silu(x64, w64, b64)
    ref.backward(dout.double())
    assert_close(out, ref, dtype, "out")
    assert_close(xd.grad, x64.grad, dtype, "dx")
    # the filter gradients are float32 sums over batch * seqlen terms that carry the input rounding
    assert_close(wd.grad, w64.grad, dtype, "dweight")
    if has_bias:
        assert_close(bd.grad, b64.grad, dtype, "dbias")


@pytest.mark.parametrize("dtype,C", [(torch.bfloat16, 64), (torch.float32, 5)])
def test_conv1d_silu_gradient_into_a_slice(dtype, C):
    """dx_place: the gradient of x lands in a slice of a wider buffer (the layer's use), bit for bit what the plain call
    returns, and the rest of the buffer stays as it was."""
    from bi_mamba2_amd.conv1d import conv1d_silu_fn
    g = torch.Generator().manual_seed(2)
    b, L, W = 2, 50, 7
    x = torch.randn(b, L, C, generator=g).to(dtype).cuda()
    w = (0.3 * torch.randn(C, 1, W, generator=g)).cuda()
    bias = (0.1 * torch.randn(C, generator=g)).cuda()
    dout = torch.randn(b, L, C, generator=g).to(dtype).cuda()
    xa = x.clone().requires_grad_(True)
    conv1d_silu_fn(xa, w, bias).backward(dout)
    wide = torch.full((b, L, C + 24), 7.0, dtype=dtype, device="cuda")
    xb = x.clone().requires_grad_(True)
    conv1d_silu_fn(xb, w, bias, dx_place=lambda: wide[..., 8:8 + C]).backward(dout)
    assert torch.equal(xb.grad, xa.grad) and torch.equal(wide[..., 8:8 + C], xa.grad)
    assert (wide[..., :8] == 7.0).all() and (wide[..., 8 + C:] == 7.0).all()


def test_conv1d_silu_errors():
    from bi_mamba2_amd.conv1d import conv1d_silu_fn
    x = torch.randn(1, 8, 4)
    with pytest.raises(Exception):
        conv1d_silu_fn(x, torch.randn(4, 1, 3))                      # CPU tensor: there is no fallback
    with pytest.raises(ValueError):
        conv1d_silu_fn(x.cuda(), torch.randn(4, 1, 4).cuda())        # even width

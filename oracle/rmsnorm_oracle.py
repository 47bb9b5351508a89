"""CPU restatement of the reference's gated RMS norm.  TEST INFRASTRUCTURE ONLY: imported by tests/, by
__graft_entry__.smoke() and by bench.py's baseline leg, never by the product path.

Follows rms_norm_ref (src/ssd/bi/layernorm_gated.py:18-39 of Hprairie/Bi-Mamba2): optional gate before the norm,
mean of squares over the whole row or over groups of `group_size` consecutive columns, weight, optional bias,
optional gate after the norm.  Written on torch tensors so that float64 inputs give a float64 result and
torch.autograd gives the gradients.

Pinned by tests/test_oracle_rmsnorm.py: against torch.nn.functional.rms_norm (no gate, one group), against a scalar
Python loop on a tiny case, the two gate orders against each other's definition, groups against the ungrouped norm
of the reshaped rows, scale invariance (norm(c*x) = norm(x) for eps = 0), and finite-difference gradcheck.
"""
import torch
import torch.nn.functional as F


def rms_norm_gated(x, weight, bias=None, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=True):
    """is_rms_norm=False: the LayerNorm of the same reference kernels (IS_RMS_NORM = False,
    src/ssd/bi/layernorm_gated.py:66-76 there) - the group mean is subtracted before the mean of squares is taken."""
    if z is not None and not norm_before_gate:
        x = x * F.silu(z)
    n = x.shape[-1]
    gs = n if group_size is None else group_size
    assert n % gs == 0
    xg = x.reshape(*x.shape[:-1], n // gs, gs)
    if not is_rms_norm:
        xg = xg - xg.mean(dim=-1, keepdim=True)
    rstd = 1.0 / torch.sqrt(xg.square().mean(dim=-1, keepdim=True) + eps)
    out = (xg * rstd).reshape(x.shape) * weight
    if bias is not None:
        out = out + bias
    if z is not None and norm_before_gate:
        out = out * F.silu(z)
    return out

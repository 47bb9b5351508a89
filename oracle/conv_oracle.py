"""CPU restatement of the layer's non-causal depthwise conv1d + SiLU.  TEST INFRASTRUCTURE ONLY: imported by tests/,
never by the product path.

Follows what the reference layer does with xBC (src/ssd/modules.py:162-164 of Hprairie/Bi-Mamba2, convolution constructed
at :68-75: nn.Conv1d(C, C, kernel_size=d_conv, groups=C, padding=d_conv // 2), then SiLU), written on channels-last
tensors as a sum of shifted copies, so that float64 inputs give a float64 result and torch.autograd gives the gradients.

Pinned by tests/test_oracle_conv.py: against torch.nn.functional.conv1d + silu (the library routine the reference calls)
on the transposed tensors, against a scalar Python loop on a tiny case, against the identity filter, and by
finite-difference gradcheck.
"""
import torch
import torch.nn.functional as F


def conv1d_silu(x, weight, bias=None):
    """x: (batch, seqlen, channels); weight: (channels, width) or (channels, 1, width), width odd; bias: (channels)."""
    channels, width = weight.shape[0], weight.shape[-1]
    assert width % 2 == 1 and x.shape[-1] == channels
    w = weight.reshape(channels, width)
    h = width // 2
    xp = F.pad(x, (0, 0, h, h))
    L = x.shape[1]
    pre = sum(xp[:, k:k + L, :] * w[:, k] for k in range(width))
    if bias is not None:
        pre = pre + bias
    return pre * torch.sigmoid(pre)

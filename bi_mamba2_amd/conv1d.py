"""Non-causal depthwise conv1d + SiLU on channels-last activations, on the HIP kernels.

It replaces ``act(conv1d(xBC.transpose(1, 2)).transpose(1, 2))`` of the reference layer (src/ssd/modules.py:162-164 of
Hprairie/Bi-Mamba2; the convolution is ``nn.Conv1d(C, C, d_conv, groups=C, padding=d_conv // 2)``, :68-75 there) with
one kernel that reads the (batch, seqlen, channels) view of the projection output as it lies and needs no transposes:

    out[b, l, c] = silu(bias[c] + sum_k weight[c, 0, k] * x[b, l + k - d_conv // 2, c])     (zero padding, d_conv odd)

There is no CPU or PyTorch fallback: CPU tensors raise, a missing library raises.
"""
import ctypes

import torch

from . import _lib
from .ops import _DT, _require_gpu


def _call(entry, p, device):
    lib = _lib.load()
    with torch.cuda.device(device):
        p.stream = torch.cuda.current_stream().cuda_stream
        rc = getattr(lib, entry)(ctypes.byref(p))
    if rc != 0:
        msg = lib.bimamba2_strerror(rc).decode()
        raise (ValueError if rc in (-1, -2) else RuntimeError)(f"{entry}: {msg} (code {rc})")


def _view3(t, name):
    """(batch, seqlen, channels) with unit stride along channels (other strides are passed on as they are)."""
    _require_gpu(t, name)
    assert t.dim() == 3, f"{name}: expected (batch, seqlen, channels)"
    return t if t.stride(-1) == 1 else t.contiguous()


def _params(x, weight, bias):
    if x.dtype not in _DT:
        raise ValueError(f"unsupported dtype {x.dtype} (need float32, bfloat16 or float16)")
    batch, seqlen, channels = x.shape
    assert weight.shape[0] == channels and weight.dim() in (2, 3), "weight: (channels, width) or (channels, 1, width)"
    width = weight.shape[-1]
    w32 = weight.detach().reshape(channels, width).float().contiguous()
    b32 = bias.detach().float().contiguous() if bias is not None else None
    p = _lib.ConvParams()
    p.batch, p.seqlen, p.channels, p.width = batch, seqlen, channels, width
    p.dtype, p.has_bias = _DT[x.dtype], int(bias is not None)
    p.x, p.x_sb, p.x_sl = x.data_ptr(), x.stride(0), x.stride(1)
    p.weight = w32.data_ptr()
    if b32 is not None:
        p.bias = b32.data_ptr()
    return p, (w32, b32)


def _conv1d_silu_fwd(x, weight, bias):
    x = _view3(x, "x")
    p, keep = _params(x, weight, bias)
    out = torch.empty(x.shape, device=x.device, dtype=x.dtype)
    p.out = out.data_ptr()
    _call("bimamba2_conv1d_silu_fwd", p, x.device)
    return out


def _conv1d_silu_bwd(dout, x, weight, bias, dx_out=None):
    """-> dx (batch, seqlen, channels), dweight (channels, width) float32, dbias (channels) float32 or None.
    dx_out: where dx is to be written (same shape and dtype as x, unit stride along channels: e.g. a slice of a wider
    buffer); a new tensor when None."""
    x, dout = _view3(x, "x"), _view3(dout, "dout")
    assert dout.shape == x.shape
    p, keep = _params(x, weight, bias)
    if dx_out is not None and (dx_out.shape != x.shape or dx_out.dtype != x.dtype or dx_out.stride(-1) != 1 or dx_out.device != x.device):
        dx_out = None
    dx = dx_out if dx_out is not None else torch.empty(x.shape, device=x.device, dtype=x.dtype)
    p.dx_sb, p.dx_sl = dx.stride(0), dx.stride(1)
    dw = torch.empty((p.channels, p.width), device=x.device, dtype=torch.float32)
    db = torch.empty((p.channels,), device=x.device, dtype=torch.float32) if bias is not None else None
    p.dout, p.dout_sb, p.dout_sl = dout.data_ptr(), dout.stride(0), dout.stride(1)
    p.dx, p.dweight = dx.data_ptr(), dw.data_ptr()
    if db is not None:
        p.dbias = db.data_ptr()
    n = _lib.load().bimamba2_conv1d_silu_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(int(n), 1), device=x.device, dtype=torch.uint8)
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    _call("bimamba2_conv1d_silu_bwd", p, x.device)
    return dx, dw, db


class Conv1dSiluFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias=None, dx_place=None):
        ctx.save_for_backward(x, weight, bias)
        ctx.dx_place = dx_place
        return _conv1d_silu_fwd(x, weight, bias)

    @staticmethod
    def backward(ctx, dout):
        x, weight, bias = ctx.saved_tensors
        dx, dw, db = _conv1d_silu_bwd(dout, x, weight, bias, dx_out=ctx.dx_place() if ctx.dx_place is not None else None)
        return dx, dw.reshape(weight.shape).to(weight.dtype), (db.to(bias.dtype) if bias is not None else None), None


def conv1d_silu_fn(x, weight, bias=None, dx_place=None):
    """x: (batch, seqlen, channels), channels contiguous (a strided view is fine); weight: (channels, 1, width) as
    nn.Conv1d keeps it, or (channels, width); bias: (channels,) or None.  width odd, at most 9.
    dx_place: optional callable, asked in the backward pass for the tensor the gradient of x is to be written into (shaped
    like x, unit stride along channels) - the layer hands out slices of one buffer for the gradients of the pieces of its
    projection output, which saves concatenating them."""
    return Conv1dSiluFn.apply(x, weight, bias, dx_place)

"""Gated RMSNorm / LayerNorm on the HIP kernels, with the reference's names (src/ssd/bi/layernorm_gated.py of
Hprairie/Bi-Mamba2): ``rmsnorm_fn`` (:383-384 there) and ``layernorm_fn`` (:380-381), the ``RMSNorm`` (:415-437) and
``LayerNorm`` (:388-412) modules and the autograd function behind them (``LayerNormFn``, :333-376).

    xg  = x                    if norm_before_gate else x * silu(z)
    xc  = xg                   (RMS norm)         or  xg - mean_group(xg)   (LayerNorm, is_rms_norm=False)
    y   = xc / sqrt(mean_group(xc^2) + eps) * weight (+ bias)
    out = y * silu(z)          if norm_before_gate else y

There is no CPU or PyTorch fallback: CPU tensors raise, a missing library raises.
"""
import ctypes

import torch

from . import _lib
from .ops import _DT, _require_gpu


def _rows(t, name):
    _require_gpu(t, name)
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(-1) != 1:
        t2 = t2.contiguous()
    return t2


def _call(entry, p, device):
    lib = _lib.load()
    with torch.cuda.device(device):
        p.stream = torch.cuda.current_stream().cuda_stream
        rc = getattr(lib, entry)(ctypes.byref(p))
    if rc != 0:
        msg = lib.bimamba2_strerror(rc).decode()
        raise (ValueError if rc in (-1, -2) else RuntimeError)(f"{entry}: {msg} (code {rc})")


def _params(x2, z2, weight, bias, eps, group_size, norm_before_gate, is_rms_norm=True):
    if x2.dtype not in _DT:
        raise ValueError(f"unsupported dtype {x2.dtype} (need float32, bfloat16 or float16)")
    p = _lib.NormParams()
    p.rows, p.cols = x2.shape
    p.group_size = group_size if group_size is not None else x2.shape[1]
    p.dtype = _DT[x2.dtype]
    p.has_z, p.has_bias, p.norm_before_gate = int(z2 is not None), int(bias is not None), int(bool(norm_before_gate))
    p.eps = float(eps)
    p.layer_norm = int(not is_rms_norm)
    p.x, p.x_rs = x2.data_ptr(), x2.stride(0)
    if z2 is not None:
        p.z, p.z_rs = z2.data_ptr(), z2.stride(0)
    p.weight = weight.data_ptr()
    if bias is not None:
        p.bias = bias.data_ptr()
    return p


def _layer_norm_fwd(x, weight, bias, eps, z=None, group_size=None, norm_before_gate=True, is_rms_norm=True):
    """x, z: (rows, cols) with unit stride along cols; weight, bias: (cols,) float32.  -> out, rstd (rows, ngroups) for the
    RMS norm; out, mean, rstd for the LayerNorm (is_rms_norm=False)."""
    rows, cols = x.shape
    gs = group_size if group_size is not None else cols
    assert cols % gs == 0
    assert weight.shape == (cols,) and (bias is None or bias.shape == (cols,))
    assert z is None or z.shape == x.shape
    p = _params(x, z, weight, bias, eps, group_size, norm_before_gate, is_rms_norm)
    out = torch.empty((rows, cols), device=x.device, dtype=x.dtype)
    rstd = torch.empty((rows, cols // gs), device=x.device, dtype=torch.float32)
    p.out, p.out_rs, p.rstd = out.data_ptr(), out.stride(0), rstd.data_ptr()
    mean = None
    if not is_rms_norm:
        mean = torch.empty_like(rstd)
        p.mean = mean.data_ptr()
    _call("bimamba2_rmsnorm_gated_fwd", p, x.device)
    return (out, rstd) if is_rms_norm else (out, mean, rstd)


def _layer_norm_bwd(dy, x, weight, bias, eps, rstd, z=None, group_size=None, norm_before_gate=True, mean=None, dz_out=None):
    """-> dx, dweight (float32), dbias (float32 or None), dz (or None).  mean: the forward's group means (LayerNorm), None
    for the RMS norm.  dz_out: where dz is to be written (rows like x, unit stride along the columns), a new tensor when
    None."""
    p = _params(x, z, weight, bias, eps, group_size, norm_before_gate, mean is None)
    if mean is not None:
        p.mean = mean.data_ptr()
    dx = torch.empty_like(x, memory_format=torch.contiguous_format)
    if dz_out is not None and (z is None or dz_out.shape != x.shape or dz_out.dtype != x.dtype or dz_out.stride(-1) != 1
                               or dz_out.device != x.device):
        dz_out = None
    dz = dz_out if dz_out is not None else (torch.empty_like(x, memory_format=torch.contiguous_format) if z is not None else None)
    dw = torch.empty((x.shape[1],), device=x.device, dtype=torch.float32)
    db = torch.empty_like(dw) if bias is not None else None
    p.dout, p.dout_rs, p.rstd = dy.data_ptr(), dy.stride(0), rstd.data_ptr()
    p.dx, p.dx_rs, p.dweight = dx.data_ptr(), dx.stride(0), dw.data_ptr()
    if dz is not None:
        p.dz, p.dz_rs = dz.data_ptr(), dz.stride(0)
    if db is not None:
        p.dbias = db.data_ptr()
    n = _lib.load().bimamba2_rmsnorm_gated_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(int(n), 1), device=x.device, dtype=torch.uint8)
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    _call("bimamba2_rmsnorm_gated_bwd", p, x.device)
    return dx, dw, db, dz


class LayerNormFn(torch.autograd.Function):
    """The reference's function of the same name: gated RMS norm (is_rms_norm=True) or gated LayerNorm."""

    @staticmethod
    def forward(ctx, x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False,
                dz_place=None):
        # dz_place: optional callable, asked in the backward pass for the tensor the gradient of z is to be written into
        # (shaped like z, unit stride along the last dimension, rows at one stride: e.g. a slice of a wider buffer)
        ctx.dz_place = dz_place
        shape = x.shape
        x2 = _rows(x, "x")
        z2 = _rows(z, "z") if z is not None else None
        if z2 is not None:
            assert z.shape == shape
            if z2.dtype != x2.dtype:
                z2 = z2.to(x2.dtype)
        w32 = weight.detach().float().contiguous()
        b32 = bias.detach().float().contiguous() if bias is not None else None
        _require_gpu(w32, "weight")
        res = _layer_norm_fwd(x2, w32, b32, eps, z=z2, group_size=group_size, norm_before_gate=norm_before_gate,
                              is_rms_norm=is_rms_norm)
        out, rstd, mean = res[0], res[-1], (None if is_rms_norm else res[1])
        ctx.save_for_backward(x2, w32, b32, rstd, z2, mean)
        ctx.shape, ctx.eps, ctx.group_size, ctx.norm_before_gate = shape, eps, group_size, norm_before_gate
        ctx.wdtype = weight.dtype
        ctx.bdtype = bias.dtype if bias is not None else None
        ctx.zdtype = z.dtype if z is not None else None
        return out.reshape(shape)

    @staticmethod
    def backward(ctx, dy):
        x2, w32, b32, rstd, z2, mean = ctx.saved_tensors
        dy2 = _rows(dy, "dy")
        if dy2.dtype != x2.dtype:
            dy2 = dy2.to(x2.dtype)
        place, dz_rows = None, None
        if ctx.dz_place is not None and z2 is not None and ctx.zdtype == x2.dtype:
            place = ctx.dz_place()
            if place is not None and tuple(place.shape) == tuple(ctx.shape) and place.stride(-1) == 1:
                try:
                    dz_rows = place.view(-1, ctx.shape[-1])          # rows at one stride, or no view exists
                except RuntimeError:
                    place = None
            else:
                place = None
        dx, dw, db, dz = _layer_norm_bwd(dy2, x2, w32, b32, ctx.eps, rstd, z=z2, group_size=ctx.group_size,
                                         norm_before_gate=ctx.norm_before_gate, mean=mean, dz_out=dz_rows)
        if dz is not None:
            dz = place if (place is not None and dz is dz_rows) else dz.reshape(ctx.shape).to(ctx.zdtype)
        return (dx.reshape(ctx.shape), dw.to(ctx.wdtype), db.to(ctx.bdtype) if db is not None else None,
                dz, None, None, None, None, None)


MAX_GROUP = 32768     # columns per normalisation group (bimamba2_rmsnorm_gated_fwd / _bwd refuse more)


def layernorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, is_rms_norm=False):
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, is_rms_norm)


def rmsnorm_fn(x, weight, bias, z=None, eps=1e-6, group_size=None, norm_before_gate=True, dz_place=None):
    return LayerNormFn.apply(x, weight, bias, z, eps, group_size, norm_before_gate, True, dz_place)


class LayerNorm(torch.nn.Module):
    """Same constructor, parameters (weight and bias) and forward as the reference's module (:388-412 there)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        super().__init__()
        if (group_size or hidden_size) > MAX_GROUP:
            raise ValueError(f"LayerNorm: groups of {group_size or hidden_size} columns exceed the {MAX_GROUP} the kernels support")
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.bias = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)
        torch.nn.init.zeros_(self.bias)

    def forward(self, x, z=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z)); plain norm without z."""
        return layernorm_fn(x, self.weight, self.bias, z=z, eps=self.eps, group_size=self.group_size,
                            norm_before_gate=self.norm_before_gate)


class RMSNorm(torch.nn.Module):
    """Same constructor, parameters and forward as the reference's module (no bias parameter)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, device=None, dtype=None):
        super().__init__()
        # the kernels hold a group of at most MAX_GROUP columns per wave (the reference's Triton kernel: 64 KB per row);
        # refuse a wider one where the module is built rather than at the first forward
        if (group_size or hidden_size) > MAX_GROUP:
            raise ValueError(f"RMSNorm: groups of {group_size or hidden_size} columns exceed the {MAX_GROUP} the kernels support")
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x, z=None, dz_place=None):
        """norm(x) * silu(z) if norm_before_gate, else norm(x * silu(z)); plain norm without z.  dz_place (not in the
        reference): see LayerNormFn.forward."""
        return rmsnorm_fn(x, self.weight, self.bias, z=z, eps=self.eps, group_size=self.group_size,
                          norm_before_gate=self.norm_before_gate, dz_place=dz_place)

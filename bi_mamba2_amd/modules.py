"""``BiMamba2`` layer around the bidirectional SSD operator.

Same constructor keywords, parameter names/shapes (so state_dicts interchange) and forward math as the
reference layer (src/ssd/modules.py:17-187): in_proj -> split [z | xBC | dt] -> softplus(dt + dt_bias) ->
non-causal depthwise conv1d + SiLU -> split x, B, C -> bidirectional SSD with D -> gated RMSNorm(y, z) ->
out_proj.  Parameters are created in the reference's order, so a seeded construction draws the same values.
The projections and the convolution are ordinary torch ops; the SSD and the gated RMS norm are the HIP operators.
"""
import ctypes
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .conv1d import conv1d_silu_fn
from .layernorm_gated import RMSNorm, rmsnorm_fn
from .ops import _DT, bimamba_chunk_scan_combined


# the gated RMS norm of the layer runs on the HIP kernels (bi_mamba2_amd/layernorm_gated.py)
RMSNormGated = RMSNorm


class _GradPieces:
    """One buffer for the gradients of the pieces a tensor is split into along its last dimension.  torch.split's backward
    concatenates the pieces' gradients, a copy of the whole projection output's gradient (100 MB at the benchmark layer);
    here the kernels that produce the large pieces write them into slices of the buffer (piece(i), asked for in the
    backward pass) and the split's backward hands the buffer on as it is."""

    # debug hook: a callable given the indices of the pieces whose gradients had to be copied into the buffer in one
    # backward pass (None, the default: nothing is recorded; the tests set it to see that the large pieces arrive in place)
    on_copied = None

    def __init__(self, like, sizes):
        self.shape, self.dtype, self.device = tuple(like.shape), like.dtype, like.device
        self.bounds = [0]
        for n in sizes:
            self.bounds.append(self.bounds[-1] + n)
        assert self.bounds[-1] == self.shape[-1]
        self.buf = None

    def piece(self, i):
        if self.buf is None:
            self.buf = torch.empty(self.shape, dtype=self.dtype, device=self.device)
        return self.buf[..., self.bounds[i]:self.bounds[i + 1]]

    def place(self, i):
        return lambda: self.piece(i)

    def take(self):
        buf, self.buf = self.buf, None
        return buf


def _cast_many(items, device):
    """items: (src, dst, op, aux) tensors (contiguous, same number of elements each pair) -> one launch."""
    p = _lib.CastParams()
    assert len(items) <= _lib.CAST_MAX
    p.count = len(items)
    for k, (src, dst, op, aux) in enumerate(items):
        it = p.item[k]
        it.src, it.dst, it.n = src.data_ptr(), dst.data_ptr(), src.numel()
        it.src_dtype, it.dst_dtype, it.op = _DT[src.dtype], _DT[dst.dtype], op
        it.aux = aux.data_ptr() if aux is not None else None
    lib = _lib.load()
    with torch.cuda.device(device):
        p.stream = torch.cuda.current_stream().cuda_stream
        rc = lib.bimamba2_cast_many(ctypes.byref(p))
    if rc != 0:
        raise RuntimeError(f"bimamba2_cast_many: {lib.bimamba2_strerror(rc).decode()} (code {rc})")


class _ParamsAsFloat32(torch.autograd.Function):
    """(A_log, D, dt_bias, conv weight, conv bias or None, norm weight) -> (A = -exp(A_log), and the others) as float32, in
    one launch, and their gradients back into the parameters' types in one launch.  The kernels of the layer compute with
    float32 parameters; when the module holds them in a 16-bit type (model.to(torch.bfloat16)) each of these maps is
    otherwise a torch op of its own, forward and backward: about twenty launches of 4 us per step."""

    @staticmethod
    def forward(ctx, *params):
        live = [t for t in params if t is not None]
        buf = torch.empty(sum(t.numel() for t in live), dtype=torch.float32, device=live[0].device)
        outs, items, at = [], [], 0
        for i, t in enumerate(params):
            if t is None:
                outs.append(None)
                continue
            o = buf[at:at + t.numel()].view(t.shape)
            at += t.numel()
            items.append((t.detach().contiguous(), o, _lib.CAST_NEG_EXP if i == 0 else _lib.CAST_COPY, None))
            outs.append(o)
        _cast_many(items, buf.device)
        ctx.meta = [(t.dtype, t.shape) if t is not None else None for t in params]
        ctx.save_for_backward(outs[0])
        ctx.mark_non_differentiable(*[o for o, need in zip(outs, ctx.needs_input_grad) if o is not None and not need])
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        (A,) = ctx.saved_tensors
        res, items = [], []
        for i, (g, meta) in enumerate(zip(grads, ctx.meta)):
            if g is None or meta is None or not ctx.needs_input_grad[i]:
                res.append(None)
                continue
            dtype, shape = meta
            g = g.float().contiguous()
            o = torch.empty(shape, dtype=dtype, device=g.device)
            items.append((g, o, _lib.CAST_MUL if i == 0 else _lib.CAST_COPY, A if i == 0 else None))   # dA_log = dA * A
            res.append(o)
        if items:
            _cast_many(items, A.device)
        return tuple(res)


class _SplitInto(torch.autograd.Function):
    """torch.split(t, sizes, dim=-1) whose backward fills a _GradPieces buffer: a gradient that already is the buffer's
    slice stays where it is, any other one is copied in (a missing one counts as zero)."""

    @staticmethod
    def forward(ctx, t, pieces):
        ctx.pieces = pieces
        b = pieces.bounds
        return tuple(t[..., b[i]:b[i + 1]] for i in range(len(b) - 1))

    @staticmethod
    def backward(ctx, *grads):
        pieces = ctx.pieces
        copied = []
        for i, g in enumerate(grads):
            dst = pieces.piece(i)
            if g is None:
                dst.zero_()
            elif not (g.data_ptr() == dst.data_ptr() and g.shape == dst.shape and g.stride() == dst.stride() and g.dtype == dst.dtype):
                dst.copy_(g)
                copied.append(i)
        if _GradPieces.on_copied is not None:
            _GradPieces.on_copied(tuple(copied))
        return pieces.take(), None


class BiMamba2(nn.Module):
    """Bidirectional Mamba-2 mixer layer; ``forward(u)`` maps (batch, seqlen, d_model) to the same shape."""

    def __init__(self, d_model, d_state=64, d_conv=7, conv_init=None, expand=2, headdim=64, ngroups=1,
                 dt_min=0.001, dt_max=0.1, dt_init_floor=1e-4, dt_limit=(0.0, float("inf")),
                 learnable_init_states=False, activation="swish", bias=False, conv_bias=True, chunk_size=256,
                 use_mem_eff_path=False, layer_idx=None, device=None, dtype=None):
        super().__init__()
        fk = {"device": device, "dtype": dtype}
        assert not use_mem_eff_path, "Mem Eff Path is not implemented yet."
        assert activation in ("silu", "swish")
        self.d_model, self.d_state, self.d_conv, self.conv_init = d_model, d_state, d_conv, conv_init
        self.expand, self.headdim, self.ngroups = expand, headdim, ngroups
        self.d_inner = expand * d_model
        assert self.d_inner % headdim == 0
        self.nheads = self.d_inner // headdim
        self.dt_limit = dt_limit
        self.learnable_init_states = learnable_init_states
        self.activation = activation
        self.chunk_size = chunk_size
        self.use_mem_eff_path = use_mem_eff_path
        self.layer_idx = layer_idx

        bc = 2 * ngroups * d_state
        # in_proj output order: [z, x, B, C, dt]
        self.in_proj = nn.Linear(d_model, 2 * self.d_inner + bc + self.nheads, bias=bias, **fk)
        conv_dim = self.d_inner + bc
        self.conv1d = nn.Conv1d(conv_dim, conv_dim, kernel_size=d_conv, groups=conv_dim, padding=d_conv // 2,
                                bias=conv_bias, **fk)
        if conv_init is not None:
            nn.init.uniform_(self.conv1d.weight, -conv_init, conv_init)
        if learnable_init_states:   # kept for state_dict compatibility; the bidirectional path has no initial state
            self.init_states = nn.Parameter(torch.zeros(self.nheads, headdim, d_state, **fk))
            self.init_states._no_weight_decay = True
        self.act = nn.SiLU()

        # dt_bias = softplus^-1 of a log-uniform sample in [dt_min, dt_max]
        dt0 = torch.exp(torch.rand(self.nheads, **fk) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min))
        dt0 = torch.clamp(dt0, min=dt_init_floor)
        self.dt_bias = nn.Parameter(dt0 + torch.log(-torch.expm1(-dt0)))
        self.dt_bias._no_weight_decay = True

        self.A_log = nn.Parameter(torch.log(torch.ones(self.nheads, dtype=torch.float32, device=device)).to(dtype=dtype))
        self.A_log._no_weight_decay = True
        self.D = nn.Parameter(torch.ones(self.nheads, device=device))
        self.D._no_weight_decay = True
        self.fc_D = nn.Linear(self.d_inner, self.nheads, bias=False, **fk)   # present in the reference, unused there too
        self.norm = RMSNormGated(self.d_inner, eps=1e-5, norm_before_gate=True, **fk)
        self.out_proj = nn.Linear(self.d_inner, d_model, bias=bias, **fk)

    def forward(self, u):
        bc = self.ngroups * self.d_state
        zxbcdt = self.in_proj(u)
        prm = (self.A_log, self.D, self.dt_bias, self.conv1d.weight, self.conv1d.bias, self.norm.weight)
        if u.is_cuda and any(t is not None and t.dtype != torch.float32 for t in prm) and all(t is None or t.dtype in _DT for t in prm):
            # 16-bit parameters: all maps to float32 (and A = -exp(A_log)) in one launch, their gradients likewise
            A, D, dt_bias, conv_w, conv_b, norm_w = _ParamsAsFloat32.apply(*prm)
        else:
            A = -torch.exp(self.A_log.float())
            D, dt_bias, conv_w, conv_b, norm_w = prm[1:]
        sizes = [self.d_inner, self.d_inner + 2 * bc, self.nheads]
        if torch.is_grad_enabled() and zxbcdt.requires_grad:
            # the gradients of z (from the norm) and of xBC (from the convolution) are written straight into their places
            # in the gradient of the projection output
            grads = _GradPieces(zxbcdt, sizes)
            z, xBC, dt = _SplitInto.apply(zxbcdt, grads)
            dz_place, dxbc_place = grads.place(0), grads.place(1)
        else:
            z, xBC, dt = torch.split(zxbcdt, sizes, dim=-1)
            dz_place = dxbc_place = None
        # conv1d + SiLU on the channels-last view, one HIP kernel (the reference transposes, calls nn.Conv1d, transposes
        # back and applies the activation, modules.py:162-164 there); self.conv1d only holds the parameters
        xBC = conv1d_silu_fn(xBC, conv_w, conv_b, dx_place=dxbc_place)
        kw = {} if tuple(self.dt_limit) == (0.0, float("inf")) else {"dt_limit": tuple(self.dt_limit)}
        if torch.is_grad_enabled() and xBC.requires_grad and self.headdim <= 128 and self.d_state <= 256:
            # likewise the operator's dx, dB, dC: slices of the gradient of the convolution's output
            g2 = _GradPieces(xBC, [self.d_inner, bc, bc])
            x, B, C = _SplitInto.apply(xBC, g2)
            kw["grad_places"] = {"dx": lambda: g2.piece(0).unflatten(-1, (self.nheads, self.headdim)),
                                 "dB": lambda: g2.piece(1).unflatten(-1, (self.ngroups, self.d_state)),
                                 "dC": lambda: g2.piece(2).unflatten(-1, (self.ngroups, self.d_state))}
        else:
            x, B, C = torch.split(xBC, [self.d_inner, bc, bc], dim=-1)
        # softplus(dt + dt_bias) (modules.py:158 there) happens inside the operator's first kernel
        y = bimamba_chunk_scan_combined(
            x.unflatten(-1, (self.nheads, self.headdim)), dt, A,
            B.unflatten(-1, (self.ngroups, self.d_state)), C.unflatten(-1, (self.ngroups, self.d_state)),
            chunk_size=self.chunk_size, D=D, z=None, dt_bias=dt_bias, dt_softplus=True, **kw)
        # (self.norm's forward, with the weight as prepared above)
        y = rmsnorm_fn(y.flatten(-2), norm_w, None, z=z, eps=self.norm.eps, group_size=self.norm.group_size,
                       norm_before_gate=self.norm.norm_before_gate, dz_place=dz_place)
        return self.out_proj(y)

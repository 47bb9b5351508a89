"""Host side of the bidirectional SSD operator: the functions of the reference's ``ssd.bi.ssd_combined`` and of its
stage wrappers, with the same names, argument meaning and error behaviour, on top of the C ABI of
libbimamba2_hip.so (include/bimamba2.h).  PyTorch is used for device memory and streams only; every device
computation is a hand-written HIP kernel.  There is no CPU path: tensors must live on a GPU.

Reference interface mirrored here (paths relative to the reference's root):
  bimamba_chunk_scan_combined / MambaChunkScanCombinedFn      src/ssd/bi/ssd_combined.py:555-593
  _mamba_chunk_scan_combined_fwd / _bwd                       src/ssd/bi/ssd_combined.py:297-475
  _chunk_cumsum_fwd, _chunk_state_fwd, _chunk_state_bwd_db,
  _chunk_cumsum_bwd                                           src/ssd/bi/ssd_chunk_state.py:699-894
  _state_passing_fwd / _bwd                                   src/ssd/bi/ssd_state_passing.py:190-248
  _bmm_chunk_fwd / _bwd                                       src/ssd/bi/ssd_bmm.py:163-262
  _chunk_scan_fwd, _chunk_scan_bwd_dz/_dstates/_dC/_dcb       src/ssd/bi/ssd_chunk_scan.py:1638-1909
"""
import math

import torch

from . import _lib
from ._lib import Params

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}
_INF = float("inf")
MAX_CHUNK_SIZE, MAX_HEADDIM = 256, 128     # BIMAMBA2_MAX_CHUNK, BIMAMBA2_MAX_HEADDIM of include/bimamba2.h
MAX_DSTATE = 256                           # BIMAMBA2_MAX_DSTATE


def _require_gpu(t, name):
    if not t.is_cuda:
        raise RuntimeError(f"{name} is on {t.device}: the bidirectional SSD kernels run on an AMD GPU only "
                           "(there is no CPU fallback)")


def _rowmajor_last(t):
    """Last dim must be contiguous for the kernels; anything else is copied."""
    return t if t.stride(-1) == 1 else t.contiguous()


def _f32c(t):
    return t.detach().to(torch.float32).contiguous()


_WS_CACHE = {}


class _Call:
    """Collects tensors into a ``bimamba2_params`` and keeps them alive until the launch has been enqueued."""

    def __init__(self, batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, dtype, device,
                 dt_dtype=torch.float32, dt_softplus=False, dt_limit=(0.0, _INF)):
        if dtype not in _DT:
            raise ValueError(f"unsupported dtype {dtype} (need float32, bfloat16 or float16)")
        if dt_dtype not in _DT:
            raise ValueError(f"unsupported dt dtype {dt_dtype}")
        p = Params()
        p.batch, p.seqlen, p.nheads, p.headdim = batch, seqlen, nheads, headdim
        p.ngroups, p.dstate, p.chunk_size = ngroups, dstate, chunk_size
        p.dtype, p.dt_dtype = _DT[dtype], _DT[dt_dtype]
        p.dt_softplus = int(bool(dt_softplus))
        p.dt_min, p.dt_max = float(dt_limit[0]), float(dt_limit[1])
        self.p, self.keep, self.device, self.dtype, self.dt_dtype = p, [], device, dtype, dt_dtype
        self.params = []       # float32 copies of A, D, dt_bias that the parameter block points at
        self.nchunks = (seqlen + chunk_size - 1) // chunk_size

    # ---- raw pointer fields -------------------------------------------------------------------------
    def put(self, field, t, dtype=None):
        if t is None:
            return None
        _require_gpu(t, field)
        if dtype is not None and t.dtype != dtype:
            raise TypeError(f"{field} must be {dtype}, got {t.dtype}")
        if not t.is_contiguous():
            raise ValueError(f"{field} must be contiguous")
        self.keep.append(t)
        setattr(self.p, field, t.data_ptr())
        return t

    def new(self, field, shape, dtype=torch.float32):
        t = torch.empty(shape, device=self.device, dtype=dtype)
        return self.put(field, t)

    def put_grad(self, field, t, shape, dtype):
        """dx, dB or dC given by the caller: (batch, seqlen, heads or groups, width) with the two inner dimensions
        contiguous; batch and position strides are passed on (a slice of a wider buffer)."""
        _require_gpu(t, field)
        if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
            raise ValueError(f"{field}: expected {tuple(shape)} {dtype}, got {tuple(t.shape)} {t.dtype}")
        if t.stride(3) != 1 or t.stride(2) != shape[3]:
            raise ValueError(f"{field}: the two inner dimensions must be contiguous")
        self.keep.append(t)
        setattr(self.p, field, t.data_ptr())
        contiguous = t.is_contiguous()
        setattr(self.p, field + "_sb", 0 if contiguous else t.stride(0))
        setattr(self.p, field + "_sl", 0 if contiguous else t.stride(1))
        return t

    # ---- strided inputs -----------------------------------------------------------------------------
    def _strided(self, field, prefix, t, dtype):
        _require_gpu(t, field)
        if t.dtype != dtype:
            t = t.to(dtype)
        t = _rowmajor_last(t)
        self.keep.append(t)
        setattr(self.p, field, t.data_ptr())
        for name, s in zip(prefix, t.stride()[:3]):
            setattr(self.p, name, s)
        return t

    def set_x(self, x):
        return self._strided("x", ("x_sb", "x_sl", "x_sh"), x, self.dtype)

    def set_z(self, z):
        if z is None:
            return None
        self.p.has_z = 1
        return self._strided("z", ("z_sb", "z_sl", "z_sh"), z, self.dtype)

    def set_dout(self, dout):
        return self._strided("dout", ("dout_sb", "dout_sl", "dout_sh"), dout, self.dtype)

    def set_B(self, B):
        return self._strided("Bm", ("B_sb", "B_sl", "B_sg"), B, self.dtype)

    def set_C(self, C):
        return self._strided("Cm", ("C_sb", "C_sl", "C_sg"), C, self.dtype)

    def set_dt(self, dt):
        _require_gpu(dt, "dt")
        self.keep.append(dt)
        self.p.dt = dt.data_ptr()
        self.p.dt_sb, self.p.dt_sl, self.p.dt_sh = dt.stride()
        return dt

    def _param(self, field, t):
        t = self.put(field, _f32c(t))
        self.params.append(t)
        return t

    def set_A(self, A):
        return self._param("A", A)

    def set_D(self, D):
        if D is None:
            return None
        self.p.has_D = 1
        self.p.D_has_hdim = int(D.dim() == 2)
        return self._param("D", D)

    def set_dt_bias(self, dt_bias):
        if dt_bias is None:
            return None
        self.p.has_dt_bias = 1
        return self._param("dt_bias", dt_bias)

    def _workspace_bytes(self, is_bwd):
        return int(_lib.load().bimamba2_workspace_bytes(self.p, int(is_bwd)))

    def workspace(self, is_bwd):
        p = self.p
        # the size depends on the problem and on which intermediates the caller brought; ask the library once per such key
        # (which kernels run, and with them what is carved, also depends on strides and on 16-byte alignment)
        al = lambda v: (v or 0) & 15
        key = (is_bwd, p.batch, p.seqlen, p.nheads, p.headdim, p.ngroups, p.dstate, p.chunk_size, p.dtype, p.has_z, p.causal,
               bool(p.dt_out), bool(p.cs_f), bool(p.states_f), bool(p.states_b), bool(p.CB), bool(p.CBT), bool(p.dCB), bool(p.dCBT),
               bool(p.dstates_f), bool(p.dout_x), bool(p.red), bool(p.dBs), bool(p.da_intra),
               p.x_sb, p.x_sl, p.x_sh, p.z_sb, p.z_sl, p.z_sh, p.dout_sb, p.dout_sl, p.dout_sh, p.B_sb, p.B_sl, p.B_sg,
               p.C_sb, p.C_sl, p.C_sg, al(p.x), al(p.z), al(p.dout), al(p.Bm), al(p.Cm), al(p.out), al(p.out_x), al(p.dx),
               al(p.states_f), al(p.states_b), al(p.dstates_f), al(p.dstates_b),
               bool(p.states16_f), bool(p.dstates16_f), p.fwd_saved, al(p.states16_f), al(p.states16_b), al(p.final_f), al(p.final_b),
               al(p.initial_f), al(p.initial_b), al(p.dfinal_f), al(p.dfinal_b), al(p.dinitial_f), al(p.dinitial_b))
        n = _WS_CACHE.get(key)
        if n is None:
            n = _WS_CACHE[key] = self._workspace_bytes(is_bwd)
        ws = torch.empty(max(int(n), 1), device=self.device, dtype=torch.uint8)
        self.keep.append(ws)
        self.p.workspace = ws.data_ptr()
        self.p.workspace_bytes = ws.numel()

    def run(self, entry):
        if torch.cuda.current_device() == self.device.index:
            self.p.stream = torch.cuda.current_stream().cuda_stream
            _lib.call(entry, self.p)
            return
        with torch.cuda.device(self.device):
            self.p.stream = torch.cuda.current_stream().cuda_stream
            _lib.call(entry, self.p)

    # ---- reuse of the input half of a call (the autograd function builds it once for forward and backward) ----
    def snapshot(self):
        """The parameter block as bytes plus the converted tensors it points at (the float32 copies of A, D, dt_bias,
        whatever their size): a call rebuilt from the snapshot uses their pointers again."""
        return bytes(self.p), list(self.params)

    @classmethod
    def from_snapshot(cls, snap, x, nchunks):
        self = cls.__new__(cls)
        self.p = Params.from_buffer_copy(snap[0])
        self.keep = list(snap[1])
        self.params = list(snap[1])
        self.device, self.dtype, self.dt_dtype = x.device, x.dtype, None
        self.nchunks = nchunks
        return self


def _check_chunk(chunk_size):
    assert chunk_size >= 32, "chunk_size must be at least 32 (as in the reference) and at most 256"


def _slices(nheads, ngroups):
    """Number of head slices whose partial dB / dC sums the kernels keep apart (8 heads per slice)."""
    return (nheads // ngroups + 7) // 8


def _bhcq(c):
    return (c.p.batch, c.p.nheads, c.nchunks, c.p.chunk_size)


# =============================================================================================================
# stage wrappers
# =============================================================================================================
def _chunk_cumsum_fwd(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, _INF)):
    """-> dA_cumsum_f, dA_cumsum_b, dt_out, each (batch, nheads, nchunks, chunk_size) float32."""
    batch, seqlen, nheads = dt.shape
    assert A.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    c = _Call(batch, seqlen, nheads, 1, 1, 1, chunk_size, torch.float32, dt.device, dt.dtype, dt_softplus, dt_limit)
    c.set_dt(dt); c.set_A(A); c.set_dt_bias(dt_bias)
    dt_out = c.new("dt_out", _bhcq(c)); cs_f = c.new("cs_f", _bhcq(c)); cs_b = c.new("cs_b", _bhcq(c))
    c.run("bimamba2_chunk_cumsum_fwd")
    return cs_f, cs_b, dt_out


def _bmm_chunk_fwd(C, B, chunk_size, output_dtype=torch.float32, with_transpose=False):
    """CB (batch, nchunks, ngroups, chunk_size, chunk_size); kept in float32 (the reference's choice too).
    with_transpose=True also returns CBT = CB.transpose(-1, -2) as a second contiguous tensor (the dx kernel
    reads CB by columns)."""
    batch, seqlen, ngroups, dstate = B.shape
    assert C.shape == B.shape
    c = _Call(batch, seqlen, ngroups, 1, ngroups, dstate, chunk_size, C.dtype, C.device)
    c.set_B(B); c.set_C(C)
    CB = c.new("CB", (batch, c.nchunks, ngroups, chunk_size, chunk_size))
    CBT = c.new("CBT", CB.shape) if with_transpose else None
    c.run("bimamba2_bmm_chunk_fwd")
    if with_transpose:
        return CB, CBT
    return CB if output_dtype in (None, torch.float32) else CB.to(output_dtype)


def _chunk_state_fwd(B, x, dt, dA_cumsum_f, dA_cumsum_b, states_in_fp32=True):
    """-> states_f, states_b (batch, nchunks, nheads, headdim, dstate) float32."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert dA_cumsum_f.shape == dt.shape and dA_cumsum_b.shape == dt.shape
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, x.dtype, x.device)
    c.set_x(x); c.set_B(B)
    c.put("dt_out", dt, torch.float32); c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    shape = (batch, nchunks, nheads, headdim, dstate)
    sf = c.new("states_f", shape); sb = c.new("states_b", shape)
    c.run("bimamba2_chunk_state_fwd")
    return sf, sb


def _state_passing_fwd(states_f, states_b, dA_cumsum_f, dA_cumsum_b, return_final_states=True):
    """Both inter-chunk recurrences in one launch.  states_* are (batch, nchunks, nheads, headdim, dstate) float32
    chunk states; returns the states entering each chunk (new tensors) and the two final states."""
    batch, nchunks, nheads, headdim, dstate = states_f.shape
    chunk_size = dA_cumsum_f.shape[-1]
    assert states_b.shape == states_f.shape
    assert dA_cumsum_f.shape == (batch, nheads, nchunks, chunk_size) and dA_cumsum_b.shape == dA_cumsum_f.shape
    c = _Call(batch, nchunks * chunk_size, nheads, headdim, 1, dstate, chunk_size, torch.float32, states_f.device)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    pf = c.put("states_f", states_f.clone(), torch.float32); pb = c.put("states_b", states_b.clone(), torch.float32)
    ff = fb = None
    if return_final_states:
        ff = c.new("final_f", (batch, nheads, headdim, dstate)); fb = c.new("final_b", (batch, nheads, headdim, dstate))
    c.run("bimamba2_state_passing_fwd")
    return pf, pb, ff, fb


def _chunk_scan_fwd(CB, x, dt, dA_cumsum_f, dA_cumsum_b, C, states_f, states_b, D=None, z=None, B=None):
    """-> out, out_x (out_x is None without z).  CB may be None when B is given and the problem is one whose scan
    kernel rebuilds CB from C and B (bimamba2_chunk_scan_reads_cb == 0); anything else raises ValueError."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = C.shape
    assert nheads % ngroups == 0
    assert C.shape == (batch, seqlen, ngroups, dstate)
    assert CB is None or CB.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    assert CB is not None or B is not None, "without CB the kernel needs B to rebuild it"
    if z is not None:
        assert z.shape == x.shape
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    assert dt.shape == (batch, nheads, nchunks, chunk_size)
    assert states_f.shape == (batch, nchunks, nheads, headdim, dstate) and states_b.shape == states_f.shape
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, x.dtype, x.device)
    c.set_x(x); c.set_C(C); c.set_z(z); c.set_D(D)
    if CB is None:
        c.set_B(B)
    c.put("CB", CB, torch.float32); c.put("dt_out", dt, torch.float32)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    c.put("states_f", states_f, torch.float32); c.put("states_b", states_b, torch.float32)
    out = c.new("out", x.shape, x.dtype)
    out_x = c.new("out_x", x.shape, x.dtype) if z is not None else None
    c.run("bimamba2_chunk_scan_fwd")
    return out, out_x


def _chunk_scan_bwd_dz(x, z, out_x, dout, chunk_size=None, D=None):
    """-> dz, dout_x = dout * silu(z)."""
    batch, seqlen, nheads, headdim = x.shape
    assert z.shape == x.shape and out_x.shape == x.shape and dout.shape == x.shape
    c = _Call(batch, seqlen, nheads, headdim, 1, 1, chunk_size or 64, x.dtype, x.device)
    c.set_z(z); c.set_dout(dout)
    c.put("out_x", out_x.contiguous(), x.dtype)
    dz = c.new("dz", x.shape, x.dtype); dout_x = c.new("dout_x", x.shape, x.dtype)
    c.run("bimamba2_chunk_scan_bwd_dz")
    return dz, dout_x


def _chunk_scan_bwd_dstates(C, dA_cumsum_f, dA_cumsum_b, dout, headdim=None):
    """-> gradient w.r.t. the states entering each chunk, both directions, float32."""
    batch, seqlen, nheads, hd = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum_f.shape
    _, _, ngroups, dstate = C.shape
    c = _Call(batch, seqlen, nheads, hd, ngroups, dstate, chunk_size, dout.dtype, dout.device)
    c.set_dout(dout); c.set_C(C)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    shape = (batch, nchunks, nheads, hd, dstate)
    df = c.new("dstates_f", shape); db = c.new("dstates_b", shape)
    c.run("bimamba2_chunk_scan_bwd_dstates")
    return df, db


def _chunk_scan_bwd_dz_dstates(z, out_x, dout, C, dA_cumsum_f, dA_cumsum_b):
    """_chunk_scan_bwd_dz and _chunk_scan_bwd_dstates as one launch -> dz, dout_x, dstates_f, dstates_b.  Raises for
    problems that only the two separate kernels cover (see include/bimamba2.h)."""
    batch, seqlen, nheads, hd = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum_f.shape
    _, _, ngroups, dstate = C.shape
    assert z.shape == dout.shape and out_x.shape == dout.shape
    c = _Call(batch, seqlen, nheads, hd, ngroups, dstate, chunk_size, dout.dtype, dout.device)
    c.set_z(z); c.set_dout(dout); c.set_C(C)
    c.put("out_x", out_x.contiguous(), dout.dtype)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    dz = c.new("dz", dout.shape, dout.dtype); dout_x = c.new("dout_x", dout.shape, dout.dtype)
    shape = (batch, nchunks, nheads, hd, dstate)
    df = c.new("dstates_f", shape); db = c.new("dstates_b", shape)
    c.run("bimamba2_chunk_scan_bwd_dz_dstates")
    return dz, dout_x, df, db


def _state_passing_bwd(states_f, states_b, dA_cumsum_f, dA_cumsum_b, dstates_f, dstates_b):
    """states_*: states entering each chunk; dstates_*: gradient w.r.t. them.
    -> gradient w.r.t. each chunk's own state (both directions) and ddA_chunk_f/b (batch, nheads, nchunks)."""
    batch, nchunks, nheads, headdim, dstate = states_f.shape
    chunk_size = dA_cumsum_f.shape[-1]
    c = _Call(batch, nchunks * chunk_size, nheads, headdim, 1, dstate, chunk_size, torch.float32, states_f.device)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    c.put("states_f", states_f, torch.float32); c.put("states_b", states_b, torch.float32)
    gf = c.put("dstates_f", dstates_f.clone(), torch.float32); gb = c.put("dstates_b", dstates_b.clone(), torch.float32)
    nsplit = (headdim * dstate + 1023) // 1024
    af = c.new("ddA_chunk_f", (batch, nheads, nchunks, nsplit)); ab = c.new("ddA_chunk_b", (batch, nheads, nchunks, nsplit))
    c.run("bimamba2_state_passing_bwd")
    return gf, gb, af.sum(-1), ab.sum(-1)


def _chunk_scan_chunk_state_bwd_dx(x, dt, dA_cumsum_f, dA_cumsum_b, B, CB, dout, dstates_f, dstates_b, D=None, dx=None,
                                   C=None):
    """-> dx, ddt_direct (batch, nheads, nchunks, chunk_size) float32, dD.  CB may be None when C is given and the
    kernel rebuilds it (see _chunk_scan_fwd)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert CB is None or CB.shape == (batch, nchunks, ngroups, chunk_size, chunk_size)
    assert CB is not None or C is not None, "without CB the kernel needs C to rebuild it"
    assert dout.shape == x.shape
    assert dstates_f.shape == (batch, nchunks, nheads, headdim, dstate) and dstates_b.shape == dstates_f.shape
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, x.dtype, x.device)
    c.set_x(x); c.set_B(B); c.set_dout(dout); c.set_D(D)
    if CB is None:
        c.set_C(C)
    else:
        c.put("CBT", CB.transpose(-1, -2).contiguous(), torch.float32)
    c.put("dt_out", dt, torch.float32)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    c.put("dstates_f", dstates_f, torch.float32); c.put("dstates_b", dstates_b, torch.float32)
    dx = c.put("dx", dx) if dx is not None else c.new("dx", x.shape, x.dtype)
    # one plane per headdim column tile of the kernel, added up here in a fixed order
    planes = int(_lib.load().bimamba2_ddt_direct_planes(c.p))
    ddt = c.new("ddt_direct", (planes,) + _bhcq(c))
    dD = None
    if D is not None:
        dD = c.new("dD", tuple(D.shape))
        c.new("red", (batch * nchunks * nheads * headdim,))
    c.run("bimamba2_chunk_scan_bwd_dx")
    ddt = ddt[0] if planes == 1 else ddt.sum(0)
    return dx, ddt, (dD.to(D.dtype) if dD is not None else None)


def _chunk_state_bwd_db(x, dt, dA_cumsum_f, dA_cumsum_b, dstates_f, dstates_b, B=None, ngroups=1):
    """-> dB state part (batch, seqlen, ngroups, dstate) float32, v_f, v_b (batch, nheads, nchunks, chunk_size):
    per-position terms whose exclusive prefix (v_f) / suffix (v_b) sums are the reference's ddA_next_f/b."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    dstate = dstates_f.shape[-1]
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, x.dtype, x.device)
    c.set_x(x); c.set_B(B)
    c.put("dt_out", dt, torch.float32); c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    c.put("dstates_f", dstates_f, torch.float32); c.put("dstates_b", dstates_b, torch.float32)
    dBs = torch.zeros(_slices(nheads, ngroups), batch, seqlen, ngroups, dstate, device=x.device, dtype=torch.float32)
    c.put("dBs", dBs)
    vf = c.new("v_f", _bhcq(c)); vb = c.new("v_b", _bhcq(c))
    c.run("bimamba2_chunk_state_bwd_db")
    return dBs, vf, vb


def _chunk_scan_bwd_dC(states_f, states_b, dA_cumsum_f, dA_cumsum_b, dout, C=None, ngroups=1):
    """-> dC state part float32, u_f, u_b: per-position terms whose inclusive suffix (u_f) / prefix (u_b) sums
    are the reference's ddA_prev_f/b."""
    batch, seqlen, nheads, headdim = dout.shape
    _, _, nchunks, chunk_size = dA_cumsum_f.shape
    dstate = states_f.shape[-1]
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, dout.dtype, dout.device)
    c.set_dout(dout); c.set_C(C)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    c.put("states_f", states_f, torch.float32); c.put("states_b", states_b, torch.float32)
    dCs = torch.zeros(_slices(nheads, ngroups), batch, seqlen, ngroups, dstate, device=dout.device, dtype=torch.float32)
    c.put("dCs", dCs)
    uf = c.new("u_f", _bhcq(c)); ub = c.new("u_b", _bhcq(c))
    c.run("bimamba2_chunk_scan_bwd_dc")
    return dCs, uf, ub


def _chunk_scan_bwd_dcb(x, dt, dA_cumsum_f, dA_cumsum_b, dout, CB, ngroups=1, B=None, C=None):
    """-> dCB (batch, nchunks, ngroups, Q, Q) float32 and the per-tile vectors (batch, nheads, nchunks, tiles, 2, 64)
    from which chunk_cumsum_bwd assembles the within-chunk part of d(dt*A) (the reference's ddA_f + ddA_b of
    its two "stable" kernels): column / row sums of off-diagonal 64x64 tiles, full contribution of diagonal ones.
    CB may be None when B and C are given and the kernel rebuilds its CB tiles (see _chunk_scan_fwd)."""
    batch, seqlen, nheads, headdim = x.shape
    _, _, nchunks, chunk_size = dt.shape
    assert CB is not None or (B is not None and C is not None), "without CB the kernel needs B and C to rebuild it"
    c = _Call(batch, seqlen, nheads, headdim, ngroups, 1 if CB is not None else B.shape[-1], chunk_size, x.dtype, x.device)
    c.set_x(x); c.set_dout(dout)
    if CB is None:
        c.set_B(B); c.set_C(C)
    c.put("CB", CB, torch.float32); c.put("dt_out", dt, torch.float32)
    c.put("cs_f", dA_cumsum_f, torch.float32); c.put("cs_b", dA_cumsum_b, torch.float32)
    nsl = max(1, min(4, nheads // ngroups // 32))      # head slices, added up in place by the kernel launcher
    dCB = c.new("dCB", (nsl, batch, nchunks, ngroups, chunk_size, chunk_size))[0]
    c.new("dCBT", (nsl, batch, nchunks, ngroups, chunk_size, chunk_size))
    nqt = (chunk_size + 63) // 64
    da = c.new("da_intra", (batch, nheads, nchunks, nqt * nqt, 2, 64))
    c.run("bimamba2_chunk_scan_bwd_dcb")
    return dCB, da


def _bmm_chunk_bwd(B, C, dCB, dBs, dCs):
    """dB = sum(dBs) + dCB^T.C and dC = sum(dCs) + dCB.B per chunk, in the dtype of B / C; dBs, dCs are the
    (slices, batch, seqlen, ngroups, dstate) partial sums of _chunk_state_bwd_db / _chunk_scan_bwd_dC."""
    batch, seqlen, ngroups, dstate = B.shape
    chunk_size = dCB.shape[-1]
    # nheads is only used to tell the kernel how many slices to add up: _slices(nheads, ngroups) must give them back
    assert dCs.shape[0] == dBs.shape[0]
    nheads = ngroups * 8 * dBs.shape[0]
    assert _slices(nheads, ngroups) == dBs.shape[0]
    c = _Call(batch, seqlen, nheads, 1, ngroups, dstate, chunk_size, B.dtype, B.device)
    c.set_B(B); c.set_C(C)
    c.put("dCB", dCB, torch.float32); c.put("dCBT", dCB.transpose(-1, -2).contiguous(), torch.float32)
    c.put("dBs", dBs, torch.float32); c.put("dCs", dCs, torch.float32)
    dB = torch.zeros(B.shape, device=B.device, dtype=B.dtype); c.put("dB", dB)
    dC = torch.zeros(B.shape, device=B.device, dtype=B.dtype); c.put("dC", dC)
    c.run("bimamba2_bmm_chunk_bwd")
    return dB, dC


def _chunk_cumsum_bwd(da_intra, u_f, u_b, v_f, v_b, ddA_chunk_f, ddA_chunk_b, ddt_direct, dt, A, dt_bias=None,
                      dt_softplus=False, dt_limit=(0.0, _INF)):
    """Assembles d(dt * A) from its pieces and takes it through the dt transform: the reference's host-side scans
    (src/ssd/bi/ssd_combined.py:456-466) and its _chunk_cumsum_bwd (src/ssd/bi/ssd_chunk_state.py:727-761) in one kernel.
    da_intra: per-tile vectors of _chunk_scan_bwd_dcb; u_*: of _chunk_scan_bwd_dC; v_*: of _chunk_state_bwd_db;
    ddA_chunk_*: (batch, nheads, nchunks) of _state_passing_bwd; ddt_direct: of _chunk_scan_chunk_state_bwd_dx; dt: the raw
    (batch, seqlen, nheads) input.  -> ddt (like dt), dA (nheads,), ddt_bias (nheads,) or None."""
    batch, seqlen, nheads = dt.shape
    _, _, nchunks, chunk_size = ddt_direct.shape
    assert u_f.shape == ddt_direct.shape and v_f.shape == ddt_direct.shape
    assert ddA_chunk_f.shape == (batch, nheads, nchunks) and ddA_chunk_b.shape == ddA_chunk_f.shape
    # headdim = dstate = 1: one partial sum per chunk in ddA_chunk_*
    c = _Call(batch, seqlen, nheads, 1, 1, 1, chunk_size, torch.float32, dt.device, dt.dtype, dt_softplus, dt_limit)
    c.set_dt(dt); c.set_A(A); c.set_dt_bias(dt_bias)
    for field, t in (("da_intra", da_intra), ("u_f", u_f), ("u_b", u_b), ("v_f", v_f), ("v_b", v_b),
                     ("ddA_chunk_f", ddA_chunk_f.reshape(batch, nheads, nchunks, 1)),
                     ("ddA_chunk_b", ddA_chunk_b.reshape(batch, nheads, nchunks, 1)), ("ddt_direct", ddt_direct)):
        c.put(field, t.contiguous(), torch.float32)
    ddt = c.new("ddt", dt.shape, dt.dtype)
    dA = c.new("dA", (nheads,))
    ddt_bias = c.new("ddt_bias", (nheads,)) if dt_bias is not None else None
    c.new("red", (2 * batch * nchunks * nheads,))
    c.run("bimamba2_chunk_cumsum_bwd")
    return ddt, dA, ddt_bias


# =============================================================================================================
# combined forward / backward
# =============================================================================================================
def _problem(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit):
    batch, seqlen, nheads, headdim = x.shape
    _, _, ngroups, dstate = B.shape
    assert nheads % ngroups == 0
    assert B.shape == (batch, seqlen, ngroups, dstate)
    assert x.shape == (batch, seqlen, nheads, headdim)
    assert dt.shape == (batch, seqlen, nheads)
    assert A.shape == (nheads,)
    assert C.shape == B.shape
    _check_chunk(chunk_size)
    if z is not None:
        assert z.shape == x.shape
    if D is not None:
        assert D.shape == (nheads, headdim) or D.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    _require_gpu(x, "x")
    c = _Call(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size, x.dtype, x.device, dt.dtype,
              dt_softplus, dt_limit)
    c.set_x(x); c.set_dt(dt); c.set_A(A); c.set_B(B); c.set_C(C)
    c.set_D(D); c.set_z(z); c.set_dt_bias(dt_bias)
    return c


_BLOB_FIELDS = ("dt_out", "cs_f", "cs_b", "states_f", "states_b")


# the same with the entering states in the library's 16-bit copies (half the size) instead of float32
_BLOB_FIELDS_COPIES = ("dt_out", "cs_f", "cs_b", "states16_f", "states16_b")


def _point_into(c, blob, offs, fields=_BLOB_FIELDS):
    """Points the five forward intermediates at their places (float offsets) inside one float32 allocation."""
    base = blob.data_ptr()
    for field, o in zip(fields, offs):
        setattr(c.p, field, base + 4 * o)
    c.keep.append(blob)


# Sequence boundaries that one chunk may hold.  The kernels separate packed sequences by an offset of BIMAMBA2_SEQ_CUT (-20)
# per boundary in the chunk's cumulative decay sums (include/bimamba2.h), whose float32 resolution therefore falls with
# the number of boundaries inside ONE chunk: 1.2e-6 relative per boundary, i.e. 4e-5 at 32 - inside the float32 contract
# of 1e-4 - and beyond it from about 40.  The result does not depend on the chunk size, so a call whose seq_idx puts more
# boundaries than this into some chunk runs with a smaller chunk (a chunk of 32 positions cannot hold more than 32).
MAX_SEQ_BOUNDARIES_PER_CHUNK = 32


def seq_boundaries_per_chunk(seq_idx, chunk_size):
    """Largest number of sequence boundaries that fall into one chunk of `chunk_size` positions, as the kernels count
    them: a change of seq_idx between positions l - 1 and l offsets the forward sums of the chunk of l and the reverse
    sums of the chunk of l - 1."""
    change = seq_idx[:, 1:] != seq_idx[:, :-1]                      # (batch, L - 1): entry l - 1 is the boundary in front of l
    if change.numel() == 0:
        return 0
    batch, n = change.shape
    pos = torch.arange(1, n + 1, device=seq_idx.device)
    nch = (n + 1 + chunk_size - 1) // chunk_size
    ones = change.to(torch.int32)
    fwd = torch.zeros(batch, nch, dtype=torch.int32, device=seq_idx.device).scatter_add_(1, (pos // chunk_size).expand(batch, n), ones)
    rev = torch.zeros(batch, nch, dtype=torch.int32, device=seq_idx.device).scatter_add_(1, ((pos - 1) // chunk_size).expand(batch, n), ones)
    return int(torch.maximum(fwd.max(), rev.max()).item())


def chunk_size_for_seq_idx(seq_idx, chunk_size):
    """The chunk size a call with this seq_idx runs with: `chunk_size` if no chunk holds more than
    MAX_SEQ_BOUNDARIES_PER_CHUNK boundaries, else the largest of 128, 64, 32 below it for which that is true.  Costs one
    device-to-host synchronisation (the count is taken on the device)."""
    for q in [chunk_size] + [c for c in (128, 64, 32) if c < chunk_size]:
        if seq_boundaries_per_chunk(seq_idx, q) <= MAX_SEQ_BOUNDARIES_PER_CHUNK:
            return q
    # (not reached with chunk sizes down to 32; kept so that a change of the limit cannot make the mechanism fail silently)
    raise ValueError(f"seq_idx puts more than {MAX_SEQ_BOUNDARIES_PER_CHUNK} sequence boundaries into every chunk size down "
                     "to 32 positions: beyond the accuracy of the packed-sequence mechanism")


def _set_seq_idx(c, seq_idx, x):
    """seq_idx: (batch, seqlen) integer tensor, constant over each packed sequence; None = one sequence per row."""
    c.p.seq_idx = None
    if seq_idx is not None:
        assert tuple(seq_idx.shape) == tuple(x.shape[:2]), "seq_idx: expected (batch, seqlen)"
        c.put("seq_idx", seq_idx.detach().to(torch.int32).contiguous(), torch.int32)


def _set_states(c, fields, states, x, B):
    """Points the two (batch, nheads, headdim, dstate) float32 fields at the given tensors (None entries stay NULL)."""
    if states is None:
        return
    shape = (x.shape[0], x.shape[2], x.shape[3], B.shape[3])
    for field, t in zip(fields, states):
        if t is not None:
            assert tuple(t.shape) == shape, f"{field}: expected {shape}, got {tuple(t.shape)}"
            c.put(field, _f32c(t), torch.float32)


def _mamba_chunk_scan_combined_fwd(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                                   dt_limit=(0.0, _INF), return_intermediates=True, keep_for_bwd=False, causal=False,
                                   initial_states=None, seq_idx=None, want_out_x=True, want_final=True):
    """Returns (out, out_x, dt_out, dA_cumsum_f, dA_cumsum_b, states_f, states_b, final_states_f, final_states_b)
    like the reference; states_* are the states entering each chunk.  With return_intermediates=False only
    out, out_x and the final states are materialised as tensors (the rest lives in a workspace).
    keep_for_bwd=True appends a tenth element: the tuple (dt_out, cs_f, cs_b, states_f, states_b, snapshot) that
    _mamba_chunk_scan_combined_bwd accepts as `saved` to skip its recomputation (snapshot: the input half of the
    parameter block, reused when the backward pass gets the same tensors).
    causal=True runs the single-direction operator (see causal_chunk_scan_combined): no reverse states, final_states_b
    is None.  initial_states = (initial_f, initial_b), each (batch, nheads, headdim, dstate) or None: the state of the
    forward recurrence in front of the first position and of the reverse recurrence behind the last one."""
    c = _problem(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit)
    c.p.causal = 1 if causal else 0
    _set_states(c, ("initial_f", "initial_b"), initial_states, x, B)
    _set_seq_idx(c, seq_idx, x)
    batch, seqlen, nheads, headdim = x.shape
    ngroups, dstate = B.shape[2], B.shape[3]
    dt_out = cs_f = cs_b = sf = sb = None
    saved = snap = None
    if keep_for_bwd and not return_intermediates:
        # what the backward pass reuses, in one allocation (five tensors cost five times the allocator's and Python's
        # overhead); the snapshot below carries the pointers
        n1 = (batch * nheads * c.nchunks * chunk_size + 63) // 64 * 64
        n2 = (batch * c.nchunks * nheads * headdim * dstate + 63) // 64 * 64
        # where the kernels can, the states entering the chunks are kept in the input's 16-bit type only
        copies = bool(_lib.load().bimamba2_state_copies(c.p))
        fields = _BLOB_FIELDS_COPIES if copies else _BLOB_FIELDS
        ns = n2 // 2 if copies else n2
        blob = torch.empty(3 * n1 + 2 * ns, device=x.device, dtype=torch.float32)
        offs = (0, n1, 2 * n1, 3 * n1, 3 * n1 + ns)
        _point_into(c, blob, offs, fields)
        snap = c.snapshot() + (offs, fields)
        saved = ("blob", blob, snap)
    else:
        snap = c.snapshot() if keep_for_bwd else None
        if return_intermediates or keep_for_bwd:
            dt_out = c.new("dt_out", _bhcq(c)); cs_f = c.new("cs_f", _bhcq(c)); cs_b = c.new("cs_b", _bhcq(c))
            sshape = (batch, c.nchunks, nheads, headdim, dstate)
            sf = c.new("states_f", sshape); sb = c.new("states_b", sshape)
        if keep_for_bwd:
            saved = (dt_out, cs_f, cs_b, sf, sb, snap)
    out = c.new("out", x.shape, x.dtype)
    # the pre-gate output is what a backward pass needs; without one (want_out_x=False) the scan kernel skips that store
    out_x = c.new("out_x", x.shape, x.dtype) if (z is not None and want_out_x) else None
    ff = c.new("final_f", (batch, nheads, headdim, dstate)) if want_final else None
    fb = c.new("final_b", (batch, nheads, headdim, dstate)) if (want_final and not causal) else None
    c.workspace(False)
    c.run("bimamba2_fwd")
    res = (out, out_x, dt_out, cs_f, cs_b, sf, sb, ff, fb)
    return res + (saved,) if keep_for_bwd else res


def _mamba_chunk_scan_combined_bwd(dout, x, dt, A, B, C, out, chunk_size, D=None, z=None, dt_bias=None,
                                   dfinal_states=None, dt_softplus=False, dt_limit=(0.0, _INF),
                                   dx=None, ddt=None, dB=None, dC=None, dz=None, recompute_output=False, saved=None,
                                   causal=False, initial_states=None, seq_idx=None):
    """Returns (dx, ddt, dA, dB, dC, dD, dz, ddt_bias).  `out` must be the pre-gate output out_x when z is
    given (it is what the autograd function saves); it is not read otherwise.  `saved` is the tuple the forward
    returns with keep_for_bwd=True; without it the forward intermediates are recomputed, as in the reference.
    dfinal_states = (dfinal_f, dfinal_b): gradients with respect to the final states (None entries count as zero).
    With initial_states = (initial_f, initial_b) given, the result has a ninth element (dinitial_f, dinitial_b)."""
    assert not recompute_output, "recompute_output is not supported"
    assert dout.shape == x.shape
    blob = None
    if saved is not None and isinstance(saved[0], str):      # ("blob", allocation, snapshot): see the forward
        blob, snap = saved[1], saved[2]
    else:
        snap = saved[5] if saved is not None and len(saved) > 5 else None
    c = None
    if snap is not None:
        # the forward's parameter block, if the tensors handed back by autograd are still the ones it describes
        c = _Call.from_snapshot(snap, x, (x.shape[1] + chunk_size - 1) // chunk_size)
        same = (c.p.x == x.data_ptr() and c.p.dt == dt.data_ptr() and c.p.Bm == B.data_ptr() and c.p.Cm == C.data_ptr()
                and (z is None or c.p.z == z.data_ptr()) and x.is_cuda)
        if not same:
            c = None
    if c is None:
        c = _problem(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit)
    c.p.causal = 1 if causal else 0
    batch, seqlen, nheads, headdim = x.shape
    c.p.initial_f = c.p.initial_b = None          # (a snapshot of the forward call may carry them)
    _set_states(c, ("initial_f", "initial_b"), initial_states, x, B)
    _set_states(c, ("dfinal_f", "dfinal_b"), dfinal_states, x, B)
    _set_seq_idx(c, seq_idx, x)
    dinit = None
    if initial_states is not None:
        sshape = (batch, nheads, headdim, B.shape[3])
        dinit = tuple(c.new(f, sshape) if t is not None else None
                      for f, t in zip(("dinitial_f", "dinitial_b"), initial_states))
    if blob is not None and x.element_size() == 2 and (dout.data_ptr() % 16 or any(s % 8 for s in dout.stride()[:3])):
        # the forward kept the 16-bit copies of the entering states only, which the kernels for aligned operands know:
        # a gradient view that breaks their alignment (e.g. a slice of a wider tensor at an odd offset) is copied
        dout = dout.contiguous()
    c.set_dout(dout)
    if blob is not None:
        _point_into(c, blob, snap[2], snap[3])
        c.p.fwd_saved = 1
    elif saved is not None:
        for name, t in zip(_BLOB_FIELDS, saved[:5]):
            c.put(name, t, torch.float32)
        c.p.fwd_saved = 1
    if z is not None:
        assert out.shape == x.shape
        c.put("out_x", out.contiguous() if out.dtype == x.dtype else out.to(x.dtype).contiguous())
        dz = c.put("dz", dz) if dz is not None else c.new("dz", x.shape, x.dtype)
    c.p.dx_sb = c.p.dx_sl = c.p.dB_sb = c.p.dB_sl = c.p.dC_sb = c.p.dC_sl = 0
    dx = c.put_grad("dx", dx, x.shape, x.dtype) if dx is not None else c.new("dx", x.shape, x.dtype)
    ddt = c.put("ddt", ddt) if ddt is not None else c.new("ddt", dt.shape, dt.dtype)
    dB = c.put_grad("dB", dB, B.shape, x.dtype) if dB is not None else c.new("dB", B.shape, x.dtype)
    dC = c.put_grad("dC", dC, C.shape, x.dtype) if dC is not None else c.new("dC", C.shape, x.dtype)
    dA = c.new("dA", (nheads,))
    dD = c.new("dD", tuple(D.shape)) if D is not None else None
    ddt_bias = c.new("ddt_bias", (nheads,)) if dt_bias is not None else None
    c.workspace(True)
    c.run("bimamba2_bwd")
    res = (dx, ddt, dA.to(A.dtype), dB.to(B.dtype), dC.to(C.dtype),
           dD.to(D.dtype) if dD is not None else None, dz,
           ddt_bias.to(dt_bias.dtype) if ddt_bias is not None else None)
    return res + (dinit,) if dinit is not None else res


# True: the autograd function keeps the forward's small and state intermediates for the backward pass (about
# 2 * batch * nchunks * nheads * headdim * dstate * 4 bytes); False: recompute them as the reference does.
KEEP_FORWARD_INTERMEDIATES = True


class MambaChunkScanCombinedFn(torch.autograd.Function):
    """Same 12 positional arguments and the same 12-tuple of gradients as the reference's autograd function
    (src/ssd/bi/ssd_combined.py:555-574)."""

    @staticmethod
    def forward(ctx, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                dt_limit=(0.0, _INF), return_final_states=False, *extra):
        # extra: nothing (as in the reference), or (initial_states_f, initial_states_b[, seq_idx[, grad_places]]) -
        # extensions
        assert len(extra) in (0, 2, 3, 4)
        initial_states, seq_idx = tuple(extra[:2]), (extra[2] if len(extra) >= 3 else None)
        ctx.grad_places = extra[3] if len(extra) == 4 else None
        ctx.seq_idx = seq_idx
        ctx.n_extra = len(extra)
        ctx.dt_dtype = dt.dtype
        init = tuple(initial_states) if any(t is not None for t in initial_states) else None
        need_bwd = any(ctx.needs_input_grad)       # False under torch.no_grad() and for inputs without requires_grad
        keep = KEEP_FORWARD_INTERMEDIATES and need_bwd
        res = _mamba_chunk_scan_combined_fwd(
            x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, dt_softplus=dt_softplus, dt_limit=dt_limit,
            return_intermediates=False, keep_for_bwd=keep, initial_states=init, seq_idx=seq_idx, want_out_x=need_bwd,
            want_final=return_final_states)
        out, out_x, ff, fb = res[0], res[1], res[7], res[8]
        # kept for the backward pass: ("blob", one allocation with dt_out, cs_f, cs_b and the states, snapshot)
        blob, ctx.snap = (res[9][1], res[9][2]) if keep else (None, None)
        ctx.n_init = len(initial_states)
        ctx.save_for_backward(out_x if z is not None else None, x, dt, A, B, C, D, z, dt_bias,
                              *(initial_states if ctx.n_init else (None, None)), blob)
        ctx.dt_softplus = dt_softplus
        ctx.chunk_size = chunk_size
        ctx.dt_limit = dt_limit
        ctx.return_final_states = return_final_states
        if not return_final_states:
            return out
        # unlike the reference (which refuses a backward pass when final states were returned), gradients flow through
        # the final states; an unused one arrives as None
        ctx.set_materialize_grads(False)
        return out, ff, fb

    @staticmethod
    def backward(ctx, dout, *dfinal):
        out_x, x, dt, A, B, C, D, z, dt_bias, init_f, init_b, blob = ctx.saved_tensors
        saved = ("blob", blob, ctx.snap) if blob is not None else None
        if dout is None:
            dout = torch.zeros_like(x)
        init = (init_f, init_b) if (init_f is not None or init_b is not None) else None
        dfin = tuple(dfinal) if any(t is not None for t in dfinal) else None
        given = {}
        if ctx.grad_places:
            # destinations for dx / dB / dC handed out by the caller (e.g. slices of one buffer); one that does not fit the
            # kernels' layout is not used
            for name, like in (("dx", x), ("dB", B), ("dC", C)):
                t = ctx.grad_places[name]() if ctx.grad_places.get(name) else None
                fits = (t is not None and tuple(t.shape) == tuple(like.shape) and t.dtype == x.dtype and like.dtype == x.dtype
                        and t.stride(3) == 1 and t.stride(2) == like.shape[3] and t.device == x.device)
                # The forward pass of a 16-bit problem keeps only the 16-bit copies of the entering states, which the
                # kernels for 16-byte aligned operands read: a destination that is not aligned that way (an odd offset into
                # a wider buffer) is not used - the kernel writes a fresh tensor and the caller copies it.
                if fits and x.element_size() == 2 and (t.data_ptr() % 16 or t.stride(0) % 8 or t.stride(1) % 8):
                    fits = False
                if fits:
                    given[name] = t
        res = _mamba_chunk_scan_combined_bwd(
            dout, x, dt, A, B, C, out_x, ctx.chunk_size, D=D, z=z, dt_bias=dt_bias, dt_softplus=ctx.dt_softplus,
            dt_limit=ctx.dt_limit, saved=saved, dfinal_states=dfin, initial_states=init, seq_idx=ctx.seq_idx, **given)
        dx, ddt, dA, dB, dC, dD, dz, ddt_bias = res[:8]
        grads = (dx, ddt, dA, dB, dC, None, dD, dz, ddt_bias, None, None, None)
        if ctx.n_init:
            grads += tuple(res[8]) if init is not None else (None, None)
        if ctx.n_extra >= 3:
            grads += (None,) * (ctx.n_extra - 2)
        return grads


def bimamba_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                                dt_limit=(0.0, _INF), return_final_states=False, initial_states_f=None,
                                initial_states_b=None, seq_idx=None, grad_places=None):
    """Bidirectional SSD:  y = SS(x) + flip(SS(flip(x))) + D*x, gated by silu(z) when z is given.

    Argument:
        x: (batch, seqlen, nheads, headdim)
        dt: (batch, seqlen, nheads)
        A: (nheads)
        B: (batch, seqlen, ngroups, dstate)
        C: (batch, seqlen, ngroups, dstate)   (dstate above the kernels' 256: computed in pieces of the state dimension)
        chunk_size: int, at least 32 (above 256 the kernels use 256: the result does not depend on it)
        D: (nheads, headdim) or (nheads,)
        z: (batch, seqlen, nheads, headdim)
        dt_bias: (nheads,)
        dt_softplus: whether to apply softplus to dt (+ dt_bias)
        dt_limit: clamp range for the transformed dt
    Return:
        initial_states_f, initial_states_b: (batch, nheads, headdim, dstate), optional - not in the reference, whose
            bidirectional path starts both recurrences from zero: the state of the forward recurrence in front of the
            first position and of the reverse recurrence behind the last one (e.g. the final states of the
            neighbouring pieces of a longer sequence).  Gradients flow into them and through the final states.
        seq_idx: (batch, seqlen) integers, optional - not in the bidirectional reference (its causal sibling has it):
            constant over each of several sequences packed one behind the other; positions with different seq_idx do
            not interact in either direction.  When some chunk would hold more than MAX_SEQ_BOUNDARIES_PER_CHUNK (32)
            sequence boundaries the call runs with a smaller chunk size (the result does not depend on it), which costs
            one device-to-host synchronisation per call with seq_idx (chunk_size_for_seq_idx).
        grad_places: {"dx": f, "dB": f, "dC": f}, optional - not in the reference: callables asked in the backward pass for
            the tensors these gradients are to be written into (shaped like x / B / C, the two inner dimensions contiguous;
            e.g. slices of one buffer, which saves concatenating them when x, B, C are pieces of one tensor).  A destination
            the kernels cannot write (wrong shape or type, inner dimensions not contiguous, for 16-bit types a base or
            batch / position stride that is not a multiple of 16 bytes) is not used, and neither are any on the routes for
            headdim > 128 and dstate > 256 (torch glue around several kernel calls): the caller then receives freshly
            allocated gradients through autograd as without this argument and copies them where it wants them.
    Return:
        out: (batch, seqlen, nheads, headdim), or (out, final_states_f, final_states_b) with
        return_final_states=True (final states are (batch, nheads, headdim, dstate) float32)
    """
    # The result does not depend on the chunk size (it only sets where the kernels cut the sequence), and the kernels'
    # chunks hold at most 256 positions: a larger chunk_size, which the reference accepts, runs with 256.
    chunk_size = min(chunk_size, MAX_CHUNK_SIZE)
    if seq_idx is not None:
        # many short packed sequences: a smaller chunk keeps the boundaries per chunk inside what the mechanism resolves
        chunk_size = chunk_size_for_seq_idx(seq_idx, chunk_size)
    headdim = x.shape[-1]
    if headdim > MAX_HEADDIM:
        # The channels of a head only share dt, A and the head's group, so a head wider than the kernels' 128 channels
        # is computed as several narrower heads with the same dt, A, dt_bias (and D), side by side in the same group.
        # Everything here is differentiable torch glue: autograd sums the pieces' gradients of dt, A, dt_bias and D.
        parts = next((k for k in range(2, headdim + 1) if headdim % k == 0 and headdim // k <= MAX_HEADDIM), None)
        assert parts is not None
        batch, seqlen, nheads, _ = x.shape
        narrow = lambda t: t.reshape(*t.shape[:-2], nheads * parts, headdim // parts) if t is not None else None
        rep = lambda t, dim: t.repeat_interleave(parts, dim=dim) if t is not None else None
        res = bimamba_chunk_scan_combined(
            narrow(x), rep(dt, 2), rep(A, 0), B, C, chunk_size, D=(narrow(D) if D is not None and D.dim() == 2 else rep(D, 0)),
            z=narrow(z), dt_bias=rep(dt_bias, 0), dt_softplus=dt_softplus, dt_limit=dt_limit, return_final_states=return_final_states,
            initial_states_f=(initial_states_f.reshape(batch, nheads * parts, headdim // parts, -1) if initial_states_f is not None else None),
            initial_states_b=(initial_states_b.reshape(batch, nheads * parts, headdim // parts, -1) if initial_states_b is not None else None),
            seq_idx=seq_idx)
        if not return_final_states:
            return res.reshape(x.shape)
        return (res[0].reshape(x.shape),) + tuple(t.reshape(batch, nheads, headdim, -1) for t in res[1:])
    dstate = B.shape[-1]
    if dstate > MAX_DSTATE:
        # The state columns do not interact: SS(x) with (B, C) is the sum over pieces of the state dimension of SS(x) with
        # that piece of B and of C.  Pieces of at most 256 columns (views: the kernels take strided B / C) go through the
        # kernels without D and gate; the sum, the D term and the gate are differentiable torch glue in float32, and the
        # final states of the pieces lie side by side.
        # The pieces run in float32 whatever the inputs' type: their outputs are summed, and 16-bit pieces, each rounded on
        # its own, would leave the sum several times the rounding error of the one pass the reference makes.
        cuts = [(n0, min(n0 + MAX_DSTATE, dstate)) for n0 in range(0, dstate, MAX_DSTATE)]
        piece = lambda t, n0, n1: t[..., n0:n1] if t is not None else None
        x32, B32, C32 = x.float(), B.float(), C.float()
        y, fins = None, []
        for n0, n1 in cuts:
            r = bimamba_chunk_scan_combined(
                x32, dt, A, piece(B32, n0, n1), piece(C32, n0, n1), chunk_size, dt_bias=dt_bias, dt_softplus=dt_softplus,
                dt_limit=dt_limit, return_final_states=return_final_states,
                initial_states_f=piece(initial_states_f, n0, n1), initial_states_b=piece(initial_states_b, n0, n1), seq_idx=seq_idx)
            if return_final_states:
                fins.append(r[1:])
                r = r[0]
            y = r if y is None else y + r
        if D is not None:
            y = y + x32 * (D.float() if D.dim() == 2 else D.float()[:, None])
        if z is not None:
            y = y * torch.nn.functional.silu(z.float())
        out = y.to(x.dtype)
        if not return_final_states:
            return out
        return out, torch.cat([f[0] for f in fins], dim=-1), torch.cat([f[1] for f in fins], dim=-1)
    if grad_places is not None:
        return MambaChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit,
                                              return_final_states, initial_states_f, initial_states_b, seq_idx, grad_places)
    if initial_states_f is None and initial_states_b is None and seq_idx is None:
        return MambaChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit,
                                              return_final_states)
    if seq_idx is None:
        return MambaChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit,
                                              return_final_states, initial_states_f, initial_states_b)
    return MambaChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit,
                                          return_final_states, initial_states_f, initial_states_b, seq_idx)


class CausalChunkScanCombinedFn(torch.autograd.Function):
    """The single-direction operator  y = SS(x) + D*x  (gated by silu(z)) from the same kernels with the reverse
    direction left out: the comparator the bidirectional pass is timed against.  It exists for the shapes whose scan
    kernels rebuild C.B^T themselves (16-bit x/B/C, headdim a multiple of 64, dstate 64, chunk_size a multiple of 64,
    16-byte aligned rows); other shapes raise.  The math is the reference's causal path
    (src/ssd/uni/ssd_combined.py:621-659 there)."""

    @staticmethod
    def forward(ctx, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False, dt_limit=(0.0, _INF)):
        keep = any(t is not None and t.requires_grad for t in (x, dt, A, B, C, D, z, dt_bias))
        res = _mamba_chunk_scan_combined_fwd(
            x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias, dt_softplus=dt_softplus, dt_limit=dt_limit,
            return_intermediates=False, keep_for_bwd=keep, causal=True, want_final=False)
        blob, ctx.snap = (res[9][1], res[9][2]) if keep else (None, None)
        ctx.save_for_backward(res[1] if z is not None else None, x, dt, A, B, C, D, z, dt_bias, blob)
        ctx.dt_softplus, ctx.chunk_size, ctx.dt_limit = dt_softplus, chunk_size, dt_limit
        return res[0]

    @staticmethod
    def backward(ctx, dout):
        out_x, x, dt, A, B, C, D, z, dt_bias, blob = ctx.saved_tensors
        saved = ("blob", blob, ctx.snap) if blob is not None else None
        dx, ddt, dA, dB, dC, dD, dz, ddt_bias = _mamba_chunk_scan_combined_bwd(
            dout, x, dt, A, B, C, out_x, ctx.chunk_size, D=D, z=z, dt_bias=dt_bias, dt_softplus=ctx.dt_softplus,
            dt_limit=ctx.dt_limit, saved=saved, causal=True)
        return dx, ddt, dA, dB, dC, None, dD, dz, ddt_bias, None, None


def causal_chunk_scan_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                               dt_limit=(0.0, _INF)):
    """Single-direction (causal) SSD with the arguments of bimamba_chunk_scan_combined; see CausalChunkScanCombinedFn."""
    return CausalChunkScanCombinedFn.apply(x, dt, A, B, C, chunk_size, D, z, dt_bias, dt_softplus, dt_limit)

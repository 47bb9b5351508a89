"""CPU-only tests of the host side: the C-ABI library loads and exports what include/bimamba2.h declares, argument
checks answer with error codes before anything is launched, and the Python mirror of the reference interface
refuses what the reference refuses.  No kernel runs here."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

from bi_mamba2_amd import _lib, ops
from bi_mamba2_amd.modules import BiMamba2

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "bimamba2.h")).read()
    declared = set(re.findall(r"\b(bimamba2_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.ALL_SYMBOLS), declared ^ set(_lib.ALL_SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.bimamba2_version() >= 100
    assert lib.bimamba2_params_size() == ctypes.sizeof(_lib.Params)


def _params(**kw):
    p = _lib.Params()
    base = dict(batch=2, seqlen=100, nheads=4, headdim=32, ngroups=2, dstate=16, chunk_size=64, dtype=_lib.BF16,
                dt_dtype=_lib.F32, dt_max=float("inf"))
    base.update(kw)
    for k, v in base.items():
        setattr(p, k, v)
    return p


def test_argument_checks_return_error_codes():
    lib = _lib.load()
    assert lib.bimamba2_fwd(None) == -1
    assert lib.bimamba2_fwd(ctypes.byref(_params())) == -3                      # no workspace
    assert lib.bimamba2_chunk_cumsum_fwd(ctypes.byref(_params())) == -1         # null pointers
    assert lib.bimamba2_fwd(ctypes.byref(_params(chunk_size=512))) == -2        # chunk too large
    assert lib.bimamba2_fwd(ctypes.byref(_params(chunk_size=16))) == -2         # chunk too small (reference: >= 32)
    assert lib.bimamba2_fwd(ctypes.byref(_params(headdim=256))) == -2
    assert lib.bimamba2_fwd(ctypes.byref(_params(nheads=3))) == -1              # heads not divisible by groups
    assert lib.bimamba2_fwd(ctypes.byref(_params(dtype=7))) == -2
    assert lib.bimamba2_bwd(ctypes.byref(_params(fwd_saved=1, workspace=1, workspace_bytes=1 << 40))) == -1
    # the forward without a workspace refuses what its built-in buffer cannot hold, before any GPU call
    big = _params(batch=16, seqlen=65536, nheads=64, headdim=64, ngroups=1, dstate=64, chunk_size=256)
    assert lib.bimamba2_fwd_static(ctypes.byref(big)) == -5
    assert lib.bimamba2_fwd_static(None) == -1
    for code in (0, -1, -2, -3, -4, -5, -99):
        assert lib.bimamba2_strerror(code)
    with pytest.raises(ValueError):
        _lib.call("bimamba2_chunk_cumsum_fwd", _params())


def test_workspace_sizes():
    lib = _lib.load()
    p = _params()
    fwd, bwd = lib.bimamba2_workspace_bytes(ctypes.byref(p), 0), lib.bimamba2_workspace_bytes(ctypes.byref(p), 1)
    nc = 2
    states = 2 * 2 * nc * 4 * 32 * 16 * 4
    assert fwd >= states and bwd > 2 * fwd - 4096
    assert lib.bimamba2_workspace_bytes(ctypes.byref(_params(chunk_size=8)), 0) == 0


def _cpu_inputs(b=1, L=64, H=2, P=4, G=1, N=4):
    return (torch.randn(b, L, H, P), torch.randn(b, L, H), -torch.rand(H), torch.randn(b, L, G, N), torch.randn(b, L, G, N))


def test_no_cpu_fallback():
    x, dt, A, B, C = _cpu_inputs()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.bimamba_chunk_scan_combined(x, dt, A, B, C, 32)


def test_shape_checks_match_the_reference():
    x, dt, A, B, C = _cpu_inputs()
    with pytest.raises(AssertionError):
        ops.bimamba_chunk_scan_combined(x, dt, A, B, C, 16)                       # chunk_size >= 32
    with pytest.raises(AssertionError):
        ops.bimamba_chunk_scan_combined(x, dt[:, :-1], A, B, C, 32)
    with pytest.raises(AssertionError):
        ops.bimamba_chunk_scan_combined(x, dt, A, B, C[..., :-1], 32)
    with pytest.raises(AssertionError):
        ops.bimamba_chunk_scan_combined(x, dt, A, B, C, 32, D=torch.randn(3))
    with pytest.raises(AssertionError):
        ops.bimamba_chunk_scan_combined(x, dt, A, B, C, 32, z=torch.randn(1, 64, 2, 5))


def test_missing_library_fails_loudly(tmp_path):
    code = ("import os; os.environ['BIMAMBA2_LIB'] = %r\n"
            "from bi_mamba2_amd import _lib\n"
            "try:\n    _lib.load()\nexcept RuntimeError as e:\n    print('RAISED', 'no CPU or PyTorch fallback' in str(e))\n") % str(tmp_path / "absent.so")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert "RAISED True" in out.stdout, out.stdout + out.stderr


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "ONE GPU" in out.stderr


def test_bimamba2_layer_parameters():
    """Same parameter names and shapes as the reference layer (src/ssd/modules.py:65-116 there)."""
    m = BiMamba2(d_model=64, d_state=16, headdim=16, ngroups=2, learnable_init_states=True)
    shapes = {k: tuple(v.shape) for k, v in m.state_dict().items()}
    d_inner, nheads, bc = 128, 8, 2 * 2 * 16
    assert shapes == {
        "in_proj.weight": (2 * d_inner + bc + nheads, 64), "conv1d.weight": (d_inner + bc, 1, 7), "conv1d.bias": (d_inner + bc,),
        "init_states": (nheads, 16, 16), "dt_bias": (nheads,), "A_log": (nheads,), "D": (nheads,),
        "fc_D.weight": (nheads, d_inner), "norm.weight": (d_inner,), "out_proj.weight": (64, d_inner)}
    assert torch.all(m.A_log == 0) and torch.all(m.D == 1)
    dt0 = torch.nn.functional.softplus(m.dt_bias)
    assert dt0.min() >= 1e-4 and dt0.max() <= 0.1 + 1e-6


def test_import_aliases():
    from ssd.bi.ssd_combined import bimamba_chunk_scan_combined, MambaChunkScanCombinedFn
    from ssd.modules import BiMamba2 as Alias
    assert bimamba_chunk_scan_combined is ops.bimamba_chunk_scan_combined
    assert MambaChunkScanCombinedFn is ops.MambaChunkScanCombinedFn and Alias is BiMamba2


def test_norm_and_conv_argument_checks():
    """The layer's two extra entry-point families check their arguments before anything is launched."""
    lib = _lib.load()
    assert lib.bimamba2_rmsnorm_gated_fwd(None) == -1 and lib.bimamba2_conv1d_silu_fwd(None) == -1
    n = _lib.NormParams()
    n.rows, n.cols, n.group_size, n.dtype = 4, 64, 48, _lib.F32
    assert lib.bimamba2_rmsnorm_gated_fwd(ctypes.byref(n)) == -1                # groups do not divide the row
    n.group_size = 64
    assert lib.bimamba2_rmsnorm_gated_fwd(ctypes.byref(n)) == -1                # null pointers
    assert lib.bimamba2_rmsnorm_gated_workspace_bytes(ctypes.byref(n)) == 0     # (0 for a problem that fails the checks)
    c = _lib.ConvParams()
    c.batch, c.seqlen, c.channels, c.width, c.dtype = 2, 16, 8, 4, _lib.BF16
    c.x = c.weight = c.out = 256                                               # never dereferenced: the width check comes first
    assert lib.bimamba2_conv1d_silu_fwd(ctypes.byref(c)) == -2                  # even filter width
    c.width = 11
    assert lib.bimamba2_conv1d_silu_fwd(ctypes.byref(c)) == -2                  # wider than the kernels are built for
    c.width, c.x = 7, None
    assert lib.bimamba2_conv1d_silu_fwd(ctypes.byref(c)) == -1                  # null input
    c.x = 256
    c.dout = c.dx = c.dweight = 256
    assert lib.bimamba2_conv1d_silu_bwd(ctypes.byref(c)) == -3                  # backward without workspace
    assert lib.bimamba2_conv1d_silu_workspace_bytes(ctypes.byref(c)) >= 2 * 16 // 56 * 8 * 8 * 4


def test_causal_flag_and_second_direction_buffers():
    """The single-direction comparator refuses a reverse final state."""
    lib = _lib.load()
    p = _params(causal=1, final_b=256, workspace=256, workspace_bytes=1 << 40)
    assert lib.bimamba2_fwd(ctypes.byref(p)) == -1


def test_state_copies_are_for_the_fast_path_only():
    """bimamba2_state_copies() says where the kernels can keep the entering states in 16-bit copies; the workspace of the
    composites holds them there, and a stage that does not know them refuses them (before any launch)."""
    lib = _lib.load()
    fast = dict(batch=2, seqlen=512, nheads=8, headdim=64, ngroups=1, dstate=64, chunk_size=256,
                x_sb=512 * 8 * 64, x_sl=8 * 64, x_sh=64, B_sb=512 * 64, B_sl=64, B_sg=64, C_sb=512 * 64, C_sl=64, C_sg=64,
                x=256, Bm=256, Cm=256)
    assert lib.bimamba2_state_copies(ctypes.byref(_params(**fast))) == 1
    assert lib.bimamba2_state_copies(ctypes.byref(_params(**dict(fast, dtype=_lib.F32)))) == 0
    assert lib.bimamba2_state_copies(ctypes.byref(_params(**dict(fast, dstate=128, B_sl=128, C_sl=128)))) == 0
    assert lib.bimamba2_state_copies(ctypes.byref(_params())) == 0
    # the copies are part of the forward workspace where they are used, and a caller who brings them saves that much
    stn = 2 * 2 * 8 * 64 * 64
    own = lib.bimamba2_workspace_bytes(ctypes.byref(_params(**fast)), 0)
    brought = lib.bimamba2_workspace_bytes(ctypes.byref(_params(**dict(fast, states16_f=256, states16_b=512))), 0)
    assert own - brought == 2 * stn * 2
    # the generic state passing (float32 problem) does not know the copies
    p = _params(cs_f=256, cs_b=256, states_f=256, states_b=256, states16_f=256, states16_b=256, dtype=_lib.F32)
    assert lib.bimamba2_state_passing_fwd(ctypes.byref(p)) == -2


def test_chunk_size_follows_the_number_of_sequence_boundaries():
    """Packed sequences: the host lowers the chunk size until no chunk holds more boundaries than the float32 cumulative sums
    resolve (runs on CPU tensors: only the count is taken here)."""
    import torch
    from bi_mamba2_amd import ops
    lim = ops.MAX_SEQ_BOUNDARIES_PER_CHUNK
    one = torch.zeros(2, 300, dtype=torch.int32)
    assert ops.seq_boundaries_per_chunk(one, 256) == 0 and ops.chunk_size_for_seq_idx(one, 256) == 256
    # a boundary in front of position l counts for the chunk of l (forward sums) and for the chunk of l - 1 (reverse sums)
    edge = torch.zeros(1, 512, dtype=torch.int32)
    edge[0, 256:] = 1
    assert ops.seq_boundaries_per_chunk(edge, 256) == 1
    four = torch.arange(512)[None].div(4, rounding_mode="floor")            # 64 boundaries per 256 positions
    assert ops.seq_boundaries_per_chunk(four, 256) == 64 and ops.seq_boundaries_per_chunk(four, 128) == 32
    assert ops.chunk_size_for_seq_idx(four, 256) == 128
    single = torch.arange(256)[None]                                        # every token its own sequence
    assert ops.chunk_size_for_seq_idx(single, 256) == 32
    assert ops.seq_boundaries_per_chunk(single, 32) <= lim
    mixed = torch.cat([torch.zeros(1, 256, dtype=torch.int64), 1 + torch.arange(256)[None].div(5, rounding_mode="floor")], dim=1)
    assert ops.chunk_size_for_seq_idx(mixed, 256) == 128                    # the densest chunk decides
    assert ops.chunk_size_for_seq_idx(four, 64) == 64                       # never above what the caller asked for

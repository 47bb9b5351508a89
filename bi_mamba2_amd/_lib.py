"""ctypes binding of libbimamba2_hip.so (the C ABI declared in include/bimamba2.h).

There is no fallback: if the library has not been built, loading raises and every operator fails loudly.
Build it with ``make -C bi_mamba2_amd/csrc`` (or ``python __graft_entry__.py``).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# BIMAMBA2_LIB lets a caller point at another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("BIMAMBA2_LIB") or os.path.join(_HERE, "libbimamba2_hip.so")

F32, BF16, F16 = 0, 1, 2

_i32, _i64, _f32, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class Params(ctypes.Structure):
    """Mirror of ``struct bimamba2_params``; the field order must match the header."""
    _fields_ = (
        [(n, _i32) for n in ("batch", "seqlen", "nheads", "headdim", "ngroups", "dstate", "chunk_size",
                             "dtype", "dt_dtype", "has_D", "D_has_hdim", "has_z", "has_dt_bias", "dt_softplus",
                             "fwd_saved", "causal")]
        + [("dt_min", _f32), ("dt_max", _f32)]
        + [(n, _i64) for n in ("x_sb", "x_sl", "x_sh", "z_sb", "z_sl", "z_sh", "dout_sb", "dout_sl", "dout_sh",
                               "B_sb", "B_sl", "B_sg", "C_sb", "C_sl", "C_sg", "dt_sb", "dt_sl", "dt_sh")]
        + [(n, _vp) for n in ("x", "dt", "Bm", "Cm", "z", "dout", "A", "D", "dt_bias",
                              "out", "out_x", "final_f", "final_b",
                              "dx", "ddt", "dB", "dC", "dz", "dA", "dD", "ddt_bias",
                              "dt_out", "cs_f", "cs_b", "CB", "dCB", "CBT", "dCBT", "states_f", "states_b",
                              "dstates_f", "dstates_b", "dout_x",
                              "ddt_direct", "u_f", "u_b", "v_f", "v_b", "da_intra",
                              "ddA_chunk_f", "ddA_chunk_b", "dBs", "dCs", "red",
                              "initial_f", "initial_b", "dfinal_f", "dfinal_b", "dinitial_f", "dinitial_b", "seq_idx",
                              "states16_f", "states16_b", "dstates16_f", "dstates16_b", "workspace")]
        + [("workspace_bytes", ctypes.c_size_t), ("stream", _vp)]
        + [(n, _i64) for n in ("dx_sb", "dx_sl", "dB_sb", "dB_sl", "dC_sb", "dC_sl")]
    )


ENTRY_POINTS = (
    "bimamba2_fwd", "bimamba2_bwd", "bimamba2_fwd_static",
    "bimamba2_chunk_cumsum_fwd", "bimamba2_bmm_chunk_fwd", "bimamba2_chunk_state_fwd",
    "bimamba2_state_passing_fwd", "bimamba2_chunk_scan_fwd",
    "bimamba2_chunk_scan_bwd_dz", "bimamba2_chunk_scan_bwd_dstates", "bimamba2_chunk_scan_bwd_dz_dstates", "bimamba2_state_passing_bwd",
    "bimamba2_chunk_scan_bwd_dx", "bimamba2_chunk_state_bwd_db", "bimamba2_chunk_scan_bwd_dc",
    "bimamba2_chunk_scan_bwd_dcb", "bimamba2_bmm_chunk_bwd", "bimamba2_chunk_cumsum_bwd",
)
NORM_ENTRY_POINTS = ("bimamba2_rmsnorm_gated_fwd", "bimamba2_rmsnorm_gated_bwd")
CONV_ENTRY_POINTS = ("bimamba2_conv1d_silu_fwd", "bimamba2_conv1d_silu_bwd")
ALL_SYMBOLS = ENTRY_POINTS + ("bimamba2_strerror", "bimamba2_version", "bimamba2_params_size",
                              "bimamba2_workspace_bytes", "bimamba2_chunk_scan_reads_cb", "bimamba2_state_copies",
                              "bimamba2_chunk_scan_heads_per_workgroup", "bimamba2_ddt_direct_planes", "bimamba2_norm_params_size",
                              "bimamba2_rmsnorm_gated_workspace_bytes", "bimamba2_conv_params_size",
                              "bimamba2_conv1d_silu_workspace_bytes", "bimamba2_cast_params_size",
                              "bimamba2_cast_many") + NORM_ENTRY_POINTS + CONV_ENTRY_POINTS

_lib = None


class NormParams(ctypes.Structure):
    """Mirror of ``struct bimamba2_norm_params`` (gated RMSNorm)."""
    _fields_ = (
        [("rows", _i64), ("cols", _i32), ("group_size", _i32), ("dtype", _i32), ("has_z", _i32), ("has_bias", _i32),
         ("norm_before_gate", _i32), ("eps", _f32), ("layer_norm", _i32)]
        + [(n, _i64) for n in ("x_rs", "z_rs", "out_rs", "dout_rs", "dx_rs", "dz_rs")]
        + [(n, _vp) for n in ("x", "z", "weight", "bias", "out", "rstd", "dout", "dx", "dz", "dweight", "dbias", "workspace")]
        + [("workspace_bytes", ctypes.c_size_t), ("stream", _vp), ("mean", _vp)]
    )


class ConvParams(ctypes.Structure):
    """Mirror of ``struct bimamba2_conv_params`` (depthwise conv1d + SiLU)."""
    _fields_ = (
        [("batch", _i64), ("seqlen", _i64), ("channels", _i32), ("width", _i32), ("dtype", _i32), ("has_bias", _i32)]
        + [(n, _i64) for n in ("x_sb", "x_sl", "dout_sb", "dout_sl")]
        + [(n, _vp) for n in ("x", "weight", "bias", "out", "dout", "dx", "dweight", "dbias", "workspace")]
        + [("workspace_bytes", ctypes.c_size_t), ("stream", _vp), ("dx_sb", _i64), ("dx_sl", _i64)]
    )


CAST_MAX = 8
CAST_COPY, CAST_NEG_EXP, CAST_MUL = 0, 1, 2


class CastItem(ctypes.Structure):
    _fields_ = [("src", _vp), ("dst", _vp), ("aux", _vp), ("n", _i64), ("src_dtype", _i32), ("dst_dtype", _i32), ("op", _i32),
                ("reserved", _i32)]


class CastParams(ctypes.Structure):
    """Mirror of ``struct bimamba2_cast_params`` (several small conversions in one launch)."""
    _fields_ = [("count", _i32), ("reserved", _i32), ("item", CastItem * CAST_MAX), ("stream", _vp)]


def load():
    """Loads the shared library once; raises RuntimeError when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built (run `make -C {_HERE}/csrc`). "
            "There is no CPU or PyTorch fallback for this operator.")
    lib = ctypes.CDLL(LIB_PATH)
    for name in ENTRY_POINTS:
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(Params)]
        fn.restype = ctypes.c_int
    lib.bimamba2_strerror.argtypes = [ctypes.c_int]
    lib.bimamba2_strerror.restype = ctypes.c_char_p
    lib.bimamba2_version.restype = ctypes.c_int
    lib.bimamba2_chunk_scan_reads_cb.argtypes = [ctypes.POINTER(Params), ctypes.c_int]
    lib.bimamba2_chunk_scan_reads_cb.restype = ctypes.c_int
    lib.bimamba2_chunk_scan_heads_per_workgroup.argtypes = [ctypes.POINTER(Params), ctypes.c_int]
    lib.bimamba2_chunk_scan_heads_per_workgroup.restype = ctypes.c_int
    lib.bimamba2_ddt_direct_planes.argtypes = [ctypes.POINTER(Params)]
    lib.bimamba2_ddt_direct_planes.restype = ctypes.c_int
    lib.bimamba2_state_copies.argtypes = [ctypes.POINTER(Params)]
    lib.bimamba2_state_copies.restype = ctypes.c_int
    lib.bimamba2_params_size.restype = ctypes.c_size_t
    if lib.bimamba2_params_size() != ctypes.sizeof(Params):
        raise RuntimeError("bimamba2_params layout mismatch between the library and its Python mirror")
    lib.bimamba2_workspace_bytes.argtypes = [ctypes.POINTER(Params), ctypes.c_int]
    lib.bimamba2_workspace_bytes.restype = ctypes.c_size_t
    for name in NORM_ENTRY_POINTS:
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(NormParams)]
        fn.restype = ctypes.c_int
    lib.bimamba2_norm_params_size.restype = ctypes.c_size_t
    if lib.bimamba2_norm_params_size() != ctypes.sizeof(NormParams):
        raise RuntimeError("bimamba2_norm_params layout mismatch between the library and its Python mirror")
    lib.bimamba2_rmsnorm_gated_workspace_bytes.argtypes = [ctypes.POINTER(NormParams)]
    lib.bimamba2_rmsnorm_gated_workspace_bytes.restype = ctypes.c_size_t
    for name in CONV_ENTRY_POINTS:
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(ConvParams)]
        fn.restype = ctypes.c_int
    lib.bimamba2_conv_params_size.restype = ctypes.c_size_t
    if lib.bimamba2_conv_params_size() != ctypes.sizeof(ConvParams):
        raise RuntimeError("bimamba2_conv_params layout mismatch between the library and its Python mirror")
    lib.bimamba2_conv1d_silu_workspace_bytes.argtypes = [ctypes.POINTER(ConvParams)]
    lib.bimamba2_conv1d_silu_workspace_bytes.restype = ctypes.c_size_t
    lib.bimamba2_cast_params_size.restype = ctypes.c_size_t
    if lib.bimamba2_cast_params_size() != ctypes.sizeof(CastParams):
        raise RuntimeError("bimamba2_cast_params layout mismatch between the library and its Python mirror")
    lib.bimamba2_cast_many.argtypes = [ctypes.POINTER(CastParams)]
    lib.bimamba2_cast_many.restype = ctypes.c_int
    _lib = lib
    return lib


def call(name, params):
    """Calls an entry point and turns a negative return code into a Python exception."""
    lib = load()
    rc = getattr(lib, name)(ctypes.byref(params))
    if rc != 0:
        msg = lib.bimamba2_strerror(rc).decode()
        exc = ValueError if rc in (-1, -2, -5) else RuntimeError
        raise exc(f"{name}: {msg} (code {rc})")

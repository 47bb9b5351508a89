"""ctypes binding of oracle/bimamba2_seq.c (scalar C restatement of the forward).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libbimamba2_seq.so")


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "all"])


def _lib():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.bimamba2_seq_forward.restype = ctypes.c_int
    return lib


def _p(t):
    if t is None:
        return ctypes.c_void_p(0), None
    a = np.ascontiguousarray(t.detach().to(torch.float64).numpy())
    return a.ctypes.data_as(ctypes.c_void_p), a


def seq_forward(x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """Returns (out, out_x, final_f, final_b) as float64 torch tensors."""
    nb, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    out = np.zeros((nb, L, H, P))
    out_x = np.zeros((nb, L, H, P))
    ff = np.zeros((nb, H, P, N))
    fb = np.zeros((nb, H, P, N))
    keep = [_p(t) for t in (x, dt, A, B, C, D, z, dt_bias)]
    px, pdt, pA, pB, pC, pD, pz, pbias = [k[0] for k in keep]
    rc = _lib().bimamba2_seq_forward(
        nb, L, H, P, G, N, px, pdt, pA, pB, pC, pD, ctypes.c_int(int(D is not None and D.dim() == 2)), pz, pbias,
        ctypes.c_int(int(dt_softplus)), ctypes.c_double(float(dt_limit[0])), ctypes.c_double(float(dt_limit[1])),
        out.ctypes.data_as(ctypes.c_void_p), out_x.ctypes.data_as(ctypes.c_void_p),
        ff.ctypes.data_as(ctypes.c_void_p), fb.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise RuntimeError(f"bimamba2_seq_forward failed with {rc}")
    return tuple(torch.from_numpy(a) for a in (out, out_x, ff, fb))

"""The oracle against the committed golden fixtures (CPU), and the HIP path against the same fixtures (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import bimamba2_oracle as O
from oracle.seq_c import seq_forward
from tests.helpers import assert_close, is_reduced

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _tiny():
    d = np.load(os.path.join(GOLD, "tiny_case.npz"))
    return {k: torch.from_numpy(d[k]) for k in d.files}


def test_oracle_matches_tiny_fixture():
    t = _tiny()
    kw = dict(D=t["in_D"], z=t["in_z"], dt_bias=t["in_dt_bias"], dt_softplus=True)
    args = (t["in_x"], t["in_dt"], t["in_A"], t["in_B"], t["in_C"])
    for fn in (O.bimamba2_sequential, lambda *a, **k: O.bimamba2_naive_chunked(*a, 32, **k), seq_forward):
        out, out_x, ff, fb = fn(*args, **kw)
        torch.testing.assert_close(out, t["out"], rtol=1e-11, atol=1e-11)
        torch.testing.assert_close(out_x, t["out_x"], rtol=1e-11, atol=1e-11)
        torch.testing.assert_close(ff, t["final_f"], rtol=1e-11, atol=1e-11)
        torch.testing.assert_close(fb, t["final_b"], rtol=1e-11, atol=1e-11)
    g = O.bimamba2_grads(t["dout"], *args, form="chunked", chunk_size=32, **kw)
    for k in ("dx", "ddt", "dA", "dB", "dC", "dD", "dz", "ddt_bias"):
        torch.testing.assert_close(g[k], t[k], rtol=1e-10, atol=1e-10)


def test_oracle_matches_config0_fixture():
    d = np.load(os.path.join(GOLD, "config0_forward.npz"))
    inp = O.make_inputs(2, 256, 4, 32, 1, 16, seed=0, dtype=torch.float32, with_z=False)
    r = {k: (v.double() if v is not None else None) for k, v in inp.items()}
    out = O.bimamba2_naive_chunked(r["x"], r["dt"], r["A"], r["B"], r["C"], 64, D=r["D"], dt_bias=r["dt_bias"], dt_softplus=True)[0]
    np.testing.assert_allclose(out.flatten()[torch.from_numpy(d["index"])].numpy(), d["values"], rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(out.sum().item(), d["total"], rtol=1e-10)
    np.testing.assert_allclose(out.sum((0, 1, 3)).numpy(), d["per_head"], rtol=1e-10)


@pytest.mark.gpu
def test_gpu_matches_tiny_fixture():
    from bi_mamba2_amd import ops
    t = _tiny()
    dev = {k: v.float().cuda() for k, v in t.items()}
    leaves = {k: dev["in_" + k].clone().requires_grad_(True) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")}
    out, ff, fb = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 32,
                                                  D=leaves["D"], z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True,
                                                  return_final_states=True)
    assert_close(out, t["out"], torch.float32, "out")
    assert_close(ff, t["final_f"], torch.float32, "final_f")
    assert_close(fb, t["final_b"], torch.float32, "final_b")
    out2 = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 32,
                                           D=leaves["D"], z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    out2.backward(dev["dout"])
    for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias"):
        assert_close(leaves[k].grad, t["d" + k], torch.float32, "d" + k, scaled=is_reduced("d" + k, torch.float32))


@pytest.mark.gpu
def test_gpu_matches_config0_fixture():
    from bi_mamba2_amd import ops
    d = np.load(os.path.join(GOLD, "config0_forward.npz"))
    inp = O.make_inputs(2, 256, 4, 32, 1, 16, seed=0, dtype=torch.float32, with_z=False)
    g = {k: (v.cuda() if v is not None else None) for k, v in inp.items()}
    out = ops.bimamba_chunk_scan_combined(g["x"], g["dt"], g["A"], g["B"], g["C"], 64, D=g["D"], dt_bias=g["dt_bias"], dt_softplus=True)
    got = out.flatten()[torch.from_numpy(d["index"]).cuda()]
    assert_close(got, torch.from_numpy(d["values"]), torch.float32, "config 0 samples")
    assert abs(out.double().sum().item() - float(d["total"])) <= 1e-4 * float(d["abs_total"])

"""Writes the golden fixtures of this directory from the CPU oracle (float64).

The reference project ships no stored vectors for this path (its tests compare two GPU implementations with each
other), so the fixtures are produced by the oracle after it has been pinned by tests/test_oracle.py; they freeze
those values against later edits of the oracle and give the GPU tests a file-based anchor.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import bimamba2_oracle as O  # noqa: E402


def tiny():
    """Every tensor of a tiny case: partial last chunk, 2 heads per group, z, D (H, P), dt_bias, softplus."""
    inp = O.make_inputs(1, 40, 4, 4, 2, 4, seed=123, dtype=torch.float32, with_z=True, D_has_hdim=True)
    r = {k: v.double() for k, v in inp.items()}
    dout = torch.randn(r["x"].shape, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    kw = dict(D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True)
    out, out_x, ff, fb = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], **kw)
    g = O.bimamba2_grads(dout, r["x"], r["dt"], r["A"], r["B"], r["C"], **kw)
    arrays = {"in_" + k: v.numpy() for k, v in r.items()}
    arrays.update(dout=dout.numpy(), out=out.numpy(), out_x=out_x.numpy(), final_f=ff.numpy(), final_b=fb.numpy())
    arrays.update({k: v.numpy() for k, v in g.items() if k != "out" and v is not None})
    np.savez_compressed(os.path.join(HERE, "tiny_case.npz"), **arrays)


def config0():
    """Baseline configuration 0 (batch 2, seqlen 256, 4 heads x 32, 1 group, dstate 16, chunk 64, float32,
    forward only, seed 0): the output at a fixed set of positions plus whole-tensor sums."""
    inp = O.make_inputs(2, 256, 4, 32, 1, 16, seed=0, dtype=torch.float32, with_z=False)
    r = {k: (v.double() if v is not None else None) for k, v in inp.items()}
    out = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], dt_bias=r["dt_bias"], dt_softplus=True)[0]
    idx = torch.randint(0, out.numel(), (512,), generator=torch.Generator().manual_seed(11))
    np.savez_compressed(os.path.join(HERE, "config0_forward.npz"), index=idx.numpy(), values=out.flatten()[idx].numpy(),
                        total=np.array(out.sum().item()), abs_total=np.array(out.abs().sum().item()),
                        per_head=out.sum((0, 1, 3)).numpy())


if __name__ == "__main__":
    tiny()
    config0()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))

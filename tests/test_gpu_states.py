"""GPU parity of the states at the ends of the sequence: initial states of both recurrences, gradients into them and
gradients through the final states (the reference's bidirectional path has none of these), against torch.autograd on
the float64 recurrence, and the cut-sequence identity at a fast-path shape."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, is_reduced, make_case, to64, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


CASES = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z
    (2, 100, 4, 16, 2, 8, 32, torch.float32, False),
    (1, 130, 2, 32, 1, 16, 64, torch.float32, True),
    (2, 300, 4, 64, 2, 64, 128, torch.bfloat16, True),
    (1, 512, 8, 64, 1, 64, 256, torch.bfloat16, False),
]


def _states(b, H, P, N, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(b, H, P, N, generator=g) * 0.5


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("keep", [True, False])
def test_initial_states_and_final_state_gradients(ops, case, keep, monkeypatch):
    monkeypatch.setattr(ops, "KEEP_FORWARD_INTERMEDIATES", keep)
    b, L, H, P, G, N, Q, dtype, z = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z)
    init = {"f": _states(b, H, P, N, 11), "b": _states(b, H, P, N, 12)}
    cot = {"f": _states(b, H, P, N, 13), "b": _states(b, H, P, N, 14)}
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    di = {k: v.cuda().requires_grad_(True) for k, v in init.items()}
    out, ff, fb = ops.bimamba_chunk_scan_combined(
        leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"], z=leaves["z"],
        dt_bias=leaves["dt_bias"], dt_softplus=True, return_final_states=True, initial_states_f=di["f"],
        initial_states_b=di["b"])
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    torch.autograd.backward([out, ff, fb], [dout.cuda(), cot["f"].cuda(), cot["b"].cuda()])

    r = {k: (v.clone().requires_grad_(True) if torch.is_tensor(v) else v) for k, v in to64(inp).items()}
    ri = {k: v.double().requires_grad_(True) for k, v in init.items()}
    ro, _, rff, rfb = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                                            dt_softplus=True, initial_states_f=ri["f"], initial_states_b=ri["b"])
    torch.autograd.backward([ro, rff, rfb], [dout.double(), cot["f"].double(), cot["b"].double()])
    # the initial states (RMS 0.5 over dstate columns) lift the 16-bit cases' outputs well above unit scale
    big = dtype != torch.float32
    assert_close(out, ro, dtype, "out", scaled=big)
    assert_close(ff, rff, dtype, "final_f", scaled=big)
    assert_close(fb, rfb, dtype, "final_b", scaled=big)
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if r[k] is not None:
            assert_close(leaves[k].grad, r[k].grad, dtype, "d" + k, scaled=big or is_reduced("d" + k, dtype))
    assert_close(di["f"].grad, ri["f"].grad, dtype, "dinitial_f", scaled=big)
    assert_close(di["b"].grad, ri["b"].grad, dtype, "dinitial_b", scaled=big)


def test_cut_sequence_equals_the_whole(ops):
    """Two pieces of a sequence, chained through their final states, reproduce the uncut operator (what a split of the
    sequence over devices, or chunked processing of a long one, relies on)."""
    b, L, H, P, G, N, Q, dtype = 2, 1024, 8, 64, 1, 64, 256, torch.bfloat16
    d = to_dev(make_case(b, L, H, P, G, N, dtype, with_z=True))
    kw = dict(D=d["D"], dt_bias=d["dt_bias"], dt_softplus=True, return_final_states=True)
    run = lambda s, **extra: ops.bimamba_chunk_scan_combined(d["x"][:, s], d["dt"][:, s], d["A"], d["B"][:, s], d["C"][:, s], Q,
                                                            z=d["z"][:, s], **kw, **extra)
    full = run(slice(0, L))
    cut = 512
    s1, s2 = slice(0, cut), slice(cut, L)
    fin_f1, fin_b2 = run(s1)[1], run(s2)[2]
    r1 = run(s1, initial_states_b=fin_b2)
    r2 = run(s2, initial_states_f=fin_f1)
    assert_close(torch.cat([r1[0], r2[0]], 1), full[0], dtype, "out")
    assert_close(r2[1], full[1], dtype, "final_f")
    assert_close(r1[2], full[2], dtype, "final_b")

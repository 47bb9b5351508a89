"""CPU tests that pin the oracle itself (no GPU, no kernels).

The three statements of the forward (literal recurrence, quadratic closed form, chunked flip-and-sum) plus
the staged composition are compared with each other, with the scalar C restatement, with special cases whose
answer is textbook arithmetic, and the autograd gradients with finite differences."""
import math

import pytest
import torch

from oracle import bimamba2_oracle as O
from oracle.seq_c import seq_forward
from tests.helpers import make_case, to64

CASES = [
    # batch, seqlen, H, P, G, N, chunk, z, D_hdim, softplus, bias, limit
    (2, 70, 4, 8, 2, 6, 32, True, False, True, True, (0.0, float("inf"))),
    (1, 33, 2, 4, 1, 3, 32, False, True, False, False, (0.0, float("inf"))),
    (2, 96, 4, 4, 4, 4, 32, False, False, True, True, (0.02, 0.3)),
    (1, 64, 6, 5, 3, 7, 64, True, True, True, False, (0.0, float("inf"))),
]


def _kw(inp, softplus, limit):
    return dict(D=inp["D"], z=inp["z"], dt_bias=inp["dt_bias"], dt_softplus=softplus, dt_limit=limit)


@pytest.mark.parametrize("case", CASES)
def test_forms_agree(case):
    b, L, H, P, G, N, Q, z, dh, sp, bias, lim = case
    inp = to64(make_case(b, L, H, P, G, N, torch.float32, with_z=z, D_has_hdim=dh, with_bias=bias))
    args = (inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"])
    kw = _kw(inp, sp, lim)
    seq = O.bimamba2_sequential(*args, **kw)
    quad = O.bimamba2_quadratic(*args, **kw)
    naive = O.bimamba2_naive_chunked(*args, Q, **kw)
    staged = O.bimamba2_staged(*args, Q, **kw)
    cseq = seq_forward(*args, **kw)
    for name, o in (("quadratic", quad), ("naive", naive), ("staged", staged), ("C", cseq)):
        torch.testing.assert_close(o[0], seq[0], rtol=1e-11, atol=1e-11, msg=lambda m: f"{name} out: {m}")
        torch.testing.assert_close(o[1], seq[1], rtol=1e-11, atol=1e-11, msg=lambda m: f"{name} out_x: {m}")
    for name, o in (("naive", naive), ("staged", staged), ("C", cseq)):
        torch.testing.assert_close(o[2], seq[2], rtol=1e-11, atol=1e-11)
        torch.testing.assert_close(o[3], seq[3], rtol=1e-11, atol=1e-11)


def test_A_zero_is_masked_matmul():
    """A = 0: every decay is 1, so y_t = sum_s (C_t.B_s) dt_s x_s (1[s<=t] + 1[s>=t])."""
    inp = to64(make_case(1, 40, 2, 3, 1, 5, with_D=False, with_bias=False))
    inp["A"] = torch.zeros(2, dtype=torch.float64)
    dtp = inp["dt"].abs()
    out = O.bimamba2_sequential(inp["x"], dtp, inp["A"], inp["B"], inp["C"])[0]
    cb = torch.einsum("btgn,bsgn->bts", inp["C"], inp["B"])
    L = 40
    mask = torch.tril(torch.ones(L, L, dtype=torch.float64)) + torch.triu(torch.ones(L, L, dtype=torch.float64))
    ref = torch.einsum("bts,bsh,bshp->bthp", cb * mask, dtp, inp["x"])
    torch.testing.assert_close(out, ref, rtol=1e-12, atol=1e-12)


def test_constant_channel_geometric_series():
    """x = B = C = 1, dt = d, A = a: y_t = d (sum_{k=0..t} r^k + sum_{k=0..L-1-t} r^k), r = e^{d a}."""
    L, d, a = 17, 0.3, -0.7
    one = torch.ones(1, L, 1, 1, dtype=torch.float64)
    out = O.bimamba2_quadratic(one, torch.full((1, L, 1), d, dtype=torch.float64), torch.tensor([a], dtype=torch.float64),
                               one.clone(), one.clone())[0]
    r = math.exp(d * a)
    ref = torch.tensor([d * ((1 - r ** (t + 1)) / (1 - r) + (1 - r ** (L - t)) / (1 - r)) for t in range(L)], dtype=torch.float64)
    torch.testing.assert_close(out.flatten(), ref, rtol=1e-12, atol=1e-12)


def test_flip_equivariance_and_linearity():
    inp = to64(make_case(2, 50, 2, 4, 1, 4, with_z=False))
    f = lambda x, dt, B, C: O.bimamba2_quadratic(x, dt, inp["A"], B, C, D=inp["D"], dt_bias=inp["dt_bias"], dt_softplus=True)[0]
    y = f(inp["x"], inp["dt"], inp["B"], inp["C"])
    yf = f(inp["x"].flip(1), inp["dt"].flip(1), inp["B"].flip(1), inp["C"].flip(1))
    torch.testing.assert_close(yf.flip(1), y, rtol=1e-11, atol=1e-11)
    y2 = f(2.5 * inp["x"], inp["dt"], inp["B"], inp["C"])
    torch.testing.assert_close(y2, 2.5 * y, rtol=1e-11, atol=1e-11)


def test_single_chunk_has_no_state_contribution():
    inp = to64(make_case(1, 32, 2, 4, 1, 4))
    dt_out, cs_f, cs_b = O.stage_chunk_cumsum(inp["dt"], inp["A"], 32, inp["dt_bias"], True)
    S_f, S_b = O.stage_chunk_state(inp["B"], inp["x"], dt_out, cs_f, cs_b)
    prev_f, prev_b, ff, fb = O.stage_state_passing(S_f, S_b, cs_f, cs_b)
    assert prev_f.abs().max() == 0 and prev_b.abs().max() == 0
    torch.testing.assert_close(ff, S_f[:, 0])
    torch.testing.assert_close(fb, S_b[:, 0])


def test_softplus_threshold_and_clamp():
    dt = torch.tensor([[[-30.0], [0.0], [19.9], [20.1], [25.0]]], dtype=torch.float64)
    out = O.dt_transform(dt, None, True, (0.0, float("inf")))
    ref = torch.tensor([math.log1p(math.exp(-30.0)), math.log(2.0), math.log1p(math.exp(19.9)), 20.1, 25.0], dtype=torch.float64)
    torch.testing.assert_close(out.flatten(), ref, rtol=1e-12, atol=0)
    out = O.dt_transform(torch.tensor([[[-1.0], [0.5], [3.0]]], dtype=torch.float64), None, False, (0.1, 2.0))
    torch.testing.assert_close(out.flatten(), torch.tensor([0.1, 0.5, 2.0], dtype=torch.float64))
    # default limits still clamp negative dt to 0 when softplus is off
    out = O.dt_transform(torch.tensor([[[-1.0]]], dtype=torch.float64), None, False)
    assert out.item() == 0.0


def test_autograd_matches_finite_differences():
    inp = to64(make_case(1, 9, 2, 2, 1, 3, with_z=True, D_has_hdim=True))
    leaves = [inp[k].clone().requires_grad_(True) for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")]

    def fn(x, dt, A, B, C, D, z, bias):
        return O.bimamba2_quadratic(x, dt, A, B, C, D=D, z=z, dt_bias=bias, dt_softplus=True, dt_limit=(0.0, 5.0))[0]

    assert torch.autograd.gradcheck(fn, leaves, eps=1e-6, atol=1e-6, rtol=1e-5)

    def fn_seq(x, dt, A, B, C, D, z, bias):
        return O.bimamba2_sequential(x, dt, A, B, C, D=D, z=z, dt_bias=bias, dt_softplus=True)[0]

    assert torch.autograd.gradcheck(fn_seq, leaves, eps=1e-6, atol=1e-6, rtol=1e-5)


def test_gradients_of_forms_agree():
    inp = to64(make_case(2, 70, 4, 4, 2, 4, with_z=True))
    dout = torch.randn(inp["x"].shape, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    kw = dict(D=inp["D"], z=inp["z"], dt_bias=inp["dt_bias"], dt_softplus=True)
    a = O.bimamba2_grads(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], form="quadratic", **kw)
    b = O.bimamba2_grads(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], form="chunked", chunk_size=32, **kw)
    for k in a:
        torch.testing.assert_close(a[k], b[k], rtol=1e-10, atol=1e-10, msg=lambda m: f"{k}: {m}")


def test_gradients_through_the_stage_functions_agree_with_the_closed_form():
    """The GPU tests of the backward stages take torch.autograd through the stage_* functions as the expected value: here
    the gradients through their composition (ragged last chunk, grouped heads) are held against the closed form's."""
    inp = to64(make_case(2, 70, 4, 4, 2, 4, with_z=True, D_has_hdim=True))
    dout = torch.randn(inp["x"].shape, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")
    leaves = {k: inp[k].clone().requires_grad_(True) for k in names}
    out = O.bimamba2_staged(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 32, D=leaves["D"], z=leaves["z"],
                            dt_bias=leaves["dt_bias"], dt_softplus=True)[0]
    out.backward(dout)
    ref = O.bimamba2_grads(dout, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                           dt_bias=inp["dt_bias"], dt_softplus=True, form="quadratic")
    for k in names:
        torch.testing.assert_close(leaves[k].grad, ref["d" + k], rtol=1e-10, atol=1e-10, msg=lambda m: f"{k}: {m}")


def test_causal_operator_against_the_plain_recurrence():
    """ssd_causal (what the single-direction comparator is checked against) against the token-by-token recurrence
    h_t = e^{dt_t A} h_{t-1} + dt_t x_t (x) B_t,  y_t = C_t . h_t + D x_t  written out here, and: the two causal passes
    (as given, and on the flipped sequence) add up to the bidirectional operator, whose diagonal term is counted twice."""
    inp = to64(make_case(2, 37, 4, 3, 2, 5, with_z=True, D_has_hdim=True))
    x, dt, A, B, C, D, z, bias = (inp[k] for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias"))
    out, out_x, final = O.ssd_causal(x, dt, A, B, C, 16, D=D, z=z, dt_bias=bias, dt_softplus=True)
    dtp = torch.nn.functional.softplus(dt + bias)
    bsz, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    y = torch.zeros_like(x)
    for b in range(bsz):
        for h in range(H):
            g = h // (H // G)
            st = torch.zeros(P, N, dtype=x.dtype)
            for t in range(L):
                st = torch.exp(dtp[b, t, h] * A[h]) * st + dtp[b, t, h] * torch.outer(x[b, t, h], B[b, t, g])
                y[b, t, h] = st @ C[b, t, g] + D[h] * x[b, t, h]
            torch.testing.assert_close(final[b, h], st, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out_x, y, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out, y * z * torch.sigmoid(z), rtol=1e-10, atol=1e-10)
    # bidirectional = causal + flip(causal(flip)); the diagonal term dt_t (C_t.B_t) x_t is in both passes
    kw = dict(dt_bias=bias, dt_softplus=True)
    yf = O.ssd_causal(x, dt, A, B, C, 16, **kw)[0]
    yb = O.ssd_causal(x.flip(1), dt.flip(1), A, B.flip(1), C.flip(1), 16, **kw)[0].flip(1)
    bi = O.bimamba2_sequential(x, dt, A, B, C, **kw)[0]
    torch.testing.assert_close(yf + yb, bi, rtol=1e-10, atol=1e-10)


def test_initial_states_make_a_split_sequence_equal_the_whole():
    """The oracle's initial states: a sequence cut in two pieces, the second started from the first's final forward
    state and the first from the second's final reverse state, reproduces the uncut result (outputs and final states)."""
    inp = to64(make_case(2, 41, 4, 3, 2, 5, with_z=True))
    x, dt, A, B, C, D, z, bias = (inp[k] for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias"))
    kw = dict(dt_bias=bias, dt_softplus=True)
    full = O.bimamba2_sequential(x, dt, A, B, C, D=D, z=z, **kw)
    cut = 17
    a = lambda t: t[:, :cut]
    b = lambda t: t[:, cut:]
    fin_f1 = O.bimamba2_sequential(a(x), a(dt), A, a(B), a(C), D=D, z=a(z), **kw)[2]
    fin_b2 = O.bimamba2_sequential(b(x), b(dt), A, b(B), b(C), D=D, z=b(z), **kw)[3]
    r1 = O.bimamba2_sequential(a(x), a(dt), A, a(B), a(C), D=D, z=a(z), initial_states_b=fin_b2, **kw)
    r2 = O.bimamba2_sequential(b(x), b(dt), A, b(B), b(C), D=D, z=b(z), initial_states_f=fin_f1, **kw)
    torch.testing.assert_close(torch.cat([r1[0], r2[0]], 1), full[0], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(r2[2], full[2], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(r1[3], full[3], rtol=1e-10, atol=1e-10)


def test_packed_sequences_equal_separate_runs():
    """The oracle's seq_idx: three sequences packed into one row give, piece by piece, what each gives on its own."""
    inp = to64(make_case(1, 40, 4, 3, 2, 5, with_z=True))
    x, dt, A, B, C, D, z, bias = (inp[k] for k in ("x", "dt", "A", "B", "C", "D", "z", "dt_bias"))
    kw = dict(dt_bias=bias, dt_softplus=True)
    bounds = [0, 13, 14, 40]
    seq_idx = torch.zeros(1, 40, dtype=torch.int64)
    for i in range(3):
        seq_idx[:, bounds[i]:bounds[i + 1]] = i
    packed = O.bimamba2_sequential(x, dt, A, B, C, D=D, z=z, seq_idx=seq_idx, **kw)[0]
    for i in range(3):
        s = slice(bounds[i], bounds[i + 1])
        alone = O.bimamba2_sequential(x[:, s], dt[:, s], A, B[:, s], C[:, s], D=D, z=z[:, s], **kw)[0]
        torch.testing.assert_close(packed[:, s], alone, rtol=1e-10, atol=1e-10)

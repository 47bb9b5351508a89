"""CPU oracle for the bidirectional SSD operator  y = SS(x) + flip(SS(flip(x))) + D*x  [* silu(z)].

THIS FILE IS TEST INFRASTRUCTURE.  Only tests, the smoke check and the benchmark's CPU-baseline leg may
import it; the shipped operator never does.  Everything here is plain torch on the CPU and works in
float64 (pass float64 tensors) so that it can serve as the "exact" side of a parity comparison.

Three independent statements of the forward math are kept side by side and cross-checked by the tests:

* ``bimamba2_sequential``  - the literal two-direction recurrence (formula: reference README.md:13-17;
  what "flip" covers and that D*x is added once: reference tests/fixtures/fwd.py:58-70).
* ``bimamba2_quadratic``   - the O(L^2) closed form (one masked decay matrix per direction).
* ``bimamba2_naive_chunked`` - the chunked causal SSD (math of reference src/ssd/uni/ssd_combined.py:621-659,
  src/ssd/uni/ssd_chunk_state.py:964-992, src/ssd/uni/ssd_state_passing.py:325-348,
  src/ssd/uni/ssd_chunk_scan.py:1791-1832) run on the inputs and on the sequence-flipped inputs and summed.
  This is also the function the benchmark times as the CPU baseline.

Gradients come from torch.autograd on any of the three (they are ordinary differentiable torch code).

The ``stage_*`` functions restate each intermediate of the chunked bidirectional algorithm (layouts as the
reference's stage wrappers return them) so that every device kernel can be checked on its own.

Pinning: the sequential form is checked against the C restatement in oracle/bimamba2_seq.c (different language,
scalar loops), the three forms against each other, against special cases with textbook answers (A = 0 turns
the operator into a plain masked matmul; a single constant channel turns it into a geometric series) and
against torch.autograd.gradcheck; see tests/test_oracle.py.  The extensions are pinned there as well:
``ssd_causal`` (the single-direction operator of the comparator) against the token-by-token recurrence written out in
the test and by "causal + flipped causal = bidirectional"; the initial states of ``bimamba2_sequential`` by the
cut-sequence identity (two pieces chained through their final states equal the uncut run); its ``seq_idx`` by "packed
sequences equal the same sequences run one by one".
"""
import math

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------------------
# dt preprocessing (reference src/ssd/bi/ssd_chunk_state.py:70-82, softplus: src/ssd/bi/softplus.py:8-17)
# --------------------------------------------------------------------------------------------------------
def dt_transform(dt, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """dt' = clamp(softplus?(dt + dt_bias), dt_min, dt_max); dt is (B, L, H)."""
    if dt_bias is not None:
        dt = dt + dt_bias.to(dt.dtype)
    if dt_softplus:
        dt = F.softplus(dt, beta=1.0, threshold=20.0)
    # the reference always applies min(max(dt, dt_min), dt_max), also with the default limits (0, inf):
    # without softplus a negative dt becomes 0 (and gets no gradient)
    return torch.clamp(dt, min=float(dt_limit[0]), max=float(dt_limit[1]))


def _expand_groups(t, nheads):
    """(B, L, G, N) -> (B, L, H, N), head h uses group h // (H/G)."""
    g = t.shape[2]
    return t.repeat_interleave(nheads // g, dim=2)


def _finish(y, x, D, z):
    if D is not None:
        Dv = D.to(y.dtype)
        y = y + x * (Dv[:, None] if Dv.dim() == 1 else Dv)
    out_x = y
    out = y if z is None else y * z * torch.sigmoid(z)
    return out, out_x


# --------------------------------------------------------------------------------------------------------
# 1. literal recurrence
# --------------------------------------------------------------------------------------------------------
def bimamba2_sequential(x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                        dt_limit=(0.0, float("inf")), initial_states_f=None, initial_states_b=None, seq_idx=None):
    """Returns (out, out_x, final_f, final_b).  Shapes: x (B,L,H,P), dt (B,L,H), A (H,), B/C (B,L,G,N).
    initial_states_f / _b (B,H,P,N): where the forward recurrence starts in front of position 0 resp. the reverse one
    behind position L-1 (zero when absent, as in the reference).  seq_idx (B,L) integers: sequences packed one behind
    the other; a recurrence restarts from zero wherever seq_idx changes (the causal reference's seq_idx semantics,
    src/ssd/uni/ssd_chunk_state.py:592-665 there, applied to both directions)."""
    bsz, L, H, P = x.shape
    dtp = dt_transform(dt, dt_bias, dt_softplus, dt_limit)
    Bh, Ch = _expand_groups(B, H), _expand_groups(C, H)
    N = Bh.shape[-1]
    decay = torch.exp(dtp * A.to(dtp.dtype))                       # (B, L, H)
    inj = (dtp[..., None, None] * x[..., :, None]) * Bh[..., None, :]  # (B, L, H, P, N)
    yf, yb = [None] * L, [None] * L
    h = x.new_zeros(bsz, H, P, N) if initial_states_f is None else initial_states_f
    for t in range(L):
        if seq_idx is not None and t > 0:
            h = h * (seq_idx[:, t] == seq_idx[:, t - 1]).to(h.dtype)[:, None, None, None]
        h = decay[:, t, :, None, None] * h + inj[:, t]
        yf[t] = (h * Ch[:, t, :, None, :]).sum(-1)
    final_f = h
    g = x.new_zeros(bsz, H, P, N) if initial_states_b is None else initial_states_b
    for t in range(L - 1, -1, -1):
        if seq_idx is not None and t < L - 1:
            g = g * (seq_idx[:, t] == seq_idx[:, t + 1]).to(g.dtype)[:, None, None, None]
        g = decay[:, t, :, None, None] * g + inj[:, t]
        yb[t] = (g * Ch[:, t, :, None, :]).sum(-1)
    final_b = g
    y = torch.stack(yf, 1) + torch.stack(yb, 1)
    out, out_x = _finish(y, x, D, z)
    return out, out_x, final_f, final_b


# --------------------------------------------------------------------------------------------------------
# 2. quadratic closed form
# --------------------------------------------------------------------------------------------------------
def bimamba2_quadratic(x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                       dt_limit=(0.0, float("inf"))):
    """Returns (out, out_x).  y_t = sum_s (C_t.B_s) M[t,s] dt'_s x_s + D x_t with
    M[t,s] = 1[s<=t] exp(sum_{r=s+1..t} a_r) + 1[s>=t] exp(sum_{r=t..s-1} a_r),  a = dt' * A."""
    bsz, L, H, P = x.shape
    dtp = dt_transform(dt, dt_bias, dt_softplus, dt_limit)
    a = (dtp * A.to(dtp.dtype)).permute(0, 2, 1)                   # (B, H, L)
    inc = torch.cumsum(a, -1)
    exc = inc - a
    tri_l = torch.tril(torch.ones(L, L, dtype=torch.bool))
    tri_u = torch.triu(torch.ones(L, L, dtype=torch.bool))
    df = inc[..., :, None] - inc[..., None, :]                      # [t, s] = sum_{s+1..t}
    db = exc[..., None, :] - exc[..., :, None]                      # [t, s] = sum_{t..s-1}
    ninf = torch.finfo(a.dtype).min
    M = torch.exp(df.masked_fill(~tri_l, ninf)) + torch.exp(db.masked_fill(~tri_u, ninf))
    Bh, Ch = _expand_groups(B, H), _expand_groups(C, H)
    cb = torch.einsum("bthn,bshn->bhts", Ch, Bh)
    y = torch.einsum("bhts,bsh,bshp->bthp", cb * M, dtp, x)
    return _finish(y, x, D, z)


# --------------------------------------------------------------------------------------------------------
# 3. chunked causal SSD, used twice (naive flip-and-sum); this is the CPU baseline
# --------------------------------------------------------------------------------------------------------
def ssd_causal_chunked(x, dtp, A, B, C, chunk_size):
    """Causal SSD on already transformed dt' (B, L, H): chunk states -> inter-chunk scan -> chunk outputs."""
    bsz, L, H, P = x.shape
    Q = chunk_size
    nc = (L + Q - 1) // Q
    pad = nc * Q - L
    if pad:
        x = F.pad(x, (0, 0, 0, 0, 0, pad))
        dtp = F.pad(dtp, (0, 0, 0, pad))
        B = F.pad(B, (0, 0, 0, 0, 0, pad))
        C = F.pad(C, (0, 0, 0, 0, 0, pad))
    Bh, Ch = _expand_groups(B, H), _expand_groups(C, H)
    N = Bh.shape[-1]
    xc = x.reshape(bsz, nc, Q, H, P)
    Bc = Bh.reshape(bsz, nc, Q, H, N)
    Cc = Ch.reshape(bsz, nc, Q, H, N)
    dtc = dtp.reshape(bsz, nc, Q, H).permute(0, 3, 1, 2)            # (B, H, nc, Q)
    cs = torch.cumsum(dtc * A.to(dtc.dtype)[None, :, None, None], -1)
    # chunk states: sum_k exp(cs[-1]-cs[k]) dt[k] x[k] (x) B[k]
    w = torch.exp(cs[..., -1:] - cs) * dtc
    states = torch.einsum("bclhn,bhcl,bclhp->bchpn", Bc, w, xc)
    # inter-chunk scan (sequential; nc is small)
    tot = cs[..., -1]                                               # (B, H, nc)
    prev = []
    s = x.new_zeros(bsz, H, P, N)
    for c in range(nc):
        prev.append(s)
        s = torch.exp(tot[:, :, c])[..., None, None] * s + states[:, c]
    prev = torch.stack(prev, 1)                                     # (B, nc, H, P, N)
    # chunk outputs
    seg = cs[..., :, None] - cs[..., None, :]                       # (B, H, nc, Q, Q)
    tri = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    Lmat = torch.exp(seg.masked_fill(~tri, torch.finfo(seg.dtype).min))
    cb = torch.einsum("bclhn,bcshn->bhcls", Cc, Bc)
    y = torch.einsum("bhcls,bhcs,bcshp->bclhp", cb * Lmat, dtc, xc)
    y = y + torch.einsum("bclhn,bchpn->bclhp", Cc, prev) * torch.exp(cs).permute(0, 2, 3, 1)[..., None]
    return y.reshape(bsz, nc * Q, H, P)[:, :L], s


def bimamba2_naive_chunked(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                           dt_limit=(0.0, float("inf"))):
    """Naive flip-and-sum path: two causal passes.  Returns (out, out_x, final_f, final_b)."""
    dtp = dt_transform(dt, dt_bias, dt_softplus, dt_limit)
    yf, final_f = ssd_causal_chunked(x, dtp, A, B, C, chunk_size)
    yb, final_b = ssd_causal_chunked(x.flip(1), dtp.flip(1), A, B.flip(1), C.flip(1), chunk_size)
    out, out_x = _finish(yf + yb.flip(1), x, D, z)
    return out, out_x, final_f, final_b


def ssd_causal(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """The single-direction operator y = SS(x) + D*x (gated by silu(z)): one causal pass of the naive path above (math of
    the reference's ssd_chunk_scan_combined_ref, src/ssd/uni/ssd_combined.py:621-659).  Returns (out, out_x, final).
    It is what the causal comparator of the HIP path is checked against."""
    dtp = dt_transform(dt, dt_bias, dt_softplus, dt_limit)
    y, final = ssd_causal_chunked(x, dtp, A, B, C, chunk_size)
    out, out_x = _finish(y, x, D, z)
    return out, out_x, final


# --------------------------------------------------------------------------------------------------------
# per-stage restatements of the chunked bidirectional algorithm (layouts of the reference stage wrappers)
# --------------------------------------------------------------------------------------------------------
def _chunks(L, Q):
    return (L + Q - 1) // Q


def _pad_seq(t, nc, Q):
    pad = nc * Q - t.shape[1]
    if pad:
        t = F.pad(t, (0, 0) * (t.dim() - 2) + (0, pad))
    return t


def stage_chunk_cumsum(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """-> dt_out, cs_f, cs_b each (B, H, nc, Q); padding positions have dt_out = 0
    (reference src/ssd/bi/ssd_chunk_state.py:35-91)."""
    bsz, L, H = dt.shape
    Q = chunk_size
    nc = _chunks(L, Q)
    dtp = dt_transform(dt, dt_bias, dt_softplus, dt_limit)
    dtp = _pad_seq(dtp, nc, Q).reshape(bsz, nc, Q, H).permute(0, 3, 1, 2)
    dA = dtp * A.to(dtp.dtype)[None, :, None, None]
    cs_f = torch.cumsum(dA, -1)
    cs_b = torch.cumsum(dA.flip(-1), -1).flip(-1)
    return dtp.contiguous(), cs_f, cs_b


def stage_bmm_chunk(C, B, chunk_size):
    """CB[b,c,g,l,s] = C_l . B_s inside chunk c (reference src/ssd/bi/ssd_bmm.py:35-91)."""
    bsz, L, G, N = B.shape
    Q = chunk_size
    nc = _chunks(L, Q)
    Bc = _pad_seq(B, nc, Q).reshape(bsz, nc, Q, G, N)
    Cc = _pad_seq(C, nc, Q).reshape(bsz, nc, Q, G, N)
    return torch.einsum("bclgn,bcsgn->bcgls", Cc, Bc)


def stage_chunk_state(B, x, dt_out, cs_f, cs_b):
    """-> S_f, S_b (B, nc, H, P, N) (reference src/ssd/bi/ssd_chunk_state.py:188-263)."""
    bsz, L, H, P = x.shape
    _, _, nc, Q = dt_out.shape
    Bc = _pad_seq(_expand_groups(B, H), nc, Q).reshape(bsz, nc, Q, H, -1)
    xc = _pad_seq(x, nc, Q).reshape(bsz, nc, Q, H, P)
    wf = torch.exp(cs_f[..., -1:] - cs_f) * dt_out
    wb = torch.exp(cs_b[..., :1] - cs_b) * dt_out
    S_f = torch.einsum("bclhn,bhcl,bclhp->bchpn", Bc, wf, xc)
    S_b = torch.einsum("bclhn,bhcl,bclhp->bchpn", Bc, wb, xc)
    return S_f, S_b


def stage_state_passing(S_f, S_b, cs_f, cs_b):
    """-> prev_f, prev_b (B, nc, H, P, N), final_f, final_b (B, H, P, N)
    (reference src/ssd/bi/ssd_state_passing.py:28-92)."""
    bsz, nc = S_f.shape[:2]
    tot = cs_f[..., -1]                      # equals cs_b[..., 0]
    prev_f, prev_b = [None] * nc, [None] * nc
    s = torch.zeros_like(S_f[:, 0])
    for c in range(nc):
        prev_f[c] = s
        s = torch.exp(tot[:, :, c])[..., None, None] * s + S_f[:, c]
    final_f = s
    s = torch.zeros_like(S_b[:, 0])
    for c in range(nc - 1, -1, -1):
        prev_b[c] = s
        s = torch.exp(cs_b[:, :, c, 0])[..., None, None] * s + S_b[:, c]
    final_b = s
    return torch.stack(prev_f, 1), torch.stack(prev_b, 1), final_f, final_b


def _intra_mask(cs_f, cs_b):
    """M[b,h,c,t,s] = 1[s<=t] e^{cs_f[t]-cs_f[s]} + 1[s>=t] e^{cs_b[t]-cs_b[s]}."""
    Q = cs_f.shape[-1]
    tri_l = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    tri_u = torch.triu(torch.ones(Q, Q, dtype=torch.bool))
    ninf = torch.finfo(cs_f.dtype).min
    df = (cs_f[..., :, None] - cs_f[..., None, :]).masked_fill(~tri_l, ninf)
    db = (cs_b[..., :, None] - cs_b[..., None, :]).masked_fill(~tri_u, ninf)
    return torch.exp(df), torch.exp(db)


def stage_chunk_scan(CB, x, dt_out, cs_f, cs_b, C, prev_f, prev_b, D=None, z=None):
    """-> out, out_x (B, L, H, P) (reference src/ssd/bi/ssd_chunk_scan.py:43-189)."""
    bsz, L, H, P = x.shape
    _, _, nc, Q = dt_out.shape
    G = C.shape[2]
    xc = _pad_seq(x, nc, Q).reshape(bsz, nc, Q, H, P)
    Cc = _pad_seq(_expand_groups(C, H), nc, Q).reshape(bsz, nc, Q, H, -1)
    Mf, Mb = _intra_mask(cs_f, cs_b)
    cbh = CB.repeat_interleave(H // G, dim=2).permute(0, 2, 1, 3, 4)   # (B, H, nc, Q, Q)
    y = torch.einsum("bhcts,bhcs,bcshp->bcthp", cbh * (Mf + Mb), dt_out, xc)
    y = y + torch.einsum("bclhn,bchpn->bclhp", Cc, prev_f) * torch.exp(cs_f).permute(0, 2, 3, 1)[..., None]
    y = y + torch.einsum("bclhn,bchpn->bclhp", Cc, prev_b) * torch.exp(cs_b).permute(0, 2, 3, 1)[..., None]
    y = y.reshape(bsz, nc * Q, H, P)[:, :L]
    return _finish(y, x, D, z)


def bimamba2_staged(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                    dt_limit=(0.0, float("inf"))):
    """The chunked bidirectional algorithm composed from the stage functions.
    Returns (out, out_x, final_f, final_b)."""
    dt_out, cs_f, cs_b = stage_chunk_cumsum(dt, A, chunk_size, dt_bias, dt_softplus, dt_limit)
    S_f, S_b = stage_chunk_state(B, x, dt_out, cs_f, cs_b)
    prev_f, prev_b, final_f, final_b = stage_state_passing(S_f, S_b, cs_f, cs_b)
    CB = stage_bmm_chunk(C, B, chunk_size)
    out, out_x = stage_chunk_scan(CB, x, dt_out, cs_f, cs_b, C, prev_f, prev_b, D, z)
    return out, out_x, final_f, final_b


# --------------------------------------------------------------------------------------------------------
# convenience: full set of gradients through autograd of the quadratic form
# --------------------------------------------------------------------------------------------------------
def bimamba2_grads(dout, x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                   dt_limit=(0.0, float("inf")), form="quadratic", chunk_size=None):
    """Returns dict with out and the gradients dx, ddt, dA, dB, dC, dD, dz, ddt_bias (None where absent)."""
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias"]
    vals = [x, dt, A, B, C, D, z, dt_bias]
    leaves = [None if v is None else v.detach().clone().requires_grad_(True) for v in vals]
    kw = dict(D=leaves[5], z=leaves[6], dt_bias=leaves[7], dt_softplus=dt_softplus, dt_limit=dt_limit)
    if form == "quadratic":
        out = bimamba2_quadratic(*leaves[:5], **kw)[0]
    elif form == "sequential":
        out = bimamba2_sequential(*leaves[:5], **kw)[0]
    elif form == "causal":
        out = ssd_causal(*leaves[:5], chunk_size, **kw)[0]
    else:
        out = bimamba2_naive_chunked(*leaves[:5], chunk_size, **kw)[0]
    present = [l for l in leaves if l is not None]
    grads = torch.autograd.grad(out, present, dout)
    res = {"out": out.detach()}
    it = iter(grads)
    for n, l in zip(names, leaves):
        res["d" + n] = None if l is None else next(it)
    return res


def make_inputs(batch, seqlen, nheads, headdim, ngroups, dstate, seed=0, dtype=torch.float32,
                with_z=False, with_D=True, D_has_hdim=False, generator=None):
    """Synthetic inputs with the benchmark distributions: x, B, C, z ~ N(0,1); A = -exp(U(log 1, log 16));
    dt ~ N(0, 0.5); dt_bias = inverse softplus of log-uniform[1e-3, 1e-1]; D ~ N(0,1).
    x, B, C, z are rounded to `dtype`; dt, A, D, dt_bias stay float32."""
    g = generator or torch.Generator().manual_seed(seed)
    x = torch.randn(batch, seqlen, nheads, headdim, generator=g).to(dtype)
    dt = 0.5 * torch.randn(batch, seqlen, nheads, generator=g)
    A = -torch.exp(torch.rand(nheads, generator=g) * math.log(16.0))
    B = torch.randn(batch, seqlen, ngroups, dstate, generator=g).to(dtype)
    C = torch.randn(batch, seqlen, ngroups, dstate, generator=g).to(dtype)
    dt0 = torch.exp(torch.rand(nheads, generator=g) * (math.log(1e-1) - math.log(1e-3)) + math.log(1e-3))
    dt_bias = dt0 + torch.log(-torch.expm1(-dt0))
    D = None
    if with_D:
        D = torch.randn((nheads, headdim) if D_has_hdim else (nheads,), generator=g)
    z = torch.randn(batch, seqlen, nheads, headdim, generator=g).to(dtype) if with_z else None
    return dict(x=x, dt=dt, A=A, B=B, C=C, D=D, z=z, dt_bias=dt_bias)

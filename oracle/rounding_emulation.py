"""The chunked bidirectional algorithm, forward and backward, written out stage by stage as explicit contractions, with a
switch that rounds where the REFERENCE's kernels round.

THIS FILE IS TEST INFRASTRUCTURE (imported by tests only).

Purpose.  The parity contract for 16-bit inputs is rtol = atol = 2e-2 against the float64 math.  A 16-bit implementation
cannot be exact: every matrix product takes operands rounded to the 16-bit type.  What error that leaves in each output and
gradient is a property of WHERE the roundings sit, and the reference fixes those places.  This module restates the
reference's stage math with exactly its rounding points, so that the size of "the reference's own error against the exact
math" can be measured per tensor on any input and put beside the HIP path's error (tests/test_rounding_emulation.py,
tests/test_gpu_rounding_envelope.py).  With rounding switched off (dtype=None) every quantity is exact float64, and the
gradients must then equal torch.autograd through the oracle's closed form - that check pins the hand-written backward
formulas below (a dropped term or a transposed index fails it).

Rounding points restated (T = the 16-bit type of x, B, C, z, dout; accumulation is float32 in the reference, float64 here -
the accumulation error is far below the operand rounding), paths relative to the reference's root:
  forward   scaled B -> T before the chunk-state product                       src/ssd/bi/ssd_chunk_state.py:243-244
            states entering the chunks -> T (out_dtype=C.dtype)                src/ssd/bi/ssd_combined.py:324-327
            masked, decayed cb * dt -> T before the product with x             src/ssd/bi/ssd_chunk_scan.py:156
            out_x, out -> T                                                    src/ssd/bi/ssd_chunk_scan.py:176-189
  backward  dout * silu(z) -> T (the dout every later kernel reads), dz -> T   src/ssd/bi/ssd_chunk_scan.py:419-440
            dout * decay -> T before the dstates product                       src/ssd/bi/ssd_chunk_scan.py:503-504
            dstates, states -> T after the backward state passing              src/ssd/bi/ssd_combined.py:392-408
            masked, decayed cb^T -> T before the product with dout; dx -> T    src/ssd/bi/ssd_combined.py:197-208
            dCB -> T inside the bmm backward (dout.to(a.dtype))                src/ssd/bi/ssd_bmm.py:143
            dB, dC -> T                                                        src/ssd/bi/ssd_combined.py:441-442
  (dt, A, D, dt_bias, the cumulative sums and every ddA / ddt term stay float32 in the reference: not rounded here.)
"""
import torch
import torch.nn.functional as F

from . import bimamba2_oracle as O


def _rounder(dtype):
    if dtype is None:
        return lambda t: t
    return lambda t: t.to(dtype).to(torch.float64)


def reference_rounded(dout, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, dt_softplus=False,
                      dt_limit=(0.0, float("inf")), dtype=torch.bfloat16):
    """All inputs float64 (x, B, C, z, dout holding values already representable in `dtype`).  Returns a dict with out and
    dx, ddt, dA, dB, dC, dD, dz, ddt_bias as the reference's chunked algorithm produces them when its matrix-product
    operands and stored tensors are rounded to `dtype` (None: no rounding, exact)."""
    rd = _rounder(dtype)
    bsz, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    Q = chunk_size
    nc = (L + Q - 1) // Q
    hpg = H // G
    pad = lambda t: O._pad_seq(t, nc, Q)
    # ---- dt transform and cumulative sums (float32 in the reference: kept exact here) ----
    dt_raw = dt if dt_bias is None else dt + dt_bias
    dt_out, cs_f, cs_b = O.stage_chunk_cumsum(dt, A, Q, dt_bias, dt_softplus, dt_limit)         # (B, H, nc, Q)
    valid = (torch.arange(nc * Q).reshape(nc, Q) < L).to(x.dtype)                              # (nc, Q)
    xc = pad(x).reshape(bsz, nc, Q, H, P)
    Bc = pad(O._expand_groups(B, H)).reshape(bsz, nc, Q, H, N)
    Cc = pad(O._expand_groups(C, H)).reshape(bsz, nc, Q, H, N)
    tot = cs_f[..., -1]                                                                          # (B, H, nc) = cs_b[..., 0]
    wf = torch.exp(cs_f[..., -1:] - cs_f) * dt_out                                               # chunk-state weights
    wb = torch.exp(cs_b[..., :1] - cs_b) * dt_out
    ef = torch.exp(cs_f).permute(0, 2, 3, 1)                                                     # (B, nc, Q, H): e^{cs_f[m]}
    eb = torch.exp(cs_b).permute(0, 2, 3, 1)
    # ---- forward ----
    Bf = rd(Bc * wf.permute(0, 2, 3, 1)[..., None])                                              # scaled B -> T
    Bb = rd(Bc * wb.permute(0, 2, 3, 1)[..., None])
    S_f = torch.einsum("bclhn,bclhp->bchpn", Bf, xc)
    S_b = torch.einsum("bclhn,bclhp->bchpn", Bb, xc)
    prev_f, prev_b, _, _ = O.stage_state_passing(S_f, S_b, cs_f, cs_b)                           # float32 recurrence
    P_f, P_b = rd(prev_f), rd(prev_b)                                                            # entering states -> T
    CBh = torch.einsum("bclhn,bcshn->bhcls", Cc, Bc)                                             # (B, H, nc, Q, Q) per head
    Mf, Mb = O._intra_mask(cs_f, cs_b)
    Mt = (Mf + Mb) * (valid[None, None, :, :, None] * valid[None, None, :, None, :])
    cbm = rd(CBh * Mt * dt_out[..., None, :])                                                    # masked cb * dt -> T
    acc = torch.einsum("bhcts,bcshp->bcthp", cbm, xc)
    acc = acc + torch.einsum("bclhn,bchpn->bclhp", Cc, P_f) * ef[..., None]
    acc = acc + torch.einsum("bclhn,bchpn->bclhp", Cc, P_b) * eb[..., None]
    y = acc.reshape(bsz, nc * Q, H, P)[:, :L]
    if D is not None:
        y = y + x * (D[:, None] if D.dim() == 1 else D)
    out_x = rd(y)
    out = rd(y * z * torch.sigmoid(z)) if z is not None else out_x
    # ---- backward ----
    dz = None
    if z is not None:
        sg = torch.sigmoid(z)
        dz = rd(dout * out_x * sg * (1 + z * (1 - sg)))
        dy32 = dout * z * sg                                                                     # float32 in the reference's dz kernel
        dy = rd(dy32)                                                                            # what every later kernel reads
    else:
        dy32 = dy = dout
    dD = None
    if D is not None:
        dD = (dy32 * x).sum((0, 1)) if D.dim() == 2 else (dy32 * x).sum((0, 1, 3))
    dyc = pad(dy).reshape(bsz, nc, Q, H, P)
    # dstates: gradient with respect to the states entering each chunk, dout * decay -> T
    dP_f = torch.einsum("bclhp,bclhn->bchpn", rd(dyc * ef[..., None]), Cc)
    dP_b = torch.einsum("bclhp,bclhn->bchpn", rd(dyc * eb[..., None]), Cc)
    # backward state passing (float32): gradient with respect to each chunk's own state, and the chunk-decay terms
    dS_f, dS_b = [None] * nc, [None] * nc
    ddA_chunk_f, ddA_chunk_b = torch.zeros_like(tot), torch.zeros_like(tot)
    g = torch.zeros_like(dP_f[:, 0])
    for c in range(nc - 1, -1, -1):          # forward direction: chunk c's state feeds chunks c+1..
        dS_f[c] = g
        d = torch.exp(tot[:, :, c])[..., None, None]
        ddA_chunk_f[:, :, c] = (g * prev_f[:, c] * d).sum((-1, -2))
        g = dP_f[:, c] + d * g
    g = torch.zeros_like(dP_b[:, 0])
    for c in range(nc):                      # reverse direction: chunk c's state feeds chunks c-1..
        dS_b[c] = g
        d = torch.exp(tot[:, :, c])[..., None, None]
        ddA_chunk_b[:, :, c] = (g * prev_b[:, c] * d).sum((-1, -2))
        g = dP_b[:, c] + d * g
    dS_f, dS_b = rd(torch.stack(dS_f, 1)), rd(torch.stack(dS_b, 1))                              # -> T
    # dx, ddt_direct
    sf = torch.exp(cs_f[..., -1:] - cs_f).permute(0, 2, 3, 1)                                    # (B, nc, Q, H): e^{cs_f[Q-1]-cs_f[m]}
    sb = torch.exp(cs_b[..., :1] - cs_b).permute(0, 2, 3, 1)
    accx = torch.einsum("bcmhn,bchpn->bcmhp", Bc, dS_f) * sf[..., None] + torch.einsum("bcmhn,bchpn->bcmhp", Bc, dS_b) * sb[..., None]
    cbt = rd((CBh * Mt).transpose(-1, -2))                                                       # [m, k] = CB[k, m] (decay of (k, m)) -> T
    accx = accx + torch.einsum("bhcmk,bckhp->bcmhp", cbt, dyc)
    dtq = dt_out.permute(0, 2, 3, 1)                                                             # (B, nc, Q, H)
    dxc = accx * dtq[..., None]
    dx = dxc.reshape(bsz, nc * Q, H, P)[:, :L]
    if D is not None:
        dx = dx + dy * (D[:, None] if D.dim() == 1 else D)
    dx = rd(dx)
    ddt_direct = (accx * xc).sum(-1)                                                             # (B, nc, Q, H)
    # dB (state part) and its decay terms; dC (state part) and its decay terms
    db_f = torch.einsum("bcmhp,bchpn->bcmhn", xc, dS_f) * (sf * dtq)[..., None]
    db_b = torch.einsum("bcmhp,bchpn->bcmhn", xc, dS_b) * (sb * dtq)[..., None]
    v_f, v_b = (db_f * Bc).sum(-1), (db_b * Bc).sum(-1)                                          # per position; ddA_next = exclusive prefix / suffix sums
    dc_f = torch.einsum("bcmhp,bchpn->bcmhn", dyc, P_f) * ef[..., None]
    dc_b = torch.einsum("bcmhp,bchpn->bcmhn", dyc, P_b) * eb[..., None]
    u_f, u_b = (dc_f * Cc).sum(-1), (dc_b * Cc).sum(-1)
    # dCB and the within-chunk decay terms from G = dout . x^T
    Gm = torch.einsum("bcthp,bcshp->bhcts", dyc, xc)
    dCBh = Gm * Mt * dt_out[..., None, :]                                                        # per head, float32
    dCB = dCBh.reshape(bsz, G, hpg, nc, Q, Q).sum(2)                                             # (B, G, nc, Q, Q)
    dCB16 = rd(dCB)                                                                              # -> T inside the bmm backward
    Bg = pad(B).reshape(bsz, nc, Q, G, N)
    Cg = pad(C).reshape(bsz, nc, Q, G, N)
    dB = torch.einsum("bgcts,bctgn->bcsgn", dCB16, Cg) + (db_f + db_b).reshape(bsz, nc, Q, G, hpg, N).sum(4)
    dC = torch.einsum("bgcts,bcsgn->bctgn", dCB16, Bg) + (dc_f + dc_b).reshape(bsz, nc, Q, G, hpg, N).sum(4)
    dB = rd(dB.reshape(bsz, nc * Q, G, N)[:, :L])
    dC = rd(dC.reshape(bsz, nc * Q, G, N)[:, :L])
    # d(dt*A) per position: every decay exponent is a sum of a = dt*A over a range of positions
    Wf = Gm * CBh * Mf * dt_out[..., None, :] * (valid[None, None, :, :, None] * valid[None, None, :, None, :])
    Wb = Gm * CBh * Mb * dt_out[..., None, :] * (valid[None, None, :, :, None] * valid[None, None, :, None, :])
    idx = torch.arange(Q)
    strict_l = (idx[:, None] > idx[None, :]).to(x.dtype)                                         # s < t
    strict_u = (idx[:, None] < idx[None, :]).to(x.dtype)
    Wf, Wb = Wf * strict_l, Wb * strict_u
    # forward pairs (t, s), s < t, carry e^{a_{s+1} + .. + a_t}: position r gets sum over s < r <= t
    colf = Wf.sum(-2)                                   # by s
    rowf = Wf.sum(-1)                                   # by t
    ddA_intra_f = torch.cumsum(colf - rowf, -1) - (colf - rowf)                                  # exclusive prefix of (col - row)
    # reverse pairs (t, s), s > t, carry e^{a_t + .. + a_{s-1}}: position r gets sum over t <= r < s
    colb = Wb.sum(-2)
    rowb = Wb.sum(-1)
    dlt = colb - rowb
    ddA_intra_b = torch.flip(torch.cumsum(torch.flip(dlt, (-1,)), -1), (-1,)) - dlt              # exclusive suffix of (col - row)
    # state terms: u (entering state read at position m: e^{cs_f[m]} = sum over positions <= m; e^{cs_b[m]} = positions >= m),
    # v (position m written into the chunk state: e^{cs_f[Q-1]-cs_f[m]} = positions > m; e^{cs_b[0]-cs_b[m]} = positions < m),
    # and the chunk totals of the inter-chunk recurrences (every position of the chunk)
    uf, ub = u_f.permute(0, 3, 1, 2), u_b.permute(0, 3, 1, 2)                                    # (B, H, nc, Q)
    vf, vb = v_f.permute(0, 3, 1, 2), v_b.permute(0, 3, 1, 2)
    rev = lambda t: torch.flip(torch.cumsum(torch.flip(t, (-1,)), -1), (-1,))
    ddA = ddA_intra_f + ddA_intra_b
    ddA = ddA + rev(uf) + torch.cumsum(ub, -1)                                                   # inclusive suffix / prefix
    ddA = ddA + (torch.cumsum(vf, -1) - vf) + (rev(vb) - vb)                                     # exclusive prefix / suffix
    ddA = ddA + (ddA_chunk_f + ddA_chunk_b)[..., None]
    # through the dt transform (reference src/ssd/bi/ssd_chunk_state.py:145-170)
    ddtp = ddA * A[None, :, None, None] + ddt_direct.permute(0, 3, 1, 2)                         # d / d(dt')
    dA = (ddA * dt_out).sum((0, 2, 3))
    ddtp = ddtp.permute(0, 2, 3, 1).reshape(bsz, nc * Q, H)[:, :L]
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    pre = dt_raw
    act = F.softplus(pre, beta=1.0, threshold=20.0) if dt_softplus else pre
    inside = ((act >= lo) & (act <= hi)).to(x.dtype)
    ddt = ddtp * inside
    if dt_softplus:
        ddt = ddt * torch.where(pre <= 20.0, torch.sigmoid(pre), torch.ones_like(pre))
    ddt_bias = ddt.sum((0, 1)) if dt_bias is not None else None
    return {"out": out, "dx": dx, "ddt": ddt, "dA": dA, "dB": dB, "dC": dC, "dD": dD, "dz": dz, "ddt_bias": ddt_bias}

"""GPU parity on the smallest and most ragged shapes: one position, a sequence shorter than a chunk on the fast-path
kernels (one partly filled chunk), a last chunk of one position, forward and backward; and the shapes beyond the kernels'
limits that the public function takes apart (heads wider than 128 channels, chunks longer than 256)."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, is_reduced, make_case, to64, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z
    (1, 1, 2, 16, 1, 8, 32, torch.float32, False),
    (2, 7, 2, 32, 2, 16, 64, torch.float32, True),
    (1, 1, 2, 64, 1, 64, 256, torch.bfloat16, True),          # fast-path kernels, one position
    (2, 40, 4, 64, 1, 64, 256, torch.bfloat16, True),         # fast-path kernels, 40 of 256 positions
    (1, 257, 2, 64, 1, 64, 256, torch.bfloat16, False),       # last chunk holds one position
    (1, 65, 2, 128, 2, 64, 64, torch.float16, True),          # two headdim tiles, last chunk of one position
]


@pytest.mark.parametrize("case", CASES)
def test_tiny_and_ragged_shapes(case):
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q, dtype, z = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z)
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    out.backward(dout.cuda())
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True)
    assert_close(out, ref["out"], dtype, "out")
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if ref["d" + k] is not None:
            assert_close(leaves[k].grad, ref["d" + k], dtype, "d" + k, scaled=is_reduced("d" + k, dtype))


WIDE = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z, D with headdim, final states
    (2, 100, 2, 256, 1, 16, 64, torch.float32, True, True, False),       # heads of 256 channels: two pieces of 128
    (1, 300, 4, 192, 2, 64, 128, torch.bfloat16, False, False, True),    # 192 channels: two pieces of 96; final states
    (1, 700, 2, 64, 1, 32, 512, torch.float32, True, False, False),      # chunk_size above the kernels' 256
    (1, 200, 2, 32, 1, 320, 64, torch.float32, True, False, True),       # dstate above the kernels' 256: pieces of 256 + 64
    (1, 300, 4, 64, 2, 384, 128, torch.bfloat16, True, True, False),     # the same in bf16: 256 + 128
]


@pytest.mark.parametrize("case", WIDE)
def test_heads_wider_and_chunks_longer_than_the_kernels(case):
    """Shapes the reference accepts beyond the kernels' limits (headdim > 128, chunk_size > 256, dstate > 256): the public
    function splits wide heads into narrower ones that share dt, A, dt_bias (and D), caps the chunk size (the result does
    not depend on it) and sums over pieces of a wide state dimension; output, final states and every gradient against the
    oracle at the shape the caller gave."""
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q, dtype, z, Dhp, fin = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z, D_has_hdim=Dhp)
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    res = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True, return_final_states=fin)
    out = res[0] if fin else res
    assert out.shape == (b, L, H, P)
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    out.backward(dout.cuda())
    r = to64(inp)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True)
    assert_close(out, ref["out"], dtype, "out")
    if fin:
        assert res[1].shape == (b, H, P, N) and res[2].shape == (b, H, P, N)
        rf = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"], dt_softplus=True)
        assert_close(res[1], rf[2], dtype, "final_f")
        assert_close(res[2], rf[3], dtype, "final_b")
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if ref["d" + k] is not None:
            assert leaves[k].grad.shape == leaves[k].shape
            # (dx of the 16-bit case: sums of up to 22 from operands with 8 bits of mantissa leave one element in 230000
            # at 1.17 x the plain bound; the criterion of the summed gradients, as in test_gpu_scan16_shapes.py)
            assert_close(leaves[k].grad, ref["d" + k], dtype, "d" + k,
                         scaled=is_reduced("d" + k, dtype) or (k == "x" and dtype != torch.float32))


BIG = [
    # batch, seqlen, H, P, G, N, z: x, z, dout and their gradients pass 2^31 elements inside the last batch row ...
    (9, 65536, 64, 64, 1, 64, True),
    # ... and here the per-chunk states (batch * nchunks * H * P * N) do too, on the kernels for other shapes
    (9, 65536, 64, 128, 2, 128, False),
]


@pytest.mark.parametrize("case", BIG)
def test_offsets_beyond_32_bits(case):
    """The last batch row of a problem whose tensors hold more than 2^31 elements must come out exactly as the same row
    computed alone (no workgroup works on more than one batch row, so every sum has the same order): an element offset
    that wraps at 32 bits anywhere in the forward or backward kernels breaks this."""
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, with_z = case
    dtype, Q = torch.bfloat16, 256
    g = torch.Generator(device="cuda").manual_seed(11)
    rn = lambda *s: torch.randn(*s, device="cuda", dtype=dtype, generator=g)
    x, Bm, Cm, dout = rn(b, L, H, P), rn(b, L, G, N), rn(b, L, G, N), rn(b, L, H, P)
    z = rn(b, L, H, P) if with_z else None
    dt = rn(b, L, H)
    A = -torch.rand(H, device="cuda", generator=g) - 0.5
    D = torch.randn(H, device="cuda", generator=g)
    dt_bias = torch.randn(H, device="cuda", generator=g) * 0.1 - 3.0
    assert x.numel() > 2 ** 31

    def run(sl):
        leaves = [t[sl].detach().requires_grad_(True) if t is not None else None for t in (x, dt, Bm, Cm, z)]
        out = ops.bimamba_chunk_scan_combined(leaves[0], leaves[1], A, leaves[2], leaves[3], Q, D=D, z=leaves[4],
                                              dt_bias=dt_bias, dt_softplus=True)
        grads = torch.autograd.grad(out, [t for t in leaves if t is not None], dout[sl])
        return [out.detach()] + list(grads)

    last = slice(b - 1, b)
    alone = run(last)
    full = run(slice(0, b))
    names = ["out", "dx", "ddt", "dB", "dC"] + (["dz"] if with_z else [])
    for name, f, a in zip(names, full, alone):
        assert torch.isfinite(a.float()).all(), name
        assert a.float().abs().max() > 0, name
        assert torch.equal(f[last], a), f"{name}: the last batch row differs from the same row computed alone"


def test_gradient_destinations_that_break_the_kernels_alignment_are_not_used():
    """grad_places at a 16-bit fast-path shape: slices of a wider buffer at an odd element offset (not 16-byte aligned) for
    dx, dB and dC.  The forward kept only the 16-bit copies of the entering states, which the aligned kernels read, so such
    a destination must be declined (fresh gradients through autograd), not turned into an unsupported-kernel error; aligned
    slices of the same buffer are written in place.  Both against the oracle."""
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q, dtype = 1, 300, 2, 64, 1, 64, 256, torch.bfloat16
    inp = make_case(b, L, H, P, G, N, dtype, with_z=True)
    r = to64(inp)
    dout = torch.randn(b, L, H, P, generator=torch.Generator().manual_seed(5)).to(dtype)
    ref = O.bimamba2_grads(dout.double(), r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                           dt_softplus=True)
    width = H * P + 2 * G * N
    for shift, in_place in ((3, False), (8, True)):
        d = to_dev(inp)
        leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
        buf = torch.zeros(b, L, width + 16, device="cuda", dtype=dtype)
        cuts = {"dx": (shift, H * P, (H, P)), "dB": (shift + H * P, G * N, (G, N)), "dC": (shift + H * P + G * N, G * N, (G, N))}
        places = {k: (lambda o=o, n=n, sh=sh: buf[..., o:o + n].unflatten(-1, sh)) for k, (o, n, sh) in cuts.items()}
        out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                              z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True, grad_places=places)
        out.backward(dout.cuda())
        for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
            assert_close(leaves[k].grad, ref["d" + k], dtype, f"d{k} (offset {shift})", scaled=is_reduced("d" + k, dtype) or k == "x")
        # (autograd clones a strided gradient into .grad, so the buffer itself tells whether the kernels wrote into it)
        for k, name in (("x", "dx"), ("B", "dB"), ("C", "dC")):
            if in_place:
                assert torch.equal(places[name](), leaves[k].grad), (name, shift)
            else:
                assert not places[name]().any(), (name, shift)

"""GPU parity of packed sequences (seq_idx), forward and backward, against float64 autograd on the oracle's recurrence
with restarts, and against running the packed sequences one by one."""
import pytest
import torch

from oracle import bimamba2_oracle as O
from tests.helpers import assert_close, is_reduced, make_case, to64, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from bi_mamba2_amd import ops
    return ops


def _seq_idx(batch, L, bounds_per_row):
    si = torch.zeros(batch, L, dtype=torch.int32)
    for b, bounds in enumerate(bounds_per_row):
        edges = [0] + list(bounds) + [L]
        for i in range(len(edges) - 1):
            si[b, edges[i]:edges[i + 1]] = i
    return si


CASES = [
    # batch, seqlen, H, P, G, N, chunk, dtype, z, boundaries per row (incl. chunk edges, a one-token sequence, none)
    (2, 100, 4, 16, 2, 8, 32, torch.float32, False, [(17, 32, 33, 64), ()]),
    (2, 300, 4, 64, 2, 64, 128, torch.bfloat16, True, [(128, 200), (1, 255, 256, 299)]),
    (1, 512, 8, 64, 1, 64, 256, torch.bfloat16, False, [(100, 256, 300)]),
    # many short sequences inside one chunk: 32 (float32) resp. 42 (bf16) boundaries per 256 positions, every one adding its cut to the
    # chunk's cumulative sums
    (2, 512, 4, 32, 2, 16, 256, torch.float32, False, [tuple(range(8, 264, 8)), tuple(range(4, 512, 8))]),
    (1, 512, 4, 64, 1, 64, 256, torch.bfloat16, True, [tuple(range(6, 510, 6))]),
    # more boundaries per 256 positions than the mechanism resolves in one chunk (64: sequences of 4 tokens; 255: every token
    # a sequence of its own): the host side runs these with a smaller chunk, float32 still held to the plain 1e-4
    (1, 512, 4, 32, 2, 16, 256, torch.float32, False, [tuple(range(4, 512, 4))]),
    (2, 256, 2, 16, 1, 8, 256, torch.float32, True, [tuple(range(1, 256)), tuple(range(2, 256, 2))]),
]


@pytest.mark.parametrize("case", CASES)
def test_packed_sequences_forward_and_backward(ops, case):
    b, L, H, P, G, N, Q, dtype, z, bounds = case
    inp = make_case(b, L, H, P, G, N, dtype, with_z=z)
    si = _seq_idx(b, L, bounds)
    d = to_dev(inp)
    leaves = {k: (v.clone().requires_grad_(True) if v is not None else None) for k, v in d.items()}
    out = ops.bimamba_chunk_scan_combined(leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], Q, D=leaves["D"],
                                          z=leaves["z"], dt_bias=leaves["dt_bias"], dt_softplus=True, seq_idx=si.cuda())
    dout = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).to(out.dtype)
    out.backward(dout.cuda())
    r = {k: (v.clone().requires_grad_(True) if torch.is_tensor(v) else v) for k, v in to64(inp).items()}
    ro = O.bimamba2_sequential(r["x"], r["dt"], r["A"], r["B"], r["C"], D=r["D"], z=r["z"], dt_bias=r["dt_bias"],
                               dt_softplus=True, seq_idx=si.long())[0]
    ro.backward(dout.double())
    # 16-bit cases: outputs up to 40 from operands rounded to 8 bits of mantissa leave a few elements per 100000 beyond the
    # plain bound (the same without seq_idx)
    big = dtype != torch.float32
    assert_close(out, ro, dtype, "out", scaled=big)
    for k in ("x", "B", "C", "z", "dt", "A", "D", "dt_bias"):
        if r[k] is not None:
            assert_close(leaves[k].grad, r[k].grad, dtype, "d" + k, scaled=is_reduced("d" + k, dtype))


def test_packed_equals_one_by_one(ops):
    b, L, H, P, G, N, Q, dtype = 1, 768, 8, 64, 1, 64, 256, torch.bfloat16
    d = to_dev(make_case(b, L, H, P, G, N, dtype, with_z=True))
    edges = [0, 200, 512, 768]
    si = _seq_idx(b, L, [edges[1:-1]]).cuda()
    kw = dict(D=d["D"], dt_bias=d["dt_bias"], dt_softplus=True)
    packed = ops.bimamba_chunk_scan_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, z=d["z"], seq_idx=si, **kw)
    for i in range(3):
        s = slice(edges[i], edges[i + 1])
        alone = ops.bimamba_chunk_scan_combined(d["x"][:, s], d["dt"][:, s], d["A"], d["B"][:, s], d["C"][:, s], Q,
                                                z=d["z"][:, s], **kw)
        assert_close(packed[:, s], alone, dtype, f"sequence {i}")

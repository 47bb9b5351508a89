"""The operator under HIP graph capture: forward + backward recorded once into a torch.cuda.CUDAGraph and replayed.  The
library only launches kernels on the caller's stream (it clears memory with a fill kernel, never with a memset node), so
a capture holds the whole pass.  Every replay is checked against the eager result, with eager work and synchronisations
between the replays."""
import pytest
import torch

from tests.helpers import make_case, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(2, 512, 4, 64, 1, 64, 256, torch.bfloat16), (1, 200, 2, 32, 1, 16, 64, torch.float32)])
def test_forward_backward_replays_match_eager(shape):
    from bi_mamba2_amd import ops
    b, L, H, P, G, N, Q, dtype = shape
    d = to_dev(make_case(b, L, H, P, G, N, dtype, with_z=True))
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")
    static = {k: d[k].clone().requires_grad_(True) for k in names}
    dout = torch.randn(d["x"].shape, generator=torch.Generator().manual_seed(3)).to(dtype).cuda()

    def step(t):
        out = ops.bimamba_chunk_scan_combined(t["x"], t["dt"], t["A"], t["B"], t["C"], Q, D=t["D"], z=t["z"], dt_bias=t["dt_bias"],
                                              dt_softplus=True)
        return (out,) + torch.autograd.grad(out, [t[k] for k in names], dout)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up on a side stream, as capture requires
        for _ in range(3):
            step(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(static)
    for rep in range(4):
        # new input values in the graph's static tensors, the same values through the eager path
        fresh = {k: (d[k] * (1.0 + 0.1 * rep) if k in ("x", "B", "C", "z") else d[k].clone()) for k in names}
        with torch.no_grad():
            for k in names:
                static[k].copy_(fresh[k])
        graph.replay()
        torch.cuda.synchronize()
        eager = step({k: fresh[k].detach().clone().requires_grad_(True) for k in names})
        torch.cuda.synchronize()
        for name, a, e in zip(("out",) + tuple("d" + k for k in names), captured, eager):
            assert torch.equal(a, e), f"replay {rep}: {name} differs from the eager result"

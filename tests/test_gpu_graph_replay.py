"""The operator under HIP graph capture: forward + backward recorded once (torch's graph-safe allocator serves the
operator's temporaries), then replayed on new input contents.  Every replay, with eager work and synchronisations in
between, must reproduce the eager result bit for bit -- without pruning, with a float threshold and with "auto"
(whose kernels use atomicMax on a scratch they initialise themselves)."""
import pytest
import torch

from conftest import make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("thr", [None, -6.0, "auto"])
@pytest.mark.parametrize("M,N", [(256, 256), (1, 700), (128, 4096)])
def test_graph_replays_equal_eager(thr, M, N):
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from forgetting_transformer import forgetting_attention
    B, H, D = 2, 4, 64
    sets = [make_inputs(B, H, M, N, D, dtype=torch.bfloat16, device="cuda", head_first=True, seed=50 + s, gate_mean=0.5)
            for s in range(3)]
    ss = torch.tensor([0, 3], device="cuda")

    def step(q, k, v, g, do):
        q, k, v, g = (x.detach().requires_grad_() for x in (q, k, v, g))
        out = forgetting_attention(q, k, v, g, head_first=True, seq_start=ss, adaptive_threshold=thr)
        out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad, g.grad

    eager = [tuple(t.clone() for t in step(*s[:5])) for s in sets]
    static = [t.clone() for t in sets[0][:5]]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up on the capture stream, as torch asks for
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(*static)
    for rnd in range(2):
        for s, want in zip(sets, eager):
            for dst, src in zip(static, s[:5]):
                dst.copy_(src)
            graph.replay()
            torch.cuda.synchronize()
            torch.randn(1 << 20, device="cuda").sum().item()        # unrelated eager work between replays
            for name, got, ref in zip(("out", "dq", "dk", "dv", "dlog_fgate"), outs, want):
                assert torch.equal(got, ref), (name, rnd, thr, M, N)

"""The ring share under HIP graph capture: the library allocates nothing, never synchronises and
launches on the caller's stream, so a forward + backward captured once can be replayed. Replays
are interleaved with eager work and synchronisations, and every replay must reproduce the eager
result bit for bit."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_captured_ring_step_replays_bit_exactly(gpu):
    from pithtrain_amd.operators.ring_attention.local import ring_backward_local, ring_forward_local

    B, S_l, Hq, Hkv, D, C, r = 1, 512, 8, 2, 128, 4, 2
    g = torch.Generator().manual_seed(5)
    mk = lambda *s: (torch.randn(*s, generator=g) * D**-0.5).to(torch.bfloat16).to(gpu)  # noqa: E731
    q = mk(B, S_l, Hq, D)
    ks = [mk(B, S_l, Hkv, D) for _ in range(C)]
    vs = [mk(B, S_l, Hkv, D) for _ in range(C)]
    dout = torch.randn(B, S_l, Hq, D, generator=g).to(torch.bfloat16).to(gpu)
    scale = D**-0.5

    def step():
        out, lse = ring_forward_local(q, ks, vs, scale, r, C, "zigzag")
        dq, dks, dvs = ring_backward_local(dout, q, out, lse, ks, vs, scale, r, C, "zigzag")
        return [out, lse, dq] + [t for t in dks + dvs if t is not None]

    def run_eager():
        return [t.clone() for t in step()]

    want = run_eager()
    # warm-up on a side stream, as graph capture requires
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()

    for replay in range(3):
        for t in captured:
            t.fill_(float("nan"))  # stale results must not pass
        # new inputs in place: a replay reads the tensors the capture saw
        if replay == 1:
            q.mul_(0.5)
            want = run_eager()
        graph.replay()
        torch.cuda.synchronize()
        for i, (got, ref) in enumerate(zip(captured, want)):
            assert torch.equal(got, ref), f"replay {replay}: tensor {i} differs from the eager result"
        # eager work between replays
        assert all(torch.equal(a, b) for a, b in zip(run_eager(), want))

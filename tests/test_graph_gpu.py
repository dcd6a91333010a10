"""Forward + one-call backward captured in a HIP graph (torch.cuda.CUDAGraph) and replayed.

The scoring and backward entry points enqueue kernels and one event record / wait pair only, so they can
be captured, the fork onto the library's second stream included.  Replays are checked against the eager
sequence step by step, with eager work and synchronisations between the replays.  The segment plan is
built outside the graph (rocPRIM's sort clears its buffers with memset nodes)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_captured_step_replays_to_the_eager_bits():
    import bench
    from smore_amd import fused
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    n, b, k, dim = 2_000_000, 1100, 1024, 200          # a step large enough for the second stream
    table0 = torch.empty((n, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q1 = torch.empty((b, dim), device="cuda").uniform_(-0.07, 0.07, generator=gen)
    q2 = torch.empty((b, dim), device="cuda").uniform_(0.0, 0.07, generator=gen)
    idx = bench.zipf_ids(n, (b, k), 1.1, gen, torch.device("cuda"))
    gs = torch.randn((b, k), device="cuda", generator=gen)
    params = fused.score_params(24.0, 0.02)
    opt = fused.adam_params(1e-4, 1)
    plan = fused.build_plan(idx, n)
    codes = fused.new_codes("box", table0, idx, q1)

    def step(w, m, v):
        score = fused.score_forward("box", w, idx, q1, q2, params, codes=codes)
        g1, g2 = fused.score_backward_fused("box", plan, w, idx, q1, q2, score, gs, params, m=m, v=v, adam=opt,
                                            codes=codes)
        return score, g1, g2

    we, me, ve = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    eager = []
    for _ in range(3):
        s, g1, g2 = step(we, me, ve)
        eager.append((s.clone(), g1.clone(), g2.clone(), we.clone(), me.clone(), ve.clone()))
    torch.cuda.synchronize()

    # one uncaptured call on a side stream first: it also creates the library's second stream, which
    # cannot be created while a capture is under way
    ws, ms, vs = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(ws, ms, vs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    wg, mg, vg = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step(wg, mg, vg)
    torch.cuda.synchronize()
    for i in range(3):
        graph.replay()
        torch.cuda.synchronize()
        torch.randn(4096, device="cuda").sum().item()          # unrelated eager work between replays
        want = eager[i]
        for name, a, c in zip(("score", "gq1", "gq2", "table", "m", "v"), want, (*out, wg, mg, vg)):
            assert torch.equal(a, c), f"replay {i}: {name} differs from the eager step"

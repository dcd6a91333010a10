"""A whole step -- segment plan, forward, one-call backward with sparse Adam -- captured in a HIP graph
(torch.cuda.CUDAGraph) and replayed.

Every entry point of the step enqueues kernels only (plus the event record / wait pair of the fork onto the
library's second stream): no memset, no library call, no allocation inside the library.  The optimizer's
per-step constants (learning rate, bias corrections) live in a two-float device buffer that the caller
rewrites between replays, because a captured launch freezes its by-value arguments.  Replays are checked
against eager steps whose learning rate and step counter advance, bit for bit, with eager work and
synchronisations between the replays."""
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
    codes = fused.new_codes("box", table0, idx, q1)
    lrs = [1e-4, 7e-5, 3e-5]                            # a learning-rate schedule on top of the step counter

    def step(w, m, v, opt):
        plan = fused.build_plan(idx, n)
        score = fused.score_forward("box", w, idx, q1, q2, params, codes=codes)
        g1, g2 = fused.score_backward_fused("box", plan, w, idx, q1, q2, score, gs, params, m=m, v=v, adam=opt,
                                            codes=codes)
        return score, g1, g2, plan

    we, me, ve = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    eager = []
    for i, lr in enumerate(lrs):
        s, g1, g2, plan = step(we, me, ve, fused.adam_params(lr, i + 1))
        eager.append((s.clone(), g1.clone(), g2.clone(), we.clone(), me.clone(), ve.clone(), plan.order.clone(),
                      plan.seg_start.clone(), plan.pair_seg.clone(), plan.n_uniq))
    torch.cuda.synchronize()

    # one uncaptured call on a side stream first: it also creates the library's second stream, which
    # cannot be created while a capture is under way
    consts = torch.zeros(2, device="cuda")
    ws, ms, vs = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(ws, ms, vs, fused.adam_params(1e-4, 1, step_consts=consts))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    wg, mg, vg = table0.clone(), torch.zeros_like(table0), torch.zeros_like(table0)
    captured = fused.adam_params(123.0, 77, step_consts=consts)   # lr / step of the capture itself must not matter
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step(wg, mg, vg, captured)
    torch.cuda.synchronize()
    for i, lr in enumerate(lrs):
        fused.set_step_consts(consts, fused.adam_params(lr, i + 1))
        graph.replay()
        torch.cuda.synchronize()
        torch.randn(4096, device="cuda").sum().item()          # unrelated eager work between replays
        want = eager[i]
        plan = out[3]
        got = (*out[:3], wg, mg, vg, plan.order, plan.seg_start, plan.pair_seg)
        assert int(plan.n_uniq_dev.item()) == want[9]
        for name, a, c in zip(("score", "gq1", "gq2", "table", "m", "v", "order", "seg_start", "pair_seg"), want, got):
            if name == "seg_start":                             # entries beyond the segment count are not written
                a, c = a[: want[9] + 1], c[: want[9] + 1]
            assert torch.equal(a, c), f"replay {i}: {name} differs from the eager step"


def test_step_constants_from_device_memory_match_the_by_value_ones():
    """Same update whether lr / step arrive in smx_opt_params or in the device buffer, for every optimizer."""
    from smore_amd import fused
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    n, p, row = 500, 3000, 64
    idx = torch.randint(0, n, (p,), device="cuda", generator=gen)
    grads = torch.randn((p, row), device="cuda", generator=gen)
    plan = fused.build_plan(idx, n)
    for kind in ("adam", "sgd", "adagrad", "rmsprop"):
        outs = []
        for from_device in (False, True):
            w = torch.linspace(-1, 1, n * row, device="cuda").reshape(n, row).contiguous()
            m, v = torch.zeros_like(w), torch.full_like(w, 0.01)
            consts = torch.zeros(2, device="cuda")
            if from_device:
                fused.set_step_consts(consts, fused.opt_params(kind, 3e-3, step=5))
                opt = fused.opt_params(kind, 99.0, step=1, step_consts=consts)
            else:
                opt = fused.opt_params(kind, 3e-3, step=5)
            fused.rows_backward(plan, grads, table=w, m=m if kind == "adam" else None, v=None if kind == "sgd" else v,
                                adam=opt)
            outs.append((w, m, v))
        for a, c in zip(*outs):
            assert torch.equal(a, c), kind

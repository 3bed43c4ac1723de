"""The operators recorded into HIP graphs: every replay, with fresh inputs written into the same buffers and
the program's own eager work and synchronisations between the replays, must give what the eager call
gives on those inputs.  Nothing in the recorded calls may allocate, copy from the host or clear memory
with a memset node; state that changes from step to step (scan descriptors, the LANS step epoch) has to
live on the device for a replay to be a new step.
"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, to_np

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                                   # warm-up outside the capture (lazy module loads)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


# (4096, 256, 16): the scan as one look-back kernel (top-1) or as count + place (top-2); (140000, 8, 64): count +
# segment sums + place, gate rows staged through LDS
@pytest.mark.parametrize("S,M,E", [(4096, 256, 16), (140000, 8, 64)])
@pytest.mark.parametrize("k,dt", [(1, torch.float32), (2, torch.bfloat16)])
def test_encode_decode_graph_replays(pkg, k, dt, S, M, E):
    ops = pkg.ops
    cf = 0.8
    data = torch.empty((S, M), dtype=dt, device="cuda")
    logits = torch.empty((S, E), dtype=torch.float32, device="cuda")
    C = ops.moe_capacity(S, E, cf * k)
    outs = (torch.empty(k * S, device="cuda"), torch.empty((2, k * S), dtype=torch.int32, device="cuda"),
            torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
            torch.empty((E, C, M), dtype=dt, device="cuda"))
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, k))
    dec = torch.empty((S, M), dtype=dt, device="cuda")
    zero = torch.zeros(E, dtype=torch.int32, device="cuda")

    def step():
        ops.moe_encode(data, logits, zero, cf, top_k=k, gate_is_logits=True, workspace=ws, out=outs)
        ops.moe_decode(outs[4], outs[0], outs[1], top_k=k, out=dec)

    def fresh(seed):
        x, lg = make_inputs(seed, S, M, E, zipf_bias=True)
        data.copy_(dev(x).to(dt))
        logits.copy_(dev(lg))

    fresh(0)
    graph = _capture(step)
    for seed in (1, 2, 3, 4):
        fresh(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs] + [dec.clone()]
        for o in outs:                         # eager work between the replays, on the same buffers
            o.fill_(1) if o.dtype != torch.int64 else o.zero_()
        dec.fill_(2)
        step()
        torch.cuda.synchronize()
        for a, b in zip(got, list(outs) + [dec]):
            assert torch.equal(a, b)
        # and the routing of the replay is the oracle's
        sel, _ = mo.select_topk(to_np(logits), k, gate_is_logits=True)
        assert np.array_equal(to_np(got[1])[0][:S] >= 0, to_np(got[1])[0][:S] == sel[0])


@pytest.mark.parametrize("schedule", ["sweeps", "resident"])
def test_lans_graph_replays(pkg, schedule):
    """One recorded LANS step replayed as steps 2, 3, 4, ... of a run (the step number is read from device
    memory) against the same steps made eagerly on a second copy of the state."""
    ops, capi = pkg.ops, pkg.capi
    shapes = [(300, 70), (8192 * 3,), (5,), (8192 * 5 + 17,), (1024, 64)]
    rng = np.random.default_rng(4)
    T = len(shapes)

    def state():
        p = [dev((rng.standard_normal(s) * 0.02).astype(np.float32)) for s in shapes]
        return p, [torch.zeros_like(x) for x in p], [torch.zeros_like(x) for x in p]

    p1, m1, v1 = state()
    p2 = [x.clone() for x in p1]
    m2, v2 = [torch.zeros_like(x) for x in p1], [torch.zeros_like(x) for x in p1]
    g = [torch.empty_like(x) for x in p1]
    sched = capi.LANS_RESIDENT if schedule == "resident" else capi.LANS_SWEEPS
    plan1 = ops.LansPlan([x.numel() for x in p1], schedule=sched)
    plan2 = ops.LansPlan([x.numel() for x in p1], schedule=sched)
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    step_dev = torch.ones((), dtype=torch.float32, device="cuda")

    def fresh(seed):
        r = np.random.default_rng(seed)
        for x, s in zip(g, shapes):
            x.copy_(dev((r.standard_normal(s) * 1e-3).astype(np.float32)))

    fresh(100)
    plan1.step(g, p1, m1, v1, 1, hyper)        # step 1 eagerly on both copies (uploads the pointer tables)
    plan2.step(g, p2, m2, v2, 1, hyper)
    torch.cuda.synchronize()
    state_before = [x.clone() for x in p1 + m1 + v1]
    graph = _capture(lambda: plan1.step(g, p1, m1, v1, 0, hyper, step_dev=step_dev))
    for a, b in zip(p1 + m1 + v1, state_before):   # the warm-up and the capture must not count as steps
        a.copy_(b)
    for n in (2, 3, 4, 5):
        fresh(100 + n)
        step_dev.fill_(float(n))
        graph.replay()
        torch.cuda.synchronize()
        plan2.step(g, p2, m2, v2, n, hyper)
        torch.cuda.synchronize()
        for a, b in zip(p1 + m1 + v1, p2 + m2 + v2):
            assert torch.equal(a, b)
        assert plan1.error() == 0 and plan2.error() == 0
    plan1.close()
    plan2.close()

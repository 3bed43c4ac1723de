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


@pytest.mark.parametrize("k,logits_in", [(1, False), (2, True)])
def test_forward_and_backward_graph_replays(pkg, k, logits_in):
    """One expert layer's dispatch forward and backward recorded as one graph: encode, decode, then the four
    backward ops and the gate gradient of the whole op, every buffer given by the caller."""
    ops = pkg.ops
    S, M, E, cf = 6000, 128, 32, 0.7
    C = ops.moe_capacity(S, E, cf * k)
    f32, i32 = torch.float32, torch.int32
    data = torch.empty((S, M), device="cuda")
    gate = torch.empty((S, E), device="cuda")
    dy = torch.empty((S, M), device="cuda")
    zero = torch.zeros(E, dtype=i32, device="cuda")
    enc = (torch.empty(k * S, device="cuda"), torch.empty((2, k * S), dtype=i32, device="cuda"),
           torch.empty(E, dtype=i32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
           torch.empty((E, C, M), device="cuda"))
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, k))
    ws_dx = torch.empty(max(int(pkg.capi.load().lancet_moe_decode_dx_workspace_bytes(E, C)), 4), dtype=torch.uint8, device="cuda")
    res = dict(dec=torch.empty((S, M), device="cuda"), d_buf=torch.empty((E, C, M), device="cuda"),
               d_gates_s=torch.empty(k * S, device="cuda"), d_data=torch.empty((S, M), device="cuda"),
               d_gate=torch.empty((S, E), device="cuda"))

    def step():
        ops.moe_encode(data, gate, zero, cf, top_k=k, gate_is_logits=logits_in, workspace=ws, out=enc)
        ops.moe_decode(enc[4], enc[0], enc[1], top_k=k, out=res["dec"])
        ops.moe_decode_dx(dy, enc[0], enc[1], E, C, top_k=k, workspace=ws_dx, out=res["d_buf"])
        ops.moe_decode_dg(dy, enc[4], enc[1], top_k=k, out=res["d_gates_s"])
        ops.moe_encode_dx(res["d_buf"], enc[1], top_k=k, out=res["d_data"])
        ops.moe_encode_dgate(res["d_gates_s"], gate, enc[1], top_k=k, gate_is_logits=logits_in, out=res["d_gate"])

    def fresh(seed):
        x, lg = make_inputs(seed, S, M, E, zipf_bias=True)
        data.copy_(dev(x))
        gate.copy_(dev(lg) if logits_in else torch.softmax(dev(lg), dim=1))
        dy.copy_(dev(np.random.default_rng(seed + 50).standard_normal((S, M)).astype(np.float32)))

    fresh(0)
    graph = _capture(step)
    for seed in (1, 2, 3):
        fresh(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = {n: t.clone() for n, t in res.items()}
        for t in list(res.values()) + [enc[0], enc[4]]:
            t.fill_(3)                         # eager work between the replays, on the same buffers
        step()
        torch.cuda.synchronize()
        for n, t in res.items():
            assert torch.equal(got[n], t), n
        want = mo.moe_encode_dgate(to_np(got["d_gates_s"]), to_np(gate), to_np(enc[1]), k, logits_in)
        scale = np.abs(want).max(axis=1, keepdims=True)
        assert (np.abs(to_np(got["d_gate"]) - want) <= 1e-5 * np.abs(want) + 2e-6 * scale).all()


@pytest.mark.parametrize("schedule", ["sweeps", "resident"])
def test_mixed_precision_lans_graph_replays(pkg, schedule):
    """The step of a 16-bit model (bf16 gradients in, bf16 parameter copies out) recorded once and replayed as
    steps 2, 3, ... against the same steps made eagerly on a second copy of the state."""
    ops, capi = pkg.ops, pkg.capi
    shapes = [(300, 70), (8192 * 3,), (5,), (8192 * 5 + 18,), (1024, 64)]
    rng = np.random.default_rng(14)
    bf16 = torch.bfloat16
    p1 = [dev((rng.standard_normal(s) * 0.02).astype(np.float32)) for s in shapes]
    p2 = [x.clone() for x in p1]
    m1, v1, m2, v2 = ([torch.zeros_like(x) for x in p1] for _ in range(4))
    low1, low2 = ([torch.zeros_like(x, dtype=bf16) for x in p1] for _ in range(2))
    g = [torch.empty_like(x, dtype=bf16) for x in p1]
    sched = capi.LANS_RESIDENT if schedule == "resident" else capi.LANS_SWEEPS
    plan1 = ops.LansPlan([x.numel() for x in p1], schedule=sched)
    plan2 = ops.LansPlan([x.numel() for x in p1], schedule=sched)
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    step_dev = torch.ones((), dtype=torch.float32, device="cuda")

    def fresh(seed):
        r = np.random.default_rng(seed)
        for x, s in zip(g, shapes):
            x.copy_(dev((r.standard_normal(s) * 1e-3).astype(np.float32)).to(bf16))

    fresh(200)
    plan1.step(g, p1, m1, v1, 1, hyper, p_lowp=low1)
    plan2.step(g, p2, m2, v2, 1, hyper, p_lowp=low2)
    torch.cuda.synchronize()
    before = [x.clone() for x in p1 + m1 + v1 + low1]
    graph = _capture(lambda: plan1.step(g, p1, m1, v1, 0, hyper, step_dev=step_dev, p_lowp=low1))
    for a, b in zip(p1 + m1 + v1 + low1, before):
        a.copy_(b)
    for n in (2, 3, 4):
        fresh(200 + n)
        step_dev.fill_(float(n))
        graph.replay()
        torch.cuda.synchronize()
        plan2.step(g, p2, m2, v2, n, hyper, p_lowp=low2)
        torch.cuda.synchronize()
        for a, b in zip(p1 + m1 + v1 + low1, p2 + m2 + v2 + low2):
            assert torch.equal(a, b)
        for lw, pp in zip(low1, p1):
            assert torch.equal(lw, pp.to(bf16))
        assert plan1.error() == 0 and plan2.error() == 0
    plan1.close()
    plan2.close()


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

"""The BASELINE.json configurations at their full sizes.

Routing integers are compared with the oracle bit for bit at full size.  The [E,C,M] buffers and
the recombined [S,M] outputs are compared through properties that hold at any size and are
evaluated on the GPU: every kept token's row is found bit-equal at its (expert, location), rows
past the used capacity are zero, decode(identity expert) returns the token scaled by its combine
weight(s).  (The oracle's own buffers are compared directly at the reduced sizes of
test_gpu_moe.py.)"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import ulp_distance, dev, make_inputs, rows_to_torch, to_np

pytestmark = pytest.mark.gpu


def check_buffer_properties(data_t, il_t, used_t, disp_t, k):
    S = data_t.shape[0]
    E, Cap, M = disp_t.shape
    il = il_t.long()
    for j in range(k):
        idx, loc = il[0, j * S:(j + 1) * S], il[1, j * S:(j + 1) * S]
        ok = idx >= 0
        assert torch.equal(disp_t[idx[ok], loc[ok]], data_t[ok])
    # kept rows per expert = used (used_in = 0), rows past them are zero
    kept = torch.bincount(il[0][il[0] >= 0], minlength=E)
    assert torch.equal(kept, used_t.long())
    tail = torch.arange(Cap, device="cuda")[None, :] >= used_t.long()[:, None]
    assert not disp_t[tail].any()


def test_config1_switch_top1_fp32(pkg):
    """S=4096, M=768 fp32, E=8, top-1, C=640, combine weight = top-1 softmax prob, seed 0."""
    S, M, E, cf = 4096, 768, 8, 1.25
    data, logits = make_inputs(0, S, M, E)
    want = mo.moe_encode(data, logits, np.zeros(E, np.int32), cf, gate_is_logits=True, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), None, cf, gate_is_logits=True)
    assert got[4].shape == (E, 640, M)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_array_equal(to_np(got[3]), want[3])
    np.testing.assert_allclose(to_np(got[0]), want[0], rtol=1e-5)
    np.testing.assert_array_equal(to_np(got[4]), want[4])
    out = pkg.ops.moe_decode(got[4], got[0], got[1])
    np.testing.assert_array_equal(to_np(out), mo.moe_decode(want[4], to_np(got[0]), want[1]))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_config2_gshard_top2_zipf(pkg, dt):
    """S=16384, M=1024, E=16, top-2, capacity factor 1.0 (C=2048), Zipf(1.2) expert bias."""
    S, M, E, cf = 16384, 1024, 16, 1.0
    data, logits = make_inputs(0, S, M, E, zipf_bias=True)
    sel, val = mo.select_topk(logits, 2, True)
    zero = np.zeros(E, np.int32)
    Cap = mo.capacity(S, E, 2 * cf)
    assert Cap == 2048
    i1, l1, u1, _ = mo.gen_location(sel[0], zero, Cap, M, E)
    i2, l2, u2, _ = mo.gen_location(sel[1], u1, Cap, M, E)
    merged = mo.moe_merge_masks([np.stack([i1, l1]), np.stack([i2, l2])], E)
    d_data = rows_to_torch(data, dt)
    got = pkg.ops.moe_encode(d_data, dev(logits), None, cf, top_k=2, gate_is_logits=True)
    np.testing.assert_array_equal(to_np(got[1]), merged)
    np.testing.assert_array_equal(to_np(got[2]), u2)
    assert (merged[0] < 0).sum() > 1000, "hot experts must overflow"
    raw = np.concatenate([val[0], val[1]])
    np.testing.assert_allclose(to_np(got[0]), mo.top2_normalize_gates(raw, merged[0]), rtol=1e-5)
    check_buffer_properties(d_data, got[1], got[2], got[4], 2)
    out = pkg.ops.moe_decode(got[4], got[0], got[1], top_k=2)
    # identity expert: out = (g1 + g2) * x with g1 + g2 = 1 where any slot was kept, else 0
    either = (got[1][0, :S] >= 0) | (got[1][0, S:] >= 0)
    x = d_data.float()
    if dt == "f32":
        assert float(((out.float() - x)[either].abs() / x[either].abs().clamp_min(1e-20)).max()) <= 2e-6
    else:   # 1 unit in the last place of bf16 (north_star's bound for the combine), counted on the bit patterns
        assert ulp_distance(out[either], d_data[either]) <= 1
    assert not out[~either].any() and (~either).any()


@pytest.mark.parametrize("P", [1, 4])
@pytest.mark.parametrize("hot_experts", [False, True])
def test_config3_batch_prioritized_bf16(pkg, P, hot_experts):
    """S=32768, M=2048 bf16, E=64, top-1, cf=1.25 (C=640), logits ~ 2*N(0,1); the drop set of the
    sort+scan is reproduced exactly, for the whole batch and for 4 partitions.  With the
    configuration's balanced logits no expert reaches its capacity (512 +- 22 tokens against
    640), so the same shape is also run with a Zipf expert bias that makes hot experts overflow."""
    S0, M, E, cf = 32768, 2048, 64, 1.25
    data, logits = make_inputs(0, S0, M, E, logit_scale=2.0, zipf_bias=hot_experts)
    gate = mo.softmax_rows(logits)           # priorities: fp32 softmax prob of the top expert
    d_data, d_gate = rows_to_torch(data, "bf16"), dev(gate)
    S = S0 // P
    kept_total = np.zeros(E, np.int64)
    for pid in range(P):
        want = mo.moe_encode_bpr(np.zeros((S0, 1), np.float32), gate, P, pid, cf * P, fast_scatter=True)
        got = pkg.ops.moe_encode_batch_prioritized(d_data, d_gate, P, pid, cf * P)
        assert got[4].shape == (E, 640, M)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[2]), want[2])
        np.testing.assert_array_equal(to_np(got[0]), want[0])
        check_buffer_properties(d_data[pid * S:(pid + 1) * S], got[1], got[2], got[4], 1)
        kept_total += want[2]
    cnt = np.bincount(np.argmax(gate, axis=1), minlength=E)
    np.testing.assert_array_equal(kept_total, np.minimum(cnt, 640))
    assert bool((cnt > 640).any()) == hot_experts


@pytest.mark.parametrize("pressure", [False, True])
def test_config4_lancet_forward_pipeline_bf16(pkg, pressure):
    """S=65536 (4 partitions of 16384), M=4096 bf16, E=32, top-2, cf=1.25 -> C=5120: encode per
    (slot, partition) in capacity order s1p0..s1p3, s2p0..s2p3 with chained used capacity, then
    moe_merge_masks + moe_redispatch, then moe_decode; must equal the un-partitioned top-2 op.
    Inputs as the configuration states them: NumPy default_rng(0), data then logits, both N(0,1), rows rounded
    to bf16 (nothing is dropped at C = 5120 then); and the same with four favoured experts, so that slots overflow."""
    ops = pkg.ops
    S0, M, E, cf, P = 65536, 4096, 32, 1.25, 4
    S = S0 // P
    rng = np.random.default_rng(0)
    data = torch.from_numpy(mo.f32_to_bf16_bits(rng.standard_normal((S0, M), dtype=np.float32)).view(np.int16)).cuda().view(torch.bfloat16)
    h_logits = rng.standard_normal((S0, E), dtype=np.float32)
    if pressure:
        h_logits[:, :4] += np.float32(0.75)
    logits = torch.from_numpy(h_logits).cuda()
    fused = ops.moe_encode(data, logits, None, cf, top_k=2, gate_is_logits=True)
    assert fused[4].shape == (E, 5120, M)
    # per-slot gate arrays: argmax = the slot's expert, max = its softmax probability
    lib = pkg.capi.load()
    import ctypes as C
    sel = torch.empty((2, S0), dtype=torch.int32, device="cuda")
    val = torch.empty((2, S0), dtype=torch.float32, device="cuda")
    assert lib.lancet_gate_topk(C.c_void_p(logits.data_ptr()), None, S0, E, 2, pkg.capi.F32, pkg.capi.GATE_IS_LOGITS,
                                C.c_void_p(sel.data_ptr()), C.c_void_p(val.data_ptr()), None) == 0
    used = torch.zeros(E, dtype=torch.int32, device="cuda")
    ils, bufs, raws = [], [], []
    for slot in range(2):
        for p in range(P):
            sl = slice(p * S, (p + 1) * S)
            gate = torch.full((S, E), -1.0, device="cuda")
            gate.scatter_(1, sel[slot, sl].long()[:, None], val[slot, sl][:, None])
            g, il, used, elems, disp = ops.moe_encode(data[sl], gate, used, 2 * cf * P)
            assert disp.shape == (E, 5120, M)
            ils.append(il), bufs.append(disp), raws.append(g)
    merged = ops.moe_merge_masks(ils, E)                 # [2, 8*S] = slot-major [2, 2*S0]
    red = ops.moe_redispatch(bufs, ils)
    del bufs
    weights = ops.moe_top2_normalize_gates(torch.cat(raws), merged)
    assert torch.equal(merged, fused[1])
    assert torch.equal(used, fused[2])
    assert torch.equal(red, fused[4])
    np.testing.assert_allclose(to_np(weights), to_np(fused[0]), rtol=1e-5)
    assert (int((merged[0] < 0).sum()) > 0) == pressure
    out_p = ops.moe_decode(red, weights, merged, top_k=2)
    out_f = ops.moe_decode(fused[4], fused[0], fused[1], top_k=2)
    diff = (out_p.view(torch.int16).int() - out_f.view(torch.int16).int()).abs().max()
    assert int(diff) <= 1
    # routing at full size against the oracle
    osel, _ = mo.select_topk(h_logits, 2, True)
    zero = np.zeros(E, np.int32)
    i1, l1, u1, _ = mo.gen_location(osel[0], zero, 5120, M, E)
    i2, l2, u2, _ = mo.gen_location(osel[1], u1, 5120, M, E)
    np.testing.assert_array_equal(to_np(merged), mo.moe_merge_masks([np.stack([i1, l1]), np.stack([i2, l2])], E))
    check_buffer_properties(data, merged, used, red, 2)


# ----------------------------------------------------------------------------- config 5: LANS at full size
def _config5_shapes():
    """24 layers x {4 x [1024,1024], 8 x [1024]}, every second layer 32 expert matrices ([1024,4096] and
    [4096,1024] x 16 experts), final norm 2 x [1024]: 674 tensors, 1,711,474,688 parameters."""
    shapes = []
    for layer in range(24):
        shapes += [(1024, 1024)] * 4 + [(1024,)] * 8
        if layer % 2 == 1:
            shapes += [(1024, 4096), (4096, 1024)] * 16
    return shapes + [(1024,)] * 2


def test_config5_lans_full_size(pkg):
    """All 674 tensors stepped 10 times by both schedules.  The oracle follows a sample of the tensors (one of
    every shape, at the list's ends and in its middle: a step is independent per tensor) through the same 10
    steps: parameters within 1e-6 of max|p| (m, v 1e-5).  Over the whole list: the norms the plan reports
    against torch's fp64 norms of the same arrays, and the two schedules against each other (2e-6)."""
    import importlib
    lo = importlib.import_module("oracle.lans_oracle")
    ops, capi = pkg.ops, pkg.capi
    free, _ = torch.cuda.mem_get_info()
    if free < 80 << 30:
        pytest.skip("needs 80 GiB of free device memory")
    shapes = _config5_shapes()
    numels = [int(np.prod(s)) for s in shapes]
    assert len(shapes) == 674 and sum(numels) == 1711474688
    gen = torch.Generator(device="cuda").manual_seed(5)
    p0 = [torch.randn(s, generator=gen, device="cuda") * 0.02 for s in shapes]
    state = {}
    for name, sched in (("sweeps", capi.LANS_SWEEPS), ("resident", capi.LANS_RESIDENT)):
        state[name] = ([x.clone() for x in p0], [torch.zeros_like(x) for x in p0], [torch.zeros_like(x) for x in p0],
                       ops.LansPlan(numels, schedule=sched))
    sample = [0, 4, 12, 16, 24, 25, 300, 341, 672, 673]              # matrices, vectors, both expert shapes, the ends
    assert {shapes[i] for i in sample} == set(shapes)
    ref_p = [to_np(p0[i]) for i in sample]
    ref_m = [np.zeros(shapes[i], np.float32) for i in sample]
    ref_v = [np.zeros(shapes[i], np.float32) for i in sample]
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    g = [torch.empty_like(x) for x in p0]
    for step in range(1, 11):
        for x in g:
            x.normal_(0.0, 1e-3, generator=gen)
        for name in ("sweeps", "resident"):
            p, m, v, plan = state[name]
            plan.step(g, p, m, v, step, hyper)
        lo.lans_step([to_np(g[i]) for i in sample], ref_p, ref_m, ref_v, step)
        if step in (1, 10):
            p, m, v, plan = state["sweeps"]
            norms = to_np(plan.norms())
            want_g = torch.stack([torch.linalg.vector_norm(x.double()) for x in g]).cpu().numpy()
            np.testing.assert_allclose(norms[0], want_g, rtol=2e-6)
    torch.cuda.synchronize()
    for name in ("sweeps", "resident"):
        p, m, v, plan = state[name]
        assert plan.error() == 0
        for k, i in enumerate(sample):
            for got, want, tol, what in ((p[i], ref_p[k], 1e-6, "p"), (m[i], ref_m[k], 1e-5, "m"), (v[i], ref_v[k], 1e-5, "v")):
                diff = np.abs(to_np(got).astype(np.float64) - want)
                err = diff.max()
                assert err <= tol * np.abs(want).max(), "%s %s[%d]: %.3e" % (name, what, i, err)
                if what == "p":
                    # element by element: 1e-6 relative, with a floor of 1e-9 of the tensor's largest entry for the
                    # entries near zero (an entry moves by about lr * |p| per step whatever its own size, so the
                    # last place of that movement, not of the entry, bounds what two evaluation orders can differ by)
                    bound = 1e-6 * np.abs(want) + 1e-9 * np.abs(want).max()
                    assert (diff <= bound).all(), "%s p[%d]: %.3e relative at the worst entry" % (
                        name, i, (diff / np.maximum(np.abs(want), 1e-30)).max())
    ps, pr = state["sweeps"][0], state["resident"][0]
    for i in range(len(shapes)):
        scale = float(ps[i].abs().max())
        assert float((ps[i] - pr[i]).abs().max()) <= 2e-6 * scale, i
        assert bool((ps[i] != p0[i]).any())                         # every tensor was stepped
    for name in ("sweeps", "resident"):
        state[name][3].close()


def test_config5_lans_mixed_precision_full_size(pkg):
    """Config 5's 674 tensors as a bf16 model trains them: bf16 gradients, fp32 master parameters and moments, and the
    model's bf16 parameters written by the same step (lancet_lans_step_mixed), resident schedule, 4 steps.  The oracle
    (cast up, lans_step, cast down: python/raf/optim/lans.py:256-257, 285-288) follows a sample of tensors of every
    shape; over the whole list every 16-bit copy must be the rounded master parameter, bit for bit."""
    import importlib
    lo = importlib.import_module("oracle.lans_oracle")
    ops, capi = pkg.ops, pkg.capi
    free, _ = torch.cuda.mem_get_info()
    if free < 50 << 30:
        pytest.skip("needs 50 GiB of free device memory")
    shapes = _config5_shapes()
    numels = [int(np.prod(s)) for s in shapes]
    gen = torch.Generator(device="cuda").manual_seed(6)
    p = [torch.randn(s, generator=gen, device="cuda") * 0.02 for s in shapes]
    m = [torch.zeros_like(x) for x in p]
    v = [torch.zeros_like(x) for x in p]
    low = [torch.zeros(s, dtype=torch.bfloat16, device="cuda") for s in shapes]
    g = [torch.empty(s, dtype=torch.bfloat16, device="cuda") for s in shapes]
    sample = [0, 4, 12, 16, 24, 25, 300, 341, 672, 673]
    ref_p = [to_np(p[i]) for i in sample]
    ref_m = [np.zeros(shapes[i], np.float32) for i in sample]
    ref_v = [np.zeros(shapes[i], np.float32) for i in sample]
    plan = ops.LansPlan(numels)
    assert plan.schedule() == capi.LANS_RESIDENT
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    for step in range(1, 5):
        for x in g:
            x.copy_(torch.empty(x.shape, device="cuda").normal_(0.0, 1e-3, generator=gen))
        plan.step(g, p, m, v, step, hyper, p_lowp=low)
        lo.lans_step_mixed([to_np(g[i]) for i in sample], ref_p, ref_m, ref_v, step, mo.round_to_bf16)
    torch.cuda.synchronize()
    assert plan.error() == 0 and plan.last_resident_slots() > 0
    for i in range(len(shapes)):
        assert torch.equal(low[i], p[i].to(torch.bfloat16)), i
    for k, i in enumerate(sample):
        for got, want, tol, what in ((p[i], ref_p[k], 1e-6, "p"), (m[i], ref_m[k], 1e-5, "m"), (v[i], ref_v[k], 1e-5, "v")):
            err = np.abs(to_np(got).astype(np.float64) - want).max()
            assert err <= tol * np.abs(want).max(), "%s[%d]: %.3e" % (what, i, err)
    plan.close()

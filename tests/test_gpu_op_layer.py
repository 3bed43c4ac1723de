"""The C++ op layer (OpEnv + dialect dispatch) on the GPU: an executor that declares, allocates,
dispatches and executes must give exactly what the oracle gives, for all six operators."""
import numpy as np
import pytest
import torch

from oracle import lans_oracle as lo
from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ex(pkg):
    return pkg.raf_executor.Executor()


def test_encode_decode_through_the_op_layer(pkg, ex):
    S, M, E, cf = 2048, 128, 32, 1.0
    data, logits = make_inputs(11, S, M, E)
    gate = mo.softmax_rows(logits)
    used0 = np.zeros(E, np.int32)
    want = mo.moe_encode(data, gate, used0, cf, fast_scatter=True)
    got = ex("raf.op.moe_encode", dev(data), dev(gate), dev(used0), cf)
    assert len(got) == 5 and got[3].dtype == torch.uint64
    for g, w in zip(got, want):
        np.testing.assert_array_equal(to_np(g), w)
    out = ex("raf.op.moe_decode", got[4], got[0], got[1])
    np.testing.assert_array_equal(to_np(out), mo.moe_decode(want[4], want[0], want[1]))
    # extension arguments: top_k = 2 on logits
    want2 = mo.moe_encode_top2(data, logits, used0, cf, gate_is_logits=True, fast_scatter=True)
    got2 = ex("raf.op.moe_encode", dev(data), dev(logits), dev(used0), cf, 2, 1)
    np.testing.assert_array_equal(to_np(got2[1]), want2[1])
    np.testing.assert_array_equal(to_np(got2[4]), want2[4])
    out2 = ex("raf.op.moe_decode", got2[4], got2[0], got2[1], 2)
    np.testing.assert_array_equal(to_np(out2), mo.moe_decode(want2[4], to_np(got2[0]), want2[1], k=2))


def test_bpr_merge_redispatch_through_the_op_layer(pkg, ex):
    S0, M, E, P = 1024, 64, 16, 4
    data, logits = make_inputs(12, S0, M, E, logit_scale=2.0)
    gate = mo.softmax_rows(logits)
    d_data, d_gate = dev(data), dev(gate)
    ils, bufs, o_ils, o_bufs = [], [], [], []
    for pid in range(P):
        got = ex("raf.op.moe_encode_batch_prioritized", d_data, d_gate, P, pid, float(P))
        want = mo.moe_encode_bpr(data, gate, P, pid, float(P), fast_scatter=True)
        for g, w in zip(got, want):
            np.testing.assert_array_equal(to_np(g), w)
        ils.append(got[1]), bufs.append(got[4]), o_ils.append(want[1]), o_bufs.append(want[4])
    merged = ex("raf.op.moe_merge_masks", ils, E)
    red = ex("raf.op.moe_redispatch", bufs, ils)
    np.testing.assert_array_equal(to_np(merged), mo.moe_merge_masks(o_ils, E))
    np.testing.assert_array_equal(to_np(red), mo.moe_redispatch(o_bufs, o_ils))


@pytest.mark.parametrize("schedule", ["sweeps", "resident"])
def test_lans_through_the_op_layer_with_cached_openv(pkg, ex, monkeypatch, schedule):
    # the OpEnv reads LANCET_LANS_SCHEDULE when it is built
    monkeypatch.setenv("LANCET_LANS_SCHEDULE", schedule)
    shapes = [(128, 64), (33,), (5000,), (3, 8192)]
    rng = np.random.default_rng(0)
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
    dg, dp, dm, dv = ([dev(a) for a in l] for l in (g, p, m, v))
    step = torch.tensor(1.0, device="cuda")
    call = ex.prepare("raf.op.lans", dg + dp + dm + dv, step, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)
    assert call.env_name == "raf.op.hip.lans" and call.arg_indices == [0, 1]
    for k in range(1, 4):           # the OpEnv is built once and executed three times
        step.fill_(float(k))
        outs = call.run()
        lo.lans_step(g, p, m, v, k)
    torch.cuda.synchronize()
    assert len(outs) == 4 * len(shapes) and outs[len(shapes)].data_ptr() == dp[0].data_ptr()   # outputs alias the inputs
    for a, b in zip(dp, p):
        assert np.abs(to_np(a).astype(np.float64) - b).max() <= 1e-6 * np.abs(b).max()
    call.close()


@pytest.mark.parametrize("full_size", [False, True])
def test_config4_pattern_both_ways_through_the_op_layer(pkg, ex, full_size):
    """Config 4's dispatch (4 token partitions, top-2) through the executor in the two forms the op layer offers:
    as the partition pass emits it (src/pass/dist_optimization/partition_exprs.cc:1709-1874: one moe_encode per
    (slot, partition) chained through used_capacity, moe_merge_masks, moe_redispatch) and rewritten to the
    routed-once form (moe_route over the whole gate, moe_scatter_tokens per partition in place on one buffer,
    moe_decode_tokens per partition).  Masks, capacities, the [E, C, M] buffer and the combined output must be
    equal, bit for bit (the weights to 1e-5: the chained form normalises them in a separate op)."""
    ops = pkg.ops
    if full_size:
        S0, M, E, cf, P, dt = 65536, 4096, 32, 1.25, 4, torch.bfloat16
    else:
        S0, M, E, cf, P, dt = 4096, 64, 8, 0.5, 4, torch.bfloat16
    S = S0 // P
    rng = np.random.default_rng(0)
    data = torch.from_numpy(rng.standard_normal((S0, M), dtype=np.float32)).cuda().to(dt)
    h_logits = rng.standard_normal((S0, E), dtype=np.float32)
    h_logits[:, :2] += np.float32(0.75)                     # favoured experts: slots overflow
    logits = torch.from_numpy(h_logits).cuda()
    zero = torch.zeros(E, dtype=torch.int32, device="cuda")
    # ---- routed once
    gates_s, il, used, elems = ex("raf.op.moe_route", logits, zero, M, cf, 2, 1)
    Cap = ops.moe_capacity(S0, E, 2 * cf)
    buf = torch.full((E, Cap, M), 7.0, dtype=dt, device="cuda")
    for p in range(P):
        out = ex("raf.op.moe_scatter_tokens", data[p * S:(p + 1) * S], il, zero, used, buf, p * S, 2, p == P - 1)
        assert out.data_ptr() == buf.data_ptr()            # in place
    starts, counts = ex("raf.op.moe_partition_ranges", il, P, E, M, 2)
    outs = [ex("raf.op.moe_decode_tokens", buf, gates_s, il, p * S, S, 2) for p in range(P)]
    # ---- as the partition pass emits it
    sel = torch.empty((2, S0), dtype=torch.int32, device="cuda")
    val = torch.empty((2, S0), dtype=torch.float32, device="cuda")
    import ctypes as C
    assert pkg.capi.load().lancet_gate_topk(C.c_void_p(logits.data_ptr()), None, S0, E, 2, pkg.capi.F32, pkg.capi.GATE_IS_LOGITS,
                                            C.c_void_p(sel.data_ptr()), C.c_void_p(val.data_ptr()), None) == 0
    u = zero
    ils, bufs, raws = [], [], []
    for slot in range(2):
        for p in range(P):
            sl = slice(p * S, (p + 1) * S)
            gate = torch.full((S, E), -1.0, device="cuda")
            gate.scatter_(1, sel[slot, sl].long()[:, None], val[slot, sl][:, None])
            g, pil, u, pel, disp = ex("raf.op.moe_encode", data[sl], gate, u, 2 * cf * P, 1, 0, 0)   # no tail zero-fill: feeds redispatch
            ils.append(pil), bufs.append(disp), raws.append(g)
    merged = ex("raf.op.moe_merge_masks", ils, E)
    red = ex("raf.op.moe_redispatch", bufs, ils)
    del bufs
    weights = ops.moe_top2_normalize_gates(torch.cat(raws), merged)
    assert bool((merged[0] < 0).any())
    assert torch.equal(merged, il) and torch.equal(u, used) and torch.equal(red, buf)
    np.testing.assert_allclose(to_np(weights), to_np(gates_s), rtol=1e-5)
    whole = ex("raf.op.moe_decode", red, gates_s, merged, 2)
    assert torch.equal(torch.cat(outs), whole)
    # the ranges are the partitions' own element counts, in capacity order
    kept = torch.stack([(il[0, j * S0 + p * S: j * S0 + (p + 1) * S].long().clamp_min(-1) + 1).bincount(minlength=E + 1)[1:]
                        for j in range(2) for p in range(P)])
    assert torch.equal(counts.view(torch.int64), kept * M)
    assert torch.equal(starts.view(torch.int64), (torch.cumsum(kept, 0) - kept) * M)


def test_gate_gradient_and_mixed_lans_through_the_op_layer(pkg, ex):
    S, M, E = 3000, 16, 16
    data, logits = make_inputs(17, S, M, E, zipf_bias=True)
    want = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 0.7, gate_is_logits=True, fast_scatter=True)
    dy = np.random.default_rng(2).standard_normal(2 * S).astype(np.float32)
    got = ex("raf.op.moe_encode_dgate", dev(dy), dev(logits), dev(want[1]), 2, 1)
    ref = mo.moe_encode_dgate(dy, logits, want[1], 2, True)
    scale = np.abs(ref).max(axis=1, keepdims=True)
    assert (np.abs(to_np(got) - ref) <= 1e-5 * np.abs(ref) + 1e-6 * scale).all()
    # lans with bf16 gradients and bf16 parameter copies (trailing tuple argument)
    shapes = [(128, 64), (33,), (2, 8192)]
    rng = np.random.default_rng(1)
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    g = [mo.round_to_bf16(rng.normal(0, 1e-3, s).astype(np.float32)) for s in shapes]
    dg = [dev(a).to(torch.bfloat16) for a in g]
    dp, dm, dv = ([dev(a) for a in l] for l in (p, m, v))
    low = [torch.zeros(s, dtype=torch.bfloat16, device="cuda") for s in shapes]
    call = ex.prepare("raf.op.lans", dg + dp + dm + dv, 1, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True, low)
    assert call.arg_indices == [0, 1, 11]
    call.run()
    torch.cuda.synchronize()
    lo.lans_step_mixed(g, p, m, v, 1, mo.round_to_bf16)
    for a, b, c in zip(dp, p, low):
        assert np.abs(to_np(a).astype(np.float64) - b).max() <= 1e-6 * np.abs(b).max()
        assert torch.equal(c, a.to(torch.bfloat16))
    call.close()


def test_executor_reports_op_errors(pkg, ex):
    with pytest.raises(pkg.raf_executor.RafError, match="matching shape in dim 0"):
        ex("raf.op.moe_encode", torch.zeros((8, 4), device="cuda"), torch.zeros((9, 2), device="cuda"),
           torch.zeros(2, dtype=torch.int32, device="cuda"), 1.0)
    with pytest.raises(pkg.raf_executor.RafError, match="float32"):
        ex("raf.op.lans", [torch.zeros(4, device="cuda", dtype=torch.float16)] * 4, 1, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)


def test_plain_c_client_of_the_c_abi():
    """tests/c_client/lancet_client.c: a C99 program that links the library and the HIP runtime only (no
    Python, no torch) and checks encode + decode on a hand-computed case."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_client", "lancet_client")
    if not os.path.exists(exe):                # normally built beforehand by __graft_entry__.build(); gcc takes 0.2 s
        subprocess.run(["make", "-C", os.path.dirname(exe)], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0, proc.stdout
    assert "match the hand-computed case" in proc.stdout


def test_op_layer_reports_a_scan_that_gave_up(pkg, ex):
    """A prepared call keeps its OpEnv and workspace across runs (RAF's interpreter cache): the workspace is set up
    by the first run only; with a wait bound of one poll the scan gives up somewhere in 512 tiles, the outputs carry
    the marks, and check() raises where the reference would have aborted; the next run is whole again."""
    import ctypes as C
    lib = pkg.capi.load()
    S, M, E = 131072, 8, 256         # 512 tiles; the look-back form of the scan is asked for below (the default forms have no waits)
    data, logits = make_inputs(13, S, M, E)
    gate = mo.softmax_rows(logits)
    want = mo.moe_encode(data, gate, np.zeros(E, np.int32), 1.0, fast_scatter=True)
    # capacity_factor, top_k, gate_is_logits, zero_tail, no noise tensor, scan as one look-back kernel
    call = ex.prepare("raf.op.moe_encode", dev(data), dev(gate), dev(np.zeros(E, np.int32)), 1.0, 1, 0, 1, 0, 1)
    try:
        got = call.run()
        call.check()
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        ws = C.c_void_p(call.workspaces[0].data_ptr())
        raised = 0
        for _ in range(3):
            assert lib.lancet_debug_scan_workspace_spin_limit(ws, 1, None) == 0
            got = call.run()
            assert lib.lancet_debug_scan_workspace_spin_limit(ws, 0, None) == 0
            il = to_np(got[1])
            marked = ((il[0] == -1) & (il[1] == -1)).any()
            try:
                call.check()
                assert not marked
            except pkg.raf_executor.RafError as e:
                raised += 1
                assert "gave up a wait" in str(e)
            got = call.run()
            call.check()              # the word was cleared by the check that raised
            np.testing.assert_array_equal(to_np(got[1]), want[1])
            np.testing.assert_array_equal(to_np(got[4]), want[4])
        assert raised > 0
    finally:
        call.close()

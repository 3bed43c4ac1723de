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

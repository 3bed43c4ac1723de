"""GPU parity tests of the MoE dispatch path: HIP kernels (through the C ABI) against the
NumPy oracle on the same seeded inputs.

Bar: expert indices, locations, used capacity, elements_per_expert and scattered rows
bit-exact; softmax gate values within 1e-5 relative; decode bit-exact in fp32 (the kernel
rounds exactly like the oracle: fp32 products, fp32 sum, no fused multiply-add) and within
1 bf16/fp16 ulp for 16-bit rows.
"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, rows_as_oracle, rows_to_torch, to_np

pytestmark = pytest.mark.gpu

GATE_RTOL = 1e-5


def check_encode(got, want, gate_exact):
    g, il, used, elems, disp = got
    wg, wil, wused, welems, wdisp = want
    np.testing.assert_array_equal(to_np(il), wil)
    np.testing.assert_array_equal(to_np(used), wused)
    np.testing.assert_array_equal(to_np(elems), welems)
    if gate_exact:
        np.testing.assert_array_equal(to_np(g), wg)
    else:
        np.testing.assert_allclose(to_np(g), wg, rtol=GATE_RTOL, atol=0)
    np.testing.assert_array_equal(to_np(disp), wdisp)


# ----------------------------------------------------------------------------- moe_encode, top-1
@pytest.mark.parametrize("S,M,E,cf", [
    (1024, 128, 32, 1.0), (2048, 128, 64, 1.0),      # reference test shapes (test_cuda_moe.py:88-91)
    (4096, 768, 8, 1.25),                             # BASELINE config 1
    (1000, 36, 7, 0.5), (255, 8, 3, 1.0), (257, 12, 5, 2.0), (1, 4, 2, 1.0), (64, 4, 1, 1.0),
    (3000, 16, 128, 1.5), (777, 20, 200, 3.0),
])
@pytest.mark.parametrize("is_logits", [False, True])
def test_encode_top1(pkg, S, M, E, cf, is_logits):
    data, logits = make_inputs(S * 7 + E, S, M, E)
    gate = logits if is_logits else mo.softmax_rows(logits)
    used0 = np.zeros(E, np.int32)
    want = mo.moe_encode(data, gate, used0, cf, gate_is_logits=is_logits, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(gate), dev(used0), cf, gate_is_logits=is_logits)
    check_encode(got, want, gate_exact=not is_logits)


def _softmax64(logits):
    x = logits.astype(np.float64)
    ex = np.exp(x - x.max(axis=1, keepdims=True))
    return ex / ex.sum(axis=1, keepdims=True)


@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("S,E,scale,close", [(4096, 32, 30.0, False), (4096, 512, 30.0, False), (4096, 32, 1.0, True),
                                             (3000, 512, 4.0, True), (300000, 64, 30.0, False)])
def test_softmax_gates_for_wide_rows_and_close_runner_ups(pkg, k, S, E, scale, close):
    """The fused softmax where it is hardest: logits of scale 30 (|x - max| of 30 to 150: the terms of the
    denominator span the whole fp32 range and the second probability is tiny), rows of 512 experts, and rows
    whose runner-up lies within 1e-3 of the maximum (every second row: exactly equal, where the first must win).
    Selection bit-exact against the oracle; probabilities (lancet_gate_topk) and the op's gates_s at 1e-5 against
    the oracle AND against a float64 softmax evaluated here.  The last shape is long enough for the rows to be
    staged through LDS (rescaled running sum)."""
    import ctypes as C
    ops, capi = pkg.ops, pkg.capi
    TINY = 1.2e-38          # below the smallest normal fp32 a probability may be flushed or lose digits
    _, logits = make_inputs(S + E + int(scale), S, 1, E, logit_scale=scale)
    if close:
        rng = np.random.default_rng(1)
        top = logits.argmax(axis=1)
        other = (top + 1 + rng.integers(0, E - 1, S)) % E
        delta = (rng.random(S) * 1e-3).astype(np.float32)
        delta[::2] = 0.0
        logits[np.arange(S), other] = logits[np.arange(S), top] - delta
    sel, val = mo.select_topk(logits, k, True)
    p64 = _softmax64(logits)
    idx = torch.empty((k, S), dtype=torch.int32, device="cuda")
    prob = torch.empty((k, S), dtype=torch.float32, device="cuda")
    d_logits = dev(logits)
    st = capi.load().lancet_gate_topk(C.c_void_p(d_logits.data_ptr()), None, S, E, k, capi.F32, capi.GATE_IS_LOGITS,
                                      C.c_void_p(idx.data_ptr()), C.c_void_p(prob.data_ptr()), None)
    assert st == 0
    np.testing.assert_array_equal(to_np(idx), sel)
    np.testing.assert_allclose(to_np(prob), val, rtol=GATE_RTOL, atol=TINY)
    rows = np.arange(S)
    for j in range(k):
        np.testing.assert_allclose(to_np(prob)[j], p64[rows, sel[j]], rtol=GATE_RTOL, atol=TINY)
    # the op itself: routing bit-exact, gates_s (k = 2: normalised after the drop) at the same bar
    zero = np.zeros(E, np.int32)
    data = np.zeros((S, 4), np.float32)
    if k == 1:
        want = mo.moe_encode(data, logits, zero, 0.9, gate_is_logits=True, fast_scatter=True)
    else:
        want = mo.moe_encode_top2(data, logits, zero, 0.9, gate_is_logits=True, fast_scatter=True)
    got = ops.moe_encode(dev(data), d_logits, None, 0.9, top_k=k, gate_is_logits=True)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_allclose(to_np(got[0]), want[0], rtol=GATE_RTOL, atol=TINY)
    if k == 1:
        np.testing.assert_allclose(to_np(got[0]), p64[rows, sel[0]], rtol=GATE_RTOL, atol=TINY)
    else:
        g = [np.where(want[1][0, j * S:(j + 1) * S] >= 0, p64[rows, sel[j]], 0.0) for j in range(2)]
        den = np.maximum(g[0] + g[1], float(mo.F32_EPS))
        np.testing.assert_allclose(to_np(got[0]), np.concatenate([g[0] / den, g[1] / den]), rtol=GATE_RTOL, atol=TINY)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_encode_top1_16bit_rows(pkg, dt):
    S, M, E = 1500, 96, 16
    data, logits = make_inputs(3, S, M, E)
    gate = mo.softmax_rows(logits)
    used0 = np.zeros(E, np.int32)
    want = mo.moe_encode(rows_as_oracle(data, dt), gate, used0, 1.0, fast_scatter=True)
    got = pkg.ops.moe_encode(rows_to_torch(data, dt), dev(gate), dev(used0), 1.0)
    check_encode(got, want, gate_exact=True)


def test_encode_rows_not_16_byte_multiple(pkg):
    """M*4 = 20 bytes and M*2 = 10 bytes per row take the element-granular path."""
    S, M, E = 600, 5, 6
    data, logits = make_inputs(4, S, M, E)
    gate = mo.softmax_rows(logits)
    used0 = np.zeros(E, np.int32)
    for dt in ("f32", "bf16"):
        want = mo.moe_encode(rows_as_oracle(data, dt), gate, used0, 1.0, fast_scatter=True)
        got = pkg.ops.moe_encode(rows_to_torch(data, dt), dev(gate), dev(used0), 1.0)
        check_encode(got, want, gate_exact=True)


def test_encode_edge_routing(pkg):
    S, M, E = 900, 8, 8
    data, logits = make_inputs(5, S, M, E, ties=True)
    # ties, an expert nobody chooses, an expert that is full on entry, one that overflows
    logits[:, 3] = -50.0
    logits[::3, 1] = 40.0
    C = mo.capacity(S, E, 1.0)
    used_in = np.array([0, 5, C, 0, C // 2, 1, C - 1, C], np.int32)
    want = mo.moe_encode(data, logits, used_in, 1.0, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), dev(used_in), 1.0)
    check_encode(got, want, gate_exact=True)
    # capacity 0: everything dropped, empty buffer
    want = mo.moe_encode(data, logits, np.zeros(E, np.int32), 0.0, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), dev(np.zeros(E, np.int32)), 0.0)
    assert got[4].shape == (E, 0, M)
    check_encode(got, want, gate_exact=True)
    # all tokens to one expert
    logits[:, 2] = 99.0
    want = mo.moe_encode(data, logits, np.zeros(E, np.int32), 1.0, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), None, 1.0)
    check_encode(got, want, gate_exact=True)


def test_encode_empty_batch(pkg):
    E, M = 4, 8
    got = pkg.ops.moe_encode(torch.empty((0, M), device="cuda"), torch.empty((0, E), device="cuda"),
                             dev(np.array([1, 0, 2, 0], np.int32)), 1.0)
    assert got[0].numel() == 0 and got[1].shape == (2, 0) and got[4].shape == (E, 0, M)
    np.testing.assert_array_equal(to_np(got[2]), [0, 0, 0, 0])   # min(used_in + 0, C = 0)


# ----------------------------------------------------------------------------- chained partitions
@pytest.mark.parametrize("P,E,S0,M", [(2, 2, 1024, 512), (4, 2, 1024, 512), (4, 16, 2048, 64), (3, 5, 999, 8)])
def test_partitioned_encode_merge_redispatch(pkg, P, E, S0, M):
    """tests/python/op/cuda/test_cuda_moe.py:384-471: partitioned == un-partitioned."""
    ops = pkg.ops
    data, logits = make_inputs(17 + P, S0, M, E)
    gate = mo.softmax_rows(logits)
    S = S0 // P
    d_data, d_gate = dev(data), dev(gate)
    used = dev(np.zeros(E, np.int32))
    ils, bufs, gs, o_ils, o_bufs = [], [], [], [], []
    o_used = np.zeros(E, np.int32)
    for p in range(P):
        sl = slice(p * S, (p + 1) * S)
        g, il, used, elems, disp = ops.moe_encode(d_data[sl].contiguous(), d_gate[sl].contiguous(), used, float(P))
        og, oil, o_used, oelems, odisp = mo.moe_encode(data[sl], gate[sl], o_used, float(P), fast_scatter=True)
        check_encode((g, il, used, elems, disp), (og, oil, o_used, oelems, odisp), gate_exact=True)
        ils.append(il), bufs.append(disp), gs.append(g), o_ils.append(oil), o_bufs.append(odisp)
    merged = ops.moe_merge_masks(ils, E)
    red = ops.moe_redispatch(bufs, ils)
    np.testing.assert_array_equal(to_np(merged), mo.moe_merge_masks(o_ils, E))
    np.testing.assert_array_equal(to_np(red), mo.moe_redispatch(o_bufs, o_ils))
    if S * P == S0:
        # against the un-partitioned op (same capacity: cf*P per partition == cf on the whole batch
        # whenever ceil(S/E)*P == ceil(S0/E))
        ref = mo.moe_encode(data, gate, np.zeros(E, np.int32), 1.0, fast_scatter=True)
        if ref[4].shape == tuple(red.shape):
            ril = ref[1].copy()
            ril[1, ril[0] < 0] = -1
            np.testing.assert_array_equal(to_np(merged), ril)
            np.testing.assert_array_equal(to_np(red), ref[4])


# ----------------------------------------------------------------------------- top-2 extension
@pytest.mark.parametrize("S,M,E,cf,dt", [(2048, 64, 16, 1.0, "f32"), (2048, 64, 16, 1.0, "bf16"),
                                         (1111, 24, 5, 0.6, "f32"), (4096, 32, 32, 1.25, "bf16"),
                                         (300, 8, 2, 0.5, "f32")])
def test_encode_top2(pkg, S, M, E, cf, dt):
    data, logits = make_inputs(S + E, S, M, E, zipf_bias=True)
    used0 = np.zeros(E, np.int32)
    want = mo.moe_encode_top2(rows_as_oracle(data, dt), logits, used0, cf, gate_is_logits=True, fast_scatter=True)
    got = pkg.ops.moe_encode(rows_to_torch(data, dt), dev(logits), dev(used0), cf, top_k=2, gate_is_logits=True)
    check_encode(got, want, gate_exact=False)
    assert (want[1][0] < 0).any(), "config must drop tokens"


def test_top2_equals_two_chained_top1_encodes(pkg):
    """The identity that defines the extension: top-2 == encode(choice 1) -> encode(choice 2,
    used = out 1) -> merge_masks -> redispatch with the reference's top-1 semantics."""
    ops = pkg.ops
    S, M, E, cf = 1536, 32, 8, 0.75
    data, logits = make_inputs(99, S, M, E, zipf_bias=True)
    probs = mo.softmax_rows(logits)
    sel, val = mo.select_topk(logits, 2, True)
    # gate arrays whose argmax is the k-th choice and whose max is that choice's probability
    gates = []
    for j in range(2):
        g = np.full((S, E), -1.0, np.float32)
        g[np.arange(S), sel[j]] = val[j]
        gates.append(g)
    d_data = dev(data)
    used = dev(np.zeros(E, np.int32))
    ils, bufs, raw = [], [], []
    for j in range(2):
        g, il, used, elems, disp = ops.moe_encode(d_data, dev(gates[j]), used, 2 * cf)
        ils.append(il), bufs.append(disp), raw.append(g)
    merged = ops.moe_merge_masks(ils, E)
    red = ops.moe_redispatch(bufs, ils)
    weights = ops.moe_top2_normalize_gates(torch.cat(raw), merged)
    fused = ops.moe_encode(d_data, dev(logits), dev(np.zeros(E, np.int32)), cf, top_k=2, gate_is_logits=True)
    np.testing.assert_array_equal(to_np(merged), to_np(fused[1]))
    np.testing.assert_array_equal(to_np(red), to_np(fused[4]))
    np.testing.assert_array_equal(to_np(used), to_np(fused[2]))
    np.testing.assert_allclose(to_np(weights), to_np(fused[0]), rtol=GATE_RTOL)
    del probs


# ----------------------------------------------------------------------------- batch prioritised
@pytest.mark.parametrize("S0,M,E,P,cf,ties", [
    (1024, 128, 32, 1, 1.0, False), (2048, 128, 64, 1, 1.0, False),   # test_cuda_moe.py:160-163
    (1024, 512, 16, 4, 4.0, False),                                    # test_cuda_moe.py:1316
    (2000, 16, 8, 1, 0.5, True), (1536, 8, 6, 3, 1.5, True), (4096, 8, 64, 4, 2.0, False),
    (700, 4, 3, 1, 5.0, False),                                        # nothing dropped
    # more keys per expert than the select kernel keeps on chip (10240): it fetches them again in every pass
    (36000, 4, 2, 1, 0.5, False), (40000, 4, 2, 4, 0.75, True),
    (19000, 4, 2, 2, 0.6, True),                                       # about that limit: one expert over, one under
    (1050000, 2, 4, 2, 0.5, True),                                     # more than 4096 tiles: the batch is read whole
])
def test_encode_bpr(pkg, S0, M, E, P, cf, ties):
    data, logits = make_inputs(S0 + P, S0, M, E, logit_scale=2.0, ties=ties)
    gate = mo.softmax_rows(logits)
    if ties:
        gate = (np.round(gate * 16) / 16).astype(np.float32)   # many equal priorities
    d_data, d_gate = dev(data), dev(gate)
    for pid in range(P):
        want = mo.moe_encode_bpr(data, gate, P, pid, cf, fast_scatter=True)
        got = pkg.ops.moe_encode_batch_prioritized(d_data, d_gate, P, pid, cf)
        check_encode(got, want, gate_exact=True)


def test_encode_bpr_on_logits_resorts_emitted_priorities(pkg):
    """With logits the priorities are softmax values computed on the device; exp() is not
    bit-portable, so the oracle re-sorts the priorities the device emitted (checked at 1e-5)."""
    S0, M, E = 4096, 16, 16
    data, logits = make_inputs(7, S0, M, E, logit_scale=2.0)
    got = pkg.ops.moe_encode_batch_prioritized(dev(data), dev(logits), 1, 0, 0.5, gate_is_logits=True)
    prio = to_np(got[0])
    want = mo.moe_encode_bpr(data, logits, 1, 0, 0.5, gate_is_logits=True, priorities=prio, fast_scatter=True)
    np.testing.assert_allclose(prio, want[0], rtol=GATE_RTOL)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_array_equal(to_np(got[4]), want[4])


# ----------------------------------------------------------------------------- decode
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("S,M,E", [(1024, 128, 32), (777, 40, 6), (300, 5, 4)])
def test_decode(pkg, dt, k, S, M, E):
    ops = pkg.ops
    data, logits = make_inputs(S + k, S, M, E, zipf_bias=True)
    rows = rows_as_oracle(data, dt)
    used0 = np.zeros(E, np.int32)
    if k == 1:
        g, il, _, _, disp = mo.moe_encode(rows, mo.softmax_rows(logits), used0, 0.8, fast_scatter=True)
    else:
        g, il, _, _, disp = mo.moe_encode_top2(rows, logits, used0, 0.8, gate_is_logits=True, fast_scatter=True)
    # an "expert" that is not the identity, so that the two slots carry different rows
    expert_out = rows_as_oracle((disp * np.float32(1.5) + np.float32(0.25)).astype(np.float32), dt)
    want32 = mo.moe_decode(expert_out, g, il, k=k)
    got = ops.moe_decode(rows_to_torch(expert_out, dt), dev(g), dev(il), top_k=k)
    if dt == "f32":
        np.testing.assert_array_equal(to_np(got), want32)
    else:
        tdt = torch.bfloat16 if dt == "bf16" else torch.float16
        want = torch.from_numpy(want32).to(tdt)
        # same fp32 value rounded once on both sides: identical bits expected; the documented
        # tolerance is 1 ulp of the storage type
        a = got.cpu().view(torch.int16).to(torch.int32)
        b = want.view(torch.int16).to(torch.int32)
        assert int((a - b).abs().max()) <= 1
    dropped = (il[0, :S] < 0) if k == 1 else ((il[0, :S] < 0) & (il[0, S:] < 0))
    assert dropped.any() and not to_np(got)[dropped].any()


def test_decode_roundtrip_identity_expert(pkg):
    """decode(encode(x), gate = 1) == x on kept tokens, 0 on dropped ones (bit-exact)."""
    ops = pkg.ops
    S, M, E = 2048, 128, 32
    data, logits = make_inputs(123, S, M, E)
    d_data = dev(data)
    g, il, used, elems, disp = ops.moe_encode(d_data, dev(mo.softmax_rows(logits)), None, 0.9)
    out = ops.moe_decode(disp, torch.ones_like(g), il)
    kept = (il[0] >= 0)
    assert torch.equal(out[kept], d_data[kept]) and not out[~kept].any() and (~kept).any()


# ----------------------------------------------------------------------------- launcher level
# the scan in each of its forms: one look-back kernel (12 tiles), count + place (79), count + segment sums + place (1172)
@pytest.mark.parametrize("S,E", [(3000, 12), (20000, 12), (300000, 64)])
def test_launch_gen_location_and_encode_forward(pkg, S, E):
    import ctypes as C
    lib = pkg.capi.load()
    M, cf = 16, 0.7
    data, logits = make_inputs(31, S, M, E)
    Cap = mo.capacity(S, E, cf)
    idx0 = np.argmax(logits, axis=1).astype(np.int32)
    used_in = np.array([0, 3] * (E // 2), np.int32)
    widx, wloc, wused, welems = mo.gen_location(idx0, used_in, Cap, M, E)
    d_idx, d_used = dev(idx0), dev(used_in)
    d_loc = torch.empty(S, dtype=torch.int32, device="cuda")
    d_uo = torch.empty(E, dtype=torch.int32, device="cuda")
    d_el = torch.empty(E, dtype=torch.int64, device="cuda")
    nws = lib.lancet_gen_location_workspace_bytes(S, E)
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    assert lib.lancet_scan_workspace_init(p(ws), nws, None) == 0
    st = lib.lancet_launch_gen_location(p(d_idx), p(d_used), p(d_loc), p(d_uo), p(d_el), Cap, S, E, M, p(ws), nws, None)
    assert st == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(d_idx), widx)
    np.testing.assert_array_equal(to_np(d_loc), wloc)
    np.testing.assert_array_equal(to_np(d_uo), wused)
    np.testing.assert_array_equal(to_np(d_el).astype(np.uint64), welems)
    # scatter with and without the used-capacity test
    d_data = dev(data)
    for capused in (d_used, None):
        out = torch.full((E, Cap, M), 7.0, device="cuda")
        st = lib.lancet_launch_encode_forward(p(d_idx), p(d_loc), p(capused) if capused is not None else None,
                                              p(d_data), p(out), S, M, Cap, E, pkg.capi.F32, None)
        assert st == 0
        torch.cuda.synchronize()
        avail = (Cap - used_in) if capused is not None else None
        np.testing.assert_array_equal(to_np(out), mo.scatter_rows(data, widx, wloc, E, Cap, avail))


@pytest.mark.parametrize("k", [1, 2])
def test_bounded_wait_flags_the_workspace(pkg, k):
    """A spin limit of 1 makes look-back waits give up at once: the kernels must still finish; a call in which a
    wait gave up sets the workspace's sticky error word and shows it in its outputs without a synchronisation
    (used_capacity = -1, and -1 for every token whose position depended on the wait); every token that is not
    marked has its correct position; the default limit leaves the word clear and the next call is whole."""
    import ctypes as C
    lib = pkg.capi.load()
    ops = pkg.ops
    S, M, E = 131072, 4, 256         # 512 tiles; scan_lookback asks for the look-back form (the default forms have no waits)
    data, logits = make_inputs(1, S, M, E)
    d_data, d_gate = dev(data), dev(logits)
    enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
    want = enc(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, k))
    ops.moe_encode(d_data, d_gate, None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=True)
    assert ws.error() == 0
    gave_up = 0
    for _ in range(3):
        assert lib.lancet_debug_scan_workspace_spin_limit(C.c_void_p(ws.buf.data_ptr()), 1, None) == 0
        got = ops.moe_encode(d_data, d_gate, None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=True)
        assert lib.lancet_debug_scan_workspace_spin_limit(C.c_void_p(ws.buf.data_ptr()), 0, None) == 0
        torch.cuda.synchronize()   # terminates
        il, used = to_np(got[1]), to_np(got[2])
        flagged = ws.error()       # 1 whenever a predecessor's word was not there at the first poll
        assert ws.error() == 0     # the reader clears the word
        marked = (il[0] == -1) & (il[1] == -1) & (want[1] != -1).any(axis=0)   # marks (a dropped slot of top-2 looks the same)
        differs = (il != want[1]).any(axis=0)
        if k == 2:
            assert not (differs & ~marked).any(), "what is not marked is right"
            assert (to_np(got[0])[marked] == 0).all()
        else:
            # dropped tokens of the top-1 op keep idx -1 and their rank: marks are (-1, -1)
            np.testing.assert_array_equal(il[:, ~((il[0] == -1) & (il[1] == -1))], want[1][:, ~((il[0] == -1) & (il[1] == -1))])
        if marked.any():           # some position was built on a wait that gave up
            gave_up += 1
            assert flagged == 1
        assert (used == -1).all() or np.array_equal(used, want[2])
        if (used == -1).all():
            assert flagged == 1
            if k == 2:
                assert (il == -1).all()
        # the workspace is ready for the next call whatever happened
        got = ops.moe_encode(d_data, d_gate, None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=True)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[2]), want[2])
        np.testing.assert_array_equal(to_np(got[4]), want[4])
        assert ws.error() == 0
    assert gave_up > 0, "512 tiles with a wait of one poll: some wait gives up"


def test_scan_epoch_wraps(pkg):
    """The call that runs with the last epoch clears the descriptor table and the epoch starts again at 1: calls
    before, at and after the wrap give the right routing, also when the table holds words tagged with the
    epochs that come round again."""
    import ctypes as C
    lib = pkg.capi.load()
    ops = pkg.ops
    ws = ops.ScanWorkspace(1 << 20)
    last = (1 << 30) - 1
    cases = [(5000, 32, 2), (9000, 16, 1), (3000, 8, 2)]
    wants = []
    for i, (S, E, k) in enumerate(cases):
        data, logits = make_inputs(400 + i, S, 8, E)
        enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
        wants.append((dev(data), dev(logits), enc(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)))

    def run_all():
        # every case as one look-back kernel (the form that draws epochs) and in the form it takes by default
        # (no look-back at these sizes: its words in the table must never pass for descriptors)
        for (S, E, k), (d, g, want) in zip(cases, wants):
            for lookback in (True, False):
                got = ops.moe_encode(d, g, None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=lookback)
                np.testing.assert_array_equal(to_np(got[1]), want[1])
                np.testing.assert_array_equal(to_np(got[2]), want[2])
                np.testing.assert_allclose(to_np(got[0]), want[0], rtol=1e-5)

    run_all()                      # epochs 1..3: their words stay in the table
    for start in (last - 4, last - 1, last):
        assert lib.lancet_debug_scan_workspace_epoch(C.c_void_p(ws.buf.data_ptr()), start, None) == 0
        for _ in range(3):
            run_all()              # crosses the wrap and meets epochs 1..3 again
    assert ws.error() == 0
    # a batch-prioritised call as the one that wraps (its scan has two counter sets and scratch behind the table)
    data, logits = make_inputs(410, 20000, 8, 16)
    gate = mo.softmax_rows(logits)
    want = mo.moe_encode_bpr(data, gate, 1, 0, 1.0, fast_scatter=True)
    assert lib.lancet_debug_scan_workspace_epoch(C.c_void_p(ws.buf.data_ptr()), last, None) == 0
    for lookback in (True, True, False, True):
        got = ops.moe_encode_batch_prioritized(dev(data), dev(gate), 1, 0, 1.0, workspace=ws, scan_lookback=lookback)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[2]), want[2])
    run_all()
    assert ws.error() == 0


def test_scan_on_a_workspace_that_is_not_set_up(pkg):
    """A call handed memory that lancet_scan_workspace_init never saw must not hang or run wild: the look-back form of
    the scan (top-1 on few tiles here) marks its outputs (-1) and sets the error word, and after the set-up the same
    memory works; the form without waits (top-2 here) keeps no state and simply gives the right result."""
    import ctypes as C
    lib = pkg.capi.load()
    capi = pkg.capi
    S, M, E = 3000, 8, 8
    data, logits = make_inputs(2, S, M, E)
    d_data, d_gate = dev(data), dev(logits)
    p = lambda t: C.c_void_p(t.data_ptr())
    for k in (1, 2):
        nws = int(lib.lancet_moe_encode_workspace_bytes(S, E, k))
        for fill in (0, 0xff):
            ws = torch.full((nws,), fill, dtype=torch.uint8, device="cuda")
            Cap = ops_cap = pkg.ops.moe_capacity(S, E, float(k))
            outs = (torch.zeros(k * S, device="cuda"), torch.zeros((2, k * S), dtype=torch.int32, device="cuda"),
                    torch.zeros(E, dtype=torch.int32, device="cuda"), torch.zeros(E, dtype=torch.int64, device="cuda"),
                    torch.zeros((E, Cap, M), device="cuda"))
            st = lib.lancet_moe_encode(p(d_data), p(d_gate), None, None, S, M, E, Cap, k, capi.F32, capi.F32, capi.GATE_IS_LOGITS,
                                       *[p(t) for t in outs], p(ws), nws, None)
            assert st == 0
            torch.cuda.synchronize()
            err = C.c_int(0)
            if k == 1:
                assert (to_np(outs[1]) == -1).all() and (to_np(outs[2]) == -1).all()
                assert (to_np(outs[4]) == 0).all(), "no token has a place: the buffer is all tail"
                assert lib.lancet_scan_workspace_error(p(ws), None, C.byref(err)) == 0 and err.value == 1
            else:
                want = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
                np.testing.assert_array_equal(to_np(outs[1]), want[1])
                np.testing.assert_array_equal(to_np(outs[4]), want[4])
            assert lib.lancet_scan_workspace_init(p(ws), nws, None) == 0
            st = lib.lancet_moe_encode(p(d_data), p(d_gate), None, None, S, M, E, Cap, k, capi.F32, capi.F32, capi.GATE_IS_LOGITS,
                                       *[p(t) for t in outs], p(ws), nws, None)
            assert st == 0
            enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
            want = enc(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
            np.testing.assert_array_equal(to_np(outs[1]), want[1])
            np.testing.assert_array_equal(to_np(outs[4]), want[4])
            assert lib.lancet_scan_workspace_error(p(ws), None, C.byref(err)) == 0 and err.value == 0


def test_top2_lookback_on_a_workspace_with_a_damaged_ticket(pkg):
    """A set-up workspace that served a healthy top-2 look-back call, then has only its ticket word damaged (as a
    call that overlapped another on the same workspace leaves it): no tile of the next call can take part, none
    publishes, and the totals row still holds the healthy call's words.  The finalisation must not take them:
    every output is marked (-1, gates 0, used_capacity -1, no elements), the error word is set, and after a new
    set-up the workspace works."""
    ops = pkg.ops
    S, M, E = 6000, 8, 16
    data, logits = make_inputs(31, S, M, E)
    d_data, d_gate = dev(data), dev(logits)
    want = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, 2))
    for _ in range(2):
        got = ops.moe_encode(d_data, d_gate, None, 1.0, top_k=2, gate_is_logits=True, workspace=ws, scan_lookback=True)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
    assert ws.error() == 0
    ws.buf.view(torch.int32)[0] = 1 << 20                       # the ticket: far beyond the launch's tiles
    got = ops.moe_encode(d_data, d_gate, None, 1.0, top_k=2, gate_is_logits=True, workspace=ws, scan_lookback=True)
    torch.cuda.synchronize()
    assert (to_np(got[1]) == -1).all() and (to_np(got[2]) == -1).all()
    assert not to_np(got[0]).any() and not to_np(got[3]).any() and not to_np(got[4]).any()
    assert ws.error() == 1
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, 2))
    got = ops.moe_encode(d_data, d_gate, None, 1.0, top_k=2, gate_is_logits=True, workspace=ws, scan_lookback=True)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    assert ws.error() == 0


def test_scan_workspace_is_reused_across_shapes(pkg):
    """One workspace, calls of different token counts, expert counts and top_k one after the other: descriptor
    words of earlier calls lie anywhere in the table and must never be taken for the running call's."""
    ops = pkg.ops
    ws = ops.ScanWorkspace(1 << 20)
    rng = np.random.default_rng(5)
    shapes = [(5000, 32, 2), (700, 8, 1), (5000, 32, 1), (2049, 64, 2), (256, 2, 2), (5000, 32, 2), (1, 4, 1), (4097, 16, 1)]
    for i, (S, E, k) in enumerate(shapes * 2):
        data, logits = make_inputs(200 + i, S, 8, E)
        enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
        want = enc(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
        # the look-back form and the forms without waits alternate on the one workspace
        got = ops.moe_encode(dev(data), dev(logits), None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=i % 2 == 0)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[2]), want[2])
        if i % 3 == 0:   # batch-prioritised calls share it too
            gate = mo.softmax_rows(logits)
            wb = mo.moe_encode_bpr(data, gate, 1, 0, 1.0, fast_scatter=True)
            gb = ops.moe_encode_batch_prioritized(dev(data), dev(gate), 1, 0, 1.0, workspace=ws, scan_lookback=i % 2 == 1)
            np.testing.assert_array_equal(to_np(gb[1]), wb[1])
    # the batch-prioritised call keeps per-token data behind its descriptor table, where a later call with a
    # larger table expects descriptors: small expert ids and arbitrary floats must not pass for them
    data, logits = make_inputs(300, 32768, 8, 8)
    gate = mo.softmax_rows(logits)
    wb = mo.moe_encode_bpr(data, gate, 1, 0, 1.0, fast_scatter=True)
    gb = ops.moe_encode_batch_prioritized(dev(data), dev(gate), 1, 0, 1.0, workspace=ws)
    np.testing.assert_array_equal(to_np(gb[1]), wb[1])
    for i, (S, E, k) in enumerate([(20000, 32, 2), (32768, 64, 1), (9000, 128, 2)]):
        data, logits = make_inputs(310 + i, S, 8, E)
        enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
        want = enc(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
        for lookback in (True, False):
            got = ops.moe_encode(dev(data), dev(logits), None, 1.0, top_k=k, gate_is_logits=True, workspace=ws, scan_lookback=lookback)
            np.testing.assert_array_equal(to_np(got[1]), want[1])
            np.testing.assert_array_equal(to_np(got[2]), want[2])
    assert ws.error() == 0


def test_encode_without_tail_zero_fill_feeds_redispatch(pkg):
    """zero_tail=False writes the used rows only: they equal the zero-filled encode's rows, the rest of
    the buffer keeps what it held, and moe_redispatch over such partition buffers is unchanged."""
    ops = pkg.ops
    S0, M, E, P = 2048, 64, 8, 4
    data, logits = make_inputs(77, S0, M, E, zipf_bias=True)
    gate = dev(mo.softmax_rows(logits))
    d_data = dev(data)
    S = S0 // P
    Cap = ops.moe_capacity(S, E, float(P))
    used_a = used_b = None
    ils, bufs_a, bufs_b = [], [], []
    for p_ in range(P):
        sl = slice(p_ * S, (p_ + 1) * S)
        a = ops.moe_encode(d_data[sl], gate[sl], used_a, float(P))
        out_b = (torch.empty(S, device="cuda"), torch.empty((2, S), dtype=torch.int32, device="cuda"),
                 torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
                 torch.full((E, Cap, M), 7.0, device="cuda"))
        b = ops.moe_encode(d_data[sl], gate[sl], used_b, float(P), zero_tail=False, out=out_b)
        kept = (a[2] - (used_a if used_a is not None else 0)).long()
        rows = torch.arange(Cap, device="cuda")[None, :] < kept[:, None]
        assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
        assert torch.equal(a[4][rows], b[4][rows]) and bool((b[4][~rows] == 7.0).all())
        used_a, used_b = a[2], b[2]
        ils.append(a[1]), bufs_a.append(a[4]), bufs_b.append(b[4])
    assert torch.equal(ops.moe_redispatch(bufs_a, ils), ops.moe_redispatch(bufs_b, ils))


# ----------------------------------------------------------------------------- redispatch_expert_input
@pytest.mark.parametrize("dt,M", [("f32", 64), ("bf16", 128), ("f32", 5)])
@pytest.mark.parametrize("P", [2, 4])
def test_redispatch_expert_input(pkg, dt, M, P):
    """tests/python/distributed/test_partitioned_moe.py:99-196 with synthetic all-to-all outputs: every
    source GPU's received rows are split over P partitions; the merge restores them.  Also counts that
    are not a multiple of M (element-granular streams) and a scale factor."""
    ops = pkg.ops
    rng = np.random.default_rng(P * 10 + M)
    C, G, LE, le = 40, 8, 2, 1
    whole = rows_as_oracle(rng.standard_normal((C, G, M), dtype=np.float32), dt)
    rows_total = rng.integers(0, C + 1, G)
    rows_total[0], rows_total[1] = 0, C
    bufs = [rows_as_oracle(rng.standard_normal((C, G, M), dtype=np.float32), dt) for _ in range(P)]
    cnts = [np.zeros(G * LE, np.uint64) for _ in range(P)]
    for g in range(G):
        edges = [0] + list(np.sort(rng.integers(0, rows_total[g] + 1, P - 1))) + [rows_total[g]]
        for p in range(P):
            n = edges[p + 1] - edges[p]
            bufs[p][:n, g, :] = whole[edges[p]:edges[p + 1], g, :]
            cnts[p][g * LE + le] = n * M
            cnts[p][g * LE + (1 - le)] = 7 * M
    d_bufs = [rows_to_torch(b, dt) for b in bufs]
    d_cnts = [dev(c.astype(np.int64)) for c in cnts]
    want = mo.moe_redispatch_expert_input(bufs, cnts, le, LE)
    got = ops.moe_redispatch_expert_input(d_bufs, d_cnts, le, LE)
    np.testing.assert_array_equal(to_np(got), want)
    for g in range(G):
        np.testing.assert_array_equal(want[:rows_total[g], g], whole[:rows_total[g], g])
    # through the op layer, 4-D [C, 1, G, M] form
    ex = pkg.raf_executor.Executor()
    got4 = ex("raf.op.moe_redispatch_expert_input", [b.reshape(C, 1, G, M) for b in d_bufs], d_cnts, le, LE)
    assert tuple(got4.shape) == (C, 1, G, M)
    np.testing.assert_array_equal(to_np(got4).reshape(C, G, M), want)
    # element-granular streams with a scale factor
    cnts2 = [rng.integers(0, (C * M) // (2 * P), G * LE).astype(np.uint64) for _ in range(P)]
    want2 = mo.moe_redispatch_expert_input(bufs, cnts2, 0, LE, scale=2)
    got2 = ops.moe_redispatch_expert_input(d_bufs, [dev(c.astype(np.int64)) for c in cnts2], 0, LE, recv_cnts_scale=2)
    np.testing.assert_array_equal(to_np(got2), want2)


# ----------------------------------------------------------------------------- sparse <-> packed copies
@pytest.mark.parametrize("dt,dims", [("f32", (6, 10, 16)), ("bf16", (8, 12, 24)), ("bf16", (5, 7, 9)), ("f32", (3, 4, 5))])
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("aligned", [True, False])
def test_sparse_packed_copies(pkg, dt, dims, axis, aligned):
    """memcpy_sparse_to_cont_3d / memcpy_cont_to_sparse_3d (sparse_memcpy.cu:11-96) against the oracle, with
    counts read through a stride and an offset; `aligned` makes every count a multiple of dim2 (whole rows, what
    elements_per_expert holds), otherwise counts are arbitrary and block offsets fall inside 16-byte granules."""
    ops = pkg.ops
    rng = np.random.default_rng(sum(dims) + axis + 2 * aligned)
    d0, d1, d2 = dims
    nb = dims[axis]
    rows = d1 if axis == 0 else d0
    stride, offset = 3, 2
    cnt = rng.integers(0, 1000, nb * stride).astype(np.uint64)
    picked = rng.integers(0, rows + 1, nb) * d2 if aligned else rng.integers(0, rows * d2 + 1, nb)
    picked[0] = 0 if nb > 1 else picked[0]
    picked[-1] = rows * d2
    cnt[offset::stride] = picked
    total = int(picked.sum())
    src = rows_as_oracle(rng.standard_normal(dims, dtype=np.float32), dt)
    dst0 = rows_as_oracle(rng.standard_normal(total + 5, dtype=np.float32), dt)
    d_cnt = dev(cnt.astype(np.int64))
    want = mo.memcpy_sparse_to_cont_3d(src, dst0, cnt, stride, offset, axis)
    got = ops.memcpy_sparse_to_cont_3d(rows_to_torch(src, dt), rows_to_torch(dst0, dt), d_cnt, stride, offset, axis)
    np.testing.assert_array_equal(to_np(got), want)
    for zero_tail in (False, True):
        buf0 = rows_as_oracle(rng.standard_normal(dims, dtype=np.float32), dt)
        want3 = mo.memcpy_cont_to_sparse_3d(want, buf0, cnt, stride, offset, axis, zero_tail=zero_tail)
        got3 = ops.memcpy_cont_to_sparse_3d(rows_to_torch(want, dt), rows_to_torch(buf0, dt), d_cnt, stride, offset,
                                            axis, zero_tail=zero_tail)
        np.testing.assert_array_equal(to_np(got3), want3)
    # a packed array shorter than the counts say: the copy stops at its end
    short = max(total - d2 - 1, 0)
    want_s = mo.memcpy_sparse_to_cont_3d(src, dst0[:short], cnt, stride, offset, axis)
    got_s = ops.memcpy_sparse_to_cont_3d(rows_to_torch(src, dt), rows_to_torch(dst0[:short].copy(), dt), d_cnt, stride,
                                         offset, axis)
    np.testing.assert_array_equal(to_np(got_s), want_s)


def test_sparse_packed_copies_scale_and_encode_counts(pkg):
    """Counts straight from an encode (elements_per_expert) pack the dispatched buffer; scale/shrink reinterpret
    the counts for another element size (sparse_memcpy.cu:33-36)."""
    ops = pkg.ops
    rng = np.random.default_rng(11)
    S, M, E = 4096, 256, 16
    x = rng.standard_normal((S, M), dtype=np.float32)
    gate = mo.softmax_rows(rng.standard_normal((S, E), dtype=np.float32) * 2)
    gates_s, indloc, used, elems, disp = ops.moe_encode(dev(x), dev(gate), torch.zeros(E, dtype=torch.int32, device="cuda"), 0.8)
    kept = int(used.sum().item())
    assert kept < S
    packed = ops.memcpy_sparse_to_cont_3d(disp, torch.empty(kept * M, device="cuda"), elems)
    want = np.concatenate([to_np(disp)[e, :int(used[e])].reshape(-1) for e in range(E)])
    np.testing.assert_array_equal(to_np(packed), want)
    back = ops.memcpy_cont_to_sparse_3d(packed, torch.full_like(disp, 3.0), elems, zero_tail=True)
    np.testing.assert_array_equal(to_np(back), to_np(disp))
    # the same counts, read as fp32 elements, drive a bf16 buffer of twice the width (scale 2)
    disp16 = rows_as_oracle(rng.standard_normal((E, disp.shape[1], 2 * M), dtype=np.float32), "bf16")
    cnt = to_np(elems).astype(np.uint64)
    want16 = mo.memcpy_sparse_to_cont_3d(disp16, np.zeros(2 * kept * M, disp16.dtype), cnt, scale=2)
    got16 = ops.memcpy_sparse_to_cont_3d(rows_to_torch(disp16, "bf16"), rows_to_torch(np.zeros(2 * kept * M, disp16.dtype), "bf16"),
                                         elems, scale_element_size_by=2)
    np.testing.assert_array_equal(to_np(got16), want16)
    want_h = mo.memcpy_sparse_to_cont_3d(disp16, np.zeros(kept * M, disp16.dtype), cnt, scale=1, shrink=2)
    got_h = ops.memcpy_sparse_to_cont_3d(rows_to_torch(disp16, "bf16"), rows_to_torch(np.zeros(kept * M, disp16.dtype), "bf16"),
                                         elems, shrink_element_size_by=2)
    np.testing.assert_array_equal(to_np(got_h), want_h)


# ----------------------------------------------------------------------------- route / scatter halves
@pytest.mark.parametrize("k,dt", [(1, "f32"), (2, "bf16"), (1, "f16")])
def test_route_then_scatter_equals_encode(pkg, k, dt):
    """lancet_moe_route + lancet_moe_scatter (the two halves of MoeEncode::Execute, moe.cc:366-380 and
    :381-395) give what moe_encode gives, with used capacity carried in."""
    ops = pkg.ops
    S, M, E, cf = 1500, 48, 12, 0.75
    data, logits = make_inputs(5 + k, S, M, E, zipf_bias=True)
    Cap = ops.moe_capacity(S, E, cf * k)
    used0 = np.zeros(E, np.int32) if k == 2 else np.random.default_rng(1).integers(0, Cap // 2, E).astype(np.int32)
    d_data, d_gate, d_used = rows_to_torch(data, dt), dev(logits), dev(used0)
    whole = ops.moe_encode(d_data, d_gate, d_used, cf, top_k=k, gate_is_logits=True)
    gates_s, indloc, used_out, elems = ops.moe_route(d_gate, d_used, M, cf, top_k=k, gate_is_logits=True)
    disp = ops.moe_scatter(d_data, indloc, d_used, used_out, E, Cap, top_k=k)
    for a, b in zip(whole, (gates_s, indloc, used_out, elems, disp)):
        assert torch.equal(a.view(torch.int64) if a.dtype == torch.uint64 else a,
                           b.view(torch.int64) if b.dtype in (torch.uint64,) else b)
    assert (to_np(indloc)[0] < 0).any()


# ----------------------------------------------------------------------------- top-2 with second-choice noise
@pytest.mark.parametrize("dt,is_logits", [("f32", True), ("bf16", True), ("f32", False)])
def test_encode_top2_with_second_choice_noise(pkg, dt, is_logits):
    """gate2_noise stands for the Gumbel sample GShard adds before the second argmax
    (docker/resources/sharded_moe.py:275-278): it moves second choices, never the first, and gate values
    still come from the un-noised gate.  Through the op function, the routing half alone and the op layer."""
    ops = pkg.ops
    S, M, E, cf = 1800, 32, 10, 0.8
    data, logits = make_inputs(77, S, M, E, zipf_bias=True)
    gate = logits if is_logits else mo.softmax_rows(logits)
    noise = np.random.default_rng(8).gumbel(size=(S, E)).astype(np.float32) * np.float32(1.0 if is_logits else 0.05)
    x = rows_as_oracle(data, dt)
    used0 = np.zeros(E, np.int32)
    want = mo.moe_encode_top2(x, gate, used0, cf, gate_is_logits=is_logits, fast_scatter=True, gate2_noise=noise)
    plain = mo.moe_encode_top2(x, gate, used0, cf, gate_is_logits=is_logits, fast_scatter=True)
    assert (want[1][0, S:] != plain[1][0, S:]).any()
    d_x, d_gate, d_noise, d_used = rows_to_torch(data, dt), dev(gate), dev(noise), dev(used0)
    got = ops.moe_encode(d_x, d_gate, d_used, cf, top_k=2, gate_is_logits=is_logits, gate2_noise=d_noise)
    check_encode(got, want, gate_exact=not is_logits)
    routed = ops.moe_route(d_gate, d_used, M, cf, top_k=2, gate_is_logits=is_logits, gate2_noise=d_noise)
    np.testing.assert_array_equal(to_np(routed[1]), want[1])
    ex = pkg.raf_executor.Executor()
    outs = ex("raf.op.moe_encode", d_x, d_gate, d_used, cf, 2, int(is_logits), 1, d_noise)
    np.testing.assert_array_equal(to_np(outs[1]), want[1])
    np.testing.assert_array_equal(to_np(outs[4]), want[4])
    with pytest.raises(ValueError):
        ops.moe_encode(d_x, d_gate, d_used, cf, top_k=1, gate2_noise=d_noise)


# ----------------------------------------------------------------------------- partition encodes into one buffer
@pytest.mark.parametrize("P,E,S0,M,dt", [(4, 8, 2048, 64, "f32"), (3, 5, 999, 24, "bf16"), (2, 2, 512, 8, "f32")])
def test_chained_encodes_into_one_buffer_equal_redispatch(pkg, P, E, S0, M, dt):
    """LANCET_ROWS_AT_USED: partition encodes chained through used_capacity write their rows behind those of
    the earlier partitions, all into one [E, C, M] buffer, the last one zero-filling what is left.  The
    buffer is bit for bit what moe_redispatch builds from separate partition buffers
    (tests/python/op/cuda/test_cuda_moe.py:384-471 protocol), and also what one encode of the whole batch gives."""
    ops = pkg.ops
    S = S0 // P
    S0 = S * P
    cf = 0.75
    data, logits = make_inputs(P + E, S0, M, E, zipf_bias=True)
    gate = mo.softmax_rows(logits)
    d_data, d_gate = rows_to_torch(data, dt), dev(gate)
    Cap = ops.moe_capacity(S, E, cf * P)
    shared = torch.full((E, Cap, M), 7.0, dtype=d_data.dtype, device="cuda")   # stale contents must not survive
    used = torch.zeros(E, dtype=torch.int32, device="cuda")
    ils, bufs = [], []
    for p in range(P):
        sl = slice(p * S, (p + 1) * S)
        sep = ops.moe_encode(d_data[sl], d_gate[sl], used, cf * P)
        outs = (torch.empty(S, device="cuda"), torch.empty((2, S), dtype=torch.int32, device="cuda"),
                torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"), shared)
        one = ops.moe_encode(d_data[sl], d_gate[sl], used, cf * P, zero_tail=(p == P - 1), rows_at_used=True, out=outs)
        assert torch.equal(one[1], sep[1]) and torch.equal(one[2], sep[2])       # routing outputs are unchanged
        ils.append(sep[1])
        bufs.append(sep[4])
        used = sep[2]
    want = ops.moe_redispatch(bufs, ils)
    assert torch.equal(shared, want)
    assert (to_np(torch.stack(ils))[:, 0] < 0).any()                             # the case drops tokens
    if ops.moe_capacity(S0, E, cf) == Cap:
        whole = ops.moe_encode(d_data, d_gate, torch.zeros(E, dtype=torch.int32, device="cuda"), cf)
        assert torch.equal(shared, whole[4])


# ----------------------------------------------------------------------------- token ranges of a whole-batch routing
@pytest.mark.parametrize("k,dt,P,S,M,E", [(2, "bf16", 4, 2048, 64, 8), (1, "f32", 3, 999, 24, 5), (2, "f32", 2, 512, 5, 4),
                                          (2, "f16", 5, 1000, 40, 16)])
@pytest.mark.parametrize("with_used_in", [False, True])
def test_token_range_scatter_and_decode_equal_the_whole_batch(pkg, k, dt, P, S, M, E, with_used_in):
    """Route the whole batch once, then move rows range by range (lancet_moe_scatter_tokens /
    lancet_moe_decode_tokens): the buffer is bit for bit the one moe_encode builds for the batch (itself checked
    against the oracle), stale contents of the shared buffer do not survive, and the ranges' decodes are the
    rows of the whole-batch decode."""
    ops = pkg.ops
    cf = 0.75
    data, logits = make_inputs(S + k, S, M, E, zipf_bias=True)
    gate = mo.softmax_rows(logits)
    d_data, d_gate = rows_to_torch(data, dt), dev(gate)
    used_in = dev(np.arange(E, dtype=np.int32) % 3) if with_used_in else None
    g, il, used, elems, disp = ops.moe_encode(d_data, d_gate, used_in, cf, top_k=k)
    want_rows = mo.moe_encode_top2 if k == 2 else mo.moe_encode
    ref = want_rows(rows_as_oracle(data, dt), gate, to_np(used_in) if with_used_in else np.zeros(E, np.int32), cf)
    np.testing.assert_array_equal(to_np(disp), ref[4])
    assert (to_np(il)[0] < 0).any()
    C = disp.shape[1]
    shared = torch.full_like(disp, 5.0)
    bounds = [S * p // P for p in range(P + 1)]
    bounds[1] += 1                                   # ranges of unequal length, one of them odd
    for p in range(P):
        lo, hi = bounds[p], bounds[p + 1]
        ops.moe_scatter_tokens(d_data[lo:hi], il, used_in, used, lo, E, C, top_k=k, zero_tail=(p == 1), out=shared)
    assert torch.equal(shared, disp)
    whole = ops.moe_decode(disp, g, il, top_k=k)
    for p in range(P):
        lo, hi = bounds[p], bounds[p + 1]
        part = ops.moe_decode_tokens(shared, g, il, lo, hi - lo, top_k=k)
        assert torch.equal(part, whole[lo:hi])
    empty = ops.moe_decode_tokens(shared, g, il, S, 0, top_k=k)
    assert empty.shape == (0, M)
    with pytest.raises(ValueError):
        ops.moe_decode_tokens(shared, g, il, S - 1, 2, top_k=k)


# ----------------------------------------------------------------------------- non-finite gates
@pytest.mark.parametrize("mode", ["top1", "top2", "bpr"])
@pytest.mark.parametrize("is_logits", [False, True])
def test_non_finite_gates_keep_the_outputs_well_formed(pkg, mode, is_logits):
    """NaN and infinities in the gate: which expert such a token goes to is not pinned by anything the
    reference holds, but the outputs must stay well formed: experts in range, kept locations below the
    capacity and distinct per expert, counts consistent, rows copied bit for bit, no bounded wait tripped;
    tokens whose row is finite route exactly as in a batch without the bad rows' values."""
    ops = pkg.ops
    S, M, E, cf = 3000, 16, 8, 0.6
    data, logits = make_inputs(77, S, M, E)
    rng = np.random.default_rng(5)
    bad = rng.random(S) < 0.2
    vals = np.array([np.nan, np.inf, -np.inf], np.float32)
    poisoned = logits.copy()
    for s in np.nonzero(bad)[0]:
        k = rng.integers(1, E + 1)
        poisoned[s, rng.choice(E, k, replace=False)] = vals[rng.integers(0, 3, k)]
    d_data = dev(data)
    if mode == "bpr":
        g, il, used, elems, disp = ops.moe_encode_batch_prioritized(d_data, dev(poisoned), 1, 0, cf, gate_is_logits=is_logits)
        k = 1
    else:
        k = 2 if mode == "top2" else 1
        g, il, used, elems, disp = ops.moe_encode(d_data, dev(poisoned), None, cf, top_k=k, gate_is_logits=is_logits)
    torch.cuda.synchronize()
    il, used, elems, disp = to_np(il), to_np(used), to_np(elems), to_np(disp)
    C = disp.shape[1]
    idx, loc = il[0], il[1]
    assert idx.min() >= -1 and idx.max() < E
    kept = idx >= 0
    assert (loc[kept] >= 0).all() and (loc[kept] < C).all()
    slots = idx[kept].astype(np.int64) * C + loc[kept]
    assert np.unique(slots).size == slots.size
    counts = np.bincount(idx[kept], minlength=E)
    np.testing.assert_array_equal(counts, used)
    np.testing.assert_array_equal(elems, used.astype(np.uint64) * M)
    for e in range(E):                                  # locations of an expert are exactly 0 .. used-1
        assert set(loc[kept & (idx == e)]) == set(range(used[e]))
    tok = np.tile(np.arange(S), k)
    np.testing.assert_array_equal(disp[idx[kept], loc[kept]], data[tok[kept]])
    assert not disp.reshape(E * C, M)[np.setdiff1d(np.arange(E * C), slots)].any()
    if mode != "bpr":
        # first choices of the finite rows are the oracle's (later tokens' locations may differ: bad rows count)
        sel, _ = mo.select_topk(logits, k, gate_is_logits=is_logits)
        first = idx[:S]
        good = ~bad & (first >= 0)
        np.testing.assert_array_equal(first[good], sel[0][good])


def test_streaming_probe_kernels(pkg, lib):
    """lancet_debug_stream (the plain read / fill / copy kernels bench.py times beside the row movers)."""
    import ctypes as C
    n = 3 * 4096
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.full((n + 4096,), 7, dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    assert lib.lancet_debug_stream(2, p(dst), p(src), n, None) == 0
    assert torch.equal(dst[:n], src) and bool((dst[n:] == 7).all())
    assert lib.lancet_debug_stream(1, p(dst), None, 4096, None) == 0
    assert not bool(dst[:4096].any()) and torch.equal(dst[4096:n], src[4096:])
    assert lib.lancet_debug_stream(0, None, p(src), n, None) == 0
    assert lib.lancet_debug_stream(2, p(dst), p(src), 100, None) == pkg.capi.ERR_SHAPE
    assert lib.lancet_debug_stream(2, None, p(src), n, None) == pkg.capi.ERR_NULL
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- rows split over several waves
@pytest.mark.parametrize("M", [252, 256, 260, 508, 516, 1001, 1024, 1028, 2050, 4104, 8200, 16392, 33000])
@pytest.mark.parametrize("dt,k", [("f32", 1), ("bf16", 2), ("f16", 1), ("f32", 2)])
def test_rows_of_every_split(pkg, M, dt, k):
    """The row movers hand a row to 1, 2, 4, 8 or 16 waves by its length (one or two 16-byte granules per lane,
    further granules in a loop).  Row lengths around every switch point, rows that are not a multiple of the
    granule (element-wise path) and rows longer than one pass of 16 waves, against the oracle."""
    ops = pkg.ops
    S, E, cf = 150, 4, 0.8
    data, logits = make_inputs(M + k, S, M, E, zipf_bias=True)
    gate = mo.softmax_rows(logits)
    rows = rows_as_oracle(data, dt)
    used0 = np.zeros(E, np.int32)
    want = (mo.moe_encode_top2 if k == 2 else mo.moe_encode)(rows, gate, used0, cf, fast_scatter=True)
    got = ops.moe_encode(rows_to_torch(data, dt), dev(gate), None, cf, top_k=k)
    check_encode(got, want, gate_exact=True)
    assert (want[1][0] < 0).any()

    def same(got_t, want32):
        if dt == "f32":
            np.testing.assert_array_equal(to_np(got_t), want32)
            return
        tdt = torch.bfloat16 if dt == "bf16" else torch.float16
        a = got_t.cpu().view(torch.int16).to(torch.int32)
        b = torch.from_numpy(want32).to(tdt).view(torch.int16).to(torch.int32)
        assert int((a - b).abs().max()) <= 1                 # one rounding of the same fp32 value on both sides

    same(ops.moe_decode(got[4], got[0], got[1], top_k=k), mo.moe_decode(want[4], want[0], want[1], k=k))
    same(ops.moe_encode_dx(got[4], got[1], top_k=k), mo.moe_encode_dx(want[4], want[1], k))


# ----------------------------------------------------------------------------- row ranges of token partitions
@pytest.mark.parametrize("k,dt,P,S,M,E", [(1, "f32", 4, 2048, 64, 8), (2, "bf16", 4, 2048, 64, 8), (2, "f32", 3, 999, 5, 5),
                                          (1, "f16", 2, 512, 24, 16), (2, "bf16", 8, 4096, 40, 32)])
def test_partition_ranges_and_range_copies(pkg, k, dt, P, S, M, E):
    """lancet_moe_partition_ranges and the sparse copies on ranges against the oracle, and the round trip they are
    for: every partition's rows packed out of the shared buffer and unpacked into an empty one rebuild the buffer."""
    ops = pkg.ops
    S -= S % P
    cf = 0.7
    data, logits = make_inputs(S + 3 * k, S, M, E, zipf_bias=True)
    gate = mo.softmax_rows(logits)
    rows = rows_as_oracle(data, dt)
    want = (mo.moe_encode_top2 if k == 2 else mo.moe_encode)(rows, gate, np.zeros(E, np.int32), cf, fast_scatter=True)
    g, il, used, elems, disp = ops.moe_encode(rows_to_torch(data, dt), dev(gate), None, cf, top_k=k)
    np.testing.assert_array_equal(to_np(il), want[1])
    w_starts, w_counts = mo.moe_partition_ranges(want[1], P, E, M, k=k)
    starts, counts = ops.moe_partition_ranges(il, P, E, M, top_k=k)
    np.testing.assert_array_equal(to_np(starts).astype(np.uint64), w_starts)
    np.testing.assert_array_equal(to_np(counts).astype(np.uint64), w_counts)
    rebuilt = torch.zeros_like(disp)
    for q in range(k * P):
        total = int(w_counts[q].sum())
        wire = torch.full((total + 3,), 5.0, dtype=disp.dtype, device="cuda")
        ops.memcpy_sparse_ranges_to_cont_3d(disp, wire, counts[q], starts[q], axis=0)
        ref = mo.memcpy_sparse_ranges_to_cont_3d(want[4], np.full(total + 3, 5.0, np.float32), w_counts[q], w_starts[q])
        np.testing.assert_array_equal(to_np(wire), ref)
        ops.memcpy_cont_to_sparse_ranges_3d(wire, rebuilt, counts[q], starts[q], axis=0)
    assert torch.equal(rebuilt, disp)
    # the ranges of one (slot, partition) as a strided view of the whole table, the way a caller picks a row
    q = k * P - 1
    wire = torch.zeros(int(w_counts[q].sum()), dtype=disp.dtype, device="cuda")
    ops.memcpy_sparse_ranges_to_cont_3d(disp, wire, counts, starts, nelements_stride=1, nelements_offset=q * E, axis=0)
    ref = mo.memcpy_sparse_ranges_to_cont_3d(want[4], np.zeros(wire.numel(), np.float32), w_counts[q], w_starts[q])
    np.testing.assert_array_equal(to_np(wire), ref)


def test_range_copies_along_axis_1(pkg):
    ops = pkg.ops
    rng = np.random.default_rng(2)
    d0, d1, d2 = 6, 5, 24
    buf = rng.standard_normal((d0, d1, d2)).astype(np.float32)
    starts = np.array([0, 24, 48, 5, 143], np.uint64)         # whole rows, a row, an odd start, the last element
    counts = np.array([48, 24, 96, 11, 1], np.uint64)
    total = int(counts.sum())
    wire = ops.memcpy_sparse_ranges_to_cont_3d(dev(buf), torch.zeros(total, device="cuda"), dev(counts.astype(np.int64)),
                                               dev(starts.astype(np.int64)), axis=1)
    np.testing.assert_array_equal(to_np(wire), mo.memcpy_sparse_ranges_to_cont_3d(buf, np.zeros(total, np.float32), counts, starts, axis=1))
    back = ops.memcpy_cont_to_sparse_ranges_3d(wire, torch.full((d0, d1, d2), 9.0, device="cuda"), dev(counts.astype(np.int64)),
                                               dev(starts.astype(np.int64)), axis=1)
    np.testing.assert_array_equal(to_np(back), mo.memcpy_cont_to_sparse_ranges_3d(to_np(wire), np.full((d0, d1, d2), 9.0, np.float32),
                                                                                 counts, starts, axis=1))
    # a range that would leave its block is clipped
    starts[2], counts[2] = 100, 1000
    wire2 = ops.memcpy_sparse_ranges_to_cont_3d(dev(buf), torch.zeros(2000, device="cuda"), dev(counts.astype(np.int64)),
                                                dev(starts.astype(np.int64)), axis=1)
    np.testing.assert_array_equal(to_np(wire2), mo.memcpy_sparse_ranges_to_cont_3d(buf, np.zeros(2000, np.float32), counts, starts, axis=1))


def test_capacity_override_gshard_formula(pkg):
    """capacity= replaces the formula: GShard's ceil(2 S / E * cf) where E does not divide S (75 against 76)."""
    S, M, E = 300, 16, 8
    data, logits = make_inputs(71, S, M, E, zipf_bias=True)
    C = mo.gshard_top2_capacity(S, E, 1.0)
    assert C == 75 and pkg.ops.moe_capacity(S, E, 2.0) == 76
    want = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, C=C, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), None, 1.0, top_k=2, gate_is_logits=True, capacity=C)
    assert got[4].shape == (E, 75, M)
    for i in (1, 2, 3, 4):
        np.testing.assert_array_equal(to_np(got[i]), want[i])
    r = pkg.ops.moe_route(dev(logits), None, M, 1.0, top_k=2, gate_is_logits=True, capacity=C)
    np.testing.assert_array_equal(to_np(r[1]), want[1])


def test_default_workspaces_are_kept_per_stream(pkg):
    """Calls without a workspace argument share one kept per (device, stream): calls on two streams that run at the
    same time must not share theirs (the look-back form keeps state in it), and scan_errors() reads them all."""
    ops = pkg.ops
    S, M, E = 6000, 32, 16           # top-1 on 24 tiles: the look-back form
    data, logits = make_inputs(77, S, M, E)
    want = mo.moe_encode(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, fast_scatter=True)
    d_data, d_gate = dev(data), dev(logits)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    before = len(ops._scan_pool)
    outs = []
    for _ in range(20):
        outs.append(ops.moe_encode(d_data, d_gate, None, 1.0, gate_is_logits=True))
        with torch.cuda.stream(side):
            outs.append(ops.moe_encode(d_data, d_gate, None, 1.0, gate_is_logits=True))
    torch.cuda.synchronize()
    assert len(ops._scan_pool) >= max(before, 2)
    keys = {k for k in ops._scan_pool if k[1] in (side.cuda_stream, torch.cuda.current_stream().cuda_stream)}
    assert len(keys) == 2
    for got in outs:
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[4]), want[4])
    assert ops.scan_errors() == 0

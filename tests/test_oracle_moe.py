"""Pins the NumPy MoE oracle with checks that do not retype its formulas:
hand-computed values, brute-force token loops, the dense einsum form of GShard
top-2, and the reference tests' own identities (partitioned == un-partitioned,
no expert above capacity, encode->decode round trip)."""
import numpy as np
import pytest
from scipy.special import softmax as sp_softmax

from oracle import moe_oracle as mo


def rng_case(seed, S, M, E, dtype=np.float32, ties=False):
    rng = np.random.default_rng(seed)
    data = rng.standard_normal((S, M)).astype(dtype)
    gate = rng.standard_normal((S, E)).astype(np.float32)
    if ties:
        gate = np.round(gate * 2) / 2  # many exact ties
    return data, gate


# ---------------------------------------------------------------- capacity
@pytest.mark.parametrize("S,E,cf,want", [
    (4096, 8, 1.25, 640),          # BASELINE config 1
    (16384, 16, 2.0, 2048),        # config 2 (top-2: 2*cf)
    (32768, 64, 1.25, 640),        # config 3
    (16384, 32, 10.0, 5120),       # config 4 per partition: 2*1.25*4
    (65536, 32, 2.5, 5120),        # config 4 un-partitioned
    (1000, 7, 1.0, 143),           # ceil(1000/7)
    (10, 4, 1.5, 4),               # int(1.5*3) = 4
    (10, 4, 0.0, 0),
    (5, 8, 1.0, 1),
])
def test_capacity_hand_cases(S, E, cf, want):
    assert mo.capacity(S, E, cf) == want


# ---------------------------------------------------------------- softmax
def test_softmax_against_scipy_and_fp64():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((257, 33)) * 4).astype(np.float32)
    p = mo.softmax_rows(x)
    ref64 = sp_softmax(x.astype(np.float64), axis=1)
    np.testing.assert_allclose(p, ref64, rtol=2e-6, atol=0)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, rtol=1e-6)
    # shift invariance (closed-form property of softmax)
    p2 = mo.softmax_rows(x + np.float32(3.0))
    np.testing.assert_allclose(p, p2, rtol=1e-5)


# ---------------------------------------------------------------- selection
def brute_topk(row, k):
    order = sorted(range(len(row)), key=lambda j: (-row[j], j))
    return order[:k]


@pytest.mark.parametrize("ties", [False, True])
def test_select_topk_bruteforce(ties):
    _, gate = rng_case(2, 300, 1, 9, ties=ties)
    idx, val = mo.select_topk(gate, 2, False)
    for s in range(gate.shape[0]):
        want = brute_topk(list(gate[s]), 2)
        assert [idx[0, s], idx[1, s]] == want
        assert val[0, s] == gate[s, want[0]] and val[1, s] == gate[s, want[1]]


def test_select_hand_ties():
    gate = np.array([[5, 5, 3], [3, 5, 5], [5, 3, 3], [3, 5, 3], [1, 1, 1]], dtype=np.float32)
    idx, _ = mo.select_topk(gate, 2)
    assert idx[0].tolist() == [0, 1, 0, 1, 0]
    assert idx[1].tolist() == [1, 2, 1, 0, 1]


def test_select_second_choice_when_rest_is_minus_inf():
    gate = np.array([[1.0, -np.inf, -np.inf], [-np.inf, -np.inf, 2.0]], dtype=np.float32)
    idx, _ = mo.select_topk(gate, 2)
    assert idx[0].tolist() == [0, 2]
    assert idx[1].tolist() == [1, 0]


# ---------------------------------------------------------------- encode (A.1)
def brute_encode(data, gate, used_in, C):
    S, M = data.shape
    E = gate.shape[1]
    counts = [0] * E
    idx = [0] * S
    loc = [0] * S
    buf = np.zeros((E, C, M), data.dtype)
    for s in range(S):
        e = brute_topk(list(gate[s]), 1)[0]
        r = counts[e]
        counts[e] += 1
        loc[s] = r
        if r >= C - used_in[e]:
            idx[s] = -1
        else:
            idx[s] = e
            buf[e, r] = data[s]
    used_out = [min(int(used_in[e]) + counts[e], C) for e in range(E)]
    elems = [(used_out[e] - int(used_in[e])) * M for e in range(E)]
    return idx, loc, used_out, elems, buf


@pytest.mark.parametrize("S,M,E,cf,seed", [(64, 8, 4, 1.0, 0), (257, 4, 8, 1.25, 1), (100, 3, 7, 0.5, 2),
                                           (33, 2, 1, 1.0, 3), (50, 2, 16, 1.0, 4)])
def test_encode_bruteforce(S, M, E, cf, seed):
    data, gate = rng_case(seed, S, M, E, ties=(seed % 2 == 1))
    rng = np.random.default_rng(seed + 100)
    C = mo.capacity(S, E, cf)
    used_in = rng.integers(0, C + 1, size=E).astype(np.int32) if seed % 2 else np.zeros(E, np.int32)
    g, il, used, elems, disp = mo.moe_encode(data, gate, used_in, cf)
    bi, bl, bu, be, bb = brute_encode(data, gate, used_in, C)
    assert il[0].tolist() == bi and il[1].tolist() == bl
    assert used.tolist() == bu and elems.tolist() == be
    assert elems.dtype == np.uint64 and il.dtype == np.int32 and g.dtype == np.float32
    np.testing.assert_array_equal(disp, bb)
    np.testing.assert_array_equal(g, gate.max(axis=1))
    # vectorised scatter == loop scatter
    np.testing.assert_array_equal(mo.scatter_rows_fast(data, il[0], il[1], E, C), disp)


def test_encode_invariants_all_tokens_one_expert():
    S, M, E = 40, 4, 4
    data, gate = rng_case(5, S, M, E)
    gate[:, 2] = 100.0
    C = mo.capacity(S, E, 1.0)  # 10
    g, il, used, elems, disp = mo.moe_encode(data, gate, np.zeros(E, np.int32), 1.0)
    assert used.tolist() == [0, 0, 10, 0]
    assert il[0].tolist() == [2] * 10 + [-1] * 30
    assert il[1].tolist() == list(range(40))          # stale ranks stay on dropped tokens
    np.testing.assert_array_equal(disp[2], data[:10])
    assert not disp[[0, 1, 3]].any()


# ---------------------------------------------------------------- chained partitions (A.3/A.4)
@pytest.mark.parametrize("P", [2, 4])
@pytest.mark.parametrize("E", [2, 8])
def test_partitioned_equals_unpartitioned(P, E):
    """tests/python/op/cuda/test_cuda_moe.py:384-471 protocol."""
    S0, M = 256, 6
    data, gate = rng_case(7, S0, M, E)
    S = S0 // P
    zero = np.zeros(E, np.int32)
    rg, ril, rused, _, rdisp = mo.moe_encode(data, gate, zero, 1.0)
    used = zero
    ils, bufs, gs = [], [], []
    for p in range(P):
        sl = slice(p * S, (p + 1) * S)
        g, il, used, _, disp = mo.moe_encode(data[sl], gate[sl], used, float(P))
        assert disp.shape == rdisp.shape
        ils.append(il), bufs.append(disp), gs.append(g)
    np.testing.assert_array_equal(used, rused)
    # no expert above capacity across the chain (test_cuda_moe.py:336-381)
    cat = np.concatenate([il[0] for il in ils])
    assert (np.bincount(cat[cat >= 0], minlength=E) <= rdisp.shape[1]).all()
    merged = mo.moe_merge_masks(ils, E)
    red = mo.moe_redispatch(bufs, ils)
    ril = ril.copy()
    ril[1, ril[0] < 0] = -1            # merge normalises stale locations to -1
    np.testing.assert_array_equal(merged, ril)
    np.testing.assert_array_equal(red, rdisp)
    np.testing.assert_array_equal(np.concatenate(gs), rg)


# ---------------------------------------------------------------- BPR (A.2)
def brute_bpr(gate, C, P, pid):
    S0, E = gate.shape
    S = S0 // P
    idx0 = [brute_topk(list(gate[s]), 1)[0] for s in range(S0)]
    g0 = [gate[s, idx0[s]] for s in range(S0)]
    keep = [False] * S0
    for e in range(E):
        toks = sorted([s for s in range(S0) if idx0[s] == e], key=lambda s: (-g0[s], s))
        for s in toks[:C]:
            keep[s] = True
    counts = [0] * E
    idx, loc = [], []
    for s in range(pid * S, (pid + 1) * S):
        if keep[s]:
            idx.append(idx0[s]), loc.append(counts[idx0[s]])
            counts[idx0[s]] += 1
        else:
            idx.append(-1), loc.append(-1)
    return idx, loc, [min(c, C) for c in counts], keep


@pytest.mark.parametrize("S0,E,P,cf,ties", [(128, 4, 1, 1.0, False), (128, 4, 1, 0.5, True), (256, 8, 4, 4.0, False),
                                            (256, 8, 4, 2.0, True), (96, 3, 2, 1.0, True)])
def test_bpr_bruteforce(S0, E, P, cf, ties):
    M = 3
    data, gate = rng_case(11, S0, M, E, ties=ties)
    C = mo.capacity(S0 // P, E, cf)
    kept_total = np.zeros(E, np.int64)
    for pid in range(P):
        g, il, used, elems, disp = mo.moe_encode_bpr(data, gate, P, pid, cf)
        bi, bl, bu, keep = brute_bpr(gate, C, P, pid)
        assert il[0].tolist() == bi and il[1].tolist() == bl and used.tolist() == bu
        assert elems.tolist() == [u * M for u in bu]
        S = S0 // P
        np.testing.assert_array_equal(g, gate.max(axis=1)[pid * S:(pid + 1) * S])
        for s in range(S):
            if bi[s] >= 0:
                np.testing.assert_array_equal(disp[bi[s], bl[s]], data[pid * S + s])
        assert np.count_nonzero(disp.any(axis=2)) <= sum(bu)
        kept_total += used
    # sum over partitions of kept == min(cnt, C): drop set independent of the partitioning
    cnt = np.bincount(np.argmax(gate, axis=1), minlength=E)
    np.testing.assert_array_equal(kept_total, np.minimum(cnt, C))


# ---------------------------------------------------------------- top-2 (A.6) vs dense GShard form
def dense_top2(logits, data, C, noise=None):
    """docker/resources/sharded_moe.py:253-324 written with dense masks; `noise` stands for the Gumbel
    sample of :275 (logits_w_noise = logits + noise, used for the second choice only)."""
    S, E = logits.shape
    gates = sp_softmax(logits.astype(np.float64), axis=1)
    i1 = np.argmax(gates, axis=1)
    mask1 = np.eye(E, dtype=np.int64)[i1]
    w_noise = logits if noise is None else (logits + noise).astype(np.float32)
    except1 = np.where(mask1.astype(bool), -np.inf, w_noise.astype(np.float64))
    i2 = np.argmax(except1, axis=1)
    mask2 = np.eye(E, dtype=np.int64)[i2]
    loc1 = np.cumsum(mask1, axis=0) - 1
    loc2 = np.cumsum(mask2, axis=0) - 1 + mask1.sum(axis=0, keepdims=True)
    mask1 = mask1 * (loc1 < C)
    mask2 = mask2 * (loc2 < C)
    l1 = (loc1 * mask1).sum(axis=1)
    l2 = (loc2 * mask2).sum(axis=1)
    g1 = (gates * mask1).sum(axis=1)
    g2 = (gates * mask2).sum(axis=1)
    den = np.maximum(g1 + g2, np.finfo(np.float32).eps)
    g1, g2 = g1 / den, g2 / den
    cw = np.zeros((S, E, C))
    for s in range(S):
        if mask1[s].any():
            cw[s, i1[s], l1[s]] += g1[s]
        if mask2[s].any():
            cw[s, i2[s], l2[s]] += g2[s]
    disp = np.einsum("sec,sm->ecm", (cw != 0).astype(np.float64), data.astype(np.float64))
    return cw, disp


@pytest.mark.parametrize("noisy", [False, True])
@pytest.mark.parametrize("S,E,cf,seed", [(48, 4, 1.0, 0), (64, 8, 0.5, 1), (40, 3, 2.0, 2)])
def test_top2_matches_dense_gshard(S, E, cf, seed, noisy):
    M = 5
    data, logits = rng_case(seed, S, M, E)
    logits[:, 0] += 1.5   # a hot expert so that slot 1 and slot 2 both overflow
    noise = np.random.default_rng(seed + 50).gumbel(size=(S, E)).astype(np.float32) if noisy else None
    C = int(np.ceil(2 * S / E * cf))
    assert C == mo.capacity(S, E, 2 * cf) or (2 * S / E * cf) != int(2 * S / E * cf)
    gates, il, used, elems, disp = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), cf,
                                                      gate_is_logits=True, C=C, gate2_noise=noise)
    cw, ddisp = dense_top2(logits, data, C, noise)
    if noisy:   # the noise changes second choices, or the case pins nothing
        plain = mo.select_topk(logits, 2, True)[0][1]
        assert (mo.select_topk(logits, 2, True, noise)[0][1] != plain).any()
    mine = np.zeros((S, E, C))
    for j in range(2):
        for s in range(S):
            e, l = il[0, j * S + s], il[1, j * S + s]
            if e >= 0:
                mine[s, e, l] += gates[j * S + s]
    np.testing.assert_allclose(mine, cw, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(disp, ddisp, rtol=0, atol=0)
    kept = np.bincount(il[0][il[0] >= 0], minlength=E)
    np.testing.assert_array_equal(used, kept)
    assert elems.tolist() == (kept * M).tolist()
    # decode of the identity expert with the combine weights == dense combine
    out = mo.moe_decode(disp, gates, il, k=2)
    want = np.einsum("sec,ecm->sm", cw, ddisp)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- decode (A.5)
def test_decode_roundtrip_and_loop_reference():
    S, M, E = 120, 6, 5
    data, gate = rng_case(21, S, M, E)
    probs = mo.softmax_rows(gate)
    g, il, used, _, disp = mo.moe_encode(data, probs, np.zeros(E, np.int32), 0.75)
    out1 = mo.moe_decode(disp, np.ones(S, np.float32), il)
    kept = il[0] >= 0
    np.testing.assert_array_equal(out1[kept], data[kept])
    assert not out1[~kept].any() and (~kept).any()
    # loop reference of test_cuda_moe.py:1157-1165
    out = mo.moe_decode(disp, g, il)
    C = disp.shape[1]
    for s in range(S):
        e, l = il[0, s], il[1, s]
        want = disp[e, l] * g[s] if (0 <= e < E and l < C) else np.zeros(M, np.float32)
        np.testing.assert_array_equal(out[s], want)


def test_bf16_rounding_helpers():
    x = np.array([1.0, 1.00390625, 1.005859375, -2.5, 3.0e38, 1e-40], dtype=np.float32)
    # 1.00390625 = 1 + 2^-8 is a tie between bf16 1.0 and 1.0078125 -> even (1.0)
    r = mo.round_to_bf16(x)
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == np.float32(1.0078125) and r[3] == -2.5
    import torch
    t = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(r, t)


# ---------------------------------------------------------------- backward ops vs torch autograd
@pytest.mark.parametrize("k", [1, 2])
def test_backward_ops_match_autograd_of_dense_forms(k):
    """Dense forms: dispatched = einsum('sec,sm->ecm', mask, x), gates_s = gate[s, idx];
    combined = einsum('sec,ecm->sm', weight_sec, expert_out).  torch autograd of those gives the four
    gradients without using the oracle's backward formulas."""
    import torch
    S, M, E = 40, 6, 4
    data, logits = rng_case(31 + k, S, M, E)
    logits[:, 0] += 1.0
    probs = mo.softmax_rows(logits)
    if k == 1:
        g, il, used, _, disp = mo.moe_encode(data, probs, np.zeros(E, np.int32), 0.75)
    else:
        g, il, used, _, disp = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 0.75, gate_is_logits=True)
    C = disp.shape[1]
    mask = np.zeros((k, S, E, C), np.float64)
    for j in range(k):
        for s in range(S):
            e, l = il[0, j * S + s], il[1, j * S + s]
            if e >= 0:
                mask[j, s, e, l] = 1.0
    rng = np.random.default_rng(5)
    # --- encode: loss = <dispatched, W> + <gates_s, w>
    W = rng.standard_normal(disp.shape)
    w = rng.standard_normal(k * S)
    x = torch.tensor(data.astype(np.float64), requires_grad=True)
    gate = torch.tensor(probs.astype(np.float64), requires_grad=True)
    tmask = torch.tensor(mask)
    dispatched = torch.einsum("jsec,sm->ecm", tmask, x)
    onehot = torch.zeros((k, S, E), dtype=torch.float64)
    sel, _ = mo.select_topk(logits, k, True)
    for j in range(k):
        kept = il[0, j * S:(j + 1) * S] >= 0
        onehot[j, np.arange(S)[kept], sel[j][kept]] = 1.0     # dropped slots get no gate gradient
    gates_s = (gate[None] * onehot).sum(dim=2).reshape(-1)
    loss = (dispatched * torch.tensor(W)).sum() + (gates_s * torch.tensor(w)).sum()
    loss.backward()
    np.testing.assert_array_equal(disp, dispatched.detach().numpy().astype(np.float32))
    np.testing.assert_allclose(mo.moe_encode_dx(W.astype(np.float32), il, k), x.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(mo.moe_encode_dg(w.astype(np.float32), il, E, k), gate.grad.numpy(), rtol=1e-6, atol=1e-7)
    # --- decode: loss = <combined, Y>
    Y = rng.standard_normal((S, M))
    eo = torch.tensor((disp * 1.5 + 0.1).astype(np.float64), requires_grad=True)
    gs = torch.tensor(g.astype(np.float64), requires_grad=True)
    weight = (tmask * gs.reshape(k, S, 1, 1)).sum(dim=0)
    combined = torch.einsum("sec,ecm->sm", weight, eo)
    (combined * torch.tensor(Y)).sum().backward()
    eo32 = eo.detach().numpy().astype(np.float32)
    np.testing.assert_allclose(mo.moe_decode(eo32, g, il, k=k), combined.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(mo.moe_decode_dx(Y.astype(np.float32), g, il, E, C, k), eo.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(mo.moe_decode_dg(Y.astype(np.float32), eo32, il, k), gs.grad.numpy(), rtol=1e-5, atol=1e-6)


def _dense_top2_weights(logits_or_probs, il, k, S, E, is_logits):
    """The gate side of top2gating (docker/resources/sharded_moe.py:253-324) in torch, fp64, dense one-hot form,
    with the selection and capacity decisions (which slots survive) taken from `il` as constants: gates = softmax
    (:260), mask_j after the capacity drop (:296-297), gates_j_s = einsum('se,se->s', gates, mask_j) (:306-307),
    denom clamped at finfo(float32).eps (:308-310), division (:311-312).  k = 1: the reference op's own
    gates_s = sum_e gate * one_hot (src/op/dialect/cuda/moe.cc:232-250), kept tokens only as its gradient rule has it."""
    import torch
    gates = torch.softmax(logits_or_probs, dim=1) if is_logits else logits_or_probs
    masks = []
    for j in range(k):
        idx = torch.as_tensor(np.asarray(il[0, j * S:(j + 1) * S]), dtype=torch.long)
        kept = idx >= 0
        m = torch.zeros((S, E), dtype=torch.float64)
        m[torch.arange(S)[kept], idx[kept]] = 1.0
        masks.append(m)
    gs = [torch.einsum("se,se->s", gates, m) for m in masks]
    if k == 1:
        return gs[0]
    denom = torch.clamp(gs[0] + gs[1], min=torch.finfo(torch.float32).eps)
    return torch.cat([gs[0] / denom, gs[1] / denom])


@pytest.mark.parametrize("is_logits", [False, True])
@pytest.mark.parametrize("k", [1, 2])
def test_gate_gradient_of_the_whole_op_matches_autograd_of_dense_top2gating(k, is_logits):
    import torch
    S, M, E = 96, 4, 6
    data, logits = rng_case(77 + k, S, M, E)
    logits[:, 1] += 1.5                                   # a hot expert: slots of both kinds get dropped
    gate_in = logits if is_logits else mo.softmax_rows(logits)
    used0 = np.zeros(E, np.int32)
    if k == 1:
        g, il, *_ = mo.moe_encode(data, gate_in, used0, 0.6, gate_is_logits=is_logits)
    else:
        g, il, *_ = mo.moe_encode_top2(data, gate_in, used0, 0.6, gate_is_logits=is_logits)
        first, second = il[0, :S] >= 0, il[0, S:] >= 0
        assert (first & ~second).any() and (~first & second).any() and (~first & ~second).any() and (first & second).any()
    rng = np.random.default_rng(9)
    w = rng.standard_normal(k * S).astype(np.float32)
    x = torch.tensor(gate_in.astype(np.float64), requires_grad=True)
    ws = _dense_top2_weights(x, il, k, S, E, is_logits)
    if k == 2 or not is_logits:
        # the dense form reproduces the forward's weights (k = 1 on logits: the forward keeps the value of dropped tokens too)
        kept = np.concatenate([il[0, j * S:(j + 1) * S] >= 0 for j in range(k)])
        np.testing.assert_allclose(ws.detach().numpy()[kept], g[kept], rtol=2e-6)
    (ws * torch.tensor(w.astype(np.float64))).sum().backward()
    got = mo.moe_encode_dgate(w, gate_in, il, k, is_logits)
    np.testing.assert_allclose(got, x.grad.numpy(), rtol=1e-9, atol=1e-12)
    if k == 1 and not is_logits:
        np.testing.assert_array_equal(got.astype(np.float32), mo.moe_encode_dg(w, il, E, 1))


def test_gate_gradient_below_the_clamp_of_the_denominator():
    """Probabilities so small that g1 + g2 < eps: the clamped denominator is a constant, d g_k = dy_k / eps
    (torch.clamp's gradient); and rows at either side of the threshold."""
    import torch
    S, E = 8, 4
    gate = np.full((S, E), 1e-9, np.float32)
    gate[:, 0] = np.float32(3e-8) * np.arange(1, S + 1, dtype=np.float32)      # g1 + g2 from 4e-8 to 2.5e-7: crosses eps
    gate[:, 2] = np.float32(1e-8)
    il = np.array([[0] * S + [2] * S, list(range(S)) * 2], np.int32)
    tot = gate[:, 0].astype(np.float64) + gate[:, 2]
    assert (tot < float(mo.F32_EPS)).any() and (tot > float(mo.F32_EPS)).any()
    w = np.linspace(-1, 2, 2 * S).astype(np.float32)
    x = torch.tensor(gate.astype(np.float64), requires_grad=True)
    (_dense_top2_weights(x, il, 2, S, E, False) * torch.tensor(w.astype(np.float64))).sum().backward()
    np.testing.assert_allclose(mo.moe_encode_dgate(w, gate, il, 2, False), x.grad.numpy(), rtol=1e-9, atol=0)


def test_gate_gradient_of_peaked_rows_has_the_closed_form_of_a_two_expert_softmax():
    """Two experts, logits (t, 0) with t up to 60: p1 = 1 / (1 + exp(-t)) and the gradient of the selected logit is
    dy p1 (1 - p1) = dy exp(-t) / (1 + exp(-t))^2, of the other one its negative; neither form subtracts.
    Evaluating p (dp - sum p dp) as written would be off by 1e-16 / (1 - p1): 2e-5 at t = 27, everything at t = 40."""
    t = np.array([0.5, 3.0, 12.0, 27.0, 40.0, 60.0])
    S = t.size
    logits = np.stack([t, np.zeros(S)], axis=1).astype(np.float32)
    il = np.array([[0] * S, list(range(S))], np.int32)
    dy = np.linspace(-2, 3, S).astype(np.float32)
    z = np.exp(-t)
    sel = dy.astype(np.float64) * z / (1 + z) ** 2
    got = mo.moe_encode_dgate(dy, logits, il, 1, True)
    np.testing.assert_allclose(got[:, 0], sel, rtol=1e-13, atol=0)
    np.testing.assert_allclose(got[:, 1], -sel, rtol=1e-13, atol=0)
    # top-2, both kept: w1 = p1 / (p1 + p2) = 1 / (1 + exp(-t)) again (a third expert far below changes nothing
    # in the ratio), so d logit1 = (dy1 - dy2) exp(-t) / (1 + exp(-t))^2, d logit2 its negative, d logit3 = 0
    logits3 = np.concatenate([logits, np.full((S, 1), -5.0, np.float32)], axis=1)
    il2 = np.array([[0] * S + [1] * S, list(range(S)) * 2], np.int32)
    dy2 = np.concatenate([dy, dy[::-1] * np.float32(0.5)]).astype(np.float32)
    sel2 = (dy2[:S].astype(np.float64) - dy2[S:]) * z / (1 + z) ** 2
    got = mo.moe_encode_dgate(dy2, logits3, il2, 2, True)
    np.testing.assert_allclose(got[:, 0], sel2, rtol=1e-12, atol=0)
    np.testing.assert_allclose(got[:, 1], -sel2, rtol=1e-12, atol=0)
    assert np.abs(got[:, 2]).max() <= 1e-15 * np.abs(sel2).max()


# ---------------------------------------------------------------- redispatch_expert_input
@pytest.mark.parametrize("P", [2, 4])
def test_redispatch_expert_input_partitioned_equals_whole(P):
    """tests/python/distributed/test_partitioned_moe.py:99-196: split every source GPU's received rows
    into P partitions (each compacted from row 0 of its own buffer); the merge restores the whole."""
    rng = np.random.default_rng(P)
    C, G, M, LE, le = 12, 3, 4, 2, 1
    whole = rng.standard_normal((C, G, M)).astype(np.float32)
    rows_total = rng.integers(0, C + 1, G)
    bufs = [np.full((C, G, M), 99.0, np.float32) for _ in range(P)]
    cnts = [np.zeros(G * LE, np.uint64) for _ in range(P)]
    for g in range(G):
        cuts = np.sort(rng.integers(0, rows_total[g] + 1, P - 1))
        edges = [0] + list(cuts) + [rows_total[g]]
        for p in range(P):
            n = edges[p + 1] - edges[p]
            bufs[p][:n, g, :] = whole[edges[p]:edges[p + 1], g, :]
            cnts[p][g * LE + le] = n * M
            cnts[p][g * LE + (1 - le)] = 12345          # the other local expert's count must be ignored
    out = mo.moe_redispatch_expert_input(bufs, cnts, le, LE)
    for g in range(G):
        np.testing.assert_array_equal(out[:rows_total[g], g], whole[:rows_total[g], g])
        assert not out[rows_total[g]:, g].any()
    # element-granular counts (not a multiple of M) and the scale factor
    cnts2 = [np.array([3, 0, 5, 0, 0, 0], np.uint64), np.array([2, 0, 1, 0, 4, 0], np.uint64)]
    out2 = mo.moe_redispatch_expert_input(bufs[:2], cnts2, 0, LE, scale=2)
    want_g0 = np.concatenate([bufs[0][:, 0].reshape(-1)[:6], bufs[1][:, 0].reshape(-1)[:4]])
    np.testing.assert_array_equal(out2[:, 0].reshape(-1)[:10], want_g0)
    assert not out2[:, 0].reshape(-1)[10:].any()


# ----------------------------------------------------------------------------- sparse <-> packed copies
def _brute_sparse_to_cont(src, dst, cnt, stride, offset, axis, scale, shrink):
    """Element-by-element restatement of the copy as one thread would do it (block offset = scaled sum of the
    earlier counts; 3-D position from the flat stream position), independent of the oracle's slicing."""
    d0, d1, d2 = src.shape
    out = dst.copy()
    for b in range(src.shape[axis]):
        before = sum(int(cnt[j * stride + offset]) for j in range(b)) * scale // shrink
        n = int(cnt[b * stride + offset]) * scale // shrink
        for t in range(n):
            if axis == 0:
                v = src[b, t // d2, t % d2]
            else:
                v = src[t // d2, b, t % d2]
            out[before + t] = v
    return out


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("scale,shrink", [(1, 1), (2, 1), (1, 2), (3, 2)])
def test_sparse_copy_matches_elementwise_definition(axis, scale, shrink):
    rng = np.random.default_rng(axis * 7 + scale + shrink)
    d0, d1, d2, stride, offset = 5, 4, 6, 3, 1
    src = rng.standard_normal((d0, d1, d2)).astype(np.float32)
    nb = src.shape[axis]
    cap = (d1 if axis == 0 else d0) * d2
    cnt = np.zeros(nb * stride, np.uint64)
    cnt[offset::stride] = rng.integers(0, cap * shrink // scale + 1, nb)
    cnt[(offset + 1) % stride::stride] = 999          # other columns must not be read
    total = sum(int(c) for c in cnt[offset::stride]) * scale // shrink
    dst = np.full(total + 3, -7.0, np.float32)
    got = mo.memcpy_sparse_to_cont_3d(src, dst, cnt, stride, offset, axis, scale, shrink)
    np.testing.assert_array_equal(got, _brute_sparse_to_cont(src, dst, cnt, stride, offset, axis, scale, shrink))
    # inverse: the valid part of every block comes back, the rest keeps the destination's bytes
    back = mo.memcpy_cont_to_sparse_3d(got, np.full_like(src, 5.0), cnt, stride, offset, axis, scale, shrink)
    offs, ns = mo.sparse_copy_extents(cnt, stride, offset, nb, scale, shrink)
    for b in range(nb):
        a = (src[b] if axis == 0 else src[:, b, :]).reshape(-1)
        r = (back[b] if axis == 0 else back[:, b, :]).reshape(-1)
        np.testing.assert_array_equal(r[:ns[b]], a[:ns[b]])
        assert (r[ns[b]:] == 5.0).all()
    z = mo.memcpy_cont_to_sparse_3d(got, np.full_like(src, 5.0), cnt, stride, offset, axis, scale, shrink, zero_tail=True)
    assert ((z == back) | (z == 0)).all() and (z[back == 5.0] == 0).all()


def test_sparse_copy_packs_encode_output():
    """elements_per_expert of an encode is exactly the count array the copy is keyed by: packing [E, C, M]
    along axis 0 gives the kept rows of every expert back to back, and unpacking restores the buffer."""
    rng = np.random.default_rng(3)
    S, M, E = 96, 8, 4
    x = rng.standard_normal((S, M)).astype(np.float32)
    gate = mo.softmax_rows(rng.standard_normal((S, E)).astype(np.float32))
    _, _, used, elems, disp = mo.moe_encode(x, gate, np.zeros(E, np.int32), 0.75)
    packed = mo.memcpy_sparse_to_cont_3d(disp, np.zeros(int(elems.sum()), np.float32), elems)
    want = np.concatenate([disp[e, :used[e]].reshape(-1) for e in range(E)])
    np.testing.assert_array_equal(packed, want)
    np.testing.assert_array_equal(mo.memcpy_cont_to_sparse_3d(packed, np.zeros_like(disp), elems), disp)


# ---------------------------------------------------------------- row ranges of partitions inside a whole-batch routing
@pytest.mark.parametrize("P,E", [(2, 2), (4, 8), (4, 3)])
def test_partition_ranges_pack_what_the_chained_partition_encodes_pack(P, E):
    """The ranges exist for one identity: what partition p owns inside the buffer of the whole-batch encode is what
    partition p's own chained encode (tests/python/op/cuda/test_cuda_moe.py:384-471 protocol) holds in its first
    rows, so packing either way gives the same stream, counts = the chained encode's elements_per_expert, and
    unpacking every partition's stream at its ranges rebuilds the whole buffer."""
    S0, M = 264, 6
    S0 -= S0 % (P * E)
    data, gate = rng_case(11 + P, S0, M, E)
    gate[:, 0] += 0.4                       # a crowded expert: the chain drops tokens
    S = S0 // P
    zero = np.zeros(E, np.int32)
    _, wil, wused, _, wdisp = mo.moe_encode(data, gate, zero, 0.75)
    starts, counts = mo.moe_partition_ranges(wil, P, E, M)
    assert (wil[0] < 0).any()
    used = zero
    rebuilt = np.zeros_like(wdisp)
    for p in range(P):
        sl = slice(p * S, (p + 1) * S)
        _, il, used, elems, disp = mo.moe_encode(data[sl], gate[sl], used, 0.75 * P)
        assert disp.shape == wdisp.shape
        np.testing.assert_array_equal(counts[p], elems)
        total = int(elems.sum())
        own = mo.memcpy_sparse_to_cont_3d(disp, np.full(total, 7, disp.dtype), elems)
        ranged = mo.memcpy_sparse_ranges_to_cont_3d(wdisp, np.full(total, 9, wdisp.dtype), counts[p], starts[p])
        np.testing.assert_array_equal(ranged, own)
        rebuilt = mo.memcpy_cont_to_sparse_ranges_3d(ranged, rebuilt, counts[p], starts[p])
    np.testing.assert_array_equal(used, wused)
    np.testing.assert_array_equal(rebuilt, wdisp)
    # the ranges tile the used rows of every expert without gaps or overlap
    np.testing.assert_array_equal(starts[0], np.zeros(E, np.uint64))
    np.testing.assert_array_equal(starts[1:], (starts + counts)[:-1])
    np.testing.assert_array_equal((starts + counts)[-1], wused.astype(np.uint64) * np.uint64(M))


def test_partition_ranges_of_a_top2_routing_hold_the_partitions_tokens_in_order():
    """top-2: rows of expert e follow each other slot-major, then by partition, then by token
    (docker/resources/sharded_moe.py:282-295: second choices are placed behind all first choices).  Every range
    must hold exactly the rows of the kept tokens of its (slot, partition, expert), in token order."""
    S0, M, E, P = 240, 5, 4, 3
    data, gate = rng_case(3, S0, M, E)
    _, il, used, _, disp = mo.moe_encode_top2(data, gate, np.zeros(E, np.int32), 0.6)
    starts, counts = mo.moe_partition_ranges(il, P, E, M, k=2)
    S = S0 // P
    assert (il[0] < 0).any()
    for j in range(2):
        for p in range(P):
            for e in range(E):
                toks = [s for s in range(p * S, (p + 1) * S) if il[0, j * S0 + s] == e]
                r0 = int(starts[j * P + p, e]) // M
                assert int(counts[j * P + p, e]) == len(toks) * M
                np.testing.assert_array_equal(disp[e, r0:r0 + len(toks)], data[toks])
                assert [int(il[1, j * S0 + s]) for s in toks] == list(range(r0, r0 + len(toks)))
    np.testing.assert_array_equal((starts + counts)[-1], used.astype(np.uint64) * np.uint64(M))


def test_top2_capacity_formula_against_gshard():
    """The top-2 extension sizes the buffer with the reference op's formula and a doubled factor,
    int(2 cf * ceil(S / E)); GShard's own is ceil(2 S / E * cf) (sharded_moe.py:267).  They agree on every
    BASELINE configuration and differ when E does not divide S or the factor is fractional; a caller that
    wants GShard's passes it as the capacity override, and the drop set then is GShard's."""
    for S, E, cf in [(16384, 16, 1.0), (65536, 32, 1.25), (4096, 8, 1.0)]:
        assert mo.capacity(S, E, 2 * cf) == mo.gshard_top2_capacity(S, E, cf)
    assert (mo.capacity(300, 8, 2.0), mo.gshard_top2_capacity(300, 8, 1.0)) == (76, 75)
    assert (mo.capacity(1000, 7, 2 * 1.1), mo.gshard_top2_capacity(1000, 7, 1.1)) == (314, 315)
    # with the override the oracle's drop set is that of the dense GShard form at that capacity
    rng = np.random.default_rng(4)
    S, E, M = 300, 8, 3
    data = rng.standard_normal((S, M), dtype=np.float32)
    logits = rng.standard_normal((S, E), dtype=np.float32)
    logits[:, 0] += 2.0
    C = mo.gshard_top2_capacity(S, E, 1.0)
    g, il, used, _, disp = mo.moe_encode_top2(data, logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True, C=C)
    assert disp.shape == (E, 75, M) and used.max() == 75
    kept1 = il[0, :S] >= 0
    first = np.argmax(logits, axis=1)
    for e in range(E):   # slot 1 keeps the first C tokens of every expert, in token order
        tok = np.flatnonzero(first == e)
        assert kept1[tok[:C]].all() and not kept1[tok[C:]].any()

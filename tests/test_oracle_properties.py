"""Property tests of the CPU oracle (hypothesis): the invariants the dispatch semantics fix, checked on
random small inputs, ragged and degenerate ones included.  Each property is independent of how the oracle
computes its answer, so a dropped term, a wrong sign or an off-by-one in it fails one of them."""
import numpy as np
from hypothesis import given, settings, strategies as st

from oracle import moe_oracle as mo

SET = dict(max_examples=60, deadline=None)


@st.composite
def routing_case(draw, max_S=80, max_E=9):
    S = draw(st.integers(0, max_S))
    E = draw(st.integers(1, max_E))
    M = draw(st.integers(1, 5))
    seed = draw(st.integers(0, 2 ** 31 - 1))
    cf = draw(st.sampled_from([0.25, 0.5, 1.0, 1.25, 2.0, 5.0]))
    rng = np.random.default_rng(seed)
    data = rng.standard_normal((S, M)).astype(np.float32)
    # quantised gate values make ties common
    gate = (np.round(rng.standard_normal((S, E)) * draw(st.sampled_from([1.0, 4.0]))) / 4).astype(np.float32)
    return data, gate, cf, rng


@settings(**SET)
@given(routing_case())
def test_encode_invariants(case):
    data, gate, cf, rng = case
    S, M = data.shape
    E = gate.shape[1]
    C = mo.capacity(S, E, cf)
    used_in = rng.integers(0, C + 1, E).astype(np.int32)
    g, il, used_out, elems, disp = mo.moe_encode(data, gate, used_in, cf)
    idx0 = np.argmax(gate, axis=1) if S else np.zeros(0, np.int64)          # first max
    np.testing.assert_array_equal(g, gate[np.arange(S), idx0])
    for e in range(E):
        toks = np.flatnonzero(idx0 == e)
        # locations count the tokens of the expert in token order, kept or not
        np.testing.assert_array_equal(il[1][toks], np.arange(len(toks)))
        room = C - int(used_in[e])
        kept = toks[:max(room, 0)]
        assert (il[0][kept] == e).all() and (il[0][toks[len(kept):]] == -1).all()
        assert used_out[e] == min(used_in[e] + len(toks), C)
        assert elems[e] == (used_out[e] - used_in[e]) * M
        # rows start at 0 in this call's own buffer; everything past them is zero
        np.testing.assert_array_equal(disp[e, :len(kept)], data[kept])
        assert not disp[e, len(kept):].any()


@settings(**SET)
@given(routing_case(), st.integers(1, 4))
def test_chained_partitions_equal_the_whole_batch(case, P):
    data, gate, cf, _ = case
    S, M = data.shape
    E = gate.shape[1]
    S -= S % P
    if S == 0:
        return
    data, gate = data[:S], gate[:S]
    whole = mo.moe_encode(data, gate, np.zeros(E, np.int32), cf)
    Cw = mo.capacity(S, E, cf)
    used = np.zeros(E, np.int32)
    ils, bufs = [], []
    Sp = S // P
    # the partitions get capacity_factor x P, as the partition pass passes it; the identity needs equal capacities
    if mo.capacity(Sp, E, cf * P) != Cw:
        return
    for p in range(P):
        _, il, used, _, disp = mo.moe_encode(data[p * Sp:(p + 1) * Sp], gate[p * Sp:(p + 1) * Sp], used, cf * P)
        ils.append(il)
        bufs.append(disp)
    merged = mo.moe_merge_masks(ils, E)
    kept_whole = whole[1][0] >= 0
    np.testing.assert_array_equal(merged[0] >= 0, kept_whole)
    np.testing.assert_array_equal(merged[0][kept_whole], whole[1][0][kept_whole])
    np.testing.assert_array_equal(merged[1][kept_whole], whole[1][1][kept_whole])
    assert (merged[1][~kept_whole] == -1).all()
    np.testing.assert_array_equal(mo.moe_redispatch(bufs, ils), whole[4])
    np.testing.assert_array_equal(used, whole[2])


@settings(**SET)
@given(routing_case(), st.integers(1, 4))
def test_bpr_keeps_the_best_tokens_whatever_the_partitioning(case, P):
    data, gate, cf, _ = case
    S0, M = data.shape
    E = gate.shape[1]
    S0 -= S0 % P
    if S0 == 0:
        return
    data, gate = data[:S0], gate[:S0]
    S = S0 // P
    C = mo.capacity(S, E, cf)
    idx0 = np.argmax(gate, axis=1)
    prio = gate[np.arange(S0), idx0]
    keep = np.zeros(S0, bool)
    for e in range(E):
        toks = np.flatnonzero(idx0 == e)
        order = sorted(toks, key=lambda s: (-prio[s], s))          # best first, ties by token
        keep[order[:C]] = True
    for pid in range(P):
        g, il, used, elems, disp = mo.moe_encode_bpr(data, gate, P, pid, cf)
        sl = slice(pid * S, (pid + 1) * S)
        np.testing.assert_array_equal(il[0] >= 0, keep[sl])
        np.testing.assert_array_equal(g, prio[sl])
        for e in range(E):
            toks = np.flatnonzero((idx0[sl] == e) & keep[sl])
            np.testing.assert_array_equal(il[1][toks], np.arange(len(toks)))
            assert used[e] == min(len(toks), C) and elems[e] == used[e] * M
            np.testing.assert_array_equal(disp[e, :len(toks)], data[sl][toks])
        assert (il[1][il[0] < 0] == -1).all()


@settings(**SET)
@given(routing_case())
def test_decode_is_the_weighted_inverse_of_encode(case):
    data, gate, cf, _ = case
    S, M = data.shape
    E = gate.shape[1]
    probs = mo.softmax_rows(gate)
    g, il, _, _, disp = mo.moe_encode(data, probs, np.zeros(E, np.int32), cf)
    out = mo.moe_decode(disp, g, il)
    kept = il[0] >= 0
    np.testing.assert_array_equal(out[kept], (data[kept] * g[kept, None]).astype(np.float32))
    assert not out[~kept].any()
    # gradients of the pair are each other's transposes: <decode(B, g), Y> == <B, decode_dx(Y, g)>
    rng = np.random.default_rng(S + E)
    Y = rng.standard_normal((S, M)).astype(np.float32)
    B = rng.standard_normal(disp.shape).astype(np.float32)
    lhs = float((mo.moe_decode(B, g, il).astype(np.float64) * Y).sum())
    rhs = float((B.astype(np.float64) * mo.moe_decode_dx(Y, g, il, E, disp.shape[1])).sum())
    assert abs(lhs - rhs) <= 1e-4 * (1 + abs(lhs))


@settings(**SET)
@given(routing_case(max_E=7))
def test_top2_is_two_chained_top1_encodes(case):
    data, gate, cf, _ = case
    S, M = data.shape
    E = gate.shape[1]
    if E < 2 or S == 0:
        return
    gates, il, used, elems, disp = mo.moe_encode_top2(data, gate, np.zeros(E, np.int32), cf)
    C = mo.capacity(S, E, 2 * cf)
    sel, val = mo.select_topk(gate, 2)
    assert (sel[0] != sel[1]).all()
    i1, l1, u1, _ = mo.gen_location(sel[0], np.zeros(E, np.int32), C, M, E)
    i2, l2, u2, _ = mo.gen_location(sel[1], u1, C, M, E)
    np.testing.assert_array_equal(used, u2)
    np.testing.assert_array_equal(il[0], np.concatenate([i1, i2]))
    # second-slot rows sit behind all first-slot rows of the expert
    for s in np.flatnonzero(i2 >= 0):
        assert il[1][S + s] == l2[s] + u1[i2[s]]
        np.testing.assert_array_equal(disp[i2[s], il[1][S + s]], data[s])
    # combine weights: post-drop values normalised to sum 1 wherever a slot survived
    tot = gates[:S] + gates[S:]
    alive = (i1 >= 0) | (i2 >= 0)
    np.testing.assert_allclose(tot[alive & (val[0] * (i1 >= 0) + val[1] * (i2 >= 0) > 1e-6)], 1.0, rtol=1e-5)
    assert not tot[~alive].any()

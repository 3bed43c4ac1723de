"""CPU restatement (NumPy) of the reference's MoE token-dispatch ops.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the HIP path is
compared against; nothing in the shipped package imports it.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may call it.

Every function restates an algorithm of the reference (paths relative to the
reference tree) and cites the lines it follows.  The style is deliberately the
one the reference's own test references use (one-hot + cumsum locations and a
Python scatter loop, tests/python/op/cuda/test_cuda_moe.py:114-137), so that
timing it gives "the NumPy reference path" of the baseline.

Parity status of each function (what pins it, beyond re-reading the source):
  capacity            closed form; hand-computed cases in tests/test_oracle_moe.py
  softmax_rows        scipy.special.softmax / fp64 evaluation at 1e-6
  select_topk         brute-force Python loop; numpy argmax first-max rule.
                      TIE-BREAK OF THE REFERENCE IS "parity unpinned": the
                      reference selects with a TVM-compiled argmax whose source
                      is absent (3rdparty/tvm is an empty submodule); its tests
                      only compare against np.argmax on tie-free random input.
                      We fix ties -> lowest expert index.
  moe_encode          brute-force token loop (tests), invariants (bijection of
                      locations onto [0,kept), used_out closed form, rows
                      bit-equal to source rows), chained-partition identity
  moe_encode_bpr      brute-force per-expert sort; partition independence of the
                      drop set.  STABILITY OF THE REFERENCE ARGSORT IS "parity
                      unpinned" (TVM argsort, source absent); we fix a stable
                      descending order, ties by ascending token id.
  moe_merge_masks /
  moe_redispatch      identity "partitioned == un-partitioned" of
                      test_cuda_moe.py:384-471
  moe_encode_top2     dense einsum form of docker/resources/sharded_moe.py:253-324
                      at tiny sizes; identity with two chained top-1 encodes
  moe_decode          round trip decode(encode(x), gate=1) == x on kept tokens
  backward ops        torch autograd through dense einsum forms of the forward
  moe_encode_dgate    torch autograd through a dense restatement of top2gating
                      (docker/resources/sharded_moe.py:253-324: softmax, capacity masks, clamp,
                      normalisation), incl. a case below the clamp; peaked rows by the
                      closed form of a two-expert softmax
"""
import numpy as np

F32_EPS = np.float32(1.1920929e-07)  # torch.finfo(torch.float32).eps, sharded_moe.py:310


# --------------------------------------------------------------------------
# T1: shape contract
# --------------------------------------------------------------------------
def capacity(S, E, capacity_factor):
    """C = int(float(cf) * ((S + E - 1) / E)): integer ceil-div, float multiply,
    truncation.  src/op/dialect/cuda/moe.cc:107-109, src/op/declare/moe.cc:46."""
    return int(np.float32(capacity_factor) * np.float32((S + E - 1) // E))


def gshard_top2_capacity(S, E, capacity_factor):
    """ceil(2 * S / E * cf) in double precision (docker/resources/sharded_moe.py:267): GShard's own top-2
    capacity.  The top-2 extension here follows the reference op's formula with the factor doubled
    (capacity(S, E, 2 * cf)); the two agree when E divides S and 2 * cf * S / E is whole."""
    import math
    return int(math.ceil((2 * S / E) * capacity_factor))


# --------------------------------------------------------------------------
# A0: gate softmax (outside the reference op; models/benchmark/pytorch/utils.py:565-573)
# --------------------------------------------------------------------------
def softmax_rows(logits):
    """p[s,:] = exp(x - max) / sum_e exp(x - max), fp32, sum taken in expert order."""
    x = np.asarray(logits, dtype=np.float32)
    ex = np.exp(x - x.max(axis=1, keepdims=True), dtype=np.float32)
    acc = np.zeros(x.shape[0], dtype=np.float32)
    for j in range(x.shape[1]):  # sequential fp32 sum over experts
        acc = acc + ex[:, j]
    return (ex / acc[:, None]).astype(np.float32)


# --------------------------------------------------------------------------
# A1 / A2 front end: top-1 / top-2 selection on the array the op is given
# --------------------------------------------------------------------------
def select_topk(gate, k=1, gate_is_logits=False, gate2_noise=None):
    """Returns (idx [k,S] int32, val [k,S] fp32).

    idx[0] = argmax_e gate[s,e] (first max; src/op/dialect/cuda/moe.cc:177-195,
    tests/python/op/cuda/test_cuda_moe.py:115).  idx[1] = argmax with idx[0]
    masked to -inf (docker/resources/sharded_moe.py:275-278); gate2_noise [S,E], if given,
    is added (fp32) to the array for that second choice alone, as the Gumbel noise of :275 is.
    val = gate[s, idx] (moe.cc:232-250: sum_e gate*onehot), or the softmax
    probability of that expert when the array holds logits."""
    g = np.asarray(gate, dtype=np.float32)
    S, E = g.shape
    rows = np.arange(S)
    prob = softmax_rows(g) if gate_is_logits else g
    idx = np.empty((k, S), dtype=np.int32)
    val = np.empty((k, S), dtype=np.float32)
    i1 = np.argmax(g, axis=1).astype(np.int32) if S else np.zeros(0, np.int32)
    idx[0] = i1
    val[0] = prob[rows, i1]
    if k == 2:
        assert E >= 2
        masked = g.copy() if gate2_noise is None else (g + np.asarray(gate2_noise, dtype=np.float32)).astype(np.float32)
        masked[rows, i1] = -np.inf
        # argmax of a row that is all -inf apart from i1 must not return i1
        i2 = np.argmax(masked, axis=1).astype(np.int32)
        clash = i2 == i1
        if clash.any():
            i2[clash] = np.where(i1[clash] == 0, 1, 0)
        idx[1] = i2
        val[1] = prob[rows, i2]
    return idx, val


def _ranks(idx0, E):
    """rank[s] = #{t < s : idx0[t] == idx0[s]}, via one-hot cumsum - 1
    (test_cuda_moe.py:116-123).  idx0 < 0 means "no expert" and gets rank 0."""
    S = idx0.shape[0]
    if S == 0:
        return np.zeros(0, np.int32), np.zeros(E, np.int64)
    onehot = idx0[:, None] == np.arange(E, dtype=np.int32)[None, :]
    cums = np.cumsum(onehot, axis=0, dtype=np.int32)
    safe = np.where(idx0 >= 0, idx0, 0)
    rank = cums[np.arange(S), safe] - 1
    rank = np.where(idx0 >= 0, rank, 0).astype(np.int32)
    return rank, cums[-1].astype(np.int64)


# --------------------------------------------------------------------------
# A3: gen_location (tutel_moe_dispatch.cu:164-212)
# --------------------------------------------------------------------------
def gen_location(idx0, used_in, C, M, E):
    """Returns (idx, loc, used_out, elems).  loc = rank among tokens of the same
    expert (written for dropped tokens too, :198); dropped <=> loc >= C - used_in
    (:199-201) -> idx = -1; used_out = min(used_in + cnt, C) (:207-209);
    elems = (used_out - used_in) * M (:210)."""
    idx0 = np.asarray(idx0, dtype=np.int32)
    used_in = np.asarray(used_in, dtype=np.int32)
    rank, cnt = _ranks(idx0, E)
    safe = np.where(idx0 >= 0, idx0, 0)
    drop = (idx0 >= 0) & (rank >= (C - used_in[safe]))
    idx = np.where(drop, -1, idx0).astype(np.int32)
    used_out = np.minimum(used_in.astype(np.int64) + cnt, C).astype(np.int32)
    elems = ((used_out.astype(np.int64) - used_in) * M).astype(np.uint64)
    return idx, rank, used_out, elems


# --------------------------------------------------------------------------
# A4: encode_forward scatter (tutel_moe_dispatch.cu:61-81, launchers :461-484)
# --------------------------------------------------------------------------
def scatter_rows(data, idx, loc, E, C, avail=None):
    """Zero [E,C,M]; for tokens with 0<=idx<E, 0<=loc<C (and loc < avail[idx] when
    given): out[idx, loc, :] = data[s, :].  The Python loop is the reference's
    test reference (test_cuda_moe.py:124-127)."""
    S, M = data.shape
    out = np.zeros((E, C, M), dtype=data.dtype)
    for s in range(S):
        e, l = int(idx[s]), int(loc[s])
        if 0 <= e < E and 0 <= l < C and (avail is None or l < avail[e]):
            out[e, l, :] = data[s, :]
    return out


def scatter_rows_fast(data, idx, loc, E, C):
    """Vectorised form of scatter_rows (same result; used where the loop is too slow)."""
    S, M = data.shape
    out = np.zeros((E, C, M), dtype=data.dtype)
    ok = (idx >= 0) & (idx < E) & (loc >= 0) & (loc < C)
    out[idx[ok], loc[ok]] = data[ok]
    return out


# --------------------------------------------------------------------------
# A.1: raf.op.moe_encode (moe.cc:346-396)
# --------------------------------------------------------------------------
def moe_encode(data, gate, used_in, capacity_factor=1.0, gate_is_logits=False,
               C=None, fast_scatter=False):
    """Returns the reference 5-tuple (src/op/declare/moe.cc:48-58):
    gates_s [S] fp32, indices_locations [2,S] int32, used_capacity [E] int32,
    elements_per_expert [E] uint64, dispatched [E,C,M]."""
    data = np.asarray(data)
    S, M = data.shape
    E = gate.shape[1]
    if C is None:
        C = capacity(S, E, capacity_factor)
    sel, val = select_topk(gate, 1, gate_is_logits)
    idx, loc, used_out, elems = gen_location(sel[0], used_in, C, M, E)
    fn = scatter_rows_fast if fast_scatter else scatter_rows
    disp = fn(data, idx, loc, E, C)
    return val[0], np.stack([idx, loc]).astype(np.int32), used_out, elems, disp


# --------------------------------------------------------------------------
# A.2: raf.op.moe_encode_batch_prioritized (moe.cc:415-729,
#      tutel_moe_dispatch.cu:259-363, test reference test_cuda_moe.py:270-309)
# --------------------------------------------------------------------------
def moe_encode_bpr(data, gate, n_partitions=1, partition_id=0, capacity_factor=1.0,
                   gate_is_logits=False, C=None, priorities=None, fast_scatter=False):
    """`priorities`, when given, replaces gates0 as the sort key (used to re-sort
    keys a device emitted, since exp() is not bit-portable)."""
    data = np.asarray(data)
    S0, M = data.shape
    E = gate.shape[1]
    P = int(n_partitions)
    S = S0 // P
    if C is None:
        C = capacity(S, E, capacity_factor)
    sel, val = select_topk(gate, 1, gate_is_logits)
    idx0, gates0 = sel[0], val[0]
    key = gates0 if priorities is None else np.asarray(priorities, dtype=np.float32)
    # descending, stable: ties keep ascending token order (moe.cc:701-719 argsort,
    # is_ascend=false; np.argsort(-x) in test_cuda_moe.py:189)
    order = np.argsort(-key.astype(np.float64), kind="stable")
    # pass 1 (:276-313): rank within expert in priority order, keep = rank < C
    rank_sorted, _ = _ranks(idx0[order], E)
    keep = np.empty(S0, dtype=bool)
    keep[order] = rank_sorted < C
    # pass 2 (:317-356): compact locations over this partition's kept tokens
    lo = partition_id * S
    pidx0 = idx0[lo:lo + S]
    pkeep = keep[lo:lo + S]
    rank_kept, cnt_kept = _ranks(np.where(pkeep, pidx0, -1).astype(np.int32), E)
    idx = np.where(pkeep, pidx0, -1).astype(np.int32)
    loc = np.where(pkeep, rank_kept, -1).astype(np.int32)
    used_out = np.minimum(cnt_kept, C).astype(np.int32)         # :358-360
    elems = (used_out.astype(np.int64) * M).astype(np.uint64)   # :361
    fn = scatter_rows_fast if fast_scatter else scatter_rows
    disp = fn(data[lo:lo + S], idx, loc, E, C)
    return gates0[lo:lo + S].copy(), np.stack([idx, loc]).astype(np.int32), used_out, elems, disp


# --------------------------------------------------------------------------
# A.3: raf.op.moe_merge_masks (moe.cc:731-823, tutel_moe_dispatch.cu:214-255)
# --------------------------------------------------------------------------
def moe_merge_masks(indlocs, E):
    P = len(indlocs)
    S = indlocs[0].shape[1]
    out = np.empty((2, P * S), dtype=np.int32)
    off = np.zeros(E, dtype=np.int64)
    for p, il in enumerate(indlocs):
        idx, loc = il[0], il[1]
        kept = idx >= 0
        safe = np.where(kept, idx, 0)
        out[0, p * S:(p + 1) * S] = np.where(kept, idx, -1)
        out[1, p * S:(p + 1) * S] = np.where(kept, loc + off[safe], -1)
        off += np.bincount(idx[kept], minlength=E)[:E]
    return out


# --------------------------------------------------------------------------
# A.4: raf.op.moe_redispatch (moe.cc:826-943, tutel_moe_dispatch.cu:365-408)
# --------------------------------------------------------------------------
def moe_redispatch(bufs, indlocs):
    """out[e, off_p[e] + r, :] = buf_p[e, r, :] for r < kept_p[e].  Rows the
    reference leaves uninitialised are defined as zero here."""
    E, C, M = bufs[0].shape
    out = np.zeros((E, C, M), dtype=bufs[0].dtype)
    off = np.zeros(E, dtype=np.int64)
    for buf, il in zip(bufs, indlocs):
        idx = il[0]
        cnt = np.bincount(idx[idx >= 0], minlength=E)[:E]
        for e in range(E):
            n = int(min(cnt[e], C - off[e]))
            if n > 0:
                out[e, off[e]:off[e] + n] = buf[e, :n]
        off += cnt
    return out


# --------------------------------------------------------------------------
# A.5: raf.op.moe_decode (moe.cc:1228-1311, tutel_moe_dispatch.cu:46-55,110-116,
#      test reference test_cuda_moe.py:1157-1165)
# --------------------------------------------------------------------------
def _to_f32(a):
    return np.asarray(a).astype(np.float32)


def moe_decode(expert_out, gates_s, indloc, k=1, round_fn=None):
    """out[s] = sum over the k slots of gates_s * expert_out[idx, loc]; products and
    the sum are fp32 (each rounded), one final rounding to the storage dtype via
    round_fn.  Slot j of token s lives at column j*S + s (slot-major)."""
    E, C, M = expert_out.shape
    S = indloc.shape[1] // k
    acc = np.zeros((S, M), dtype=np.float32)
    x = _to_f32(expert_out)
    for j in range(k):
        idx = indloc[0, j * S:(j + 1) * S]
        loc = indloc[1, j * S:(j + 1) * S]
        g = np.asarray(gates_s[j * S:(j + 1) * S], dtype=np.float32)
        ok = (idx >= 0) & (idx < E) & (loc >= 0) & (loc < C)
        rows = np.zeros((S, M), dtype=np.float32)
        rows[ok] = x[idx[ok], loc[ok]] * g[ok, None]
        acc = rows if j == 0 else (acc + rows).astype(np.float32)
    return acc if round_fn is None else round_fn(acc)


# --------------------------------------------------------------------------
# A.6: top-2 extension (docker/resources/sharded_moe.py:253-324, no Gumbel noise)
# --------------------------------------------------------------------------
def moe_encode_top2(data, gate, used_in, capacity_factor=1.0, gate_is_logits=False,
                    C=None, fast_scatter=False, gate2_noise=None, gate_round=None):
    """GShard top-2 expressed as two chained reference top-1 encodes, merged:
    slot 1 with used_in, slot 2 with used_out(slot 1); merged layout is what
    moe_merge_masks/moe_redispatch give for the two calls.  Capacity follows the
    reference formula with capacity_factor' = 2*capacity_factor
    (sharded_moe.py:267).  Combine weights are taken after the drop and
    normalised by max(g1+g2, eps) (:296-312).  gate_round (a 16-bit gate array: the
    function that rounds fp32 to its type, result as fp32): the two raw gate values
    are what a gates_s array of that type holds, i.e. rounded, before the fp32
    normalisation; rounding the returned weights to the type is the caller's."""
    data = np.asarray(data)
    S, M = data.shape
    E = gate.shape[1]
    if C is None:
        C = capacity(S, E, 2.0 * capacity_factor)
    sel, val = select_topk(gate, 2, gate_is_logits, gate2_noise)
    if gate_round is not None:
        val = gate_round(val).astype(np.float32)
    used_in = np.asarray(used_in, dtype=np.int32)
    i1, l1, used1, _ = gen_location(sel[0], used_in, C, M, E)
    i2, l2, used2, _ = gen_location(sel[1], used1, C, M, E)
    merged = moe_merge_masks([np.stack([i1, l1]), np.stack([i2, l2])], E)
    g1 = np.where(i1 >= 0, val[0], np.float32(0)).astype(np.float32)
    g2 = np.where(i2 >= 0, val[1], np.float32(0)).astype(np.float32)
    den = np.maximum((g1 + g2).astype(np.float32), F32_EPS)
    gates = np.concatenate([g1 / den, g2 / den]).astype(np.float32)
    fn = scatter_rows_fast if fast_scatter else scatter_rows
    disp = fn(np.concatenate([data, data]), merged[0], merged[1], E, C)
    elems = ((used2.astype(np.int64) - used_in) * M).astype(np.uint64)
    return gates, merged, used2, elems, disp


def top2_normalize_gates(raw_gates, merged_idx):
    """Combine weights from raw per-slot gate values and merged (post-drop) indices."""
    S = raw_gates.shape[0] // 2
    g1 = np.where(merged_idx[:S] >= 0, raw_gates[:S], np.float32(0)).astype(np.float32)
    g2 = np.where(merged_idx[S:] >= 0, raw_gates[S:], np.float32(0)).astype(np.float32)
    den = np.maximum((g1 + g2).astype(np.float32), F32_EPS)
    return np.concatenate([g1 / den, g2 / den]).astype(np.float32)


# --------------------------------------------------------------------------
# bf16 helpers (round-to-nearest-even on the fp32 bit pattern)
# --------------------------------------------------------------------------
def f32_to_bf16_bits(a):
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = np.isnan(np.asarray(a, dtype=np.float32))
    out = rounded.astype(np.uint16)
    out[nan] = 0x7FC0
    return out


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to_bf16(a):
    """fp32 -> nearest bf16 value, returned as fp32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a))


def round_to_f16(a):
    """fp32 -> nearest fp16 value (round to nearest even), returned as fp32."""
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


# --------------------------------------------------------------------------
# backward ops (gradients wired by src/op/grad/moe.cc:30-93)
# Pinned in tests/test_oracle_moe.py against torch autograd of the dense einsum forms.
# --------------------------------------------------------------------------
def _valid(indloc, k, E, C):
    idx, loc = indloc[0], indloc[1]
    return (idx >= 0) & (idx < E) & (loc >= 0) & (loc < C)


def moe_encode_dx(dy, indloc, k=1):
    """dx[s] = sum over slots of dy[idx, loc] (encode_backward_data_kernel,
    tutel_moe_dispatch.cu:46-55,88-94); products with the unit gate are exact."""
    E, C, M = dy.shape
    S = indloc.shape[1] // k
    return moe_decode(dy, np.ones(k * S, np.float32), indloc, k=k)


def moe_encode_dg(dy_gates_s, indloc, n_experts, k=1):
    """grad_gates[S,E]: zero, then grad[s, idx] = dy (encode_backward_gate_kernel, :96-105,499-506)."""
    S = indloc.shape[1] // k
    out = np.zeros((S, n_experts), np.float32)
    for j in range(k):
        idx = indloc[0, j * S:(j + 1) * S]
        ok = (idx >= 0) & (idx < n_experts)
        out[np.arange(S)[ok], idx[ok]] = dy_gates_s[j * S:(j + 1) * S][ok]
    return out


def moe_encode_dgate(dy_gates_s, gate, indloc, k=1, gate_is_logits=False):
    """Gradient of the [S,E] gate input of moe_encode / moe_encode_top2 given the gradient of the op's OUTPUT
    gates_s [k*S]; fp64 arithmetic on the fp32 inputs.  What MoeEncodeGrad (src/op/grad/moe.cc:30-58) gives for the
    reference's one form (k = 1 on probabilities: moe_encode_dg), extended to what the top-2 op does to a gate
    value (docker/resources/sharded_moe.py:296-312): g_j = p[s, i_j] * mask_j (masks after the capacity drop),
    w_j = g_j / clamp(g_1 + g_2, min=eps); torch.clamp passes the gradient where the sum is >= eps and none
    below.  With gate_is_logits the array holds logits and p = softmax(logits) (:260), differentiated too.
    Pinned in tests/test_oracle_moe.py by torch autograd through a dense restatement of top2gating, and for peaked
    rows by the closed form of a two-expert softmax."""
    gate = np.asarray(gate, np.float64)
    S, E = gate.shape
    dy = np.asarray(dy_gates_s, np.float64)
    if gate_is_logits:
        ex = np.exp(gate - gate.max(axis=1, keepdims=True))
        p = ex / ex.sum(axis=1, keepdims=True)
    else:
        p = gate
    rows = np.arange(S)
    idx = [np.asarray(indloc[0, j * S:(j + 1) * S]) for j in range(k)]
    kept = [(i >= 0) & (i < E) for i in idx]
    safe = [np.where(m, i, 0) for i, m in zip(idx, kept)]
    g = [np.where(m, p[rows, i], 0.0) for i, m in zip(safe, kept)]
    if k == 1:
        d = [np.where(kept[0], dy[:S], 0.0)]
    else:
        eps = float(F32_EPS)
        tot = g[0] + g[1]
        live = (g[0].astype(np.float32) + g[1].astype(np.float32)) >= F32_EPS   # the forward's own fp32 sum decides
        den2 = np.where(live, tot * tot, 1.0)
        d1 = np.where(live, (dy[:S] - dy[S:]) * g[1] / den2, dy[:S] / eps)
        d2 = np.where(live, (dy[S:] - dy[:S]) * g[0] / den2, dy[S:] / eps)
        d = [np.where(kept[0], d1, 0.0), np.where(kept[1], d2, 0.0)]
    dp = np.zeros((S, E), np.float64)
    for j in range(k):
        np.add.at(dp, (rows, safe[j]), d[j])
    if not gate_is_logits:
        return dp
    out = p * (dp - (p * dp).sum(axis=1, keepdims=True))
    # The entries that carry a slot gradient again, without 1 - p_j as a difference: in a peaked row (p_j within
    # 1e-11 of 1) that difference loses five of fp64's digits.  1 - p_j is the sum of the OTHER exponentials over
    # the whole sum, and d_j (1 - p_j) - sum_{l != j} p_l d_l is the same number as d_j - sum_l p_l d_l.
    tot = ex.sum(axis=1)
    for j in range(k):
        others = ex.copy()
        others[rows, safe[j]] = 0.0
        rest = others.sum(axis=1) / tot
        cross = sum((p[rows, safe[l]] * d[l] for l in range(k) if l != j), np.zeros(S))
        val = p[rows, safe[j]] * (d[j] * rest - cross)
        out[rows[kept[j]], safe[j][kept[j]]] = val[kept[j]]
    return out


def moe_decode_dx(dy, gates_s, indloc, n_experts, capacity, k=1, round_fn=None):
    """grad_expert_out[idx, loc] = gates_s * dy[s], zero elsewhere (decode_backward_data_kernel,
    :118-124,523-533: memset + atomicAdd onto distinct rows)."""
    S, M = dy.shape
    out = np.zeros((n_experts, capacity, M), np.float32)
    ok = _valid(indloc, k, n_experts, capacity)
    tok = np.tile(np.arange(S), k)
    g = np.asarray(gates_s, np.float32)
    out[indloc[0][ok], indloc[1][ok]] = _to_f32(dy)[tok[ok]] * g[ok, None]
    return out if round_fn is None else round_fn(out)


def moe_decode_dg(dy, expert_out, indloc, k=1):
    """grad_gates_s[i] = <expert_out[idx, loc], dy[s]> (decode_backward_gate_kernel, :126-157), 0 for
    dropped slots.  fp64 accumulation here; the device sums fp32 partials in a tree."""
    E, C, M = expert_out.shape
    S = dy.shape[0]
    ok = _valid(indloc, k, E, C)
    tok = np.tile(np.arange(S), k)
    out = np.zeros(k * S, np.float64)
    a = _to_f32(expert_out).astype(np.float64)
    b = _to_f32(dy).astype(np.float64)
    out[ok] = np.einsum("nm,nm->n", a[indloc[0][ok], indloc[1][ok]], b[tok[ok]])
    return out.astype(np.float32)


# --------------------------------------------------------------------------
# moe_redispatch_expert_input (moe.cc:945-1073, tutel_moe_dispatch.cu:436-456)
# Pinned in tests/test_oracle_moe.py by the reference's own protocol: the merge of P row-compacted
# partitions equals the un-partitioned buffer on the received rows.
# --------------------------------------------------------------------------
def moe_redispatch_expert_input(bufs, recv_cnts, local_expert_id, n_local_experts, scale=1):
    """bufs[p]: [C, G, M]; recv_cnts[p]: uint64 [G*LE] element counts.  For source g the element
    streams of the partitions are concatenated; stream element x -> out[x // M, g, x % M].  Rows the
    reference leaves untouched are zero here."""
    C, G, M = bufs[0].shape
    out = np.zeros((C, G, M), bufs[0].dtype)
    for g in range(G):
        stream = []
        for buf, cnt in zip(bufs, recv_cnts):
            n = int(cnt[g * n_local_experts + local_expert_id]) * scale
            stream.append(buf[:, g, :].reshape(-1)[:n])
        flat = np.concatenate(stream)[:C * M]
        col = np.zeros(C * M, bufs[0].dtype)
        col[:flat.size] = flat
        out[:, g, :] = col.reshape(C, M)
    return out


# ----------------------------------------------------------------------------- sparse <-> packed copies
def sparse_copy_extents(nelements_per_dim, stride, offset, nblocks, scale=1, shrink=1):
    """(off_b, n_b) of sparse_memcpy.cu:16-36: the counts of the blocks before b are summed first and the sum
    is then scaled; the block's own count is scaled by itself."""
    c = [int(nelements_per_dim[b * stride + offset]) for b in range(nblocks)]
    offs, run = [], 0
    for b in range(nblocks):
        offs.append(run * scale // shrink)
        run += c[b]
    return offs, [x * scale // shrink for x in c]


def _sparse_block_view(buf, axis, b):
    # the block's elements in stream order: INDEX3Ddim0 / INDEX3Ddim1, sparse_memcpy.cu:43-46
    return buf[b].reshape(-1) if axis == 0 else buf[:, b, :].reshape(-1)


def memcpy_sparse_to_cont_3d(src, dst, nelements_per_dim, stride=1, offset=0, axis=0, scale=1, shrink=1):
    """memcpy_sparse_to_cont_3d_dim{0,1}_kernel, sparse_memcpy.cu:48-53: returns dst (1-D) with the packed
    stream written; what the stream does not cover keeps dst's values.  Counts are clipped to the block and
    to dst (the source would run out of bounds)."""
    out = np.array(dst, copy=True).reshape(-1)
    nb = src.shape[axis]
    offs, ns = sparse_copy_extents(nelements_per_dim, stride, offset, nb, scale, shrink)
    for b in range(nb):
        blk = _sparse_block_view(src, axis, b)
        n = max(0, min(ns[b], blk.size, out.size - offs[b]))
        out[offs[b]:offs[b] + n] = blk[:n]
    return out


def memcpy_cont_to_sparse_3d(src, dst, nelements_per_dim, stride=1, offset=0, axis=0, scale=1, shrink=1,
                             zero_tail=False):
    """memcpy_cont_to_sparse_3d_dim{0,1}_kernel, sparse_memcpy.cu:55-60: returns dst (3-D) with every block's
    first n_b elements taken from the packed stream; the rest keeps dst's values (zero with zero_tail)."""
    out = np.array(dst, copy=True)
    flat = np.asarray(src).reshape(-1)
    nb = out.shape[axis]
    offs, ns = sparse_copy_extents(nelements_per_dim, stride, offset, nb, scale, shrink)
    for b in range(nb):
        blk = np.array(_sparse_block_view(out, axis, b), copy=True)
        n = max(0, min(ns[b], blk.size, flat.size - offs[b]))
        blk[:n] = flat[offs[b]:offs[b] + n]
        if zero_tail:
            blk[n:] = 0
        if axis == 0:
            out[b] = blk.reshape(out.shape[1], out.shape[2])
        else:
            out[:, b, :] = blk.reshape(out.shape[0], out.shape[2])
    return out



# --------------------------------------------------------------------------
# Row ranges of token partitions inside a whole-batch routing, and the sparse copies on ranges.  No counterpart in
# the reference; pinned in tests/test_oracle_moe.py by the identity they exist for: packing the ranges of
# partition p out of the whole-batch buffer gives what packing partition p's own chained encode gives
# (tests/python/op/cuda/test_cuda_moe.py:384-471 protocol + sparse_memcpy.cu semantics).
# --------------------------------------------------------------------------
def moe_partition_ranges(indloc, n_partitions, n_experts, M, k=1):
    """(starts, counts) uint64 [k*P, E] in elements: counts[j*P+p][e] = M * #kept tokens of partition p with slot-j
    expert e; starts = running sum over the rows before (slot-major, then partition: the capacity order)."""
    S = indloc.shape[1] // k
    Sp = S // n_partitions
    Q = k * n_partitions
    counts = np.zeros((Q, n_experts), np.uint64)
    for j in range(k):
        for p in range(n_partitions):
            idx = indloc[0, j * S + p * Sp: j * S + (p + 1) * Sp]
            kept = idx[(idx >= 0) & (idx < n_experts)]
            counts[j * n_partitions + p] = np.bincount(kept, minlength=n_experts).astype(np.uint64) * np.uint64(M)
    starts = np.zeros_like(counts)
    starts[1:] = np.cumsum(counts, axis=0, dtype=np.uint64)[:-1]
    return starts, counts


def memcpy_sparse_ranges_to_cont_3d(src, dst, counts, starts, axis=0):
    """Packs elements [start_b, start_b + n_b) of every block b (stream order of the block) into dst."""
    out = np.array(dst, copy=True).reshape(-1)
    off = 0
    for b in range(src.shape[axis]):
        blk = _sparse_block_view(src, axis, b)
        s0 = min(int(starts[b]), blk.size)
        n = max(0, min(int(counts[b]), blk.size - s0, out.size - off))
        out[off:off + n] = blk[s0:s0 + n]
        off += int(counts[b])
    return out


def memcpy_cont_to_sparse_ranges_3d(src, dst, counts, starts, axis=0):
    """The inverse: only the ranges of dst are written."""
    out = np.array(dst, copy=True)
    flat = np.asarray(src).reshape(-1)
    off = 0
    for b in range(out.shape[axis]):
        blk = np.array(_sparse_block_view(out, axis, b), copy=True)
        s0 = min(int(starts[b]), blk.size)
        n = max(0, min(int(counts[b]), blk.size - s0, flat.size - off))
        blk[s0:s0 + n] = flat[off:off + n]
        if axis == 0:
            out[b] = blk.reshape(out.shape[1], out.shape[2])
        else:
            out[:, b, :] = blk.reshape(out.shape[0], out.shape[2])
        off += int(counts[b])
    return out

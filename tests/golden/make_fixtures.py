"""Writes tests/golden/*.npz: small seeded input/output vectors of every operator of the path.

The reference tree stores no golden vectors for this path (its tests compare a CUDA run with an
inline NumPy reference and keep nothing), so these vectors are produced by this repository's
NumPy oracle after it has passed tests/test_oracle_*.py (brute force, dense GShard form, paper
fp64 LANS).  They freeze the oracle's behaviour: a later edit of the oracle that changes any
output fails tests/test_golden.py, and the HIP path is checked against the same files.

    python tests/golden/make_fixtures.py            # writes the files that do not exist yet (existing ones stay frozen)
    python tests/golden/make_fixtures.py --force    # rewrites all of them
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import lans_oracle as lo  # noqa: E402
from oracle import moe_oracle as mo  # noqa: E402


def inputs(seed, S, M, E, ties=False, hot=False):
    rng = np.random.default_rng(seed)
    data = rng.standard_normal((S, M), dtype=np.float32)
    logits = rng.standard_normal((S, E), dtype=np.float32)
    if hot:
        logits[:, 0] += np.float32(1.5)
    if ties:
        logits = (np.round(logits * 2) / 2).astype(np.float32)
    return data, logits


def main():
    out = {}
    # moe_encode, top-1, on probabilities, with a used-capacity vector
    data, logits = inputs(1, 64, 8, 4, hot=True)
    gate = mo.softmax_rows(logits)
    used = np.array([0, 3, 16, 1], np.int32)
    r = mo.moe_encode(data, gate, used, 1.0)
    out["encode_top1"] = dict(data=data, gate=gate, used_in=used, cf=np.float32(1.0), gates_s=r[0], indloc=r[1],
                              used_out=r[2], elems=r[3], dispatched=r[4])
    # moe_encode on tied logits (first-max rule)
    data, logits = inputs(2, 48, 4, 8, ties=True)
    r = mo.moe_encode(data, logits, np.zeros(8, np.int32), 0.5)
    out["encode_top1_ties"] = dict(data=data, gate=logits, used_in=np.zeros(8, np.int32), cf=np.float32(0.5),
                                   gates_s=r[0], indloc=r[1], used_out=r[2], elems=r[3], dispatched=r[4])
    # top-2 extension on logits
    data, logits = inputs(3, 60, 8, 6, hot=True)
    r = mo.moe_encode_top2(data, logits, np.zeros(6, np.int32), 0.75, gate_is_logits=True)
    out["encode_top2"] = dict(data=data, gate=logits, cf=np.float32(0.75), gates_s=r[0], indloc=r[1], used_out=r[2],
                              elems=r[3], dispatched=r[4])
    dec = mo.moe_decode(r[4] * np.float32(2.0), r[0], r[1], k=2)
    out["decode_top2"] = dict(expert_out=r[4] * np.float32(2.0), gates_s=r[0], indloc=r[1], out=dec)
    # batch prioritised, two partitions, tied priorities
    data, logits = inputs(4, 64, 4, 4, hot=True)
    gate = (np.round(mo.softmax_rows(logits) * 8) / 8).astype(np.float32)
    for pid in range(2):
        r = mo.moe_encode_bpr(data, gate, 2, pid, 1.0)
        out["bpr_p%d" % pid] = dict(data=data, gate=gate, n_partitions=np.int32(2), partition_id=np.int32(pid),
                                    cf=np.float32(1.0), gates_s=r[0], indloc=r[1], used_out=r[2], elems=r[3],
                                    dispatched=r[4])
    # chained partitions + merge + redispatch
    data, logits = inputs(5, 96, 4, 3, hot=True)
    gate = mo.softmax_rows(logits)
    used = np.zeros(3, np.int32)
    ils, bufs = [], []
    for p in range(3):
        sl = slice(p * 32, (p + 1) * 32)
        r = mo.moe_encode(data[sl], gate[sl], used, 2.0)
        used = r[2]
        ils.append(r[1]), bufs.append(r[4])
    out["merge_redispatch"] = dict(indlocs=np.stack(ils), bufs=np.stack(bufs), n_experts=np.int32(3),
                                   merged=mo.moe_merge_masks(ils, 3), redispatched=mo.moe_redispatch(bufs, ils))
    # decode top-1
    r = mo.moe_encode(data, gate, np.zeros(3, np.int32), 0.5)
    out["decode_top1"] = dict(expert_out=r[4], gates_s=r[0], indloc=r[1], out=mo.moe_decode(r[4], r[0], r[1]))
    # LANS: 3 tensors, 3 steps
    rng = np.random.default_rng(6)
    shapes = [(5, 7), (3,), (40,)]
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    lans = {"p0_%d" % i: a.copy() for i, a in enumerate(p)}
    for step in (1, 2, 3):
        g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
        for i, a in enumerate(g):
            lans["g%d_%d" % (step, i)] = a
        lo.lans_step(g, p, m, v, step)
    for i in range(3):
        lans["p3_%d" % i], lans["m3_%d" % i], lans["v3_%d" % i] = p[i], m[i], v[i]
    out["lans"] = lans
    # gate gradient of the whole op: top-1 / top-2, on probabilities / on logits, with dropped slots of every kind
    data, logits = inputs(7, 72, 2, 6, hot=True)
    dgate = dict(logits=logits)
    rng = np.random.default_rng(8)
    for k in (1, 2):
        for is_logits in (0, 1):
            gate = logits if is_logits else mo.softmax_rows(logits)
            enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
            il = enc(data, gate, np.zeros(6, np.int32), 0.6, gate_is_logits=bool(is_logits))[1]
            dy = rng.standard_normal(k * 72).astype(np.float32)
            tag = "k%d_l%d" % (k, is_logits)
            dgate["gate_" + tag], dgate["indloc_" + tag], dgate["dy_" + tag] = gate, il, dy
            dgate["grad_" + tag] = mo.moe_encode_dgate(dy, gate, il, k, bool(is_logits))
    out["encode_dgate"] = dgate
    # LANS of a bf16 model: bf16 gradients, fp32 master state, bf16 copies of the new parameters; 3 tensors, 3 steps
    rng = np.random.default_rng(9)
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    mixed = {"p0_%d" % i: a.copy() for i, a in enumerate(p)}
    for step in (1, 2, 3):
        g = [mo.round_to_bf16(rng.normal(0, 1e-3, s).astype(np.float32)) for s in shapes]
        for i, a in enumerate(g):
            mixed["g%d_%d" % (step, i)] = a
        low = lo.lans_step_mixed(g, p, m, v, step, mo.round_to_bf16)
    for i in range(3):
        mixed["p3_%d" % i], mixed["m3_%d" % i], mixed["v3_%d" % i], mixed["low3_%d" % i] = p[i], m[i], v[i], low[i]
    out["lans_mixed"] = mixed
    force = "--force" in sys.argv[1:]
    for name, arrays in out.items():
        path = os.path.join(HERE, name + ".npz")
        if os.path.exists(path) and not force:
            print("kept ", name)
            continue
        np.savez_compressed(path, **arrays)
        print("wrote", name, sum(a.nbytes for a in arrays.values()), "bytes")


if __name__ == "__main__":
    main()

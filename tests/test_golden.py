"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the NumPy oracle
must still reproduce them (CPU), and the HIP path must reproduce them on the GPU."""
import os

import numpy as np
import pytest

from oracle import lans_oracle as lo
from oracle import moe_oracle as mo

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gold(name):
    with np.load(os.path.join(GOLD, name + ".npz")) as z:
        return {k: z[k] for k in z.files}


def eq5(got, f):
    np.testing.assert_array_equal(got[1], f["indloc"])
    np.testing.assert_array_equal(got[2], f["used_out"])
    np.testing.assert_array_equal(got[3], f["elems"])
    np.testing.assert_array_equal(got[4], f["dispatched"])


def test_oracle_reproduces_fixtures():
    for name in ("encode_top1", "encode_top1_ties"):
        f = gold(name)
        got = mo.moe_encode(f["data"], f["gate"], f["used_in"], float(f["cf"]))
        eq5(got, f)
        np.testing.assert_array_equal(got[0], f["gates_s"])
    f = gold("encode_top2")
    got = mo.moe_encode_top2(f["data"], f["gate"], np.zeros(f["gate"].shape[1], np.int32), float(f["cf"]), gate_is_logits=True)
    eq5(got, f)
    np.testing.assert_array_equal(got[0], f["gates_s"])
    for pid in range(2):
        f = gold("bpr_p%d" % pid)
        eq5(mo.moe_encode_bpr(f["data"], f["gate"], 2, pid, float(f["cf"])), f)
    f = gold("merge_redispatch")
    np.testing.assert_array_equal(mo.moe_merge_masks(list(f["indlocs"]), 3), f["merged"])
    np.testing.assert_array_equal(mo.moe_redispatch(list(f["bufs"]), list(f["indlocs"])), f["redispatched"])
    for name, k in (("decode_top1", 1), ("decode_top2", 2)):
        f = gold(name)
        np.testing.assert_array_equal(mo.moe_decode(f["expert_out"], f["gates_s"], f["indloc"], k=k), f["out"])
    f = gold("lans")
    p = [f["p0_%d" % i].copy() for i in range(3)]
    m = [np.zeros_like(a) for a in p]
    v = [np.zeros_like(a) for a in p]
    for step in (1, 2, 3):
        lo.lans_step([f["g%d_%d" % (step, i)] for i in range(3)], p, m, v, step)
    for i in range(3):
        np.testing.assert_array_equal(p[i], f["p3_%d" % i])
        np.testing.assert_array_equal(m[i], f["m3_%d" % i])
        np.testing.assert_array_equal(v[i], f["v3_%d" % i])


def test_oracle_reproduces_the_gradient_and_mixed_precision_fixtures():
    f = gold("encode_dgate")
    for k in (1, 2):
        for is_logits in (0, 1):
            tag = "k%d_l%d" % (k, is_logits)
            got = mo.moe_encode_dgate(f["dy_" + tag], f["gate_" + tag], f["indloc_" + tag], k, bool(is_logits))
            np.testing.assert_array_equal(got, f["grad_" + tag])
            assert (f["indloc_" + tag][0] < 0).any() and np.abs(f["grad_" + tag]).max() > 0
    f = gold("lans_mixed")
    p = [f["p0_%d" % i].copy() for i in range(3)]
    m = [np.zeros_like(a) for a in p]
    v = [np.zeros_like(a) for a in p]
    for step in (1, 2, 3):
        low = lo.lans_step_mixed([f["g%d_%d" % (step, i)] for i in range(3)], p, m, v, step, mo.round_to_bf16)
    for i in range(3):
        np.testing.assert_array_equal(p[i], f["p3_%d" % i])
        np.testing.assert_array_equal(low[i], f["low3_%d" % i])
        np.testing.assert_array_equal(mo.round_to_bf16(f["p3_%d" % i]), f["low3_%d" % i])


@pytest.mark.gpu
def test_hip_path_reproduces_the_gradient_and_mixed_precision_fixtures(pkg):
    import torch
    from tests.gpu_util import dev, to_np
    ops = pkg.ops
    f = gold("encode_dgate")
    for k in (1, 2):
        for is_logits in (0, 1):
            tag = "k%d_l%d" % (k, is_logits)
            got = to_np(ops.moe_encode_dgate(dev(f["dy_" + tag]), dev(f["gate_" + tag]), dev(f["indloc_" + tag]), top_k=k,
                                             gate_is_logits=bool(is_logits)))
            want = f["grad_" + tag]
            scale = np.abs(want).max(axis=1, keepdims=True)
            assert (np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6 * scale).all()
    f = gold("lans_mixed")
    p = [dev(f["p0_%d" % i]) for i in range(3)]
    m = [torch.zeros_like(a) for a in p]
    v = [torch.zeros_like(a) for a in p]
    low = [torch.zeros_like(a, dtype=torch.bfloat16) for a in p]
    for step in (1, 2, 3):
        g = [dev(f["g%d_%d" % (step, i)]).to(torch.bfloat16) for i in range(3)]
        ops.lans(g + p + m + v, step, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True, p_lowp=low)
    for i in range(3):
        want = f["p3_%d" % i]
        assert np.abs(to_np(p[i]).astype(np.float64) - want).max() <= 1e-6 * np.abs(want).max()
        assert torch.equal(low[i], p[i].to(torch.bfloat16))
        ulp = (low[i].cpu().view(torch.int16).int() - torch.from_numpy(f["low3_%d" % i]).to(torch.bfloat16).view(torch.int16).int()).abs().max()
        assert int(ulp) <= 1


@pytest.mark.gpu
def test_hip_path_reproduces_fixtures(pkg):
    import torch
    from tests.gpu_util import dev, to_np
    ops = pkg.ops
    for name in ("encode_top1", "encode_top1_ties"):
        f = gold(name)
        got = ops.moe_encode(dev(f["data"]), dev(f["gate"]), dev(f["used_in"]), float(f["cf"]))
        eq5([to_np(t) for t in got], f)
        np.testing.assert_array_equal(to_np(got[0]), f["gates_s"])
    f = gold("encode_top2")
    got = ops.moe_encode(dev(f["data"]), dev(f["gate"]), None, float(f["cf"]), top_k=2, gate_is_logits=True)
    eq5([to_np(t) for t in got], f)
    np.testing.assert_allclose(to_np(got[0]), f["gates_s"], rtol=1e-5)
    for pid in range(2):
        f = gold("bpr_p%d" % pid)
        got = ops.moe_encode_batch_prioritized(dev(f["data"]), dev(f["gate"]), 2, pid, float(f["cf"]))
        eq5([to_np(t) for t in got], f)
    f = gold("merge_redispatch")
    ils = [dev(a) for a in f["indlocs"]]
    bufs = [dev(a) for a in f["bufs"]]
    np.testing.assert_array_equal(to_np(ops.moe_merge_masks(ils, 3)), f["merged"])
    np.testing.assert_array_equal(to_np(ops.moe_redispatch(bufs, ils)), f["redispatched"])
    for name, k in (("decode_top1", 1), ("decode_top2", 2)):
        f = gold(name)
        out = ops.moe_decode(dev(f["expert_out"]), dev(f["gates_s"]), dev(f["indloc"]), top_k=k)
        np.testing.assert_array_equal(to_np(out), f["out"])
    f = gold("lans")
    p = [dev(f["p0_%d" % i]) for i in range(3)]
    m = [torch.zeros_like(a) for a in p]
    v = [torch.zeros_like(a) for a in p]
    for step in (1, 2, 3):
        g = [dev(f["g%d_%d" % (step, i)]) for i in range(3)]
        ops.lans(g + p + m + v, step, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)
    for i in range(3):
        want = f["p3_%d" % i]
        assert np.abs(to_np(p[i]).astype(np.float64) - want).max() <= 1e-6 * np.abs(want).max()
        # m and v: 1e-5 relative, with a floor of 1e-6 of the tensor's largest entry (an entry of m in which
        # beta1 * m and (1 - beta1) * g / ||g|| cancel carries the last-place difference of ||g||, whose sum order
        # differs between schedules, at its full absolute size)
        for got_t, name in ((m[i], "m3_%d" % i), (v[i], "v3_%d" % i)):
            np.testing.assert_allclose(to_np(got_t), f[name], rtol=1e-5, atol=1e-6 * np.abs(f[name]).max())

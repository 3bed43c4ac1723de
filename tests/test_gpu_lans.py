"""GPU parity tests of the fused multi-tensor LANS step against the NumPy oracle.

Bar (BASELINE.json): parameters within 1e-6 relative after 10 steps.  Relative is taken per
tensor against the largest parameter magnitude (an elementwise relative error is undefined
for parameters that pass through zero); m and v are checked at 1e-5."""
import numpy as np
import pytest
import torch

from oracle import lans_oracle as lo
from tests.gpu_util import dev, to_np

pytestmark = pytest.mark.gpu

P_RTOL = 1e-6


def make_state(seed, shapes):
    rng = np.random.default_rng(seed)
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    return rng, p, m, v


def assert_close_scaled(got, want, rtol, what):
    scale = np.abs(want).max()
    err = np.abs(got.astype(np.float64) - want.astype(np.float64)).max()
    assert err <= rtol * max(scale, 1e-30), "%s: max err %.3e vs scale %.3e" % (what, err, scale)


def run_both(pkg, shapes, steps, seed=0, **hyper):
    rng, p, m, v = make_state(seed, shapes)
    dp, dm, dv = [dev(a) for a in p], [dev(a) for a in m], [dev(a) for a in v]
    args = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-6, bias_correction=1, weight_decay=0.01,
                grad_averaging=1, mode=1, normalize_grad=True)
    args.update(hyper)
    for step in range(1, steps + 1):
        g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
        dg = [dev(a) for a in g]
        lo.lans_step(g, p, m, v, step, **args)
        pkg.ops.lans(dg + dp + dm + dv, step, args["lr"], args["beta1"], args["beta2"], args["eps"],
                     args["bias_correction"], args["weight_decay"], args["grad_averaging"], args["mode"],
                     args["normalize_grad"])
        for a, b in zip(dg, g):   # g is not modified
            np.testing.assert_array_equal(to_np(a), b)
    for i in range(len(shapes)):
        assert_close_scaled(to_np(dp[i]), p[i], P_RTOL, "p[%d]" % i)
        assert_close_scaled(to_np(dm[i]), m[i], 1e-5, "m[%d]" % i)
        assert_close_scaled(to_np(dv[i]), v[i], 1e-5, "v[%d]" % i)
    return dp, dm, dv


def test_lans_gpt2_like_list_ten_steps(pkg):
    # a scaled-down slice of BASELINE config 5: matrices, biases/norms, sizes that are not a
    # multiple of 4 or of the chunk, a tensor spanning several chunks
    shapes = [(256, 256), (256, 1024), (1024, 256), (256,), (256,), (1000, 33), (7,), (1,), (16384 * 3 + 5,)]
    run_both(pkg, shapes, 10)


def test_lans_reference_test_shapes(pkg):
    # tests/python/optim/test_lans.py:140-161 (one 2x2 tensor, 4 steps) and :94-137
    # (conv 6x3x5x5, bn w/b 6, linear w/b: the >= 3 tensor case)
    run_both(pkg, [(2, 2)], 4, seed=1)
    run_both(pkg, [(6, 3, 5, 5), (6,), (6,), (10, 84), (10,)], 2, seed=2)


@pytest.mark.parametrize("hyper", [
    dict(mode=0), dict(weight_decay=0.0), dict(normalize_grad=False), dict(bias_correction=0),
    dict(grad_averaging=0), dict(mode=0, weight_decay=0.0, normalize_grad=False),
    dict(lr=5e-2, beta1=0.8, beta2=0.99, eps=1e-8),
    # mode 0 with weight decay: wd * p joins the scaled gradient before the moments (multi_tensor_lans.cu:287-297)
    dict(mode=0, weight_decay=0.25, lr=0.1, beta1=0.5, beta2=0.5, bias_correction=0),
])
def test_lans_flags(pkg, hyper):
    run_both(pkg, [(300, 40), (129,), (64, 64)], 5, seed=3, **hyper)


def test_lans_zero_norm_special_cases(pkg):
    """||g|| == 0 (no normalisation, u = wd*p) and ||p|| == 0 (ratio = lr)."""
    shapes = [(50,), (60,)]
    p = [np.linspace(-1, 1, 50).astype(np.float32), np.zeros(60, np.float32)]
    g = [np.zeros(50, np.float32), np.linspace(-1, 1, 60).astype(np.float32)]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    dg, dp, dm, dv = ([dev(a) for a in l] for l in (g, p, m, v))
    lo.lans_step(g, p, m, v, 1)
    pkg.ops.lans(dg + dp + dm + dv, 1, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)
    for i in range(2):
        assert_close_scaled(to_np(dp[i]), p[i], P_RTOL, "p[%d]" % i)
    np.testing.assert_allclose(to_np(dp[0]), np.linspace(-1, 1, 50) * (1 - 1e-3), rtol=1e-6, atol=1e-9)


def test_lans_unaligned_tensors_and_device_step(pkg):
    """Tensors that start 4 bytes past a 16-byte boundary take the scalar path; the step may be
    a device scalar (as the reference passes it)."""
    n = 5000
    rng = np.random.default_rng(9)
    host = [rng.normal(0, s, n).astype(np.float32) for s in (1e-3, 0.02)]
    g, p = host[0].copy(), host[1].copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    store = [torch.zeros(n + 1, device="cuda") for _ in range(4)]
    views = [s[1:] for s in store]
    for t, a in zip(views, (g, p, m, v)):
        t.copy_(torch.from_numpy(a))
    assert views[0].data_ptr() % 16 == 4
    step = torch.tensor(3.0, device="cuda")
    lo.lans_step([g], [p], [m], [v], 3)
    pkg.ops.lans(views, step, 1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)
    assert_close_scaled(to_np(views[1]), p, P_RTOL, "p")
    assert_close_scaled(to_np(views[2]), m, 1e-5, "m")


def test_lans_norms_and_plan_reuse(pkg):
    shapes = [(64, 64), (100,)]
    rng, p, m, v = make_state(5, shapes)
    g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
    plan = pkg.ops.LansPlan([a.size for a in p])
    hyper = pkg.capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    dg, dp, dm, dv = ([dev(a) for a in l] for l in (g, p, m, v))
    want = lo.lans_step(g, p, m, v, 1)
    plan.step(dg, dp, dm, dv, 1, hyper)
    np.testing.assert_allclose(to_np(plan.norms()).T, np.array(want, np.float32), rtol=2e-6)
    # new gradient tensors (different pointers) on the second step
    g2 = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
    lo.lans_step(g2, p, m, v, 2)
    plan.step([dev(a) for a in g2], dp, dm, dv, 2, hyper)
    for i in range(2):
        assert_close_scaled(to_np(dp[i]), p[i], P_RTOL, "p[%d]" % i)
    plan.close()


def _fresh_state(numels, seed, offset=0):
    """g, p, m, v as lists of separately allocated (so 16-byte aligned) tensors; with `offset`, every tensor is
    a view that starts `offset` elements into its allocation."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    def alloc(n, std):
        t = torch.zeros(n + offset, device="cuda")
        if std:
            t.normal_(0, std, generator=gen)
        return t[offset:]
    return [[alloc(n, std) for n in numels] for std in (1e-3, 0.02, 0, 0)]


def test_lans_resident_schedule(pkg):
    """The persistent-kernel schedule must terminate, leave its error word clear, be reproducible and agree
    with the three-sweep schedule to fp32 rounding of the per-chunk sums.  Tensors that are whole multiples
    of the 8192-parameter chunk go through the kernel (one chunk, several, a quarter of a round, a whole round
    of 512), the others through the sweeps of the same step."""
    capi = pkg.capi
    numels = [1000, 65536, 5, 1 << 20, 3 * 8192, 8193, 1, (2 << 20) + 17, 8192, 8192, 4 << 20, 2 << 20, 8192 * 131]
    resident_chunks = sum(n // 8192 for n in numels if n % 8192 == 0)
    results = []
    for schedule in (capi.LANS_SWEEPS, None, None):            # None: what a new plan has
        state = _fresh_state(numels, 7)
        plan = pkg.ops.LansPlan(numels, schedule=schedule)
        hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
        for step in (1, 2, 3):
            plan.step(*state, step, hyper)
        torch.cuda.synchronize()
        assert plan.error() == 0
        if schedule is None:                                    # padding included, so at least the chunks
            assert plan.last_resident_slots() >= resident_chunks
        else:
            assert plan.last_resident_slots() == 0
        results.append((state, plan.norms()))
        plan.close()
    for la, lb in zip(results[1][0], results[2][0]):          # run to run: the same bits
        for a, b in zip(la, lb):
            assert torch.equal(a, b)
    assert torch.equal(results[1][1], results[2][1])
    for name, la, lb in zip("gpmv", results[0][0], results[1][0]):
        for i, (a, b) in enumerate(zip(la, lb)):
            scale = max(a.abs().max().item(), 1e-30)
            assert (a - b).abs().max().item() <= 2e-6 * scale, (name, i)
    torch.testing.assert_close(results[0][1], results[1][1], rtol=2e-6, atol=0)


def test_lans_resident_step_with_an_unaligned_tensor_runs_as_sweeps(pkg):
    """The resident kernel moves float4s: a step in which an array of one of its tensors is not 16-byte
    aligned goes through the sweeps instead, with the sweeps' bits."""
    capi = pkg.capi
    numels = [8192 * 4, 100, 8192]
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    out = []
    for schedule, offset in ((capi.LANS_SWEEPS, 1), (capi.LANS_RESIDENT, 1), (capi.LANS_RESIDENT, 0)):
        state = _fresh_state(numels, 9, offset)
        plan = pkg.ops.LansPlan(numels, schedule=schedule)
        plan.step(*state, 1, hyper)
        plan.step(*state, 2, hyper)
        torch.cuda.synchronize()
        assert plan.error() == 0
        out.append((state, plan.last_resident_slots()))
        plan.close()
    assert out[0][1] == 0 and out[1][1] == 0 and out[2][1] >= 5
    for la, lb in zip(out[0][0], out[1][0]):
        for a, b in zip(la, lb):
            assert torch.equal(a, b)


def test_lans_resident_give_up_is_fail_safe_and_sticky(pkg):
    """With publication switched off (test hook) every wait of the resident kernel runs into its bound: the
    kernel must still end, write no parameter, flag the plan; the next step must be refused until the error
    has been read; after that the plan works again."""
    capi = pkg.capi
    numels = [1 << 20, 8192 * 3, 8192]
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    state = _fresh_state(numels, 13)
    before = [[t.clone() for t in lst] for lst in state]
    plan = pkg.ops.LansPlan(numels)
    plan.debug(spin_limit=8, flags=1)
    plan.step(*state, 1, hyper)
    torch.cuda.synchronize()
    # nothing was published, so no workgroup learned ||g||: stage M never ran, and nothing at all was written
    for la, lb in zip(state, before):
        for a, b in zip(la, lb):
            assert torch.equal(a, b)
    with pytest.raises(capi.LancetError) as info:          # refused on the host, nothing launched
        plan.step(*state, 2, hyper)
    assert info.value.status == capi.ERR_STALLED
    assert plan.error() == 1                                # read ...
    assert plan.error() == 0                                # ... and cleared
    plan.debug(spin_limit=0, flags=0)
    plan.step(*state, 1, hyper)
    torch.cuda.synchronize()
    assert plan.error() == 0
    ref = [[t.clone() for t in lst] for lst in before]
    other = pkg.ops.LansPlan(numels)
    other.step(*ref, 1, hyper)
    torch.cuda.synchronize()
    for la, lb in zip(state, ref):
        for a, b in zip(la, lb):
            assert torch.equal(a, b)
    plan.close()
    other.close()


@pytest.mark.parametrize("with_grad_norms", [False, True])
def test_lans_steps_queued_behind_a_stalled_step_touch_nothing(pkg, with_grad_norms):
    """A training loop that never synchronises has steps 2 and 3 queued before the host can see that step 1 stalled
    (and a replayed graph never asks the host): such steps must see the error on the device and leave every array
    alone, in both schedules, until the error has been read.  With the caller's gradient norms stage M of step 1
    runs (moments written) and only its parameters stay unwritten: the half-applied state a later step must not
    build on.  The host-side refusal is switched off here (debug flag 2) so that the steps really are launched."""
    capi = pkg.capi
    numels = [1 << 20, 8192 * 3, 8192, 1000]             # the last one goes through the sweeps of the same step
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    state = _fresh_state(numels, 17)
    before = [[t.clone() for t in lst] for lst in state]
    norms = torch.stack([torch.linalg.vector_norm(g.double()).float() for g in state[0]]) if with_grad_norms else None
    plan = pkg.ops.LansPlan(numels)
    plan.debug(spin_limit=8, flags=1 | 2)                 # nothing is published: every wait gives up
    plan.step(*state, 1, hyper, grad_norms=norms)
    torch.cuda.synchronize()
    after1 = [[t.clone() for t in lst] for lst in state]
    for i in range(3):                                    # the resident kernel's tensors: no parameter was written
        assert torch.equal(state[1][i], before[1][i])
        assert torch.equal(state[2][i], before[2][i]) != with_grad_norms     # moments: written only when ||g|| was known
    assert not torch.equal(state[1][3], before[1][3])     # the sweeps' tensor of step 1 is independent of the stall
    plan.debug(spin_limit=0, flags=2)                     # a healthy device from here on; the host still does not look
    plan.step(*state, 2, hyper, grad_norms=norms)
    plan.step(*state, 3, hyper, grad_norms=norms)
    plan.set_schedule(capi.LANS_SWEEPS)
    plan.step(*state, 4, hyper, grad_norms=norms)
    torch.cuda.synchronize()
    for la, lb in zip(state, after1):
        for a, b in zip(la, lb):
            assert torch.equal(a, b)                      # steps 2 to 4 were skipped as a whole
    plan.set_schedule(capi.LANS_RESIDENT)
    plan.debug(spin_limit=0, flags=0)
    with pytest.raises(capi.LancetError):                 # the host-side refusal is back
        plan.step(*state, 2, hyper, grad_norms=norms)
    assert plan.error() == 1 and plan.error() == 0
    plan.step(*state, 2, hyper, grad_norms=norms)         # and the plan works again
    torch.cuda.synchronize()
    assert plan.error() == 0
    for i in range(4):
        assert not torch.equal(state[1][i], after1[1][i])
    plan.close()


def _rounder(name):
    from oracle import moe_oracle as mo
    return {"f32": (lambda a: a), "bf16": mo.round_to_bf16, "f16": mo.round_to_f16}[name]


_TORCH = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


@pytest.mark.parametrize("schedule", ["sweeps", "resident"])
@pytest.mark.parametrize("gdt,pdt", [("bf16", "bf16"), ("f16", "f16"), ("f32", "bf16"), ("bf16", None), ("f16", "bf16")])
def test_lans_mixed_precision_step(pkg, schedule, gdt, pdt):
    """The step of a 16-bit model: gradients in bf16 / fp16, fp32 master parameters and moments, and the model's
    16-bit copy of every new parameter written by the same step, against the oracle's restatement of what the
    reference's optimizer does around its op (cast the gradients up, lans, cast the parameters down,
    python/raf/optim/lans.py:256-257, 285-288).  Master parameters within 1e-6 after 10 steps as for the fp32 step;
    the 16-bit copies bit-equal to the rounded master.  Shapes: the reference's own test lists
    (tests/python/optim/test_lans.py:94-161) and tensors the resident kernel takes."""
    capi = pkg.capi
    for seed, shapes in enumerate([[(2, 2)], [(6, 3, 5, 5), (6,), (6,), (10, 84), (10,)],
                                   [(3 * 8192,), (300, 70), (2, 8192), (8192 + 5,), (8192,)]]):
        rng, p, m, v = make_state(20 + seed, shapes)
        dp, dm, dv = [dev(a) for a in p], [dev(a) for a in m], [dev(a) for a in v]
        dlow = [torch.full(s, 7.0, dtype=_TORCH[pdt], device="cuda") for s in shapes] if pdt else None
        plan = pkg.ops.LansPlan([a.size for a in p], schedule=capi.LANS_SWEEPS if schedule == "sweeps" else None)
        hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
        for step in range(1, 11):
            g = [_rounder(gdt)(rng.normal(0, 1e-3, s).astype(np.float32)).astype(np.float32) for s in shapes]
            dg = [dev(a).to(_TORCH[gdt]) for a in g]
            for a, b in zip(dg, g):
                np.testing.assert_array_equal(to_np(a), b)            # the device holds exactly the oracle's gradients
            low = lo.lans_step_mixed(g, p, m, v, step, _rounder(pdt) if pdt else None)
            plan.step(dg, dp, dm, dv, step, hyper, p_lowp=dlow)
            if dlow is not None:
                for a, b in zip(dlow, dp):                            # bit-equal to the rounded master, every step
                    assert torch.equal(a, b.to(_TORCH[pdt]))
        assert plan.error() == 0
        if schedule == "resident" and seed == 2:
            assert plan.last_resident_slots() >= 6
        for i in range(len(shapes)):
            assert_close_scaled(to_np(dp[i]), p[i], P_RTOL, "p[%d]" % i)
            assert_close_scaled(to_np(dm[i]), m[i], 1e-5, "m[%d]" % i)
            assert_close_scaled(to_np(dv[i]), v[i], 1e-5, "v[%d]" % i)
            if pdt:                                                    # and against the oracle's casts: one ulp of the type
                from tests.gpu_util import ulp_distance
                assert ulp_distance(dlow[i], torch.from_numpy(low[i]).to(_TORCH[pdt]).cuda()) <= 1
        plan.close()


def test_lans_mixed_precision_rejects_and_aligns(pkg):
    """p, m, v stay float32; 16-bit arrays of a resident tensor that are not 8-byte aligned send the step through
    the sweeps (element path), with the same result."""
    capi = pkg.capi
    numels = [8192 * 2, 100]
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    out = []
    for offset in (0, 1):
        g, p, m, v = _fresh_state(numels, 23, 0)
        store = [torch.zeros(n + offset, dtype=torch.bfloat16, device="cuda") for n in numels]
        g16 = [s[offset:] for s in store]
        for a, b in zip(g16, g):
            a.copy_(b)
        low_store = [torch.zeros(n + offset, dtype=torch.bfloat16, device="cuda") for n in numels]
        low = [s[offset:] for s in low_store]
        plan = pkg.ops.LansPlan(numels)
        plan.step(g16, p, m, v, 1, hyper, p_lowp=low)
        plan.step(g16, p, m, v, 2, hyper, p_lowp=low)
        torch.cuda.synchronize()
        assert plan.error() == 0
        assert (plan.last_resident_slots() > 0) == (offset == 0)
        out.append((p, low))
        for a, b in zip(low, p):
            assert torch.equal(a, b.to(torch.bfloat16))
        with pytest.raises(ValueError):
            plan.step(g16, [x.to(torch.bfloat16) for x in p], m, v, 3, hyper)
        plan.close()
    for a, b in zip(out[0][0], out[1][0]):
        scale = float(a.abs().max())
        assert float((a - b).abs().max()) <= 2e-6 * scale


def test_lans_resident_schedule_against_oracle(pkg):
    capi = pkg.capi
    rng = np.random.default_rng(5)
    shapes = [(300, 100), (8192,), (17,), (4, 8192), (8192 * 2 + 3,)]
    g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    dg, dp, dm, dv = ([dev(a) for a in lst] for lst in (g, p, m, v))
    plan = pkg.ops.LansPlan([a.size for a in g], schedule=capi.LANS_RESIDENT)
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    for step in range(1, 11):
        lo.lans_step(g, p, m, v, step)
        plan.step(dg, dp, dm, dv, step, hyper)
    assert plan.error() == 0
    assert plan.last_resident_slots() >= 5                  # the (8192,) and (4, 8192) tensors
    for i in range(len(shapes)):
        assert_close_scaled(to_np(dp[i]), p[i], P_RTOL, "p[%d]" % i)
        assert_close_scaled(to_np(dm[i]), m[i], P_RTOL, "m[%d]" % i)
        assert_close_scaled(to_np(dv[i]), v[i], P_RTOL, "v[%d]" % i)
    plan.close()


def test_lans_resident_schedule_with_tensors_that_do_not_fit(pkg):
    """Tensors with more chunks than the kernel takes go through the sweeps inside the same step; the
    caller sees one step, norms in the order of its lists, and the same values as the pure sweeps schedule."""
    capi = pkg.capi
    probe = pkg.ops.LansPlan([1024, 1024])
    limit, largest = probe.resident_capacity()
    probe.close()
    assert largest == 1 and limit >= 256
    big = (limit + 1) * 8192
    numels = [1024, big, 65536, big + 3 * 8192 + 5, 8192]
    results = []
    for schedule in (capi.LANS_SWEEPS, capi.LANS_RESIDENT):
        state = _fresh_state(numels, 11)
        plan = pkg.ops.LansPlan(numels, schedule=schedule)
        assert plan.resident_capacity() == (limit, limit + 5)
        hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
        for step in (1, 2):
            plan.step(*state, step, hyper)
        torch.cuda.synchronize()
        assert plan.error() == 0
        assert plan.last_resident_slots() == (9 if schedule == capi.LANS_RESIDENT else 0)
        results.append((state, plan.norms()))
        plan.close()
    for name, la, lb in zip("gpmv", results[0][0], results[1][0]):
        for i, (a, b) in enumerate(zip(la, lb)):
            assert (a - b).abs().max().item() <= 2e-6 * max(a.abs().max().item(), 1e-30), (name, i)
    torch.testing.assert_close(results[0][1], results[1][1], rtol=2e-6, atol=0)
    # the two large tensors took the same kernels under both schedules: the same bits
    for i in (1, 3):
        assert torch.equal(results[0][0][1][i], results[1][0][1][i])
    # a plan made only of tensors that do not fit has no use for the resident kernel and starts with the sweeps
    only_big = pkg.ops.LansPlan([big])                       # no memory is touched by creating a plan
    with pytest.raises(RuntimeError):
        only_big.set_schedule(capi.LANS_RESIDENT)
    only_big.close()


def test_lans_resident_schedule_beside_other_work(pkg):
    """The resident kernel's workgroups wait for one another, so they must all get onto the chip: with
    another stream keeping compute units busy they get there as that work retires, the waits stay within
    their bound (error word 0) and the result is the one an idle GPU gives."""
    capi = pkg.capi
    numels = [4 << 20, 1 << 20, 4 << 20, 1024, 3 << 20]
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)

    def state():
        gen = torch.Generator(device="cuda").manual_seed(3)
        total = sum(numels)
        flat = [torch.empty(total, device="cuda").normal_(0, s, generator=gen) for s in (1e-3, 0.02)]
        flat += [torch.zeros(total, device="cuda") for _ in range(2)]
        return flat, [list(torch.split(t, numels)) for t in flat]

    flat_a, views_a = state()
    plan = pkg.ops.LansPlan(numels, schedule=capi.LANS_RESIDENT)
    for step in (1, 2, 3):
        plan.step(*views_a, step, hyper)
    torch.cuda.synchronize()
    assert plan.error() == 0
    assert plan.last_resident_slots() >= (12 << 20) // 8192

    flat_b, views_b = state()
    side = torch.cuda.Stream()
    x = torch.randn(64 << 20, device="cuda")
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    for step in (1, 2, 3):
        with torch.cuda.stream(side):
            for _ in range(6):                      # streaming work that occupies every compute unit
                torch.mul(x, 1.0001, out=y)
                torch.add(y, 1.0, out=x)
        plan.step(*views_b, step, hyper)
    torch.cuda.synchronize()
    assert plan.error() == 0
    for a, b in zip(flat_a, flat_b):
        assert torch.equal(a, b)
    plan.close()


def test_stepper_trains_a_small_model_like_the_reference_optimizer(pkg):
    """LansStepper is the counterpart of raf.optim.lans.LANS (python/raf/optim/lans.py:44-103): it owns m, v and the
    step counter, takes the parameters' .grad, and leaves out parameters without a gradient.  Five training
    steps of a two-layer model against the oracle fed with the same gradients."""
    torch.manual_seed(0)
    w1 = (torch.randn(64, 32, device="cuda") * 0.1).requires_grad_(True)
    b1 = torch.zeros(32, device="cuda", requires_grad=True)
    w2 = (torch.randn(32, 8, device="cuda") * 0.1).requires_grad_(True)
    unused = torch.ones(5, device="cuda", requires_grad=True)          # never reached by the loss: .grad stays None
    params = [w1, b1, w2, unused]
    opt = pkg.ops.LansStepper(params, lr=2e-3, weight_decay=0.05)
    ref_p = [to_np(p.detach()) for p in params[:3]]
    ref_m = [np.zeros_like(a) for a in ref_p]
    ref_v = [np.zeros_like(a) for a in ref_p]
    x = torch.randn(128, 64, device="cuda")
    y = torch.randn(128, 8, device="cuda")
    losses = []
    for step in range(1, 6):
        for p in params:
            p.grad = None
        loss = ((torch.tanh(x @ w1 + b1) @ w2 - y) ** 2).mean()
        loss.backward()
        losses.append(float(loss.detach()))
        lo.lans_step([to_np(p.grad) for p in params[:3]], ref_p, ref_m, ref_v, step, lr=2e-3, weight_decay=0.05)
        opt.step()
    assert losses[-1] < losses[0]
    for p, want in zip(params[:3], ref_p):
        assert_close_scaled(to_np(p.detach()), want, 5e-6, "parameter")   # gradients feed back: errors compound
    np.testing.assert_array_equal(to_np(unused.detach()), np.ones(5, np.float32))
    with pytest.raises(ValueError):
        opt.step([None])


def test_stepper_keeps_master_weights_for_a_16_bit_model(pkg):
    """Parameters in bfloat16: the stepper keeps float32 master copies, feeds the 16-bit gradients as they are and
    lets the step write the model's parameters (python/raf/optim/lans.py:256-257, 285-288 does it with casts around
    the op).  Against the oracle's mixed step fed with the same gradients."""
    from oracle import moe_oracle as mo
    torch.manual_seed(1)
    w1 = (torch.randn(64, 32, device="cuda") * 0.1).to(torch.bfloat16).requires_grad_(True)
    w2 = (torch.randn(32, 8, device="cuda") * 0.1).to(torch.bfloat16).requires_grad_(True)
    params = [w1, w2]
    opt = pkg.ops.LansStepper(params, lr=2e-3, weight_decay=0.05)
    assert opt.mixed and opt.master[0].dtype == torch.float32
    ref_p = [to_np(p.detach()) for p in params]
    ref_m = [np.zeros_like(a) for a in ref_p]
    ref_v = [np.zeros_like(a) for a in ref_p]
    x = torch.randn(128, 64, device="cuda").to(torch.bfloat16)
    y = torch.randn(128, 8, device="cuda")
    for step in range(1, 5):
        for p in params:
            p.grad = None
        loss = ((torch.tanh(x @ w1) @ w2).float() - y).pow(2).mean()
        loss.backward()
        assert w1.grad.dtype == torch.bfloat16
        low = lo.lans_step_mixed([to_np(p.grad) for p in params], ref_p, ref_m, ref_v, step, mo.round_to_bf16, lr=2e-3, weight_decay=0.05)
        opt.step()
        for p, master, want in zip(params, opt.master, low):
            assert torch.equal(p.detach(), master.to(torch.bfloat16))
        # the model's parameters feed the next gradients: keep the oracle on the device's values
        for a, master in zip(ref_p, opt.master):
            assert_close_scaled(to_np(master), a, 2e-6, "master parameter")
            a[...] = to_np(master)

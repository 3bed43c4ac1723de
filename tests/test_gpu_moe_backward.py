"""GPU parity tests of the MoE backward ops (moe_encode_dx/dg, moe_decode_dx/dg) against the NumPy
oracle (itself pinned against torch autograd in tests/test_oracle_moe.py).

Bar: encode_dx, encode_dg and fp32 decode_dx are copies or single fp32 products -> bit-exact;
16-bit decode_dx within 1 ulp; decode_dg is a length-M dot product summed in a different order than
the oracle's fp64 sum -> 1e-5 of sum|a_i*b_i|."""
import copy

import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, rows_as_oracle, rows_to_torch, to_np

pytestmark = pytest.mark.gpu


def routed(S, M, E, k, dt, seed):
    data, logits = make_inputs(seed, S, M, E, zipf_bias=True)
    rows = rows_as_oracle(data, dt)
    used0 = np.zeros(E, np.int32)
    if k == 1:
        return rows, mo.moe_encode(rows, mo.softmax_rows(logits), used0, 0.7, fast_scatter=True)
    return rows, mo.moe_encode_top2(rows, logits, used0, 0.7, gate_is_logits=True, fast_scatter=True)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("S,M,E", [(1024, 128, 32), (777, 40, 6), (300, 5, 4)])
def test_backward_ops(pkg, dt, k, S, M, E):
    ops = pkg.ops
    rows, (g, il, used, elems, disp) = routed(S, M, E, k, dt, S + 3 * k)
    C = disp.shape[1]
    rng = np.random.default_rng(S)
    dy_buf = rows_as_oracle(rng.standard_normal(disp.shape, dtype=np.float32), dt)
    dy_tok = rows_as_oracle(rng.standard_normal((S, M), dtype=np.float32), dt)
    dy_gate = rng.standard_normal(k * S, dtype=np.float32)
    d_il, d_g = dev(il), dev(g)
    assert (il[0] < 0).any()
    # encode_dx: gather (k = 2: fp32 sum of two rows, rounded once)
    got = ops.moe_encode_dx(rows_to_torch(dy_buf, dt), d_il, top_k=k)
    want = mo.moe_encode_dx(dy_buf, il, k)
    if dt == "f32" or k == 1:
        np.testing.assert_array_equal(to_np(got), rows_as_oracle(want, dt))
    else:
        tdt = torch.bfloat16 if dt == "bf16" else torch.float16
        diff = (got.cpu().view(torch.int16).int() - torch.from_numpy(want).to(tdt).view(torch.int16).int()).abs().max()
        assert int(diff) <= 1
    # encode_dg
    got = ops.moe_encode_dg(dev(dy_gate), d_il, E, top_k=k)
    np.testing.assert_array_equal(to_np(got), mo.moe_encode_dg(dy_gate, il, E, k))
    # decode_dx
    got = ops.moe_decode_dx(rows_to_torch(dy_tok, dt), d_g, d_il, E, C, top_k=k)
    want = mo.moe_decode_dx(dy_tok, g, il, E, C, k)
    if dt == "f32":
        np.testing.assert_array_equal(to_np(got), want)
    else:
        tdt = torch.bfloat16 if dt == "bf16" else torch.float16
        diff = (got.cpu().view(torch.int16).int() - torch.from_numpy(want).to(tdt).view(torch.int16).int()).abs().max()
        assert int(diff) <= 1
    # decode_dg
    got = to_np(ops.moe_decode_dg(rows_to_torch(dy_tok, dt), rows_to_torch(disp, dt), d_il, top_k=k))
    want = mo.moe_decode_dg(dy_tok, disp, il, k)
    ok = (il[0] >= 0)
    tok = np.tile(np.arange(S), k)
    scale = np.zeros(k * S)
    scale[ok] = np.abs(disp[il[0][ok], il[1][ok]].astype(np.float64) * dy_tok[tok[ok]]).sum(axis=1)
    assert (np.abs(got.astype(np.float64) - want) <= 1e-5 * scale + 1e-30).all()
    assert not got[~ok].any()


def _gate_rounder(gdt):
    return {"f32": lambda a: a, "bf16": mo.round_to_bf16, "f16": mo.round_to_f16}[gdt]


def _check_gate_gradient(pkg, logits, il, k, is_logits, gdt, seed):
    """lancet_moe_encode_dgate against the oracle (fp64 on the same, rounded, inputs).  fp32 gates: 1e-5 relative,
    plus 1e-6 of the row's largest slot gradient for the entries where the selected term and the row's mean cancel.
    16-bit gates: one unit in the last place of the type, or that same absolute floor."""
    ops = pkg.ops
    S, E = logits.shape
    rnd = _gate_rounder(gdt)
    gate_in = rnd(logits if is_logits else mo.softmax_rows(logits)).astype(np.float32)
    dy = rnd(np.random.default_rng(seed).standard_normal(k * S).astype(np.float32)).astype(np.float32)
    want = mo.moe_encode_dgate(dy, gate_in, il, k, is_logits)
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[gdt]
    got = ops.moe_encode_dgate(dev(dy).to(tdt), dev(gate_in).to(tdt), dev(il), top_k=k, gate_is_logits=is_logits)
    assert got.dtype == tdt and got.shape == (S, E)
    scale = np.abs(want).max(axis=1, keepdims=True)          # the selected entries carry the row's largest values
    if gdt == "f32":
        err = np.abs(to_np(got).astype(np.float64) - want)
        assert (err <= 1e-5 * np.abs(want) + 1e-6 * scale + 1e-30).all(), float((err / (np.abs(want) + 1e-30)).max())
    else:
        w16 = torch.from_numpy(want).to(tdt)
        a, b = got.cpu().view(torch.int16).to(torch.int32), w16.view(torch.int16).to(torch.int32)
        a, b = torch.where(a < 0, -(a & 0x7fff), a), torch.where(b < 0, -(b & 0x7fff), b)
        close = torch.from_numpy(np.abs(to_np(got).astype(np.float64) - want) <= 1e-6 * scale)
        assert bool((((a - b).abs() <= 1) | close).all())
    dead = np.stack([il[0, j * S:(j + 1) * S] < 0 for j in range(k)]).all(axis=0)
    assert not to_np(got)[dead].any()                         # a token with no kept slot gets no gradient
    return got


@pytest.mark.parametrize("gdt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("is_logits", [False, True])
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("S,E", [(1024, 32), (777, 6), (300, 5), (2048, 512)])
def test_gate_gradient_of_the_whole_op(pkg, gdt, is_logits, k, S, E):
    """E = 5 (rows that are no whole 16-byte granules) takes the element path, the others the 16-byte one."""
    data, logits = make_inputs(S + E, S, 1, E, zipf_bias=True)
    rnd = _gate_rounder(gdt)
    gate_in = rnd(logits if is_logits else mo.softmax_rows(logits)).astype(np.float32)
    used0 = np.zeros(E, np.int32)
    if k == 1:
        il = mo.moe_encode(data, gate_in, used0, 0.7, gate_is_logits=is_logits, fast_scatter=True)[1]
    else:
        il = mo.moe_encode_top2(data, gate_in, used0, 0.7, gate_is_logits=is_logits, fast_scatter=True)[1]
    assert (il[0] < 0).any() and (il[0] >= 0).any()
    got = _check_gate_gradient(pkg, logits, il, k, is_logits, gdt, S)
    if k == 1 and not is_logits:     # the reference's own rule (moe_encode_dg) is this case
        dy = dev(rnd(np.random.default_rng(S).standard_normal(S).astype(np.float32)).astype(np.float32)).to(got.dtype)
        assert torch.equal(got, pkg.ops.moe_encode_dg(dy, dev(il), E))


@pytest.mark.parametrize("shape", ["config2", "config4_pressure"])
def test_gate_gradient_at_the_baseline_shapes(pkg, shape):
    """Config 2 (S=16384, E=16, Zipf bias: more than 1000 dropped slots) and config 4's shape with four favoured
    experts (S=65536, E=32, C=5120: slots overflow), top-2 on logits, fp32 gate; routing taken from the HIP op."""
    if shape == "config2":
        S, E, cf = 16384, 16, 1.0
        _, logits = make_inputs(0, S, 1, E, zipf_bias=True)
    else:
        S, E, cf = 65536, 32, 1.25
        rng = np.random.default_rng(0)
        logits = rng.standard_normal((S, E), dtype=np.float32)
        logits[:, :4] += np.float32(0.75)
    _, il, _, _ = pkg.ops.moe_route(dev(logits), None, 8, cf, top_k=2, gate_is_logits=True)
    il = to_np(il)
    assert (il[0] < 0).sum() > (1000 if shape == "config2" else 0)
    _check_gate_gradient(pkg, logits, il, 2, True, "f32", 11)


def test_gate_gradient_below_the_clamp_and_for_large_logits(pkg):
    """Rows whose two kept values add up to less than eps (the clamped denominator is a constant), and logits of
    scale 30, where a row's probabilities span 60 orders of magnitude."""
    S, E = 512, 8
    rng = np.random.default_rng(4)
    gate = (rng.random((S, E), dtype=np.float32) * np.linspace(1e-8, 3e-7, S, dtype=np.float32)[:, None]).astype(np.float32)
    _, il, *_ = mo.moe_encode_top2(np.zeros((S, 1), np.float32), gate, np.zeros(E, np.int32), 1.0, fast_scatter=True)
    sel, val = mo.select_topk(gate, 2)
    tot = val[0].astype(np.float64) + val[1]
    assert (tot < 1.19e-7).sum() > 10 and (tot > 1.2e-7).sum() > 10
    dy = rng.standard_normal(2 * S).astype(np.float32)
    got = to_np(pkg.ops.moe_encode_dgate(dev(dy), dev(gate), dev(il), top_k=2))
    want = mo.moe_encode_dgate(dy, gate, il, 2, False)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)
    _, logits = make_inputs(3, 1024, 1, 32, logit_scale=30.0)
    il = mo.moe_encode_top2(np.zeros((1024, 1), np.float32), logits, np.zeros(32, np.int32), 0.8, gate_is_logits=True,
                            fast_scatter=True)[1]
    _check_gate_gradient(pkg, logits, il, 2, True, "f32", 5)


@pytest.mark.parametrize("scale", [4.0, 12.0, 30.0])
def test_gate_gradient_of_peaked_rows_keeps_its_relative_accuracy(pkg, scale):
    """Top-1 on logits whose rows are peaked (the selected probability within 1e-3 ... 1e-30 of 1): the gradient
    of the selected logit is dy p (1 - p).  The kernel forms 1 - p from the sum of the other exponentials, not as
    a difference, so EVERY entry stays within 2e-5 relative of the oracle, with no floor tied to the row (a plain
    fp32 softmax backward is off by 6e-8 / (1 - p) there); 1e-37 covers results that underflow."""
    S, E = 2048, 32
    _, logits = make_inputs(int(scale), S, 1, E, logit_scale=scale)
    il = mo.moe_encode(np.zeros((S, 1), np.float32), logits, np.zeros(E, np.int32), 0.9, gate_is_logits=True, fast_scatter=True)[1]
    p_top = mo.softmax_rows(logits).max(axis=1)
    assert (p_top > 1 - 1e-4).sum() >= (50 if scale > 4 else 0)
    dy = np.random.default_rng(9).standard_normal(S).astype(np.float32)
    got = to_np(pkg.ops.moe_encode_dgate(dev(dy), dev(logits), dev(il), top_k=1, gate_is_logits=True))
    want = mo.moe_encode_dgate(dy, logits, il, 1, True)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-37)
    # two experts: the closed form dy exp(-t) / (1 + exp(-t))^2 for the selected logit, its negative for the other
    t = np.linspace(0.25, 80.0, 320).astype(np.float32)
    two = np.stack([np.zeros_like(t), t], axis=1)
    il2 = np.array([[1] * t.size, list(range(t.size))], np.int32)
    dy2 = np.random.default_rng(10).standard_normal(t.size).astype(np.float32)
    got = to_np(pkg.ops.moe_encode_dgate(dev(dy2), dev(two), dev(il2), top_k=1, gate_is_logits=True))
    z = np.exp(-t.astype(np.float64))
    sel = dy2 * z / (1 + z) ** 2
    np.testing.assert_allclose(got[:, 1], sel, rtol=2e-5, atol=1e-37)
    np.testing.assert_allclose(got[:, 0], -sel, rtol=2e-5, atol=1e-37)


def test_backward_matches_autograd_through_forward_ops(pkg):
    """End to end: gradients of sum(decode(expert(encode(x))) * Y) with an elementwise expert, taken
    with the backward ops, against torch autograd of the same computation written with torch indexing."""
    ops = pkg.ops
    S, M, E = 512, 64, 8
    data, logits = make_inputs(5, S, M, E)
    x = dev(data)
    gate = dev(mo.softmax_rows(logits))
    g, il, used, elems, disp = ops.moe_encode(x, gate, None, 0.8)
    C = disp.shape[1]
    y = ops.moe_decode(disp * 2.0, g, il)
    Y = torch.randn_like(y)
    # backward with the ops
    d_expert_out = ops.moe_decode_dx(Y, g, il, E, C)
    d_gates_s = ops.moe_decode_dg(Y, disp * 2.0, il)
    d_x = ops.moe_encode_dx(d_expert_out * 2.0, il)
    d_gate = ops.moe_encode_dg(d_gates_s, il, E)
    # autograd reference
    xr = x.clone().double().requires_grad_(True)
    gr = gate.clone().double().requires_grad_(True)
    idx, loc = il[0].long(), il[1].long()
    kept = idx >= 0
    gs = gr[torch.arange(S, device="cuda"), idx.clamp_min(0)]
    yr = torch.zeros((S, M), dtype=torch.float64, device="cuda")
    yr[kept] = xr[kept] * 2.0 * gs[kept, None]
    (yr * Y.double()).sum().backward()
    torch.testing.assert_close(d_x.double(), xr.grad, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(d_gate.double(), gr.grad, rtol=1e-5, atol=1e-5)


def _dense_layer(x, logits, W, il, C):
    """The MoE layer in DeepSpeed's einsum form (docker/resources/sharded_moe.py:315-322 and the
    'sec,sm->ecm' / 'sec,ecm->sm' products of MOELayer.forward), fp64, with the routing decisions
    (expert, location of every kept token) taken as constants."""
    S, E = logits.shape
    gate = torch.softmax(logits, dim=1)
    idx, loc = il[0].long(), il[1].long()
    kept = idx >= 0
    mask = torch.zeros((S, E, C), dtype=torch.float64, device=x.device)
    mask[torch.arange(S, device=x.device)[kept], idx[kept], loc[kept]] = 1.0
    gates_s = (gate * mask.sum(2)).sum(1)
    disp = torch.einsum("sec,sm->ecm", mask, x)
    expert_out = torch.tanh(torch.bmm(disp, W))
    return torch.einsum("sec,ecm->sm", mask * gates_s[:, None, None], expert_out)


@pytest.mark.parametrize("bpr", [False, True])
def test_autograd_wiring_of_a_whole_layer(pkg, bpr):
    """softmax -> moe_encode -> per-expert matmul + tanh -> moe_decode, differentiated by torch.autograd through
    the gradient rules of src/op/grad/moe.cc, against the dense einsum form of the same layer in fp64."""
    grad = pkg.grad
    S, M, E = 384, 32, 6
    data, logits_np = make_inputs(21, S, M, E, zipf_bias=True)
    rng = np.random.default_rng(3)
    W0 = dev((rng.standard_normal((E, M, M)) / np.sqrt(M)).astype(np.float32))
    Y = dev(rng.standard_normal((S, M)).astype(np.float32))
    x = dev(data).requires_grad_(True)
    logits = dev(logits_np).requires_grad_(True)
    W = W0.clone().requires_grad_(True)
    gate = torch.softmax(logits, dim=1)
    if bpr:
        gates_s, il, used, elems, disp = grad.moe_encode_batch_prioritized(x, gate, 1, 0, 0.75)
    else:
        gates_s, il, used, elems, disp = grad.moe_encode(x, gate, None, 0.75)
    assert not il.requires_grad and disp.requires_grad and gates_s.requires_grad
    assert bool((il[0] < 0).any())                                   # some tokens are dropped
    out = grad.moe_decode(torch.tanh(torch.bmm(disp, W)), gates_s, il)
    (out * Y).sum().backward()

    xr = x.detach().double().requires_grad_(True)
    lr = logits.detach().double().requires_grad_(True)
    Wr = W0.double().requires_grad_(True)
    ref = _dense_layer(xr, lr, Wr, il, disp.shape[1])
    torch.testing.assert_close(out.detach().double(), ref.detach(), rtol=1e-5, atol=1e-5)
    (ref * Y.double()).sum().backward()
    torch.testing.assert_close(x.grad.double(), xr.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(logits.grad.double(), lr.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(W.grad.double(), Wr.grad, rtol=1e-4, atol=1e-5)


def test_autograd_wiring_of_a_prioritized_partition(pkg):
    """moe_encode_batch_prioritized sees the whole batch and encodes one partition: the tokens of the other
    partitions get zero gradient, the partition's own tokens the gradient of the plain rule."""
    grad, ops = pkg.grad, pkg.ops
    S0, M, E, P, pid = 512, 16, 4, 4, 2
    data, logits_np = make_inputs(8, S0, M, E)
    x = dev(data).requires_grad_(True)
    gate = dev(mo.softmax_rows(logits_np)).requires_grad_(True)
    gates_s, il, used, elems, disp = grad.moe_encode_batch_prioritized(x, gate, P, pid, 0.5)
    wd, wg = torch.randn_like(disp), torch.randn_like(gates_s)
    ((disp * wd).sum() + (gates_s * wg).sum()).backward()
    S = S0 // P
    own = slice(pid * S, (pid + 1) * S)
    assert torch.equal(x.grad[own], ops.moe_encode_dx(wd, il))
    assert torch.equal(gate.grad[own], ops.moe_encode_dg(wg, il, E))
    rest = torch.ones(S0, dtype=torch.bool, device="cuda")
    rest[own] = False
    assert not bool(x.grad[rest].any()) and not bool(gate.grad[rest].any())


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("top_k,fused", [(1, False), (1, True), (2, False), (2, True)])
def test_moe_layer_module_against_a_dense_layer(pkg, dt, top_k, fused):
    """Gate / Experts / MOELayerImpl (the reference's layer, models/benchmark/pytorch/utils.py:529-634) on the HIP
    operators: output and all parameter gradients against the same layer written densely with one-hot masks in
    torch (the form of the reference's FakeMoeEncodeOp / FakeMoeDecodeOp, :349-370,454-462; for top_k = 2 the
    masks, clamp and normalisation of docker/resources/sharded_moe.py:296-322), in fp64.  fused: the gate module
    hands over logits and the operator runs the softmax."""
    ml = pkg.moe_layer
    torch.manual_seed(3)
    B, L, M, E, H = 4, 96, 32, 4, 48
    expert = torch.nn.Sequential(torch.nn.Linear(M, H), torch.nn.GELU(), torch.nn.Linear(H, M))
    layer = ml.MOELayerImpl(ml.Gate(M, E, softmax=not fused), ml.Experts(expert, 1, M, E), 1, E, capacity_factor=0.75 / top_k,
                            top_k=top_k, fused_softmax=fused).cuda()
    for i, e in enumerate(layer.experts.experts):            # the copies start equal: make the experts differ
        for p in e.parameters():
            p.data.add_(0.05 * (i + 1) * torch.randn_like(p))
    layer = layer.to(dt)
    x = torch.randn(B, L, M, device="cuda").to(dt).requires_grad_(True)
    Y = torch.randn(B, L, M, device="cuda")
    out = layer(x)
    assert out.shape == x.shape and out.dtype == dt
    (out.float() * Y).sum().backward()

    # dense fp64 layer with the same parameters and the same routing decisions
    ref = copy.deepcopy(layer).double()
    xr = x.detach().double().requires_grad_(True)
    flat = xr.reshape(-1, M)
    gate = torch.softmax(ref.gate.wg(flat), dim=1)
    S = flat.shape[0]
    C = pkg.ops.moe_capacity(S, E, 0.75)
    with torch.no_grad():
        _, il, _, _, _ = pkg.ops.moe_encode(x.detach().reshape(-1, M).contiguous(), layer.gate(x.detach().reshape(-1, M)), None,
                                            0.75 / top_k, top_k=top_k, gate_is_logits=fused)
    assert bool((il[0] < 0).any())
    masks, weights = [], []
    for j in range(top_k):
        idx, loc = il[0, j * S:(j + 1) * S].long(), il[1, j * S:(j + 1) * S].long()
        kept = idx >= 0
        mask = torch.zeros((S, E, C), dtype=torch.float64, device="cuda")
        mask[torch.arange(S, device="cuda")[kept], idx[kept], loc[kept]] = 1.0
        masks.append(mask)
        weights.append((gate * mask.sum(2)).sum(1))
    if top_k == 2:
        denom = torch.clamp(weights[0] + weights[1], min=torch.finfo(torch.float32).eps)
        weights = [w / denom for w in weights]
    disp = torch.einsum("sec,sm->ecm", sum(masks), flat)
    eo = torch.stack([ref.experts.experts[e](disp[e]) for e in range(E)])
    combine = sum(m * w[:, None, None] for m, w in zip(masks, weights))
    want = torch.einsum("sec,ecm->sm", combine, eo).reshape(B, L, M)
    (want * Y.double()).sum().backward()
    tol = dict(rtol=1e-4, atol=1e-5) if dt == torch.float32 else dict(rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(out.detach().double(), want.detach(), **tol)
    torch.testing.assert_close(x.grad.double(), xr.grad, **tol)
    for (n, a), (_, b) in zip(layer.named_parameters(), ref.named_parameters()):
        assert a.grad is not None, n
        scale = float(b.grad.abs().max())
        err = float((a.grad.double() - b.grad).abs().max())
        assert err <= (1e-4 if dt == torch.float32 else 5e-2) * max(scale, 1e-6), (n, err, scale)

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
def test_moe_layer_module_against_a_dense_layer(pkg, dt):
    """Gate / Experts / MOELayerImpl (the reference's layer, models/benchmark/pytorch/utils.py:529-634) on the HIP
    operators: output and all parameter gradients against the same layer written densely with one-hot masks in
    torch (the form of the reference's FakeMoeEncodeOp / FakeMoeDecodeOp, :349-370,454-462), in fp64."""
    ml = pkg.moe_layer
    torch.manual_seed(3)
    B, L, M, E, H = 4, 96, 32, 4, 48
    expert = torch.nn.Sequential(torch.nn.Linear(M, H), torch.nn.GELU(), torch.nn.Linear(H, M))
    layer = ml.MOELayerImpl(ml.Gate(M, E), ml.Experts(expert, 1, M, E), 1, E, capacity_factor=0.75).cuda()
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
        _, il, _, _, _ = pkg.ops.moe_encode(x.detach().reshape(-1, M).contiguous(), layer.gate(x.detach().reshape(-1, M)), None, 0.75)
    idx, loc = il[0].long(), il[1].long()
    kept = idx >= 0
    assert bool((~kept).any())
    mask = torch.zeros((S, E, C), dtype=torch.float64, device="cuda")
    mask[torch.arange(S, device="cuda")[kept], idx[kept], loc[kept]] = 1.0
    gates_s = (gate * mask.sum(2)).sum(1)
    disp = torch.einsum("sec,sm->ecm", mask, flat)
    eo = torch.stack([ref.experts.experts[e](disp[e]) for e in range(E)])
    want = torch.einsum("sec,ecm->sm", mask * gates_s[:, None, None], eo).reshape(B, L, M)
    (want * Y.double()).sum().backward()
    tol = dict(rtol=1e-4, atol=1e-5) if dt == torch.float32 else dict(rtol=5e-2, atol=5e-2)
    torch.testing.assert_close(out.detach().double(), want.detach(), **tol)
    torch.testing.assert_close(x.grad.double(), xr.grad, **tol)
    for (n, a), (_, b) in zip(layer.named_parameters(), ref.named_parameters()):
        assert a.grad is not None, n
        scale = float(b.grad.abs().max())
        err = float((a.grad.double() - b.grad).abs().max())
        assert err <= (1e-4 if dt == torch.float32 else 5e-2) * max(scale, 1e-6), (n, err, scale)

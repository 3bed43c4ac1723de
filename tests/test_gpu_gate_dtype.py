"""Gate arrays in the token dtype (the reference's kernels take `__dtype* gates1_s`,
src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:110-116,126-157, and mixed-precision graphs feed a half
gate, python/raf/amp/type_hints.py:97,105): every op that reads or writes gate values, with fp16 and bf16
gates, against the oracle run on the rounded gate.  Indices, locations, used capacity and rows bit-exact;
gate values: the fp32 result rounded once to the gate type (bit-exact where the op only selects, 1 unit in the
last place of the gate type after a softmax or a normalisation, whose fp32 value the oracle and the device
form with different exp implementations)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import TORCH_DT, dev, make_inputs, rows_as_oracle, to_np

pytestmark = pytest.mark.gpu

ROUND = {"bf16": mo.round_to_bf16, "f16": mo.round_to_f16}


def ulp_diff(got_t, want_f32, gd):
    """Largest distance, in units of the last place of the 16-bit type, between a GPU tensor of that type and
    the fp32 values rounded to it."""
    want_t = torch.from_numpy(np.ascontiguousarray(want_f32)).to(TORCH_DT[gd])
    a = got_t.cpu().view(torch.int16).to(torch.int32)
    b = want_t.view(torch.int16).to(torch.int32)
    # order-preserving image of the sign-magnitude patterns
    a = torch.where(a < 0, -(a & 0x7fff), a)
    b = torch.where(b < 0, -(b & 0x7fff), b)
    return int((a - b).abs().max()) if a.numel() else 0


@pytest.mark.parametrize("gd", ["bf16", "f16"])
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("logits", [False, True])
def test_encode_and_decode_with_a_half_gate(pkg, gd, k, logits):
    """16-bit gates tie massively (bf16 has 8 bits of mantissa): the first maximum must win in both slots."""
    ops = pkg.ops
    S, M, E, cf = 6000, 64, 16, 0.8
    data, raw = make_inputs(11 + k, S, M, E, zipf_bias=True)
    gate32 = raw if logits else mo.softmax_rows(raw)
    gate = ROUND[gd](gate32)                      # what the device holds
    if not logits:
        sel = mo.select_topk(gate, k)[0]
        top = np.sort(gate, axis=1)[:, -k:]
        assert (np.sum(gate >= top[:, :1], axis=1) > k).any(), "the rounded gate should hold ties among the leaders"
    used_in = np.arange(E, dtype=np.int32) % 3
    if k == 1:
        want = mo.moe_encode(data, gate, used_in, cf, gate_is_logits=logits, fast_scatter=True)
    else:
        want = mo.moe_encode_top2(data, gate, used_in, cf, gate_is_logits=logits, fast_scatter=True, gate_round=ROUND[gd])
    d_gate = dev(gate).to(TORCH_DT[gd])
    assert np.array_equal(to_np(d_gate), gate)
    got = ops.moe_encode(dev(data), d_gate, dev(used_in), cf, top_k=k, gate_is_logits=logits)
    assert got[0].dtype == TORCH_DT[gd]
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_array_equal(to_np(got[3]), want[3])
    np.testing.assert_array_equal(to_np(got[4]), want[4])
    exact = k == 1 and not logits                 # a selected value, stored as it came
    assert ulp_diff(got[0], want[0], gd) <= (0 if exact else 1)
    # decode with the device's own gates_s against the oracle on exactly those values
    expert_out = np.random.default_rng(3).standard_normal(want[4].shape, dtype=np.float32)
    out = ops.moe_decode(dev(expert_out), got[0], got[1], top_k=k)
    np.testing.assert_array_equal(to_np(out), mo.moe_decode(expert_out, to_np(got[0]), want[1], k=k))
    # routing alone and selection alone agree with the fused op
    r = ops.moe_route(d_gate, dev(used_in), M, cf, top_k=k, gate_is_logits=logits)
    assert torch.equal(r[0], got[0]) and torch.equal(r[1], got[1]) and torch.equal(r[2], got[2])


@pytest.mark.parametrize("gd", ["bf16", "f16"])
def test_gate_topk_and_noise_with_a_half_gate(pkg, gd):
    import ctypes as C
    lib, capi = pkg.capi.load(), pkg.capi
    S, E = 3000, 24                               # 24 halves = 48 bytes per row: rows are not all 16-byte aligned
    _, raw = make_inputs(5, S, 4, E)
    gate = ROUND[gd](mo.softmax_rows(raw))
    noise = ROUND[gd](np.random.default_rng(9).gumbel(size=(S, E)).astype(np.float32))
    code = {"bf16": capi.BF16, "f16": capi.F16}[gd]
    p = lambda t: C.c_void_p(t.data_ptr())
    d_gate, d_noise = dev(gate).to(TORCH_DT[gd]), dev(noise).to(TORCH_DT[gd])
    for nz in (None, d_noise):
        idx = torch.empty((2, S), dtype=torch.int32, device="cuda")
        val = torch.empty((2, S), dtype=TORCH_DT[gd], device="cuda")
        assert lib.lancet_gate_topk(p(d_gate), p(nz) if nz is not None else None, S, E, 2, code, 0, p(idx), p(val), None) == 0
        wi, wv = mo.select_topk(gate, 2, False, None if nz is None else noise)
        np.testing.assert_array_equal(to_np(idx), wi)
        np.testing.assert_array_equal(to_np(val), wv)


@pytest.mark.parametrize("gd", ["bf16", "f16"])
def test_batch_prioritized_with_a_half_gate(pkg, gd):
    """Priorities are the rounded gate values: many equal priorities, ties go to the lower token index."""
    ops = pkg.ops
    S0, M, E, P = 8192, 32, 8, 2
    data, raw = make_inputs(21, S0, M, E, logit_scale=2.0)
    gate = ROUND[gd](mo.softmax_rows(raw))
    for pid in range(P):
        want = mo.moe_encode_bpr(data, gate, P, pid, 0.6, fast_scatter=True)
        got = ops.moe_encode_batch_prioritized(dev(data), dev(gate).to(TORCH_DT[gd]), P, pid, 0.6)
        assert got[0].dtype == TORCH_DT[gd]
        for i in (1, 2, 3, 4):
            np.testing.assert_array_equal(to_np(got[i]), want[i])
        np.testing.assert_array_equal(to_np(got[0]), want[0])
    assert len(np.unique(gate.max(axis=1))) < S0 // 4, "rounded priorities should repeat"


@pytest.mark.parametrize("gd", ["bf16", "f16"])
@pytest.mark.parametrize("k", [1, 2])
def test_backward_ops_with_half_gates(pkg, gd, k):
    ops = pkg.ops
    S, M, E, cf = 2048, 64, 8, 0.7
    data, raw = make_inputs(31, S, M, E, zipf_bias=True)
    gate = ROUND[gd](mo.softmax_rows(raw))
    enc = mo.moe_encode_top2 if k == 2 else mo.moe_encode
    kw = {"gate_round": ROUND[gd]} if k == 2 else {}
    want = enc(data, gate, np.zeros(E, np.int32), cf, fast_scatter=True, **kw)
    il = want[1]
    Cap = want[4].shape[1]
    rng = np.random.default_rng(7)
    gates_s = ROUND[gd](want[0])
    d_il, d_g = dev(il), dev(gates_s).to(TORCH_DT[gd])
    # moe_encode_dg: gradient of gates_s scattered into [S, E], in the gradient's own 16-bit type
    dy_g = ROUND[gd](rng.standard_normal(k * S, dtype=np.float32))
    got = ops.moe_encode_dg(dev(dy_g).to(TORCH_DT[gd]), d_il, E, top_k=k)
    assert got.dtype == TORCH_DT[gd]
    np.testing.assert_array_equal(to_np(got), mo.moe_encode_dg(dy_g, il, E, k=k))
    # moe_decode_dx: rows of dy weighted by the half gates (fp32 product, one rounding to the row type)
    dy = rng.standard_normal((S, M), dtype=np.float32)
    got = ops.moe_decode_dx(dev(dy), d_g, d_il, E, Cap, top_k=k)
    np.testing.assert_array_equal(to_np(got), mo.moe_decode_dx(dy, gates_s, il, E, Cap, k=k))
    # moe_decode_dg: fp32 dot products, rounded once to the gate type (sum order differs: 1 unit in the last place)
    expert_out = rng.standard_normal((E, Cap, M), dtype=np.float32)
    got = ops.moe_decode_dg(dev(dy), dev(expert_out), d_il, top_k=k, gate_dtype=TORCH_DT[gd])
    assert got.dtype == TORCH_DT[gd]
    assert ulp_diff(got, mo.moe_decode_dg(dy, expert_out, il, k=k), gd) <= 1
    # top-2 combine weights from raw half values
    if k == 2:
        rawg = ROUND[gd](rng.random(2 * S, dtype=np.float32))
        got = ops.moe_top2_normalize_gates(dev(rawg).to(TORCH_DT[gd]), d_il)
        assert ulp_diff(got, mo.top2_normalize_gates(rawg, il[0]), gd) <= 0


def test_op_layer_takes_a_half_gate(pkg):
    """The C++ op layer declares gates_s in the gate's dtype and runs the half-gate kernels (it used to reject
    anything but float32, which forced a cast node into mixed-precision graphs)."""
    run = pkg.raf_executor.Executor()
    S, M, E = 1024, 32, 8
    data, raw = make_inputs(41, S, M, E)
    gate = mo.round_to_f16(mo.softmax_rows(raw))
    d_data, d_gate = dev(data).half(), dev(gate).half()
    used = torch.zeros(E, dtype=torch.int32, device="cuda")
    out = run("raf.op.moe_encode", d_data, d_gate, used, 1.0)
    want = mo.moe_encode(rows_as_oracle(data, "f16"), gate, np.zeros(E, np.int32), 1.0, fast_scatter=True)
    assert out[0].dtype == torch.float16
    np.testing.assert_array_equal(to_np(out[0]), want[0])
    np.testing.assert_array_equal(to_np(out[1]), want[1])
    np.testing.assert_array_equal(to_np(out[4]), want[4])
    dec = run("raf.op.moe_decode", out[4], out[0], out[1])
    np.testing.assert_array_equal(to_np(dec), mo.moe_decode(want[4], want[0], want[1], round_fn=mo.round_to_f16))


# From 512 tiles of 256 tokens on, gate rows longer than a cache line are read a wave's 64 rows at a time, 128 bytes
# of each, and passed through LDS; with logits the softmax denominator is then formed in the same walk as the
# selection (rescaled sum).  Row lengths: whole 128-byte chunks, a short last chunk, a single granule in the last.
@pytest.mark.parametrize("gd,E", [("f32", 64), ("f32", 100), ("f32", 36), ("bf16", 72), ("bf16", 128), ("f16", 200), ("f16", 68)])
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("logits", [False, True])
def test_selection_on_long_batches_of_long_rows(pkg, gd, E, k, logits):
    import ctypes as C
    ops, capi, lib = pkg.ops, pkg.capi, pkg.capi.load()
    S, M, cf = 131072 + 37, 4, 0.7            # 513 tiles, the last one ragged
    rng = np.random.default_rng(E + k)
    raw = rng.standard_normal((S, E), dtype=np.float32) * np.float32(2.0)
    raw[:, rng.integers(E)] += np.float32(1.5)
    data = rng.standard_normal((S, M), dtype=np.float32)
    gate32 = raw if logits else mo.softmax_rows(raw)
    gate = gate32 if gd == "f32" else ROUND[gd](gate32)
    rnd = None if gd == "f32" else ROUND[gd]
    used_in = (np.arange(E, dtype=np.int32) % 5) if k == 1 else np.zeros(E, np.int32)
    if k == 1:
        want = mo.moe_encode(data, gate, used_in, cf, gate_is_logits=logits, fast_scatter=True)
    else:
        want = mo.moe_encode_top2(data, gate, used_in, cf, gate_is_logits=logits, fast_scatter=True, gate_round=rnd)
    tdt = torch.float32 if gd == "f32" else TORCH_DT[gd]
    d_gate = dev(gate).to(tdt)
    got = ops.moe_encode(dev(data), d_gate, dev(used_in), cf, top_k=k, gate_is_logits=logits)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_array_equal(to_np(got[4]), want[4])
    if gd == "f32":
        np.testing.assert_allclose(to_np(got[0]), want[0], rtol=1e-5, atol=0)
    else:
        assert ulp_diff(got[0], want[0], gd) <= (0 if (k == 1 and not logits) else 1)
    # selection alone (lancet_gate_topk) takes the same path
    code = {"f32": capi.F32, "bf16": capi.BF16, "f16": capi.F16}[gd]
    p = lambda t: C.c_void_p(t.data_ptr())
    idx = torch.empty((k, S), dtype=torch.int32, device="cuda")
    val = torch.empty((k, S), dtype=tdt, device="cuda")
    assert lib.lancet_gate_topk(p(d_gate), None, S, E, k, code, capi.GATE_IS_LOGITS if logits else 0, p(idx), p(val), None) == 0
    wi, wv = mo.select_topk(gate, k, logits, None)
    np.testing.assert_array_equal(to_np(idx), wi)
    if not logits:
        np.testing.assert_array_equal(to_np(val).astype(np.float32), wv)


def test_batch_prioritized_on_a_long_batch_of_long_rows(pkg):
    S0, M, E, P = 140000, 4, 96, 2
    rng = np.random.default_rng(77)
    gate = mo.softmax_rows(rng.standard_normal((S0, E), dtype=np.float32) * np.float32(2.0))
    data = rng.standard_normal((S0, M), dtype=np.float32)
    for pid in range(P):
        want = mo.moe_encode_bpr(data, gate, P, pid, 0.8, fast_scatter=True)
        got = pkg.ops.moe_encode_batch_prioritized(dev(data), dev(gate), P, pid, 0.8)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[2]), want[2])
        np.testing.assert_array_equal(to_np(got[0]), want[0])

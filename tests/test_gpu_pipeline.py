"""The partitioned encode / exchange / decode pipeline on two streams against the un-partitioned operators
(the identity the reference tests for chained partitions, tests/python/op/cuda/test_cuda_moe.py:384-471)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, rows_as_oracle, rows_to_torch, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt,S,M,E,P,cf", [("f32", 4096, 64, 8, 4, 0.75), ("bf16", 8192, 256, 16, 2, 1.0),
                                           ("bf16", 16384, 512, 32, 8, 0.5)])
def test_pipeline_equals_unpartitioned_ops(pkg, dt, S, M, E, P, cf):
    ops = pkg.ops
    rng = np.random.default_rng(S + P)
    x = rows_as_oracle(rng.standard_normal((S, M), dtype=np.float32), dt)
    logits = rng.standard_normal((S, E), dtype=np.float32) * 2
    d_x, d_gate = rows_to_torch(x, dt), dev(logits)
    layer = pkg.pipeline.PartitionedMoeLayer(S, M, E, P, cf, dtype=d_x.dtype, gate_is_logits=True)
    piped = layer.run(d_x, d_gate).clone()
    masks = [m.clone() for m in layer.kept_masks()]
    serial = layer.run_serial(d_x, d_gate).clone()
    assert torch.equal(piped, serial)
    # a second pass over the same buffers (stale rows in the receive buffers must not leak)
    x2 = rows_as_oracle(rng.standard_normal((S, M), dtype=np.float32), dt)
    layer.run(rows_to_torch(x2, dt), d_gate)
    piped_again = layer.run(d_x, d_gate)
    assert torch.equal(piped_again, piped)
    # un-partitioned: one encode over all S tokens with the same total capacity, then decode
    assert ops.moe_capacity(S, E, cf) == layer.C
    gates_s, indloc, used, elems, disp = ops.moe_encode(d_x, d_gate, torch.zeros(E, dtype=torch.int32, device="cuda"),
                                                        cf, gate_is_logits=True)
    whole = ops.moe_decode(disp, gates_s, indloc)
    assert torch.equal(piped, whole)
    # the partitions keep exactly the tokens the whole batch keeps
    merged = ops.moe_merge_masks(masks, E)
    kept_whole = to_np(indloc)[0] >= 0
    np.testing.assert_array_equal(to_np(merged)[0] >= 0, kept_whole)
    assert 0 < kept_whole.sum() < S                      # the case drops tokens
    # the same partitions as token ranges of one whole-batch routing, exchanged at their row ranges
    layer.out.fill_(3.0), layer.once.send.fill_(4.0), layer.once.recv.fill_(5.0), layer.once.out.fill_(6.0)
    once = layer.run_routed_once(d_x, d_gate).clone()
    assert torch.equal(once, whole)
    assert torch.equal(layer.once.recv, disp) and torch.equal(layer.once.whole[1], indloc)
    layer.run_routed_once(rows_to_torch(x2, dt), d_gate)
    assert torch.equal(layer.run_routed_once(d_x, d_gate), whole)
    # and the oracle agrees on the decode of the kept tokens
    want = mo.moe_decode(to_np(disp), to_np(gates_s), to_np(indloc),
                         round_fn=None if dt == "f32" else mo.round_to_bf16)
    np.testing.assert_array_equal(to_np(piped), want)


def test_concurrent_calls_on_separate_streams_share_no_state(pkg):
    """Eight encode + decode pairs issued on eight streams at once, each with its own workspace and outputs
    (the library keeps no state between calls), repeated a few times: every result equals the one the same
    call gives when it runs alone."""
    import numpy as np
    from tests.gpu_util import dev, make_inputs
    ops = pkg.ops
    S, M, E, cf = 8192, 512, 16, 0.9
    jobs = []
    for i in range(8):
        k = 1 + i % 2
        data, logits = make_inputs(40 + i, S, M, E, zipf_bias=bool(i & 2))
        d_data = dev(data).to(torch.bfloat16 if i % 3 else torch.float32)
        d_logits = dev(logits)
        alone = ops.moe_encode(d_data, d_logits, None, cf, top_k=k, gate_is_logits=True)
        alone_out = ops.moe_decode(alone[4], alone[0], alone[1], top_k=k)
        outs = tuple(torch.empty_like(t) if t.dtype != torch.uint64 else torch.empty(t.shape, dtype=torch.int64, device="cuda")
                     for t in alone)
        ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, k))
        torch.cuda.synchronize()   # set up on this stream, used on the streams below
        jobs.append((k, d_data, d_logits, alone, alone_out, outs, ws, torch.empty_like(alone_out), torch.cuda.Stream()))
    torch.cuda.synchronize()
    for _ in range(3):
        for k, d_data, d_logits, _, _, outs, ws, dec, stream in jobs:
            with torch.cuda.stream(stream):
                ops.moe_encode(d_data, d_logits, None, cf, top_k=k, gate_is_logits=True, workspace=ws, out=outs)
                ops.moe_decode(outs[4], outs[0], outs[1], top_k=k, out=dec)
        torch.cuda.synchronize()
        for k, _, _, alone, alone_out, outs, ws, dec, _ in jobs:
            for a, b in zip(alone, outs):
                assert torch.equal(a.view(torch.int64) if a.dtype == torch.uint64 else a, b)
            assert torch.equal(alone_out, dec)
            for t in outs:
                t.zero_()
            dec.zero_()
        torch.cuda.synchronize()            # the clears run on the default stream


@pytest.mark.parametrize("dt,S,M,E,P,cf", [("bf16", 8192, 256, 16, 4, 0.6), ("f32", 3000, 40, 6, 3, 1.0), ("f16", 4096, 64, 32, 8, 0.4)])
def test_routed_once_pipeline_top2_equals_unpartitioned_ops(pkg, dt, S, M, E, P, cf):
    """RoutedOnceMoeLayer with top-2 routing: one routing of the batch, per partition a scatter of its tokens (both
    slots), the exchange of the rows it owns (one range per slot and expert) and a decode, against moe_encode +
    moe_decode over the whole batch, twice over the same buffers."""
    ops = pkg.ops
    rng = np.random.default_rng(S + P)
    x = rows_as_oracle(rng.standard_normal((S, M), dtype=np.float32), dt)
    logits = rng.standard_normal((S, E), dtype=np.float32) * 2
    d_x, d_gate = rows_to_torch(x, dt), dev(logits)
    layer = pkg.pipeline.RoutedOnceMoeLayer(S, M, E, P, cf, top_k=2, dtype=d_x.dtype, gate_is_logits=True)
    layer.send.fill_(4.0), layer.recv.fill_(5.0), layer.out.fill_(6.0)
    got = layer.run(d_x, d_gate).clone()
    gates_s, indloc, used, elems, disp = ops.moe_encode(d_x, d_gate, None, cf, top_k=2, gate_is_logits=True)
    whole = ops.moe_decode(disp, gates_s, indloc, top_k=2)
    assert torch.equal(got, whole) and torch.equal(layer.recv, disp)
    assert bool((indloc[0] < 0).any())
    x2 = rows_as_oracle(rng.standard_normal((S, M), dtype=np.float32), dt)
    layer.run(rows_to_torch(x2, dt), d_gate)
    assert torch.equal(layer.run(d_x, d_gate), whole)

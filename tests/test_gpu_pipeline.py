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
    # and the oracle agrees on the decode of the kept tokens
    want = mo.moe_decode(to_np(disp), to_np(gates_s), to_np(indloc),
                         round_fn=None if dt == "f32" else mo.round_to_bf16)
    np.testing.assert_array_equal(to_np(piped), want)

"""lancet_moe_encode_noalloc (static device scratch, no allocation) against lancet_moe_encode, through the
C ABI: identical outputs, bit for bit, on two calls in a row, the second with a smaller input, both in the scan's
look-back form (the one form that keeps state: the shared scratch still holds the first call's descriptors under
the second call's table), then once more with top-1 and a used capacity; and at the largest size the scratch holds."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, to_np

pytestmark = pytest.mark.gpu


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(None)


def _outputs(S, M, E, Cap, k, dtype):
    return (torch.full((k * S,), -7.0, dtype=torch.float32, device="cuda"),
            torch.full((2, k * S), -7, dtype=torch.int32, device="cuda"),
            torch.full((E,), -7, dtype=torch.int32, device="cuda"),
            torch.full((E,), -7, dtype=torch.int64, device="cuda"),
            torch.full((E, Cap, M), -7.0, dtype=dtype, device="cuda"))


def _encode_both(pkg, lib, data, gate, used_in, cf, k, flags):
    capi = pkg.capi
    S, M = data.shape
    E = gate.shape[1]
    Cap = int(lib.lancet_moe_capacity(S, E, cf * (2.0 if k == 2 else 1.0)))
    dt = {torch.float32: capi.F32, torch.bfloat16: capi.BF16}[data.dtype]
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ref = _outputs(S, M, E, Cap, k, data.dtype)
    ws_bytes = lib.lancet_moe_encode_workspace_bytes(S, E, k)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    assert lib.lancet_scan_workspace_init(_p(ws), ws_bytes, st) == 0
    rc = lib.lancet_moe_encode(_p(data), _p(gate), None, _p(used_in), S, M, E, Cap, k, dt, capi.F32, flags, *[_p(t) for t in ref],
                               _p(ws), ws_bytes, st)
    assert rc == 0, capi.status_string(rc)
    got = _outputs(S, M, E, Cap, k, data.dtype)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.lancet_moe_encode_noalloc(_p(data), _p(gate), None, _p(used_in), S, M, E, Cap, k, dt, capi.F32, flags,
                                       *[_p(t) for t in got], st)
    assert rc == 0, capi.status_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return ref, got, Cap


def test_noalloc_encode_equals_encode_on_two_calls_in_a_row(pkg, lib):
    capi = pkg.capi
    # first call: top-2 on logits, bf16 rows; second call: smaller batch, fewer experts (fewer tiles and
    # counters than the descriptors the first call left in the scratch)
    for seed, (S, M, E, k, dtype) in enumerate([(5000, 256, 32, 2, torch.bfloat16), (1300, 64, 8, 2, torch.bfloat16)]):
        data, logits = make_inputs(100 + seed, S, M, E)
        d_data = dev(data).to(dtype)
        ref, got, Cap = _encode_both(pkg, lib, d_data, dev(logits), None, 1.0, k, capi.GATE_IS_LOGITS | capi.SCAN_LOOKBACK)
        for name, r, g in zip(("gates_s", "indices_locations", "used_capacity", "elements_per_expert", "dispatched"), ref, got):
            assert torch.equal(r.view(torch.uint8), g.view(torch.uint8)), (seed, name)
        # and both equal the oracle's routing
        want = mo.moe_encode_top2(mo.round_to_bf16(data), logits, np.zeros(E, np.int32), 1.0, gate_is_logits=True,
                                  fast_scatter=True)
        np.testing.assert_array_equal(to_np(got[1]), want[1])
        np.testing.assert_array_equal(to_np(got[4]), want[4])
    # third call: top-1 with a used capacity, fp32 rows, gate probabilities
    S, M, E = 777, 20, 16
    data, logits = make_inputs(7, S, M, E)
    gate = mo.softmax_rows(logits)
    used = np.arange(E, dtype=np.int32) % 5
    ref, got, Cap = _encode_both(pkg, lib, dev(data), dev(gate), dev(used), 1.0, 1, 0)
    for r, g in zip(ref, got):
        assert torch.equal(r.view(torch.uint8), g.view(torch.uint8))
    want = mo.moe_encode(data, gate, used, 1.0, fast_scatter=True)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[4]), want[4])


def test_noalloc_encode_at_the_limit_of_its_scratch(pkg, lib):
    """S = 65536, E = 512, top-2 is the largest power-of-two batch whose table fits (256 tiles x 1024 counters);
    one tile more is rejected."""
    capi = pkg.capi
    S, M, E, k = 65536, 8, 512, 2
    assert lib.lancet_moe_encode_workspace_bytes(S, E, k) <= capi.NOALLOC_SCRATCH_BYTES
    assert lib.lancet_moe_encode_workspace_bytes(S + 1, E, k) > capi.NOALLOC_SCRATCH_BYTES
    data, logits = make_inputs(12, S, M, E)
    d_data, d_logits = dev(data).to(torch.bfloat16), dev(logits)
    for flags in (capi.GATE_IS_LOGITS, capi.GATE_IS_LOGITS | capi.SCAN_LOOKBACK):
        ref, got, Cap = _encode_both(pkg, lib, d_data, d_logits, None, 1.0, k, flags)
        for r, g in zip(ref, got):
            assert torch.equal(r.view(torch.uint8), g.view(torch.uint8))
        assert int((got[1][0] >= 0).sum()) > S
    one = torch.zeros(1, device="cuda")
    rc = lib.lancet_moe_encode_noalloc(_p(one), _p(one), None, None, S + 1, M, E, 8, k, capi.BF16, capi.F32, 0, _p(one), _p(one),
                                       _p(one), _p(one), _p(one), None)
    assert rc == capi.ERR_SCRATCH


def test_noalloc_encode_rejects_sizes_beyond_its_scratch(pkg, lib):
    capi = pkg.capi
    assert capi.NOALLOC_SCRATCH_BYTES == (2 << 20) + 4096     # LANCET_NOALLOC_SCRATCH_BYTES of the header
    S, E, k = 1 << 20, 512, 2          # 4096 tiles x 1024 counters x 4 B = 16 MiB of descriptors
    assert lib.lancet_moe_encode_workspace_bytes(S, E, k) > capi.NOALLOC_SCRATCH_BYTES
    one = torch.zeros(1, device="cuda")
    rc = lib.lancet_moe_encode_noalloc(_p(one), _p(one), None, None, S, 4, E, 8, k, capi.F32, capi.F32, 0, _p(one), _p(one), _p(one),
                                       _p(one), _p(one), None)
    assert rc == capi.ERR_SCRATCH
    assert "scratch" in capi.status_string(rc)

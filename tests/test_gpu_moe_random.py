"""Seeded random sweep of the dispatch path against the oracle: shapes the hand-picked cases do not reach
(expert counts up to the 512 the kernels support, token counts around tile and wave boundaries, rows that
are and are not 16-byte multiples, used capacity carried in, every storage type), end to end through
encode -> decode and the batch-prioritized encode.  Same bar as the other parity tests: integers and rows
bit-exact, gates 1e-5 relative, 16-bit decode within one unit in the last place."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, make_inputs, rows_as_oracle, rows_to_torch, to_np

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    S = int(rng.choice([1, 63, 64, 65, 255, 256, 257, 511, 1000, 1537, 2048, 3001]))
    E = int(rng.choice([1, 2, 3, 7, 8, 31, 33, 64, 65, 100, 255, 256, 257, 400, 512]))
    M = int(rng.choice([1, 3, 4, 8, 20, 36, 64, 72, 130]))
    dt = str(rng.choice(["f32", "bf16", "f16"]))
    k = int(rng.choice([1, 2])) if E >= 2 else 1
    cf = float(rng.choice([0.25, 0.5, 1.0, 1.5, 4.0]))
    return rng, S, M, E, dt, k, cf


@pytest.mark.parametrize("seed", range(32))
def test_encode_decode_random(pkg, seed):
    rng, S, M, E, dt, k, cf = _case(seed)
    print("case", seed, dict(S=S, M=M, E=E, dt=dt, k=k, cf=cf), flush=True)
    data, logits = make_inputs(seed, S, M, E, logit_scale=float(rng.choice([0.5, 2.0])), zipf_bias=bool(rng.integers(2)))
    x = rows_as_oracle(data, dt)
    Cap = mo.capacity(S, E, cf * k)
    used0 = rng.integers(0, max(Cap, 1) + 1, E).astype(np.int32) if k == 1 and rng.integers(2) else np.zeros(E, np.int32)
    if k == 1:
        want = mo.moe_encode(x, logits, used0, cf, gate_is_logits=True, fast_scatter=True)
    else:
        want = mo.moe_encode_top2(x, logits, used0, cf, gate_is_logits=True, fast_scatter=True)
    got = pkg.ops.moe_encode(rows_to_torch(data, dt), dev(logits), dev(used0), cf, top_k=k, gate_is_logits=True)
    g, il, used, elems, disp = got
    np.testing.assert_array_equal(to_np(il), want[1])
    np.testing.assert_array_equal(to_np(used), want[2])
    np.testing.assert_array_equal(to_np(elems), want[3])
    np.testing.assert_allclose(to_np(g), want[0], rtol=1e-5, atol=0)
    np.testing.assert_array_equal(to_np(disp), want[4])
    # decode of the buffer the GPU produced, with the GPU's own gates (so the comparison is exact in fp32)
    round_fn = {"f32": None, "bf16": mo.round_to_bf16, "f16": lambda a: a.astype(np.float16).astype(np.float32)}[dt]
    want_dec = mo.moe_decode(to_np(disp), to_np(g), to_np(il), k=k, round_fn=round_fn)
    got_dec = to_np(pkg.ops.moe_decode(disp, g, il, top_k=k))
    if dt == "f32":
        np.testing.assert_array_equal(got_dec, want_dec)
    else:
        ulp = np.maximum(np.abs(want_dec), 1e-30) * (2.0 ** -7 if dt == "bf16" else 2.0 ** -10)
        assert (np.abs(got_dec - want_dec) <= ulp).all()


@pytest.mark.parametrize("seed", range(12))
def test_encode_bpr_random(pkg, seed):
    rng = np.random.default_rng(2000 + seed)
    P = int(rng.choice([1, 2, 3, 4]))
    S0 = P * int(rng.choice([1, 50, 256, 300, 777]))
    E = int(rng.choice([1, 2, 5, 16, 64, 130, 512]))
    M = int(rng.choice([1, 4, 12, 64]))
    cf = float(rng.choice([0.5, 1.0, 2.0])) * P
    ties = bool(rng.integers(2))
    print("case", seed, dict(S0=S0, M=M, E=E, P=P, cf=cf, ties=ties), flush=True)
    data, logits = make_inputs(seed, S0, M, E, logit_scale=2.0, ties=ties)
    gate = mo.softmax_rows(logits)
    if ties:
        gate = (np.round(gate * 8) / 8).astype(np.float32)
    d_data, d_gate = dev(data), dev(gate)
    for pid in range(P):
        want = mo.moe_encode_bpr(data, gate, P, pid, cf, fast_scatter=True)
        g, il, used, elems, disp = pkg.ops.moe_encode_batch_prioritized(d_data, d_gate, P, pid, cf)
        np.testing.assert_array_equal(to_np(il), want[1])
        np.testing.assert_array_equal(to_np(used), want[2])
        np.testing.assert_array_equal(to_np(elems), want[3])
        np.testing.assert_array_equal(to_np(g), want[0])
        np.testing.assert_array_equal(to_np(disp), want[4])


@pytest.mark.parametrize("S,E,k,cf,skew", [(300001, 512, 2, 1.0, 3.0), (262144, 2, 2, 0.3, 0.0), (100000, 100, 1, 2.5, 1.0),
                                           (65536, 256, 2, 0.3, 3.0), (300001, 3, 1, 1.0, 0.0), (262144, 64, 1, 0.3, 3.0)])
def test_routing_over_many_tiles(pkg, S, E, k, cf, skew, scan_lookback=False):
    """Long batches: more than a thousand scan tiles, look-back windows of a couple of rows (E = 512, top-2) up
    to hundreds, a crowded expert, chained used capacity; every output against the oracle (M = 4 keeps the
    oracle's row movement small)."""
    rng = np.random.default_rng(S + E + k)
    M = 4
    logits = rng.standard_normal((S, E), dtype=np.float32)
    logits[:, rng.integers(E)] += np.float32(skew)
    data = rng.standard_normal((S, M), dtype=np.float32)
    used0 = np.zeros(E, np.int32)
    if k == 1:
        used0 = rng.integers(0, max(mo.capacity(S, E, cf), 1) + 1, E).astype(np.int32)
    want = (mo.moe_encode_top2 if k == 2 else mo.moe_encode)(data, logits, used0, cf, gate_is_logits=True, fast_scatter=True)
    got = pkg.ops.moe_encode(dev(data), dev(logits), dev(used0), cf, top_k=k, gate_is_logits=True, scan_lookback=scan_lookback)
    np.testing.assert_array_equal(to_np(got[1]), want[1])
    np.testing.assert_array_equal(to_np(got[2]), want[2])
    np.testing.assert_array_equal(to_np(got[3]), want[3])
    np.testing.assert_allclose(to_np(got[0]), want[0], rtol=1e-5, atol=0)
    np.testing.assert_array_equal(to_np(got[4]), want[4])


# one counter set on at most 32 tiles: one look-back kernel; tiles x counters up to 32768: two kernels without waits;
# beyond: three (segment sums between count and place).  Every case also as one look-back kernel.
@pytest.mark.parametrize("S,E,k,cf,skew", [
    (32768, 512, 2, 1.0, 2.0),    # 128 tiles x 1024 counters: two pairs of counters per thread and row, segments of 32
    (8192, 512, 2, 1.0, 2.0),     # 32 x 1024 = 32768: the last size at which every tile adds up all rows
    (8193, 512, 2, 1.0, 2.0),     # one tile more: segment sums
    (49152, 256, 2, 0.5, 3.0),    # 192 x 512: one pair per thread, rows read eight at a time
    (8448, 100, 1, 1.5, 1.0),     # 33 tiles, 50 pairs (do not divide the workgroup: sums through LDS atomics)
    (8192, 100, 1, 1.5, 1.0),     # 32 tiles, one set: look-back
    (20000, 64, 1, 0.7, 2.0),     # 79 x 64: 32 pairs, several rows per thread and a remainder
    (9000, 7, 1, 1.0, 0.0),       # odd counter count: the last pair's high half is empty
    (5000, 3, 2, 1.0, 0.0), (300, 2, 2, 2.0, 0.0), (1, 2, 2, 1.0, 0.0),
    (786432, 16, 1, 1.0, 1.0),    # 3072 tiles: more tiles than run at once; segments of 64, the last one short
    (300001, 1, 1, 0.5, 0.0),     # one expert: one counter per tile, 1172 tiles, segment table behind an odd-sized table
    (262145, 33, 2, 1.0, 2.0),    # 1025 tiles in segments of 64 (the 17th holds one tile), 66 counters
])
def test_every_form_of_the_scan_at_its_boundaries(pkg, S, E, k, cf, skew):
    test_routing_over_many_tiles(pkg, S, E, k, cf, skew)
    test_routing_over_many_tiles(pkg, S, E, k, cf, skew, scan_lookback=True)

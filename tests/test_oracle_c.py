"""The C restatement (OpenMP, the timed CPU baseline) must agree with the NumPy oracle:
integers and moved rows bit for bit, softmax values to 1e-6, LANS to 1e-6."""
import subprocess
import os

import numpy as np
import pytest

from oracle import lans_oracle as lo
from oracle import moe_oracle as mo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def co():
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    from oracle import c_oracle
    c_oracle.load()
    return c_oracle


@pytest.mark.parametrize("k,is_logits,bf16", [(1, False, False), (1, True, True), (2, True, False), (2, True, True)])
@pytest.mark.parametrize("S,M,E,cf", [(700, 12, 8, 0.6), (2048, 16, 32, 1.0), (5, 3, 2, 1.0)])
def test_c_encode_decode_match_numpy(co, k, is_logits, bf16, S, M, E, cf):
    rng = np.random.default_rng(S + k)
    data = rng.standard_normal((S, M), dtype=np.float32)
    logits = rng.standard_normal((S, E), dtype=np.float32)
    logits[:, 0] += 1.0
    gate = logits if is_logits else mo.softmax_rows(logits)
    used_in = rng.integers(0, 3, E).astype(np.int32)
    if bf16:
        data = mo.round_to_bf16(data)
    Cap = mo.capacity(S, E, cf * k)
    if k == 1:
        want = mo.moe_encode(data, gate, used_in, C=Cap, gate_is_logits=is_logits)
    else:
        want = mo.moe_encode_top2(data, gate, used_in, C=Cap, gate_is_logits=is_logits)
    cdata = mo.f32_to_bf16_bits(data) if bf16 else data
    got = co.moe_encode(cdata, gate, used_in, Cap, k, is_logits)
    np.testing.assert_array_equal(got[1], want[1])
    np.testing.assert_array_equal(got[2], want[2])
    np.testing.assert_array_equal(got[3], want[3])
    np.testing.assert_allclose(got[0], want[0], rtol=1e-6 if is_logits else 0)
    gdisp = mo.bf16_bits_to_f32(got[4]) if bf16 else got[4]
    np.testing.assert_array_equal(gdisp, want[4])
    out = co.moe_decode(got[4], want[0], want[1], k)
    ref = mo.moe_decode(want[4], want[0], want[1], k, round_fn=mo.round_to_bf16 if bf16 else None)
    np.testing.assert_array_equal(mo.bf16_bits_to_f32(out) if bf16 else out, ref)


@pytest.mark.parametrize("hyper", [dict(), dict(mode=0), dict(weight_decay=0.0, normalize_grad=False),
                                   dict(bias_correction=0, grad_averaging=0)])
def test_c_lans_matches_numpy(co, hyper):
    rng = np.random.default_rng(0)
    shapes = [(40, 30), (17,), (3000,), (1,)]
    p = [rng.normal(0, 0.02, s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    p2, m2, v2 = ([a.copy() for a in l] for l in (p, m, v))
    for step in range(1, 6):
        g = [rng.normal(0, 1e-3, s).astype(np.float32) for s in shapes]
        n1 = lo.lans_step(g, p, m, v, step, **hyper)
        n2 = co.lans_step(g, p2, m2, v2, step, **hyper)
        np.testing.assert_allclose(n2, np.array(n1, np.float32), rtol=1e-6)
    for a, b in zip(p + m + v, p2 + m2 + v2):
        np.testing.assert_allclose(b, a, rtol=1e-6, atol=1e-12)


def test_thread_count_is_reported(co):
    assert co.num_threads() >= 1

"""The dispatch path on buffers beyond 32-bit offsets: an [E, C, M] buffer of more than 2^31 elements
(more than 4 GiB), where the reference's 32-bit index arithmetic (tutel_moe_dispatch.cu:61-70) stops.

At this size the oracle checks the routing integers (they only depend on the [S, E] gate); the rows
are checked on the GPU with size-independent properties: every kept token's row sits at its
(expert, location) bit for bit, every other buffer row is zero, decode with unit gates returns the
kept rows and zeros, the backward scatter rebuilds the buffer, two chained half-batch encodes followed
by moe_redispatch rebuild it, and packing + unpacking the used rows rebuilds it.
"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as mo
from tests.gpu_util import dev, to_np

pytestmark = pytest.mark.gpu

S, M, E, CF = 393216, 8192, 8, 1.25


def _bits(t):
    return t.view(torch.int16)


@pytest.fixture(scope="module")
def big(pkg):
    ops = pkg.ops
    free, _ = torch.cuda.mem_get_info()
    if free < 48 << 30:
        pytest.skip("needs 48 GiB of free device memory")
    rng = np.random.default_rng(91)
    logits = rng.standard_normal((S, E), dtype=np.float32)
    logits[:, 3] += np.float32(0.5)                      # one crowded expert, so that tokens are dropped
    gate = mo.softmax_rows(logits)
    gen = torch.Generator(device="cuda").manual_seed(17)
    data = torch.randn((S, M), generator=gen, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    zero = torch.zeros(E, dtype=torch.int32, device="cuda")
    out = ops.moe_encode(data, dev(gate), zero, CF)
    torch.cuda.synchronize()
    return ops, gate, data, out


def test_buffer_is_beyond_32_bit_offsets(big):
    _, _, _, (_, _, _, _, disp) = big
    assert disp.numel() > 2 ** 31 and disp.numel() * disp.element_size() > 2 ** 32


def test_routing_equals_oracle(big):
    ops, gate, data, (g, il, used, elems, disp) = big
    C = ops.moe_capacity(S, E, CF)
    wg, wil, wused, welems = _route(gate, C)
    np.testing.assert_array_equal(to_np(il), wil)
    np.testing.assert_array_equal(to_np(used), wused)
    np.testing.assert_array_equal(to_np(elems), welems)
    np.testing.assert_array_equal(to_np(g), wg)
    assert (wil[0] < 0).any() and wused.max() == C       # the case drops tokens and fills an expert


def _route(gate, C):
    """Top-1 routing of the oracle without its row movement (which would need the 6 GiB batch on the host)."""
    idx, val = mo.select_topk(gate, 1)
    idx, loc, used, elems = mo.gen_location(idx[0].copy(), np.zeros(E, np.int32), C, M, E)
    return val[0], np.stack([idx, loc]), used, elems


def test_rows_sit_at_their_locations_and_the_rest_is_zero(big):
    ops, _, data, (_, il, used, _, disp) = big
    C = disp.shape[1]
    idx, loc = il[0].long(), il[1].long()
    kept = idx >= 0
    rows = disp.view(E * C, M)
    slot = idx[kept] * C + loc[kept]
    assert torch.equal(_bits(rows[slot]), _bits(data[kept]))
    assert slot.unique().numel() == slot.numel()
    unused = torch.ones(E * C, dtype=torch.bool, device="cuda")
    unused[slot] = False
    assert int(unused.sum()) == E * C - int(used.sum())
    assert not bool(_bits(rows[unused]).any())


def test_decode_with_unit_gates_returns_the_kept_rows(big):
    ops, _, data, (_, il, _, _, disp) = big
    out = ops.moe_decode(disp, torch.ones(S, device="cuda"), il)
    kept = il[0] >= 0
    assert torch.equal(_bits(out[kept]), _bits(data[kept]))
    assert not bool(_bits(out[~kept]).any())


def test_backward_scatter_rebuilds_the_buffer(big):
    ops, _, data, (_, il, _, _, disp) = big
    C = disp.shape[1]
    got = ops.moe_decode_dx(data, torch.ones(S, device="cuda"), il, E, C)
    assert torch.equal(_bits(got), _bits(disp))
    dx = ops.moe_encode_dx(disp, il)
    kept = il[0] >= 0
    assert torch.equal(_bits(dx[kept]), _bits(data[kept])) and not bool(_bits(dx[~kept]).any())


def test_chained_halves_and_redispatch_rebuild_the_buffer(big):
    ops, gate, data, (_, il, used, _, disp) = big
    h = S // 2
    d_gate = dev(gate)
    zero = torch.zeros(E, dtype=torch.int32, device="cuda")
    a = ops.moe_encode(data[:h], d_gate[:h], zero, CF * 2, zero_tail=False)
    b = ops.moe_encode(data[h:], d_gate[h:], a[2], CF * 2, zero_tail=False)
    assert a[4].shape == disp.shape and torch.equal(b[2], used)
    got = ops.moe_redispatch([a[4], b[4]], [a[1], b[1]])
    assert torch.equal(_bits(got), _bits(disp))
    merged = ops.moe_merge_masks([a[1], b[1]], E)
    kept = il[0] >= 0
    assert torch.equal(merged[0], il[0]) and torch.equal(merged[1][kept], il[1][kept])
    assert bool((merged[1][~kept] == -1).all())          # a dropped token's location is -1 after the merge


def test_pack_and_unpack_rebuild_the_buffer(big):
    ops, _, _, (_, _, used, elems, disp) = big
    total = int(elems.sum())
    assert total == int(used.sum()) * M and total > 2 ** 31
    wire = torch.empty(total, dtype=disp.dtype, device="cuda")
    ops.memcpy_sparse_to_cont_3d(disp, wire, elems, axis=0)
    C = disp.shape[1]
    first = torch.cat([disp[e, :int(used[e])].reshape(-1) for e in range(E)])
    assert torch.equal(_bits(wire), _bits(first))
    back = torch.full_like(disp, 3.0)
    ops.memcpy_cont_to_sparse_3d(wire, back, elems, axis=0, zero_tail=True)
    assert torch.equal(_bits(back), _bits(disp))

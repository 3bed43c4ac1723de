"""Gradient wiring of the MoE dispatch operators, as RAF registers it (src/op/grad/moe.cc:30-93), for callers
that differentiate with torch.autograd.

  moe_encode, moe_encode_batch_prioritized (MoeEncodeGrad, :30-58):
      d data = moe_encode_dx(dy[4], y[1]);  d gate = moe_encode_dg(dy[0], y[1], E);  used_capacity: none
  moe_decode (MoeDecodeGrad, :60-90):
      d data = moe_decode_dx(dy, gate, indices_locations, E, C);  d gate = moe_decode_dg(dy, data, indices_locations)

The wrappers cover what the reference differentiates: top-1 ops on a gate that holds probabilities.  Every
gradient is computed by the HIP backward kernels; nothing here falls back to torch arithmetic.
"""
import torch

from . import ops


class _MoeEncode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, gate, used_capacity, capacity_factor, bpr):
        if bpr is None:
            out = ops.moe_encode(data, gate, used_capacity, capacity_factor)
        else:
            out = ops.moe_encode_batch_prioritized(data, gate, bpr[0], bpr[1], capacity_factor)
        gates_s, indloc, used, elems, disp = out
        ctx.save_for_backward(indloc)
        ctx.n_experts = gate.shape[1]
        ctx.bpr = bpr
        ctx.data_shape, ctx.data_dtype = data.shape, data.dtype
        ctx.mark_non_differentiable(indloc, used, elems)
        return gates_s, indloc, used, elems, disp

    @staticmethod
    def backward(ctx, d_gates_s, _d_indloc, _d_used, _d_elems, d_disp):
        (indloc,) = ctx.saved_tensors
        dx = ops.moe_encode_dx(d_disp.contiguous(), indloc)
        dg = ops.moe_encode_dg(d_gates_s.contiguous(), indloc, ctx.n_experts)
        if ctx.bpr is not None:
            # the op saw the whole batch and encoded one partition of it: the other tokens get no gradient
            # (the reference's rule returns the partition-sized arrays as they are)
            P, pid = ctx.bpr
            S = indloc.shape[1]
            full_x = torch.zeros(ctx.data_shape, dtype=ctx.data_dtype, device=dx.device)
            full_g = torch.zeros((ctx.data_shape[0], ctx.n_experts), dtype=dg.dtype, device=dx.device)
            full_x[pid * S:(pid + 1) * S] = dx
            full_g[pid * S:(pid + 1) * S] = dg
            dx, dg = full_x, full_g
        return dx, dg, None, None, None


class _MoeDecode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, gate, indices_locations):
        ctx.save_for_backward(data, gate, indices_locations)
        return ops.moe_decode(data, gate, indices_locations)

    @staticmethod
    def backward(ctx, dy):
        data, gate, indloc = ctx.saved_tensors
        E, C, _ = data.shape
        dy = dy.contiguous()
        return ops.moe_decode_dx(dy, gate, indloc, E, C), ops.moe_decode_dg(dy, data, indloc, gate_dtype=gate.dtype), None


def moe_encode(data, gate, used_capacity=None, capacity_factor=1.0):
    """Differentiable raf.op.moe_encode: gradients flow to data (through dispatched) and to gate (through gates_s)."""
    return _MoeEncode.apply(data, gate, used_capacity, float(capacity_factor), None)


def moe_encode_batch_prioritized(data, gate, n_partitions=1, partition_id=0, capacity_factor=1.0):
    """Differentiable raf.op.moe_encode_batch_prioritized (same gradient as moe_encode, src/op/grad/moe.cc:58)."""
    return _MoeEncode.apply(data, gate, None, float(capacity_factor), (int(n_partitions), int(partition_id)))


def moe_decode(data, gate, indices_locations):
    """Differentiable raf.op.moe_decode: gradients flow to data (expert outputs) and to gate (gates_s)."""
    return _MoeDecode.apply(data, gate, indices_locations)

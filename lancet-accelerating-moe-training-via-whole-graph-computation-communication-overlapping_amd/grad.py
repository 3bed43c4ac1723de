"""Gradient wiring of the MoE dispatch operators, as RAF registers it (src/op/grad/moe.cc:30-93), for callers
that differentiate with torch.autograd.

  moe_encode, moe_encode_batch_prioritized (MoeEncodeGrad, :30-58):
      d data = moe_encode_dx(dy[4], y[1]);  d gate = moe_encode_dg(dy[0], y[1], E);  used_capacity: none
  moe_decode (MoeDecodeGrad, :60-90):
      d data = moe_decode_dx(dy, gate, indices_locations, E, C);  d gate = moe_decode_dg(dy, data, indices_locations)

The reference differentiates the one form of the op it has: top-1 on a gate that holds probabilities.  The forms
this library adds (top_k = 2 with GShard's normalised combine weights, docker/resources/sharded_moe.py:253-324, and
the softmax fused into the op, gate_is_logits) do more to a gate value than select it, so their gate gradient is
    d gate = moe_encode_dgate(dy[0], gate, y[1])
which goes back through the normalisation and the softmax (ops.moe_encode_dgate); moe_decode's rules take top_k.
Every gradient is computed by the HIP backward kernels; nothing here falls back to torch arithmetic.
"""
import torch

from . import ops


class _MoeEncode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, gate, used_capacity, capacity_factor, bpr, top_k=1, gate_is_logits=False, gate2_noise=None,
                capacity=None):
        if bpr is None:
            out = ops.moe_encode(data, gate, used_capacity, capacity_factor, top_k=top_k, gate_is_logits=gate_is_logits,
                                 gate2_noise=gate2_noise, capacity=capacity)
        else:
            out = ops.moe_encode_batch_prioritized(data, gate, bpr[0], bpr[1], capacity_factor, gate_is_logits=gate_is_logits)
        gates_s, indloc, used, elems, disp = out
        # the plain rule needs the mask only; the forms that transform the gate value need the gate too
        ctx.whole_op = top_k == 2 or gate_is_logits
        ctx.save_for_backward(indloc, gate if ctx.whole_op else None)
        ctx.n_experts = gate.shape[1]
        ctx.bpr = bpr
        ctx.top_k, ctx.gate_is_logits = top_k, gate_is_logits
        ctx.data_shape, ctx.data_dtype = data.shape, data.dtype
        ctx.mark_non_differentiable(indloc, used, elems)
        return gates_s, indloc, used, elems, disp

    @staticmethod
    def backward(ctx, d_gates_s, _d_indloc, _d_used, _d_elems, d_disp):
        indloc, gate = ctx.saved_tensors
        dx = ops.moe_encode_dx(d_disp.contiguous(), indloc, top_k=ctx.top_k)
        if not ctx.whole_op:
            dg = ops.moe_encode_dg(d_gates_s.contiguous(), indloc, ctx.n_experts)
        elif ctx.bpr is None:
            dg = ops.moe_encode_dgate(d_gates_s.contiguous(), gate, indloc, ctx.top_k, ctx.gate_is_logits)
        else:
            P, pid = ctx.bpr
            S = indloc.shape[1]
            dg = ops.moe_encode_dgate(d_gates_s.contiguous(), gate[pid * S:(pid + 1) * S], indloc, 1, ctx.gate_is_logits)
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
        return dx, dg, None, None, None, None, None, None, None


class _MoeDecode(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, gate, indices_locations, top_k=1):
        ctx.save_for_backward(data, gate, indices_locations)
        ctx.top_k = top_k
        return ops.moe_decode(data, gate, indices_locations, top_k=top_k)

    @staticmethod
    def backward(ctx, dy):
        data, gate, indloc = ctx.saved_tensors
        E, C, _ = data.shape
        dy = dy.contiguous()
        return (ops.moe_decode_dx(dy, gate, indloc, E, C, top_k=ctx.top_k),
                ops.moe_decode_dg(dy, data, indloc, top_k=ctx.top_k, gate_dtype=gate.dtype), None, None)


def moe_encode(data, gate, used_capacity=None, capacity_factor=1.0, top_k=1, gate_is_logits=False, gate2_noise=None,
               capacity=None):
    """Differentiable raf.op.moe_encode: gradients flow to data (through dispatched) and to gate (through gates_s);
    with top_k = 2 or gate_is_logits the gate gradient goes back through the normalisation of the combine weights
    and through the fused softmax.  gate2_noise only moves the second choice and gets no gradient."""
    return _MoeEncode.apply(data, gate, used_capacity, float(capacity_factor), None, int(top_k), bool(gate_is_logits),
                            gate2_noise, capacity)


def moe_encode_batch_prioritized(data, gate, n_partitions=1, partition_id=0, capacity_factor=1.0, gate_is_logits=False):
    """Differentiable raf.op.moe_encode_batch_prioritized (same gradient as moe_encode, src/op/grad/moe.cc:58)."""
    return _MoeEncode.apply(data, gate, None, float(capacity_factor), (int(n_partitions), int(partition_id)), 1,
                            bool(gate_is_logits), None, None)


def moe_decode(data, gate, indices_locations, top_k=1):
    """Differentiable raf.op.moe_decode: gradients flow to data (expert outputs) and to gate (gates_s)."""
    return _MoeDecode.apply(data, gate, indices_locations, int(top_k))

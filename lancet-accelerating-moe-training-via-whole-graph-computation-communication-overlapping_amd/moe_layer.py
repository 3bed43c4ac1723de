"""The MoE layer that calls the dispatch path, with the reference's module names (models/benchmark/pytorch/utils.py:
Gate :565-573, Experts :529-562, MOELayerImpl :576-634), on one GPU.

The reference's layer runs torch-CPU stand-ins of the operators (FakeMoeEncodeOp / FakeMoeDecodeOp, :313-501) and
an all-to-all on either side of the experts.  Here the operators are the HIP ones, differentiated through the
gradient rules of grad.py; with one GPU in the job the all-to-all is the identity (world_size = 1), so the
dispatched buffer [E, C, M] goes to the experts as [1, E, C, M] and comes back the same way.
"""
import copy

import torch
import torch.nn.functional as F

from . import grad


class Gate(torch.nn.Module):
    """Linear(model_dim, num_experts, bias=False) + softmax over the experts, in fp32 (the op takes an fp32 gate).
    softmax=False leaves the logits to the operator, which then runs the softmax itself, fused into its selection
    (MOELayerImpl(fused_softmax=True))."""

    def __init__(self, model_dim, num_experts, softmax=True):
        super().__init__()
        self.wg = torch.nn.Linear(model_dim, num_experts, bias=False)
        self.softmax = softmax

    def forward(self, input):
        logits = self.wg(input).float()
        return F.softmax(logits, dim=1) if self.softmax else logits


class Experts(torch.nn.Module):
    """num_local_experts copies of `expert`; input and output [world_size, num_local_experts, C, M]."""

    def __init__(self, expert, world_size, hidden_size, num_local_experts=1):
        super().__init__()
        self.experts = torch.nn.ModuleList([copy.deepcopy(expert) for _ in range(num_local_experts)])
        self.num_local_experts = num_local_experts
        self.world_size = world_size
        self.hidden_size = hidden_size
        for e in self.experts:
            for _, param in e.named_parameters():
                param.allreduce = False          # expert parameters are not data-parallel (utils.py:541-544)

    def forward(self, inputs):
        outs = []
        for chunk, expert in zip(inputs.chunk(self.num_local_experts, dim=1), self.experts):
            G, _, C, M = chunk.shape
            out = expert(chunk.reshape(G * C, M))
            if isinstance(out, tuple):
                out = out[0]
            outs.append(out.reshape(G, 1, C, self.hidden_size))
        return torch.cat(outs, dim=1)


class MOELayerImpl(torch.nn.Module):
    """gate -> moe_encode -> experts -> moe_decode (GShard Algorithm 2 as the reference lays it out, :585-634).
    top_k = 2 routes every token to two experts with GShard's normalised combine weights
    (docker/resources/sharded_moe.py:253-324, no second-choice noise); fused_softmax=True expects a gate module that
    returns logits (Gate(..., softmax=False))."""

    def __init__(self, gate, experts, world_size=1, num_local_experts=1, capacity_factor=1.0, top_k=1,
                 fused_softmax=False):
        super().__init__()
        if world_size != 1:
            raise ValueError("one GPU per job here: the all-to-all on either side of the experts is not built")
        if top_k not in (1, 2):
            raise ValueError("top_k must be 1 or 2")
        self.gate = gate
        self.experts = experts
        self.world_size = world_size
        self.num_local_experts = num_local_experts
        self.capacity_factor = capacity_factor
        self.top_k = top_k
        self.fused_softmax = fused_softmax

    def forward(self, input_tensor):
        d_model = input_tensor.shape[-1]
        reshaped_input = input_tensor.reshape(-1, d_model)
        gate_weights = self.gate(reshaped_input)
        gates_s, indices_locations, _, _, dispatched_input = grad.moe_encode(
            reshaped_input.contiguous(), gate_weights, None, self.capacity_factor, top_k=self.top_k,
            gate_is_logits=self.fused_softmax)
        dispatched_input = dispatched_input.reshape(self.world_size, self.num_local_experts, -1, d_model)
        expert_output = self.experts(dispatched_input)
        expert_output = expert_output.reshape(self.world_size * self.num_local_experts, -1, d_model).contiguous()
        combined_output = grad.moe_decode(expert_output, gates_s, indices_locations, top_k=self.top_k)
        return combined_output.reshape(input_tensor.shape)

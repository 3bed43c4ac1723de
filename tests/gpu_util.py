"""Helpers shared by the GPU parity tests: seeded inputs in the shapes BASELINE.json names and
conversions between NumPy (oracle side) and torch GPU tensors (HIP side)."""
import numpy as np
import torch

from oracle import moe_oracle as mo

TORCH_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def make_inputs(seed, S, M, E, logit_scale=1.0, zipf_bias=False, ties=False):
    """data ~ N(0,1) fp32 [S,M]; logits ~ scale*N(0,1) (+ per-expert Zipf(1.2) bias scaled to [0,3])."""
    rng = np.random.default_rng(seed)
    data = rng.standard_normal((S, M), dtype=np.float32)
    logits = (rng.standard_normal((S, E), dtype=np.float32) * np.float32(logit_scale)).astype(np.float32)
    if zipf_bias:
        r = np.arange(1, E + 1, dtype=np.float64)
        bias = 3.0 * (r ** -1.2 - E ** -1.2) / (1.0 - E ** -1.2) if E > 1 else np.zeros(1)
        logits = (logits + bias[rng.permutation(E)].astype(np.float32)[None, :]).astype(np.float32)
    if ties:
        logits = (np.round(logits * 2) / 2).astype(np.float32)
    return data, logits


def rows_to_torch(data_f32, dt):
    """fp32 host rows -> GPU tensor of storage type dt (round to nearest even)."""
    return torch.from_numpy(data_f32).cuda().to(TORCH_DT[dt])


def rows_as_oracle(data_f32, dt):
    """The values the GPU tensor of rows_to_torch holds, as fp32 NumPy."""
    if dt == "f32":
        return data_f32
    if dt == "bf16":
        return mo.round_to_bf16(data_f32)
    return data_f32.astype(np.float16).astype(np.float32)


def to_np(t):
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.float().cpu().numpy()
    if t.dtype == torch.uint64:
        return t.view(torch.int64).cpu().numpy().astype(np.uint64)
    return t.cpu().numpy()


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def ulp_distance(a, b):
    """Largest distance between two 16-bit float GPU tensors of one dtype, in units of the last place (the
    sign-magnitude bit patterns mapped to integers in value order)."""
    x, y = a.view(torch.int16).to(torch.int32), b.view(torch.int16).to(torch.int32)
    x = torch.where(x < 0, -(x & 0x7fff), x)
    y = torch.where(y < 0, -(y & 0x7fff), y)
    return int((x - y).abs().max()) if x.numel() else 0

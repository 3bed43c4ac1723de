"""The RAF operators of the dispatch/optimizer path (six forward ops, four MoE backward ops) over
torch tensors on the GPU.

Names, positional argument order and defaults follow the reference's schemas
(scripts/src_codegen/def_schema.py:642-698, 726-742); output tuples follow
src/op/declare/moe.cc.  Extensions are trailing keyword arguments only (top_k,
gate_is_logits, workspace, out).  torch supplies device memory and the current
stream; all computation is done by the HIP kernels behind the C ABI.
"""
import ctypes as C
import functools
import os

import torch

from . import capi

_DTYPES = {torch.float32: capi.F32, torch.bfloat16: capi.BF16, torch.float16: capi.F16}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Handle of the current device's current stream, as the integer a void* argument takes.  A small call costs
    about as much on the host as on the device, so this goes straight to torch's C entry points where they exist."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    """Device address of a tensor (None = null pointer); the typed entry points of capi take it as void*."""
    return t.data_ptr() if t is not None else None


def _dtype_code(t):
    if t.dtype not in _DTYPES:
        raise TypeError("token rows must be float32, bfloat16 or float16, got %s" % t.dtype)
    return _DTYPES[t.dtype]


def _gate_code(t, name="gate"):
    """Gate arrays (gate, gate2_noise, gates_s and their gradients) are float32, or a half type as a
    mixed-precision graph has them (python/raf/amp/type_hints.py:97,105); arithmetic on them is fp32."""
    if t.dtype not in _DTYPES:
        raise TypeError("%s must be float32, bfloat16 or float16, got %s" % (name, t.dtype))
    return _DTYPES[t.dtype]


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _dev(t, name):
    _need(t.is_cuda, "%s must live on the GPU" % name)
    _need(t.is_contiguous(), "%s must be contiguous" % name)


def _workspace(nbytes, device, given):
    if given is not None:
        _need(given.is_cuda and given.dtype == torch.uint8 and given.numel() >= nbytes,
              "workspace must be a uint8 GPU tensor of at least %d bytes" % nbytes)
        return given
    return torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device=device)


class ScanWorkspace:
    """Device memory of the position scan (moe_encode, moe_route, moe_encode_batch_prioritized, gen_location).

    The scan keeps a few words of state in its workspace from call to call (launch epoch, ticket), so that no
    call spends a launch on clearing it: the memory is set up once, here, on the current stream, and every call
    leaves it ready for the next.  One workspace serves one call at a time: calls that may overlap (different
    streams) need a workspace each.  No counterpart in the reference, whose scan kernel keeps no state
    (tutel_moe_dispatch.cu:164-212)."""

    def __init__(self, nbytes, device="cuda"):
        nbytes = (max(int(nbytes), 8192) + 7) // 8 * 8
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        capi.check(capi.load().lancet_scan_workspace_init(_p(self.buf), nbytes, _stream()), "lancet_scan_workspace_init")

    @property
    def nbytes(self):
        return self.buf.numel()

    def error(self):
        """1 when a call on this workspace gave up a wait (its outputs then hold -1 for the tokens concerned and
        for used_capacity) since the last read, else 0; synchronises the current stream and clears the word."""
        err = C.c_int(0)
        capi.check(capi.load().lancet_scan_workspace_error(_p(self.buf), _stream(), C.byref(err)),
                   "lancet_scan_workspace_error")
        return int(err.value)


_scan_pool = {}


def _scan_workspace(nbytes, device, given):
    """The workspace a scan call uses: the caller's ScanWorkspace, or one kept per (device, stream) and grown on
    demand (calls on one stream run one after the other, so they can share)."""
    if given is not None:
        if not isinstance(given, ScanWorkspace):
            raise TypeError("workspace of a scan call must be an ops.ScanWorkspace (it is set up once and carries "
                            "state from call to call), got %s" % type(given).__name__)
        _need(given.buf.device == device and given.nbytes >= nbytes,
              "workspace must live on the data's GPU and hold at least %d bytes" % nbytes)
        return given
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, _raw_stream(idx) if _raw_stream is not None else torch.cuda.current_stream(device).cuda_stream)
    ws = _scan_pool.get(key)
    if ws is None or ws.nbytes < nbytes:
        with torch.cuda.device(device):
            ws = ScanWorkspace(max(int(nbytes), 1 << 16), device)
        _scan_pool[key] = ws
    return ws


def scan_errors():
    """Number of scan workspaces kept by this module on which a wait gave up since the last check
    (synchronises).  The reference aborts on any failure (src/common/cuda_utils.h:18-22); here the outputs of a
    failed call hold -1 and this is the check a caller makes where it synchronises anyway."""
    return sum(ws.error() for ws in list(_scan_pool.values()))


@functools.lru_cache(maxsize=256)
def moe_capacity(S, E, capacity_factor):
    """C = int(float(cf) * ceil(S / E)) (src/op/dialect/cuda/moe.cc:107-109)."""
    return int(capi.load().lancet_moe_capacity(int(S), int(E), float(capacity_factor)))


def _check_encode_inputs(data, gate):
    _dev(data, "data"), _dev(gate, "gate")
    _need(data.dim() == 2, "Expected input data to be 2D.")
    _need(gate.dim() == 2, "Expected input gate to be 2D.")
    _need(data.shape[0] == gate.shape[0], "Input data and gate should have matching shape in dim 0.")
    _gate_code(gate)
    return _dtype_code(data)


@functools.lru_cache(maxsize=256)
def moe_encode_workspace_bytes(S, E, top_k=1):
    return int(capi.load().lancet_moe_encode_workspace_bytes(int(S), int(E), int(top_k)))


def _flags(gate_is_logits, zero_tail, rows_at_used=False, scan_lookback=False):
    return ((capi.GATE_IS_LOGITS if gate_is_logits else 0) | (0 if zero_tail else capi.NO_TAIL_ZERO) |
            (capi.ROWS_AT_USED if rows_at_used else 0) | (capi.SCAN_LOOKBACK if scan_lookback else 0))


def _check_noise(gate2_noise, gate, top_k):
    if gate2_noise is None:
        return
    _dev(gate2_noise, "gate2_noise")
    _need(top_k == 2, "gate2_noise only exists for the second choice (top_k = 2)")
    _need(gate2_noise.shape == gate.shape and gate2_noise.dtype == gate.dtype, "gate2_noise must have the gate's shape and dtype")


def moe_encode(data, gate, used_capacity, capacity_factor=1.0, top_k=1, gate_is_logits=False,
               zero_tail=True, gate2_noise=None, rows_at_used=False, workspace=None, out=None, capacity=None,
               scan_lookback=False):
    """raf.op.moe_encode(data, gate, used_capacity, capacity_factor=1.0).

    Returns (gates_s [k*S] f32, indices_locations [2, k*S] i32, used_capacity [E] i32,
    elements_per_expert [E] u64, dispatched [E, C, M]).  With top_k = 2 the capacity follows
    GShard: capacity_factor is doubled before the reference formula is applied; gate2_noise [S, E], if
    given, is added to the gate for the second choice alone (the Gumbel noise of
    docker/resources/sharded_moe.py:275, drawn by the caller).  rows_at_used=True writes the rows of expert e
    from row used_capacity[e] on: chained partition encodes that pass the same `dispatched` buffer (out=) fill
    it the way moe_redispatch would, the last one with zero_tail=True, the others without.  zero_tail=False
    leaves rows past the used capacity unwritten (partition buffers that only feed moe_redispatch).
    capacity, if given, is used as it is instead of the reference formula: GShard's own top-2 capacity is
    ceil(2 * S / E * capacity_factor) (docker/resources/sharded_moe.py:267), which differs from
    int(2 * capacity_factor * ceil(S / E)) when E does not divide S or the factor is fractional
    (S = 300, E = 8, factor 1: 75 against 76).  scan_lookback=True runs the position scan as one kernel with a
    look-back between its tiles whatever the size (LANCET_SCAN_LOOKBACK)."""
    lib = capi.load()
    dt = _check_encode_inputs(data, gate)
    S, M = data.shape
    E = gate.shape[1]
    _need(top_k in (1, 2), "top_k must be 1 or 2")
    _check_noise(gate2_noise, gate, top_k)
    cf = float(capacity_factor) * (2.0 if top_k == 2 else 1.0)
    Cap = moe_capacity(S, E, cf) if capacity is None else int(capacity)
    _need(Cap >= 0, "capacity must not be negative")
    if used_capacity is not None:
        _dev(used_capacity, "used_capacity")
        _need(used_capacity.dim() == 1 and used_capacity.numel() == E and used_capacity.dtype == torch.int32,
              "Input used_capacity should be 1-D int32 of length E.")
    dev = data.device
    if out is None:
        gates_s = torch.empty(top_k * S, dtype=gate.dtype, device=dev)
        indloc = torch.empty((2, top_k * S), dtype=torch.int32, device=dev)
        used_out = torch.empty(E, dtype=torch.int32, device=dev)
        elems = torch.empty(E, dtype=torch.int64, device=dev)
        disp = torch.empty((E, Cap, M), dtype=data.dtype, device=dev)
    else:
        gates_s, indloc, used_out, elems, disp = out
    ws = _scan_workspace(moe_encode_workspace_bytes(S, E, top_k), dev, workspace)
    _need(gates_s.dtype == gate.dtype, "gates_s takes the gate's dtype")
    st = lib.lancet_moe_encode(_p(data), _p(gate), _p(gate2_noise), _p(used_capacity), S, M, E, Cap, top_k, dt,
                               _gate_code(gate), _flags(gate_is_logits, zero_tail, rows_at_used, scan_lookback), _p(gates_s), _p(indloc),
                               _p(used_out), _p(elems), _p(disp), _p(ws.buf), ws.nbytes, _stream())
    capi.check(st, "lancet_moe_encode")
    return gates_s, indloc, used_out, elems.view(torch.uint64) if elems.dtype == torch.int64 else elems, disp


def moe_route(gate, used_capacity, M, capacity_factor=1.0, top_k=1, gate_is_logits=False, gate2_noise=None,
              workspace=None, out=None, capacity=None, scan_lookback=False):
    """The routing half of moe_encode (selection + position scan, src/op/dialect/cuda/moe.cc:366-380), so that
    a caller can run it ahead of, or beside, the row movement of another partition.  M only scales
    elements_per_expert.  Returns (gates_s, indices_locations, used_capacity, elements_per_expert)."""
    lib = capi.load()
    _dev(gate, "gate")
    _need(gate.dim() == 2, "gate must be 2-D")
    gd = _gate_code(gate)
    S, E = gate.shape
    _need(top_k in (1, 2), "top_k must be 1 or 2")
    _check_noise(gate2_noise, gate, top_k)
    Cap = moe_capacity(S, E, float(capacity_factor) * (2.0 if top_k == 2 else 1.0)) if capacity is None else int(capacity)
    dev = gate.device
    if out is None:
        out = (torch.empty(top_k * S, dtype=gate.dtype, device=dev),
               torch.empty((2, top_k * S), dtype=torch.int32, device=dev),
               torch.empty(E, dtype=torch.int32, device=dev), torch.empty(E, dtype=torch.int64, device=dev))
    gates_s, indloc, used_out, elems = out[:4]
    ws = _scan_workspace(moe_encode_workspace_bytes(S, E, top_k), dev, workspace)
    _need(gates_s.dtype == gate.dtype, "gates_s takes the gate's dtype")
    st = lib.lancet_moe_route(_p(gate), _p(gate2_noise), _p(used_capacity), S, int(M), E, Cap, top_k, gd, _flags(gate_is_logits, True, False, scan_lookback),
                              _p(gates_s), _p(indloc), _p(used_out), _p(elems), _p(ws.buf), ws.nbytes, _stream())
    capi.check(st, "lancet_moe_route")
    return gates_s, indloc, used_out, elems


def moe_scatter(data, indices_locations, used_in, used_out, n_experts, capacity, top_k=1, zero_tail=True,
                rows_at_used=False, out=None):
    """The row-movement half of moe_encode (launch_encode_forward, moe.cc:381-395) on routing produced by
    moe_route: returns dispatched [E, C, M]."""
    lib = capi.load()
    _dev(data, "data")
    _need(data.dim() == 2, "Expected input data to be 2D.")
    S = _check_indloc(indices_locations, top_k)
    _need(S == data.shape[0], "indices_locations and data disagree on the token count")
    M = data.shape[1]
    if out is None:
        out = torch.empty((n_experts, capacity, M), dtype=data.dtype, device=data.device)
    st = lib.lancet_moe_scatter(_p(data), _p(indices_locations), _p(used_in), _p(used_out), S, M, int(n_experts),
                                int(capacity), top_k, _dtype_code(data), _flags(False, zero_tail, rows_at_used), _p(out),
                                _stream())
    capi.check(st, "lancet_moe_scatter")
    return out


def moe_scatter_tokens(data, indices_locations, used_in, used_out, token_first, n_experts, capacity, top_k=1,
                       zero_tail=True, out=None):
    """Row movement of tokens [token_first, token_first + len(data)) of a whole-batch routing
    (moe_route over all S_total tokens): data holds the rows of those tokens, `out` is the whole [E, C, M]
    buffer and the rows go to their final places.  The calls of all token ranges together give the buffer of
    one moe_encode over the batch; one of them passes zero_tail=True, the others False.  used_in / used_out are
    what the routing call took and returned (used_in None = zeros)."""
    lib = capi.load()
    _dev(data, "data")
    _need(data.dim() == 2, "Expected input data to be 2D.")
    S_total = _check_indloc(indices_locations, top_k)
    n, M = data.shape
    _need(0 <= token_first and token_first + n <= S_total, "token range outside the routed batch")
    if out is None:
        out = torch.empty((n_experts, capacity, M), dtype=data.dtype, device=data.device)
    st = lib.lancet_moe_scatter_tokens(_p(data), _p(indices_locations), _p(used_in), _p(used_out), S_total, int(token_first), n, M,
                                       int(n_experts), int(capacity), top_k, _dtype_code(data),
                                       _flags(False, zero_tail), _p(out), _stream())
    capi.check(st, "lancet_moe_scatter_tokens")
    return out


def moe_decode_tokens(data, gate, indices_locations, token_first, n_tokens, top_k=1, out=None):
    """moe_decode of tokens [token_first, token_first + n_tokens) of a whole-batch routing: gate [k*S_total] and
    indices_locations [2, k*S_total] cover the batch, the result is [n_tokens, M]."""
    lib = capi.load()
    _dev(data, "data"), _dev(gate, "gate")
    _need(data.dim() == 3, "Expected input data to be 3D.")
    _need(gate.dim() == 1, "gate must be 1-D")
    S_total = _check_indloc(indices_locations, top_k)
    _need(gate.shape[0] == top_k * S_total, "gate and indices_locations disagree on the token count")
    _need(0 <= token_first and 0 <= n_tokens and token_first + n_tokens <= S_total, "token range outside the routed batch")
    E, Cap, M = data.shape
    if out is None:
        out = torch.empty((n_tokens, M), dtype=data.dtype, device=data.device)
    st = lib.lancet_moe_decode_tokens(_p(data), _p(gate), _p(indices_locations), S_total, int(token_first),
                                      int(n_tokens), M, E, Cap, top_k, _dtype_code(data), _gate_code(gate), _p(out), _stream())
    capi.check(st, "lancet_moe_decode_tokens")
    return out


@functools.lru_cache(maxsize=256)
def moe_encode_bpr_workspace_bytes(S0, E, n_partitions=1):
    return int(capi.load().lancet_moe_encode_bpr_workspace_bytes(int(S0), int(E), int(n_partitions)))


def moe_encode_batch_prioritized(data, gate, n_partitions=1, partition_id=0, capacity_factor=1.0,
                                 gate_is_logits=False, zero_tail=True, workspace=None, out=None, scan_lookback=False):
    """raf.op.moe_encode_batch_prioritized(data, gate, n_partitions=1, partition_id=0,
    capacity_factor=1.0): data/gate are the whole batch, the outputs cover partition
    partition_id (S = S0 / n_partitions tokens)."""
    lib = capi.load()
    dt = _check_encode_inputs(data, gate)
    S0, M = data.shape
    E = gate.shape[1]
    _need(n_partitions > 0, "n_partitions should be greater than 0.")
    _need(0 <= partition_id < n_partitions, "partition_id should be less than n_partitions.")
    S = S0 // n_partitions
    Cap = moe_capacity(S, E, capacity_factor)
    dev = data.device
    if out is None:
        gates_s = torch.empty(S, dtype=gate.dtype, device=dev)
        indloc = torch.empty((2, S), dtype=torch.int32, device=dev)
        used_out = torch.empty(E, dtype=torch.int32, device=dev)
        elems = torch.empty(E, dtype=torch.int64, device=dev)
        disp = torch.empty((E, Cap, M), dtype=data.dtype, device=dev)
    else:
        gates_s, indloc, used_out, elems, disp = out
    ws = _scan_workspace(moe_encode_bpr_workspace_bytes(S0, E, n_partitions), dev, workspace)
    _need(gates_s.dtype == gate.dtype, "gates_s takes the gate's dtype")
    st = lib.lancet_moe_encode_bpr(_p(data), _p(gate), S0, M, E, Cap, n_partitions, partition_id, dt, _gate_code(gate),
                                   _flags(gate_is_logits, zero_tail, False, scan_lookback), _p(gates_s), _p(indloc),
                                   _p(used_out), _p(elems), _p(disp), _p(ws.buf), ws.nbytes, _stream())
    capi.check(st, "lancet_moe_encode_bpr")
    return gates_s, indloc, used_out, elems.view(torch.uint64) if elems.dtype == torch.int64 else elems, disp


def moe_decode(data, gate, indices_locations, top_k=1, out=None):
    """raf.op.moe_decode(data [E,C,M], gate [k*S], indices_locations [2, k*S]) -> [S, M]."""
    lib = capi.load()
    _dev(data, "data"), _dev(gate, "gate"), _dev(indices_locations, "indices_locations")
    _need(data.dim() == 3, "Expected input data to be 3D.")
    _need(gate.dim() == 1, "Expected input gate to be 1D.")
    gd = _gate_code(gate)
    _need(indices_locations.dtype == torch.int32 and indices_locations.dim() == 2 and
          indices_locations.shape[0] == 2 and indices_locations.shape[1] == gate.shape[0],
          "indices_locations must be int32 [2, k*S]")
    dt = _dtype_code(data)
    E, Cap, M = data.shape
    _need(gate.shape[0] % top_k == 0, "gate length must be a multiple of top_k")
    S = gate.shape[0] // top_k
    if out is None:
        out = torch.empty((S, M), dtype=data.dtype, device=data.device)
    st = lib.lancet_moe_decode(_p(data), _p(gate), _p(indices_locations), S, M, E, Cap, top_k, dt, gd, _p(out),
                               _stream())
    capi.check(st, "lancet_moe_decode")
    return out


def _check_indloc(indices_locations, top_k):
    _dev(indices_locations, "indices_locations")
    _need(indices_locations.dtype == torch.int32 and indices_locations.dim() == 2 and indices_locations.shape[0] == 2,
          "indices_locations must be int32 [2, k*S]")
    _need(top_k in (1, 2) and indices_locations.shape[1] % top_k == 0, "top_k must be 1 or 2 and divide the mask length")
    return indices_locations.shape[1] // top_k


def moe_encode_dx(dy, indices_locations, top_k=1, out=None):
    """raf.op.moe_encode_dx(dy [E,C,M], indices_locations [2, k*S]) -> [S, M]."""
    lib = capi.load()
    _dev(dy, "dy")
    _need(dy.dim() == 3, "Input dy should be 3-D.")
    S = _check_indloc(indices_locations, top_k)
    E, Cap, M = dy.shape
    if out is None:
        out = torch.empty((S, M), dtype=dy.dtype, device=dy.device)
    st = lib.lancet_moe_encode_dx(_p(dy), _p(indices_locations), S, M, E, Cap, top_k, _dtype_code(dy), _p(out), _stream())
    capi.check(st, "lancet_moe_encode_dx")
    return out


def moe_encode_dg(dy, indices_locations, n_experts, top_k=1, out=None):
    """raf.op.moe_encode_dg(dy [k*S], indices_locations, n_experts) -> [S, E] of dy's dtype."""
    lib = capi.load()
    _dev(dy, "dy")
    _need(dy.dim() == 1, "Input dy should be 1-D.")
    S = _check_indloc(indices_locations, top_k)
    _need(dy.shape[0] == top_k * S, "dy and indices_locations disagree")
    if out is None:
        out = torch.empty((S, n_experts), dtype=dy.dtype, device=dy.device)
    _need(out.dtype == dy.dtype, "the gate gradient takes dy's dtype")
    st = lib.lancet_moe_encode_dg(_p(dy), _p(indices_locations), S, n_experts, top_k, _gate_code(dy, "dy"), _p(out), _stream())
    capi.check(st, "lancet_moe_encode_dg")
    return out


def moe_encode_dgate(dy, gate, indices_locations, top_k=1, gate_is_logits=False, out=None):
    """Gate gradient of moe_encode(..., top_k, gate_is_logits) as a whole: dy [k*S] is the gradient of the op's output
    gates_s, gate [S, E] the op's gate input, the result [S, E] the gradient with respect to that input, through the
    top-2 normalisation (docker/resources/sharded_moe.py:304-312) and, with gate_is_logits, the fused softmax.  With
    top_k = 1 on probabilities it is moe_encode_dg (src/op/grad/moe.cc:30-58)."""
    lib = capi.load()
    _dev(dy, "dy"), _dev(gate, "gate")
    _need(dy.dim() == 1 and gate.dim() == 2, "dy must be 1-D and gate 2-D")
    S = _check_indloc(indices_locations, top_k)
    _need(dy.shape[0] == top_k * S and gate.shape[0] == S, "dy, gate and indices_locations disagree")
    _need(dy.dtype == gate.dtype, "dy takes the gate's dtype")
    if out is None:
        out = torch.empty_like(gate)
    _need(out.dtype == gate.dtype and out.shape == gate.shape and out.is_contiguous(), "the gradient has the gate's shape and dtype")
    st = lib.lancet_moe_encode_dgate(_p(dy), _p(gate), _p(indices_locations), S, gate.shape[1], top_k, _gate_code(gate),
                                     capi.GATE_IS_LOGITS if gate_is_logits else 0, _p(out), _stream())
    capi.check(st, "lancet_moe_encode_dgate")
    return out


def moe_decode_dx(dy, gate, indices_locations, n_experts, capacity, top_k=1, workspace=None, out=None):
    """raf.op.moe_decode_dx(dy [S,M], gate [k*S], indices_locations, n_experts, capacity) -> [E, C, M]."""
    lib = capi.load()
    _dev(dy, "dy"), _dev(gate, "gate")
    _need(dy.dim() == 2, "Input dy should be 2-D.")
    _need(gate.dim() == 1, "gate must be 1-D")
    S = _check_indloc(indices_locations, top_k)
    _need(dy.shape[0] == S and gate.shape[0] == top_k * S, "dy, gate and indices_locations disagree")
    M = dy.shape[1]
    if out is None:
        out = torch.empty((n_experts, capacity, M), dtype=dy.dtype, device=dy.device)
    ws_bytes = int(lib.lancet_moe_decode_dx_workspace_bytes(n_experts, capacity))
    ws = _workspace(ws_bytes, dy.device, workspace)
    st = lib.lancet_moe_decode_dx(_p(dy), _p(gate), _p(indices_locations), S, M, n_experts, capacity, top_k,
                                  _dtype_code(dy), _gate_code(gate), _p(out), _p(ws), ws.numel(), _stream())
    capi.check(st, "lancet_moe_decode_dx")
    return out


def moe_decode_dg(dy, data, indices_locations, top_k=1, gate_dtype=torch.float32, out=None):
    """raf.op.moe_decode_dg(dy [S,M], data [E,C,M], indices_locations) -> [k*S] of gate_dtype (the dtype of the
    gates_s the gradient belongs to; the reference gives it dy's dtype, src/op/declare/moe.cc:239)."""
    lib = capi.load()
    _dev(dy, "dy"), _dev(data, "data")
    _need(dy.dim() == 2 and data.dim() == 3 and dy.dtype == data.dtype and dy.shape[1] == data.shape[2],
          "dy must be [S,M] and data [E,C,M] of one dtype")
    S = _check_indloc(indices_locations, top_k)
    _need(dy.shape[0] == S, "dy and indices_locations disagree")
    E, Cap, M = data.shape
    if out is None:
        out = torch.empty(top_k * S, dtype=gate_dtype, device=dy.device)
    st = lib.lancet_moe_decode_dg(_p(dy), _p(data), _p(indices_locations), S, M, E, Cap, top_k, _dtype_code(dy),
                                  _gate_code(out, "the gate gradient"), _p(out), _stream())
    capi.check(st, "lancet_moe_decode_dg")
    return out


def moe_top2_normalize_gates(raw_gates, merged_indices_locations):
    """Combine weights of the top-2 extension from per-slot raw gate values [2S] and the merged
    indices_locations [2, 2S]."""
    lib = capi.load()
    S = raw_gates.shape[0] // 2
    out = torch.empty_like(raw_gates)
    st = lib.lancet_moe_top2_normalize_gates(_p(raw_gates), _p(merged_indices_locations), S, _gate_code(raw_gates, "raw_gates"),
                                             _p(out), _stream())
    capi.check(st, "lancet_moe_top2_normalize_gates")
    return out


def moe_merge_masks(indices_locations, n_experts, workspace=None, out=None):
    """raf.op.moe_merge_masks(indices_locations: tuple of [2,S], n_experts) -> [2, P*S]."""
    lib = capi.load()
    P = len(indices_locations)
    _need(P >= 1, "need at least one partition")
    for il in indices_locations:
        _dev(il, "indices_locations")
        _need(il.dim() == 2 and il.shape == indices_locations[0].shape and il.dtype == torch.int32,
              "Expected input indices_locations to be 2D int32 of equal shape.")
    S = indices_locations[0].shape[1]
    dev = indices_locations[0].device
    if out is None:
        out = torch.empty((2, P * S), dtype=torch.int32, device=dev)
    ws_bytes = int(lib.lancet_moe_merge_masks_workspace_bytes(P, n_experts))
    ws = _workspace(ws_bytes, dev, workspace)
    ptrs = capi.ptr_array([il.data_ptr() for il in indices_locations])
    st = lib.lancet_moe_merge_masks(ptrs, P, S, n_experts, _p(out), _p(ws), ws.numel(), _stream())
    capi.check(st, "lancet_moe_merge_masks")
    return out


def moe_redispatch(data, indices_locations, workspace=None, out=None):
    """raf.op.moe_redispatch(data: tuple of [E,C,M], indices_locations: tuple of [2,S]) -> [E,C,M]."""
    lib = capi.load()
    P = len(indices_locations)
    _need(P >= 1 and len(data) == P, "data and indices_locations must have one entry per partition")
    for d in data:
        _dev(d, "data")
        _need(d.dim() in (3, 4) and d.shape == data[0].shape and d.dtype == data[0].dtype,
              "Expected input data to be 3 or 4D of equal shape.")
    for il in indices_locations:
        _dev(il, "indices_locations")
        _need(il.dim() == 2 and il.dtype == torch.int32, "Expected input indices_locations to be 2D.")
    shape = tuple(data[0].shape)
    if len(shape) == 4:   # [G, LE, C, M]
        E, Cap, M = shape[0] * shape[1], shape[2], shape[3]
    else:
        E, Cap, M = shape
    S = indices_locations[0].shape[1]
    dt = _dtype_code(data[0])
    dev = data[0].device
    if out is None:
        out = torch.empty(shape, dtype=data[0].dtype, device=dev)
    ws_bytes = int(lib.lancet_moe_redispatch_workspace_bytes(P, E))
    ws = _workspace(ws_bytes, dev, workspace)
    dptrs = capi.ptr_array([d.data_ptr() for d in data])
    iptrs = capi.ptr_array([il.data_ptr() for il in indices_locations])
    st = lib.lancet_moe_redispatch(dptrs, iptrs, P, S, M, Cap, E, dt, _p(out), _p(ws), ws.numel(), _stream())
    capi.check(st, "lancet_moe_redispatch")
    return out


def moe_redispatch_expert_input(data, recv_cnts, local_expert_id, n_local_experts, recv_cnts_scale=1, out=None):
    """raf.op.moe_redispatch_expert_input(data: tuple, recv_cnts: tuple, local_expert_id, n_local_experts,
    recv_cnts_scale=1): data[p] is [C, G, M] (or [C, 1, G, M] / [C*G, M]), recv_cnts[p] uint64 [G*LE]."""
    lib = capi.load()
    P = len(data)
    _need(P >= 1 and len(recv_cnts) == P, "data and recv_cnts must have one entry per partition")
    for d in data:
        _dev(d, "data")
        _need(d.shape == data[0].shape and d.dtype == data[0].dtype, "partition buffers must agree")
    for c in recv_cnts:
        _dev(c, "recv_cnts")
        _need(c.dim() == 1 and c.dtype in (torch.int64, getattr(torch, "uint64", torch.int64)) and
              c.shape == recv_cnts[0].shape, "Expected recv_cnts to be 1-D 64-bit counts of equal length.")
    shape = tuple(data[0].shape)
    n = recv_cnts[0].shape[0]
    _need(n % n_local_experts == 0, "recv_cnts length must be G x n_local_experts")
    if len(shape) == 4:      # [C, 1, G, M]
        _need(shape[1] == 1, "4D Input data should have dim 1 at axis 1.")
        Cap, G, M = shape[0], shape[2], shape[3]
    elif len(shape) == 3:    # [C, G, M]
        Cap, G, M = shape
    else:                    # [C x G, M]
        _need(len(shape) == 2, "Input data should be 2,3 or 4-D.")
        G = n // n_local_experts
        Cap, M = shape[0] // G, shape[1]
    _need(n // G == n_local_experts, "Expected input recv_cnts to be 1D of size G x LE.")
    if out is None:
        out = torch.empty(shape, dtype=data[0].dtype, device=data[0].device)
    dptrs = capi.ptr_array([d.data_ptr() for d in data])
    cptrs = capi.ptr_array([c.data_ptr() for c in recv_cnts])
    st = lib.lancet_moe_redispatch_expert_input(dptrs, cptrs, P, int(local_expert_id), int(n_local_experts), Cap, M, G,
                                                int(recv_cnts_scale), _dtype_code(data[0]), _p(out), _stream())
    capi.check(st, "lancet_moe_redispatch_expert_input")
    return out


def _sparse_copy_args(buf, packed, nelements_per_dim, nelements_stride, nelements_offset, axis):
    _dev(buf, "sparse buffer"), _dev(packed, "packed array"), _dev(nelements_per_dim, "nelements_per_dim")
    _need(buf.dim() == 3, "the sparse buffer must be 3-D")
    _need(axis in (0, 1), "Axis %d not supported." % axis)
    _need(buf.dtype == packed.dtype and buf.is_contiguous() and packed.is_contiguous(), "dtype / layout mismatch")
    _need(nelements_per_dim.dtype in (torch.int64, getattr(torch, "uint64", torch.int64)) and
          nelements_per_dim.is_contiguous(), "nelements_per_dim must be contiguous 64-bit counts")
    return tuple(buf.shape), packed.numel(), nelements_per_dim.numel()


def memcpy_sparse_to_cont_3d(src, dst, nelements_per_dim, nelements_stride=1, nelements_offset=0, axis=0,
                             scale_element_size_by=1, shrink_element_size_by=1):
    """launch_memcpy_sparse_to_cont_3d (src/op/dialect/cuda/kernels/sparse_memcpy.cu:62-85): packs the valid
    elements of every block along `axis` of src[dim0, dim1, dim2] into dst (written in place, returned)."""
    lib = capi.load()
    (d0, d1, d2), n_dst, n_cnt = _sparse_copy_args(src, dst, nelements_per_dim, nelements_stride, nelements_offset, axis)
    st = lib.lancet_memcpy_sparse_to_cont_3d(_p(src), _p(dst), _p(nelements_per_dim), n_cnt, int(nelements_stride),
                                             int(nelements_offset), int(axis), d0, d1, d2, n_dst,
                                             int(scale_element_size_by), int(shrink_element_size_by), _dtype_code(src),
                                             _stream())
    capi.check(st, "lancet_memcpy_sparse_to_cont_3d")
    return dst


def memcpy_cont_to_sparse_3d(src, dst, nelements_per_dim, nelements_stride=1, nelements_offset=0, axis=0,
                             scale_element_size_by=1, shrink_element_size_by=1, zero_tail=False):
    """launch_memcpy_cont_to_sparse_3d (sparse_memcpy.cu:62-85): the inverse; dst[dim0, dim1, dim2] is written in
    place.  zero_tail clears the part of every block the copy does not reach (the reference leaves it)."""
    lib = capi.load()
    (d0, d1, d2), n_src, n_cnt = _sparse_copy_args(dst, src, nelements_per_dim, nelements_stride, nelements_offset, axis)
    st = lib.lancet_memcpy_cont_to_sparse_3d(_p(src), _p(dst), _p(nelements_per_dim), n_cnt, int(nelements_stride),
                                             int(nelements_offset), int(axis), d0, d1, d2, n_src,
                                             int(scale_element_size_by), int(shrink_element_size_by), _dtype_code(dst),
                                             capi.ZERO_TAIL if zero_tail else 0, _stream())
    capi.check(st, "lancet_memcpy_cont_to_sparse_3d")
    return dst


def memcpy_sparse_ranges_to_cont_3d(src, dst, nelements_per_dim, starts_per_dim, nelements_stride=1, nelements_offset=0,
                                    axis=0):
    """memcpy_sparse_to_cont_3d on row ranges: block b contributes its elements [start_b, start_b + n_b) (both
    arrays indexed b*stride + offset).  Packs what one token partition owns inside a shared buffer."""
    lib = capi.load()
    (d0, d1, d2), n_dst, n_cnt = _sparse_copy_args(src, dst, nelements_per_dim, nelements_stride, nelements_offset, axis)
    _dev(starts_per_dim, "starts_per_dim")
    _need(starts_per_dim.dtype == nelements_per_dim.dtype and starts_per_dim.numel() == n_cnt and
          starts_per_dim.is_contiguous(), "starts_per_dim must match nelements_per_dim")
    st = lib.lancet_memcpy_sparse_ranges_to_cont_3d(_p(src), _p(dst), _p(nelements_per_dim), _p(starts_per_dim), n_cnt,
                                                    int(nelements_stride), int(nelements_offset), int(axis), d0, d1, d2,
                                                    n_dst, _dtype_code(src), _stream())
    capi.check(st, "lancet_memcpy_sparse_ranges_to_cont_3d")
    return dst


def memcpy_cont_to_sparse_ranges_3d(src, dst, nelements_per_dim, starts_per_dim, nelements_stride=1, nelements_offset=0,
                                    axis=0):
    """The inverse of memcpy_sparse_ranges_to_cont_3d: only the ranges are written."""
    lib = capi.load()
    (d0, d1, d2), n_src, n_cnt = _sparse_copy_args(dst, src, nelements_per_dim, nelements_stride, nelements_offset, axis)
    _dev(starts_per_dim, "starts_per_dim")
    _need(starts_per_dim.dtype == nelements_per_dim.dtype and starts_per_dim.numel() == n_cnt and
          starts_per_dim.is_contiguous(), "starts_per_dim must match nelements_per_dim")
    st = lib.lancet_memcpy_cont_to_sparse_ranges_3d(_p(src), _p(dst), _p(nelements_per_dim), _p(starts_per_dim), n_cnt,
                                                    int(nelements_stride), int(nelements_offset), int(axis), d0, d1, d2,
                                                    n_src, _dtype_code(dst), _stream())
    capi.check(st, "lancet_memcpy_cont_to_sparse_ranges_3d")
    return dst


def moe_partition_ranges(indices_locations, n_partitions, n_experts, M, top_k=1, workspace=None, out=None):
    """Row ranges of n_partitions equal token partitions inside a whole-batch routing: returns (starts, counts), each
    int64 [top_k * n_partitions, E] in elements (rows x M), rows ordered slot-major then partition."""
    lib = capi.load()
    S_total = _check_indloc(indices_locations, top_k)
    _need(n_partitions >= 1 and S_total % n_partitions == 0, "the token count must divide into n_partitions")
    Q = top_k * int(n_partitions)
    dev = indices_locations.device
    if out is None:
        out = (torch.empty((Q, n_experts), dtype=torch.int64, device=dev), torch.empty((Q, n_experts), dtype=torch.int64, device=dev))
    starts, counts = out
    ws = _workspace(lib.lancet_moe_partition_ranges_workspace_bytes(top_k, int(n_partitions), int(n_experts)), dev, workspace)
    st = lib.lancet_moe_partition_ranges(_p(indices_locations), S_total, top_k, int(n_partitions), int(n_experts), int(M),
                                         _p(starts), _p(counts), _p(ws), ws.numel(), _stream())
    capi.check(st, "lancet_moe_partition_ranges")
    return starts, counts


# ------------------------------------------------------------------------------------ LANS
class LansPlan:
    """Owns the native plan of one parameter set (what the reference's LansImpl constructor
    captures, src/op/dialect/cuda/lans.cc:28-83)."""

    def __init__(self, numels, schedule=None):
        lib = capi.load()
        self.numels = [int(n) for n in numels]
        arr = (C.c_int64 * len(self.numels))(*self.numels)
        handle = C.c_void_p()
        capi.check(lib.lancet_lans_plan_create(arr, len(self.numels), C.byref(handle)), "lancet_lans_plan_create")
        self._h = handle
        self._lib = lib
        if schedule is not None:
            self.set_schedule(schedule)

    def set_schedule(self, schedule):
        """capi.LANS_RESIDENT (what a new plan has when a tensor fits the resident kernel; raises on a plan
        with no such tensor) or capi.LANS_SWEEPS (no workgroup waits for another)."""
        capi.check(self._lib.lancet_lans_plan_set_schedule(self._h, int(schedule)), "lancet_lans_plan_set_schedule")

    def schedule(self):
        """The schedule the next step runs: capi.LANS_RESIDENT or capi.LANS_SWEEPS."""
        n = C.c_int(-1)
        capi.check(self._lib.lancet_lans_plan_schedule(self._h, C.byref(n)), "lancet_lans_plan_schedule")
        return n.value

    def resident_capacity(self):
        """(chunks the resident schedule holds at once, chunks of this plan's largest tensor)."""
        wg, mx = C.c_int(0), C.c_int(0)
        capi.check(self._lib.lancet_lans_plan_resident_capacity(self._h, C.byref(wg), C.byref(mx)),
                   "lancet_lans_plan_resident_capacity")
        return wg.value, mx.value

    def error(self):
        """Reads and clears the plan's sticky error (synchronises the current stream)."""
        err = C.c_int(-1)
        capi.check(self._lib.lancet_lans_plan_error(self._h, _stream(), C.byref(err)), "lancet_lans_plan_error")
        return err.value

    def debug(self, spin_limit=0, flags=0):
        """Test hook (include/lancet_hip_debug.h): bound of the resident schedule's waits, bit 0 = nothing
        is published."""
        capi.check(self._lib.lancet_lans_plan_debug(self._h, int(spin_limit), int(flags)), "lancet_lans_plan_debug")

    def last_resident_slots(self):
        """Test hook: chunk slots the resident kernel took in the last step (0: sweeps only)."""
        n = C.c_int(-1)
        capi.check(self._lib.lancet_lans_plan_debug_last_resident(self._h, C.byref(n)),
                   "lancet_lans_plan_debug_last_resident")
        return n.value

    def close(self):
        if self._h is not None:
            self._lib.lancet_lans_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def step(self, g, p, m, v, step, hyper, step_dev=None, grad_norms=None, p_lowp=None):
        """One LANS step.  p, m, v are float32 (the master parameters and the moments); g is float32, or bfloat16 /
        float16 as the backward pass of a 16-bit model leaves it (one type for the whole list; widened inside the
        step, which is what casting the gradients to float32 first would give); p_lowp: optional list of bfloat16 /
        float16 tensors that receive the new parameters rounded to that type (the model's own copies), written in
        the same pass as p.  grad_norms: optional float32 GPU tensor [T] of ||g_i|| in list order (skips the
        step's own pass over g).  Raises LancetError(ERR_STALLED) when an earlier step of the resident
        schedule gave up a wait, until error() has been read."""
        T = len(self.numels)
        if grad_norms is not None:
            _need(grad_norms.is_cuda and grad_norms.dtype == torch.float32 and grad_norms.numel() == T and
                  grad_norms.is_contiguous(), "grad_norms must be a contiguous float32 GPU tensor of T values")
        _need(len(g) == len(p) == len(m) == len(v) == T, "tensor lists must have one entry per planned tensor")
        _need(p_lowp is None or len(p_lowp) == T, "p_lowp must have one entry per planned tensor")
        g_dtype = g[0].dtype if T else torch.float32
        _need(g_dtype in _DTYPES, "gradients must be float32, bfloat16 or float16")
        lowp_dtype = p_lowp[0].dtype if p_lowp else torch.bfloat16
        _need(lowp_dtype in (torch.bfloat16, torch.float16), "p_lowp must be bfloat16 or float16")
        for lst, dt in ((g, g_dtype), (p, torch.float32), (m, torch.float32), (v, torch.float32)) + (((p_lowp, lowp_dtype),) if p_lowp else ()):
            for t, n in zip(lst, self.numels):
                _need(t.is_cuda and t.is_contiguous() and t.dtype == dt and t.numel() == n,
                      "LANS tensors must be contiguous GPU tensors of the planned sizes: p, m, v float32, every gradient of "
                      "one type, every 16-bit parameter copy of one type")
        arrs = [capi.ptr_array([t.data_ptr() for t in lst]) for lst in (g, p, m, v)]
        if g_dtype == torch.float32 and not p_lowp:
            st = self._lib.lancet_lans_step(self._h, arrs[0], arrs[1], arrs[2], arrs[3], int(step),
                                            _p(step_dev), C.byref(hyper), _p(grad_norms), _stream())
            capi.check(st, "lancet_lans_step")
            return
        low = capi.ptr_array([t.data_ptr() for t in p_lowp]) if p_lowp else None
        st = self._lib.lancet_lans_step_mixed(self._h, arrs[0], _DTYPES[g_dtype], arrs[1], arrs[2], arrs[3], low,
                                              _DTYPES[lowp_dtype], int(step), _p(step_dev), C.byref(hyper), _p(grad_norms),
                                              _stream())
        capi.check(st, "lancet_lans_step_mixed")

    def norms(self):
        """[4, T] float32: (||g||, ||p||, ||u_m||, ||u_g||) of the last step."""
        out = torch.empty((4, len(self.numels)), dtype=torch.float32, device="cuda")
        capi.check(self._lib.lancet_lans_plan_norms(self._h, _p(out), _stream()), "lancet_lans_plan_norms")
        return out


_PLANS = {}


def lans(tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction, weight_decay, grad_averaging,
         mode, normalize_grad, p_lowp=None):
    """raf.op.lans(tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction,
    weight_decay, grad_averaging, mode, normalize_grad).

    tensor_list = [g.. | p.. | m.. | v..] (python/raf/optim/lans.py:76-103); p, m, v are updated
    in place and the output tuple aliases the inputs (src/op/declare/optimizer.cc:46-62).  `step` is a Python number or a
    0-dim float32 GPU tensor (the reference passes a tensor; it is read on the device).  Trailing extension for a
    16-bit model: the gradients may be bfloat16 / float16 and p_lowp, a list of T 16-bit tensors, receives the new
    parameters in that type (what the casts around the op do in python/raf/optim/lans.py:256-257, 285-288)."""
    n = len(tensor_list)
    _need(n % 4 == 0 and n > 0, "tensor_list must hold 4 lists of equal length")
    T = n // 4
    g, p, m, v = (list(tensor_list[i * T:(i + 1) * T]) for i in range(4))
    key = (tuple(t.numel() for t in g), g[0].device.index)
    plan = _PLANS.get(key)
    if plan is None:
        plan = _PLANS[key] = LansPlan(key[0])
        # LANCET_LANS_SCHEDULE=sweeps: for a device this process shares with kernels of unbounded duration
        if os.environ.get("LANCET_LANS_SCHEDULE") == "sweeps":
            plan.set_schedule(capi.LANS_SWEEPS)
    hyper = capi.LansHyper(float(learning_rate), float(beta1), float(beta2), float(eps), int(bias_correction),
                           float(weight_decay), int(grad_averaging), int(mode), int(bool(normalize_grad)))
    if torch.is_tensor(step):
        _need(step.is_cuda and step.dtype == torch.float32 and step.numel() == 1, "step tensor must be a float32 GPU scalar")
        plan.step(g, p, m, v, 0, hyper, step_dev=step, p_lowp=p_lowp)
    else:
        plan.step(g, p, m, v, int(step), hyper, p_lowp=p_lowp)
    return tuple(tensor_list)


class LansStepper:
    """Minimal counterpart of raf.optim.lans.LANS (python/raf/optim/lans.py:44-103): owns m, v and
    the step counter (starting at 1) and feeds [g.., p.., m.., v..] in the reference's order."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-6, weight_decay=0.01, bias_correction=True,
                 grad_averaging=True, mode=True, normalize_grad=True):
        self.params = list(params)
        # a 16-bit model: float32 master copies are what the step updates, and it writes the model's own
        # parameters, rounded, in the same pass (the reference keeps float32 parameters and casts around the op,
        # python/raf/optim/lans.py:256-257, 285-288)
        self.mixed = bool(self.params) and self.params[0].dtype in (torch.bfloat16, torch.float16)
        _need(all(p.dtype == self.params[0].dtype for p in self.params), "parameters must share one dtype")
        self.master = [p.detach().float() for p in self.params] if self.mixed else None
        self.m = [torch.zeros_like(p, dtype=torch.float32) for p in self.params]
        self.v = [torch.zeros_like(p, dtype=torch.float32) for p in self.params]
        self.hyper = (lr, betas[0], betas[1], eps, int(bias_correction), weight_decay, int(grad_averaging),
                      int(mode), bool(normalize_grad))
        self._step = 1

    def step(self, grads=None):
        """grads: one gradient per parameter, None for a parameter without one (it is left out of the step, as
        python/raf/optim/lans.py:82-84 leaves out parameters whose .grad is None); default: the parameters' .grad."""
        if grads is None:
            grads = [p.grad for p in self.params]
        grads = list(grads)
        _need(len(grads) == len(self.params), "one gradient (or None) per parameter")
        live = [i for i, g in enumerate(grads) if g is not None]
        if live:
            pick = lambda lst: [lst[i] for i in live]
            # the update writes the parameters in place, outside autograd
            if self.mixed:
                lans(pick(grads) + pick(self.master) + pick(self.m) + pick(self.v), self._step, *self.hyper,
                     p_lowp=[p.detach() for p in pick(self.params)])
            else:
                lans(pick(grads) + [p.detach() for p in pick(self.params)] + pick(self.m) + pick(self.v), self._step,
                     *self.hyper)
        self._step += 1

"""A minimal executor over the C++ op layer (raf_hip/): what RAF's interpreter does for one
primitive call (src/impl/interpreter.cc:246-328) - run the op's Declare to learn the outputs,
allocate them, dispatch to the highest-priority dialect op, allocate the workspaces its OpEnv
requested, and Execute on the current stream.  Device memory comes from torch.

    ex = Executor()
    gates_s, indloc, used, elems, buf = ex("raf.op.moe_encode", data, gate, used_capacity, 1.25)

PreparedCall keeps the OpEnv alive for repeated execution on the same buffers, like the VM's
OpEnv cache (src/impl/vm/vm.cc:1209-1255).
"""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "liblancet_raf_ops.so")

_DL = {torch.float32: (2, 32), torch.float16: (2, 16), torch.bfloat16: (4, 16), torch.int32: (0, 32),
       torch.int64: (0, 64), torch.uint8: (1, 8), torch.bool: (1, 8)}
if hasattr(torch, "uint64"):
    _DL[torch.uint64] = (1, 64)
_FROM_DL = {(2, 32): torch.float32, (2, 16): torch.float16, (4, 16): torch.bfloat16, (0, 32): torch.int32,
            (0, 64): torch.int64, (1, 64): torch.int64}

_lib = None


class RafError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("liblancet_raf_ops.so is not built (%s); run build.py" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
    sig = {
        "raf_hip_last_error": (C.c_char_p, []),
        "raf_hip_call_create": (vp, [C.c_char_p]),
        "raf_hip_call_destroy": (None, [vp]),
        "raf_hip_push_tensor": (ci, [vp, vp, ci, ci, ci, ci, C.POINTER(i64)]),
        "raf_hip_push_int": (ci, [vp, i64]),
        "raf_hip_push_float": (ci, [vp, C.c_double]),
        "raf_hip_push_bool": (ci, [vp, ci]),
        "raf_hip_begin_tuple": (ci, [vp]),
        "raf_hip_end_tuple": (ci, [vp]),
        "raf_hip_declare": (ci, [vp]),
        "raf_hip_num_outputs": (ci, [vp]),
        "raf_hip_output_is_tuple": (ci, [vp]),
        "raf_hip_output_info": (ci, [vp, ci, C.POINTER(ci), C.POINTER(ci), C.POINTER(i64), C.POINTER(vp)]),
        "raf_hip_set_output_data": (ci, [vp, ci, vp]),
        "raf_hip_dispatch": (ci, [vp]),
        "raf_hip_env_name": (C.c_char_p, [vp]),
        "raf_hip_num_workspaces": (ci, [vp]),
        "raf_hip_workspace_bytes": (i64, [vp, ci]),
        "raf_hip_bind_workspace": (ci, [vp, ci, vp]),
        "raf_hip_check_device_status": (ci, [vp]),
        "raf_hip_num_arg_indices": (ci, [vp]),
        "raf_hip_arg_index": (ci, [vp, ci]),
        "raf_hip_set_stream": (None, [ci, vp]),
        "raf_hip_execute": (ci, [vp]),
        "raf_hip_push_dialect_preference": (ci, [C.c_char_p]),
        "raf_hip_pop_dialect_preference": (ci, []),
        "raf_hip_num_registered_ops": (ci, []),
        "raf_hip_registered_op": (C.c_char_p, [ci]),
        "raf_hip_dispatch_list": (C.c_char_p, [C.c_char_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise RafError(load().raf_hip_last_error().decode())


def registered_ops():
    lib = load()
    return [lib.raf_hip_registered_op(i).decode() for i in range(lib.raf_hip_num_registered_ops())]


def dispatch_list(base_op):
    """[(dialect_op, plevel), ...] in dispatch order under the current dialect preference."""
    s = load().raf_hip_dispatch_list(base_op.encode()).decode()
    return [(e.split(":")[0], int(e.split(":")[1])) for e in s.split(";") if e]


class dialect_preference:
    """with dialect_preference(["hip"]): ...  (python/raf/testing/common.py:254-272 with_dialect)."""

    def __init__(self, dialects):
        self.dialects = list(dialects)

    def __enter__(self):
        _check(load().raf_hip_push_dialect_preference(",".join(self.dialects).encode()))

    def __exit__(self, *exc):
        _check(load().raf_hip_pop_dialect_preference())


class PreparedCall:
    def __init__(self, op_name, args):
        lib = load()
        self._lib = lib
        self._h = lib.raf_hip_call_create(op_name.encode())
        self._keep = []      # tensors that must outlive the call
        self._inputs = {}
        try:
            for a in args:
                self._push(a)
            _check(lib.raf_hip_declare(self._h))
            self.outputs = self._allocate_outputs()
            _check(lib.raf_hip_dispatch(self._h))
            self.env_name = lib.raf_hip_env_name(self._h).decode()
            self.arg_indices = [lib.raf_hip_arg_index(self._h, i) for i in range(lib.raf_hip_num_arg_indices(self._h))]
            self.workspaces = []
            for i in range(lib.raf_hip_num_workspaces(self._h)):
                nbytes = int(lib.raf_hip_workspace_bytes(self._h, i))
                ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
                self.workspaces.append(ws)
                _check(lib.raf_hip_bind_workspace(self._h, i, C.c_void_p(ws.data_ptr())))
        except Exception:
            self.close()
            raise

    def _push(self, a):
        lib, h = self._lib, self._h
        if torch.is_tensor(a):
            if not a.is_cuda or not a.is_contiguous():
                raise RafError("tensor arguments must be contiguous GPU tensors")
            code, bits = _DL[a.dtype]
            shape = (C.c_int64 * max(a.dim(), 1))(*a.shape)
            self._keep.append(a)
            self._inputs[a.data_ptr()] = a
            _check(lib.raf_hip_push_tensor(h, C.c_void_p(a.data_ptr()), a.device.index or 0, code, bits, a.dim(), shape))
        elif isinstance(a, bool):
            _check(lib.raf_hip_push_bool(h, int(a)))
        elif isinstance(a, int):
            _check(lib.raf_hip_push_int(h, a))
        elif isinstance(a, float):
            _check(lib.raf_hip_push_float(h, a))
        elif isinstance(a, (list, tuple)):
            _check(lib.raf_hip_begin_tuple(h))
            for x in a:
                self._push(x)
            _check(lib.raf_hip_end_tuple(h))
        else:
            raise RafError("unsupported argument type %r" % type(a))

    def _allocate_outputs(self):
        lib, h = self._lib, self._h
        outs = []
        for i in range(lib.raf_hip_num_outputs(h)):
            code, bits, data = C.c_int(), C.c_int(), C.c_void_p()
            shape = (C.c_int64 * 8)()
            nd = lib.raf_hip_output_info(h, i, C.byref(code), C.byref(bits), shape, C.byref(data))
            if data.value:   # in-place output: aliases an input tensor
                outs.append(self._inputs[data.value])
                continue
            dt = _FROM_DL[(code.value, bits.value)]
            t = torch.empty(tuple(shape[d] for d in range(nd)), dtype=dt, device="cuda")
            _check(lib.raf_hip_set_output_data(h, i, C.c_void_p(t.data_ptr())))
            if (code.value, bits.value) == (1, 64) and hasattr(torch, "uint64"):
                t = t.view(torch.uint64)
            outs.append(t)
        if not lib.raf_hip_output_is_tuple(h):
            return outs[0]
        return tuple(outs)

    def run(self):
        self._lib.raf_hip_set_stream(torch.cuda.current_device(), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        _check(self._lib.raf_hip_execute(self._h))
        return self.outputs

    def check(self):
        """Raises if the device recorded a failure in work this call launched (a bounded wait that gave up);
        synchronises the current stream."""
        _check(self._lib.raf_hip_check_device_status(self._h))

    def close(self):
        if self._h is not None:
            self._lib.raf_hip_call_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Executor:
    def prepare(self, op_name, *args):
        return PreparedCall(op_name, args)

    def __call__(self, op_name, *args):
        call = PreparedCall(op_name, args)
        try:
            out = call.run()
            call.check()          # synchronises; the reference would have aborted on a device-side failure
            return out
        finally:
            # outputs are torch tensors and stay valid; the OpEnv (and, for lans, its plan) goes away.
            # Work already enqueued only touches caller-owned memory and the workspaces kept below.
            torch.cuda.current_stream().synchronize()
            call.close()

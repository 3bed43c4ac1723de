"""ctypes bindings of the C ABI declared in include/lancet_hip.h.

The library is loaded from <package>/lib/liblancet_hip.so (built in-tree by build.py).
There is no fallback: a missing library raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "liblancet_hip.so")

F32, BF16, F16 = 0, 1, 2
GATE_IS_LOGITS = 1
NO_TAIL_ZERO = 2
ABI_VERSION = 8
ZERO_TAIL = 4
ROWS_AT_USED = 8
SCAN_LOOKBACK = 16
LANS_SWEEPS, LANS_RESIDENT = 0, 1
MAX_EXPERTS = 512
MAX_PARTITIONS = 64

OK = 0
(ERR_NULL, ERR_SHAPE, ERR_DTYPE, ERR_WORKSPACE, ERR_ALIGN, ERR_TOPK, ERR_PARTITION, ERR_PLAN, ERR_SCRATCH,
 ERR_STALLED) = range(-1, -11, -1)
NOALLOC_SCRATCH_BYTES = (2 << 20) + 4096


class LansHyper(C.Structure):
    _fields_ = [("learning_rate", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float),
                ("eps", C.c_float), ("bias_correction", C.c_int), ("weight_decay", C.c_float),
                ("grad_averaging", C.c_int), ("mode", C.c_int), ("normalize_grad", C.c_int)]


class LancetError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__("%s failed: status %d (%s)" % (what, status, status_string(status)))


_vp, _i64, _int, _u32, _sz, _f32 = C.c_void_p, C.c_int64, C.c_int, C.c_uint, C.c_size_t, C.c_float

# name -> (restype, argtypes); every symbol include/lancet_hip.h declares
SIGNATURES = {
    "lancet_abi_version": (_int, []),
    "lancet_status_string": (C.c_char_p, [_int]),
    "lancet_moe_capacity": (_i64, [_i64, _i64, _f32]),
    "lancet_gate_topk": (_int, [_vp, _vp, _i64, _i64, _int, _int, _u32, _vp, _vp, _vp]),
    "lancet_gen_location_workspace_bytes": (_sz, [_i64, _i64]),
    "lancet_launch_gen_location": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "lancet_launch_encode_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "lancet_moe_encode_workspace_bytes": (_sz, [_i64, _i64, _int]),
    "lancet_moe_encode": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _u32,
                                 _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "lancet_moe_encode_noalloc": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _u32,
                                         _vp, _vp, _vp, _vp, _vp, _vp]),
    "lancet_moe_route": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _u32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "lancet_moe_scatter": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _u32, _vp, _vp]),
    "lancet_moe_encode_bpr_workspace_bytes": (_sz, [_i64, _i64, _int]),
    "lancet_moe_encode_bpr": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _u32,
                                     _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "lancet_moe_scatter_tokens": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _u32, _vp, _vp]),
    "lancet_moe_decode_tokens": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp]),
    "lancet_memcpy_sparse_ranges_to_cont_3d": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _int, _int, _i64, _i64, _i64, _i64, _int, _vp]),
    "lancet_memcpy_cont_to_sparse_ranges_3d": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _int, _int, _i64, _i64, _i64, _i64, _int, _vp]),
    "lancet_moe_partition_ranges_workspace_bytes": (_sz, [_int, _int, _i64]),
    "lancet_moe_partition_ranges": (_int, [_vp, _i64, _int, _int, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "lancet_debug_scatter_dest": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp, _vp]),
    "lancet_debug_decode_dest": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp]),
    "lancet_debug_stream": (_int, [_int, _vp, _vp, _sz, _vp]),
    "lancet_debug_stream_4r3w": (_int, [_vp, _vp, _vp, _vp, _sz, _vp]),
    "lancet_moe_decode": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp]),
    "lancet_moe_redispatch_expert_input": (_int, [C.POINTER(_vp), C.POINTER(_vp), _int, _int, _int, _i64, _i64, _i64,
                                                  _int, _int, _vp, _vp]),
    "lancet_memcpy_sparse_to_cont_3d": (_int, [_vp, _vp, _vp, _i64, _int, _int, _int, _i64, _i64, _i64, _i64, _int, _int,
                                               _int, _vp]),
    "lancet_memcpy_cont_to_sparse_3d": (_int, [_vp, _vp, _vp, _i64, _int, _int, _int, _i64, _i64, _i64, _i64, _int, _int,
                                               _int, _u32, _vp]),
    "lancet_moe_encode_dx": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp, _vp]),
    "lancet_moe_encode_dg": (_int, [_vp, _vp, _i64, _i64, _int, _int, _vp, _vp]),
    "lancet_moe_encode_dgate": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _u32, _vp, _vp]),
    "lancet_moe_decode_dx_workspace_bytes": (_sz, [_i64, _i64]),
    "lancet_moe_decode_dx": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp, _sz, _vp]),
    "lancet_moe_decode_dg": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp, _vp]),
    "lancet_moe_top2_normalize_gates": (_int, [_vp, _vp, _i64, _int, _vp, _vp]),
    "lancet_moe_merge_masks_workspace_bytes": (_sz, [_int, _i64]),
    "lancet_moe_merge_masks": (_int, [C.POINTER(_vp), _int, _i64, _i64, _vp, _vp, _sz, _vp]),
    "lancet_moe_redispatch_workspace_bytes": (_sz, [_int, _i64]),
    "lancet_moe_redispatch": (_int, [C.POINTER(_vp), C.POINTER(_vp), _int, _i64, _i64, _i64, _i64, _int,
                                     _vp, _vp, _sz, _vp]),
    "lancet_lans_plan_create": (_int, [C.POINTER(_i64), _int, C.POINTER(_vp)]),
    "lancet_lans_plan_destroy": (_int, [_vp]),
    "lancet_lans_step": (_int, [_vp, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                _int, _vp, C.POINTER(LansHyper), _vp, _vp]),
    "lancet_lans_step_mixed": (_int, [_vp, C.POINTER(_vp), _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                      _int, _int, _vp, C.POINTER(LansHyper), _vp, _vp]),
    "lancet_lans_plan_norms": (_int, [_vp, _vp, _vp]),
    "lancet_lans_plan_schedule": (_int, [_vp, C.POINTER(_int)]),
    "lancet_lans_plan_set_schedule": (_int, [_vp, _int]),
    "lancet_lans_plan_error": (_int, [_vp, _vp, C.POINTER(_int)]),
    "lancet_lans_debug_chunk_table": (_i64, [C.POINTER(_i64), _int, _int, _int, _vp, _i64, C.POINTER(_i64)]),
    "lancet_lans_plan_debug": (_int, [_vp, _u32, _u32]),
    "lancet_lans_plan_debug_last_resident": (_int, [_vp, C.POINTER(_int)]),
    "lancet_lans_plan_resident_capacity": (_int, [_vp, C.POINTER(_int), C.POINTER(_int)]),
    "lancet_debug_scan_workspace_spin_limit": (_int, [_vp, _u32, _vp]),
    "lancet_debug_scan_workspace_epoch": (_int, [_vp, _u32, _vp]),
    "lancet_scan_workspace_init": (_int, [_vp, _sz, _vp]),
    "lancet_scan_call_is_stateful": (_int, [_i64, _i64, _int, _u32, _int]),
    "lancet_scan_workspace_error": (_int, [_vp, _vp, C.POINTER(_int)]),
}

_lib = None


def load():
    """Returns the ctypes library with typed entry points; raises if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "liblancet_hip.so is not built (%s). Run `python %s` first; there is no fallback path."
            % (LIB_PATH, os.path.join(HERE, "build.py")))
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError = header and library disagree
        fn.restype = res
        fn.argtypes = args
    got = lib.lancet_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError("liblancet_hip.so has ABI version %d, expected %d" % (got, ABI_VERSION))
    _lib = lib
    return lib


def status_string(status):
    return load().lancet_status_string(int(status)).decode()


def check(status, what):
    if status != 0:
        raise LancetError(status, what)


def ptr_array(ptrs):
    arr = (_vp * len(ptrs))()
    for i, p in enumerate(ptrs):
        arr[i] = p
    return arr

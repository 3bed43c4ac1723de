"""ctypes wrapper of the C restatement (oracle/c/lancet_oracle.c).  TEST INFRASTRUCTURE ONLY."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "liblancet_oracle.so")
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("C oracle not built: run `make -C oracle`")
        _lib = C.CDLL(LIB_PATH)
        _lib.oracle_num_threads.restype = C.c_int
        _lib.oracle_moe_encode.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def num_threads():
    return int(load().oracle_num_threads())


def set_num_threads(n):
    load().oracle_set_num_threads(C.c_int(int(n)))


def moe_encode(data, gate, used_in, Cap, k=1, is_logits=False):
    """data: float32 [S,M] or uint16 (bf16 bit patterns) [S,M]."""
    lib = load()
    S, M = data.shape
    E = gate.shape[1]
    dtype = 0 if data.dtype == np.float32 else 1
    gates = np.empty(k * S, np.float32)
    il = np.empty((2, k * S), np.int32)
    used_out = np.empty(E, np.int32)
    elems = np.empty(E, np.uint64)
    disp = np.empty((E, Cap, M), data.dtype)
    data = np.ascontiguousarray(data)
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    used_in = None if used_in is None else np.ascontiguousarray(used_in, dtype=np.int32)
    rc = lib.oracle_moe_encode(_p(data), _p(gate), _p(used_in), C.c_int64(S), C.c_int64(M), C.c_int(E),
                               C.c_int(Cap), C.c_int(k), C.c_int(dtype), C.c_int(int(is_logits)), _p(gates),
                               _p(il), _p(used_out), _p(elems), _p(disp))
    if rc != 0:
        raise MemoryError("oracle_moe_encode")
    return gates, il, used_out, elems, disp


def moe_decode(expert_out, gates, il, k=1):
    lib = load()
    E, Cap, M = expert_out.shape
    S = il.shape[1] // k
    dtype = 0 if expert_out.dtype == np.float32 else 1
    out = np.empty((S, M), expert_out.dtype)
    lib.oracle_moe_decode(_p(np.ascontiguousarray(expert_out)), _p(np.ascontiguousarray(gates, dtype=np.float32)),
                          _p(np.ascontiguousarray(il, dtype=np.int32)), C.c_int64(S), C.c_int64(M), C.c_int(E),
                          C.c_int(Cap), C.c_int(k), C.c_int(dtype), _p(out))
    return out


def lans_step(g, p, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-6, bias_correction=1,
              weight_decay=0.01, grad_averaging=1, mode=1, normalize_grad=True, scratch=None):
    """In place on the float32 arrays of p, m, v.  Returns norms [T,4]."""
    lib = load()
    T = len(g)
    numels = np.array([a.size for a in g], np.int64)
    if scratch is None:
        scratch = np.empty(2 * int(numels.max()), np.float32)
    norms = np.empty((T, 4), np.float32)

    def tab(lst):
        return (C.c_void_p * T)(*[a.ctypes.data for a in lst])
    lib.oracle_lans_step(tab(g), tab(p), tab(m), tab(v), _p(numels), C.c_int(T), C.c_int(int(step)),
                         C.c_float(lr), C.c_float(beta1), C.c_float(beta2), C.c_float(eps),
                         C.c_int(int(bias_correction)), C.c_float(weight_decay), C.c_int(int(grad_averaging)),
                         C.c_int(int(mode)), C.c_int(int(bool(normalize_grad))), _p(scratch), _p(norms))
    return norms

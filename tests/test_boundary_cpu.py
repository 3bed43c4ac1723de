"""CPU-side checks of the drop-in boundary: the C-ABI library exports every symbol the header
declares, rejects bad arguments with a status (never aborts), and the C++ op layer registers the
six operators under RAF's names with RAF's output contract.  No kernel is launched."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols(name="lancet_hip.h"):
    text = open(os.path.join(ROOT, "include", name)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lancet_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.capi.load()
    names = header_symbols()
    hooks = header_symbols("lancet_hip_debug.h")
    assert len(names) >= 25
    for n in names + hooks:
        assert hasattr(lib, n), "liblancet_hip.so does not export %s" % n
    assert sorted(pkg.capi.SIGNATURES) == sorted(names + hooks), "capi.SIGNATURES and the headers disagree"
    header = open(os.path.join(ROOT, "include", "lancet_hip.h")).read()
    assert lib.lancet_abi_version() == pkg.capi.ABI_VERSION == int(re.search(r"#define LANCET_ABI_VERSION (\d+)", header).group(1))
    # test and measurement hooks live in their own header; the operator surface declares none
    assert not [n for n in names if "debug" in n] and all("debug" in n for n in hooks)


def test_capacity_formula(pkg):
    cap = pkg.ops.moe_capacity
    assert cap(4096, 8, 1.25) == 640 and cap(16384, 16, 2.0) == 2048 and cap(32768, 64, 1.25) == 640
    assert cap(65536, 32, 2.5) == 5120 and cap(16384, 32, 10.0) == 5120 and cap(10, 4, 1.5) == 4
    # no capacity: no experts, a negative token count, a product that no int holds, a factor that is no number
    assert cap(16, 0, 1.0) == -1 and cap(-1, 4, 1.0) == -1 and cap(2 ** 62, 1, 3.0e30) == -1
    assert cap(1 << 40, 1, 1.0) == -1 and cap(16, 4, float("nan")) == -1 and cap(16, 4, float("inf")) == -1
    # the ceiling division itself cannot overflow
    assert cap(2 ** 63 - 1, 3, 1e-10) == int(np.float32(1e-10) * np.float32((2 ** 63 - 1 + 2) // 3))


def test_workspace_sizes_and_argument_rejection(pkg):
    lib, capi = pkg.capi.load(), pkg.capi
    assert lib.lancet_moe_encode_workspace_bytes(65536, 32, 2) == 32 + 256 * 64 * 8   # header + one 64-bit word per tile and counter
    assert lib.lancet_moe_encode_workspace_bytes(0, 4, 1) == 32 + 1 * 4 * 8
    assert lib.lancet_moe_encode_workspace_bytes(10, 0, 1) == 0
    one = C.c_void_p(16)  # never dereferenced: every call below is rejected before any launch
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 2, 4, 1, 99, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_DTYPE
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 2, 4, 1, capi.F32, 7, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_DTYPE                     # gate dtype
    st = lib.lancet_moe_encode(one, C.c_void_p(18), None, None, 8, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_ALIGN                     # an fp32 gate at a 2-byte address ...
    st = lib.lancet_moe_encode(one, C.c_void_p(18), None, None, 8, 4, 2, 4, 3, capi.F32, capi.BF16, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_TOPK                      # ... which a 16-bit gate may have (the next check rejects top_k)
    assert lib.lancet_moe_decode(one, one, one, 8, 4, 2, 4, 1, capi.F32, 9, one, None) == capi.ERR_DTYPE
    assert lib.lancet_moe_decode_dg(one, one, one, 8, 4, 2, 4, 1, capi.F32, 9, one, None) == capi.ERR_DTYPE
    assert lib.lancet_moe_encode_dg(one, one, 8, 2, 1, 9, one, None) == capi.ERR_DTYPE
    assert lib.lancet_gate_topk(one, None, 8, 2, 1, 9, 0, one, one, None) == capi.ERR_DTYPE
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 2, 4, 3, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_TOPK
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 1, 4, 2, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_TOPK                      # top-2 needs two experts
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 8, None)
    assert st == capi.ERR_WORKSPACE
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, None, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_NULL
    st = lib.lancet_moe_encode(one, one, None, None, -1, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_SHAPE
    st = lib.lancet_moe_encode(one, one, None, None, 8, 4, 1000, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 30, None)
    assert st == capi.ERR_SHAPE                     # more experts than LANCET_MAX_EXPERTS
    st = lib.lancet_moe_encode(C.c_void_p(18), one, None, None, 8, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_ALIGN
    st = lib.lancet_moe_encode(one, one, one, None, 8, 4, 2, 4, 1, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_TOPK                      # noise for a second choice that does not exist
    st = lib.lancet_moe_encode_bpr(one, one, 8, 4, 2, 4, 2, 2, capi.F32, capi.F32, 0, one, one, one, one, one, one, 1 << 20, None)
    assert st == capi.ERR_PARTITION
    ptrs = capi.ptr_array([16] * 70)
    assert lib.lancet_moe_merge_masks(ptrs, 70, 8, 2, one, one, 1 << 20, None) == capi.ERR_PARTITION
    # sparse <-> packed copies: axis 2 is not supported (sparse_memcpy.cu:78-81), counts must cover every block
    assert lib.lancet_memcpy_sparse_to_cont_3d(one, one, one, 8, 1, 0, 2, 4, 4, 4, 64, 1, 1, capi.F32, None) == capi.ERR_SHAPE
    assert lib.lancet_memcpy_sparse_to_cont_3d(one, one, one, 4, 2, 0, 0, 4, 4, 4, 64, 1, 1, capi.F32, None) == capi.ERR_SHAPE
    assert lib.lancet_memcpy_sparse_to_cont_3d(one, one, one, 8, 1, 0, 0, 4, 4, 4, 64, 0, 1, capi.F32, None) == capi.ERR_SHAPE
    assert lib.lancet_memcpy_cont_to_sparse_3d(one, None, one, 8, 1, 0, 0, 4, 4, 4, 64, 1, 1, capi.F32, 0, None) == capi.ERR_NULL
    assert lib.lancet_memcpy_cont_to_sparse_3d(one, one, C.c_void_p(12), 8, 1, 0, 1, 4, 4, 4, 64, 1, 1, capi.BF16, 0, None) == capi.ERR_ALIGN
    assert lib.lancet_memcpy_cont_to_sparse_3d(one, one, one, 8, 1, 0, 1, 4, 0, 4, 64, 1, 1, capi.BF16, 0, None) == capi.OK
    # token ranges of a whole-batch routing: the range must lie inside the batch
    sc, dc = lib.lancet_moe_scatter_tokens, lib.lancet_moe_decode_tokens
    assert sc(one, one, None, one, 64, 60, 8, 4, 2, 4, 1, capi.F32, 0, one, None) == capi.ERR_SHAPE
    assert sc(one, one, None, one, 64, -1, 8, 4, 2, 4, 1, capi.F32, 0, one, None) == capi.ERR_SHAPE
    assert sc(one, one, None, None, 64, 0, 8, 4, 2, 4, 1, capi.F32, 0, one, None) == capi.ERR_NULL   # tail fill needs used_out
    assert sc(one, one, None, one, 64, 0, 8, 4, 2, 4, 3, capi.F32, 0, one, None) == capi.ERR_TOPK
    assert sc(one, one, None, one, 64, 0, 8, 4, 2, 4, 1, 7, 0, one, None) == capi.ERR_DTYPE
    assert dc(one, one, one, 64, 57, 8, 4, 2, 4, 1, capi.F32, capi.F32, one, None) == capi.ERR_SHAPE
    assert dc(one, None, one, 64, 0, 8, 4, 2, 4, 1, capi.F32, capi.F32, one, None) == capi.ERR_NULL
    assert dc(one, one, one, 64, 0, 8, 4, 2, 4, 1, capi.F32, capi.F32, C.c_void_p(6), None) == capi.ERR_ALIGN
    # row ranges of token partitions
    pr = lib.lancet_moe_partition_ranges
    assert lib.lancet_moe_partition_ranges_workspace_bytes(2, 4, 8) == 2 * 4 * 8 * 4
    assert pr(one, 64, 1, 3, 8, 4, one, one, one, 1 << 20, None) == capi.ERR_PARTITION      # 64 tokens, 3 partitions
    assert pr(one, 64, 2, 40, 8, 4, one, one, one, 1 << 20, None) == capi.ERR_PARTITION     # 2 x 40 > LANCET_MAX_PARTITIONS
    assert pr(one, 64, 3, 4, 8, 4, one, one, one, 1 << 20, None) == capi.ERR_TOPK
    assert pr(one, 64, 1, 4, 8, 4, one, one, one, 8, None) == capi.ERR_WORKSPACE
    assert pr(one, 64, 1, 4, 8, 4, None, one, one, 1 << 20, None) == capi.ERR_NULL
    rc_ = lib.lancet_memcpy_sparse_ranges_to_cont_3d
    assert rc_(one, one, one, None, 8, 1, 0, 0, 4, 4, 4, 64, capi.F32, None) == capi.ERR_NULL       # ranges need starts
    assert rc_(one, one, one, C.c_void_p(20), 8, 1, 0, 0, 4, 4, 4, 64, capi.F32, None) == capi.ERR_ALIGN
    assert lib.lancet_memcpy_cont_to_sparse_ranges_3d(one, one, one, one, 8, 1, 0, 2, 4, 4, 4, 64, capi.F32, None) == capi.ERR_SHAPE
    assert lib.lancet_lans_plan_destroy(None) == capi.ERR_PLAN
    assert "workspace" in capi.status_string(capi.ERR_WORKSPACE)


# ----------------------------------------------------------------------------- C++ op layer
def _declare(rx, op, pushes):
    lib = rx.load()
    h = lib.raf_hip_call_create(op.encode())
    for kind, val in pushes:
        if kind == "t":
            dtype, shape = val
            code, bits = dtype
            arr = (C.c_int64 * len(shape))(*shape)
            assert lib.raf_hip_push_tensor(h, C.c_void_p(256), 0, code, bits, len(shape), arr) == 0
        elif kind == "i":
            assert lib.raf_hip_push_int(h, val) == 0
        elif kind == "f":
            assert lib.raf_hip_push_float(h, val) == 0
        elif kind == "(":
            assert lib.raf_hip_begin_tuple(h) == 0
        elif kind == ")":
            assert lib.raf_hip_end_tuple(h) == 0
    rc = lib.raf_hip_declare(h)
    outs = []
    if rc == 0:
        for i in range(lib.raf_hip_num_outputs(h)):
            code, bits, data = C.c_int(), C.c_int(), C.c_void_p()
            shape = (C.c_int64 * 8)()
            nd = lib.raf_hip_output_info(h, i, C.byref(code), C.byref(bits), shape, C.byref(data))
            outs.append(((code.value, bits.value), tuple(shape[d] for d in range(nd))))
    return h, rc, outs


F32, BF16, I32, U64 = (2, 32), (4, 16), (0, 32), (1, 64)


def test_op_layer_registers_the_six_operators(pkg):
    rx = pkg.raf_executor
    ops = rx.registered_ops()
    for name in ("moe_encode", "moe_encode_batch_prioritized", "moe_decode", "moe_merge_masks", "moe_redispatch", "lans",
                 "moe_encode_dx", "moe_encode_dg", "moe_decode_dx", "moe_decode_dg", "moe_redispatch_expert_input"):
        assert "raf.op." + name in ops
        assert rx.dispatch_list("raf.op." + name) == [("raf.op.hip." + name, 20)]   # plevel 20 as cuda/moe.cc:411
    with rx.dialect_preference(["cuda"]):
        assert rx.dispatch_list("raf.op.moe_encode") == []
    with rx.dialect_preference(["cuda", "hip"]):
        assert rx.dispatch_list("raf.op.moe_encode") == [("raf.op.hip.moe_encode", 20)]


def test_declare_reproduces_the_output_contract(pkg):
    """src/op/declare/moe.cc:26-213 / src/op/ty/moe.cc: shapes and dtypes of every output."""
    rx = pkg.raf_executor
    lib = rx.load()
    S, M, E = 4096, 768, 8
    h, rc, outs = _declare(rx, "raf.op.moe_encode", [("t", (F32, (S, M))), ("t", (F32, (S, E))), ("t", (I32, (E,))), ("f", 1.25)])
    assert rc == 0 and outs == [(F32, (S,)), (I32, (2, S)), (I32, (E,)), (U64, (E,)), (F32, (E, 640, M))]
    assert lib.raf_hip_dispatch(h) == 0 and lib.raf_hip_env_name(h) == b"raf.op.hip.moe_encode"
    assert lib.raf_hip_num_workspaces(h) == 1
    assert lib.raf_hip_workspace_bytes(h, 0) == pkg.capi.load().lancet_moe_encode_workspace_bytes(S, E, 1)
    assert [lib.raf_hip_arg_index(h, i) for i in range(lib.raf_hip_num_arg_indices(h))] == [0, 1, 2]
    lib.raf_hip_call_destroy(h)
    # top-2 extension: slot-major outputs, doubled capacity factor, bf16 buffer
    h, rc, outs = _declare(rx, "raf.op.moe_encode", [("t", (BF16, (16384, 1024))), ("t", (F32, (16384, 16))),
                                                     ("t", (I32, (16,))), ("f", 1.0), ("i", 2), ("i", 1)])
    assert rc == 0 and outs == [(F32, (32768,)), (I32, (2, 32768)), (I32, (16,)), (U64, (16,)), (BF16, (16, 2048, 1024))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_encode_batch_prioritized",
                           [("t", (BF16, (32768, 2048))), ("t", (F32, (32768, 64))), ("i", 4), ("i", 1), ("f", 5.0)])
    assert rc == 0 and outs == [(F32, (8192,)), (I32, (2, 8192)), (I32, (64,)), (U64, (64,)), (BF16, (64, 640, 2048))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_merge_masks", [("(", 0)] + [("t", (I32, (2, 100)))] * 4 + [(")", 0), ("i", 8)])
    assert rc == 0 and outs == [(I32, (2, 400))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_redispatch", [("(", 0)] + [("t", (BF16, (8, 50, 64)))] * 2 + [(")", 0), ("(", 0)] +
                           [("t", (I32, (2, 100)))] * 2 + [(")", 0)])
    assert rc == 0 and outs == [(BF16, (8, 50, 64))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_decode", [("t", (F32, (8, 50, 64))), ("t", (F32, (100,))), ("t", (I32, (2, 100)))])
    assert rc == 0 and outs == [(F32, (100, 64))]
    lib.raf_hip_call_destroy(h)
    # backward ops (src/op/declare/moe.cc:165-247)
    h, rc, outs = _declare(rx, "raf.op.moe_encode_dx", [("t", (BF16, (8, 50, 64))), ("t", (I32, (2, 100)))])
    assert rc == 0 and outs == [(BF16, (100, 64))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_encode_dg", [("t", (F32, (100,))), ("t", (I32, (2, 100))), ("i", 8)])
    assert rc == 0 and outs == [(F32, (100, 8))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_decode_dx", [("t", (BF16, (100, 64))), ("t", (F32, (100,))), ("t", (I32, (2, 100))), ("i", 8), ("i", 50)])
    assert rc == 0 and outs == [(BF16, (8, 50, 64))]
    assert lib.raf_hip_dispatch(h) == 0 and lib.raf_hip_workspace_bytes(h, 0) == 8 * 50 * 4
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_decode_dg", [("t", (F32, (100, 64))), ("t", (F32, (8, 50, 64))), ("t", (I32, (2, 100)))])
    assert rc == 0 and outs == [(F32, (100,))]
    lib.raf_hip_call_destroy(h)


def test_declare_of_the_routed_once_ops_and_the_gate_gradient(pkg):
    """The operators a graph rewrite for this dialect introduces (no base op of these names in the reference):
    moe_route, moe_scatter_tokens (in place on the shared buffer), moe_decode_tokens, moe_partition_ranges,
    moe_encode_dgate."""
    rx = pkg.raf_executor
    lib, capi = rx.load(), pkg.capi.load()
    S, M, E, P = 65536, 4096, 32, 4
    h, rc, outs = _declare(rx, "raf.op.moe_route", [("t", (F32, (S, E))), ("t", (I32, (E,))), ("i", M), ("f", 1.25), ("i", 2), ("i", 1)])
    assert rc == 0 and outs == [(F32, (2 * S,)), (I32, (2, 2 * S)), (I32, (E,)), (U64, (E,))]
    assert lib.raf_hip_dispatch(h) == 0 and lib.raf_hip_env_name(h) == b"raf.op.hip.moe_route"
    assert lib.raf_hip_workspace_bytes(h, 0) == capi.lancet_moe_encode_workspace_bytes(S, E, 2)
    assert [lib.raf_hip_arg_index(h, i) for i in range(lib.raf_hip_num_arg_indices(h))] == [0, 1]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_scatter_tokens",
                           [("t", (BF16, (S // P, M))), ("t", (I32, (2, 2 * S))), ("t", (I32, (E,))), ("t", (I32, (E,))),
                            ("t", (BF16, (E, 5120, M))), ("i", S // P), ("i", 2), ("i", 0)])
    assert rc == 0 and outs == [(BF16, (E, 5120, M))]              # the buffer itself
    assert lib.raf_hip_dispatch(h) == 0 and lib.raf_hip_num_workspaces(h) == 0
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_decode_tokens",
                           [("t", (BF16, (E, 5120, M))), ("t", (F32, (2 * S,))), ("t", (I32, (2, 2 * S))), ("i", S // P), ("i", S // P), ("i", 2)])
    assert rc == 0 and outs == [(BF16, (S // P, M))]
    lib.raf_hip_call_destroy(h)
    h, rc, outs = _declare(rx, "raf.op.moe_partition_ranges", [("t", (I32, (2, 2 * S))), ("i", P), ("i", E), ("i", M), ("i", 2)])
    assert rc == 0 and outs == [(U64, (2 * P, E)), (U64, (2 * P, E))]
    assert lib.raf_hip_dispatch(h) == 0
    assert lib.raf_hip_workspace_bytes(h, 0) == capi.lancet_moe_partition_ranges_workspace_bytes(2, P, E)
    lib.raf_hip_call_destroy(h)
    for gd in (F32, BF16):
        h, rc, outs = _declare(rx, "raf.op.moe_encode_dgate", [("t", (gd, (2 * S,))), ("t", (gd, (S, E))), ("t", (I32, (2, 2 * S))), ("i", 2), ("i", 1)])
        assert rc == 0 and outs == [(gd, (S, E))]
        lib.raf_hip_call_destroy(h)
    h, rc, _ = _declare(rx, "raf.op.moe_decode_tokens",
                        [("t", (F32, (8, 50, 64))), ("t", (F32, (100,))), ("t", (I32, (2, 100))), ("i", 90), ("i", 20)])
    assert rc != 0 and b"token range outside the routed batch" in lib.raf_hip_last_error()
    lib.raf_hip_call_destroy(h)


def test_gate_typed_outputs_follow_the_gate(pkg):
    """A deliberate difference from the reference's Declare, which types gates_s float32 whatever the gate is
    (src/op/declare/moe.cc:54) and the gradient of gates_s like dy (:239): here gates_s and its gradient take the
    gate's type, which is what the reference's kernels are instantiated on (`__dtype* gates1_s`,
    tutel_moe_dispatch.cu:110-116).  With the float32 gate the reference's models feed, both rules give float32;
    under mixed precision a graph typed by the reference's rule needs a cast behind the op."""
    rx = pkg.raf_executor
    lib = rx.load()
    for gd in (F32, BF16):
        h, rc, outs = _declare(rx, "raf.op.moe_encode", [("t", (BF16, (512, 64))), ("t", (gd, (512, 8))), ("t", (I32, (8,)))])
        assert rc == 0 and outs[0] == (gd, (512,)) and outs[4] == (BF16, (8, 64, 64))
        lib.raf_hip_call_destroy(h)
    # moe_decode_dg: float32 unless the trailing gate_dtype argument names a half type (never dy's type by itself)
    for code, want in ((None, F32), (1, BF16)):
        args = [("t", (BF16, (100, 64))), ("t", (BF16, (8, 50, 64))), ("t", (I32, (2, 100)))] + ([("i", 1), ("i", code)] if code is not None else [])
        h, rc, outs = _declare(rx, "raf.op.moe_decode_dg", args)
        assert rc == 0 and outs == [(want, (100,))]
        lib.raf_hip_call_destroy(h)


def test_op_layer_errors_are_reported_not_fatal(pkg):
    rx = pkg.raf_executor
    lib = rx.load()
    h, rc, _ = _declare(rx, "raf.op.moe_encode", [("t", (F32, (10, 4))), ("t", (F32, (11, 2))), ("t", (I32, (2,)))])
    assert rc != 0 and b"matching shape in dim 0" in lib.raf_hip_last_error()
    lib.raf_hip_call_destroy(h)
    h, rc, _ = _declare(rx, "raf.op.moe_encode_batch_prioritized", [("t", (F32, (10, 4))), ("t", (F32, (10, 2))), ("i", 2), ("i", 2)])
    assert rc != 0 and b"partition_id should be less than n_partitions" in lib.raf_hip_last_error()
    lib.raf_hip_call_destroy(h)
    h, rc, _ = _declare(rx, "raf.op.not_an_op", [])
    assert rc != 0 and b"no FRAFDeclare" in lib.raf_hip_last_error()
    lib.raf_hip_call_destroy(h)
    with rx.dialect_preference(["cuda"]):
        h, rc, _ = _declare(rx, "raf.op.moe_decode", [("t", (F32, (8, 50, 64))), ("t", (F32, (100,))), ("t", (I32, (2, 100)))])
        assert rc == 0 and lib.raf_hip_dispatch(h) != 0
        assert b"Cannot find a valid dispatch" in lib.raf_hip_last_error()
        lib.raf_hip_call_destroy(h)


# ----------------------------------------------------------------------------- LANS task queue
def _chunk_table(pkg, numels, limit=1 << 30, round_=1 << 30):
    """(tensor of every chunk slot in ticket order, -1 = padding; slots the resident kernel hands out)."""
    lib = pkg.capi.load()
    arr = (C.c_int64 * len(numels))(*numels)
    n = lib.lancet_lans_debug_chunk_table(arr, len(numels), limit, round_, None, 0, None)
    ctensor = np.empty(max(n, 1), np.int32)
    nres = C.c_int64(-1)
    assert lib.lancet_lans_debug_chunk_table(arr, len(numels), limit, round_, ctensor.ctypes.data_as(C.c_void_p), n,
                                             C.byref(nres)) == n
    return ctensor[:n], nres.value


def _simulate_resident(ctensor, workers, rng, publish=True):
    """The resident LANS kernel as a state machine.  Every workgroup runs passes of
        draw a slot | M(s1), publish its three sums | N(drawn slot), publish its sum of g^2 |
        wait for the M sums of every chunk of s0's tensor and the N sums of every chunk of s2's | U(s0) | rotate
    on the chunk slots it draws in ticket order (s0 <- s1 <- s2 <- drawn; the first two passes find s0 and s1
    empty).  Stage M of a slot needs no wait of its own: the norm of its tensor was formed at the wait of the
    pass before, when the slot was s2.  Padding slots (-1) pass every stage at once.  Only `workers`
    workgroups run (the others never get onto the chip and draw nothing); they are advanced in random
    order.  Returns True when every chunk has been through U, False when no workgroup can move (on the
    device: the bounded waits give up).  publish=False: the test hook that withholds every sum."""
    n = len(ctensor)
    real = ctensor[ctensor >= 0]
    size = np.bincount(real, minlength=int(real.max()) + 1 if len(real) else 1)
    sums_n, sums_m = np.zeros_like(size), np.zeros_like(size)
    state = {"ticket": 0, "done": 0}

    class WG:
        def __init__(self):
            self.s = [None, None, None]
            self.drawn = None
            self.waiting = False

    def is_real(x):
        return x is not None and x >= 0

    wgs = [WG() for _ in range(workers)]
    live = set(range(workers))
    while live:
        moved = False
        for i in rng.permutation(sorted(live)):
            w = wgs[i]
            s0, s1, s2 = w.s
            if not w.waiting:                               # draw, stage M on s1, stage N on the drawn slot
                w.drawn = None
                if state["ticket"] < n:
                    w.drawn = int(ctensor[state["ticket"]])
                    state["ticket"] += 1
                if publish and is_real(s1):
                    sums_m[s1] += 1
                if publish and is_real(w.drawn):
                    sums_n[w.drawn] += 1
                w.waiting = True
                moved = True
            elif (not is_real(s0) or sums_m[s0] == size[s0]) and (not is_real(s2) or sums_n[s2] == size[s2]):
                if is_real(s0):                             # stage U on s0
                    state["done"] += 1
                w.s = [s1, s2, w.drawn]
                w.waiting = False
                moved = True
                if all(x is None for x in w.s):
                    live.discard(i)
        if not moved:
            return False
    return state["done"] == len(real)


@pytest.mark.parametrize("case", ["config5", "random", "tiny"])
def test_lans_resident_schedule_drains(pkg, case):
    """A workgroup of the resident schedule waits only for chunks of tensors it holds, slots are handed out in
    order, and a workgroup has drawn two slots by the time it first waits for one of them: the kernel drains
    whenever the running workgroups are at least half the chunks of the largest tensor, and stalls with fewer
    (and always when nothing is published)."""
    import bench
    rng = np.random.default_rng(0)
    if case == "config5":
        numels = [int(np.prod(s)) for s in bench.lans_shapes()][:40]
    elif case == "random":
        numels = [int(x) * 8192 for x in rng.integers(0, 70, 60)] + [0, 1, 8192, 8193, 70 * 8192 - 1]
    else:
        numels = [8192, 2 * 8192, 3 * 8192]
    chunks = [(x + 8191) // 8192 for x in numels]
    whole = [i for i, x in enumerate(numels) if x % 8192 == 0]
    largest = max(chunks[i] for i in whole)
    for round_ in (largest, largest + 3, 4 * largest):
        ctensor, nres = _chunk_table(pkg, numels, largest, round_)
        real = ctensor[ctensor >= 0]
        np.testing.assert_array_equal(np.bincount(real, minlength=len(numels)), chunks)   # every chunk exactly once
        res = ctensor[:nres]
        # the kernel takes the tensors that are whole chunks (and fit); the others follow, without padding
        assert set(res[res >= 0].tolist()) == {i for i in whole if chunks[i] > 0}
        assert (ctensor[nres:] >= 0).all()
        for i in set(res[res >= 0].tolist()):             # chunks of a tensor are consecutive slots of ONE round
            where = np.flatnonzero(res == i)
            assert where[-1] - where[0] + 1 == len(where) and where[0] // round_ == where[-1] // round_
        sizes = [chunks[i] for i in dict.fromkeys(res[res >= 0].tolist())]
        assert sizes == sorted(sizes, reverse=True)       # largest tensors first
        for workers in ((largest + 1) // 2, round_, round_ + 5):
            assert _simulate_resident(res, workers, rng)
    ctensor, nres = _chunk_table(pkg, numels, largest, largest)
    if largest > 2:
        assert not _simulate_resident(ctensor[:nres], (largest + 1) // 2 - 1, rng)
    assert not _simulate_resident(ctensor[:nres], largest, rng, publish=False)


def test_lans_plan_orders_tensors_that_do_not_fit_last(pkg):
    """Tensors with more chunks than the resident kernel takes, or that are not whole chunks, come after all
    the others in the plan's slot order, without padding, and are left to the sweeps; every chunk of every
    tensor appears exactly once."""
    numels = [8192, 5 * 8192, 8192 * 40 + 1, 8192, 8192 * 41, 8192 * 40, 0, 7 * 8192, 100]
    limit = 40
    ctensor, nres = _chunk_table(pkg, numels, limit, limit)
    chunks = [(n + 8191) // 8192 for n in numels]
    real = ctensor[ctensor >= 0]
    np.testing.assert_array_equal(np.bincount(real, minlength=len(numels)), chunks)
    fits = [i for i, n in enumerate(numels) if n % 8192 == 0 and chunks[i] <= limit]
    assert set(ctensor[:nres]) - {-1} == {i for i in fits if chunks[i] > 0}
    # rounds of 40 slots: [tensor 5 (40)] [tensor 7 (7), tensor 1 (5), tensors 0 and 3 (1 each)]: no padding needed
    assert nres == sum(chunks[i] for i in fits) and (ctensor[:nres] >= 0).all()
    assert list(dict.fromkeys(ctensor[:nres])) == [5, 7, 1, 0, 3]
    assert list(dict.fromkeys(ctensor[nres:])) == [2, 4, 8] and (ctensor[nres:] >= 0).all()   # list order, no padding
    assert _simulate_resident(ctensor[:nres], limit, np.random.default_rng(1))
    # a tensor that does not fit into what is left of a round starts the next one
    ctensor, nres = _chunk_table(pkg, [3 * 8192, 3 * 8192, 3 * 8192], 4, 4)
    assert ctensor.tolist() == [0, 0, 0, -1, 1, 1, 1, -1, 2, 2, 2] and nres == 11


def test_missing_library_is_an_error_not_a_fallback(pkg, monkeypatch, tmp_path):
    """Without the built library every operator raises; nothing routes to a CPU implementation."""
    capi = pkg.capi
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "liblancet_hip.so"))
    with pytest.raises(RuntimeError, match="not built"):
        capi.load()
    pkg.ops.moe_capacity.cache_clear()   # sizes are cached per shape; every operator loads the library first
    with pytest.raises(RuntimeError, match="not built"):
        pkg.ops.moe_capacity(16, 4, 1.0)
    src = open(os.path.join(os.path.dirname(capi.__file__), "ops.py")).read()
    assert "oracle" not in src and "numpy" not in src          # the operator layer never imports the checker


def test_header_is_plain_c_and_the_c_client_links():
    """include/lancet_hip.h must compile as C99 and as C++11 on its own; the C client under tests/c_client
    builds against the in-tree library with gcc (it runs in the GPU tests)."""
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hdr = os.path.join(root, "include", "lancet_hip.h")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", hdr], check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c++", hdr],
                   check=True)
    if not os.path.isdir("/opt/rocm/include"):
        pytest.skip("HIP runtime headers are not installed")
    build_dir = os.path.join(root, "tests", "c_client")
    subprocess.run(["make", "-C", build_dir, "-B"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    assert os.path.exists(os.path.join(build_dir, "lancet_client")) and shutil.which("gcc")


def test_op_layer_under_address_and_undefined_behaviour_sanitizers():
    """The C++ op layer (raf_hip/) built with -fsanitize=address,undefined and run on host memory for every operator
    of the hip dialect, against a host-only stand-in for the C ABI whose calls touch every byte the kernels touch
    (tests/c_client/op_layer_san.cc): a wrong shape, dtype or size in the op layer is a sanitizer report.  The
    reference builds its host code under the same sanitizers (cmake/modules/Sanitizer.cmake:13-40)."""
    import subprocess
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_client")
    subprocess.run(["make", "-C", here, "op_layer_san"], check=True, stdout=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([os.path.join(here, "op_layer_san")], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "every operator ran under the sanitizers" in proc.stdout
    assert "ERROR: AddressSanitizer" not in proc.stdout and "runtime error" not in proc.stdout

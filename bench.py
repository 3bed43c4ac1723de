"""Benchmark of the MoE dispatch path and the fused LANS step on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: raf.op.moe_encode
(routing + scatter) followed by raf.op.moe_decode at the headline shape of BASELINE.json
(S=65536 tokens, M=4096 bf16, E=32 experts, top-2, capacity factor 1.25 -> C=5120), inputs
resident in HBM.  Prints ONE JSON line: metric / value / unit (tokens per second of encode + decode),
`roofline` (the scatter kernel against 8 TB/s of HBM, timed with HIP events), `ops`, `backward`,
`config4_partitioned`, `pipeline`, `lans` (per-phase and side workloads) and `cpu_baseline` (the C/OpenMP
restatement of the reference's algorithm timed on this host).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-lans] [--no-cpu]
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG_NAME = "lancet-accelerating-moe-training-via-whole-graph-computation-communication-overlapping_amd"

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--tokens", type=int, default=65536)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--experts", type=int, default=32)
    ap.add_argument("--no-lans", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--lans-scale", type=float, default=1.0, help="fraction of the 24-layer LANS tensor list")
    ap.add_argument("--lans-schedule", default=None, choices=["sweeps", "resident"],
                    help="time only this LANS schedule (profiling)")
    ap.add_argument("--only", default="all", choices=["all", "scatter", "scatter_dest", "decode", "decode_dest", "route", "route_forms", "copy", "stream_copy", "lans", "lans_mixed", "dgate"],
                    help="profiling aid: run just one kernel family (prints a short JSON line)")
    return ap.parse_args()


def event_ms(fn, iters):
    """Average duration in ms of fn() over `iters` calls, HIP events on the launch stream."""
    import torch
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def hbm_probe(lib, iters):
    """What plain streaming kernels reach on this device, measured beside the row movers, over 1 GiB: the
    library's own probe kernels (lancet_debug_stream: one 16-byte non-temporal access per thread, workgroups in
    address order, the shape that streams fastest here) and torch's copy_ / zero_ for comparison.  The row
    movers' fractions of the 8 TB/s peak are to be read against these."""
    import ctypes as C
    import torch
    n = 1 << 30
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    p = lambda t: C.c_void_p(t.data_ptr())

    def run(kind):
        assert lib.lancet_debug_stream(kind, p(dst), p(src), n, None) == 0

    out = {"bytes": n}
    for name, kind, nbytes in (("read_GBps", 0, n), ("fill_GBps", 1, n), ("copy_GBps", 2, 2 * n)):
        run(kind)
        out[name] = round(nbytes / event_ms(lambda: run(kind), iters) / 1e6, 1)
    dst.copy_(src), dst.zero_()
    out["torch_copy_GBps"] = round(2 * n / event_ms(lambda: dst.copy_(src), iters) / 1e6, 1)
    out["torch_fill_GBps"] = round(n / event_ms(lambda: dst.zero_(), iters) / 1e6, 1)
    out["copy_frac_of_peak"] = round(out["copy_GBps"] / HBM_PEAK_GBS, 4)
    del src, dst
    return out


def lans_shapes(scale=1.0):
    """BASELINE config 5: 24 layers x {4 x [1024,1024], 4 x [1024] biases, 4 x [1024] norms},
    12 MoE layers x 16 experts x {[1024,4096],[4096,1024]}, final norm 2 x [1024]:
    674 tensors, 1.7115e9 parameters."""
    layers = max(1, int(round(24 * scale)))
    shapes = []
    for layer in range(layers):
        shapes += [(1024, 1024)] * 4 + [(1024,)] * 8
        if layer % 2 == 1 or layers == 1:
            shapes += [(1024, 4096), (4096, 1024)] * 16
    shapes += [(1024,)] * 2
    return shapes


def bench_lans(ops, capi, steps, warmup, scale, only_schedule=None):
    import torch
    shapes = lans_shapes(scale)
    numels = [int(torch.Size(s).numel()) for s in shapes]
    total = sum(numels)
    gen = torch.Generator(device="cuda").manual_seed(0)
    flat = {}
    for name, std in (("g", 1e-3), ("p", 0.02)):
        flat[name] = torch.empty(total, device="cuda").normal_(0, std, generator=gen)
    flat["m"] = torch.zeros(total, device="cuda")
    flat["v"] = torch.zeros(total, device="cuda")
    views = {k: list(torch.split(t, numels)) for k, t in flat.items()}
    hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
    state = {"step": 1}
    timed = {}
    default = None
    for name, schedule in (("default", None), ("sweeps", capi.LANS_SWEEPS), ("resident", capi.LANS_RESIDENT)):
        if only_schedule and name != only_schedule:
            continue
        plan = ops.LansPlan(numels)
        if schedule is None:      # what a new plan runs
            default = "resident" if plan.schedule() == capi.LANS_RESIDENT else "sweeps"
            plan.close()
            continue
        try:
            plan.set_schedule(schedule)
        except RuntimeError:      # no tensor fits the resident schedule on this device
            plan.close()
            continue

        def one():
            plan.step(views["g"], views["p"], views["m"], views["v"], state["step"], hyper)
            state["step"] += 1

        for _ in range(warmup):
            one()
        timed[name] = event_ms(one, steps)
        if plan.error() != 0:
            raise RuntimeError("LANS schedule %s flagged a wait that gave up" % name)
        plan.close()
    primary = default if default in timed else min(timed, key=timed.get)
    ms = timed[primary]
    gbs = 28.0 * total / (ms * 1e-3) / 1e9
    mixed = None
    if not only_schedule:
        mixed = bench_lans_mixed(ops, capi, numels, flat, views, hyper, state, steps, warmup, ms)
    # the ceiling: what the memory system gives a kernel with the step's access pattern and none of its
    # dependencies (4 arrays read, 3 written, one float4 per thread and array), over the same number of elements
    import ctypes as C
    lib = capi.load()
    n4 = total // 1024 * 1024
    ptr = lambda t: C.c_void_p(t.data_ptr())
    keep = {k: flat[k].clone() for k in ("p", "m", "v")}

    def plain():
        assert lib.lancet_debug_stream_4r3w(ptr(flat["g"]), ptr(flat["p"]), ptr(flat["m"]), ptr(flat["v"]), n4, None) == 0

    plain()
    ceiling_ms = event_ms(plain, max(steps, 3))
    for k in keep:
        flat[k].copy_(keep[k])
    ceiling_gbs = 28.0 * n4 / (ceiling_ms * 1e-3) / 1e9
    traffic = profile_figure("lans_traffic_bytes_per_param")
    return {"tensors": len(shapes), "params": total, "ms_per_step": round(ms, 4), "schedule": primary,
            "schedule_is_default": primary == default,
            "ms_per_step_by_schedule": {k: round(v, 4) for k, v in timed.items()},
            "algorithmic_GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "bytes_per_param_algorithmic": 28,
            "ceiling": {"what": "plain 4-read/3-write streaming kernel over the same elements, timed in this run",
                        "ms": round(ceiling_ms, 4), "GBps": round(ceiling_gbs, 1),
                        "frac_of_hbm_peak": round(ceiling_gbs / HBM_PEAK_GBS, 4),
                        "step_over_ceiling": round(ms / ceiling_ms, 4)},
            # HBM bytes per parameter from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload
            # (profiles/lans_traffic.json); null when that file is absent
            "bytes_per_param_traffic_measured": traffic,
            "bytes_per_param_traffic_source": "profiles/lans_traffic.json (rocprofv3 --pmc runs of this workload; not measured by this process)",
            "mixed_precision": mixed,
            "steps": steps}


def bench_lans_mixed(ops, capi, numels, flat, views, hyper, state, steps, warmup, ms_fp32):
    """The step of a bf16 model on the same tensor list: bf16 gradients read as they are, fp32 master parameters
    and moments, and the bf16 copy of every new parameter written by the same kernel (lancet_lans_step_mixed):
    2 + 24 + 2 = 28 bytes per parameter.  Beside it the three-pass form the reference's optimizer runs
    (python/raf/optim/lans.py:256-257, 285-288): cast the gradients to fp32, the fp32 step, cast the new parameters
    to bf16, here with one torch cast over each flat array (6 + 28 + 6 = 40 bytes per parameter)."""
    import torch
    total = sum(numels)
    g16 = flat["g"].to(torch.bfloat16)
    low = torch.empty(total, dtype=torch.bfloat16, device="cuda")
    g16_views, low_views = list(torch.split(g16, numels)), list(torch.split(low, numels))
    plan = ops.LansPlan(numels)

    def one():
        plan.step(g16_views, views["p"], views["m"], views["v"], state["step"], hyper, p_lowp=low_views)
        state["step"] += 1

    for _ in range(warmup):
        one()
    ms = event_ms(one, steps)
    if plan.error() != 0:
        raise RuntimeError("the mixed-precision LANS step flagged a wait that gave up")
    if not torch.equal(low, flat["p"].to(torch.bfloat16)):
        raise RuntimeError("16-bit parameter copies differ from the rounded master parameters")
    schedule = "resident" if plan.schedule() == capi.LANS_RESIDENT else "sweeps"
    plan.close()
    g32 = torch.empty(total, device="cuda")
    plan32 = ops.LansPlan(numels)
    g32_views = list(torch.split(g32, numels))

    def three_pass():
        g32.copy_(g16)
        plan32.step(g32_views, views["p"], views["m"], views["v"], state["step"], hyper)
        low.copy_(flat["p"])
        state["step"] += 1

    for _ in range(warmup):
        three_pass()
    ms3 = event_ms(three_pass, steps)
    plan32.close()
    gbs = 28.0 * total / (ms * 1e-3) / 1e9
    return {"what": "bf16 gradients in, fp32 master p / m / v, bf16 copies of the new parameters out, one pass",
            "schedule": schedule, "ms_per_step": round(ms, 4), "bytes_per_param_algorithmic": 28,
            "algorithmic_GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "three_pass_form": {"what": "torch cast of the flat bf16 gradients to fp32, the fp32 step, torch cast of the "
                                        "flat new parameters to bf16 (40 bytes per parameter)",
                                "ms_per_step": round(ms3, 4), "bytes_per_param": 40,
                                "GBps_of_its_own_bytes": round(40.0 * total / (ms3 * 1e-3) / 1e9, 1)},
            "speedup_over_three_pass": round(ms3 / ms, 3), "ms_fp32_step": round(ms_fp32, 4),
            # from rocprofv3 --pmc runs of `--only lans_mixed` (profiles/lans_traffic.json), not measured by this process
            "bytes_per_param_traffic_measured": (profile_figure("lans_traffic_bytes_per_param") or {}).get("resident_mixed_bf16")}


def profile_figure(key):
    """A figure that comes from a profiler run rather than from this process: read from profiles/*.json."""
    import json
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "lans_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(key)
    except (OSError, ValueError):
        return None


def headline_inputs(S, M, E):
    """The headline's host arrays: NumPy default_rng(0), generation order data then logits, both N(0,1) fp32; the token
    rows rounded to bf16 (nearest even).  The same arrays are uploaded for the GPU legs and timed by the CPU baseline."""
    import numpy as np
    from oracle import moe_oracle as mo
    rng = np.random.default_rng(0)
    data_bits = mo.f32_to_bf16_bits(rng.standard_normal((S, M), dtype=np.float32))
    logits = rng.standard_normal((S, E), dtype=np.float32)
    return data_bits, logits


def cpu_baseline(data_bits, logits, cf, budget_s=10.0):
    """The CPU restatement of the reference's algorithm timed on the host cores of this box, on the arrays the GPU
    legs ran on: whole top-2 encode + decode passes of the C restatement (oracle/c/lancet_oracle.c) with all the
    cores this process may use (repeated until the time budget is used, at least 2 passes, median) and with one
    thread (2 passes); and the NumPy restatement in the style of the reference's own test references (one-hot +
    cumsum locations, Python scatter loop; one core) on BASELINE config 1, the case the reference's CPU path runs."""
    import numpy as np
    from oracle import c_oracle, moe_oracle as mo
    S, M = data_bits.shape
    E = logits.shape[1]
    cores = len(os.sched_getaffinity(0))
    Cap = mo.capacity(S, E, 2 * cf)

    def c_passes(threads, budget, most):
        c_oracle.set_num_threads(threads)
        times = []
        t_all = time.perf_counter()
        while len(times) < 2 or (time.perf_counter() - t_all < budget and len(times) < most):
            t0 = time.perf_counter()
            g, il, _, _, disp = c_oracle.moe_encode(data_bits, logits, None, Cap, 2, True)
            out = c_oracle.moe_decode(disp, g, il, 2)
            times.append(time.perf_counter() - t0)
            del out, disp
        return sorted(times)[len(times) // 2], len(times)

    t_all, n_all = c_passes(cores, budget_s, 50)
    t_one, n_one = c_passes(1, 0.0, 2)
    c_oracle.set_num_threads(cores)
    # config 1: S=4096, M=768 fp32, E=8, top-1, cf 1.25 (C=640), seed 0, data then logits
    rng = np.random.default_rng(0)
    d1 = rng.standard_normal((4096, 768), dtype=np.float32)
    l1 = rng.standard_normal((4096, 8), dtype=np.float32)
    times = []
    for _ in range(6):   # 1 warm-up + median of 5
        t0 = time.perf_counter()
        g, il, _, _, disp = mo.moe_encode(d1, l1, np.zeros(8, np.int32), 1.25, gate_is_logits=True)
        mo.moe_decode(disp, g, il, k=1)
        times.append(time.perf_counter() - t0)
    t_np = sorted(times[1:])[2]
    numpy_more = numpy_side_configs()
    return {"value": round(S / t_all, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "C/OpenMP restatement, %d whole top-2 encode+decode passes over the headline's own arrays "
                      "(S=%d M=%d E=%d, median %.3f s per pass, %d threads)" % (n_all, S, M, E, t_all, cores),
            "threads_all": {"threads": cores, "s_per_pass": round(t_all, 4), "tokens_per_s": round(S / t_all, 1), "passes": n_all},
            "threads_1": {"threads": 1, "s_per_pass": round(t_one, 4), "tokens_per_s": round(S / t_one, 1), "passes": n_one},
            "numpy_config1": {"what": "NumPy restatement in the reference tests' style (one-hot + cumsum, Python scatter "
                                      "loop), top-1 encode + decode, S=4096 M=768 fp32 E=8 C=640, one core, median of 5",
                              "s_per_pass": round(t_np, 4), "tokens_per_s": round(4096 / t_np, 1)},
            "numpy_config2": numpy_more.get("config2"), "numpy_config3": numpy_more.get("config3")}


def numpy_side_configs(limit_s=60.0):
    """The NumPy restatement (reference tests' style, one core) on BASELINE configs 2 and 3, encode + decode per pass:
    one warm-up pass, then the median of 3, unless the warm-up alone shows that the leg would not finish within
    limit_s (then the record says so)."""
    import numpy as np
    from oracle import moe_oracle as mo
    out = {}

    def leg(name, what, S, make, run):
        args = make()
        t0 = time.perf_counter()
        run(*args)
        first = time.perf_counter() - t0
        if first * 4 > limit_s:
            out[name] = {"what": what, "skipped": "one pass takes %.1f s: four would not finish within %.0f s" % (first, limit_s)}
            return
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            run(*args)
            times.append(time.perf_counter() - t0)
        t = sorted(times)[1]
        out[name] = {"what": what, "s_per_pass": round(t, 4), "tokens_per_s": round(S / t, 1)}

    def make2():
        rng = np.random.default_rng(0)
        S, M, E = 16384, 1024, 16
        data = rng.standard_normal((S, M), dtype=np.float32)
        logits = rng.standard_normal((S, E), dtype=np.float32)
        r = np.arange(1, E + 1, dtype=np.float64)
        bias = 3.0 * (r ** -1.2 - E ** -1.2) / (1.0 - E ** -1.2)
        return data, (logits + bias[rng.permutation(E)].astype(np.float32)[None, :]).astype(np.float32)

    def run2(data, logits):
        g, il, _, _, disp = mo.moe_encode_top2(data, logits, np.zeros(16, np.int32), 1.0, gate_is_logits=True)
        mo.moe_decode(disp, g, il, k=2)

    def make3():
        rng = np.random.default_rng(0)
        S, M, E = 32768, 2048, 64
        data = mo.round_to_bf16(rng.standard_normal((S, M), dtype=np.float32))
        return data, mo.softmax_rows(rng.standard_normal((S, E), dtype=np.float32) * np.float32(2.0))

    def run3(data, gate):
        g, il, _, _, disp = mo.moe_encode_bpr(data, gate, 1, 0, 1.25)
        mo.moe_decode(disp, g, il, k=1)

    leg("config2", "top-2 encode + decode, S=16384 M=1024 fp32 E=16 C=2048, Zipf expert bias, one core", 16384, make2, run2)
    leg("config3", "batch-prioritised encode + decode, S=32768 M=2048 (bf16 values held as fp32) E=64 C=640, one core",
        32768, make3, run3)
    return out


def host_memory_available_gb():
    """MemAvailable of /proc/meminfo in GB (0 when it cannot be read)."""
    try:
        with open("/proc/meminfo") as f:
            for line in f:
                if line.startswith("MemAvailable:"):
                    return int(line.split()[1]) * 1024 / 1e9
    except (OSError, ValueError):
        pass
    return 0.0


def cpu_baseline_lans(hyper_steps=2):
    """C/OpenMP LANS on the host: the whole 674-tensor list of config 5 when the host has 48 GB available (the four
    arrays take 27.4 GB), else the 32 expert tensors of one MoE layer (134M parameters); the record says which."""
    import numpy as np
    from oracle import c_oracle
    cores = len(os.sched_getaffinity(0))
    c_oracle.set_num_threads(cores)
    avail = host_memory_available_gb()
    full = avail >= 48.0
    shapes = lans_shapes(1.0) if full else [(1024, 4096), (4096, 1024)] * 16
    rng = np.random.default_rng(0)
    # one random draw per distinct shape, copied to every tensor of that shape: the time of a step does not depend
    # on the values, and drawing 3.4e9 normals would take longer than the timed steps
    draw = {}
    for sh in set(shapes):
        draw[sh] = (rng.standard_normal(sh, dtype=np.float32) * np.float32(0.02), rng.standard_normal(sh, dtype=np.float32) * np.float32(1e-3))
    p = [draw[sh][0].copy() for sh in shapes]
    g = [draw[sh][1].copy() for sh in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    total = sum(a.size for a in p)
    scratch = np.empty(2 * max(a.size for a in p), np.float32)
    c_oracle.lans_step(g, p, m, v, 1, scratch=scratch)
    t0 = time.perf_counter()
    for k in range(hyper_steps):
        c_oracle.lans_step(g, p, m, v, 2 + k, scratch=scratch)
    dt = (time.perf_counter() - t0) / hyper_steps
    return {"params": total, "tensors": len(shapes), "ms_per_step": round(dt * 1e3, 2), "cores": cores,
            "algorithmic_GBps": round(28.0 * total / dt / 1e9, 2), "ns_per_param": round(dt / total * 1e9, 3),
            "kind": "port", "host_memory_available_GB": round(avail, 1),
            "sample": ("C/OpenMP restatement, the whole config 5 list (674 tensors), %d timed steps after one warm-up" % hyper_steps) if full
            else "C/OpenMP restatement, one MoE layer's 32 expert tensors (the host has less than 48 GB available for the whole list)"}


def bench_config4_partitioned(pkg, ops, lib, capi, data, logits, S, M, E, cf, iters):
    """BASELINE config 4 as configured: 4 token partitions x 2 slots encoded in capacity order
    (s1p0..s1p3, s2p0..s2p3) with chained used capacity, moe_merge_masks, moe_redispatch, moe_decode.
    Per-slot gate arrays are prepared outside the timed region."""
    import ctypes as C
    import torch
    P = 4
    Sp = S // P
    sel = torch.empty((2, S), dtype=torch.int32, device="cuda")
    val = torch.empty((2, S), dtype=torch.float32, device="cuda")
    assert lib.lancet_gate_topk(C.c_void_p(logits.data_ptr()), None, S, E, 2, capi.F32, capi.GATE_IS_LOGITS,
                                C.c_void_p(sel.data_ptr()), C.c_void_p(val.data_ptr()), None) == 0
    gates, parts = [], []
    for slot in range(2):
        for pi in range(P):
            sl = slice(pi * Sp, (pi + 1) * Sp)
            g = torch.full((Sp, E), -1.0, device="cuda")
            g.scatter_(1, sel[slot, sl].long()[:, None], val[slot, sl][:, None])
            gates.append(g)
            parts.append(data[sl])
    Cap = ops.moe_capacity(Sp, E, 2 * cf * P)
    outs = [(torch.empty(Sp, device="cuda"), torch.empty((2, Sp), dtype=torch.int32, device="cuda"),
             torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
             torch.empty((E, Cap, M), dtype=data.dtype, device="cuda")) for _ in range(2 * P)]
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(Sp, E, 1))
    zero = torch.zeros(E, dtype=torch.int32, device="cuda")
    merged = torch.empty((2, 2 * S), dtype=torch.int32, device="cuda")
    red = torch.empty((E, Cap, M), dtype=data.dtype, device="cuda")
    dec = torch.empty((S, M), dtype=data.dtype, device="cuda")
    mws = torch.empty(1 << 16, dtype=torch.uint8, device="cuda")

    def encodes():
        used = zero
        for i in range(2 * P):
            ops.moe_encode(parts[i], gates[i], used, 2 * cf * P, zero_tail=False, workspace=ws, out=outs[i])
            used = outs[i][2]

    ils = [o[1] for o in outs]
    bufs = [o[4] for o in outs]

    def merge():
        ops.moe_merge_masks(ils, E, workspace=mws, out=merged)

    def redispatch():
        ops.moe_redispatch(bufs, ils, workspace=mws, out=red)

    encodes(), merge(), redispatch()
    weights = ops.moe_top2_normalize_gates(torch.cat([o[0] for o in outs]), merged)

    def decode():
        ops.moe_decode(red, weights, merged, top_k=2, out=dec)

    t = {name: event_ms(fn, iters) for name, fn in (("encode_x8", encodes), ("merge_masks", merge),
                                                     ("redispatch", redispatch), ("decode", decode))}

    # the same eight encodes writing straight into one shared buffer (rows behind those of the earlier
    # calls, the last call zero-fills what is left): no redispatch pass
    shared_outs = [o[:4] + (red,) for o in outs]

    def encodes_shared():
        used = zero
        for i in range(2 * P):
            ops.moe_encode(parts[i], gates[i], used, 2 * cf * P, zero_tail=(i == 2 * P - 1), rows_at_used=True,
                           workspace=ws, out=shared_outs[i])
            used = outs[i][2]

    want_red = red.clone()
    encodes_shared()
    if not torch.equal(red, want_red):
        raise RuntimeError("shared-buffer encodes differ from moe_redispatch")
    t_shared = event_ms(encodes_shared, iters)

    # the whole sequences in one timed region, launched op by op and replayed from a captured graph (no host
    # work between launches: what a compiled caller sees)
    def sequence():
        encodes(), merge(), redispatch(), decode()

    def sequence_shared():
        encodes_shared(), merge(), decode()

    def graph_ms(fn):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        return event_ms(g.replay, iters)

    seq = {"ms_sequence": round(event_ms(sequence, iters), 4), "ms_graph_replay": round(graph_ms(sequence), 4)}
    seq_shared = {"ms_sequence": round(event_ms(sequence_shared, iters), 4),
                  "ms_graph_replay": round(graph_ms(sequence_shared), 4)}
    if not torch.equal(red, want_red):
        raise RuntimeError("graph replay of the shared-buffer encodes differs from moe_redispatch")
    # the same partitions with the batch routed once: one top-2 routing call over all S tokens (the gate is
    # all it needs), then one scatter per partition straight to the final rows (each token row read once for
    # both slots) and one decode per partition; no merge_masks, no redispatch
    r_g = torch.empty(2 * S, device="cuda")
    r_il = torch.empty((2, 2 * S), dtype=torch.int32, device="cuda")
    r_used = torch.empty(E, dtype=torch.int32, device="cuda")
    r_elems = torch.empty(E, dtype=torch.int64, device="cuda")
    r_ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, 2))
    r_buf = torch.full_like(red, 9.0)
    r_dec = torch.empty_like(dec)

    def routed_once():
        ops.moe_route(logits, None, M, cf, top_k=2, gate_is_logits=True, workspace=r_ws, out=(r_g, r_il, r_used, r_elems))
        for pi in range(P):
            ops.moe_scatter_tokens(data[pi * Sp:(pi + 1) * Sp], r_il, None, r_used, pi * Sp, E, Cap, top_k=2,
                                   zero_tail=(pi == P - 1), out=r_buf)
        for pi in range(P):
            ops.moe_decode_tokens(r_buf, r_g, r_il, pi * Sp, Sp, top_k=2, out=r_dec[pi * Sp:(pi + 1) * Sp])

    routed_once()
    if not torch.equal(r_buf, want_red):
        raise RuntimeError("partition scatters of the once-routed batch differ from moe_redispatch")
    if not torch.equal(r_il[0], merged[0]) or not torch.equal(r_il[1][merged[0] >= 0], merged[1][merged[0] >= 0]):
        raise RuntimeError("whole-batch routing differs from the merged partition masks")
    decode()
    if not torch.equal(r_dec, dec):
        raise RuntimeError("partition decodes of the once-routed batch differ from moe_decode")
    seq_routed = {"ms_sequence": round(event_ms(routed_once, iters), 4), "ms_graph_replay": round(graph_ms(routed_once), 4)}

    # ... and with the exchange staged as well: every partition packs the rows it owns in the shared send buffer
    # (one range per slot and expert) and unpacks them into the shared receive buffer its decode reads
    once = pkg.pipeline.RoutedOnceMoeLayer(S, M, E, P, cf, top_k=2, dtype=data.dtype, gate_is_logits=True)
    once.run(data, logits)
    if not torch.equal(once.recv, want_red) or not torch.equal(once.out, dec):
        raise RuntimeError("routed-once pipeline with exchange differs from the merged / redispatched result")
    seq_routed["ms_with_exchange_three_streams"] = round(event_ms(lambda: once.run(data, logits), iters), 4)
    del once

    kept = int((merged[0] >= 0).sum())
    b = data.element_size()
    # algorithmic bytes: partition encodes S*E*4 + S*M*b (each token row once per slot here: x2) + kept*M*b,
    # merge 2*(kS)*8, redispatch kept*M*b + E*C*M*b, decode kept*M*b + S*M*b + kS*12
    alg = (S * E * 4 + S * M * b + kept * M * b) + 2 * (2 * S) * 8 + (kept * M * b + E * Cap * M * b) + \
          (kept * M * b + S * M * b + 2 * S * 12)
    total = sum(t.values())
    total_shared = t_shared + t["merge_masks"] + t["decode"]
    alg_shared = (S * E * 4 + 2 * S * M * b + E * Cap * M * b) + 2 * (2 * S) * 8 + (kept * M * b + S * M * b + 2 * S * 12)
    return {"workload": "4 partitions x 2 slots -> merge_masks -> redispatch -> decode, S=%d M=%d E=%d C=%d" % (S, M, E, Cap),
            "ms": {k: round(v, 4) for k, v in t.items()}, "ms_total": round(total, 4),
            "tokens_per_s": round(S / (total * 1e-3), 1), "algorithmic_bytes": alg,
            "frac_of_hbm_peak": round(alg / (total * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "whole_sequence": dict(seq, frac_of_hbm_peak_graph=round(alg / (seq["ms_graph_replay"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)),
            "shared_buffer": {"what": "the eight encodes write into one [E,C,M] buffer at their final rows "
                                      "(LANCET_ROWS_AT_USED), no redispatch pass; the buffer is verified equal",
                              "ms": {"encode_x8": round(t_shared, 4), "merge_masks": round(t["merge_masks"], 4),
                                     "decode": round(t["decode"], 4)},
                              "ms_total": round(total_shared, 4), "tokens_per_s": round(S / (total_shared * 1e-3), 1),
                              "algorithmic_bytes": alg_shared,
                              "whole_sequence": dict(seq_shared, frac_of_hbm_peak_graph=round(
                                  alg_shared / (seq_shared["ms_graph_replay"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)),
                              "frac_of_hbm_peak": round(alg_shared / (total_shared * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
            "routed_once": dict(seq_routed, what="one top-2 routing call over the whole batch, then one scatter and one "
                                "decode per partition on token ranges of that routing (lancet_moe_scatter_tokens / "
                                "_decode_tokens): rows go straight to their final places, each token row is read once; "
                                "buffer, mask and output verified equal to the merged / redispatched ones",
                                tokens_per_s=round(S / (seq_routed["ms_sequence"] * 1e-3), 1),
                                algorithmic_bytes=alg_shared - S * M * b - 2 * (2 * S) * 8,
                                frac_of_hbm_peak=round((alg_shared - S * M * b - 2 * (2 * S) * 8) /
                                                       (seq_routed["ms_sequence"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)),
            "note": "token rows are read once per slot (two passes) in this call pattern; "
                    "partition encodes write used rows only (zero_tail=False), redispatch zero-fills the merged tail.  "
                    "The sequence is 8 encodes x (2 routing kernels + 1 scatter) + merge_masks (clear, count, merge) + redispatch "
                    "(clear, count, row mover) + decode: 31 dependent launches of which 21 are minimum-length kernels of "
                    "3-10 us that the used_capacity chain serialises, so 0.12-0.15 ms of the 1.15-1.2 ms moves no rows: "
                    "0.59-0.61 of peak is this call pattern's floor, run to run.  routed_once (raf.op.moe_route + moe_scatter_tokens + "
                    "moe_decode_tokens in the op layer) is the supported form of the same dispatch."}


def bench_pipeline(pkg, data, logits, S, M, E, cf, iters):
    """Partitioned top-1 encode -> exchange (pack / unpack keyed by elements_per_expert) -> decode, 4 partitions,
    issued on one stream and on three (routing running ahead, exchange of partition i beside the scatter of
    partition i+1)."""
    layer = pkg.pipeline.PartitionedMoeLayer(S, M, E, 4, cf, dtype=data.dtype, gate_is_logits=True)
    layer.run_serial(data, logits)
    layer.run(data, logits)
    layer.run_routed_once(data, logits)
    t_serial = event_ms(lambda: layer.run_serial(data, logits), iters)
    t_piped = event_ms(lambda: layer.run(data, logits), iters)
    t_once = event_ms(lambda: layer.run_routed_once(data, logits), iters)
    return {"workload": "4 partitions, top-1, S=%d M=%d E=%d C=%d" % (S, M, E, layer.C),
            "ms_one_stream": round(t_serial, 4), "ms_three_streams": round(t_piped, 4),
            "ms_routed_once_three_streams": round(t_once, 4),
            "note": "every stage but routing is HBM-bound on one GPU, so the streams share one memory system and "
                    "the event hops cost more than the overlap returns; the pattern pays when the exchange is a real "
                    "all-to-all over xGMI"}


def bench_other_configs(ops, iters):
    """BASELINE configs 1-3 (parity-test cases) timed for reference: encode + decode per pass; config 1 also
    replayed from a captured graph, which removes the launch gaps that dominate at that size."""
    import numpy as np
    import torch
    out = {}

    def run(name, S, M, E, cf, k, dtype, bpr=False, zipf=False, scale=1.0, graph=False):
        rng = np.random.default_rng(0)
        data = torch.from_numpy(rng.standard_normal((S, M), dtype=np.float32)).cuda().to(dtype)
        logits = rng.standard_normal((S, E), dtype=np.float32) * np.float32(scale)
        if zipf:
            r = np.arange(1, E + 1, dtype=np.float64)
            bias = 3.0 * (r ** -1.2 - E ** -1.2) / (1.0 - E ** -1.2)
            logits = logits + bias[rng.permutation(E)].astype(np.float32)[None, :]
        gate = torch.from_numpy(logits.astype(np.float32)).cuda()
        if bpr:
            gate = torch.softmax(gate, dim=1)
        Cap = ops.moe_capacity(S, E, cf * k)
        bufs = (torch.empty(k * S, device="cuda"), torch.empty((2, k * S), dtype=torch.int32, device="cuda"),
                torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
                torch.empty((E, Cap, M), dtype=dtype, device="cuda"))
        ws = ops.ScanWorkspace(max(ops.moe_encode_workspace_bytes(S, E, k), ops.moe_encode_bpr_workspace_bytes(S, E, 1)))
        dec = torch.empty((S, M), dtype=dtype, device="cuda")

        def step():
            if bpr:
                ops.moe_encode_batch_prioritized(data, gate, 1, 0, cf, workspace=ws, out=bufs)
            else:
                ops.moe_encode(data, gate, None, cf, top_k=k, gate_is_logits=True, workspace=ws, out=bufs)
            ops.moe_decode(bufs[4], bufs[0], bufs[1], top_k=k, out=dec)

        step()
        ms = event_ms(step, iters)
        kept = int((bufs[1][0] >= 0).sum())
        b = data.element_size()
        alg = (S * E * 4 + S * M * b + E * Cap * M * b + k * S * 12 + E * 12) + (kept * M * b + S * M * b + k * S * 12)
        rec = {"ms": round(ms, 4), "tokens_per_s": round(S / (ms * 1e-3), 1), "kept_slots": kept, "slots": k * S,
               "algorithmic_bytes": alg, "frac_of_hbm_peak": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        if graph:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                step()
            g.replay()
            rec["ms_graph_replay"] = round(event_ms(g.replay, iters), 4)
        out[name] = rec

    run("config1_top1_fp32", 4096, 768, 8, 1.25, 1, torch.float32, graph=True)
    run("config2_top2_fp32", 16384, 1024, 16, 1.0, 2, torch.float32, zipf=True)
    run("config2_top2_bf16", 16384, 1024, 16, 1.0, 2, torch.bfloat16, zipf=True)
    run("config3_bpr_bf16", 32768, 2048, 64, 1.25, 1, torch.bfloat16, bpr=True, scale=2.0)
    return out


def bench_backward(ops, data, outs, dec, S, M, E, Cap, K, kept, iters):
    """The four backward ops at the headline shape (dy buffers reuse forward tensors as values)."""
    import torch
    b = data.element_size()
    g, il, disp = outs[0], outs[1], outs[4]
    dx = torch.empty_like(data)
    dgate = torch.empty((S, E), device="cuda")
    dbuf = torch.empty_like(disp)
    dgs = torch.empty(K * S, device="cuda")
    ws = torch.empty(E * Cap * 4, dtype=torch.uint8, device="cuda")
    logits = torch.randn((S, E), device="cuda")
    res = {}
    for name, fn, nbytes in (
            ("encode_dx", lambda: ops.moe_encode_dx(disp, il, top_k=K, out=dx), kept * M * b + S * M * b + K * S * 8),
            ("encode_dg", lambda: ops.moe_encode_dg(g, il, E, top_k=K, out=dgate), S * E * 4 + K * S * 8),
            # the gate gradient of the op the headline runs (top-2 on logits): through the normalisation and the softmax
            ("encode_dgate", lambda: ops.moe_encode_dgate(g, logits, il, top_k=K, gate_is_logits=True, out=dgate),
             2 * S * E * 4 + K * S * 8),
            ("decode_dx", lambda: ops.moe_decode_dx(dec, g, il, E, Cap, top_k=K, workspace=ws, out=dbuf),
             kept * M * b + E * Cap * M * b + K * S * 12 + 2 * E * Cap * 4),
            ("decode_dg", lambda: ops.moe_decode_dg(dec, disp, il, top_k=K, out=dgs), 2 * kept * M * b + K * S * 12)):
        fn()
        ms = event_ms(fn, iters)
        res[name] = {"ms": round(ms, 4), "algorithmic_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                     "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    return res


def bench_expert_input(ops, M, iters):
    """moe_redispatch_expert_input at the shape one of 8 expert-parallel ranks would see for BASELINE config 4:
    G = 8 source ranks, 4 local experts, capacity 5120, 4 token partitions, bf16 rows; every partition brings
    about a quarter of the rows of each source rank.  Algorithmic bytes: received rows read once, the whole
    [C, G, M] output written once (rows past the received ones are zero-filled)."""
    import torch
    P, G, LE, Cap = 4, 8, 4, 5120
    gen = torch.Generator(device="cuda").manual_seed(9)
    data = [torch.empty((Cap, G, M), device="cuda", dtype=torch.bfloat16).normal_(0, 1, generator=gen) for _ in range(P)]
    rows = torch.randint(Cap // P - 200, Cap // P, (P, G * LE), generator=gen, device="cuda")
    cnts = [(rows[p] * M).to(torch.int64) for p in range(P)]
    out = torch.empty((Cap, G, M), device="cuda", dtype=torch.bfloat16)
    fn = lambda: ops.moe_redispatch_expert_input(data, cnts, 1, LE, out=out)
    fn()
    ms = event_ms(fn, iters)
    received = int(rows.view(P, G, LE)[:, :, 1].sum())
    nbytes = received * M * 2 + Cap * G * M * 2
    return {"workload": "P=%d G=%d LE=%d C=%d M=%d bf16, local expert 1" % (P, G, LE, Cap, M), "ms": round(ms, 4),
            "received_rows": received, "algorithmic_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
            "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py measures one GPU's share of the dispatch path; this build has no multi-GPU "
            "path (no collectives are part of it). Run with --gpus 1.")
        sys.exit(2)
    import numpy as np
    import torch
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    pkg = importlib.import_module(PKG_NAME)
    ops, capi = pkg.ops, pkg.capi
    lib = capi.load()
    import ctypes as C

    if args.only == "copy":
        # calibration for the HBM byte counters: a plain copy of known size (1 GiB read + 1 GiB written)
        n = 1 << 30
        src = torch.zeros(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.warmup):
            dst.copy_(src)
        ms = event_ms(lambda: dst.copy_(src), args.steps)
        print(json.dumps({"only": "copy", "bytes_read": n, "bytes_written": n, "ms": round(ms, 4),
                          "GBps": round(2 * n / ms / 1e6, 1)}), flush=True)
        return
    if args.only == "stream_copy":
        # the library's own plain copy (lancet_debug_stream: one 16-byte non-temporal access per thread, workgroups
        # in address order) over 1 GiB: the kernel the scatter's counters are read against
        n = 1 << 30
        src = torch.zeros(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        run = lambda: lib.lancet_debug_stream(2, C.c_void_p(dst.data_ptr()), C.c_void_p(src.data_ptr()), n, None)
        for _ in range(args.warmup):
            assert run() == 0
        ms = event_ms(run, args.steps)
        print(json.dumps({"only": "stream_copy", "bytes_read": n, "bytes_written": n, "ms": round(ms, 4),
                          "GBps": round(2 * n / ms / 1e6, 1)}), flush=True)
        return
    if args.only == "route_forms":
        # Routing alone (selection + position scan, lancet_moe_route) over token and expert counts from the side
        # configurations to long batches, in the form the library picks (look-back on few tiles of top-1, else two
        # or three kernels without waits) and as one look-back kernel (LANCET_SCAN_LOOKBACK).
        rows = []
        for S, E, k in [(4096, 8, 1), (16384, 16, 2), (32768, 64, 1), (65536, 32, 2), (65536, 64, 1), (131072, 32, 2),
                        (262144, 32, 2), (65536, 256, 2), (131072, 256, 2), (262144, 64, 2), (524288, 64, 1),
                        (1048576, 16, 1), (1048576, 64, 1), (2097152, 16, 1), (262144, 256, 1), (131072, 512, 1)]:
            gate = torch.randn((S, E), device="cuda")
            out = ops.moe_route(gate, None, 8, 1.25, top_k=k, gate_is_logits=True)
            ref = [t.clone() for t in out]
            t = {}
            for name, lb in (("default", False), ("look_back", True)):
                run = lambda: ops.moe_route(gate, None, 8, 1.25, top_k=k, gate_is_logits=True, out=out, scan_lookback=lb)
                for _ in range(max(args.warmup, 2)):
                    run()
                t[name] = event_ms(run, max(args.steps, 20))
                assert all(torch.equal(a, b) for a, b in zip(out, ref)), "the forms of the scan disagree"
            tiles = (S + 255) // 256
            form = "look-back" if (k == 1 and tiles <= 32) else ("count+place" if tiles * k * E <= 32768 else "count+segsum+place")
            rows.append({"tokens": S, "experts": E, "top_k": k, "tiles": tiles, "default_form": form,
                         "gate_rows_staged": bool(tiles >= 512 and E * 4 > 128),
                         "us_default": round(t["default"] * 1e3, 1), "us_look_back": round(t["look_back"] * 1e3, 1),
                         "gate_GBps_default": round(S * E * 4 / t["default"] / 1e6, 1)})
            del gate, out, ref
        print(json.dumps({"only": "route_forms", "rows": rows}), flush=True)
        return
    if args.only == "lans":
        print(json.dumps({"only": "lans", "lans": bench_lans(ops, capi, args.steps, args.warmup, args.lans_scale,
                                                               args.lans_schedule)}),
              flush=True)
        return
    if args.only == "lans_mixed":
        # the mixed-precision step alone (bf16 gradients in, bf16 parameter copies out), for profiler runs
        shapes = lans_shapes(args.lans_scale)
        numels = [int(torch.Size(s).numel()) for s in shapes]
        total = sum(numels)
        gen = torch.Generator(device="cuda").manual_seed(0)
        g16 = torch.empty(total, device="cuda").normal_(0, 1e-3, generator=gen).to(torch.bfloat16)
        pm = torch.empty(total, device="cuda").normal_(0, 0.02, generator=gen)
        m, v = torch.zeros(total, device="cuda"), torch.zeros(total, device="cuda")
        low = torch.empty(total, dtype=torch.bfloat16, device="cuda")
        lists = [list(torch.split(t, numels)) for t in (g16, pm, m, v, low)]
        hyper = capi.LansHyper(1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1)
        plan = ops.LansPlan(numels)
        if args.lans_schedule:
            plan.set_schedule(capi.LANS_SWEEPS if args.lans_schedule == "sweeps" else capi.LANS_RESIDENT)
        state = {"step": 1}

        def one():
            plan.step(lists[0], lists[1], lists[2], lists[3], state["step"], hyper, p_lowp=lists[4])
            state["step"] += 1

        for _ in range(args.warmup):
            one()
        ms = event_ms(one, args.steps)
        assert plan.error() == 0
        print(json.dumps({"only": "lans_mixed", "params": total, "ms_per_step": round(ms, 4), "steps": args.steps + args.warmup,
                          "algorithmic_GBps": round(28.0 * total / ms / 1e6, 1)}), flush=True)
        return

    S, M, E, K, cf = args.tokens, args.hidden, args.experts, 2, 1.25
    b = 2  # bf16
    Cap = ops.moe_capacity(S, E, 2 * cf)
    h_data_bits, h_logits = headline_inputs(S, M, E)
    data = torch.from_numpy(h_data_bits.view(np.int16)).cuda().view(torch.bfloat16)
    logits = torch.from_numpy(h_logits).cuda()
    used_in = torch.zeros(E, dtype=torch.int32, device="cuda")
    outs = (torch.empty(K * S, device="cuda"), torch.empty((2, K * S), dtype=torch.int32, device="cuda"),
            torch.empty(E, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int64, device="cuda"),
            torch.empty((E, Cap, M), dtype=torch.bfloat16, device="cuda"))
    ws = ops.ScanWorkspace(ops.moe_encode_workspace_bytes(S, E, K))
    dec = torch.empty((S, M), dtype=torch.bfloat16, device="cuda")

    def encode():
        return ops.moe_encode(data, logits, used_in, cf, top_k=K, gate_is_logits=True, workspace=ws, out=outs)

    def decode():
        return ops.moe_decode(outs[4], outs[0], outs[1], top_k=K, out=dec)

    def step():
        encode()
        decode()

    # ---- parity gate at full size: routing bit-exact against the oracle, rows by properties
    from oracle import moe_oracle as mo
    step()
    torch.cuda.synchronize()
    sel, val = mo.select_topk(h_logits, 2, True)
    zero = np.zeros(E, np.int32)
    i1, l1, u1, _ = mo.gen_location(sel[0], zero, Cap, M, E)
    i2, l2, u2, _ = mo.gen_location(sel[1], u1, Cap, M, E)
    merged = mo.moe_merge_masks([np.stack([i1, l1]), np.stack([i2, l2])], E)
    il = outs[1].cpu().numpy()
    assert np.array_equal(il, merged), "routing differs from the oracle at full size"
    assert np.array_equal(outs[2].cpu().numpy(), u2)
    kept = int((merged[0] >= 0).sum())
    il_t = outs[1].long()
    for j in range(K):
        idx, loc = il_t[0, j * S:(j + 1) * S], il_t[1, j * S:(j + 1) * S]
        ok = idx >= 0
        assert torch.equal(outs[4][idx[ok], loc[ok]], data[ok]), "scattered rows differ from the token rows"
    used = outs[2].long()
    tail_mask = torch.arange(Cap, device="cuda")[None, :] >= used[:, None]
    assert not outs[4][tail_mask].any(), "rows past the used capacity are not zero"
    either = (il_t[0, :S] >= 0) | (il_t[0, S:] >= 0)
    # identity expert + normalised weights: decode returns the token (g1 + g2 = 1) within 1 unit in the last place
    # of bf16, counted on the bit patterns (sign-magnitude patterns mapped to integers in value order)
    def ordered(t):
        i = t.view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7fff), i)
    assert int((ordered(dec[either]) - ordered(data[either])).abs().max()) <= 1, "encode -> decode round trip broken"
    assert not dec[~either].any()
    log("parity gate ok: S=%d M=%d E=%d C=%d kept=%d of %d slots" % (S, M, E, Cap, kept, K * S))

    # ---- timed region: K steps, wall clock bracketed by synchronisation
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- per-op / per-kernel durations with HIP events on the launch stream
    n = max(args.steps, 10)
    ms_enc = event_ms(encode, n)
    ms_dec = event_ms(decode, n)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: C.c_void_p(t.data_ptr())

    def scatter_only():
        st = lib.lancet_moe_scatter(p(data), p(outs[1]), p(used_in), p(outs[2]), S, M, E, Cap, K, capi.BF16, 0,
                                    p(outs[4]), stream)
        assert st == 0

    def route_only():
        st = lib.lancet_moe_route(p(logits), None, p(used_in), S, M, E, Cap, K, capi.F32, capi.GATE_IS_LOGITS, p(outs[0]),
                                  p(outs[1]), p(outs[2]), p(outs[3]), p(ws.buf), ws.nbytes, stream)
        assert st == 0

    if args.only in ("scatter_dest", "decode_dest"):
        # the row movers fed with one routing word per slot (lancet_debug_scatter_dest / _decode_dest): checked equal
        # to the operator calls, then timed alone (for a counter run beside --only scatter / decode)
        il_t = outs[1]
        dest = torch.where(il_t[0] >= 0, il_t[0] * Cap + il_t[1], torch.full_like(il_t[0], -1)).contiguous()
        want = (outs[4] if args.only == "scatter_dest" else dec).clone()

        def one_word():
            if args.only == "scatter_dest":
                st = lib.lancet_debug_scatter_dest(p(data), p(dest), p(used_in), p(outs[2]), S, M, E, Cap, K, capi.BF16, p(outs[4]), stream)
            else:
                st = lib.lancet_debug_decode_dest(p(outs[4]), p(outs[0]), p(dest), S, M, E, Cap, K, capi.BF16, capi.F32, p(dec), stream)
            assert st == 0

        one_word()
        assert torch.equal(outs[4] if args.only == "scatter_dest" else dec, want), "the one-word form differs from the operator"
        for _ in range(args.warmup):
            one_word()
        ms = event_ms(one_word, args.steps)
        print(json.dumps({"only": args.only, "ms": round(ms, 4), "steps": args.steps}), flush=True)
        return
    if args.only == "dgate":
        grad = torch.empty_like(logits)
        fn = lambda: ops.moe_encode_dgate(outs[0], logits, outs[1], top_k=K, gate_is_logits=True, out=grad)
        for _ in range(args.warmup):
            fn()
        ms = event_ms(fn, args.steps)
        print(json.dumps({"only": "dgate", "ms": round(ms, 4), "steps": args.steps, "algorithmic_bytes": 2 * S * E * 4 + K * S * 8}), flush=True)
        return
    if args.only in ("scatter", "decode", "route"):
        fn = {"scatter": scatter_only, "decode": decode, "route": route_only}[args.only]
        for _ in range(args.warmup):
            fn()
        ms = event_ms(fn, args.steps)
        print(json.dumps({"only": args.only, "ms": round(ms, 4), "steps": args.steps}), flush=True)
        return
    ms_route = event_ms(route_only, n)
    encode()
    ms_scatter = event_ms(scatter_only, n)

    enc_bytes = S * E * 4 + S * M * b + E * Cap * M * b + K * S * 12 + E * 12
    dec_bytes = kept * M * b + S * M * b + K * S * 12
    scatter_bytes = S * M * b + E * Cap * M * b + K * S * 8 + E * 8
    gbs = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    scatter_gbs = gbs(scatter_bytes, ms_scatter)
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "scatter_rows_headline_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")

    result = {
        "metric": "moe_dispatch_tokens_per_sec_encode_plus_decode",
        "value": round(S / (ms_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "un-partitioned top-2 moe_encode + moe_decode, S=%d M=%d bf16 E=%d C=%d "
                               "(BASELINE config 4 shape, headline)" % (S, M, E, Cap),
                   "tokens": S, "hidden": M, "experts": E, "capacity": Cap, "top_k": K,
                   "kept_slots": kept, "gate": "fp32 logits, softmax fused"},
        "roofline": {"bound": "hbm", "kernel": "scatter_rows_kernel<u32x4,2> (encode_forward)",
                     "achieved": round(scatter_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(scatter_gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": "profiles/scatter_rows_headline_traffic.json: HBM bytes per launch from rocprofv3 --pmc "
                                       "FETCH_SIZE / WRITE_SIZE runs of this workload (a stored figure, not measured by this process)",
                     "algorithmic_bytes_per_launch": scatter_bytes, "avg_launch_ms": round(ms_scatter, 4)},
        "ops": {
            "encode": {"ms": round(ms_enc, 4), "algorithmic_bytes": enc_bytes,
                       "GBps": round(gbs(enc_bytes, ms_enc), 1),
                       "frac": round(gbs(enc_bytes, ms_enc) / HBM_PEAK_GBS, 4)},
            "decode": {"ms": round(ms_dec, 4), "algorithmic_bytes": dec_bytes,
                       "GBps": round(gbs(dec_bytes, ms_dec), 1),
                       "frac": round(gbs(dec_bytes, ms_dec) / HBM_PEAK_GBS, 4)},
            "route_scan": {"ms": round(ms_route, 4)},
            "encode_plus_decode_frac": round(gbs(enc_bytes + dec_bytes, ms_enc + ms_dec) / HBM_PEAK_GBS, 4),
        },
    }
    result["hbm_probe"] = hbm_probe(lib, n)
    result["backward"] = bench_backward(ops, data, outs, dec, S, M, E, Cap, K, kept, n)
    del dec, outs
    torch.cuda.empty_cache()
    result["config4_partitioned"] = bench_config4_partitioned(pkg, ops, lib, capi, data, logits, S, M, E, cf, max(5, n // 2))
    result["expert_input_merge"] = bench_expert_input(ops, M, max(10, n))
    result["pipeline"] = bench_pipeline(pkg, data, logits, S, M, E, cf, max(5, n // 2))
    result["other_configs"] = bench_other_configs(ops, max(10, n))
    del data
    torch.cuda.empty_cache()
    if not args.no_lans:
        result["lans"] = bench_lans(ops, capi, max(3, min(args.steps, 10)), max(1, min(args.warmup, 2)),
                                    args.lans_scale)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(h_data_bits, h_logits, cf)
        if "lans" in result:
            result["lans"]["cpu_baseline"] = cpu_baseline_lans()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()

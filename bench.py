#!/usr/bin/env python3
"""Benchmark of the Q8_0 decode GEMV path on one MI355X.

A "step" is one token-step of the Qwen3-0.6B projection set at decode batch B:
(q, k, v, o, gate, up, down) x 28 layers + the tied 151936-row lm_head = 197
Q8_0 x Q8_0 GEMVs over 633 MB of distinct weights (more than the 256 MB
Infinity Cache, so every step streams from HBM).  Weights and quantized
activations are resident in HBM before the timed region starts.

  --mode grouped     (default) the whole projection set in ONE launch of the GEMV kernel
  --mode per_matmul  197 launches per step, one per matrix (the call pattern of the Kernel trait)
  --mode layer       113 launches per step: [q,k,v] [o] [gate,up] [down] per layer + lm_head,
                     the grouping a dependent decode step allows

Prints one JSON line.  `value` = algorithmic bytes per step / wall time per step.
`roofline` prices the GEMV kernel from two HIP events recorded on the launch
stream at the two ends of the timed region (launch gaps included).  `cpu_baseline` times the restated reference CPU path
(the checker's AVX2 kernels over a persistent-thread row partition) on the same
weights and activations in this process.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
HBM_PEAK_GBS = 8000.0
INT8_MFMA_PEAK_TOPS = 5000.0  # dense int8 MFMA


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class HipEvents:
    """hipEvent timing on a given stream (the null stream here), via libamdhip64."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]

    def create(self):
        ev = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(ev)) == 0
        return ev

    def record(self, ev, stream=None):
        assert self.hip.hipEventRecord(ev, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return ms.value


def physical_cores():
    try:
        seen = set()
        phys = core = None
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":")[1].strip()
            elif line.startswith("core id"):
                core = line.split(":")[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    seen.add((phys, core))
                phys = core = None
        if seen:
            return len(seen)
    except OSError:
        pass
    return os.cpu_count() or 1


THREADS_OVERRIDE = None  # --threads


def cpu_threads():
    """Threads of the CPU legs: the host's physical core count, unless the job's own CPU share is smaller.  The
    share is what OMP_NUM_THREADS says (the scheduler of a shared GPU host sets it to the cores that belong to the
    job, and asks worker pools to stay within it whatever /proc/cpuinfo shows); --threads overrides both."""
    detected = physical_cores()
    info = {"physical_cores_detected": detected, "logical_cpus": os.cpu_count()}
    if THREADS_OVERRIDE:
        info.update(threads_used=THREADS_OVERRIDE, thread_cap=None, thread_cap_source="--threads")
        return THREADS_OVERRIDE, info
    cap = None
    try:
        cap = int(os.environ.get("OMP_NUM_THREADS", ""))
    except ValueError:
        pass
    used = min(detected, cap) if cap and cap > 0 else detected
    info.update(threads_used=used, thread_cap=cap,
                thread_cap_source="OMP_NUM_THREADS: this job's share of the host's cores" if cap else None)
    return used, info


def build_projection_set(pkg, batch, keep_host):
    """Uploads the 197 weights and their quantized activations; returns problem records."""
    synth, K, H = pkg.synth, pkg.kernel, pkg.hip
    shapes = []
    for layer in range(synth.QWEN3_0_6B_LAYERS):
        for name, n_out, n_in in synth.QWEN3_0_6B_LAYER:
            shapes.append((f"blk.{layer}.{name}", n_out, n_in, layer))
    name, n_out, n_in = synth.QWEN3_0_6B_LM_HEAD
    shapes.append((name, n_out, n_in, -1))
    problems = []
    t0 = time.time()
    for i, (name, n_out, n_in, layer) in enumerate(shapes):
        w = synth.q8_0_weight(synth.seed_for(1, i), n_out, n_in)
        x = synth.activations(synth.seed_for(1, 0x8000 + i), batch, n_in)
        kernel = K.Q8Kernel(w, n_in, n_out)
        d_x = H.DeviceBuffer.from_array(x)
        d_q8 = H.DeviceBuffer(batch * n_in)
        d_sc = H.DeviceBuffer(batch * (n_in // 32) * 4)
        d_y = H.DeviceBuffer(batch * n_out * 4)
        # the activation is quantized by the device quantizer (x86-64 rounding), as a decode step would
        H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q8.ptr, d_sc.ptr, batch, n_in, H.ROUND_TIES_EVEN, None))
        H.check(H.lib.rmi_hip_synchronize())
        rec = dict(name=name, n_out=n_out, n_in=n_in, layer=layer, kernel=kernel, d_q8=d_q8, d_sc=d_sc, d_y=d_y)
        if keep_host:
            rec["w"] = w
            rec["q8"] = d_q8.to_array(np.uint8, (batch, n_in))
            rec["sc"] = d_sc.to_array(np.float32, (batch, n_in // 32))
        d_x.free()
        problems.append(rec)
    log(f"[bench] uploaded {len(problems)} weights in {time.time() - t0:.1f}s")
    return problems


def make_group(H, recs, batch, order="avx2"):
    n = len(recs)
    arr = lambda vals: (C.c_void_p * n)(*vals)  # noqa: E731
    create = H.lib.rmi_hip_gemv_group_create_neon if order == "neon" else H.lib.rmi_hip_gemv_group_create
    g = create(n, arr([r["kernel"].w.handle for r in recs]), arr([r["d_q8"].ptr for r in recs]),
               arr([r["d_sc"].ptr for r in recs]), arr([r["d_y"].ptr for r in recs]), batch)
    if not g:
        raise RuntimeError(H.last_error())
    return g


def group_maxt(H, g):
    """Third template argument of the kernel a group launches: 64 (one wave per workgroup) or 512."""
    wg, waves = C.c_uint32(), C.c_uint32()
    H.check(H.lib.rmi_hip_gemv_group_shape(g, C.byref(wg), C.byref(waves)))
    return "64" if waves.value == 1 else "512"


def layer_groups(H, problems, batch, order="avx2"):
    """[q,k,v] [o] [gate,up] [down] per layer, then lm_head: what a dependent decode step can fuse."""
    groups = []
    by_layer = {}
    for r in problems:
        by_layer.setdefault(r["layer"], []).append(r)
    for layer in sorted(k for k in by_layer if k >= 0):
        rs = {r["name"].split(".")[-1]: r for r in by_layer[layer]}
        for names in (("attn_q", "attn_k", "attn_v"), ("attn_output",), ("ffn_gate", "ffn_up"), ("ffn_down",)):
            groups.append(make_group(H, [rs[n] for n in names], batch, order))
    groups.append(make_group(H, by_layer[-1], batch, order))
    return groups


def cpu_baseline(problems, batch, alg_bytes):
    """The restated reference CPU path on the same weights: 10 warm-ups, 15 samples, median
    (the reference's methodology, src/bin/micro_bench.rs:32-33, 94-152)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import rmi_oracle as oracle

    if not oracle.have_avx2():
        return None
    cores, core_info = cpu_threads()
    pool = oracle.Pool(cores)
    outs = [np.zeros((batch, r["n_out"]), np.float32) for r in problems]

    def step():
        for r, out in zip(problems, outs):
            pool.matmul_q8_0(r["w"], r["q8"], r["sc"], out, r["n_in"], r["n_out"], batch)

    t_budget = time.time()
    for _ in range(10):
        step()
        if time.time() - t_budget > 20:
            break
    samples = []
    for _ in range(15):
        t0 = time.perf_counter()
        step()
        samples.append(time.perf_counter() - t0)
        if time.time() - t_budget > 40:
            break
    pool.close()
    med = statistics.median(samples)
    return {
        "value": round(alg_bytes / med / 1e9, 2),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{len(samples)} full token-steps (197 GEMVs, {alg_bytes / 1e6:.0f} MB each) after warm-up, median; "
                  f"restated reference AVX2 kernels, (ith,nth) row partition over {cores} persistent threads",
        "ms_per_step": round(med * 1e3, 3),
        "token_steps_per_s": round(1.0 / med, 2),
        **core_info,
    }, outs


def gemv_kernel_name(batch):
    """The x86-64-order GEMV the library launches for this many tokens: from four on, the one with its dots on the
    matrix cores."""
    return "gemv_q8_0_x4_kernel" if batch >= 4 else "gemv_q8_0_kernel"


def read_traffic(name, case=""):
    """HBM bytes per launch as rocprofv3 --pmc measured them when profiles/<name>_pmc.txt was recorded: a figure
    read back from that file, not measured by this run.  A file that covers several workloads names the case in the
    key ("traffic_bytes_per_launch_m512:").  Returns {"traffic": bytes or None, "traffic_source": ..}."""
    rel = os.path.join("profiles", f"{name}_pmc.txt")
    key = f"traffic_bytes_per_launch{'_' + case if case else ''}:"
    try:
        for line in open(os.path.join(ROOT, rel)):
            if line.startswith(key):
                return {"traffic": float(line.split(":")[1]),
                        "traffic_source": f"{rel} (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, recorded earlier; "
                                          "not measured in this run)"}
    except OSError:
        pass
    return {"traffic": None, "traffic_source": None}


def copy_calibration(H, args):
    """A plain copy kernel of known size, five launches: what rocprofv3 --pmc traffic counters are scaled against."""
    if not args.copy_calibration_mb:
        return
    nbytes = args.copy_calibration_mb << 20
    src, dst = H.DeviceBuffer(nbytes), H.DeviceBuffer(nbytes)
    for _ in range(5):
        H.check(H.lib.rmi_hip_copy_dev(dst.ptr, src.ptr, nbytes, None))
    H.check(H.lib.rmi_hip_synchronize())
    src.free()
    dst.free()


SETTLE_MS = 150.0  # least device time of the settling phase, ms
# Untimed steps of the last time_region call that asked for settled clocks (beyond its W warm-up steps).
LAST_SETTLE_STEPS = 0


def settle(H, ev, fn, min_ms, max_ms=1000.0, chunk=20):
    """Untimed steps until the device's clocks have settled under this load: chunks of `chunk` steps until at least
    `min_ms` of device time have passed and three chunks in a row lie within 1 % (at most `max_ms`).  The chip
    raises its clocks over the first tens of milliseconds of a compute-bound load: the tiled GEMM at 2048 tokens
    takes 53 us a step in its second 50 steps and 43.5 us from the 600th on; an HBM-bound launch does not change."""
    ev_a, ev_b = ev.create(), ev.create()
    total, n, last = 0.0, 0, []
    while total < max_ms:
        ev.record(ev_a)
        for _ in range(chunk):
            fn()
        ev.record(ev_b)
        H.check(H.lib.rmi_hip_synchronize())
        ms = ev.elapsed_ms(ev_a, ev_b)
        total += ms
        n += chunk
        last = (last + [ms / chunk])[-3:]
        if total >= min_ms and len(last) == 3 and max(last) - min(last) <= 0.01 * min(last):
            break
    return n


def time_region(H, ev, fn, steps, warmup, settle_ms=0.0):
    """W untimed warm-up steps (and, with settle_ms, further untimed steps until the clocks have settled: their
    number is left in LAST_SETTLE_STEPS), then exactly K timed steps between a device synchronisation on both sides.
    Returns (host wall seconds per step, device ms per step from two HIP events on the launch stream)."""
    global LAST_SETTLE_STEPS
    for _ in range(warmup):
        fn()
    LAST_SETTLE_STEPS = settle(H, ev, fn, settle_ms) if settle_ms else 0
    ev_a, ev_b = ev.create(), ev.create()
    H.check(H.lib.rmi_hip_synchronize())
    t0 = time.perf_counter()
    ev.record(ev_a)
    for _ in range(steps):
        fn()
    ev.record(ev_b)
    H.check(H.lib.rmi_hip_synchronize())
    wall = (time.perf_counter() - t0) / steps
    return wall, ev.elapsed_ms(ev_a, ev_b) / steps


def base_result(args, metric, unit, value, wall, dtype, config):
    return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(wall * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": config}


def run_projection_set(args, pkg, ev):
    H, synth = pkg.hip, pkg.synth
    dev_name, cus, hbm = H.device_info()
    batch = args.batch
    neon = args.order == "neon"  # the small-batch MFMA kernel; the CPU leg below restates the AVX2 order only
    want_cpu = not args.no_cpu_baseline and not neon
    problems = build_projection_set(pkg, batch, keep_host=want_cpu)
    alg_bytes = sum(synth.q8_0_gemv_bytes(r["n_out"], r["n_in"], batch) for r in problems)
    flops = sum(2 * r["n_out"] * r["n_in"] * batch for r in problems)

    group_all = make_group(H, problems, batch, args.order)
    groups_layer = layer_groups(H, problems, batch, args.order)
    gemv_dev = H.lib.rmi_hip_gemv_q8_0_neon_dev if neon else H.lib.rmi_hip_gemv_q8_0_dev

    def step_grouped():
        H.check(H.lib.rmi_hip_gemv_group_run_dev(group_all, None))

    def step_per_matmul():
        for r in problems:
            H.check(gemv_dev(r["kernel"].w.handle, r["d_q8"].ptr, r["d_sc"].ptr, r["d_y"].ptr, batch, r["n_out"], 0,
                             r["n_out"], None))

    def step_layer():
        for g in groups_layer:
            H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))

    modes = {"grouped": (step_grouped, 1), "per_matmul": (step_per_matmul, len(problems)),
             "layer": (step_layer, len(groups_layer))}

    copy_calibration(H, args)

    fn, launches = modes[args.mode]
    wall, dev_ms = time_region(H, ev, fn, args.steps, args.warmup, args.settle_ms if batch > 1 else 0.0)
    settled = LAST_SETTLE_STEPS
    value = alg_bytes / wall / 1e9
    achieved = alg_bytes / (dev_ms * 1e-3) / 1e9  # bytes per launch / average launch duration, summed over the step
    result = base_result(args, "Q8_0 GEMV HBM GB/s, Qwen3-0.6B shapes, 1 GPU", "GB/s", round(value, 1), wall,
                         "int8 dot4 -> f32", {
        "workload": f"Qwen3-0.6B per-token projection set (7x28 + lm_head = 197 Q8_0 GEMVs, 633 MB of weights), "
                    f"decode batch {batch}, launch mode {args.mode}"
                    + (", NEON accumulation order on the matrix cores" if neon else ""),
        "batch": batch,
        "launches_per_step": launches,
        "algorithmic_bytes_per_step": alg_bytes,
        # the reference's own count (src/bin/micro_bench.rs:170-171, 203-204): weights + 5 bytes per input element
        "reference_convention_bytes_per_step": sum(r["n_out"] * (r["n_in"] // 32 * 34) + 5 * r["n_in"] * batch for r in problems),
        "flops_per_step": flops,
        "device": dev_name.strip(),
        "compute_units": cus,
    })
    result["warmup"] = args.warmup + settled  # untimed steps in all (batches of two and more wait for settled clocks)
    result.update({
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "gbs_by_reference_convention": round(result["config"]["reference_convention_bytes_per_step"] / wall / 1e9, 1),
        "token_steps_per_s": round(1.0 / wall, 1),
        "gflops": round(flops / wall / 1e9, 1),
        "roofline": {
            "bound": "hbm",
            "kernel": ("gemv_q8_0_mfma_kernel<%d,%s>" % ((batch + 15) // 16, "true" if args.mode != "per_matmul" else "false"))
                      if neon else
                      "%s<%d,%s,%s>" % (gemv_kernel_name(batch), batch, "true" if args.mode != "per_matmul" else "false",
                                        group_maxt(H, group_all) if args.mode == "grouped" else "*"),
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "avg_launch_us": round(dev_ms * 1e3 / launches, 3),
            "algorithmic_bytes_per_launch": round(alg_bytes / launches),
            **(read_traffic(f"gemv_q8_0_{args.mode}_qwen3_0.6b") if batch == 1 and not neon else
               read_traffic(f"gemv_q8_0_mfma_grouped_qwen3_0.6b_batch{batch}") if neon and args.mode == "grouped" else
               {"traffic": None}),
        },
    })

    if args.extra:
        extra = {}
        for mode, (fn2, l2) in modes.items():
            if mode == args.mode:
                continue
            w2, d2 = time_region(H, ev, fn2, max(5, args.steps // 5), 3)
            extra[mode] = {"GB/s": round(alg_bytes / w2 / 1e9, 1), "ms_per_step": round(w2 * 1e3, 4),
                           "device_ms_per_step": round(d2, 4), "launches_per_step": l2,
                           "token_steps_per_s": round(1.0 / w2, 1)}
        result["other_launch_modes"] = extra

    if want_cpu:
        got = cpu_baseline(problems, batch, alg_bytes)
        if got:
            result["cpu_baseline"], cpu_outs = got
            # the timed GPU step and the CPU baseline computed the same numbers
            step_grouped()
            H.check(H.lib.rmi_hip_synchronize())
            worst = 0
            for r, ref in zip(problems, cpu_outs):
                gpu = r["d_y"].to_array(np.float32, (batch, r["n_out"]))
                worst = max(worst, int(np.count_nonzero(gpu.view(np.uint32) != ref.view(np.uint32))))
            result["cpu_baseline"]["gpu_outputs_differing_from_cpu"] = worst
        else:
            result["cpu_baseline"] = None
    return result


def run_small_batches(args, pkg, ev):
    """The projection set at decode batch 2, 4, 8 and 16 in one grouped launch each: the GEMV in the x86-64 kernel's
    order at 2, 4 and 8 tokens (what Kernel::forward_batched runs by default), the small-batch kernel on the matrix
    cores (aarch64 kernel's order) at 8 and 16.  After each timed region every output of the launch is compared
    with the CPU checker's result in the same order, bit for bit."""
    H, synth = pkg.hip, pkg.synth
    check = not args.no_cpu_baseline
    problems = build_projection_set(pkg, 16, keep_host=check)  # smaller batches use the first tokens
    oracle = None
    if check:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        from concurrent.futures import ThreadPoolExecutor
        cores, _ = cpu_threads()
    out = {}
    for label, order, batch in (("batch2_x86_order", "avx2", 2), ("batch4_x86_order", "avx2", 4),
                                ("batch8_x86_order", "avx2", 8), ("batch8_aarch64_order", "neon", 8),
                                ("batch16_aarch64_order", "neon", 16)):
        group = make_group(H, problems, batch, order)

        def step(g=group):
            H.check(H.lib.rmi_hip_gemv_group_run_dev(g, None))

        # a step is 0.13 ms: 200 of them after 50 untimed ones and as many more as the clocks take to settle (the
        # launches of four tokens and more are bound by the vector ALU), so that the figure is the steady state
        steps, warmup = 200, 50
        wall, dev_ms = time_region(H, ev, step, steps, warmup, SETTLE_MS)
        warmup += LAST_SETTLE_STEPS
        alg = sum(synth.q8_0_gemv_bytes(r["n_out"], r["n_in"], batch) for r in problems)
        achieved = alg / (dev_ms * 1e-3) / 1e9
        out[label] = {
            "workload": f"Qwen3-0.6B projection set (197 Q8_0 GEMVs), decode batch {batch}, one grouped launch, "
                        + ("x86-64 accumulation order (GEMV)" if order == "avx2" else
                           "aarch64 accumulation order (small-batch kernel on the matrix cores)"),
            "value": round(alg / wall / 1e9, 1), "unit": "GB/s", "ms_per_step": round(wall * 1e3, 4),
            "steps": steps, "warmup": warmup, "token_steps_per_s": round(batch / wall, 1), "algorithmic_bytes_per_step": alg,
            "roofline": {"bound": "hbm",
                         "kernel": "%s<%d,true,%s>" % (gemv_kernel_name(batch), batch, group_maxt(H, group)) if order == "avx2"
                                   else "gemv_q8_0_mfma_kernel<%d,true>" % ((batch + 15) // 16),
                         "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "avg_launch_us": round(dev_ms * 1e3, 3)}}
        if oracle is not None and (order == "neon" or oracle.have_avx2()):
            variant = oracle.NEON if order == "neon" else oracle.AVX2

            H.check(H.lib.rmi_hip_synchronize())
            gpu_outs = [r["d_y"].to_array(np.float32, (batch, r["n_out"])) for r in problems]

            def differing(pair, batch=batch, variant=variant):
                r, gpu = pair
                worst = 0
                for t in range(batch):
                    ref = oracle.matmul_q8_0_quantized(r["w"], r["q8"][t], r["sc"][t], r["n_in"], r["n_out"], variant)
                    worst = max(worst, int(np.count_nonzero(gpu[t].view(np.uint32) != ref.view(np.uint32))))
                return worst

            with ThreadPoolExecutor(cores) as ex:  # the checker's C loops release the interpreter lock
                out[label]["gpu_outputs_differing_from_cpu"] = max(ex.map(differing, zip(problems, gpu_outs)))
        H.lib.rmi_hip_gemv_group_destroy(group)
    return out


def run_single_gemv(args, pkg, ev):
    """One Q8_0 GEMV per launch, W[3072 x 1024], decode batch 1: the reference's own micro-benchmark case
    (src/bin/micro_bench.rs:154-175).  A 3.3 MB weight would stay in the 256 MB last-level cache if launched again
    and again, so the launches walk a pool of 160 separate copies in HBM (535 MB) in turn and every launch streams
    its weight from HBM; one step = one launch, its time = the span between two HIP events on the launch stream
    divided by the launches between them."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    dev_name, cus, hbm = H.device_info()
    n_out, n_in, copies = 3072, 1024, 160
    w = synth.q8_0_weight(synth.seed_for(0, 0), n_out, n_in)
    x = synth.activations(synth.seed_for(0, 0x8000), 1, n_in)
    kernels = [K.Q8Kernel(w, n_in, n_out) for _ in range(copies)]
    d_x = H.DeviceBuffer.from_array(x)
    d_q8, d_sc, d_y = H.DeviceBuffer(n_in), H.DeviceBuffer(n_in // 32 * 4), H.DeviceBuffer(n_out * 4)
    H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q8.ptr, d_sc.ptr, 1, n_in, H.ROUND_TIES_EVEN, None))
    H.check(H.lib.rmi_hip_synchronize())
    state = {"i": 0}

    def step():
        k = kernels[state["i"] % copies]
        state["i"] += 1
        H.check(H.lib.rmi_hip_gemv_q8_0_dev(k.w.handle, d_q8.ptr, d_sc.ptr, d_y.ptr, 1, n_out, 0, n_out, None))

    steps, warmup = max(args.steps, 4 * copies), copies
    wall, dev_ms = time_region(H, ev, step, steps, warmup)
    alg = synth.q8_0_gemv_bytes(n_out, n_in, 1)
    ref_bytes = n_out * (n_in // 32 * 34) + 5 * n_in  # the reference's own count, micro_bench.rs:170-171, 203-204
    achieved = alg / (dev_ms * 1e-3) / 1e9
    timed = argparse.Namespace(steps=steps, warmup=warmup)
    result = base_result(timed, "Q8_0 GEMV HBM GB/s, single 3072x1024 matrix per launch, 1 GPU", "GB/s",
                         round(alg / wall / 1e9, 1), wall, "int8 dot4 -> f32", {
        "workload": f"single Q8_0 GEMV W[{n_out}x{n_in}], decode batch 1, one launch per step over a pool of {copies} "
                    f"separate weight copies in HBM ({copies * synth.q8_0_weight_bytes(n_out, n_in) / 1e6:.0f} MB) taken in turn",
        "launches_per_step": 1, "algorithmic_bytes_per_step": alg, "reference_convention_bytes_per_step": ref_bytes,
        "device": dev_name.strip(), "compute_units": cus})
    result["gbs_by_reference_convention"] = round(ref_bytes / wall / 1e9, 1)
    result["gflops"] = round(2.0 * n_in * n_out / wall / 1e9, 1)
    result["roofline"] = {"bound": "hbm", "kernel": "gemv_q8_0_deep_kernel<4>", "achieved": round(achieved, 1),
                          "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                          "avg_launch_us": round(dev_ms * 1e3, 3), "algorithmic_bytes_per_launch": alg, "traffic": None,
                          "limit": "0.42 us of HBM time per launch against the 2.4 us a launch costs in a stream of "
                                   "back-to-back launches: launch-bound; the grouped launch of the headline is the remedy"}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            q8, sc = d_q8.to_array(np.uint8, (1, n_in)), d_sc.to_array(np.float32, (1, n_in // 32))
            out = np.zeros((1, n_out), np.float32)
            for _ in range(10):
                pool.matmul_q8_0(w, q8, sc, out, n_in, n_out, 1)
            samples = []
            for _ in range(15):
                t0 = time.perf_counter()
                for _ in range(20):
                    pool.matmul_q8_0(w, q8, sc, out, n_in, n_out, 1)
                samples.append((time.perf_counter() - t0) / 20)
            pool.close()
            med = statistics.median(samples)
            step()
            H.check(H.lib.rmi_hip_synchronize())
            gpu = d_y.to_array(np.float32, (1, n_out))
            result["cpu_baseline"] = {
                "value": round(alg / med / 1e9, 2), "unit": "GB/s", "cores": cores, **core_info, "kind": "port",
                "sample": "10 warm-ups, 15 samples of 20 calls, median (micro_bench.rs:32-33, 94-152); the one weight "
                          "stays in the CPU's caches between calls, as in the reference's own run",
                "us_per_call": round(med * 1e6, 2), "gbs_by_reference_convention": round(ref_bytes / med / 1e9, 2),
                "gpu_outputs_differing_from_cpu": int(np.count_nonzero(gpu.view(np.uint32) != out.view(np.uint32)))}
    for k in kernels:
        k.w.free()
    return result


def compact(r):
    """A sub-record of the default line: the figure, its workload, its roofline and its CPU leg."""
    keep = {"workload": r["config"]["workload"], "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
            "steps": r["steps"], "warmup": r["warmup"], "roofline": r["roofline"]}
    if r.get("other_mode"):
        keep["other_mode"] = r["other_mode"]
    if r.get("ffn_stacked_gate_up"):
        keep["ffn_stacked_gate_up"] = r["ffn_stacked_gate_up"]
    if r.get("cpu_baseline"):
        keep["cpu_baseline"] = r["cpu_baseline"]
    return keep


def run_gemm(args, pkg, ev):
    """Prefill GEMM: X[M x 1024] . W[3072 x 1024]^T and X[M x 3072] . W[1024 x 3072]^T, Q8_0 both sides.
    One step = both products on activations already quantized in HBM."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    dev_name, cus, hbm = H.device_info()
    M = args.tokens
    recs = []
    for i, (n_out, n_in) in enumerate([(3072, 1024), (1024, 3072)]):
        w = synth.q8_0_weight(synth.seed_for(2, i), n_out, n_in)
        x = synth.activations(synth.seed_for(2, 0x8000 + i), M, n_in)
        k = K.Q8Kernel(w, n_in, n_out)
        d_x = H.DeviceBuffer.from_array(x)
        d_q8, d_sc, d_y = H.DeviceBuffer(M * n_in), H.DeviceBuffer(M * n_in // 32 * 4), H.DeviceBuffer(M * n_out * 4)
        H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q8.ptr, d_sc.ptr, M, n_in, H.ROUND_TIES_EVEN, None))
        H.check(H.lib.rmi_hip_synchronize())
        recs.append(dict(w=w, x=x, k=k, d_q8=d_q8, d_sc=d_sc, d_y=d_y, n_out=n_out, n_in=n_in))

    # "fast": the library picks, per product, the k-split kernel (few tokens, long rows) or the tiled kernel; every
    # output within the reference's tolerance.  "exact": always the tiled kernel, the aarch64 kernel's single chain.
    fast = args.gemm_mode == "fast"
    entry = H.lib.rmi_hip_gemm_q8_0_fast_dev if fast else H.lib.rmi_hip_gemm_q8_0_dev
    other = H.lib.rmi_hip_gemm_q8_0_dev if fast else H.lib.rmi_hip_gemm_q8_0_fast_dev

    def step(fn=entry):
        for r in recs:
            H.check(fn(r["k"].w.handle, r["d_q8"].ptr, r["d_sc"].ptr, r["d_y"].ptr, M, r["n_out"], None))

    copy_calibration(H, args)
    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup, args.settle_ms)
    settled = LAST_SETTLE_STEPS
    ops = sum(2.0 * M * r["n_in"] * r["n_out"] for r in recs)
    value = ops / wall / 1e12
    achieved = ops / (dev_ms * 1e-3) / 1e12
    result = base_result(args, "Q8_0 prefill GEMM TOP/s (int8 MFMA), Qwen3-0.6B FFN shapes, 1 GPU", "TOP/s",
                         round(value, 1), wall, "int8 MFMA -> f32", {
        "workload": f"Q8_0 GEMM M={M} tokens: X[Mx1024].W[3072x1024]^T and X[Mx3072].W[1024x3072]^T, "
                    f"per-block f32 rescale, 2 launches per step, "
                    + ("kernel chosen per product (k-split or tiled), outputs within 1e-4 + 1e-4|ref|" if fast else
                       "tiled kernel, aarch64 accumulation order bit for bit"),
        "tokens": M, "launches_per_step": 2, "ops_per_step": ops, "device": dev_name.strip(), "compute_units": cus})
    result["roofline"] = {"bound": "mfma", "kernel": "gemm_q8_0_ksplit_kernel / gemm_q8_0_kernel" if fast else "gemm_q8_0_kernel",
                          "achieved": round(achieved, 1), "peak": INT8_MFMA_PEAK_TOPS,
                          "unit": "TOP/s", "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4),
                          "avg_launch_us": round(dev_ms * 1e3 / 2, 3),
                          **(read_traffic("gemm_q8_0_m2048_qwen3_0.6b_ffn") if M == 2048 else
                             read_traffic("gemm_q8_0_m64_m512_qwen3_0.6b_ffn", f"m{M}"))}
    result["warmup"] = args.warmup + settled  # untimed steps in all: the W asked for and those the clocks took to settle
    w2, d2 = time_region(H, ev, lambda: step(other), args.steps, args.warmup, args.settle_ms)
    result["other_mode"] = {"mode": "exact (tiled kernel, single chain)" if fast else "fast (kernel chosen per product)",
                            "value": round(ops / w2 / 1e12, 1), "unit": "TOP/s", "avg_launch_us": round(d2 * 1e3 / 2, 3)}
    # The FFN as a host runs it after fuse_vstack (src/ops/quant/fuse.rs:25-64): gate and up are one stacked weight,
    # one product of twice the rows, then down: three products' operations in two launches.
    kg = K.Q8Kernel(synth.q8_0_weight(synth.seed_for(2, 7), 6144, 1024), 1024, 6144)
    d_yg = H.DeviceBuffer(M * 6144 * 4)

    def ffn(fn):
        H.check(fn(kg.w.handle, recs[0]["d_q8"].ptr, recs[0]["d_sc"].ptr, d_yg.ptr, M, 6144, None))
        H.check(fn(recs[1]["k"].w.handle, recs[1]["d_q8"].ptr, recs[1]["d_sc"].ptr, recs[1]["d_y"].ptr, M, 1024, None))

    ffn_ops = 2.0 * M * 1024 * 6144 + 2.0 * M * 3072 * 1024
    result["ffn_stacked_gate_up"] = {"workload": f"X[Mx1024].[W_gate ; W_up][6144x1024]^T, then X[Mx3072].W_down[1024x3072]^T, M={M}: "
                                                 "2 launches, the operations of 3 products", "ops_per_step": ffn_ops, "unit": "TOP/s"}
    for name, fn in (("fast", H.lib.rmi_hip_gemm_q8_0_fast_dev), ("exact", H.lib.rmi_hip_gemm_q8_0_dev)):
        wf, df = time_region(H, ev, lambda: ffn(fn), args.steps, args.warmup, args.settle_ms)
        result["ffn_stacked_gate_up"][name] = {"value": round(ffn_ops / wf / 1e12, 1), "us_per_step": round(df * 1e3, 3)}
    d_yg.free()
    kg.w.free()
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            mt = min(M, 256)  # bounded sample: the first `mt` tokens of both products
            outs, qs = [], []
            for r in recs:
                q8 = r["d_q8"].to_array(np.uint8, (M, r["n_in"]))[:mt].copy()
                sc = r["d_sc"].to_array(np.float32, (M, r["n_in"] // 32))[:mt].copy()
                qs.append((q8, sc))
                outs.append(np.zeros((mt, r["n_out"]), np.float32))
            samples = []
            for it in range(4):
                t0 = time.perf_counter()
                for r, (q8, sc), out in zip(recs, qs, outs):
                    pool.matmul_q8_0(r["w"], q8, sc, out, r["n_in"], r["n_out"], mt)
                samples.append(time.perf_counter() - t0)
            pool.close()
            med = statistics.median(samples[1:])
            step()
            H.check(H.lib.rmi_hip_synchronize())
            worst = 0.0
            for r, out in zip(recs, outs):
                gpu = r["d_y"].to_array(np.float32, (M, r["n_out"]))[:mt]
                worst = max(worst, float(np.max(np.abs(gpu - out) / (1e-4 + 1e-4 * np.abs(out)))))
            result["cpu_baseline"] = {
                "value": round(ops * mt / M / med / 1e12, 4), "unit": "TOP/s", "cores": cores, **core_info, "kind": "port",
                "sample": f"first {mt} of {M} tokens of both products, one GEMV per token (the reference has no GEMM), "
                          f"restated AVX2 kernels over {cores} threads, median of 3",
                "max_err_over_tolerance": round(worst, 4)}
    return result


def run_q4k(args, pkg, ev):
    return run_kquant(args, pkg, ev, "q4_k")


def run_q6k(args, pkg, ev):
    return run_kquant(args, pkg, ev, "q6_k")


def run_kquant(args, pkg, ev, fmt):
    """Q4_K / Q6_K x Q8_K decode GEMV at 1.7B-class FFN shapes (gate/up 6144x2048, down 2048x6144), 28 layers of
    distinct weights (594 / 867 MB) so that every step streams from HBM; one grouped launch, or one per matrix with
    --mode per_matmul."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    q6 = fmt == "q6_k"
    name = "Q6_K" if q6 else "Q4_K"
    make_weight = synth.q6_k_weight if q6 else synth.q4_k_weight
    kernel_cls = K.Q6_KKernel if q6 else K.Q4_KKernel
    group_create = H.lib.rmi_hip_gemv_group_create_q6_k if q6 else H.lib.rmi_hip_gemv_group_create_q4_k
    gemv_dev = H.lib.rmi_hip_gemv_q6_k_q8k_dev if q6 else H.lib.rmi_hip_gemv_q4_k_q8k_dev
    gemv_bytes = synth.q6_k_gemv_bytes if q6 else synth.q4_k_gemv_bytes
    dev_name, cus, hbm = H.device_info()
    batch = args.batch
    recs = []
    shapes = [(6144, 2048), (6144, 2048), (2048, 6144)] * 28
    for i, (n_out, n_in) in enumerate(shapes):
        w = make_weight(synth.seed_for(3, i), n_out, n_in)
        x = synth.activations(synth.seed_for(3, 0x8000 + i), batch, n_in)
        k = kernel_cls(w, n_in, n_out)
        d_x = H.DeviceBuffer.from_array(x)
        d_d, d_q, d_b = H.DeviceBuffer(batch * n_in // 256 * 4), H.DeviceBuffer(batch * n_in), H.DeviceBuffer(batch * n_in // 16 * 2)
        d_y = H.DeviceBuffer(batch * n_out * 4)
        H.check(H.lib.rmi_hip_quantize_row_q8_k_dev(d_x.ptr, d_d.ptr, d_q.ptr, d_b.ptr, batch, n_in, None))
        H.check(H.lib.rmi_hip_synchronize())
        d_x.free()
        recs.append(dict(w=w if not args.no_cpu_baseline else None, k=k, d_d=d_d, d_q=d_q, d_b=d_b, d_y=d_y, n_out=n_out,
                         n_in=n_in))

    n = len(recs)
    arr = lambda vals: (C.c_void_p * n)(*vals)  # noqa: E731
    group = group_create(n, arr([r["k"].w.handle for r in recs]), arr([r["d_d"].ptr for r in recs]),
                         arr([r["d_q"].ptr for r in recs]), arr([r["d_b"].ptr for r in recs]),
                         arr([r["d_y"].ptr for r in recs]), batch)
    if not group:
        raise RuntimeError(H.last_error())

    def step_per_matmul():
        for r in recs:
            H.check(gemv_dev(r["k"].w.handle, r["d_d"].ptr, r["d_q"].ptr, r["d_b"].ptr, r["d_y"].ptr, batch, r["n_out"], 0,
                             r["n_out"], None))

    def step_grouped():
        H.check(H.lib.rmi_hip_gemv_group_run_dev(group, None))

    grouped = args.mode != "per_matmul"
    step = step_grouped if grouped else step_per_matmul
    launches = 1 if grouped else n
    copy_calibration(H, args)
    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup)
    alg = sum(gemv_bytes(r["n_out"], r["n_in"], batch) for r in recs)
    value = alg / wall / 1e9
    achieved = alg / (dev_ms * 1e-3) / 1e9
    result = base_result(args, f"{name} x Q8_K GEMV HBM GB/s, 1.7B-class FFN shapes, 1 GPU", "GB/s", round(value, 1), wall,
                         "int8 dot4 -> f32", {
        "workload": f"{name} GEMV, 28 layers x (gate 6144x2048, up 6144x2048, down 2048x6144), decode batch {batch}, "
                    + ("one grouped launch" if grouped else "one launch per matrix"), "batch": batch,
        "launches_per_step": launches,
        "algorithmic_bytes_per_step": alg, "device": dev_name.strip(), "compute_units": cus})
    result["roofline"] = {"bound": "hbm", "kernel": f"gemv_{fmt}_kernel<{batch},{'true' if grouped else 'false'},{group_maxt(H, group) if grouped else '*'}>",
                          "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(achieved / HBM_PEAK_GBS, 4),
                          "avg_launch_us": round(dev_ms * 1e3 / launches, 3),
                          **(read_traffic(f"gemv_{fmt}_grouped_1.7b_ffn") if grouped and batch == 1 else {"traffic": None})}
    if not args.no_cpu_baseline and batch == 1:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            host = [(r["d_d"].to_array(np.float32, (r["n_in"] // 256,)), r["d_q"].to_array(np.int8, (r["n_in"],)),
                     r["d_b"].to_array(np.int16, (r["n_in"] // 16,)), np.zeros(r["n_out"], np.float32)) for r in recs]
            samples = []
            for it in range(6):
                t0 = time.perf_counter()
                for r, (d, q, b, out) in zip(recs, host):
                    (pool.matmul_q6k_q8k if q6 else pool.matmul_q4k_q8k)(r["w"], d, q, b, out, r["n_in"], r["n_out"])
                samples.append(time.perf_counter() - t0)
            pool.close()
            med = statistics.median(samples[1:])
            step()
            H.check(H.lib.rmi_hip_synchronize())
            worst = max(int(np.count_nonzero(r["d_y"].to_array(np.float32, (r["n_out"],)).view(np.uint32)
                                             != out.view(np.uint32))) for r, (_, _, _, out) in zip(recs, host))
            result["cpu_baseline"] = {"value": round(alg / med / 1e9, 2), "unit": "GB/s", "cores": cores, **core_info, "kind": "port",
                                      "sample": f"5 full steps (84 GEMVs, {alg / 1e6:.0f} MB), restated AVX2 "
                                                f"vec_dot_{fmt.replace('_', '')}_q8k over {cores} threads, median",
                                      "gpu_outputs_differing_from_cpu": worst}
    return result


def run_q4_0(args, pkg, ev):
    """Q4_0 x Q8_0 decode GEMV at the 1.7B-class FFN shapes of the Q4_K / Q6_K workloads (gate/up 6144x2048, down
    2048x6144), 28 layers of distinct weights (595 MB) so that every step streams from HBM; one grouped launch, or
    one per matrix with --mode per_matmul."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    dev_name, cus, hbm = H.device_info()
    batch = args.batch
    recs = []
    shapes = [(6144, 2048), (6144, 2048), (2048, 6144)] * 28
    for i, (n_out, n_in) in enumerate(shapes):
        w = synth.q4_0_weight(synth.seed_for(5, i), n_out, n_in)
        x = synth.activations(synth.seed_for(5, 0x8000 + i), batch, n_in)
        k = K.Q4_0Kernel(w, n_in, n_out)
        d_x = H.DeviceBuffer.from_array(x)
        d_q, d_s, d_y = H.DeviceBuffer(batch * n_in), H.DeviceBuffer(batch * n_in // 32 * 4), H.DeviceBuffer(batch * n_out * 4)
        H.check(H.lib.rmi_hip_quantize_q8_0_dev(d_x.ptr, d_q.ptr, d_s.ptr, batch, n_in, H.ROUND_TIES_EVEN, None))
        H.check(H.lib.rmi_hip_synchronize())
        d_x.free()
        recs.append(dict(w=w if not args.no_cpu_baseline else None, k=k, d_q=d_q, d_s=d_s, d_y=d_y, n_out=n_out, n_in=n_in))

    n = len(recs)
    arr = lambda vals: (C.c_void_p * n)(*vals)  # noqa: E731
    group = H.lib.rmi_hip_gemv_group_create(n, arr([r["k"].w.handle for r in recs]), arr([r["d_q"].ptr for r in recs]),
                                            arr([r["d_s"].ptr for r in recs]), arr([r["d_y"].ptr for r in recs]), batch)
    if not group:
        raise RuntimeError(H.last_error())

    def step_per_matmul():
        for r in recs:
            H.check(H.lib.rmi_hip_gemv_q4_0_dev(r["k"].w.handle, r["d_q"].ptr, r["d_s"].ptr, r["d_y"].ptr, batch, r["n_out"],
                                                0, r["n_out"], None))

    def step_grouped():
        H.check(H.lib.rmi_hip_gemv_group_run_dev(group, None))

    grouped = args.mode != "per_matmul"
    step = step_grouped if grouped else step_per_matmul
    launches = 1 if grouped else n
    copy_calibration(H, args)
    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup)
    alg = sum(synth.q4_0_gemv_bytes(r["n_out"], r["n_in"], batch) for r in recs)
    achieved = alg / (dev_ms * 1e-3) / 1e9
    result = base_result(args, "Q4_0 x Q8_0 GEMV HBM GB/s, 1.7B-class FFN shapes, 1 GPU", "GB/s", round(alg / wall / 1e9, 1),
                         wall, "int8 dot4 -> f32", {
        "workload": f"Q4_0 GEMV, 28 layers x (gate 6144x2048, up 6144x2048, down 2048x6144), decode batch {batch}, "
                    + ("one grouped launch" if grouped else "one launch per matrix"), "batch": batch,
        "launches_per_step": launches, "algorithmic_bytes_per_step": alg, "device": dev_name.strip(),
        "compute_units": cus})
    result["roofline"] = {"bound": "hbm", "kernel": f"gemv_q4_0_kernel<{batch},{'true' if grouped else 'false'},{group_maxt(H, group) if grouped else '*'}>",
                          "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(achieved / HBM_PEAK_GBS, 4), "avg_launch_us": round(dev_ms * 1e3 / launches, 3),
                          **(read_traffic("gemv_q4_0_grouped_1.7b_ffn") if grouped and batch == 1 else {"traffic": None})}
    if not args.no_cpu_baseline and batch == 1:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            host = [(r["d_q"].to_array(np.uint8, (r["n_in"],)), r["d_s"].to_array(np.float32, (r["n_in"] // 32,)),
                     np.zeros(r["n_out"], np.float32)) for r in recs]
            samples = []
            for it in range(6):
                t0 = time.perf_counter()
                for r, (q, sc, out) in zip(recs, host):
                    pool.matmul_q4_0(r["w"], q, sc, out, r["n_in"], r["n_out"])
                samples.append(time.perf_counter() - t0)
            pool.close()
            med = statistics.median(samples[1:])
            step()
            H.check(H.lib.rmi_hip_synchronize())
            worst = max(int(np.count_nonzero(r["d_y"].to_array(np.float32, (r["n_out"],)).view(np.uint32)
                                             != out.view(np.uint32))) for r, (_, _, out) in zip(recs, host))
            result["cpu_baseline"] = {"value": round(alg / med / 1e9, 2), "unit": "GB/s", "cores": cores, **core_info, "kind": "port",
                                      "sample": f"5 full steps (84 GEMVs, {alg / 1e6:.0f} MB), restated AVX2 "
                                                f"matmul_q4_0_vs_q8_0 over {cores} threads, median",
                                      "gpu_outputs_differing_from_cpu": worst}
    return result


def run_qlinear(args, pkg, ev):
    """QuantizedLinear::forward (src/core/model.rs:65-91): f32 activation, Q4_K weight dequantised on the fly, one
    strictly sequential f32 sum per output row.  One step = the three FFN products of a 1.7B-class layer (gate, up
    6144x2048, down 2048x6144).  The bound is neither HBM nor the matrix cores but the add chain: n_in dependent f32
    adds per row, about 8.4 clocks each on one lane; rows run side by side."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    dev_name, cus, hbm = H.device_info()
    recs = []
    for i, (n_out, n_in) in enumerate([(6144, 2048), (6144, 2048), (2048, 6144)]):
        w = synth.q4_k_weight(synth.seed_for(3, i), n_out, n_in)
        x = synth.activations(synth.seed_for(3, 0x8000 + i), 1, n_in).reshape(-1)
        k = K.Q4_KKernel(w, n_in, n_out)
        recs.append(dict(w=w, x=x, k=k, d_x=H.DeviceBuffer.from_array(x), d_y=H.DeviceBuffer(n_out * 4), n_out=n_out,
                         n_in=n_in))

    def step():
        for r in recs:
            H.check(H.lib.rmi_hip_quantized_linear_forward_dev(r["k"].w.handle, r["d_x"].ptr, r["d_y"].ptr, None))

    copy_calibration(H, args)
    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup)
    alg = sum(r["n_out"] * (r["n_in"] // 256) * 144 + 4 * r["n_in"] + 4 * r["n_out"] for r in recs)
    achieved = alg / (dev_ms * 1e-3) / 1e9
    chain_us = sum(r["n_in"] * 8.4 / 2.0e3 for r in recs)  # at 2.0 GHz under load
    result = base_result(args, "QuantizedLinear::forward (Q4_K dequantise-and-dot) GB/s, 1.7B-class FFN shapes, 1 GPU", "GB/s",
                         round(alg / wall / 1e9, 1), wall, "f32 (sequential sum per row)", {
        "workload": "QuantizedLinear::forward, gate and up (6144x2048) and down (2048x6144), f32 activation, 3 launches per step",
        "launches_per_step": 3, "algorithmic_bytes_per_step": alg, "device": dev_name.strip(), "compute_units": cus})
    result["roofline"] = {"bound": "hbm", "kernel": "q4_k_dequant_dot_split_kernel", "achieved": round(achieved, 1),
                          "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                          "avg_launch_us": round(dev_ms * 1e3 / 3, 3), "traffic": None,
                          "limit": "one dependent f32 add per element and row (the reference's summation order): "
                                   f"{chain_us:.1f} us per step at 8.4 clocks an add and 2.0 GHz, whatever the bandwidth",
                          "add_chain_us_per_step": round(chain_us, 1)}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        samples, worst = [], 0
        step()
        H.check(H.lib.rmi_hip_synchronize())
        for it in range(2):
            t0 = time.perf_counter()
            refs = [oracle.quantized_linear_forward(r["w"], r["x"], r["n_in"], r["n_out"]) for r in recs]
            samples.append(time.perf_counter() - t0)
        for r, ref in zip(recs, refs):
            worst = max(worst, int(np.count_nonzero(r["d_y"].to_array(np.float32, (r["n_out"],)).view(np.uint32)
                                                    != ref.view(np.uint32))))
        result["cpu_baseline"] = {"value": round(alg / min(samples) / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": "2 full steps of the restated forward_dequant (dequantise the weight, then "
                                            "the sequential dot per row), one thread as the reference runs it, best",
                                  "gpu_outputs_differing_from_cpu": worst}
    return result


def run_q4k_gemm(args, pkg, ev):
    """Q4_K prefill: X[M x 2048] through gate and up (6144 x 2048 each) and X[M x 6144] through down (2048 x 6144),
    Q8_K activations already quantized in HBM; one step = the three products."""
    H, synth, K = pkg.hip, pkg.synth, pkg.kernel
    dev_name, cus, hbm = H.device_info()
    M = args.tokens
    recs = []
    for i, (n_out, n_in) in enumerate([(6144, 2048), (6144, 2048), (2048, 6144)]):
        w = synth.q4_k_weight(synth.seed_for(3, i), n_out, n_in)
        x = synth.activations(synth.seed_for(3, 0x8000 + i), M, n_in)
        k = K.Q4_KKernel(w, n_in, n_out)
        d_x = H.DeviceBuffer.from_array(x)
        d_d, d_q, d_b = H.DeviceBuffer(M * n_in // 256 * 4), H.DeviceBuffer(M * n_in), H.DeviceBuffer(M * n_in // 16 * 2)
        d_y = H.DeviceBuffer(M * n_out * 4)
        H.check(H.lib.rmi_hip_quantize_row_q8_k_dev(d_x.ptr, d_d.ptr, d_q.ptr, d_b.ptr, M, n_in, None))
        H.check(H.lib.rmi_hip_synchronize())
        d_x.free()
        recs.append(dict(w=w, k=k, d_d=d_d, d_q=d_q, d_b=d_b, d_y=d_y, n_out=n_out, n_in=n_in))

    def step():
        for r in recs:
            H.check(H.lib.rmi_hip_gemm_q4_k_q8k_dev(r["k"].w.handle, r["d_d"].ptr, r["d_q"].ptr, r["d_b"].ptr,
                                                    r["d_y"].ptr, M, r["n_out"], None))

    copy_calibration(H, args)
    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup, args.settle_ms)
    settled = LAST_SETTLE_STEPS
    ops = sum(2.0 * M * r["n_in"] * r["n_out"] for r in recs)
    achieved = ops / (dev_ms * 1e-3) / 1e12
    result = base_result(args, "Q4_K x Q8_K prefill GEMM TOP/s (int8 MFMA), 1.7B-class FFN shapes, 1 GPU", "TOP/s",
                         round(ops / wall / 1e12, 1), wall, "int8 MFMA -> f32", {
        "workload": f"Q4_K GEMM M={M} tokens: gate, up (6144x2048) and down (2048x6144), 3 launches per step",
        "tokens": M, "launches_per_step": 3, "ops_per_step": ops, "device": dev_name.strip(), "compute_units": cus})
    result["roofline"] = {"bound": "mfma", "kernel": "gemm_q4_k_kernel", "achieved": round(achieved, 1),
                          "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s", "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4),
                          "avg_launch_us": round(dev_ms * 1e3 / 3, 3), **read_traffic("gemm_q4_k_m512_m2048_1.7b_ffn", f"m{M}")}
    # The FFN as a host runs it after fuse_vstack (src/ops/quant/fuse.rs:25-64): gate and up are one stacked weight of
    # twice the rows, then down: the same operations in two launches.
    kg = K.Q4_KKernel(synth.q4_k_weight(synth.seed_for(3, 7), 12288, 2048), 2048, 12288)
    d_yg = H.DeviceBuffer(M * 12288 * 4)

    def ffn():
        r = recs[0]
        H.check(H.lib.rmi_hip_gemm_q4_k_q8k_dev(kg.w.handle, r["d_d"].ptr, r["d_q"].ptr, r["d_b"].ptr, d_yg.ptr, M, 12288, None))
        r = recs[2]
        H.check(H.lib.rmi_hip_gemm_q4_k_q8k_dev(r["k"].w.handle, r["d_d"].ptr, r["d_q"].ptr, r["d_b"].ptr, r["d_y"].ptr, M, 2048, None))

    result["warmup"] = args.warmup + settled  # untimed steps in all: the W asked for and those the clocks took to settle
    wf, df = time_region(H, ev, ffn, args.steps, args.warmup, args.settle_ms)
    result["ffn_stacked_gate_up"] = {"workload": f"X[Mx2048].[W_gate ; W_up][12288x2048]^T, then X[Mx6144].W_down[2048x6144]^T, M={M}: "
                                                 "2 launches, the same operations", "ops_per_step": ops,
                                     "value": round(ops / wf / 1e12, 1), "unit": "TOP/s", "us_per_step": round(df * 1e3, 3)}
    d_yg.free()
    kg.w.free()
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            mt = min(M, 64)  # bounded sample: the first `mt` tokens of the three products
            t_cpu, worst = 0.0, 0.0
            step()
            H.check(H.lib.rmi_hip_synchronize())
            for r in recs:
                got = r["d_y"].to_array(np.float32, (M, r["n_out"]))[:mt]
                dd = r["d_d"].to_array(np.float32, (M, r["n_in"] // 256))
                qq = r["d_q"].to_array(np.int8, (M, r["n_in"]))
                bb = r["d_b"].to_array(np.int16, (M, r["n_in"] // 16))
                out = np.zeros(r["n_out"], np.float32)
                for t in range(mt):
                    t0 = time.perf_counter()
                    pool.matmul_q4k_q8k(r["w"], dd[t], qq[t], bb[t], out, r["n_in"], r["n_out"])
                    t_cpu += time.perf_counter() - t0
                    worst = max(worst, float(np.max(np.abs(got[t] - out) / (1e-4 + 1e-4 * np.abs(out)))))
            pool.close()
            ops_cpu = sum(2.0 * mt * r["n_in"] * r["n_out"] for r in recs)
            result["cpu_baseline"] = {"value": round(ops_cpu / t_cpu / 1e12, 4), "unit": "TOP/s", "cores": cores,
                                      **core_info, "kind": "port",
                                      "sample": f"first {mt} of {M} tokens of the three products, one GEMV per token (the "
                                                f"reference has no GEMM), restated AVX2 vec_dot_q4k_q8k over {cores} threads",
                                      "max_err_over_tolerance": round(worst, 4)}
    return result


def run_attention(args, pkg, ev):
    """One attention launch of a Qwen3-0.6B layer over the F16 cache (16 query heads, 8 key/value heads, head
    dimension 128; src/models/qwen3.rs:876-933), output quantized to Q8_0, at --keys cached positions.  One step =
    one call of rmi_hip_attention_f16_quantize_q8_0_dev.  Neither HBM nor the matrix cores bound it: the reference's
    f64 sums and its sequential f32 sum of the softmax weights do (about 8.4 clocks per key on one lane)."""
    H = pkg.hip
    dev_name, cus, hbm = H.device_info()
    n_head, n_kv, hd, n_keys = 16, 8, 128, args.keys
    kv_stride = n_kv * hd
    rng = np.random.default_rng(1234)
    q = rng.normal(0, 1, n_head * hd).astype(np.float16).view(np.uint16)
    kc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
    vc = rng.normal(0, 1, (n_keys, kv_stride)).astype(np.float16).view(np.uint16)
    d_q, d_k, d_v = (H.DeviceBuffer.from_array(a) for a in (q, kc, vc))
    d_o, d_s = H.DeviceBuffer(n_head * hd), H.DeviceBuffer(n_head * hd // 32 * 4)

    def step():
        H.check(H.lib.rmi_hip_attention_f16_quantize_q8_0_dev(d_q.ptr, d_k.ptr, d_v.ptr, n_keys, kv_stride, n_head, n_kv,
                                                              hd, hd, d_o.ptr, d_s.ptr, 0, None))

    wall, dev_ms = time_region(H, ev, step, args.steps, args.warmup)
    alg = 2 * n_keys * kv_stride * 2 + n_head * hd * 2 + n_head * hd + n_head * hd // 32 * 4
    achieved = alg / (dev_ms * 1e-3) / 1e9
    result = base_result(args, "F16-KV attention launch, Qwen3-0.6B layer shape, keys per second, 1 GPU", "keys/s",
                         round(n_keys / wall), wall, "f16 x f16 -> f64 sums, f32 softmax", {
        "workload": f"attention over {n_keys} cached positions, 16 heads / 8 kv heads x 128, one launch per step",
        "keys": n_keys, "algorithmic_bytes_per_step": alg, "device": dev_name.strip(), "compute_units": cus})
    result["us_per_launch"] = round(dev_ms * 1e3, 3)
    result["ns_per_key"] = round(dev_ms * 1e6 / n_keys, 2)
    result["roofline"] = {"bound": "hbm", "kernel": "attention128_quant_kernel / attn128_scores_kernel + attn128_weights_pv_kernel",
                          "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(achieved / HBM_PEAK_GBS, 4), "avg_launch_us": round(dev_ms * 1e3, 3), "traffic": None,
                          "limit": "the reference's sequential f32 sum of the softmax weights: "
                                   f"{n_keys * 8.4 / 2.0e3:.1f} us at 8.4 clocks a key and 2.0 GHz, whatever the bandwidth"}
    return result


def run_decode(args, pkg, ev):
    """End-to-end greedy decode, device-resident: a random-init Qwen3-0.6B-architecture model written as a
    synthetic Q8_0 GGUF, 512 prompt tokens (fed one per step, as the reference's generate_inner does) plus 128
    generated ones = 639 token-steps per generation.  One bench step = one generation."""
    import tempfile
    H = pkg.hip
    dev_name, cus, hbm = H.device_info()
    n_prompt, n_new = 512, 128
    tmp = tempfile.mkdtemp(prefix="rmi_bench_")
    path = os.path.join(tmp, "synthetic-qwen3-0.6b-q8_0.gguf")
    pkg.gguf.write_synthetic_qwen3(path, seed=4)
    f = pkg.gguf.GGUFFile(path)
    tensors = {name: t[2] for name, t in f.tensors.items()}
    sess = pkg.decode.Qwen3Session(f.metadata, tensors, capacity=n_prompt + n_new)
    prompt = np.random.default_rng(7).integers(0, 151936, n_prompt, dtype=np.uint32)
    token_steps = n_prompt + n_new - 1
    last = {}

    def step():
        last.update(sess.generate(prompt, n_new))

    for _ in range(args.warmup):
        step()
    H.check(H.lib.rmi_hip_synchronize())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()  # each generation ends with its own synchronisation
    H.check(H.lib.rmi_hip_synchronize())
    wall = (time.perf_counter() - t0) / args.steps
    per_token = wall / token_steps
    synth = pkg.synth
    alg = sum(synth.q8_0_gemv_bytes(n_out, n_in) for _, n_out, n_in in synth.QWEN3_0_6B_LAYER) * 28 + \
        synth.q8_0_gemv_bytes(151936, 1024)
    result = base_result(args, "decode token-steps/s, Qwen3-0.6B Q8_0, 512 prompt + 128 greedy tokens, 1 GPU", "tok/s",
                         round(token_steps / wall, 1), wall, "int8 dot4 -> f32 (F16 KV cache)", {
        "workload": "device-resident greedy decode of a synthetic Q8_0 GGUF (Qwen3-0.6B architecture, 28 layers, "
                    "vocab 151936), 512 prompt positions (128 to a pass) + 127 generated tokens = 639 token-steps per "
                    "generation, logits computed at every position; one bench step = one generation",
        "token_steps_per_generation": token_steps, "launches_per_token_step": 1 + 5 * 28 + 4,
        "device": dev_name.strip(), "compute_units": cus})
    result["ms_per_token_step"] = round(per_token * 1e3, 4)
    # the two phases apart: the prompt (positions known in advance: the session takes them 128 to a pass, each
    # position's logits still computed and bit-identical to its own step) and the generated tokens (one step each)
    if args.no_phases:
        t_prompt = None
    else:
        t_prompt = min(sess.generate(prompt, 1)["seconds"] for _ in range(2))
    if t_prompt is not None:
        t_all = min(last["seconds"], sess.generate(prompt, n_new)["seconds"])
        result["phases"] = {"prompt_positions_per_s": round(n_prompt / t_prompt, 1), "prompt_ms_per_position": round(t_prompt / n_prompt * 1e3, 4),
                            "generated_tokens_per_s": round((n_new - 1) / (t_all - t_prompt), 1),
                            "generated_ms_per_token": round((t_all - t_prompt) / (n_new - 1) * 1e3, 4)}
        sess.set_prompt_passes(False)
        t_steps = sess.generate(prompt, n_new)["seconds"]
        sess.set_prompt_passes(True)
        result["phases"]["every_position_its_own_step_tok_s"] = round(token_steps / t_steps, 1)
    # HBM bytes against time for the generated tokens, each of which reads every weight once; the prompt passes
    # read a weight once for 128 positions, so the whole generation's time per token-step would flatter the figure
    if t_prompt is not None:
        per_generated = (t_all - t_prompt) / (n_new - 1)
        basis = "generated tokens (one step each, 512-638 cached positions)"
    else:
        per_generated = per_token
        basis = "whole generation, prompt passes included (they read a weight once for 128 positions: an upper bound)"
    achieved = alg / per_generated / 1e9
    result["roofline"] = {"bound": "hbm", "kernel": "Q8_0 GEMV kernels (4 per layer + lm_head = 113 launches per token-step)",
                          "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(achieved / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_token_step": alg,
                          "basis": basis, "ms_per_token_step": round(per_generated * 1e3, 4),
                          "traffic": None,
                          "note": "a generated token is 144 dependent launches of 3-13 us each, launch-latency-bound, not "
                                  "HBM-bound; the bytes are those of one weight read per token-step"}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import rmi_oracle as oracle
        if oracle.have_avx2():
            cores, core_info = cpu_threads()
            pool = oracle.Pool(cores)
            cpu = oracle.Qwen3Decoder(f.metadata, tensors, pool).generate(prompt, n_new)
            pool.close()
            result["cpu_baseline"] = {
                "value": round(token_steps / cpu["seconds"], 1), "unit": "tok/s", "cores": cores, **core_info, "kind": "port",
                "sample": f"one full generation ({token_steps} token-steps) of the restated Qwen3Session loop with the "
                          f"restated AVX2 matmuls over {cores} threads",
                "gpu_tokens_equal_cpu_tokens": bool(np.array_equal(cpu["tokens"], last["tokens"])),
                "gpu_argmax_equal_cpu_argmax_all_steps": bool(np.array_equal(cpu["argmax"], last["argmax"]))}
    sess.close()
    del f, tensors
    try:
        os.remove(path)
        os.rmdir(tmp)
    except OSError:
        pass
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 50; 500 for the q4_0 / q4k / q6k GEMV workloads, whose compute-heavy kernels "
                         "read 10-15 %% slower until the clocks have settled, a few hundred launches in)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps before (default 10; 100 for q4_0 / q4k / q6k).  Left at its default, the compute-bound "
                         "workloads (GEMM, Q4_K GEMM, batches of two and more) add untimed steps until the clocks have "
                         "settled and report the total as `warmup`; given, it is exactly the number asked for")
    ap.add_argument("--workload", choices=["projection_set", "single_gemv", "gemm", "q4_0", "q4k", "q6k", "q4k_gemm", "qlinear", "attention", "decode"], default="projection_set",
                    help="projection_set: the headline Q8_0 decode GEMV workload (default); gemm: Q8_0 prefill GEMM; "
                         "q4_0: Q4_0 x Q8_0 decode GEMV; q4k / q6k: Q4_K / Q6_K x Q8_K decode GEMV; q4k_gemm: Q4_K prefill GEMM (M = --tokens); qlinear: QuantizedLinear::forward (Q4_K dequantise-and-dot, f32 activation); decode: end-to-end device-resident greedy decode "
                         "(one step = one 639-token-step generation)")
    ap.add_argument("--batch", type=int, default=1, help="decode batch (1..8 tokens; 1..64 with --order neon)")
    ap.add_argument("--order", choices=["avx2", "neon"], default="avx2",
                    help="projection_set: accumulation order of the reference's x86-64 kernel (GEMV, the default) or of "
                         "its aarch64 kernel (small-batch kernel on the matrix cores)")
    ap.add_argument("--tokens", type=int, default=2048, help="prefill tokens M for --workload gemm")
    ap.add_argument("--gemm-mode", choices=["fast", "exact"], default="fast",
                    help="gemm: 'fast' lets the library split the blocks of a row over the waves of a workgroup where the "
                         "tile grid is smaller than the chip (outputs within the reference's tolerance); 'exact' keeps the "
                         "aarch64 kernel's single f32 chain per output, bit for bit")
    ap.add_argument("--keys", type=int, default=4096, help="cached positions for --workload attention")
    ap.add_argument("--mode", choices=["grouped", "per_matmul", "layer"], default="grouped")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration-mb", type=int, default=0,
                    help="also launch the plain copy kernel on this many MiB, 5 times, outside the timed region "
                         "(the known-size kernel that rocprofv3 --pmc traffic counters are scaled against)")
    ap.add_argument("--extra", action="store_true", help="also time the other launch modes, outside the timed region")
    ap.add_argument("--no-phases", action="store_true",
                    help="decode: skip the extra generations that time the prompt and the generated tokens apart")
    ap.add_argument("--no-decode", action="store_true",
                    help="projection_set only: skip the end-to-end decode figure that is attached to the JSON line")
    ap.add_argument("--no-configs", action="store_true",
                    help="projection_set only: skip the sub-records of the other benchmark configurations (batch 8 / 16, "
                         "prefill GEMM at M = 64 / 512 / 2048, Q4_K GEMV and GEMM) that the default run attaches")
    ap.add_argument("--threads", type=int, default=0,
                    help="threads of the CPU baseline legs (default: the host's physical cores, capped by OMP_NUM_THREADS)")
    args = ap.parse_args()
    global THREADS_OVERRIDE
    THREADS_OVERRIDE = args.threads or None
    # compute-bound workloads wait for settled clocks unless the warm-up is given on the command line (then it is
    # exactly the W asked for)
    args.settle_ms = SETTLE_MS if args.warmup is None else 0.0
    long_run = args.workload in ("q4_0", "q4k", "q6k")
    if args.steps is None:
        args.steps = 500 if long_run else 50
    if args.warmup is None:
        args.warmup = 100 if long_run else 10
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here shards across GPUs", file=sys.stderr)
        sys.exit(2)

    pkg = importlib.import_module("rust-model-inference_amd")
    pkg.init(int(os.environ.get("LOCAL_RANK", "0")))
    ev = HipEvents()
    run = {"projection_set": run_projection_set, "single_gemv": run_single_gemv, "gemm": run_gemm, "q4_0": run_q4_0, "q4k": run_q4k, "q6k": run_q6k, "q4k_gemm": run_q4k_gemm, "qlinear": run_qlinear,
           "attention": run_attention, "decode": run_decode}[args.workload]
    result = run(args, pkg, ev)
    if args.workload == "projection_set" and not args.no_decode and args.batch == 1:
        # the second half of the headline metric: end-to-end decode tok/s of the same model shape, measured
        # after (and outside) the timed GEMV region
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup = 2, 1
        d = run_decode(sub, pkg, ev)
        result["decode"] = {"value": d["value"], "unit": d["unit"], "ms_per_token_step": d["ms_per_token_step"], "phases": d.get("phases"),
                            "workload": d["config"]["workload"], "generations_timed": sub.steps,
                            "roofline": d["roofline"], "cpu_baseline": d.get("cpu_baseline")}
    if args.workload == "projection_set" and not args.no_configs and args.batch == 1 and args.mode == "grouped" \
            and args.order == "avx2":
        # the other benchmark configurations, each measured like the headline (own warm-up, own timed steps between
        # synchronisations, HIP events on the launch stream), after and outside the headline's timed region
        configs = {}
        t_cfg = time.time()
        sub = argparse.Namespace(**vars(args))
        sub.copy_calibration_mb = 0
        configs["single_gemv_3072x1024"] = compact(run_single_gemv(sub, pkg, ev))
        configs.update(run_small_batches(args, pkg, ev))
        for m in (64, 512, 2048):
            sub = argparse.Namespace(**vars(args))
            sub.tokens, sub.steps, sub.warmup, sub.copy_calibration_mb, sub.settle_ms = m, 50, 10, 0, SETTLE_MS
            configs[f"gemm_m{m}"] = compact(run_gemm(sub, pkg, ev))
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup, sub.batch, sub.copy_calibration_mb = 300, 100, 1, 0
        configs["q4k_gemv"] = compact(run_q4k(sub, pkg, ev))
        sub = argparse.Namespace(**vars(args))
        sub.tokens, sub.steps, sub.warmup, sub.copy_calibration_mb, sub.settle_ms = 512, 50, 10, 0, SETTLE_MS
        configs["q4k_gemm_m512"] = compact(run_q4k_gemm(sub, pkg, ev))
        result["configs"] = configs
        log(f"[bench] other configurations measured in {time.time() - t_cfg:.1f}s")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()

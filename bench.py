#!/usr/bin/env python3
"""Benchmark of the optimizer-step hot path on one MI355X.

A "step" is one optimizer step over the whole synthetic parameter list of the chosen
workload, with weights, gradients and state already resident in HBM.  The default workload
is the headline configuration: Adam with weight decay 1e-4 over 1,012,301,824 fp32
parameters in 400 tensors shaped like transformer blocks.

Prints ONE JSON line: params updated per second (whole job), ms per step, the roofline of
the dominant kernel (algorithmic bytes per launch / launch duration measured with HIP
events on the library's own stream, against MI355X's 8 TB/s HBM peak), the same figures for
the mixed-precision (fp16 gradient) Adam step ("amp": the form that updates in place, which
StepAMP runs by default, and the one-pass form over ping-pong state; each also without the
per-step host wait under "async"), and the CPU oracle timed on this host's cores on a bounded
sample of the same workload.

Without --workload, every benchmark configuration runs, each in a process of its own.  The one
line printed is then a short one (under 2 KB): the headline configuration's record, and under
"configs" the figures of configurations 1 to 4; the full records go to a file the line names
(--workload all adds the L-BFGS workloads and the buffer primitives; --workload NAME runs one
workload in this process and prints its full record).
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "go-metal_amd"))      # workloads.py: the configurations' tensor lists

HBM_PEAK_GBS = 8000.0
RECORDS_FILE = os.path.join("gpurun_out", "bench_configs.json")     # full per-configuration records of the default run
LINE_LIMIT = 1960         # bytes of the default run's final line: the driver keeps the tail of stdout
ROTATE_C3 = 6            # copies of the 25M list stepped in turn by the default run: 6 x 300-400 MB
STATE_PHASES = (512 << 10, 1536 << 10, 1 << 20)     # host/memory_manager.hpp, kStatePhases


def state_phase(j, nbytes):
    """Where MemoryManager.AllocateStateBuffer starts the j-th state buffer of a tensor: at its own phase modulo
    2 MiB when the request falls into the 16 MiB tier or above (more than 4 MiB), anywhere otherwise."""
    return STATE_PHASES[j % len(STATE_PHASES)] if nbytes > (4 << 20) else None

# algorithmic bytes per parameter per step: every stream read once and / or written once
BYTES_PER_PARAM = {"sgd": 20, "adam": 28, "rmsprop": 20, "adagrad": 20, "adadelta": 28, "nadam": 28,
                   "adam_amp": 28}


# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this
# file (summary and commands: profiles/adam_c5_1b_hbm_traffic.md); None where not measured.
MEASURED_HBM_TRAFFIC = {("c5", "adam"): 2.8359e10,
                        # the launches of one in-place mixed-precision step: check 2.026e9 + update 2.8345e10
                        ("c5", "adam_amp"): 3.0385e10,
                        # the one-pass step over ping-pong state: a single update launch
                        ("c5", "adam_amp_one_pass"): 2.8375e10,
                        # configs 3 and 4 (profiles/c3_c4_hbm_traffic.md)
                        ("c3-rmsprop", "rmsprop"): 5.0643e8, ("c3-adagrad", "adagrad"): 5.0644e8,
                        ("c3-adadelta", "adadelta"): 7.0642e8, ("c3-nadam", "nadam"): 7.0640e8,
                        ("c4", "adam"): 3.5019e9, ("c4", "adam_amp"): 3.7522e9, ("c4", "adam_amp_one_pass"): 3.5039e9,
                        # bytes per step, summed over the passes of a 10-pair step (profiles/lbfgs_c5_1b_hbm_traffic.md)
                        ("lbfgs-c5", 10): 352.68 * 1012301824}
TRAFFIC_SOURCE = {("lbfgs-c5", 10): "profiles/lbfgs_c5_1b_hbm_traffic.md"}
TRAFFIC_SOURCE.update({k: "profiles/adam_c5_1b_hbm_traffic.md" for k in MEASURED_HBM_TRAFFIC if k[0] == "c5"})
TRAFFIC_SOURCE.update({k: "profiles/c3_c4_hbm_traffic.md" for k in MEASURED_HBM_TRAFFIC if k[0][:2] in ("c3", "c4")})


def traffic_fields(key):
    """roofline.traffic and where it comes from: HBM bytes per launch from separate rocprofv3 counter runs of this
    file (FETCH_SIZE, then WRITE_SIZE), copied from the named summary; this run does not read counters."""
    if key not in MEASURED_HBM_TRAFFIC:
        return {"traffic": None, "traffic_source": "not measured for this workload"}
    return {"traffic": MEASURED_HBM_TRAFFIC[key],
            "traffic_source": f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, summary in "
                              f"{TRAFFIC_SOURCE[key]}; a constant from that profile, not measured by this run"}

from workloads import amp_125m_sizes, cnn_sizes, ragged_sizes, transformer_block_sizes  # noqa: E402

WORKLOADS = {
    # name: (description, sizes(), rule, hyper, gradient std)
    "c1": ("config1: Adam, one flat tensor of 1,048,576 params", lambda: [1 << 20], "adam",
           dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0), 1e-2),
    "c2-sgd": ("config2: SGD-momentum over the 16-tensor CNN list (1,143,690 params)", cnn_sizes, "sgd",
               dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=False), 1e-3),
    "c2-adam": ("config2: Adam over the 16-tensor CNN list (1,143,690 params)", cnn_sizes, "adam",
                dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0), 1e-3),
    "c3-rmsprop": ("config3: RMSprop, 25M params in 160 ragged tensors", ragged_sizes, "rmsprop",
                   dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0, centered=False), 1e-3),
    "c3-adagrad": ("config3: AdaGrad, 25M params in 160 ragged tensors", ragged_sizes, "adagrad",
                   dict(lr=0.01, eps=1e-10, weight_decay=0.0), 1e-3),
    "c3-adadelta": ("config3: AdaDelta, 25M params in 160 ragged tensors", ragged_sizes, "adadelta",
                    dict(rho=0.9, eps=1e-6, weight_decay=0.0), 1e-3),
    "c3-nadam": ("config3: NAdam, 25M params in 160 ragged tensors", ragged_sizes, "nadam",
                 dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0), 1e-3),
    "c4": ("config4: mixed-precision Adam, 125M params in 60 tensors", amp_125m_sizes, "adam",
           dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0), 1e-4),
    "c5": ("config5: Adam + weight decay 1e-4, 1,012,301,824 params in 400 transformer-block tensors",
           transformer_block_sizes, "adam",
           dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4), 1e-4),
}


def checker():
    """The CPU oracle's Python binding (tests/oracle_lib.py).  Only the cpu_baseline legs call this: nothing on
    the GPU path of this file imports from tests/ or touches the oracle."""
    tests_dir = os.path.join(ROOT, "tests")
    if tests_dir not in sys.path:
        sys.path.insert(0, tests_dir)
    from oracle_lib import oracle
    return oracle()


def cpu_model():
    """The host CPU's model name (reported beside the CPU baseline)."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def time_steps(dev, launch, steps, warmup):
    """W untimed steps, then exactly K steps bracketed by a device synchronisation on both
    sides.  Returns (wall ms per step, HIP-event ms per launch)."""
    for _ in range(warmup):
        launch()
    dev.synchronize()
    t0 = time.perf_counter()
    dev.lib.gm_timer_start(dev.handle)
    for _ in range(steps):
        launch()
    event_ms = dev.lib.gm_timer_stop(dev.handle)     # records the stop event and waits for it
    dev.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, event_ms / steps


def per_launch_times(dev, launch, steps):
    """HIP-event time of each of `steps` launches taken one at a time: (median ms, min ms)."""
    times = []
    for _ in range(steps):
        dev.lib.gm_timer_start(dev.handle)
        launch()
        times.append(dev.lib.gm_timer_stop(dev.handle))
    return float(np.median(times)), float(min(times))


def cpu_baseline_amp(sizes, hyper, grad_std, budget_params=96_000_000, target_seconds=3.0):
    """The oracle's mixed-precision Adam step (clean steps: check, unscale, update, fp16 copy) on this host."""
    o = checker()
    threads = min(16, os.cpu_count() or 1)
    chosen, total = [], 0
    for n in sizes:
        if chosen and total + n > budget_params:
            break
        chosen.append(n)
        total += n
    rng = np.random.default_rng(2)
    w = [rng.standard_normal(n, dtype=np.float32) * np.float32(0.02) for n in chosen]
    m = [np.zeros(n, np.float32) for n in chosen]
    v = [np.zeros(n, np.float32) for n in chosen]
    w16 = [np.zeros(n, np.uint16) for n in chosen]
    g16 = [(rng.standard_normal(n, dtype=np.float32) * np.float32(grad_std * 65536.0)).astype(np.float16).view(np.uint16)
           for n in chosen]
    st = o.amp_state(65536.0, 2.0, 0.5, 1 << 30)
    step = lambda: o.adam_amp(w, g16, m, v, w16, state=st, nthreads=threads, **hyper)
    step()
    t0 = time.perf_counter()
    step()
    one = max(time.perf_counter() - t0, 1e-4)
    steps = int(min(1_000_000, max(3, target_seconds / one)))
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    dt = time.perf_counter() - t0
    return {"value": total * steps / dt, "unit": "params/s", "cores": threads, "kind": "port",
            "sample_params": total, "sample_steps": steps, "sample_seconds": dt,
            "sample": f"first {len(chosen)} tensors ({total} params) of the workload, {steps} mixed-precision steps in "
                      f"{dt:.1f} s, oracle/oracle.c (eight-lane AVX2 + F16C form where the host has them) with OpenMP "
                      f"on {threads} threads of {os.cpu_count()} ({cpu_model()})"}


def cpu_baseline(sizes, rule, hyper, grad_std, budget_params=96_000_000, target_seconds=12.0):
    """The CPU oracle (a C port of the reference's update equations, OpenMP over elements) on
    this host, on the leading tensors of the same workload up to ~budget_params, for about
    target_seconds of CPU work."""
    checker()
    from harness import OracleRun
    threads = min(16, os.cpu_count() or 1)
    chosen, total = [], 0
    for n in sizes:
        if chosen and total + n > budget_params:
            break
        chosen.append(n)
        total += n
    rng = np.random.default_rng(1)
    w = [rng.standard_normal(n, dtype=np.float32) * np.float32(0.02) for n in chosen]
    g = [rng.standard_normal(n, dtype=np.float32) * np.float32(grad_std) for n in chosen]
    run = OracleRun(rule, hyper, w, nthreads=threads)
    run.step(g)                                   # warm-up (page faults, thread pool)
    t0 = time.perf_counter()
    run.step(g)
    one = max(time.perf_counter() - t0, 1e-4)
    steps = int(min(1_000_000, max(3, target_seconds / one)))
    t0 = time.perf_counter()
    for _ in range(steps):
        run.step(g)
    dt = time.perf_counter() - t0
    return {"value": total * steps / dt, "unit": "params/s", "cores": threads, "kind": "port",
            "sample_params": total, "sample_steps": steps, "sample_seconds": dt,
            "sample": f"first {len(chosen)} tensors ({total} params) of the workload, {steps} steps in "
                      f"{dt:.1f} s, oracle/oracle.c with OpenMP on {threads} threads of {os.cpu_count()} "
                      f"({cpu_model()})"}


LBFGS_WORKLOADS = {
    # name: (description, sizes(), history size)
    "lbfgs-c3": ("L-BFGS, history 10 (all pairs valid), 25M params in 160 ragged tensors", ragged_sizes, 10),
    "lbfgs-c5": ("L-BFGS, history 10 (all pairs valid), 1,012,301,824 params in 400 transformer-block tensors",
                 transformer_block_sizes, 10),
}


def lbfgs_bytes_per_param(valid_pairs):
    """Algorithmic HBM bytes per parameter of one L-BFGS step with a non-empty history: every pass reads its
    operands once and writes its result once.  The last pass is the update: it reads r (or nothing, when no
    pair is valid: r = -g is formed from the gradient it reads anyway), w, g and writes p, w, old_g, s_cur,
    y_prev.  No valid pair: 8 + 20 = 28.  c valid pairs: first dot product (8: q = -g is not stored) + c
    backward (16; the last one 12, its dot operand y_0 being the buffer its axpy reads) + c forward (16; the last
    one 12, no dot) + update (12 + 20)."""
    c = valid_pairs
    return 28 if c == 0 else 8 + (16 * c - 4) + (16 * c - 4) + 32


def bench_lbfgs(args, pkg, dev):
    lib, D = dev.lib, dev.handle
    desc, sizes_fn, m = LBFGS_WORKLOADS[args.workload]
    if args.history > 0:
        desc = desc.replace(f"history {m}", f"history {args.history}")
        m = args.history
    sizes = sizes_fn()
    n, params = len(sizes), sum(sizes)
    fill = lambda h, k, seed, std: lib.gm_fill_normal_f32(D, h, k, seed, 0.0, std)

    def tensor_list(seed, std):
        hs = [dev.alloc(4 * k) for k in sizes]
        for i, k in enumerate(sizes):
            fill(hs[i], k, seed + i, std)
        print(f"filled a list of {len(sizes)} tensors", file=sys.stderr, flush=True)
        return hs

    w, g = tensor_list(0x1000, 0.02), tensor_list(0x2000, 1e-2)
    old_g, direction = tensor_list(0x3000, 1e-2), tensor_list(0x4000, 1e-2)
    s = [tensor_list(0x10000 * (h + 1), 1e-2) for h in range(m)]
    y = [tensor_list(0x10000 * (h + 1) + 0x8000, 1e-2) for h in range(m)]
    rho_value = np.full(1, 1e-3, np.float32)
    rho = [dev.from_numpy(rho_value) for _ in range(m)]
    alpha = dev.alloc(4 * m, zero=True)
    dev.synchronize()
    arr = pkg.handle_array
    cw, cg, co, cd = arr(w), arr(g), arr(old_g), arr(direction)
    cs, cy, cr = arr([b for h in s for b in h]), arr([b for h in y for b in h]), arr(rho)
    bs = pkg.int_array([4 * k for k in sizes])
    step_size = ctypes.c_float()
    state = {"index": 0}

    def launch(count, valid=True):
        # a step with index i ends by clearing rho[i - 1] (its y is g - g); put the value back before the
        # next step so that every pair stays valid
        idx = state["index"]
        if count and valid:
            dev.upload(rho[(idx - 2) % m], rho_value)
        rc = lib.execute_lbfgs_step_mpsgraph(D, cw, cg, co, cd, cs, cy, cr, alpha, n, bs, m, count, idx, 0.01,
                                             1e-4, 0.9, 20, 1.0, 1.0, ctypes.byref(step_size))
        if rc != 0:
            raise RuntimeError(f"L-BFGS step failed rc={rc}: {lib.gm_last_error().decode()}")
        state["index"] = (idx + 1) % m

    full_wall, full_event = time_steps(dev, lambda: launch(m), args.steps, args.warmup)
    live = sum(1 for h in rho if dev.to_numpy(h, 1)[0] != 0.0)
    if live < m - 1:
        raise RuntimeError(f"only {live} of {m} history pairs stayed valid during the timed steps")
    # the history the reference's own optimizer produces: every rho is 0, a step is update + curvature
    for h in rho:
        dev.upload(h, np.zeros(1, np.float32))
    plain_wall, plain_event = time_steps(dev, lambda: launch(m, valid=False), args.steps, args.warmup)
    bpp = lbfgs_bytes_per_param(m)
    achieved = params * bpp / (full_event * 1e-3) / 1e9
    plain = params * lbfgs_bytes_per_param(0) / (plain_event * 1e-3) / 1e9
    result = {
        "metric": f"params updated/sec (L-BFGS step, {m} history pairs) + achieved HBM GB/s",
        "value": params / (full_wall * 1e-3), "unit": "params/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": full_wall, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 (dot products accumulated in f64)", "data": "synthetic",
        "config": {"workload": desc, "tensors": n, "params": params, "rule": "lbfgs", "history_size": m},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, **traffic_fields((args.workload, m)),
                     "kernel": "lbfgs_stream_kernel (all passes)",
                     "bytes_per_param": bpp, "kernel_ms": full_event,
                     "note": "time covers every pass of the step, the tree reductions between them and the "
                             "read-back of the pair flags"},
        "all_pairs_invalid_step": {"ms_per_step": plain_wall, "bytes_per_param": lbfgs_bytes_per_param(0),
                               "achieved": plain, "frac": plain / HBM_PEAK_GBS},
    }
    if args.no_cpu_baseline:
        result["cpu_baseline"] = None
    else:
        result["cpu_baseline"] = lbfgs_cpu_baseline(sizes, m)
    dev.close()
    print(json.dumps(result))


def bench_placement(args, pkg, dev):
    """Where the state buffers start against where hipMalloc would put them: the fp32 Adam step over the 1.012B list
    in several layouts of device memory (a spacer of a different size in front of the lists each time, which moves
    every later allocation), once with the two moment streams allocated plainly, exact sizes, stream after stream,
    and once with them at the phases the optimizers use.  Same weights and gradients for both."""
    lib, D = dev.lib, dev.handle
    from workloads import transformer_block_sizes
    sizes = transformer_block_sizes()
    n, params = len(sizes), sum(sizes)
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    bs = pkg.int_array([4 * s for s in sizes])
    rows = []
    spacers = [0, 3 << 20, 34 << 20, 129 << 20, (512 << 20) + (6 << 20), (1 << 30) + (77 << 20)]
    for spacer in spacers:
        pad = dev.alloc(spacer) if spacer else 0
        w = [dev.alloc(4 * s) for s in sizes]
        g = [dev.alloc(4 * s) for s in sizes]
        plain = [[dev.alloc(4 * s, zero=True) for s in sizes] for _ in range(2)]
        placed = [[dev.alloc(4 * s, zero=True, phase=state_phase(j, 4 * s)) for s in sizes] for j in range(2)]
        for k, s in enumerate(sizes):
            lib.gm_fill_normal_f32(D, w[k], s, 0x6D657461 + k, 0.0, 0.02)
            lib.gm_fill_normal_f32(D, g[k], s, 0x12345 + k, 0.0, 1e-4)
        dev.synchronize()
        cw, cg = pkg.handle_array(w), pkg.handle_array(g)
        row = {"spacer_bytes": spacer}
        t = {"t": 0}
        for name, states in (("plain", plain), ("placed", placed), ("plain_again", plain), ("placed_again", placed)):
            cm, cv = pkg.handle_array(states[0]), pkg.handle_array(states[1])

            def launch():
                t["t"] += 1
                rc = lib.execute_adam_step_mpsgraph(D, cw, cg, cm, cv, n, bs, hyper["lr"], hyper["beta1"], hyper["beta2"],
                                                    hyper["eps"], hyper["weight_decay"], t["t"])
                if rc != 0:
                    raise RuntimeError(f"adam step failed rc={rc}: {lib.gm_last_error().decode()}")
            _, ms = time_steps(dev, launch, args.steps, max(args.warmup, 5))
            row[name] = {"kernel_ms": ms, "frac": params * 28 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        rows.append(row)
        for h in w + g + plain[0] + plain[1] + placed[0] + placed[1] + ([pad] if pad else []):
            dev.free(h)
    mean = lambda key: sum((r[key]["frac"] + r[key + "_again"]["frac"]) / 2 for r in rows) / len(rows)
    result = {"metric": "fraction of HBM peak of the fp32 Adam step by placement of the state buffers",
              "unit": "fraction of 8 TB/s", "n_gpus": 1, "steps": args.steps, "warmup": max(args.warmup, 5),
              "config": {"workload": "placement: 1,012,301,824 params in 400 tensors, six layouts of device memory",
                         "state_phases": list(STATE_PHASES[:2])},
              "plain_mean": mean("plain"), "placed_mean": mean("placed"),
              "plain_range": [min(min(r["plain"]["frac"], r["plain_again"]["frac"]) for r in rows),
                              max(max(r["plain"]["frac"], r["plain_again"]["frac"]) for r in rows)],
              "placed_range": [min(min(r["placed"]["frac"], r["placed_again"]["frac"]) for r in rows),
                               max(max(r["placed"]["frac"], r["placed_again"]["frac"]) for r in rows)],
              "layouts": rows}
    dev.close()
    print(json.dumps(result))


def bench_primitives(args, pkg, dev):
    """Buffer primitives of the boundary on one large buffer each: zero fill, fp32 <-> fp16 conversion,
    device-to-device copy (HBM-bound, timed with HIP events on the library's stream) and the host copies
    in both directions (PCIe-bound, wall time; the caller's array is ordinary pageable memory)."""
    lib, D = dev.lib, dev.handle
    elems = 1 << 28                                   # 1 GiB of fp32, 512 MiB of fp16
    f32, f16, f32b = dev.alloc(4 * elems), dev.alloc(2 * elems), dev.alloc(4 * elems)
    lib.gm_fill_normal_f32(D, f32, elems, 0x51, 0.0, 1.0)
    dev.synchronize()
    shape = pkg.int_array([elems])
    F32, F16 = 0, 2

    def checked(rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed rc={rc}: {lib.gm_last_error().decode()}")

    cases = {
        "zero_metal_buffer": (lambda: checked(lib.zero_metal_buffer(D, f32b, 4 * elems), "zero"), 4 * elems),
        "convert_tensor_type f32->f16": (lambda: checked(lib.convert_tensor_type(f32, f16, shape, 1, F32, F16, D),
                                                         "convert"), 6 * elems),
        "convert_tensor_type f16->f32": (lambda: checked(lib.convert_tensor_type(f16, f32b, shape, 1, F16, F32, D),
                                                         "convert"), 6 * elems),
        "copy_buffer_to_buffer_sync": (lambda: checked(lib.copy_buffer_to_buffer_sync(f32, f32b, 0, 0, 4 * elems),
                                                       "copy"), 8 * elems),
        "gm_copy_probe (16-byte copy kernel)": (lambda: checked(lib.gm_copy_probe(D, f32b, f32, 4 * elems), "probe"),
                                                8 * elems),
    }
    table = {}
    for name, (launch, nbytes) in cases.items():
        wall_ms, event_ms = time_steps(dev, launch, args.steps, args.warmup)
        gbs = nbytes / (event_ms * 1e-3) / 1e9
        table[name] = {"bytes": nbytes, "kernel_ms": event_ms, "ms_per_call": wall_ms, "achieved": gbs,
                       "frac": gbs / HBM_PEAK_GBS}
        print(f"{name}: {event_ms:.4f} ms, {gbs:.0f} GB/s", file=sys.stderr, flush=True)

    host_elems = 1 << 26                              # 256 MiB
    host = np.random.default_rng(3).standard_normal(host_elems, dtype=np.float32)
    back = np.empty_like(host)
    fp = ctypes.POINTER(ctypes.c_float)
    pcie = {}
    for name, call in (("copy_float32_array_to_metal_buffer",
                        lambda: lib.copy_float32_array_to_metal_buffer(f32, host.ctypes.data_as(fp), host_elems)),
                       ("copy_metal_buffer_to_float32_array",
                        lambda: lib.copy_metal_buffer_to_float32_array(f32, back.ctypes.data_as(fp), host_elems))):
        checked(call(), name)
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            checked(call(), name)
        dt = (time.perf_counter() - t0) / reps
        pcie[name] = {"bytes": 4 * host_elems, "ms_per_call": dt * 1e3, "achieved": 4 * host_elems / dt / 1e9,
                      "unit": "GB/s", "bound": "pcie, pageable host memory"}
    if not np.array_equal(host, back):
        raise RuntimeError("host round trip changed the data")

    result = {"metric": "achieved HBM GB/s of the buffer primitives (% of peak)", "unit": "GB/s", "n_gpus": 1,
              "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None, "dtype": "f32 / f16 / bytes", "data": "synthetic",
              "config": {"workload": f"buffer primitives on {elems} elements", "elements": elems}}
    head = table["convert_tensor_type f32->f16"]
    result["value"] = head["achieved"]
    result["ms_per_step"] = head["ms_per_call"]
    result["roofline"] = {"bound": "hbm", "achieved": head["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": head["frac"], **traffic_fields(None), "kernel": "convert_f32_to_f16_kernel",
                          "kernel_ms": head["kernel_ms"]}
    result["primitives"] = table
    result["host_copies"] = pcie
    if args.no_cpu_baseline:
        result["cpu_baseline"] = None
    else:
        o = checker()
        threads = min(16, os.cpu_count() or 1)
        sample = host
        o.f32_to_f16(sample, nthreads=threads)
        t0, reps = time.perf_counter(), 0
        while time.perf_counter() - t0 < 10.0:
            o.f32_to_f16(sample, nthreads=threads)
            reps += 1
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": 6 * host_elems * reps / dt / 1e9, "unit": "GB/s", "cores": threads,
                                  "kind": "port",
                                  "sample": f"fp32->fp16 conversion of {host_elems} elements, {reps} calls in "
                                            f"{dt:.1f} s, oracle/oracle.c on {threads} threads ({cpu_model()})"}
    for h in (f32, f16, f32b):
        dev.free(h)
    dev.close()
    print(json.dumps(result))


def lbfgs_cpu_baseline(sizes, m, budget_params=6_000_000, target_seconds=12.0):
    """The reference's algorithm as it runs it: one CPU thread, running fp32 sums
    (oracle/oracle_lbfgs.c in reference order), on the leading tensors of the workload."""
    o = checker()
    chosen, total = [], 0
    for k in sizes:
        if chosen and total + k > budget_params:
            break
        chosen.append(k)
        total += k
    rng = np.random.default_rng(1)
    r = lambda std: [rng.standard_normal(k, dtype=np.float32) * np.float32(std) for k in chosen]
    st = {"w": r(0.02), "old_g": r(1e-2), "dir": r(1e-2), "s": [r(1e-2) for _ in range(m)],
          "y": [r(1e-2) for _ in range(m)], "rho": np.full(m, 1e-3, np.float32), "alpha": np.zeros(m, np.float32)}
    g = r(1e-2)
    steps, index, dt = 0, 0, 0.0
    while dt < target_seconds and steps < 2000:
        st["rho"][:] = 1e-3
        t0 = time.perf_counter()
        o.lbfgs_step(st, g, m, m, index, 0.01, 0)
        dt += time.perf_counter() - t0
        index = (index + 1) % m
        steps += 1
    return {"value": total * steps / dt, "unit": "params/s", "cores": 1, "kind": "port",
            "sample": f"first {len(chosen)} tensors ({total} params) of the workload, {steps} steps in {dt:.1f} s, "
                      "oracle/oracle_lbfgs.c in the reference's summation order on one thread (the reference "
                      f"runs this step as a single-threaded CPU loop); host: {cpu_model()}"}


BASELINE_CONFIGS = ["c5", "c1", "c2-sgd", "c2-adam", "c3-rmsprop", "c3-adagrad", "c3-adadelta", "c3-nadam", "c4"]


def _sig(x, digits=5):
    """A number with `digits` significant digits (the final line is kept short; full precision is in the file);
    an integer where that loses nothing, which prints shorter."""
    if x is None or isinstance(x, (str, bool)) or x == 0:
        return x
    r = float(f"{x:.{digits}g}")
    return int(r) if abs(r) >= 10 ** digits else r


def compact_line(results, records_file):
    """The one line the default run prints LAST, under 2 KB: the headline configuration's record (config 5, fp32
    Adam) with its roofline and CPU baseline, the two forms of the mixed-precision step over the same list, and per
    other configuration only the figures (ms per step, params/s, fraction of peak, kernel ms, CPU params/s).  The
    full per-configuration records, prose fields included, are in `records_file`."""
    h = results["c5"]
    roof = h["roofline"]
    line = {
        "metric": h["metric"], "value": _sig(h["value"], 7), "unit": h["unit"], "n_gpus": 1, "steps": h["steps"],
        "warmup": h["warmup"], "ms_per_step": _sig(h["ms_per_step"], 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": h["config"]["workload"], "tensors": h["config"]["tensors"], "params": h["config"]["params"]},
        "roofline": {"bound": "hbm", "achieved": _sig(roof["achieved"], 6), "peak": roof["peak"], "unit": "GB/s",
                     "frac": _sig(roof["frac"]), "traffic": roof.get("traffic"), "kernel": roof["kernel"],
                     "kernel_ms": _sig(roof["kernel_ms"], 6), "bytes_per_param": roof["bytes_per_param"]},
    }
    cpu = h.get("cpu_baseline")
    line["cpu_baseline"] = None if cpu is None else {
        "value": _sig(cpu["value"]), "unit": cpu["unit"], "cores": cpu["cores"], "kind": cpu["kind"],
        "sample": (f"{cpu['sample_params']} params x {cpu['sample_steps']} steps, {cpu['sample_seconds']:.1f} s, oracle.c OpenMP"
                   if "sample_params" in cpu else cpu["sample"][:64])}
    amp = h.get("amp")
    if amp:
        form = lambda r: {"frac": _sig(r["roofline"]["frac"], 4), "ms_per_step": _sig(r["ms_per_step"], 4)}
        line["amp"] = {"default": amp["default_form"], "one_pass": form(amp["one_pass"]), "in_place": form(amp["in_place"]),
                       "bytes_per_param": 28}
    configs = {}
    for name, r in results.items():
        if name == "c5":
            continue
        rr = r.get("roofline") or {}
        c = {"ms_per_step": _sig(r.get("ms_per_step"), 4), "steps": r.get("steps"), "value": _sig(r.get("value"), 4),
             "frac": _sig(rr.get("frac"), 4), "kernel_ms": _sig(rr.get("kernel_ms"), 4)}
        if rr.get("frac_hbm") is not None:
            c["frac_hbm"] = _sig(rr["frac_hbm"], 4)
        if r.get("one_pass"):
            c["frac_one_pass"] = _sig(r["one_pass"]["roofline"]["frac"], 4)
        cb = r.get("cpu_baseline")
        c["cpu"] = _sig(cb["value"], 3) if cb else None
        configs[name] = c
    line["configs"] = configs
    line["records"] = records_file

    def render():
        text = json.dumps(line, separators=(",", ":"))
        # integers that end in six or more zeros in exponent form: 235100000000 -> 2351e8 (the same JSON number)
        return re.sub(r"(?<=[:\[,])(\d+?)(0{6,})(?=[,}\]])", lambda m: f"{m.group(1)}e{len(m.group(2))}", text)

    # the limit holds by construction: if the figures print longer than expected, the least needed fields go
    def shorten_sample():
        if line["cpu_baseline"]:
            line["cpu_baseline"]["sample"] = line["cpu_baseline"]["sample"][:24]
    trims = [shorten_sample] + [lambda key=key: [c.pop(key, None) for c in configs.values()]
                                for key in ("kernel_ms", "steps", "cpu")]
    text = render()
    while len(text) > LINE_LIMIT and trims:
        trims.pop(0)()
        text = render()
    return text


def run_children(args, names):
    """Each named workload as a child process, started before this process has made any GPU call (it never
    makes one).  The full records go to the file RECORDS_FILE names; the last line printed is the headline
    configuration's, with the other configurations' figures under "configs" (compact_line)."""
    import subprocess
    results = {}
    for name in names:
        # Steps over the smaller lists take 5 to 500 us, and the first few hundred launches after the device
        # has been idle run slower: those workloads get at least 300 warm-up steps so that the timed ones
        # show the kernels at their steady rate.  Their CPU samples are 3 s each, the headline's 12 s.
        headline = name in ("c5", "lbfgs-c5", "primitives")
        warmup = args.warmup if headline else max(args.warmup, 300)
        # ... and at least 200 timed steps, so that the one wait at the end of the timed region (about 40 us)
        # does not show in a per-step figure of a few microseconds; every record states its own counts
        steps = args.steps if headline or name == "lbfgs-c3" else max(args.steps, 200)
        cmd = [sys.executable, os.path.abspath(__file__), "--workload", name, "--steps", str(steps),
               "--warmup", str(warmup), "--cpu-seconds", str(args.cpu_seconds if name == "c5" else min(args.cpu_seconds, 3.0))]
        if name.startswith("c3-"):
            cmd += ["--rotate", str(ROTATE_C3)]
        if args.no_cpu_baseline:
            cmd.append("--no-cpu-baseline")
        print(f"running {name}", file=sys.stderr, flush=True)
        out = subprocess.run(cmd, check=True, stdout=subprocess.PIPE, text=True).stdout
        results[name] = json.loads(out.strip().splitlines()[-1])
    os.makedirs(os.path.dirname(os.path.join(ROOT, RECORDS_FILE)), exist_ok=True)
    with open(os.path.join(ROOT, RECORDS_FILE), "w") as f:
        json.dump(results, f, indent=1)
    print(compact_line(results, RECORDS_FILE), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="", choices=[""] + sorted(WORKLOADS) + sorted(LBFGS_WORKLOADS) + ["primitives", "placement", "all"],
                    help="one workload in this process.  Default: the five benchmark configurations in turn, each in a "
                         "process of its own; the line printed is the headline configuration's (c5) with the others "
                         "under 'configs'.  'all': the same plus the L-BFGS workloads and the buffer primitives")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU time of the oracle sample (cpu_baseline)")
    ap.add_argument("--amp-check-order", default="", help="mixed-precision overflow check, for re-measurement: "
                    "'NT,REV' with NT 1/0 = non-temporal loads on/off and REV 1/0 = walk the table backwards")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-amp", action="store_true")
    ap.add_argument("--rotate", type=int, default=0,
                    help="also step K independent copies of the list in turn (K x footprint beyond the 256 MB memory-side "
                         "cache), so that no stream of a step is still cached from the step before: roofline.frac_hbm")
    ap.add_argument("--history", type=int, default=0, help="L-BFGS workloads: history size (default 10)")
    ap.add_argument("--rule", default="", choices=["", "sgd", "adam", "rmsprop", "adagrad", "adadelta", "nadam"],
                    help="run another update rule (with the benchmark configurations' hyper-parameters for it) over the workload's list")
    # launch-shape overrides (gm_set_tuning) for comparing lane widths and chunk sizes; 0 / -1 = default
    ap.add_argument("--chunk", type=int, default=0, help="elements per chunk")
    ap.add_argument("--vec", type=int, default=0, help="fp32 elements per lane: 1, 2 or 4 (0: chosen per launch)")
    ap.add_argument("--nontemporal", type=int, default=-1, help="1 / 0: non-temporal hint on / off")
    ap.add_argument("--lanes", type=int, default=0, help="lanes per workgroup of the update kernels: 128 or 256")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the optimizer step shards without communication, and this "
                 "build runs and reports a single MI355X (--gpus 1).")

    if args.workload == "":
        return run_children(args, BASELINE_CONFIGS)
    if args.workload == "all":
        return run_children(args, BASELINE_CONFIGS + sorted(LBFGS_WORKLOADS) + ["primitives"])

    from __graft_entry__ import load_package
    pkg = load_package()
    dev = pkg.Device()                 # raises if the library is not built or no GPU is visible
    lib, D = dev.lib, dev.handle
    if lib.gm_set_tuning(D, args.chunk, args.nontemporal, args.vec) != 0:
        sys.exit("invalid --chunk / --vec combination (a chunk is a power-of-two multiple of 256 * vec elements)")
    if lib.gm_set_workgroup_lanes(D, args.lanes) != 0:
        sys.exit("invalid --lanes (128 or 256)")
    if args.amp_check_order:
        nt_flag, rev_flag = (int(x) for x in args.amp_check_order.split(","))
        lib.gm_set_amp_check_order(D, nt_flag, rev_flag)

    if args.workload in LBFGS_WORKLOADS:
        return bench_lbfgs(args, pkg, dev)
    if args.workload == "primitives":
        return bench_primitives(args, pkg, dev)
    if args.workload == "placement":
        return bench_placement(args, pkg, dev)

    desc, sizes_fn, rule, hyper, grad_std = WORKLOADS[args.workload]
    if args.rule and args.rule != rule:
        rule = args.rule
        hyper = next(h for (_, _, r, h, _) in WORKLOADS.values() if r == rule)
        desc += f" [rule overridden: {rule}]"
    sizes = sizes_fn()
    n = len(sizes)
    params = sum(sizes)
    nstate = {"sgd": 1, "adam": 2, "rmsprop": 1, "adagrad": 1, "adadelta": 2, "nadam": 2}[rule]

    # ---- synthetic data, generated on the device ----
    w = [dev.alloc(4 * s) for s in sizes]
    g = [dev.alloc(4 * s) for s in sizes]
    # state buffers as the optimizers allocate them (memory.MemoryManager.AllocateStateBuffer): the j-th state of a
    # tensor starts at its own phase modulo 2 MiB, away from the weights' and gradients' 2 MiB-aligned starts
    states = [[dev.alloc(4 * s, zero=True, phase=state_phase(j, 4 * s)) for s in sizes] for j in range(nstate)]
    for k, s in enumerate(sizes):
        lib.gm_fill_normal_f32(D, w[k], s, 0x6D657461 + k, 0.0, 0.02)
        lib.gm_fill_normal_f32(D, g[k], s, 0x12345 + k, 0.0, grad_std)
    dev.synchronize()
    cw, cg = pkg.handle_array(w), pkg.handle_array(g)
    cs = [pkg.handle_array(s) for s in states]
    bs = pkg.int_array([4 * s for s in sizes])
    counter = {"t": 0}

    def launch_fp32():
        counter["t"] += 1
        t = counter["t"]
        h = hyper
        if rule == "adam":
            rc = lib.execute_adam_step_mpsgraph(D, cw, cg, cs[0], cs[1], n, bs, h["lr"], h["beta1"], h["beta2"],
                                                h["eps"], h["weight_decay"], t)
        elif rule == "nadam":
            rc = lib.execute_nadam_step_mpsgraph(D, cw, cg, cs[0], cs[1], n, bs, h["lr"], h["beta1"], h["beta2"],
                                                 h["eps"], h["weight_decay"], t)
        elif rule == "sgd":
            rc = lib.execute_sgd_step_mpsgraph(D, cw, cg, cs[0], n, bs, h["lr"], h["momentum"],
                                               h["weight_decay"], int(h["nesterov"]), t)
        elif rule == "rmsprop":
            rc = lib.execute_rmsprop_step_mpsgraph(D, cw, cg, cs[0], None, None, n, bs, h["lr"], h["alpha"],
                                                   h["eps"], h["weight_decay"], h["momentum"], False, t)
        elif rule == "adagrad":
            rc = lib.execute_adagrad_step_mpsgraph(D, cw, cg, cs[0], n, bs, h["lr"], h["eps"], h["weight_decay"])
        else:
            rc = lib.execute_adadelta_step_mpsgraph(D, cw, cg, cs[0], cs[1], n, bs, h["rho"], h["eps"],
                                                    h["weight_decay"])
        if rc != 0:
            raise RuntimeError(f"{rule} step failed rc={rc}: {lib.gm_last_error().decode()}")

    wall_ms, event_ms = time_steps(dev, launch_fp32, args.steps, args.warmup)
    median_ms, min_ms = per_launch_times(dev, launch_fp32, args.steps)
    bpp = BYTES_PER_PARAM[rule]
    achieved = params * bpp / (event_ms * 1e-3) / 1e9

    # ---- the same step over K independent copies of the list in turn: an HBM figure for lists that would
    # otherwise stay (partly) in the 256 MB memory-side cache from one step to the next ----
    rotated = None
    if args.rotate > 1:
        copies = [(cw, cg, cs)]
        for c in range(1, args.rotate):
            w2 = [dev.alloc(4 * s) for s in sizes]
            g2 = [dev.alloc(4 * s) for s in sizes]
            st2 = [[dev.alloc(4 * s, zero=True, phase=state_phase(j, 4 * s)) for s in sizes] for j in range(nstate)]
            for k, s in enumerate(sizes):
                lib.gm_fill_normal_f32(D, w2[k], s, 0x6D657461 + k + 7919 * c, 0.0, 0.02)
                lib.gm_fill_normal_f32(D, g2[k], s, 0x12345 + k + 7919 * c, 0.0, grad_std)
            copies.append((pkg.handle_array(w2), pkg.handle_array(g2), [pkg.handle_array(x) for x in st2]))
        dev.synchronize()
        turn = {"i": 0}

        def launch_rotating():
            nonlocal cw, cg, cs
            cw, cg, cs = copies[turn["i"] % len(copies)]
            turn["i"] += 1
            launch_fp32()

        rot_steps = -(-args.steps // len(copies)) * len(copies)       # every copy the same number of times
        rot_wall, rot_event = time_steps(dev, launch_rotating, rot_steps, max(args.warmup, len(copies)))
        cw, cg, cs = copies[0]
        rotated = {"copies": len(copies), "steps": rot_steps, "ms_per_step": rot_wall, "kernel_ms": rot_event,
                   "footprint_bytes": len(copies) * params * 4 * (2 + nstate)}

    # measured ceiling: plain 16-byte copy kernel over 1 GiB (an HBM figure whatever the workload's size), same run
    probe_bytes = 1 << 30
    src, dst = dev.alloc(probe_bytes), dev.alloc(probe_bytes)
    _, copy_ms = time_steps(dev, lambda: lib.gm_copy_probe(D, dst, src, probe_bytes), 10, 3)
    copy_gbs = 2 * probe_bytes / (copy_ms * 1e-3) / 1e9
    dev.free(src)
    dev.free(dst)

    result = {
        "metric": "params updated/sec (Adam fp32 multi-tensor step) + achieved HBM GB/s (% of peak)"
                  if rule == "adam" else f"params updated/sec ({rule} multi-tensor step) + achieved HBM GB/s",
        "value": params / (wall_ms * 1e-3),
        "unit": "params/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": desc, "tensors": n, "params": params, "rule": rule, "hyper": hyper,
                   "launch": {"chunk": args.chunk or "auto", "vec": args.vec or "auto", "lanes": args.lanes or "auto",
                              "nontemporal": args.nontemporal != 0}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, **traffic_fields((args.workload, rule)),
                     "kernel": f"multi_tensor_update_kernel<{rule}>", "bytes_per_param": bpp,
                     "kernel_ms": event_ms, "kernel_ms_median": median_ms, "kernel_ms_min": min_ms,
                     "copy_kernel_gbs": copy_gbs,
                     "frac_of_copy_kernel": achieved / copy_gbs},
    }
    result["config"]["state_placement"] = ("state buffers of more than 4 MiB start at phases of their own modulo 2 MiB, "
                                            "as the optimizers allocate them: " + ", ".join(str(p) for p in STATE_PHASES[:nstate]))
    footprint = params * 4 * (2 + nstate)            # every stream of the step, in bytes
    result["roofline"]["footprint_bytes"] = footprint
    if rotated:
        hbm = params * bpp / (rotated["kernel_ms"] * 1e-3) / 1e9
        result["roofline"].update({"frac_hbm": hbm / HBM_PEAK_GBS, "achieved_hbm": hbm, "rotated": rotated,
                                   "frac_of_copy_kernel": hbm / copy_gbs})
    if footprint < 256 * 1024 * 1024:
        result["roofline"]["note"] = (f"the step's {footprint / 1e6:.0f} MB stay in the 256 MB memory-side cache between "
                                      "steps and the kernel is a few microseconds of launch latency: 'achieved' counts "
                                      "algorithmic bytes per second, it is not an HBM figure for this workload")
    elif footprint < 1 << 30:
        result["roofline"]["note"] = (f"the step's {footprint / 1e6:.0f} MB are of the order of the 256 MB memory-side "
                                      "cache, which serves part of every step from what the step before left there: 'frac' "
                                      "is faster than HBM alone would allow; 'frac_hbm' (--rotate: independent copies of "
                                      "the list stepped in turn) is the HBM figure")

    # ---- mixed-precision Adam on the same list (fp16 gradients, fp16 weight copy) ----
    if rule == "adam" and not args.no_amp:
        g16 = [dev.alloc(2 * s) for s in sizes]
        w16 = [dev.alloc(2 * s) for s in sizes]
        for k, s in enumerate(sizes):
            lib.gm_fill_normal_f16(D, g16[k], s, 0x777 + k, 0.0, grad_std, 65536.0)
        dev.synchronize()
        cg16, cw16 = pkg.handle_array(g16), pkg.handle_array(w16)
        amp = lib.gm_amp_state_create(D, 65536.0, 2.0, 0.5, 2000)
        skipped, scale, tracker = ctypes.c_int(), ctypes.c_float(), ctypes.c_int()
        amp_t = {"t": 0, "skipped": 0}

        def launch_amp():
            rc = lib.execute_adam_amp_step(D, cw, cg16, cs[0], cs[1], cw16, n, bs, hyper["lr"], hyper["beta1"],
                                           hyper["beta2"], hyper["eps"], hyper["weight_decay"], amp_t["t"] + 1,
                                           amp, ctypes.byref(skipped), ctypes.byref(scale), ctypes.byref(tracker))
            if rc != 0:
                raise RuntimeError(f"mixed-precision step failed rc={rc}: {lib.gm_last_error().decode()}")
            if skipped.value:
                amp_t["skipped"] += 1
            else:
                amp_t["t"] += 1

        amp_wall, amp_event = time_steps(dev, launch_amp, args.steps, args.warmup)
        amp_achieved = params * BYTES_PER_PARAM["adam_amp"] / (amp_wall * 1e-3) / 1e9
        result["amp"] = {
            "value": params / (amp_wall * 1e-3), "unit": "params/s", "ms_per_step": amp_wall,
            "dtype": "f32 master state, f16 gradients and weight copy", "skipped_steps": amp_t["skipped"],
            "roofline": {"bound": "hbm", "achieved": amp_achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": amp_achieved / HBM_PEAK_GBS, "bytes_per_param": 28,
                         "bytes_per_param_moved": 30, **traffic_fields((args.workload, "adam_amp")),
                         "kernel": "amp_overflow_check_kernel + amp_adam_update_kernel",
                         "kernel_ms": amp_event,
                         "note": "step time covers the overflow-check launch and the update launch, whose first "
                                 "workgroup also advances the loss-scale state; each call returns once the host "
                                 "has seen the step's outcome"},
        }
        # the same step without the per-step read-back: the device keeps the step count
        lib.gm_amp_state_set_step_count(amp, amp_t["t"])

        def launch_amp_async():
            rc = lib.execute_adam_amp_step_async(D, cw, cg16, cs[0], cs[1], cw16, n, bs, hyper["lr"], hyper["beta1"],
                                                 hyper["beta2"], hyper["eps"], hyper["weight_decay"], amp)
            if rc != 0:
                raise RuntimeError(f"asynchronous mixed-precision step failed rc={rc}: {lib.gm_last_error().decode()}")

        async_wall, async_event = time_steps(dev, launch_amp_async, args.steps, args.warmup)
        async_achieved = params * BYTES_PER_PARAM["adam_amp"] / (async_event * 1e-3) / 1e9
        result["amp"]["async"] = {
            "value": params / (async_wall * 1e-3), "unit": "params/s", "ms_per_step": async_wall,
            "kernel_ms": async_event, "achieved": async_achieved, "frac": async_achieved / HBM_PEAK_GBS,
            "max_steps_in_flight": lib.gm_amp_state_max_in_flight(amp),
            "note": "execute_adam_amp_step_async: no host wait per step; HIP-event time per step over the timed steps",
        }
        lib.gm_amp_state_destroy(amp)

        # ---- the same step in one pass over ping-pong state (two sets of weights and moments) ----
        # the second set as EnablePingPong allocates it: weights 1 MiB off, moments at their counterparts' phases
        shadow = [[dev.alloc(4 * s, phase=ph if 4 * s > (4 << 20) else None) for s in sizes]
                  for ph in (1 << 20, STATE_PHASES[0], STATE_PHASES[1])]
        c_shadow = [pkg.handle_array(hs) for hs in shadow]
        amp2 = lib.gm_amp_state_create(D, 65536.0, 2.0, 0.5, 2000)
        lib.gm_amp_state_set_step_count(amp2, amp_t["t"])
        cur = ctypes.c_int()
        fused_t = {"t": amp_t["t"], "skipped": 0}

        def launch_fused():
            rc = lib.execute_adam_amp_step_fused(D, cw, cs[0], cs[1], c_shadow[0], c_shadow[1], c_shadow[2], cg16, cw16, n,
                                                 bs, hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"],
                                                 hyper["weight_decay"], fused_t["t"] + 1, amp2, ctypes.byref(skipped),
                                                 ctypes.byref(scale), ctypes.byref(tracker), ctypes.byref(cur))
            if rc != 0:
                raise RuntimeError(f"one-pass mixed-precision step failed rc={rc}: {lib.gm_last_error().decode()}")
            fused_t["skipped" if skipped.value else "t"] += 1

        def launch_fused_async():
            rc = lib.execute_adam_amp_step_fused_async(D, cw, cs[0], cs[1], c_shadow[0], c_shadow[1], c_shadow[2], cg16,
                                                       cw16, n, bs, hyper["lr"], hyper["beta1"], hyper["beta2"],
                                                       hyper["eps"], hyper["weight_decay"], amp2)
            if rc != 0:
                raise RuntimeError(f"one-pass asynchronous step failed rc={rc}: {lib.gm_last_error().decode()}")

        fused_wall, fused_event = time_steps(dev, launch_fused, args.steps, args.warmup)
        fa_wall, fa_event = time_steps(dev, launch_fused_async, args.steps, args.warmup)
        fused_achieved = params * 28 / (fused_wall * 1e-3) / 1e9
        fa_achieved = params * 28 / (fa_event * 1e-3) / 1e9
        result["amp"]["one_pass"] = {
            "entry_point": "execute_adam_amp_step_fused",
            "value": params / (fused_wall * 1e-3), "unit": "params/s", "ms_per_step": fused_wall,
            "skipped_steps": fused_t["skipped"],
            "roofline": {"bound": "hbm", "achieved": fused_achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": fused_achieved / HBM_PEAK_GBS, "bytes_per_param": 28, "bytes_per_param_moved": 28,
                         **traffic_fields((args.workload, "adam_amp_one_pass")),
                         "kernel": "amp_adam_fused_kernel + amp_finalize_repair_kernel",
                         "kernel_ms": fused_event,
                         "note": "weights and moments kept twice (ping-pong): the step reads the current set and "
                                 "writes the other, so a dropped step needs no second read of the gradients; each "
                                 "step is synchronous"},
            "async": {"value": params / (fa_wall * 1e-3), "unit": "params/s", "ms_per_step": fa_wall,
                      "kernel_ms": fa_event, "achieved": fa_achieved, "frac": fa_achieved / HBM_PEAK_GBS,
                      "max_steps_in_flight": lib.gm_amp_state_max_in_flight(amp2)},
        }
        lib.gm_amp_state_destroy(amp2)
        # StepAMP runs the in-place form unless the caller asked for ping-pong state (EnablePingPong): the in-place
        # form keeps the caller's own fp32 weight buffers current after every step, the one-pass form does not.
        in_place = result["amp"]
        one_pass = in_place.pop("one_pass")
        one_pass["dtype"] = in_place["dtype"]
        one_pass["form"] = ("one pass over ping-pong state: weights and moments kept twice (+12 B/param of HBM), "
                            "execute_adam_amp_step_fused / EnablePingPong")
        in_place["form"] = "in place: one set of state, the gradients read twice (execute_adam_amp_step, the default of StepAMP)"
        result["amp"] = {"default_form": "in_place", "in_place": in_place, "one_pass": one_pass}
        if not args.no_cpu_baseline and args.workload in ("c4", "c5"):
            result["amp"]["cpu_baseline"] = cpu_baseline_amp(sizes, hyper, grad_std, target_seconds=min(args.cpu_seconds, 3.0))

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(sizes, rule, hyper, grad_std, target_seconds=args.cpu_seconds)
    else:
        result["cpu_baseline"] = None

    if args.workload == "c4" and "amp" in result:
        # configuration 4 IS the mixed-precision step: the form StepAMP runs by default leads, the one-pass form and
        # the fp32 step over the same list follow
        amp_part = result.pop("amp")
        lead = amp_part[amp_part["default_form"]]
        fp32_part = {k: result[k] for k in ("value", "unit", "ms_per_step", "dtype", "roofline", "cpu_baseline")}
        result.update({"metric": "params updated/sec (mixed-precision Adam step, fp16 gradients and weight copy) + "
                                 "achieved HBM GB/s (% of peak)",
                       "value": lead["value"], "ms_per_step": lead["ms_per_step"], "dtype": lead["dtype"],
                       "roofline": lead["roofline"], "cpu_baseline": amp_part.get("cpu_baseline"),
                       "skipped_steps": lead["skipped_steps"], "async": lead["async"],
                       "form": lead["form"], "default_form": amp_part["default_form"],
                       "in_place": amp_part["in_place"], "one_pass": amp_part["one_pass"], "fp32_adam": fp32_part})

    dev.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()

"""Shared test harness: drives one update rule over a tensor list through the C ABI (GPU)
and through the CPU oracle, with the same call shape, so parity tests compare like with like."""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from __graft_entry__ import load_package  # noqa: E402
from oracle_lib import oracle  # noqa: E402

STATE_NAMES = {
    "sgd": ["m"], "adam": ["m", "v"], "rmsprop": ["s", "b", "ga"],
    "adagrad": ["s"], "adadelta": ["s", "a"], "nadam": ["m", "v"],
}


def states_for(rule, hyper):
    if rule == "sgd":
        return ["m"] if hyper["momentum"] > 0 else []
    if rule == "rmsprop":
        names = ["s"]
        if hyper["momentum"] > 0:
            names.append("b")
        if hyper["centered"]:
            names.append("ga")
        return names
    return STATE_NAMES[rule]


def progress(message):
    """A line for whoever watches a long GPU test from outside: pytest captures stdout, so the line also goes
    to a file the GPU job's output folder carries back (and that marks the job as alive)."""
    print(message, flush=True)
    try:
        folder = os.path.join(ROOT, "gpurun_out")
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "test_progress.log"), "a") as f:
            f.write(message + "\n")
    except OSError:
        pass


_GPU = None


def gpu_device():
    """The process-wide Device, or None when the library or a GPU is missing."""
    global _GPU
    if _GPU is None:
        try:
            _GPU = load_package().Device()
        except Exception as e:  # noqa: BLE001
            _GPU = e
    return None if isinstance(_GPU, Exception) else _GPU


def ulp_distance(a, b):
    """Units in the last place between two float32 arrays (finite values, same sign handling
    via the monotone integer mapping)."""
    def key(x):
        i = x.view(np.int32).astype(np.int64)
        return np.where(i < 0, np.int64(-2147483648) - i, i)
    return np.abs(key(np.ascontiguousarray(a)) - key(np.ascontiguousarray(b)))


class OracleRun:
    """A parameter list updated by the CPU oracle."""

    def __init__(self, rule, hyper, weights, nthreads=1):
        self.rule, self.h, self.nthreads = rule, hyper, nthreads
        self.w = [np.array(a, dtype=np.float32, copy=True) for a in weights]
        self.state = {k: [np.zeros(a.size, np.float32) for a in self.w] for k in states_for(rule, hyper)}
        self.step_count = 0

    def step(self, grads):
        o, h, r, nt = oracle(), self.h, self.rule, self.nthreads
        self.step_count += 1
        t = self.step_count
        for k, (w, g) in enumerate(zip(self.w, grads)):
            s = {name: arr[k] for name, arr in self.state.items()}
            if r == "sgd":
                o.sgd(w, g, s.get("m"), h["lr"], h["momentum"], h["weight_decay"], h["nesterov"], nt)
            elif r == "adam":
                o.adam(w, g, s["m"], s["v"], h["lr"], h["beta1"], h["beta2"], h["eps"], h["weight_decay"], t, nt)
            elif r == "rmsprop":
                o.rmsprop(w, g, s["s"], s.get("b"), s.get("ga"), h["lr"], h["alpha"], h["eps"],
                          h["weight_decay"], h["momentum"], h["centered"], nt)
            elif r == "adagrad":
                o.adagrad(w, g, s["s"], h["lr"], h["eps"], h["weight_decay"], nt)
            elif r == "adadelta":
                o.adadelta(w, g, s["s"], s["a"], h["rho"], h["eps"], h["weight_decay"], nt)
            elif r == "nadam":
                o.nadam(w, g, s["m"], s["v"], h["lr"], h["beta1"], h["beta2"], h["eps"], h["weight_decay"], t, nt)
            else:
                raise ValueError(r)

    def snapshot(self):
        out = {"w": self.w}
        out.update(self.state)
        return out


class GpuRun:
    """The same parameter list updated by libgometal_hip.so through the C ABI."""

    def __init__(self, dev, rule, hyper, weights):
        self.dev, self.rule, self.h = dev, rule, hyper
        self.pkg = load_package()
        self.sizes = [int(np.asarray(a).size) for a in weights]
        self.n = len(weights)
        self.w = [dev.from_numpy(np.asarray(a, dtype=np.float32)) for a in weights]
        self.state = {k: [dev.alloc(max(4 * n, 4), zero=True) for n in self.sizes]
                      for k in states_for(rule, hyper)}
        self.g = [dev.alloc(max(4 * n, 4)) for n in self.sizes]
        self.byte_sizes = self.pkg.int_array([4 * n for n in self.sizes])
        self.c_w = self.pkg.handle_array(self.w)
        self.c_g = self.pkg.handle_array(self.g)
        self.c_state = {k: self.pkg.handle_array(v) for k, v in self.state.items()}
        self.step_count = 0

    def upload_grads(self, grads):
        for h, g in zip(self.g, grads):
            if g.size:
                self.dev.upload(h, np.asarray(g, dtype=np.float32))

    def launch(self):
        """One step on the gradients currently in the device gradient buffers."""
        lib, h, r, d = self.dev.lib, self.h, self.rule, self.dev.handle
        self.step_count += 1
        t = self.step_count
        cs = self.c_state
        if r == "sgd":
            rc = lib.execute_sgd_step_mpsgraph(d, self.c_w, self.c_g, cs.get("m"), self.n, self.byte_sizes,
                                               h["lr"], h["momentum"], h["weight_decay"],
                                               int(bool(h["nesterov"])), t)
        elif r == "adam":
            rc = lib.execute_adam_step_mpsgraph(d, self.c_w, self.c_g, cs["m"], cs["v"], self.n,
                                                self.byte_sizes, h["lr"], h["beta1"], h["beta2"], h["eps"],
                                                h["weight_decay"], t)
        elif r == "rmsprop":
            rc = lib.execute_rmsprop_step_mpsgraph(d, self.c_w, self.c_g, cs["s"], cs.get("b"), cs.get("ga"),
                                                   self.n, self.byte_sizes, h["lr"], h["alpha"], h["eps"],
                                                   h["weight_decay"], h["momentum"], bool(h["centered"]), t)
        elif r == "adagrad":
            rc = lib.execute_adagrad_step_mpsgraph(d, self.c_w, self.c_g, cs["s"], self.n, self.byte_sizes,
                                                   h["lr"], h["eps"], h["weight_decay"])
        elif r == "adadelta":
            rc = lib.execute_adadelta_step_mpsgraph(d, self.c_w, self.c_g, cs["s"], cs["a"], self.n,
                                                    self.byte_sizes, h["rho"], h["eps"], h["weight_decay"])
        elif r == "nadam":
            rc = lib.execute_nadam_step_mpsgraph(d, self.c_w, self.c_g, cs["m"], cs["v"], self.n,
                                                 self.byte_sizes, h["lr"], h["beta1"], h["beta2"], h["eps"],
                                                 h["weight_decay"], t)
        else:
            raise ValueError(r)
        assert rc == 0, (r, rc, lib.gm_last_error())

    def step(self, grads):
        self.upload_grads(grads)
        self.launch()

    def snapshot(self):
        out = {"w": [self.dev.to_numpy(h, n) for h, n in zip(self.w, self.sizes)]}
        for k, handles in self.state.items():
            out[k] = [self.dev.to_numpy(h, n) for h, n in zip(handles, self.sizes)]
        return out

    def close(self):
        for h in self.w + self.g + [x for v in self.state.values() for x in v]:
            self.dev.free(h)


def compare_snapshots(got, want, max_ulp=0, context=""):
    """Asserts every array of two snapshots agrees to max_ulp; returns the worst distance seen."""
    worst = 0
    for name, arrays in want.items():
        for k, ref in enumerate(arrays):
            g = got[name][k]
            assert g.shape == ref.shape, (context, name, k, g.shape, ref.shape)
            if ref.size == 0:
                continue
            if np.array_equal(g.view(np.uint32), ref.view(np.uint32)):
                continue
            assert np.all(np.isfinite(g) == np.isfinite(ref)), (context, name, k, "finite mask")
            fin = np.isfinite(ref)
            d = int(ulp_distance(g[fin], ref[fin]).max()) if fin.any() else 0
            worst = max(worst, d)
            assert d <= max_ulp, f"{context} {name}[{k}]: {d} ulp > {max_ulp}"
    return worst


def amp_step_gpu(dev, pkg, handles, byte_sizes, n, hyper, step_count, amp_handle):
    """handles: dict of C arrays w, g16, m, v, w16.  Returns (skipped, scale, tracker)."""
    skipped, scale, tracker = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1)
    rc = dev.lib.execute_adam_amp_step(
        dev.handle, handles["w"], handles["g16"], handles["m"], handles["v"], handles["w16"], n,
        byte_sizes, hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"], hyper["weight_decay"],
        step_count, amp_handle, ctypes.byref(skipped), ctypes.byref(scale), ctypes.byref(tracker))
    assert rc == 0, (rc, dev.lib.gm_last_error())
    return skipped.value, scale.value, tracker.value

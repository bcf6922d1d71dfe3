"""The mixed-precision configurations at their stated size and length.

config 4: 125,000,000 parameters in 60 tensors, 5000 steps, fp16 gradients N(0, 1e-4) x the current loss
scale regenerated on the device for every step, +inf / -inf / NaN written into one random element on a
seeded 0.5 % of steps, loss scale 65536 with backoff x0.5 and growth x2 every 2000 clean steps.
config 5 (mixed-precision variant): 1,012,301,824 parameters in 400 tensors, weight decay 1e-4, 20 steps.

A third schedule (growth every 100 clean steps, an injection on about 1 % of 1000 steps) makes the scale move up
and down at full size with gradients that never underflow.

Every step's (skipped, scale, clean-step counter, step count) must equal the CPU oracle's, and weights,
moments and the fp16 weight copy are compared bit for bit at checkpoints (every 500 steps / steps 1, 10, 20).
The oracle consumes the very gradients the device generated (read back once per step) and runs in a worker
thread one step behind the GPU, so the run takes about as long as the oracle alone.  Both forms of the step (in
place, and in one pass over ping-pong state) run every schedule side by side, each on device state of its own, over
the same gradients and against the one oracle run: a step computes the same thing in either form."""
import ctypes
import os
import queue
import threading
import time

import numpy as np
import pytest

from harness import gpu_device, progress
from oracle_lib import oracle
from workloads import amp_125m_sizes, transformer_block_sizes
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
NTHREADS = min(16, os.cpu_count() or 1)


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


class DeviceForm:
    """One form of the step with device state of its own: "in_place" (execute_adam_amp_step over one set of
    weights and moments) or "one_pass" (execute_adam_amp_step_fused over ping-pong state: two sets on the device,
    the fp16 copy kept as half of the current weights from the start)."""

    def __init__(self, dev, pkg, form, sizes, offsets, w_host, w16_from_weights, loss_scale):
        self.dev, self.pkg, self.lib, self.D = dev, pkg, dev.lib, dev.handle
        self.form, self.sizes, self.offsets = form, sizes, offsets
        total = int(offsets[-1])
        arr = pkg.handle_array
        self.d_w = [dev.from_numpy(a) for a in w_host]
        self.d_m = [dev.alloc(4 * s, zero=True) for s in sizes]
        self.d_v = [dev.alloc(4 * s, zero=True) for s in sizes]
        self.d_w16 = dev.alloc(2 * total, zero=True)
        self.c_w, self.c_m, self.c_v = arr(self.d_w), arr(self.d_m), arr(self.d_v)
        self.c_w16 = arr([self.d_w16 + 2 * int(off) for off in offsets[:-1]])
        self.shadow = []
        if form == "one_pass":
            self.shadow = [[dev.alloc(4 * s) for s in sizes] for _ in range(3)]
            self.c_shadow = [arr(hs) for hs in self.shadow]
        if w16_from_weights:
            for k in range(len(sizes)):
                assert self.lib.convert_tensor_type(self.d_w[k], self.d_w16 + 2 * int(offsets[k]),
                                                    pkg.int_array([sizes[k]]), 1, 0, 2, self.D) == 0
        self.bs = pkg.int_array([4 * s for s in sizes])
        self.amp = self.lib.gm_amp_state_create(self.D, *loss_scale)
        assert self.amp
        self.current, self.applied, self.trace = 0, 0, []

    def step(self, k, c_g16, hyper):
        lib, n = self.lib, len(self.sizes)
        skipped, sc, tracker = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1)
        if self.form == "one_pass":
            cur = ctypes.c_int(-1)
            rc = lib.execute_adam_amp_step_fused(self.D, self.c_w, self.c_m, self.c_v, self.c_shadow[0], self.c_shadow[1],
                                                 self.c_shadow[2], c_g16, self.c_w16, n, self.bs, hyper["lr"],
                                                 hyper["beta1"], hyper["beta2"], hyper["eps"], hyper["weight_decay"],
                                                 self.applied + 1, self.amp, ctypes.byref(skipped), ctypes.byref(sc),
                                                 ctypes.byref(tracker), ctypes.byref(cur))
            self.current ^= 0 if skipped.value else 1
            assert cur.value == self.current, (k, cur.value, self.current)
        else:
            rc = lib.execute_adam_amp_step(self.D, self.c_w, c_g16, self.c_m, self.c_v, self.c_w16, n, self.bs,
                                           hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"],
                                           hyper["weight_decay"], self.applied + 1, self.amp, ctypes.byref(skipped),
                                           ctypes.byref(sc), ctypes.byref(tracker))
        assert rc == 0, (self.form, rc, lib.gm_last_error())
        self.applied += 0 if skipped.value else 1
        self.trace.append((skipped.value, sc.value, tracker.value, self.applied))
        return sc.value

    def compare(self, context, w_host, m_host, v_host, w16_host):
        dev, n = self.dev, len(self.sizes)
        now = (self.d_w, self.d_m, self.d_v) if self.current == 0 else tuple(self.shadow)
        for name_, dh, host in (("w", now[0], w_host), ("m", now[1], m_host), ("v", now[2], v_host)):
            for k in range(n):
                got = dev.to_numpy(dh[k], self.sizes[k])
                assert np.array_equal(got.view(np.uint32), host[k].view(np.uint32)), (context, self.form, name_, k)
        got16 = dev.to_numpy(self.d_w16, int(self.offsets[-1]), np.uint16)
        for k in range(n):
            assert np.array_equal(got16[self.offsets[k]:self.offsets[k + 1]], w16_host[k]), (context, self.form, "w16", k)

    def free(self):
        self.lib.gm_amp_state_destroy(self.amp)
        for h in self.d_w + self.d_m + self.d_v + [self.d_w16] + [x for hs in self.shadow for x in hs]:
            self.dev.free(h)


def run_schedule(dev, name, sizes, hyper, steps, inject_at, checkpoints, seed, forms=("in_place", "one_pass"),
                 loss_scale=(65536.0, 2.0, 0.5, 2000)):
    """Runs every form in `forms` over the same per-step gradients, each on device state of its own, against one run
    of the oracle (the forms differ in how the device gets there, not in what a step computes), and returns the
    per-step trace they all share.  loss_scale: (initial scale, growth factor, backoff factor, growth interval).
    inject_at: {step index: (tensor, element, fp16 bits)}; checkpoints: step indices (0-based) after which all
    buffers of every form are compared."""
    pkg, lib, D, o = load_package(), dev.lib, dev.handle, oracle()
    n, total = len(sizes), sum(sizes)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    rng = np.random.default_rng(seed)
    w_host = [rng.standard_normal(s, dtype=np.float32) * np.float32(0.02) for s in sizes]
    # the one-pass step needs fp16 copy = half(weights) from the start; the in-place step does not care, so when both
    # run they start from that, and the in-place step alone starts from a zeroed copy
    w16_from_weights = "one_pass" in forms
    d_g16 = dev.alloc(2 * total)
    c_g16 = pkg.handle_array([d_g16 + 2 * int(off) for off in offsets[:-1]])
    device_forms = []

    # ---- oracle side
    m_host = [np.zeros(s, np.float32) for s in sizes]
    v_host = [np.zeros(s, np.float32) for s in sizes]
    w16_host = [a.astype(np.float16).view(np.uint16) if w16_from_weights else np.zeros(s, np.uint16)
                for a, s in zip(w_host, sizes)]
    st = o.amp_state(*loss_scale)
    g_buffers = [np.empty((2 * total + 3) // 4, np.uint32) for _ in range(2)]
    free_buffers, work = queue.Queue(), queue.Queue(maxsize=1)
    for b in range(2):
        free_buffers.put(b)
    oracle_trace, failure = [], []

    def oracle_worker():
        try:
            while True:
                item = work.get()
                if item is None:
                    return
                b = item
                g = g_buffers[b].view(np.uint16)
                g16 = [g[offsets[k]:offsets[k + 1]] for k in range(n)]
                skipped = o.adam_amp(w_host, g16, m_host, v_host, w16_host, state=st, nthreads=NTHREADS, **hyper)
                oracle_trace.append((skipped, float(np.float32(st.scale)), st.growth_tracker, int(st.step_count)))
                free_buffers.put(b)
        except Exception as e:  # noqa: BLE001
            failure.append(e)
            free_buffers.put(-1)

    worker = threading.Thread(target=oracle_worker, daemon=True)
    worker.start()

    def drain():
        """Waits until the oracle has applied every step handed to it."""
        held = [free_buffers.get(), free_buffers.get()]
        assert not failure, failure
        for b in held:
            free_buffers.put(b)

    def first_difference(got):
        return next((i, a, b_) for i, (a, b_) in enumerate(zip(got, oracle_trace)) if a != b_)

    scale = loss_scale[0]
    t0 = time.time()
    try:
        for form in forms:
            device_forms.append(DeviceForm(dev, pkg, form, sizes, offsets, w_host, w16_from_weights, loss_scale))
        for k in range(steps):
            # this step's gradients at the current loss scale, made on the device
            assert lib.gm_fill_normal_f16(D, d_g16, total, 0xC4000000 + 7919 * k + seed, 0.0, 1e-4, scale) == 0
            if k in inject_at:
                t, e, bits = inject_at[k]
                tmp = dev.from_numpy(np.array([bits, 0], np.uint16))
                assert lib.copy_buffer_to_buffer_sync(tmp, d_g16, 0, 2 * (int(offsets[t]) + e), 2) == 0
                dev.free(tmp)
            b = free_buffers.get()
            assert b >= 0 and not failure, failure
            words = g_buffers[b].size
            assert lib.copy_metal_buffer_to_int32_array(d_g16, g_buffers[b].ctypes.data_as(ctypes.c_void_p), words) == 0
            scales = [f.step(k, c_g16, hyper) for f in device_forms]
            assert len(set(scales)) == 1, (k, scales)
            scale = scales[0]
            work.put(b)
            if k % 50 == 0:
                progress(f"{name}: step {k + 1} of {steps}, scale {scale}, {time.time() - t0:.0f} s")
            if k in checkpoints:
                drain()
                for f in device_forms:
                    f.compare(f"{name} after step {k + 1}", w_host, m_host, v_host, w16_host)
                    assert f.trace == oracle_trace, (f.form, first_difference(f.trace))
        drain()
        assert len(oracle_trace) == steps
        for f in device_forms:
            assert f.trace == oracle_trace, (f.form, first_difference(f.trace))
        want_skips = sorted(inject_at)
        assert [i for i, t in enumerate(oracle_trace) if t[0]] == want_skips
        return list(oracle_trace)
    finally:
        work.put(None)
        worker.join(timeout=60)
        for f in device_forms:
            f.free()
        dev.free(d_g16)


def config4_injections(sizes):
    rng = np.random.default_rng(0x6D657461 + 4)
    chosen = np.flatnonzero(rng.random(5000) < 0.005)
    inject = {}
    for j, k in enumerate(chosen):
        t = int(rng.integers(0, len(sizes)))
        inject[int(k)] = (t, int(rng.integers(0, sizes[t])), [0x7C00, 0xFC00, 0x7E00][j % 3])
    assert len(inject) > 10
    return inject


def test_config4_full_size_5000_steps(dev):
    """The in-place step and the one-pass ping-pong step, both over the full 5000-step schedule at full size."""
    sizes = amp_125m_sizes()
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)
    inject = config4_injections(sizes)
    trace = run_schedule(dev, "config 4", sizes, hyper, 5000, inject, {499 + 500 * i for i in range(10)}, seed=4)
    # In this schedule the scale only ever drops: a growth needs 2000 clean steps in a row, and with an injection
    # on 0.5 % of steps that happens with probability 4e-5.  The scale ends at 65536 / 2^len(inject), and from
    # about step 3500 on half(N(0, 1e-4) x scale) underflows to zero.  Growth, and gradients that stay alive to the
    # end, are what test_full_size_growth_and_backoff below is for.
    scales = [t[1] for t in trace]
    assert all(b <= a for a, b in zip(scales, scales[1:])) and scales[-1] == 65536.0 / 2.0 ** len(inject)
    assert trace[-1][3] == 5000 - len(inject)


def growth_schedule(steps, sizes, seed, rate=0.01):
    """Injections on a seeded `rate` of the steps, and the loss-scale trajectory they produce from 65536 with growth
    x2 every 100 clean steps and backoff x0.5, computed here by a plain state machine: (inject, scales, growths,
    backoffs)."""
    rng = np.random.default_rng(seed)
    chosen = np.flatnonzero(rng.random(steps) < rate)
    inject = {}
    for j, k in enumerate(chosen):
        t = int(rng.integers(0, len(sizes)))
        inject[int(k)] = (t, int(rng.integers(0, sizes[t])), [0x7C00, 0xFC00, 0x7E00][j % 3])
    scale, tracker, scales, growths, backoffs = 65536.0, 0, [], 0, 0
    for k in range(steps):
        if k in inject:
            scale, tracker, backoffs = scale * 0.5, 0, backoffs + 1
        else:
            tracker += 1
            if tracker == 100:
                scale, tracker, growths = scale * 2.0, 0, growths + 1
        scales.append(scale)
    return inject, scales, growths, backoffs


def test_full_size_growth_and_backoff(dev):
    """125,000,000 parameters in 60 tensors, 1000 steps, growth every 100 clean steps, an inf / NaN on about 1 % of
    steps: the scale goes up and down several times and stays between 2^10 and 2^20, so the fp16 gradients
    N(0, 1e-4) x scale never underflow and every applied step is a real update to the end of the run.  Every
    step's (skipped, scale, clean-step counter, step count) and, at three checkpoints, every buffer equal the
    oracle's, for the in-place step and for the one-pass step over ping-pong state."""
    sizes = amp_125m_sizes()
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)
    inject, scales, growths, backoffs = growth_schedule(1000, sizes, seed=0x6D657461 + 45)
    assert growths >= 3 and backoffs >= 3 and 2.0 ** 10 <= min(scales) and max(scales) <= 2.0 ** 20, (growths, backoffs, min(scales), max(scales))
    trace = run_schedule(dev, "growth and backoff", sizes, hyper, 1000, inject, {332, 665, 999}, seed=44,
                         loss_scale=(65536.0, 2.0, 0.5, 100))
    got = [t[1] for t in trace]
    assert got == scales
    ups = sum(1 for a, b in zip(got, got[1:]) if b > a)
    downs = sum(1 for a, b in zip(got, got[1:]) if b < a)
    assert ups >= 3 and downs >= 3 and min(got) >= 2.0 ** 10 and max(got) <= 2.0 ** 20
    assert trace[-1][3] == 1000 - len(inject)


def test_config5_mixed_precision_full_size_20_steps(dev):
    """1,012,301,824 parameters, both forms; the very first step is dropped, so the one-pass step's repair of the
    fp16 copy runs before any step has been applied."""
    sizes = transformer_block_sizes()
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    inject = {0: (7, 5, 0x7C00), 6: (len(sizes) - 3, 1234, 0xFC00), 13: (2, 4096 * 11008 - 1, 0x7E00)}
    trace = run_schedule(dev, "config 5 mixed precision", sizes, hyper, 20, inject, {0, 1, 9, 19}, seed=5)
    assert [t[0] for t in trace].count(1) == 3 and trace[-1][1] == 8192.0 and trace[-1][3] == 17


def test_a_tensor_of_the_largest_size_the_abi_can_name(dev):
    """2^29 - 1 elements (2^31 - 4 bytes of fp32, the largest C int in bytes that is a whole number of floats) next to
    a three-element tensor and a 2^28-element one, both forms, three steps; the middle step is dropped for a NaN in
    the large tensor's last element."""
    sizes = [2 ** 29 - 1, 3, 2 ** 28]
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    trace = run_schedule(dev, "largest tensor", sizes, hyper, 3, {1: (0, sizes[0] - 1, 0x7E00)}, {0, 1, 2}, seed=6)
    assert [t[0] for t in trace] == [0, 1, 0] and trace[-1][1] == 32768.0 and trace[-1][3] == 2

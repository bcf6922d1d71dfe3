"""Mixed-precision Adam on the GPU against the CPU oracle: the skip / loss-scale sequence must be
bit-exact over the whole run; weights, moments and the fp16 weight copy are held to 0 ulp."""
import ctypes
import json
import os

import numpy as np
import pytest

from harness import amp_step_gpu, gpu_device
from oracle_lib import oracle
from workloads import amp_125m_sizes
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "optimizer_kat.json")) as f:
    KAT = json.load(f)
NTHREADS = min(16, os.cpu_count() or 1)
HYPER = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


class AmpPair:
    """The same tensor list on the GPU (C ABI) and in the oracle."""

    def __init__(self, dev, weights, hyper, amp_cfg=(65536.0, 2.0, 0.5, 2000), nthreads=1):
        self.dev, self.pkg, self.h, self.nthreads = dev, load_package(), hyper, nthreads
        self.sizes = [w.size for w in weights]
        self.n = len(weights)
        self.w = [np.array(w, np.float32, copy=True) for w in weights]
        self.m = [np.zeros(s, np.float32) for s in self.sizes]
        self.v = [np.zeros(s, np.float32) for s in self.sizes]
        self.w16 = [np.zeros(s, np.uint16) for s in self.sizes]
        self.st = oracle().amp_state(*amp_cfg)
        self.d = {"w": [dev.from_numpy(w) for w in self.w],
                  "m": [dev.alloc(4 * s, zero=True) for s in self.sizes],
                  "v": [dev.alloc(4 * s, zero=True) for s in self.sizes],
                  "w16": [dev.alloc(2 * s, zero=True) for s in self.sizes],
                  "g16": [dev.alloc(2 * s) for s in self.sizes]}
        self.c = {k: self.pkg.handle_array(v) for k, v in self.d.items()}
        self.bs = self.pkg.int_array([4 * s for s in self.sizes])
        self.amp = dev.lib.gm_amp_state_create(dev.handle, *amp_cfg)
        assert self.amp
        self.gpu_steps = 0

    def step(self, g16, upload=True):
        if upload:
            for h, g in zip(self.d["g16"], g16):
                self.dev.upload(h, g)
        got = amp_step_gpu(self.dev, self.pkg, self.c, self.bs, self.n, self.h, self.gpu_steps + 1, self.amp)
        if not got[0]:
            self.gpu_steps += 1
        want_skipped = oracle().adam_amp(self.w, g16, self.m, self.v, self.w16, state=self.st,
                                         nthreads=self.nthreads, **self.h)
        want = (want_skipped, float(np.float32(self.st.scale)), self.st.growth_tracker)
        assert got == want, (got, want)
        assert self.gpu_steps == self.st.step_count
        return got[0]

    def compare(self, context=""):
        for name, host, dtype in (("w", self.w, np.float32), ("m", self.m, np.float32), ("v", self.v, np.float32),
                                  ("w16", self.w16, np.uint16)):
            for k, ref in enumerate(host):
                got = self.dev.to_numpy(self.d[name][k], ref.size, dtype)
                assert np.array_equal(got.view(np.uint8), ref.view(np.uint8)), (context, name, k)

    def close(self):
        self.dev.lib.gm_amp_state_destroy(self.amp)
        for v in self.d.values():
            for h in v:
                self.dev.free(h)


@pytest.mark.parametrize("case", KAT["amp_cases"], ids=[c["name"] for c in KAT["amp_cases"]])
def test_amp_golden_vectors(dev, case):
    h, a = case["hyper"], case["amp"]
    w0 = [np.array(t, np.uint32).view(np.float32) for t in case["w0"]]
    pair = AmpPair(dev, w0, h, (a["init_scale"], a["growth_factor"], a["backoff_factor"], a["growth_interval"]))
    try:
        for k, step in enumerate(case["g16"]):
            skipped = pair.step([np.array(t, np.uint16) for t in step])
            exp = case["expect"][k]
            assert skipped == exp["skipped"]
            for ti in range(pair.n):
                assert dev.to_numpy(pair.d["w"][ti], pair.sizes[ti]).view(np.uint32).tolist() == exp["w"][ti]
                assert dev.to_numpy(pair.d["w16"][ti], pair.sizes[ti], np.uint16).tolist() == exp["w16"][ti]
    finally:
        pair.close()


def test_config4_skip_and_scale_sequence_5000_steps(dev):
    """The 5000-step schedule of config 4 (60 tensors, loss scale 65536, backoff x0.5, growth x2
    every 2000 clean steps, +-inf / NaN injected into one random element on a seeded 0.5 % of steps)
    with every tensor at 1/1000 of its size, so the oracle keeps pace: every step's
    (skipped, scale, clean-step counter, step count) must equal the oracle's, and p / m / v / fp16
    copy are compared bit for bit every 500 steps."""
    rng = np.random.default_rng(0x6D657461 + 4)
    sizes = [max(1, s // 1000) for s in amp_125m_sizes()]
    w = [rng.normal(0, 0.02, s).astype(np.float32) for s in sizes]
    pool = [[rng.normal(0, 1e-4, s).astype(np.float32) for s in sizes] for _ in range(8)]
    inject = rng.random(5000) < 0.005
    pair = AmpPair(dev, w, HYPER)
    skipped_total = 0
    try:
        for k in range(5000):
            scale = np.float32(pair.st.scale)
            g16 = [(g * scale).astype(np.float16).view(np.uint16) for g in pool[k % len(pool)]]
            if inject[k]:
                t = int(rng.integers(0, len(sizes)))
                g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][skipped_total % 3]
            skipped_total += pair.step(g16)
            if (k + 1) % 500 == 0:
                pair.compare(f"step {k + 1}")
        assert skipped_total == int(inject.sum()) and skipped_total > 10
        assert pair.st.step_count == 5000 - skipped_total
    finally:
        pair.close()


def device_normal_f16(dev, sizes, seed, std, scale):
    """fp16 gradient tensors generated on the device; returns (handles, host copies)."""
    handles, host = [], []
    for k, s in enumerate(sizes):
        h = dev.alloc(2 * s)
        assert dev.lib.gm_fill_normal_f16(dev.handle, h, s, seed + k, 0.0, std, scale) == 0
        handles.append(h)
        host.append(dev.to_numpy(h, s, np.uint16))
    return handles, host


def poke_half(dev, handle, index, bits):
    """Overwrites one fp16 element of a device buffer (2-byte device-to-device copy)."""
    tmp = dev.from_numpy(np.array([bits, 0], np.uint16))
    assert dev.lib.copy_buffer_to_buffer_sync(tmp, handle, 0, 2 * index, 2) == 0
    dev.free(tmp)


@pytest.mark.parametrize("name,sizes_fn,weight_decay", [
    ("config4_125m", amp_125m_sizes, 0.0),
])
def test_amp_full_size(dev, name, sizes_fn, weight_decay):
    """The 125M-parameter list in a few steps (the whole 5000-step schedule and the 1.012B-parameter list
    are in tests/test_gpu_amp_full.py): clean step, a step with an injected -inf (every buffer must stay
    byte-identical), a step with a NaN, two clean steps; then p / m / v / fp16 copy against the oracle,
    bit for bit."""
    sizes = sizes_fn()
    hyper = dict(HYPER, weight_decay=weight_decay)
    rng = np.random.default_rng(17)
    w = [rng.standard_normal(s, dtype=np.float32) * np.float32(0.02) for s in sizes]
    pair = AmpPair(dev, w, hyper, nthreads=NTHREADS)
    for h in pair.d["g16"]:
        dev.free(h)
    g_handles, g_host = device_normal_f16(dev, sizes, 0xABC, 1e-4, 65536.0)
    pair.d["g16"] = g_handles
    pair.c["g16"] = pair.pkg.handle_array(g_handles)
    try:
        assert pair.step(g_host, upload=False) == 0
        victim = len(sizes) - 3
        clean = int(g_host[victim][12345 % sizes[victim]])
        for bits in (0xFC00, 0x7E00):
            poke_half(dev, g_handles[victim], 12345 % sizes[victim], bits)
            g_host[victim][12345 % sizes[victim]] = bits
            assert pair.step(g_host, upload=False) == 1
        pair.compare("after skipped steps")          # includes: nothing moved since the clean step
        poke_half(dev, g_handles[victim], 12345 % sizes[victim], clean)
        g_host[victim][12345 % sizes[victim]] = clean
        assert pair.step(g_host, upload=False) == 0
        assert pair.step(g_host, upload=False) == 0
        assert float(np.float32(pair.st.scale)) == 16384.0 and pair.st.step_count == 3
        pair.compare("final")
    finally:
        pair.close()


def test_async_steps_equal_the_synchronous_sequence(dev):
    """execute_adam_amp_step_async in bursts the host does not wait for: the device picks the bias
    corrections by its own applied-step count.  After every burst the counters, and every few bursts
    all buffers, must equal the oracle's (which is what the synchronous step is held to)."""
    pkg = load_package()
    lib, D = dev.lib, dev.handle
    rng = np.random.default_rng(0xA51)
    sizes = [3_000_000, 4096, 2_000_000, 77, 1_500_000]
    n, burst, bursts = len(sizes), 12, 24
    amp_cfg = (1024.0, 2.0, 0.5, 7)                      # short growth interval: the scale moves often
    w = [rng.normal(0, 0.02, s).astype(np.float32) for s in sizes]
    pair = AmpPair(dev, w, dict(HYPER, weight_decay=1e-4), amp_cfg, nthreads=NTHREADS)
    grads = [[rng.normal(0, 1e-3, s).astype(np.float32) for s in sizes] for _ in range(3)]
    # one set of device gradient buffers per step of a burst, so that nothing is uploaded between steps
    g16_dev = [[dev.alloc(2 * s) for s in sizes] for _ in range(burst)]
    g16_arr = [pkg.handle_array(hs) for hs in g16_dev]
    h = pair.h
    assert lib.gm_amp_state_set_step_count(pair.amp, 0) == 0
    try:
        skipped_total = 0
        for b in range(bursts):
            # the oracle runs the burst first: it fixes the scale each step's gradients are made with
            for j in range(burst):
                scale = np.float32(pair.st.scale)
                g16 = [(g * scale).astype(np.float16).view(np.uint16) for g in grads[(b + j) % 3]]
                if rng.random() < 0.12:
                    t = int(rng.integers(0, n))
                    g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][(b + j) % 3]
                for hd, g in zip(g16_dev[j], g16):
                    dev.upload(hd, g)
                skipped_total += oracle().adam_amp(pair.w, g16, pair.m, pair.v, pair.w16, state=pair.st,
                                                   nthreads=NTHREADS, **h)
            print(f"burst {b}: issuing {burst} steps", flush=True)
            for j in range(burst):
                rc = lib.execute_adam_amp_step_async(D, pair.c["w"], g16_arr[j], pair.c["m"], pair.c["v"],
                                                     pair.c["w16"], n, pair.bs, h["lr"], h["beta1"], h["beta2"],
                                                     h["eps"], h["weight_decay"], pair.amp)
                assert rc == 0, (rc, lib.gm_last_error())
            scale, tracker, applied, skipped = ctypes.c_float(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            assert lib.gm_amp_state_query(pair.amp, ctypes.byref(scale), ctypes.byref(tracker),
                                          ctypes.byref(applied), ctypes.byref(skipped)) == 0
            assert (scale.value, tracker.value, applied.value, skipped.value) == \
                (float(np.float32(pair.st.scale)), pair.st.growth_tracker, pair.st.step_count, skipped_total), b
            if b % 6 == 5 or b == bursts - 1:
                pair.compare(f"burst {b}")
        assert 10 < skipped_total < burst * bursts - 50
        # the host did run ahead: without it the bias table is never more than one entry long
        assert lib.gm_amp_state_max_in_flight(pair.amp) >= 2
        # a synchronous step continues from the same counters
        scale = np.float32(pair.st.scale)
        g16 = [(g * scale).astype(np.float16).view(np.uint16) for g in grads[0]]
        pair.gpu_steps = pair.st.step_count
        assert pair.step(g16) == 0
        pair.compare("synchronous step after the bursts")
    finally:
        pair.close()
        for hs in g16_dev:
            for hd in hs:
                dev.free(hd)


@pytest.mark.parametrize("vec,lanes", [(2, 0), (4, 0), (1, 128), (2, 128), (4, 128)])
def test_amp_launch_shape_variants_are_bit_identical(dev, vec, lanes):
    """The mixed-precision step in every selectable lane width and workgroup size, over ragged sizes with an
    overflow step in the middle: the same bits and the same skip / scale sequence as the oracle."""
    lib = dev.lib
    rng = np.random.default_rng(17)
    sizes = [1, 2, 3, 7, 255, 257, 1023, 4097, 70001]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    assert lib.gm_set_tuning(dev.handle, 0, -1, vec) == 0
    assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
    try:
        pair = AmpPair(dev, w, dict(HYPER, weight_decay=1e-4), (1024.0, 2.0, 0.5, 3))
        try:
            for t in range(6):
                g16 = [(rng.normal(0, 1e-3, n) * 1024.0).astype(np.float16).view(np.uint16) for n in sizes]
                if t == 2:
                    g16[5][100] = 0x7C00          # +inf in one element of one tensor: the step is dropped
                assert pair.step(g16) == (t == 2)
                pair.compare(f"vec={vec} lanes={lanes} step={t}")
        finally:
            pair.close()
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0


def test_amp_over_many_tiny_tensors(dev):
    """400 tensors of 1 to 700 elements: 256-element chunks, so the overflow check runs one small workgroup per
    chunk; an inf in the last element of the last tensor must still drop the whole step."""
    rng = np.random.default_rng(43)
    sizes = [int(x) for x in rng.integers(1, 701, 400)]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    pair = AmpPair(dev, w, HYPER, (4096.0, 2.0, 0.5, 2))
    try:
        for t in range(5):
            g16 = [(rng.normal(0, 1e-3, n) * 4096.0).astype(np.float16).view(np.uint16) for n in sizes]
            if t == 1:
                g16[-1][-1] = 0xFC00          # -inf
            assert pair.step(g16) == (t == 1)
        pair.compare("tiny tensors")
    finally:
        pair.close()


@pytest.mark.parametrize("misalign", [0, 1])
def test_overflow_anywhere_in_a_list_of_few_large_chunks_is_seen(dev, misalign):
    """One tensor of a million elements is cut into sixteen 65536-element chunks, and the in-place step's check then
    runs several workgroups per chunk, each over a run of 2048-element rows: an inf / NaN at the first and last
    element of the tensor, of a chunk, of a row, in the ragged tail and at random places must each drop the step
    (and a clean step in between must not).  misalign: the gradient view starts 2 bytes off, which takes the
    element-by-element path."""
    lib, pkg = dev.lib, load_package()
    n = (1 << 20) + 77
    rng = np.random.default_rng(91 + misalign)
    w = rng.normal(0, 0.02, n).astype(np.float32)
    bufs = {"w": dev.from_numpy(w), "m": dev.alloc(4 * n, zero=True), "v": dev.alloc(4 * n, zero=True),
            "w16": dev.alloc(2 * n, zero=True)}
    g_parent = dev.alloc(2 * n + 16)
    g_view = g_parent + 2 * misalign
    c = {k: pkg.handle_array([h]) for k, h in bufs.items()}
    c["g16"] = pkg.handle_array([g_view])
    bs = pkg.int_array([4 * n])
    amp = lib.gm_amp_state_create(dev.handle, 1024.0, 2.0, 0.5, 1000)
    clean = (rng.normal(0, 1e-3, n) * 1024.0).astype(np.float16).view(np.uint16)
    places = [0, 1, 2047, 2048, 65535, 65536, 65536 + 2047, 15 * 65536, (1 << 20) - 1, 1 << 20, n - 9, n - 1]
    places += [int(x) for x in rng.integers(0, n, 12)]
    try:
        applied = 0
        for k, place in enumerate(places):
            g = clean.copy()
            g[place] = [0x7C00, 0xFC00, 0x7E01][k % 3]
            padded = np.zeros(n + 8, np.uint16)
            padded[misalign:misalign + n] = g
            dev.upload(g_parent, padded)
            got = amp_step_gpu(dev, pkg, c, bs, 1, HYPER, applied + 1, amp)
            assert got[0] == 1, (place, got)
            if k % 4 == 0:                               # a clean step between dropped ones
                padded[misalign:misalign + n] = clean
                dev.upload(g_parent, padded)
                got = amp_step_gpu(dev, pkg, c, bs, 1, HYPER, applied + 1, amp)
                assert got[0] == 0, (place, got)
                applied += 1
        assert np.array_equal(dev.to_numpy(bufs["w"], n) != w, np.ones(n, bool)) or applied > 0
    finally:
        lib.gm_amp_state_destroy(amp)
        for h in list(bufs.values()) + [g_parent]:
            dev.free(h)


def test_a_list_without_elements_still_advances_the_loss_scale_state(dev):
    """Every tensor empty: there is no check or update launch to carry the epilogue, yet each step counts as
    applied (no gradient overflowed), the clean-step counter runs and the scale grows at the interval, with and
    without the host waiting for the step."""
    lib, pkg = dev.lib, load_package()
    bufs = {k: [dev.alloc(16, zero=True) for _ in range(2)] for k in ("w", "g16", "m", "v", "w16")}
    c = {k: pkg.handle_array(v) for k, v in bufs.items()}
    bs = pkg.int_array([0, 0])
    amp = lib.gm_amp_state_create(dev.handle, 1024.0, 2.0, 0.5, 3)
    st = oracle().amp_state(1024.0, 2.0, 0.5, 3)
    none = [np.zeros(0, np.float32)] * 2
    none16 = [np.zeros(0, np.uint16)] * 2
    try:
        for t in range(4):
            got = amp_step_gpu(dev, pkg, c, bs, 2, HYPER, t + 1, amp)
            want = oracle().adam_amp(none, none16, none, none, none16, state=st, **HYPER)
            assert got == (want, float(np.float32(st.scale)), st.growth_tracker) and want == 0
        assert (float(np.float32(st.scale)), st.growth_tracker, st.step_count) == (2048.0, 1, 4)
        for t in range(3):
            rc = lib.execute_adam_amp_step_async(dev.handle, c["w"], c["g16"], c["m"], c["v"], c["w16"], 2, bs,
                                                 HYPER["lr"], HYPER["beta1"], HYPER["beta2"], HYPER["eps"],
                                                 HYPER["weight_decay"], amp)
            assert rc == 0, (rc, lib.gm_last_error())
        scale, tracker, applied, skipped = ctypes.c_float(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        assert lib.gm_amp_state_query(amp, ctypes.byref(scale), ctypes.byref(tracker), ctypes.byref(applied),
                                      ctypes.byref(skipped)) == 0
        assert (scale.value, tracker.value, applied.value, skipped.value) == (4096.0, 1, 7, 0)
    finally:
        lib.gm_amp_state_destroy(amp)
        for hs in bufs.values():
            for h in hs:
                dev.free(h)


@pytest.mark.parametrize("seed", range(10))
def test_random_lists_scales_and_injections(dev, seed):
    """Tensor lists, initial scales, growth intervals, hyper-parameters and non-finite injections (+inf, -inf, two
    NaN patterns) drawn from a seeded generator; eight steps each: the skip / scale sequence and every buffer agree
    with the oracle bit for bit."""
    rng = np.random.default_rng(9000 + seed)
    nt = int(rng.integers(1, 10))
    sizes = [int(x) for x in np.exp(rng.uniform(0, np.log(200_000), nt)).astype(int)]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    hyper = dict(lr=float(10 ** rng.uniform(-4, -1)), beta1=0.9, beta2=0.999, eps=1e-8,
                 weight_decay=float(rng.choice([0.0, 1e-4, 0.01])))
    pair = AmpPair(dev, w, hyper, (float(2.0 ** rng.integers(0, 17)), 2.0, 0.5, int(rng.integers(1, 5))))
    try:
        for _ in range(8):
            with np.errstate(all="ignore"):
                g16 = [(rng.normal(0, 1e-3, n) * pair.st.scale).astype(np.float16).view(np.uint16) for n in sizes]
            if rng.random() < 0.3:
                k = int(rng.integers(0, nt))
                g16[k][int(rng.integers(0, sizes[k]))] = int(rng.choice([0x7C00, 0xFC00, 0x7E00, 0xFFFF]))
            pair.step(g16)
        pair.compare(f"seed {seed}")
    finally:
        pair.close()


def test_loss_scale_stays_finite_and_normal(dev):
    """Gradients that never overflow make the scale grow at every interval; it must stop at the largest
    finite power of two (not +inf, where inf * 0.5 = inf would hold it for good and 1 / scale = 0 would
    zero every gradient), and a run of overflows must stop at the smallest normal number.  Device state
    machine against the oracle's, every step."""
    w0 = [np.linspace(-0.5, 0.5, 300).astype(np.float32), np.full(5, 0.25, np.float32)]
    pair = AmpPair(dev, w0, HYPER, (2.0 ** 125, 2.0, 0.5, 1))
    try:
        zero = [np.zeros(s, np.uint16) for s in pair.sizes]
        scales = []
        for _ in range(5):
            assert pair.step(zero) == 0
            scales.append(float(pair.st.scale))
        assert scales == [2.0 ** 126] + [2.0 ** 127] * 4
        pair.compare("scale at its ceiling")
    finally:
        pair.close()
    pair = AmpPair(dev, w0, HYPER, (2.0 ** -124, 2.0, 0.5, 1000))
    try:
        bad = [np.zeros(s, np.uint16) for s in pair.sizes]
        bad[1][4] = 0xFC00
        scales = []
        for _ in range(5):
            assert pair.step(bad) == 1
            scales.append(float(pair.st.scale))
        assert scales == [2.0 ** -125] + [2.0 ** -126] * 4
        pair.compare("scale at its floor")
    finally:
        pair.close()

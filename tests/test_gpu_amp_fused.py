"""The one-pass (ping-pong) mixed-precision Adam step against the CPU oracle.

execute_adam_amp_step_fused keeps weights and moments twice and writes the set that is not current; the
oracle updates in place.  After every step the CURRENT set (and the fp16 weight copy, kept as half of the
current weights from the start) must equal the oracle's buffers bit for bit, the skip / scale / counter
sequence must be the oracle's, and the set that is current must alternate with every applied step and stay
put on a dropped one."""
import ctypes

import numpy as np
import pytest

from harness import gpu_device
from oracle_lib import oracle
from workloads import amp_125m_sizes
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
HYPER = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
GARBAGE = np.float32(-7.5e9)          # what the non-current set holds before its first use


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


def half_bits(a):
    with np.errstate(over="ignore"):
        return a.astype(np.float16).view(np.uint16)


class FusedPair:
    """One tensor list as two device sets plus the fp16 streams, and the same list in the oracle."""

    def __init__(self, dev, weights, hyper, amp_cfg=(65536.0, 2.0, 0.5, 2000), nthreads=1):
        self.dev, self.h, self.nthreads = dev, hyper, nthreads
        self.sizes = [w.size for w in weights]
        self.n = len(weights)
        self.w = [np.array(w, np.float32, copy=True) for w in weights]
        self.m = [np.zeros(s, np.float32) for s in self.sizes]
        self.v = [np.zeros(s, np.float32) for s in self.sizes]
        self.w16 = [half_bits(w) for w in self.w]                      # the invariant holds from the start
        self.st = oracle().amp_state(*amp_cfg)
        junk = lambda: [dev.from_numpy(np.full(max(s, 1), GARBAGE, np.float32)) for s in self.sizes]
        self.sets = [{"w": [dev.from_numpy(w) for w in self.w], "m": [dev.alloc(max(4 * s, 4), zero=True) for s in self.sizes],
                      "v": [dev.alloc(max(4 * s, 4), zero=True) for s in self.sizes]},
                     {"w": junk(), "m": junk(), "v": junk()}]
        self.g16 = [dev.alloc(max(2 * s, 2)) for s in self.sizes]
        self.d_w16 = [dev.from_numpy(h) if h.size else dev.alloc(2) for h in self.w16]
        arr = pkg.handle_array
        self.c = [{k: arr(v) for k, v in s.items()} for s in self.sets]
        self.c_g16, self.c_w16 = arr(self.g16), arr(self.d_w16)
        self.bs = pkg.int_array([4 * s for s in self.sizes])
        self.amp = dev.lib.gm_amp_state_create(dev.handle, *amp_cfg)
        assert self.amp
        self.current = 0

    def gpu_step(self):
        skipped, scale, tracker, cur = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1), ctypes.c_int(-1)
        a, b, h = self.c[0], self.c[1], self.h
        rc = self.dev.lib.execute_adam_amp_step_fused(
            self.dev.handle, a["w"], a["m"], a["v"], b["w"], b["m"], b["v"], self.c_g16, self.c_w16, self.n, self.bs,
            h["lr"], h["beta1"], h["beta2"], h["eps"], h["weight_decay"], int(self.st.step_count) + 1, self.amp,
            ctypes.byref(skipped), ctypes.byref(scale), ctypes.byref(tracker), ctypes.byref(cur))
        assert rc == 0, (rc, self.dev.lib.gm_last_error())
        return skipped.value, scale.value, tracker.value, cur.value

    def step(self, g16):
        for hd, g in zip(self.g16, g16):
            if g.size:
                self.dev.upload(hd, g)
        got = self.gpu_step()
        want_skipped = oracle().adam_amp(self.w, g16, self.m, self.v, self.w16, state=self.st, nthreads=self.nthreads,
                                         **self.h)
        if not want_skipped:
            self.current ^= 1
        want = (want_skipped, float(np.float32(self.st.scale)), self.st.growth_tracker, self.current)
        assert got == want, (got, want)
        return got[0]

    def compare(self, context=""):
        cur = self.sets[self.current]
        for name, host in (("w", self.w), ("m", self.m), ("v", self.v)):
            for k, ref in enumerate(host):
                got = self.dev.to_numpy(cur[name][k], ref.size)
                assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (context, name, k)
        for k, ref in enumerate(self.w16):
            got = self.dev.to_numpy(self.d_w16[k], ref.size, np.uint16)
            assert np.array_equal(got, ref), (context, "w16", k)

    def close(self):
        self.dev.lib.gm_amp_state_destroy(self.amp)
        for s in self.sets:
            for hs in s.values():
                for h in hs:
                    self.dev.free(h)
        for h in self.g16 + self.d_w16:
            self.dev.free(h)


def scaled_g16(rng, sizes, scale, std=1e-3):
    return [half_bits((rng.normal(0, std, n) * scale).astype(np.float32)) for n in sizes]


@pytest.mark.parametrize("chunk,vec,lanes", [(0, 0, 0), (0, 2, 128), (0, 4, 256), (256, 1, 128), (1024, 4, 256),
                                             (65536, 2, 256)])
def test_fused_step_in_every_launch_shape(dev, chunk, vec, lanes):
    """Ragged sizes, a dropped step first of all (nothing is current but the initial set), drops in the middle,
    the loss scale growing every third clean step."""
    lib = dev.lib
    rng = np.random.default_rng(61)
    sizes = [1, 2, 3, 7, 0, 255, 256, 257, 1023, 4097, 65536, 70001]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    assert lib.gm_set_tuning(dev.handle, chunk, -1, vec) == 0 and lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
    try:
        pair = FusedPair(dev, w, HYPER, (1024.0, 2.0, 0.5, 3))
        try:
            for t in range(9):
                g16 = scaled_g16(rng, sizes, np.float32(pair.st.scale))
                if t in (0, 4, 5):
                    victim = [11, 0, 5][t % 3]
                    g16[victim][-1] = [0x7C00, 0xFC00, 0x7E01][t % 3]
                assert pair.step(g16) == (t in (0, 4, 5))
                pair.compare(f"chunk={chunk} vec={vec} lanes={lanes} step={t}")
            assert pair.st.step_count == 6 and pair.current == 0
        finally:
            pair.close()
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0 and lib.gm_set_workgroup_lanes(dev.handle, 0) == 0


def test_fused_step_5000_step_schedule_at_reduced_size(dev):
    """The schedule of configuration 4 (0.5 % of steps with an injected inf / NaN, backoff x0.5, growth x2 every
    2000 clean steps) with every tensor at 1/1000 of its size: every step's record and, every 500 steps, every
    buffer of the current set."""
    rng = np.random.default_rng(0x6D657461 + 4)
    sizes = [max(1, s // 1000) for s in amp_125m_sizes()]
    w = [rng.normal(0, 0.02, s).astype(np.float32) for s in sizes]
    pool = [[rng.normal(0, 1e-4, s).astype(np.float32) for s in sizes] for _ in range(8)]
    inject = rng.random(5000) < 0.005
    pair = FusedPair(dev, w, dict(HYPER, weight_decay=0.0))
    skipped_total = 0
    try:
        for k in range(5000):
            scale = np.float32(pair.st.scale)
            g16 = [half_bits(g * scale) for g in pool[k % len(pool)]]
            if inject[k]:
                t = int(rng.integers(0, len(sizes)))
                g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][skipped_total % 3]
            skipped_total += pair.step(g16)
            if (k + 1) % 500 == 0:
                pair.compare(f"step {k + 1}")
        assert skipped_total == int(inject.sum()) and pair.st.step_count == 5000 - skipped_total
    finally:
        pair.close()


def test_fused_async_bursts(dev):
    """The run-ahead form in bursts the host does not wait for: the device picks the bias corrections and the
    set to read by its own state.  Counters after every burst, buffers after every few."""
    lib, D = dev.lib, dev.handle
    rng = np.random.default_rng(0xF05)
    sizes = [300_000, 4096, 200_000, 77]
    burst, bursts = 10, 12
    w = [rng.normal(0, 0.02, s).astype(np.float32) for s in sizes]
    pair = FusedPair(dev, w, HYPER, (1024.0, 2.0, 0.5, 7))
    g_dev = [[dev.alloc(2 * s) for s in sizes] for _ in range(burst)]
    g_arr = [pkg.handle_array(hs) for hs in g_dev]
    a, b, h = pair.c[0], pair.c[1], pair.h
    try:
        skipped_total = 0
        for bi in range(bursts):
            for j in range(burst):
                g16 = scaled_g16(rng, sizes, np.float32(pair.st.scale))
                if rng.random() < 0.15:
                    t = int(rng.integers(0, len(sizes)))
                    g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][(bi + j) % 3]
                for hd, g in zip(g_dev[j], g16):
                    dev.upload(hd, g)
                sk = oracle().adam_amp(pair.w, g16, pair.m, pair.v, pair.w16, state=pair.st, **h)
                skipped_total += sk
                pair.current ^= 0 if sk else 1
            for j in range(burst):
                rc = lib.execute_adam_amp_step_fused_async(D, a["w"], a["m"], a["v"], b["w"], b["m"], b["v"], g_arr[j],
                                                           pair.c_w16, pair.n, pair.bs, h["lr"], h["beta1"], h["beta2"],
                                                           h["eps"], h["weight_decay"], pair.amp)
                assert rc == 0, (rc, lib.gm_last_error())
            scale, tracker, applied, skipped = ctypes.c_float(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            assert lib.gm_amp_state_query(pair.amp, ctypes.byref(scale), ctypes.byref(tracker), ctypes.byref(applied),
                                          ctypes.byref(skipped)) == 0
            assert (scale.value, tracker.value, applied.value, skipped.value) == \
                (float(np.float32(pair.st.scale)), pair.st.growth_tracker, pair.st.step_count, skipped_total), bi
            assert lib.gm_amp_state_current_set(pair.amp) == pair.current
            if bi % 4 == 3:
                pair.compare(f"burst {bi}")
        assert 5 < skipped_total < burst * bursts - 30
    finally:
        pair.close()
        for hs in g_dev:
            for hd in hs:
                dev.free(hd)


def test_fused_step_argument_errors(dev):
    lib, D = dev.lib, dev.handle
    n = 1000
    bufs = {k: dev.alloc(4 * n, zero=True) for k in ("wa", "ma", "va", "wb", "mb", "vb")}
    g16, short = dev.alloc(2 * n, zero=True), dev.alloc(4 * n - 64, zero=True)
    arr = pkg.handle_array
    bs = pkg.int_array([4 * n])
    amp = lib.gm_amp_state_create(D, 65536.0, 2.0, 0.5, 2000)
    sk = ctypes.c_int()

    def call(device=D, wb=bufs["wb"], vb_array=True, state=amp):
        return lib.execute_adam_amp_step_fused(
            device, arr([bufs["wa"]]), arr([bufs["ma"]]), arr([bufs["va"]]), arr([wb]), arr([bufs["mb"]]),
            arr([bufs["vb"]]) if vb_array else None, arr([g16]), None, 1, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, state,
            ctypes.byref(sk), None, None, None)

    try:
        assert call(device=0) == -1
        assert call(state=0) == -16
        assert call(vb_array=False) == -4
        assert call(wb=0) == -4
        assert call(wb=short) == -4 and b"shorter" in lib.gm_last_error()
        before = dev.to_numpy(bufs["wa"], n).copy()
        assert call() == 0 and sk.value == 0                      # no fp16 copy requested: allowed
        assert lib.gm_amp_state_current_set(amp) == 1
        assert np.array_equal(dev.to_numpy(bufs["wa"], n), before)   # the set that was current is only read
    finally:
        lib.gm_amp_state_destroy(amp)
        for h in list(bufs.values()) + [g16, short]:
            dev.free(h)


def test_fused_step_refuses_sets_whose_skipped_tensors_differ(dev):
    """Two tensors of one size, the first one's weight buffer too short in set A only and the second one's in set B
    only: each set skips one tensor, so chunk counts, chunk sizes and element totals of the two layouts agree, and
    pairing them chunk for chunk would read one tensor and write the other.  The step is refused (-4) and nothing is
    written."""
    lib, D = dev.lib, dev.handle
    n = 5000
    arr = pkg.handle_array
    full = {k: [dev.from_numpy(np.full(n, 1.5 + i, np.float32)) for i in range(2)] for k in ("wa", "ma", "va", "wb", "mb", "vb")}
    short = [dev.from_numpy(np.full(n - 16, 9.0, np.float32)) for _ in range(2)]
    g16 = [dev.alloc(2 * n, zero=True) for _ in range(2)]
    w16 = [dev.from_numpy(np.full(n, 0x3C00, np.uint16)) for _ in range(2)]
    bs = pkg.int_array([4 * n, 4 * n])
    amp = lib.gm_amp_state_create(D, 65536.0, 2.0, 0.5, 2000)
    sk = ctypes.c_int(-1)
    try:
        wa = [short[0], full["wa"][1]]
        wb = [full["wb"][0], short[1]]
        rc = lib.execute_adam_amp_step_fused(D, arr(wa), arr(full["ma"]), arr(full["va"]), arr(wb), arr(full["mb"]),
                                             arr(full["vb"]), arr(g16), arr(w16), 2, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1,
                                             amp, ctypes.byref(sk), None, None, None)
        assert rc == -4 and b"same tensors" in lib.gm_last_error(), (rc, lib.gm_last_error())
        assert lib.gm_amp_state_current_set(amp) == 0
        for k, hs in full.items():
            for i, h in enumerate(hs):
                assert np.all(dev.to_numpy(h, n) == np.float32(1.5 + i)), (k, i)
        for h in w16:
            assert np.all(dev.to_numpy(h, n, np.uint16) == 0x3C00)
        # the same tensor short in both sets is skipped in both: allowed, and the other tensor is stepped
        wb2 = [short[1], full["wb"][1]]
        rc = lib.execute_adam_amp_step_fused(D, arr(wa), arr(full["ma"]), arr(full["va"]), arr(wb2), arr(full["mb"]),
                                             arr(full["vb"]), arr(g16), arr(w16), 2, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1,
                                             amp, ctypes.byref(sk), None, None, None)
        assert rc == 0 and sk.value == 0, (rc, lib.gm_last_error())
        assert np.all(dev.to_numpy(full["wb"][0], n) == np.float32(1.5))          # tensor 0: skipped, untouched
        assert np.all(dev.to_numpy(full["mb"][0], n) == np.float32(1.5))
        assert not np.all(dev.to_numpy(full["mb"][1], n) == np.float32(2.5))      # tensor 1: set B written
    finally:
        lib.gm_amp_state_destroy(amp)
        for hs in list(full.values()) + [short, g16, w16]:
            for h in hs:
                dev.free(h)


def test_in_place_and_one_pass_steps_share_one_loss_scale_state(dev):
    """Both forms advance the same device state and tell an overflow by the same per-step stamp: alternated on one
    list (the in-place step working on whichever set is current), with dropped steps next to each other, before
    and after applied ones and across the change of form, the sequence is the oracle's and nothing of an earlier
    step's overflow leaks into a later one."""
    lib = dev.lib
    rng = np.random.default_rng(77)
    sizes = [1, 255, 4096, 70001]
    pair = FusedPair(dev, [rng.standard_normal(s).astype(np.float32) for s in sizes], HYPER, (1024.0, 2.0, 0.5, 3))
    poisoned = {1, 2, 5, 8, 9, 10, 14}
    forms = "FFIIFIFFIIFIIFFIFI"           # F: one pass, I: in place
    try:
        for k, form in enumerate(forms):
            g16 = scaled_g16(rng, sizes, pair.st.scale)
            if k in poisoned:
                t = k % len(sizes)
                g16[t][(k * 37) % sizes[t]] = [0x7C00, 0xFC00, 0x7E00][k % 3]
            if form == "F":
                assert pair.step(g16) == (1 if k in poisoned else 0)
            else:
                for hd, g in zip(pair.g16, g16):
                    dev.upload(hd, g)
                cur = pair.c[pair.current]
                skipped, scale, tracker = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1)
                rc = lib.execute_adam_amp_step(dev.handle, cur["w"], pair.c_g16, cur["m"], cur["v"], pair.c_w16, pair.n,
                                               pair.bs, HYPER["lr"], HYPER["beta1"], HYPER["beta2"], HYPER["eps"],
                                               HYPER["weight_decay"], int(pair.st.step_count) + 1, pair.amp,
                                               ctypes.byref(skipped), ctypes.byref(scale), ctypes.byref(tracker))
                assert rc == 0, (rc, lib.gm_last_error())
                want = oracle().adam_amp(pair.w, g16, pair.m, pair.v, pair.w16, state=pair.st, **HYPER)
                assert (skipped.value, scale.value, tracker.value) == (want, float(np.float32(pair.st.scale)),
                                                                        pair.st.growth_tracker), (k, form)
                assert want == (1 if k in poisoned else 0)
                assert lib.gm_amp_state_current_set(pair.amp) == pair.current      # an in-place step never flips it
            pair.compare(f"step {k} ({form})")
    finally:
        pair.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_mix_of_forms_waits_and_state_edits(dev, seed):
    """One loss-scale state driven by a random program: bursts of one to six steps, each burst in place or in one
    pass, waited for step by step or run ahead, with injected overflows, and between bursts now and then a restored
    scale / clean-step counter or a step count set by the host.  The device keeps its state in two records that
    swap roles with every step and tells finished steps by stamps in pinned memory: after every burst the counters,
    the current set and every buffer must be the oracle's."""
    lib, D = dev.lib, dev.handle
    rng = np.random.default_rng(0xA11CE + seed)
    sizes = [int(x) for x in rng.choice([1, 63, 256, 1000, 4097, 70001, 150_000], size=int(rng.integers(2, 6)))]
    interval = int(rng.integers(2, 6))
    pair = FusedPair(dev, [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes], HYPER, (4096.0, 2.0, 0.5, interval))
    g_dev = [[dev.alloc(2 * n) for n in sizes] for _ in range(6)]
    g_arr = [pkg.handle_array(hs) for hs in g_dev]
    h = pair.h
    skipped_total = 0
    try:
        for burst in range(30):
            one_pass = bool(rng.integers(0, 2))
            waited = bool(rng.integers(0, 2))
            length = int(rng.integers(1, 7))
            in_set = pair.current                        # an in-place burst works on the set current at its start
            expected = []
            for j in range(length):
                g16 = scaled_g16(rng, sizes, np.float32(pair.st.scale))
                if rng.random() < 0.25:
                    t = int(rng.integers(0, len(sizes)))
                    g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][(burst + j) % 3]
                for hd, g in zip(g_dev[j], g16):
                    dev.upload(hd, g)
                count_before = int(pair.st.step_count)
                sk = oracle().adam_amp(pair.w, g16, pair.m, pair.v, pair.w16, state=pair.st, **h)
                skipped_total += sk
                if one_pass and not sk:
                    pair.current ^= 1
                expected.append((sk, float(np.float32(pair.st.scale)), pair.st.growth_tracker, pair.current, count_before + 1))
            a, b, cur = pair.c[0], pair.c[1], pair.c[in_set]
            for j in range(length):
                skipped, scale, tracker, now = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1), ctypes.c_int(-1)
                if one_pass and waited:
                    rc = lib.execute_adam_amp_step_fused(D, a["w"], a["m"], a["v"], b["w"], b["m"], b["v"], g_arr[j],
                                                         pair.c_w16, pair.n, pair.bs, h["lr"], h["beta1"], h["beta2"],
                                                         h["eps"], h["weight_decay"], expected[j][4], pair.amp,
                                                         ctypes.byref(skipped), ctypes.byref(scale), ctypes.byref(tracker),
                                                         ctypes.byref(now))
                    assert (skipped.value, scale.value, tracker.value, now.value) == expected[j][:4], (burst, j)
                elif one_pass:
                    rc = lib.execute_adam_amp_step_fused_async(D, a["w"], a["m"], a["v"], b["w"], b["m"], b["v"], g_arr[j],
                                                               pair.c_w16, pair.n, pair.bs, h["lr"], h["beta1"],
                                                               h["beta2"], h["eps"], h["weight_decay"], pair.amp)
                elif waited:
                    rc = lib.execute_adam_amp_step(D, cur["w"], g_arr[j], cur["m"], cur["v"], pair.c_w16, pair.n, pair.bs,
                                                   h["lr"], h["beta1"], h["beta2"], h["eps"], h["weight_decay"],
                                                   expected[j][4], pair.amp, ctypes.byref(skipped), ctypes.byref(scale),
                                                   ctypes.byref(tracker))
                    assert (skipped.value, scale.value, tracker.value) == expected[j][:3], (burst, j)
                else:
                    rc = lib.execute_adam_amp_step_async(D, cur["w"], g_arr[j], cur["m"], cur["v"], pair.c_w16, pair.n,
                                                         pair.bs, h["lr"], h["beta1"], h["beta2"], h["eps"],
                                                         h["weight_decay"], pair.amp)
                assert rc == 0, (rc, lib.gm_last_error(), burst, j)
            scale, tracker, applied, skipped = ctypes.c_float(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            assert lib.gm_amp_state_query(pair.amp, ctypes.byref(scale), ctypes.byref(tracker), ctypes.byref(applied),
                                          ctypes.byref(skipped)) == 0
            assert (scale.value, tracker.value, applied.value, skipped.value) == \
                (float(np.float32(pair.st.scale)), pair.st.growth_tracker, pair.st.step_count, skipped_total), (burst, one_pass, waited)
            assert lib.gm_amp_state_current_set(pair.amp) == pair.current
            pair.compare(f"seed {seed} burst {burst}")
            edit = rng.random()
            if edit < 0.15:                               # a checkpoint's scale and counter are restored
                new_scale = float(2.0 ** int(rng.integers(8, 15)))
                new_tracker = int(rng.integers(0, interval))
                assert lib.gm_amp_state_set(pair.amp, new_scale, new_tracker) == 0
                pair.st.scale, pair.st.growth_tracker = new_scale, new_tracker
            elif edit < 0.3:                              # the optimizer's step count is set by the host
                new_count = int(rng.integers(0, 3000))
                assert lib.gm_amp_state_set_step_count(pair.amp, new_count) == 0
                pair.st.step_count = new_count
        assert skipped_total > 5
    finally:
        pair.close()
        for hs in g_dev:
            for hd in hs:
                dev.free(hd)

"""Out-of-bounds guards around every stream of the update kernels.

Each stream of a rule (weights, gradients, every state, the fp16 streams of the mixed-precision
step) is ONE parent buffer in which the tensors lie back to back, separated and bracketed by guard
gaps filled with a sentinel.  The handles passed to the step are views into that parent, some
16-byte aligned (vector lanes) and some only element aligned (scalar tails).  After several steps
every guard must still hold the sentinel bit for bit: a write one element before a tensor, one past
its end, or a whole slice into its neighbour shows up here, for every lane width, workgroup size and
chunk size the library can launch, for both segments of a two-segment plan, and for the
allocation-free step.  The tensors themselves are compared with the CPU oracle."""
import ctypes

import numpy as np
import pytest

from harness import OracleRun, gpu_device, states_for
from oracle_lib import oracle
from workloads import two_segment_sizes
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()

GUARD = 64                       # elements of sentinel on each side of every tensor, at least
F32_SENTINEL = np.uint32(0x7FC5A5A5)     # a NaN pattern no update produces
F16_SENTINEL = np.uint16(0x7E5A)
EDGE_SIZES = [1, 2, 3, 63, 64, 65, 255, 256, 257, 511, 513, 1023, 1024, 1025, 4095, 4096, 4097,
              16383, 16385, 65535, 65536, 65537, 70001]

RULES = [
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=1e-4, nesterov=True)),
    ("sgd", dict(lr=0.01, momentum=0.0, weight_decay=0.0, nesterov=False)),
    ("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0, centered=False)),
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=1e-4, momentum=0.9, centered=True)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=0.0)),
    ("adadelta", dict(rho=0.9, eps=1e-6, weight_decay=0.0)),
    ("nadam", dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)),
]
# (chunk, vec, lanes): 0 = the library's own choice
SHAPES = [(0, 0, 0), (0, 1, 256), (0, 2, 128), (0, 4, 256), (256, 1, 128), (1024, 4, 256), (65536, 2, 256)]


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


class Packed:
    """One stream: a parent buffer [guard][t0][guard][t1]...[guard] and the view handle of each tensor.
    Even tensors start 16-byte aligned, odd ones wherever the previous guard ends."""

    def __init__(self, dev, sizes, dtype, fill=None):
        self.dev, self.sizes, self.dtype = dev, sizes, np.dtype(dtype)
        self.sentinel = F32_SENTINEL if self.dtype.itemsize == 4 else F16_SENTINEL
        raw = np.uint32 if self.dtype.itemsize == 4 else np.uint16
        per16 = 16 // self.dtype.itemsize
        self.offsets, pos = [], 0
        for i, n in enumerate(sizes):
            pos += GUARD
            if i % 2 == 0:
                pos = (pos + per16 - 1) // per16 * per16
            elif pos % 2 == 0:
                pos += 1                      # odd element offset: no vector access is legal here
            self.offsets.append(pos)
            pos += n
        self.total = pos + GUARD
        self.host = np.full(self.total, self.sentinel, raw)
        for i, (off, n) in enumerate(zip(self.offsets, sizes)):
            self.host[off:off + n] = 0 if fill is None else np.ascontiguousarray(fill[i]).view(raw)
        self.parent = dev.from_numpy(self.host)
        self.views = [self.parent + off * self.dtype.itemsize for off in self.offsets]
        self.mask = np.ones(self.total, bool)
        for off, n in zip(self.offsets, sizes):
            self.mask[off:off + n] = False

    def upload(self, arrays):
        raw = self.host.dtype
        for off, n, a in zip(self.offsets, self.sizes, arrays):
            self.host[off:off + n] = np.ascontiguousarray(a).view(raw)
        self.dev.upload(self.parent, self.host)

    def read(self):
        """(list of tensors, True when every guard element still holds the sentinel)."""
        got = self.dev.to_numpy(self.parent, self.total, self.host.dtype)
        guards_ok = bool(np.all(got[self.mask] == self.sentinel))
        return [got[off:off + n].view(self.dtype) for off, n in zip(self.offsets, self.sizes)], guards_ok

    def bad_guards(self):
        got = self.dev.to_numpy(self.parent, self.total, self.host.dtype)
        return np.flatnonzero(self.mask & (got != self.sentinel))[:8].tolist()

    def free(self):
        self.dev.free(self.parent)


def launch(dev, rule, h, c, n, bs, t, fn=None):
    lib, d = dev.lib, dev.handle
    if rule == "sgd":
        return lib.execute_sgd_step_mpsgraph(d, c["w"], c["g"], c.get("m"), n, bs, h["lr"], h["momentum"],
                                             h["weight_decay"], int(h["nesterov"]), t)
    if rule == "adam":
        return (fn or lib.execute_adam_step_mpsgraph)(d, c["w"], c["g"], c["m"], c["v"], n, bs, h["lr"], h["beta1"],
                                                      h["beta2"], h["eps"], h["weight_decay"], t)
    if rule == "nadam":
        return lib.execute_nadam_step_mpsgraph(d, c["w"], c["g"], c["m"], c["v"], n, bs, h["lr"], h["beta1"],
                                               h["beta2"], h["eps"], h["weight_decay"], t)
    if rule == "rmsprop":
        return lib.execute_rmsprop_step_mpsgraph(d, c["w"], c["g"], c["s"], c.get("b"), c.get("ga"), n, bs, h["lr"],
                                                 h["alpha"], h["eps"], h["weight_decay"], h["momentum"],
                                                 bool(h["centered"]), t)
    if rule == "adagrad":
        return lib.execute_adagrad_step_mpsgraph(d, c["w"], c["g"], c["s"], n, bs, h["lr"], h["eps"], h["weight_decay"])
    return lib.execute_adadelta_step_mpsgraph(d, c["w"], c["g"], c["s"], c["a"], n, bs, h["rho"], h["eps"],
                                              h["weight_decay"])


def run_guarded(dev, rule, hyper, sizes, steps, seed, fn=None, context=""):
    rng = np.random.default_rng(seed)
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    names = ["w", "g"] + states_for(rule, hyper)
    streams = {k: Packed(dev, sizes, np.float32, fill=w0 if k == "w" else None) for k in names}
    c = {k: pkg.handle_array(s.views) for k, s in streams.items()}
    bs = pkg.int_array([4 * n for n in sizes])
    cpu = OracleRun(rule, hyper, w0)
    try:
        for t in range(1, steps + 1):
            grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
            streams["g"].upload(grads)
            rc = launch(dev, rule, hyper, c, len(sizes), bs, t, fn)
            assert rc == 0, (context, rc, dev.lib.gm_last_error())
            cpu.step(grads)
        want = cpu.snapshot()
        for k, s in streams.items():
            tensors, guards_ok = s.read()
            assert guards_ok, f"{context}: stream {k} wrote into a guard at parent elements {s.bad_guards()}"
            if k == "g":
                continue
            for i, (a, b) in enumerate(zip(tensors, want[k])):
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (context, k, i, sizes[i])
    finally:
        for s in streams.values():
            s.free()


@pytest.mark.parametrize("rule,hyper", RULES, ids=[f"{r}-{i}" for i, (r, _) in enumerate(RULES)])
def test_guards_survive_every_rule_in_every_launch_shape(dev, rule, hyper):
    lib = dev.lib
    try:
        for chunk, vec, lanes in SHAPES:
            assert lib.gm_set_tuning(dev.handle, chunk, -1, vec) == 0, (chunk, vec)
            assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
            run_guarded(dev, rule, hyper, EDGE_SIZES, steps=3, seed=101,
                        context=f"{rule} chunk={chunk} vec={vec} lanes={lanes}")
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0


def test_guards_survive_the_allocation_free_step(dev):
    hyper = RULES[2][1]
    lib = dev.lib
    try:
        for chunk, vec, lanes in SHAPES:
            assert lib.gm_set_tuning(dev.handle, chunk, -1, vec) == 0
            assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
            run_guarded(dev, "adam", hyper, EDGE_SIZES, steps=3, seed=103, fn=lib.execute_adam_step_noalloc,
                        context=f"noalloc chunk={chunk} vec={vec} lanes={lanes}")
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0


def test_guards_survive_a_two_segment_plan(dev):
    """A list the planner cuts into two segments (one 120M-element tensor in 65536-element chunks, 80 small
    tensors in a segment of their own; tests/test_planner_bounds.py checks that this list does get two):
    guards around every small tensor and around the large one."""
    hyper = RULES[2][1]
    sizes = two_segment_sizes()
    rng = np.random.default_rng(7)
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    g0 = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
    streams = {k: Packed(dev, sizes, np.float32, fill={"w": w0, "g": g0}.get(k)) for k in ("w", "g", "m", "v")}
    c = {k: pkg.handle_array(s.views) for k, s in streams.items()}
    bs = pkg.int_array([4 * n for n in sizes])
    cpu = OracleRun("adam", hyper, w0, nthreads=min(16, __import__("os").cpu_count() or 1))
    try:
        for t in (1, 2):
            assert launch(dev, "adam", hyper, c, len(sizes), bs, t) == 0, dev.lib.gm_last_error()
            cpu.step(g0)
        want = cpu.snapshot()
        for k, s in streams.items():
            tensors, guards_ok = s.read()
            assert guards_ok, f"two segments: stream {k} wrote into a guard at {s.bad_guards()}"
            if k != "g":
                for i, (a, b) in enumerate(zip(tensors, want[k])):
                    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (k, i, sizes[i])
    finally:
        for s in streams.values():
            s.free()


@pytest.mark.parametrize("chunk,vec,lanes", SHAPES)
def test_guards_survive_the_mixed_precision_step(dev, chunk, vec, lanes):
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    lib, o = dev.lib, oracle()
    sizes = EDGE_SIZES
    rng = np.random.default_rng(113)
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    w16 = [np.zeros(n, np.uint16) for n in sizes]
    streams = {"w": Packed(dev, sizes, np.float32, fill=w), "m": Packed(dev, sizes, np.float32),
               "v": Packed(dev, sizes, np.float32), "g16": Packed(dev, sizes, np.float16),
               "w16": Packed(dev, sizes, np.float16)}
    c = {k: pkg.handle_array(s.views) for k, s in streams.items()}
    bs = pkg.int_array([4 * n for n in sizes])
    amp = lib.gm_amp_state_create(dev.handle, 65536.0, 2.0, 0.5, 2000)
    st = o.amp_state()
    assert amp
    try:
        assert lib.gm_set_tuning(dev.handle, chunk, -1, vec) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
        for k_step in range(4):
            g16 = [(rng.normal(0, 1e-4, n) * 65536.0).astype(np.float16).view(np.uint16) for n in sizes]
            if k_step == 2:
                g16[-1][-1] = 0x7C00          # the very last element of the list: the step is dropped
            streams["g16"].upload(g16)
            skipped, scale, tracker = ctypes.c_int(-1), ctypes.c_float(0), ctypes.c_int(-1)
            rc = lib.execute_adam_amp_step(dev.handle, c["w"], c["g16"], c["m"], c["v"], c["w16"], len(sizes), bs,
                                           hyper["lr"], hyper["beta1"], hyper["beta2"], hyper["eps"],
                                           hyper["weight_decay"], int(st.step_count) + 1, amp, ctypes.byref(skipped),
                                           ctypes.byref(scale), ctypes.byref(tracker))
            assert rc == 0, (rc, lib.gm_last_error())
            want = o.adam_amp(w, g16, m, v, w16, state=st, **hyper)
            assert skipped.value == want == (1 if k_step == 2 else 0)
        for name, host in (("w", w), ("m", m), ("v", v), ("w16", w16), ("g16", None)):
            tensors, guards_ok = streams[name].read()
            assert guards_ok, f"mixed precision chunk={chunk} vec={vec} lanes={lanes}: stream {name} wrote into " \
                              f"a guard at {streams[name].bad_guards()}"
            if host is not None:
                for i, (a, b) in enumerate(zip(tensors, host)):
                    assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (name, i, sizes[i])
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0
        lib.gm_amp_state_destroy(amp)
        for s in streams.values():
            s.free()


@pytest.mark.parametrize("chunk,vec,lanes", SHAPES)
def test_guards_survive_the_one_pass_mixed_precision_step(dev, chunk, vec, lanes):
    """The ping-pong step writes the set that is not current: guards around every tensor of BOTH sets and of
    the two fp16 streams, over applied and dropped steps (so that each set is written at least twice)."""
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    lib, o = dev.lib, oracle()
    sizes = EDGE_SIZES
    rng = np.random.default_rng(127)
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    w16 = [a.astype(np.float16).view(np.uint16) for a in w]
    names = ("wa", "ma", "va", "wb", "mb", "vb")
    streams = {k: Packed(dev, sizes, np.float32, fill=w if k == "wa" else None) for k in names}
    streams["g16"] = Packed(dev, sizes, np.float16)
    streams["w16"] = Packed(dev, sizes, np.float16, fill=w16)
    c = {k: pkg.handle_array(s.views) for k, s in streams.items()}
    bs = pkg.int_array([4 * n for n in sizes])
    amp = lib.gm_amp_state_create(dev.handle, 65536.0, 2.0, 0.5, 2000)
    st = o.amp_state()
    assert amp
    current = 0
    try:
        assert lib.gm_set_tuning(dev.handle, chunk, -1, vec) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
        for k_step in range(6):
            g16 = [(rng.normal(0, 1e-4, n) * np.float32(st.scale)).astype(np.float16).view(np.uint16) for n in sizes]
            if k_step in (1, 4):
                g16[k_step][0] = 0x7E00
            streams["g16"].upload(g16)
            skipped, cur = ctypes.c_int(-1), ctypes.c_int(-1)
            rc = lib.execute_adam_amp_step_fused(dev.handle, c["wa"], c["ma"], c["va"], c["wb"], c["mb"], c["vb"], c["g16"],
                                                 c["w16"], len(sizes), bs, hyper["lr"], hyper["beta1"], hyper["beta2"],
                                                 hyper["eps"], hyper["weight_decay"], int(st.step_count) + 1, amp,
                                                 ctypes.byref(skipped), None, None, ctypes.byref(cur))
            assert rc == 0, (rc, lib.gm_last_error())
            want = o.adam_amp(w, g16, m, v, w16, state=st, **hyper)
            current ^= 0 if want else 1
            assert (skipped.value, cur.value) == (want, current) and want == (1 if k_step in (1, 4) else 0)
        assert current == 0
        for name, s in streams.items():
            tensors, guards_ok = s.read()
            assert guards_ok, f"one pass chunk={chunk} vec={vec} lanes={lanes}: stream {name} wrote into a guard at " \
                              f"{s.bad_guards()}"
            host = {"wa": w, "ma": m, "va": v, "w16": w16}.get(name)
            if host is not None:
                for i, (a, b) in enumerate(zip(tensors, host)):
                    assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (name, i, sizes[i])
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0
        lib.gm_amp_state_destroy(amp)
        for s in streams.values():
            s.free()

"""Learning-rate schedules reaching the kernels, and the plan cache staying put.

The reference's engine asks its scheduler for the epoch's rate and fans it out to the optimizer
(engine/model_engine.go:2345-2390, training/scheduler.go:38-180); the optimizer passes its
LearningRate to the native step on every call.  Here the rate is a kernel argument, so a step after
UpdateLearningRate must use the new value bit-exactly and must not lay out a new chunk table.  The
expected rates come from a restatement of the reference's formulas in this file, not from the
library."""
import ctypes
import math

import numpy as np
import pytest

from harness import GpuRun, OracleRun, compare_snapshots, gpu_device
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()

SHAPES = [[32, 3, 3, 3], [32], [300, 17], [1], [70000]]
KINDS = {
    "adam": ([1e-3, 0.9, 0.999, 1e-8, 1e-4], dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
    "sgd": ([0.01, 0.9, 1e-4, 0], dict(lr=0.01, momentum=0.9, weight_decay=1e-4, nesterov=False)),
}
STEPS = 24


@pytest.fixture(scope="module")
def env():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    dev.lib.gmo_initialize_global_memory_manager(dev.handle)
    mm = dev.lib.gmo_get_global_memory_manager()
    assert mm
    return dev, mm


def plan_stats(dev):
    builds, tables, cached = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_int()
    assert dev.lib.gm_plan_cache_stats(dev.handle, ctypes.byref(builds), ctypes.byref(tables), ctypes.byref(cached)) == 0
    return builds.value, tables.value, cached.value


# ---- the reference's schedules, restated (training/scheduler.go) ----
def step_lr(epoch, base, step_size=3, gamma=0.5):                      # :38-41
    return base * math.pow(gamma, float(epoch // step_size))


def cosine_lr(epoch, base, t_max=20, eta_min=1e-5):                    # :91-97
    if epoch >= t_max:
        return eta_min
    return eta_min + (base - eta_min) * (1 + math.cos(math.pi * epoch / t_max)) / 2


class Plateau:                                                          # :131-170, mode "min"
    def __init__(self, factor=0.5, patience=2, threshold=1e-4):
        self.factor, self.patience, self.threshold = factor, patience, threshold
        self.best, self.bad, self.started = 0.0, 0, False

    def step(self, metric, lr):
        if not self.started:
            self.best, self.started = metric, True
            return lr
        if metric < self.best - self.threshold:
            self.best, self.bad = metric, 0
        else:
            self.bad += 1
        if self.bad >= self.patience:
            self.bad = 0
            return lr * self.factor
        return lr


METRICS = [1.0, 0.9, 0.95, 0.95, 0.8, 0.8, 0.8, 0.8, 0.7, 0.71, 0.72, 0.6] * 2


@pytest.mark.parametrize("schedule", ["StepLR", "CosineAnnealingLR", "ReduceLROnPlateau"])
@pytest.mark.parametrize("kind", ["adam", "sgd"])
def test_scheduled_learning_rate_reaches_the_step_exactly(env, kind, schedule):
    dev, mm = env
    lib = dev.lib
    cfg, hyper = KINDS[kind]
    base = float(np.float32(cfg[0]))
    rng = np.random.default_rng(41)
    sizes = [int(np.prod(s)) for s in SHAPES]
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    opt = pkg.HostOptimizer(kind, cfg, SHAPES, mm, dev.handle)
    assert opt.error is None, opt.error
    weights = [dev.from_numpy(w) for w in w0]
    gbufs = [dev.alloc(4 * n) for n in sizes]
    assert opt.SetWeightBuffers(weights) is None
    cpu = OracleRun(kind, dict(hyper), w0)
    sched = {"StepLR": lambda: lib.gmo_scheduler_new(0, 3, 0.5, 0.0, None),
             "CosineAnnealingLR": lambda: lib.gmo_scheduler_new(2, 20, 1e-5, 0.0, None),
             "ReduceLROnPlateau": lambda: lib.gmo_scheduler_new(3, 2, 0.5, 1e-4, b"min")}[schedule]()
    assert sched and lib.gmo_scheduler_name(sched) == schedule.encode()
    plateau, current = Plateau(), base
    seen = set()
    try:
        builds_after_first = None
        for epoch in range(STEPS):
            # engine: scheduler -> UpdateLearningRate(float32(lr)) -> Step
            if schedule == "ReduceLROnPlateau":
                previous = current
                current = plateau.step(METRICS[epoch], previous)
                assert lib.gmo_scheduler_plateau_step(sched, METRICS[epoch], previous) == current
                want_lr = current
            else:
                want_lr = step_lr(epoch, base) if schedule == "StepLR" else cosine_lr(epoch, base)
            got_lr = lib.gmo_scheduler_apply(sched, opt.handle, epoch, 0, base)
            assert got_lr == want_lr, (epoch, got_lr, want_lr)
            assert opt.field("LearningRate") == np.float32(want_lr)
            seen.add(float(np.float32(want_lr)))
            grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
            for h, g in zip(gbufs, grads):
                dev.upload(h, g)
            assert opt.Step(gbufs) is None
            cpu.h["lr"] = float(np.float32(want_lr))
            cpu.step(grads)
            if epoch == 0:
                builds_after_first = plan_stats(dev)[0]
            if epoch in (0, 7, STEPS - 1):
                for k, n in enumerate(sizes):
                    assert np.array_equal(dev.to_numpy(weights[k], n).view(np.uint32), cpu.w[k].view(np.uint32)), \
                        (schedule, kind, epoch, k)
        assert len(seen) >= 4, "the schedule must actually move the rate"
        # one chunk table for the whole run: the rate travels as a kernel argument
        assert plan_stats(dev)[0] == builds_after_first
        for name in cpu.state:
            st = {"m": "momentum", "v": "variance"}[name]
            for k, n in enumerate(sizes):
                got = dev.to_numpy(opt.state_buffer(st, k), n)
                assert np.array_equal(got.view(np.uint32), cpu.state[name][k].view(np.uint32)), (name, k)
    finally:
        lib.gmo_scheduler_free(sched)
        opt.Cleanup()
        opt.free()
        for h in weights + gbufs:
            dev.free(h)


ADAM = KINDS["adam"][1]


def test_unrelated_allocations_leave_cached_plans_alone(env):
    """A caller that allocates and frees a scratch buffer between steps: the step's plan survives; freeing
    a buffer the plan does use drops exactly that plan; table memory is reused, not reallocated."""
    dev, _ = env
    rng = np.random.default_rng(43)
    sizes = [70001, 5, 4097, 262147, 1023]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    gpu, cpu = GpuRun(dev, "adam", ADAM, w), OracleRun("adam", ADAM, w)
    other = GpuRun(dev, "adam", ADAM, [w[0]])            # a second optimizer whose plan must survive too
    ocpu = OracleRun("adam", ADAM, [w[0]])
    try:
        grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
        gpu.step(grads)
        cpu.step(grads)
        other.step([grads[0]])
        ocpu.step([grads[0]])
        builds0, tables0, _ = plan_stats(dev)
        for t in range(12):
            scratch = dev.alloc(4096 * (t + 1))
            dev.free(scratch)
            gpu.launch()
            cpu.step(grads)
            other.launch()
            ocpu.step([grads[0]])
        assert plan_stats(dev)[:2] == (builds0, tables0)
        compare_snapshots(gpu.snapshot(), cpu.snapshot(), 0, "after unrelated frees")
        compare_snapshots(other.snapshot(), ocpu.snapshot(), 0, "second optimizer after unrelated frees")

        # a gradient buffer of the first list is replaced: its plan goes, the other optimizer's stays
        fresh = dev.from_numpy(grads[2])
        dev.free(gpu.g[2])
        gpu.g[2] = fresh
        gpu.c_g = pkg.handle_array(gpu.g)
        other.launch()
        ocpu.step([grads[0]])
        assert plan_stats(dev)[0] == builds0
        gpu.launch()
        cpu.step(grads)
        builds1, tables1, _ = plan_stats(dev)
        assert builds1 == builds0 + 1
        assert tables1 == tables0, "the dropped plan's table slot is reused"
        compare_snapshots(gpu.snapshot(), cpu.snapshot(), 0, "after replacing a gradient buffer")
        compare_snapshots(other.snapshot(), ocpu.snapshot(), 0, "second optimizer")
    finally:
        gpu.close()
        other.close()


def test_a_freed_address_that_comes_back_shorter_is_revalidated(env):
    """The reason plans are dropped at all: the same address may be handed out again with another
    length, and a tensor whose buffer is shorter than its size must be skipped
    (bridge_optimizer.m:427-436), not updated from a stale table."""
    dev, _ = env
    lib = dev.lib
    n = 100_000
    rng = np.random.default_rng(47)
    w0 = rng.normal(0, 0.02, n).astype(np.float32)
    g0 = rng.normal(0, 1e-3, n).astype(np.float32)
    w, m, v = dev.from_numpy(w0), dev.alloc(4 * n, zero=True), dev.alloc(4 * n, zero=True)
    g = dev.from_numpy(g0)
    bs = pkg.int_array([4 * n])
    arr = pkg.handle_array

    def step(gh, t):
        return lib.execute_adam_step_mpsgraph(dev.handle, arr([w]), arr([gh]), arr([m]), arr([v]), 1, bs, 1e-3, 0.9,
                                              0.999, 1e-8, 0.0, t)

    try:
        assert step(g, 1) == 0
        after_one = dev.to_numpy(w, n)
        assert not np.array_equal(after_one, w0)
        dev.free(g)
        # ask for the same address again with half the length (the allocator usually returns it; if not,
        # the step below is an ordinary one and the test only checks the general behaviour)
        g_short = dev.alloc(2 * n)
        dev.upload(g_short, g0[: n // 2])
        assert step(g_short, 2) == 0
        assert np.array_equal(dev.to_numpy(w, n), after_one), "a tensor with a short buffer is skipped"
        dev.free(g_short)
    finally:
        for h in (w, m, v):
            dev.free(h)

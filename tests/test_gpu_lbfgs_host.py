"""The mirror of optimizer/lbfgs.go on the GPU: what optimizer/lbfgs_test.go checks (construction,
buffer sizes, counters, statistics, error strings) plus the Step sequence against the oracle."""
import numpy as np
import pytest

from harness import gpu_device
from lbfgs_cases import F, same_bits
from oracle_lib import oracle
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
SHAPES = [[10, 5], [5], [5, 1]]           # lbfgs_test.go:48-52, 348-352


@pytest.fixture(scope="module")
def env():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    dev.lib.gmo_initialize_global_memory_manager(dev.handle)
    mm = dev.lib.gmo_get_global_memory_manager()
    assert mm
    return dev, mm


def make(env, history=5, step=1.0, shapes=SHAPES):
    dev, mm = env
    cfg = pkg.HostLBFGS.default_config()
    opt = pkg.HostLBFGS((history,) + cfg[1:5] + (step,), shapes, mm, dev.handle)
    assert opt.error is None, opt.error
    return opt


def test_creation_and_buffer_sizes(env):                    # lbfgs_test.go:34-99, 334-376
    dev, _ = env
    opt = make(env)
    try:
        assert opt.GetStep() == 0 and opt.history()[:2] == (0, 0)
        assert [opt.buffer_size(k) for k in range(3)] == [200, 20, 20]
        assert opt.buffer_size(3) == -1
        for h in range(5):
            assert opt.buffer("rho", h)
            for k, n in enumerate([50, 5, 5]):
                for which in ("s", "y"):
                    assert not dev.to_numpy(opt.buffer(which, h, k), n).any()
        assert not opt.buffer("s", 5, 0) and opt.buffer("alpha")
        for k, n in enumerate([50, 5, 5]):
            assert not dev.to_numpy(opt.buffer("old_gradient", 0, k), n).any()
            assert not dev.to_numpy(opt.buffer("search_dir", 0, k), n).any()
        assert opt.GetStats() == {"step": 0, "history_size": 5, "history_used": 0, "prev_loss": 0.0}
    finally:
        opt.Cleanup()
        opt.free()


def test_invalid_config(env):                                # lbfgs_test.go:101-129
    dev, mm = env
    cfg = pkg.HostLBFGS.default_config()
    assert pkg.HostLBFGS((0,) + cfg[1:], [[10, 5]], mm, dev.handle).error == "history size must be positive, got 0"
    assert pkg.HostLBFGS((-3,) + cfg[1:], [[10, 5]], mm, dev.handle).error == "history size must be positive, got -3"


def test_set_weight_buffers_command_pool_and_learning_rate(env):     # lbfgs_test.go:164-219, 502-556
    dev, _ = env
    opt = make(env)
    try:
        bufs = [dev.alloc(200), dev.alloc(20), dev.alloc(20)]
        assert opt.SetWeightBuffers(bufs) is None
        assert [opt.buffer("weight", 0, k) for k in range(3)] == bufs
        assert opt.SetWeightBuffers(bufs[:2]) == "expected 3 weight buffers, got 2"
        assert not opt.uses_pooling()
        opt.SetCommandPool(0x2000)
        assert opt.uses_pooling()
        opt.SetCommandPool(0)
        assert not opt.uses_pooling()
        assert opt.UpdateLearningRate(0.01) == "L-BFGS does not use a fixed learning rate; it uses line search"
        # Step validation, lbfgs_test.go:558-576
        assert opt.Step(bufs[:1], 0.5) == "gradient buffers length (1) doesn't match weight buffers length (3)"
        assert opt.GetStep() == 0
        for b in bufs:
            dev.free(b)
    finally:
        opt.Cleanup()
        opt.free()


@pytest.mark.parametrize("pooled", [False, True])
def test_step_sequence_matches_oracle(env, pooled):
    dev, _ = env
    m, step = 3, 0.5
    sizes = [50, 5, 5]
    opt = make(env, history=m, step=step)
    rng = np.random.default_rng(31)
    w0 = [rng.standard_normal(n).astype(F) for n in sizes]
    z = lambda: [np.zeros(n, F) for n in sizes]
    ref = {"w": [t.copy() for t in w0], "old_g": z(), "dir": z(), "s": [z() for _ in range(m)],
           "y": [z() for _ in range(m)], "rho": np.zeros(m, F), "alpha": np.zeros(m, F)}
    wb = [dev.from_numpy(t) for t in w0]
    gb = [dev.alloc(4 * n) for n in sizes]
    try:
        assert opt.SetWeightBuffers(wb) is None
        if pooled:
            opt.SetCommandPool(0x2000)
        count = index = 0
        for k in range(7):
            g = [(rng.standard_normal(n) * 0.1).astype(F) for n in sizes]
            for b, t in zip(gb, g):
                dev.upload(b, t)
            loss = float(F(1.0 / (k + 1)))
            assert opt.Step(gb, loss) is None
            assert oracle().lbfgs_step(ref, g, m, count, index, step, 1)[0] == 0
            index, count = (index + 1) % m, min(count + 1, m)
            assert opt.history() == (count, index, step)
            assert opt.GetStats() == {"step": k + 1, "history_size": m, "history_used": count, "prev_loss": loss}
        for i, n in enumerate(sizes):
            assert same_bits(dev.to_numpy(wb[i], n), ref["w"][i])
            assert same_bits(dev.to_numpy(opt.buffer("old_gradient", 0, i), n), ref["old_g"][i])
            assert same_bits(dev.to_numpy(opt.buffer("search_dir", 0, i), n), ref["dir"][i])
            for h in range(m):
                assert same_bits(dev.to_numpy(opt.buffer("s", h, i), n), ref["s"][h][i])
                assert same_bits(dev.to_numpy(opt.buffer("y", h, i), n), ref["y"][h][i])
        assert same_bits(np.concatenate([dev.to_numpy(opt.buffer("rho", h), 1) for h in range(m)]), ref["rho"])
        assert same_bits(dev.to_numpy(opt.buffer("alpha"), m), ref["alpha"])
    finally:
        for b in wb + gb:
            dev.free(b)
        opt.Cleanup()
        opt.free()


def test_step_error_is_wrapped_like_the_go_code(env):       # lbfgs.go:279-281, bridge.go:2057-2059
    dev, _ = env
    opt = make(env, history=2)
    gb = [dev.alloc(200), dev.alloc(20), dev.alloc(20)]
    try:
        # weight buffers never set: nil handles reach the native step
        assert opt.Step(gb, 1.0) == "L-BFGS step failed: L-BFGS MPSGraph step failed with error code: -8"
        assert opt.GetStep() == 1          # the Go code increments before the native call (lbfgs.go:251)
        assert opt.history()[:2] == (0, 0)
    finally:
        for b in gb:
            dev.free(b)
        opt.Cleanup()
        opt.free()


def test_cleanup_returns_every_buffer_to_the_pool(env):     # lbfgs_test.go:302-332
    dev, mm = env
    import ctypes
    def allocated(pool):
        a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        rc = dev.lib.gmo_pool_stats(mm, pool, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
        return (a.value, b.value) if rc == 0 else (0, 0)
    opt = make(env, history=4)
    avail_mid, alloc_mid = allocated(1024)
    opt.Cleanup()
    avail_after, alloc_after = allocated(1024)
    # 4 x (3 s + 3 y + rho) + alpha + 3 old gradients + 3 directions = 35 buffers, all in the 1 KiB pool
    assert avail_after - avail_mid == 35
    opt.Cleanup()                          # idempotent
    assert allocated(1024) == (avail_after, alloc_after)
    opt.free()

"""Buffers placed at a phase (gm_allocate_buffer_phased): the allocator's contract, and that the optimizers put the
state buffers of large tensors at the phases host/memory_manager.hpp names, pool them by phase and compute the same
bits with them."""
import ctypes

import numpy as np
import pytest

from harness import OracleRun, gpu_device
from oracle_lib import oracle
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
PERIOD = 2 << 20
MIB = 1 << 20
STATE_PHASES = (512 * 1024, 1536 * 1024, 1 * MIB)


@pytest.fixture(scope="module")
def env():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    dev.lib.gmo_initialize_global_memory_manager(dev.handle)
    mm = dev.lib.gmo_get_global_memory_manager()
    assert mm
    return dev, mm


def test_phased_allocation_contract(env):
    dev, _ = env
    lib, D = dev.lib, dev.handle
    for size, phase in ((MIB, 0), (MIB + 4, 256), (5 * MIB + 12, MIB), (64 * MIB, PERIOD - 256), (2 * MIB, MIB + 512 * 1024)):
        h = lib.gm_allocate_buffer_phased(D, size, 1, phase)
        assert h and h % PERIOD == phase, (size, phase, hex(h))
        assert lib.gm_buffer_length(h) == (size + 15) // 16 * 16
        # the whole length is usable and the range checks of the primitives see it
        data = np.arange(size // 4, dtype=np.float32)
        dev.upload(h, data)
        assert np.array_equal(dev.to_numpy(h, size // 4), data)
        assert lib.zero_metal_buffer(D, h, size) == 0
        assert not dev.to_numpy(h, size // 4).any()
        assert lib.zero_metal_buffer(D, h, size + 64) != 0
        other = dev.alloc(size)
        assert lib.copy_buffer_to_buffer_sync(other, h, 0, 0, size) == 0
        assert lib.copy_buffer_to_buffer_sync(other, h, 0, 64, size) != 0          # would run past the end
        dev.free(other)
        lib.deallocate_metal_buffer(h)
        assert lib.gm_buffer_length(h) == 0
    # small requests ignore the phase (nothing to gain, 2 MiB to lose)
    h = lib.gm_allocate_buffer_phased(D, 4096, 1, MIB)
    assert h and lib.gm_buffer_length(h) == 4096
    lib.deallocate_metal_buffer(h)
    for bad in (-256, 100, PERIOD, PERIOD + 256):
        assert lib.gm_allocate_buffer_phased(D, 2 * MIB, 1, bad) == 0
    assert lib.gm_allocate_buffer_phased(0, 2 * MIB, 1, MIB) == 0 and lib.gm_allocate_buffer_phased(D, 0, 1, MIB) == 0


CASES = [
    ("adam", [1e-3, 0.9, 0.999, 1e-8, 1e-4], dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4),
     ["momentum", "variance"], ["m", "v"]),
    ("rmsprop", [0.01, 0.99, 1e-8, 1e-4, 0.9, 1], dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=1e-4, momentum=0.9, centered=True),
     ["squared_grad_avg", "momentum", "gradient_avg"], ["s", "b", "ga"]),
    ("sgd", [0.01, 0.9, 0.0, 0], dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=False), ["momentum"], ["m"]),
    ("adadelta", [0.9, 1e-6, 0.0], dict(rho=0.9, eps=1e-6, weight_decay=0.0), ["squared_grad_avg", "squared_update_avg"], ["s", "a"]),
]
SHAPES = [[1200, 1024], [100], [2048, 1024]]      # 4.9 MB and 8.4 MB: the 16 MiB tier, the smallest that is placed


@pytest.mark.parametrize("kind,cfg,hyper,state_types,names", CASES, ids=[c[0] for c in CASES])
def test_state_buffers_of_large_tensors_sit_at_their_phases(env, kind, cfg, hyper, state_types, names):
    dev, mm = env
    sizes = [int(np.prod(s)) for s in SHAPES]
    rng = np.random.default_rng(5)
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    seen = []
    for round_ in range(2):
        opt = pkg.HostOptimizer(kind, cfg, SHAPES, mm, dev.handle)
        assert opt.error is None, opt.error
        dev.lib.gmo_set_log_progress(opt.handle, 0)
        handles = [[opt.state_buffer(t, k) for k in range(len(sizes))] for t in state_types]
        for j, hs in enumerate(handles):
            assert hs[0] % PERIOD == STATE_PHASES[j] and hs[2] % PERIOD == STATE_PHASES[j], (kind, j, [hex(h) for h in hs])
            assert dev.lib.gm_buffer_length(hs[0]) >= 4 * sizes[0]
        seen.append(handles)
        weights = [dev.from_numpy(w) for w in w0]
        gbufs = [dev.alloc(4 * n) for n in sizes]
        assert opt.SetWeightBuffers(weights) is None
        cpu = OracleRun(kind, hyper, w0)
        for step in range(3):
            grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
            for h, g in zip(gbufs, grads):
                dev.upload(h, g)
            assert opt.Step(gbufs) is None
            cpu.step(grads)
        for k, n in enumerate(sizes):
            assert np.array_equal(dev.to_numpy(weights[k], n).view(np.uint32), cpu.w[k].view(np.uint32)), (kind, k)
            for j, name in enumerate(names):
                assert np.array_equal(dev.to_numpy(handles[j][k], n).view(np.uint32), cpu.state[name][k].view(np.uint32)), (kind, name, k)
        opt.Cleanup()
        opt.free()
        for h in weights + gbufs:
            dev.free(h)
    # the released buffers went back to the pools of their phases: the second optimizer got buffers at the same phases
    # out of the same set of handles
    for j in range(len(state_types)):
        assert {seen[0][j][0], seen[0][j][2]} == {seen[1][j][0], seen[1][j][2]}, (kind, j)


def test_ping_pong_sets_sit_at_their_phases(env):
    dev, mm = env
    sizes = [int(np.prod(s)) for s in SHAPES]
    rng = np.random.default_rng(6)
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    opt = pkg.HostOptimizer("adam", [1e-3, 0.9, 0.999, 1e-8, 0.0], SHAPES, mm, dev.handle)
    assert opt.error is None, opt.error
    weights = [dev.from_numpy(w) for w in w0]
    g16 = [dev.from_numpy((rng.normal(0, 1e-4, n) * 1024.0).astype(np.float16).view(np.uint16)) for n in sizes]
    w16 = [dev.from_numpy(w.astype(np.float16).view(np.uint16)) for w in w0]
    assert opt.SetWeightBuffers(weights) is None
    assert opt.EnableMixedPrecision(1024.0, 2.0, 0.5, 2000) is None
    assert opt.EnablePingPong() is None
    skipped, err = opt.StepAMP(g16, w16)
    assert err is None and not skipped and opt.current_set() == 1
    # the shadow set is current now: its weights start 1 MiB off, its moments at the phases of their counterparts
    for k in (0, 2):
        assert opt.state_buffer("weight", k) % PERIOD == 1 * MIB and opt.state_buffer("weight", k) != weights[k]
        assert opt.state_buffer("momentum", k) % PERIOD == STATE_PHASES[0]
        assert opt.state_buffer("variance", k) % PERIOD == STATE_PHASES[1]
    opt.Cleanup()
    opt.free()
    for h in weights + g16 + w16:
        dev.free(h)

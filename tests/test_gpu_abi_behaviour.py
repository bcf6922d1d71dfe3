"""Return codes, skip rules and launch-shape variants of the step entry points on the GPU."""
import ctypes
import threading

import numpy as np
import pytest

from harness import GpuRun, OracleRun, compare_snapshots, gpu_device
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
ADAM = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


@pytest.fixture
def four(dev):
    """Two tensors with weight / gradient / two state buffers each."""
    sizes = [1000, 37]
    bufs = {k: [dev.from_numpy(np.full(n, v, np.float32)) for n in sizes]
            for k, v in (("w", 1.0), ("g", 0.5), ("a", 0.0), ("b", 0.0))}
    yield sizes, bufs
    for v in bufs.values():
        for h in v:
            dev.free(h)


def arr(handles):
    return pkg.handle_array(handles)


def test_nil_handles_fail_with_the_reference_codes(dev, four):
    sizes, b = four
    lib, D = dev.lib, dev.handle
    bs = pkg.int_array([4 * n for n in sizes])
    hole = [b["a"][0], 0]
    # Adam / NAdam: any nil among w, g, m, v -> -4 and nothing is updated (bridge_optimizer.m:411-414, 2075-2078)
    assert lib.execute_adam_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(hole), arr(b["b"]), 2, bs,
                                          1e-3, 0.9, 0.999, 1e-8, 0.0, 1) == -4
    assert lib.execute_nadam_step_mpsgraph(D, arr(b["w"]), arr(hole), arr(b["a"]), arr(b["b"]), 2, bs,
                                           2e-3, 0.9, 0.999, 1e-8, 0.0, 1) == -4
    assert np.all(dev.to_numpy(b["w"][0], sizes[0]) == 1.0)
    assert b"nil" in lib.gm_last_error()
    # RMSProp: -4 required, -5 momentum > 0 without buffer, -6 centered without buffer (.m:736-753)
    assert lib.execute_rmsprop_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(hole), None, None, 2, bs,
                                             0.01, 0.99, 1e-8, 0.0, 0.0, False, 1) == -4
    assert lib.execute_rmsprop_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), None, None, 2, bs,
                                             0.01, 0.99, 1e-8, 0.0, 0.9, False, 1) == -5
    assert lib.execute_rmsprop_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), arr(b["b"]), arr(hole), 2, bs,
                                             0.01, 0.99, 1e-8, 0.0, 0.9, True, 1) == -6
    assert lib.execute_rmsprop_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), None, arr(hole), 2, bs,
                                             0.01, 0.99, 1e-8, 0.0, 0.0, True, 1) == -6
    assert np.all(dev.to_numpy(b["w"][0], sizes[0]) == 1.0)
    # mixed precision: -16 without a loss-scale state, -4 for a nil handle
    sk = ctypes.c_int()
    assert lib.execute_adam_amp_step(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), arr(b["b"]), None, 2, bs,
                                     1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0, ctypes.byref(sk), None, None) == -16
    amp = lib.gm_amp_state_create(D, 65536.0, 2.0, 0.5, 2000)
    assert lib.execute_adam_amp_step(D, arr(b["w"]), arr(hole), arr(b["a"]), arr(b["b"]), None, 2, bs,
                                     1e-3, 0.9, 0.999, 1e-8, 0.0, 1, amp, ctypes.byref(sk), None, None) == -4
    lib.gm_amp_state_destroy(amp)


def test_sgd_and_adagrad_skip_tensors_with_nil_handles(dev, four):
    """bridge_optimizer.m:199-202: a nil weight or gradient skips that tensor, the call succeeds."""
    sizes, b = four
    lib, D = dev.lib, dev.handle
    bs = pkg.int_array([4 * n for n in sizes])
    assert lib.execute_sgd_step_mpsgraph(D, arr(b["w"]), arr([b["g"][0], 0]), None, 2, bs, 0.5, 0.0, 0.0, 0, 1) == 0
    assert np.all(dev.to_numpy(b["w"][0], sizes[0]) == 0.75)       # 1 - 0.5 * 0.5
    assert np.all(dev.to_numpy(b["w"][1], sizes[1]) == 1.0)        # skipped
    # momentum requested but one tensor has no momentum buffer: that tensor takes the vanilla rule
    assert lib.execute_sgd_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr([b["a"][0], 0]), 2, bs,
                                         0.5, 0.9, 0.0, 0, 2) == 0
    assert np.all(dev.to_numpy(b["a"][0], sizes[0]) == 0.5)        # m = 0.9 * 0 + g
    assert np.all(dev.to_numpy(b["w"][1], sizes[1]) == 0.75)
    assert lib.execute_adagrad_step_mpsgraph(D, arr([0, b["w"][1]]), arr(b["g"]), arr(b["b"]), 2, bs,
                                             0.01, 1e-10, 0.0) == 0
    assert np.all(dev.to_numpy(b["b"][0], sizes[0]) == 0.0)        # skipped: state untouched
    assert np.all(dev.to_numpy(b["b"][1], sizes[1]) == 0.25)       # s = g^2


def test_tensor_longer_than_its_allocation_is_skipped(dev, four):
    """bridge_optimizer.m:427-436: a buffer shorter than buffer_sizes[i] skips the tensor (no fault)."""
    sizes, b = four
    lib, D = dev.lib, dev.handle
    too_big = pkg.int_array([4 * sizes[0], 4 * 1000])              # second tensor really has 37 elements
    assert lib.execute_adam_step_mpsgraph(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), arr(b["b"]), 2, too_big,
                                          1e-3, 0.9, 0.999, 1e-8, 0.0, 1) == 0
    assert np.all(dev.to_numpy(b["w"][1], sizes[1]) == 1.0)
    assert not np.all(dev.to_numpy(b["w"][0], sizes[0]) == 1.0)


def test_pooled_adam_and_queue_handles(dev, four):
    sizes, b = four
    lib, D = dev.lib, dev.handle
    bs = pkg.int_array([4 * n for n in sizes])
    q = lib.create_command_queue(D)
    assert q != 0
    assert lib.execute_adam_step_mpsgraph_pooled(D, arr(b["w"]), arr(b["g"]), arr(b["a"]), arr(b["b"]), 2, bs,
                                                 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, q) == 0
    assert not np.all(dev.to_numpy(b["w"][0], sizes[0]) == 1.0)
    lib.release_command_queue(q)
    lib.release_command_queue(0)


@pytest.mark.parametrize("chunk,nt,vec,lanes", [(0, 1, 2, 0), (0, 1, 4, 0), (0, 0, 1, 0), (256, 1, 1, 0), (1024, 0, 4, 0),
                                                (4096, 1, 2, 0), (65536, 1, 4, 0), (0, 1, 1, 128), (256, 1, 1, 128),
                                                (4096, 1, 2, 256), (0, 0, 4, 128), (0, 1, 0, 256), (0, 1, 0, 128)])
def test_launch_shape_variants_are_bit_identical(dev, chunk, nt, vec, lanes):
    """Every selectable launch shape (lane width 1 / 2 / 4, workgroups of 128 / 256 lanes, chunk size,
    non-temporal hint) computes the same bits, including on streams that are only 4-byte aligned (handles
    offset into a parent buffer)."""
    lib = dev.lib
    rng = np.random.default_rng(5)
    sizes = [1, 2, 3, 5, 255, 257, 1023, 4097, 70001, 262147]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    assert lib.gm_set_tuning(dev.handle, chunk, nt, vec) == 0
    assert lib.gm_set_workgroup_lanes(dev.handle, lanes) == 0
    try:
        for rule, hyper in (("adam", ADAM), ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=False)),
                            ("adadelta", dict(rho=0.9, eps=1e-6, weight_decay=0.0))):
            gpu, cpu = GpuRun(dev, rule, hyper, w), OracleRun(rule, hyper, w)
            for _ in range(3):
                grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
                gpu.step(grads)
                cpu.step(grads)
            compare_snapshots(gpu.snapshot(), cpu.snapshot(), 0, f"{rule} chunk={chunk} nt={nt} vec={vec} lanes={lanes}")
            gpu.close()
        # misaligned views: element 1 of each parent buffer (4-byte aligned only; not registry handles)
        n = 5000
        parents = {k: dev.from_numpy(np.zeros(n + 1, np.float32)) for k in "wgmv"}
        host = {k: np.zeros(n, np.float32) for k in "wgmv"}
        host["w"][:] = rng.normal(0, 0.02, n)
        host["g"][:] = rng.normal(0, 1e-3, n)
        for k in "wg":
            dev.upload(parents[k], np.concatenate([[np.float32(7)], host[k]]).astype(np.float32))
        views = {k: pkg.handle_array([parents[k] + 4]) for k in "wgmv"}
        assert lib.execute_adam_step_mpsgraph(dev.handle, views["w"], views["g"], views["m"], views["v"], 1,
                                              pkg.int_array([4 * n]), 1e-3, 0.9, 0.999, 1e-8, 1e-4, 1) == 0
        cpu = OracleRun("adam", ADAM, [host["w"]])
        cpu.step([host["g"]])
        got = dev.to_numpy(parents["w"], n + 1)
        assert got[0] == 7 and np.array_equal(got[1:].view(np.uint32), cpu.w[0].view(np.uint32))
        for h in parents.values():
            dev.free(h)
    finally:
        assert lib.gm_set_tuning(dev.handle, 0, -1, 0) == 0
        assert lib.gm_set_workgroup_lanes(dev.handle, 0) == 0
    assert lib.gm_set_workgroup_lanes(dev.handle, 64) == -1 and lib.gm_set_workgroup_lanes(dev.handle, 192) == -1
    assert lib.gm_set_tuning(dev.handle, 1000, 1, 1) == -1 and lib.gm_set_tuning(dev.handle, 0, 1, 3) == -1
    assert lib.gm_set_tuning(dev.handle, 768, 1, 1) == -1          # 3 slices: not a power of two


def test_two_threads_step_two_optimizers(dev):
    """Entry points may be called from any thread; two parameter lists stepped concurrently stay exact."""
    rng = np.random.default_rng(9)
    sizes = [30000, 513, 70000]
    runs, oracles, grads = [], [], []
    for t in range(2):
        w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
        runs.append(GpuRun(dev, "adam", ADAM, w))
        oracles.append(OracleRun("adam", ADAM, w))
        grads.append([[rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes] for _ in range(20)])
    errors = []

    def work(t):
        try:
            for g in grads[t]:
                runs[t].step(g)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for t in range(2):
        for g in grads[t]:
            oracles[t].step(g)
        compare_snapshots(runs[t].snapshot(), oracles[t].snapshot(), 0, f"thread {t}")
        runs[t].close()


def test_ordering_against_a_callers_stream(dev):
    """Gradients produced on the caller's own HIP stream, the step on the library's stream, the
    result consumed on the caller's stream again: ordered by gm_wait_for_stream / gm_signal_stream
    alone, no host wait in between."""
    hip = ctypes.CDLL("/opt/rocm/lib/libamdhip64.so")
    hip.hipStreamCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
    hip.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
    hip.hipHostMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t, ctypes.c_uint]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipHostFree.argtypes = [ctypes.c_void_p]
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream), 1) == 0          # hipStreamNonBlocking
    n = 8_000_000
    nbytes = 4 * n
    pin_g, pin_out = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipHostMalloc(ctypes.byref(pin_g), nbytes, 0) == 0
    assert hip.hipHostMalloc(ctypes.byref(pin_out), nbytes, 0) == 0
    g = np.ctypeslib.as_array(ctypes.cast(pin_g, ctypes.POINTER(ctypes.c_float)), shape=(n,))
    out = np.ctypeslib.as_array(ctypes.cast(pin_out, ctypes.POINTER(ctypes.c_float)), shape=(n,))
    rng = np.random.default_rng(21)
    w0 = rng.normal(0, 0.02, n).astype(np.float32)
    w, gbuf = dev.from_numpy(w0), dev.alloc(nbytes)
    lib, D = dev.lib, dev.handle
    bs = pkg.int_array([nbytes])
    want = w0.copy()
    try:
        for step in range(3):
            g[:] = rng.normal(0, 1e-2, n).astype(np.float32)
            want = want - np.float32(0.1) * g
            assert hip.hipMemcpyAsync(gbuf, pin_g, nbytes, 1, stream) == 0       # H2D on the caller's stream
            assert lib.gm_wait_for_stream(D, stream) == 0
            assert lib.execute_sgd_step_mpsgraph(D, arr([w]), arr([gbuf]), None, 1, bs, 0.1, 0.0, 0.0, 0, step + 1) == 0
            assert lib.gm_signal_stream(D, stream) == 0
            assert hip.hipMemcpyAsync(pin_out, w, nbytes, 2, stream) == 0        # D2H on the caller's stream
            assert hip.hipStreamSynchronize(stream) == 0                         # the pinned gradient is reused next
            assert np.array_equal(out.view(np.uint32), want.view(np.uint32)), step
        assert lib.gm_wait_for_stream(0, stream) == -1
    finally:
        dev.synchronize()
        hip.hipStreamDestroy(stream)
        hip.hipHostFree(pin_g)
        hip.hipHostFree(pin_out)
        dev.free(w)
        dev.free(gbuf)


def test_gradient_handles_that_change_every_step(dev):
    """A caller whose gradient buffers are new on every step (more distinct sets than the plan cache holds)
    makes the library rebuild its chunk table each time and evict the oldest plan: every step stays exact."""
    rng = np.random.default_rng(23)
    sizes = [70001, 5, 4097, 262147, 1023]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    gpu, cpu = GpuRun(dev, "adam", ADAM, w), OracleRun("adam", ADAM, w)
    sets = 24
    grads = [[rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes] for _ in range(sets)]
    handles = [[dev.from_numpy(g) for g in gs] for gs in grads]
    own = gpu.c_g
    try:
        for t in range(3 * sets):
            k = (7 * t) % sets
            gpu.c_g = pkg.handle_array(handles[k])
            gpu.launch()
            cpu.step(grads[k])
            if t % 17 == 0 or t == 3 * sets - 1:
                compare_snapshots(gpu.snapshot(), cpu.snapshot(), 0, f"step {t}")
    finally:
        gpu.c_g = own
        gpu.close()
        for hs in handles:
            for h in hs:
                dev.free(h)

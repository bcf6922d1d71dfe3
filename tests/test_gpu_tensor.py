"""memory.Tensor on the GPU (the Go tests for it are all skipped in the reference,
memory/memory_test.go:315-683) and the engine's precomputed-gradient step."""
import ctypes

import numpy as np
import pytest

from harness import OracleRun, gpu_device
from oracle_lib import oracle
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
vp = ctypes.c_void_p
F32, I32, F16 = 0, 1, 2
GPU = 1


@pytest.fixture(scope="module")
def env():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    dev.lib.gmo_initialize_global_memory_manager(dev.handle)
    return dev


def new_tensor(lib, shape, dtype=F32):
    t = lib.gmo_tensor_new(pkg.int_array(shape), len(shape), dtype, GPU)
    assert t, lib.gmo_last_error()
    return t


def fill(lib, t, data):
    a = np.ascontiguousarray(data, dtype=np.float32)
    assert lib.gmo_tensor_copy_float32_data(t, a.ctypes.data_as(vp), a.size) == 0, lib.gmo_last_error()


def read(lib, t, n):
    out = np.empty(n, np.float32)
    assert lib.gmo_tensor_to_float32_slice(t, out.ctypes.data_as(vp), n) == n, lib.gmo_last_error()
    return out


def test_tensor_lifecycle_and_reference_counting(env):
    lib = env.lib
    t = new_tensor(lib, [3, 4])
    assert lib.gmo_tensor_size(t) == 48 and lib.gmo_tensor_ref_count(t) == 1 and lib.gmo_tensor_buffer(t) != 0
    assert lib.gmo_tensor_retain(t) == t and lib.gmo_tensor_ref_count(t) == 2
    lib.gmo_tensor_release(t)
    assert lib.gmo_tensor_ref_count(t) == 1 and lib.gmo_tensor_buffer(t) != 0
    lib.gmo_tensor_release(t)
    assert lib.gmo_tensor_ref_count(t) == 0 and lib.gmo_tensor_buffer(t) == 0
    assert lib.gmo_tensor_retain(t) == 0          # Go panics with "tensor already released"
    lib.gmo_tensor_release(t)                     # releasing again is a no-op
    lib.gmo_tensor_free(t)


def test_copy_data_and_errors(env):
    lib = env.lib
    t = new_tensor(lib, [2, 5])
    data = np.arange(10, dtype=np.float32) * np.float32(0.25)
    fill(lib, t, data)
    assert np.array_equal(read(lib, t, 10), data)
    assert lib.gmo_tensor_copy_float32_data(t, data.ctypes.data_as(vp), 9) == -1
    assert lib.gmo_last_error().decode() == "data length 9 doesn't match tensor shape [2 5] (expected 10 elements)"
    h = new_tensor(lib, [2, 5], F16)
    assert lib.gmo_tensor_copy_float32_data(h, data.ctypes.data_as(vp), 10) == -1
    assert lib.gmo_last_error().decode() == "tensor data type is 2, expected Float32 (0)"
    for x in (t, h):
        lib.gmo_tensor_release(x)
        lib.gmo_tensor_free(x)


def test_convert_to_and_copy_from(env):
    lib = env.lib
    n = 4099
    rng = np.random.default_rng(2)
    data = (rng.standard_normal(n) * 3).astype(np.float32)
    t = new_tensor(lib, [n])
    fill(lib, t, data)
    same = lib.gmo_tensor_convert_to(t, F32)              # same type: retained, not copied
    assert same == t and lib.gmo_tensor_ref_count(t) == 2
    lib.gmo_tensor_release(t)
    half = lib.gmo_tensor_convert_to(t, F16)
    assert half and half != t and lib.gmo_tensor_dtype(half) == F16 and lib.gmo_tensor_size(half) == 2 * n
    bits = env.to_numpy(lib.gmo_tensor_buffer(half), n, np.uint16)
    assert np.array_equal(bits, oracle().f32_to_f16(data))
    back = lib.gmo_tensor_convert_to(half, F32)
    assert np.array_equal(read(lib, back, n), oracle().f16_to_f32(bits))
    assert lib.gmo_tensor_convert_to(t, I32) == 0         # only fp32 <-> fp16 is supported (bridge_memory.m:413-416)
    assert lib.gmo_last_error().decode() == \
        "failed to convert tensor type: failed to convert tensor type with error code: -3"
    # CopyFrom: device-to-device, with the reference's compatibility checks (tensor.go:248-291)
    dst = new_tensor(lib, [n])
    assert lib.gmo_tensor_copy_from(dst, t) == 0
    assert np.array_equal(read(lib, dst, n), data)
    other = new_tensor(lib, [n, 1])
    assert lib.gmo_tensor_copy_from(other, t) == -1
    assert lib.gmo_last_error().decode() == f"tensor shape dimensions don't match: dst [{n} 1] vs src [{n}]"
    assert lib.gmo_tensor_copy_from(half, t) == -1
    assert lib.gmo_last_error().decode() == "tensor data types don't match: dst 2 vs src 0"
    for x in (t, half, back, dst, other):
        lib.gmo_tensor_release(x)
        lib.gmo_tensor_free(x)


def test_execute_step_with_precomputed_gradients(env):
    """engine/training_engine.go:100-147 with tensors from the pool, against the oracle."""
    dev, lib = env, env.lib
    mm = lib.gmo_get_global_memory_manager()
    shapes = [[64, 32], [32], [1000]]
    sizes = [int(np.prod(s)) for s in shapes]
    rng = np.random.default_rng(4)
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)
    opt = pkg.HostOptimizer("adam", [1e-3, 0.9, 0.999, 1e-8, 0.0], shapes, mm, dev.handle)
    assert opt.error is None
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    wt = [new_tensor(lib, s) for s in shapes]
    gt = [new_tensor(lib, s) for s in shapes]
    for t, w in zip(wt, w0):
        fill(lib, t, w)
    cpu = OracleRun("adam", hyper, w0)
    for _ in range(4):
        grads = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
        for t, g in zip(gt, grads):
            fill(lib, t, g)
        assert lib.gmo_execute_step_with_precomputed_gradients(opt.handle, pkg.handle_array(wt), 3,
                                                               pkg.handle_array(gt), 3) == 0, lib.gmo_last_error()
        cpu.step(grads)
    assert opt.GetStepCount() == 4
    for t, n, ref in zip(wt, sizes, cpu.w):
        assert np.array_equal(read(lib, t, n).view(np.uint32), ref.view(np.uint32))
    opt.Cleanup()
    opt.free()
    for x in wt + gt:
        lib.gmo_tensor_release(x)
        lib.gmo_tensor_free(x)


def test_tensor_string(env):                                  # memory_test.go:608-629 (skipped there: needs a GPU)
    lib = env.lib
    t = new_tensor(lib, [2, 3])
    p = lib.gmo_tensor_string(t)
    text = ctypes.string_at(p).decode()
    lib.gmo_free_string(p)
    assert text.startswith("Tensor{shape=[2 3], dtype=0, device=1, refs=1, gen=") and text.endswith("}")
    lib.gmo_tensor_release(t)
    lib.gmo_tensor_free(t)


def test_tensor_with_a_zero_dimension(env):                   # memory_test.go:697-720 (skipped there)
    lib = env.lib
    t = new_tensor(lib, [0, 5])
    assert lib.gmo_tensor_size(t) == 0
    out = np.empty(4, np.float32)
    assert lib.gmo_tensor_to_float32_slice(t, out.ctypes.data_as(vp), 4) < 0
    assert lib.gmo_last_error().decode() == "tensor has invalid shape: [0 5]"       # tensor.go:352-354
    lib.gmo_tensor_release(t)
    lib.gmo_tensor_free(t)


def test_reference_counting_from_many_threads(env):           # memory_test.go:417-455 (skipped there)
    import threading
    lib = env.lib
    t = new_tensor(lib, [10, 10])
    workers, rounds = 10, 100

    def work():
        for _ in range(rounds):
            assert lib.gmo_tensor_retain(t) == t
            lib.gmo_tensor_release(t)

    threads = [threading.Thread(target=work) for _ in range(workers)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert lib.gmo_tensor_ref_count(t) == 1
    lib.gmo_tensor_release(t)
    assert lib.gmo_tensor_ref_count(t) == 0
    lib.gmo_tensor_free(t)

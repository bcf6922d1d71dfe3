"""Headline configuration at full size: Adam with L2 weight decay 1e-4 (applied in the reference's
order) over 1,012,301,824 fp32 parameters in 400 transformer-block tensors, 20 steps, against the
CPU oracle.  Bit-exact (the stated tolerance is <= 2 ulp).  The other five rules run over the same
list for three steps."""
import os

import numpy as np
import pytest

from harness import GpuRun, OracleRun, gpu_device, progress, states_for
from workloads import transformer_block_sizes

pytestmark = pytest.mark.gpu
NTHREADS = min(16, os.cpu_count() or 1)


def run_full_size(rule, hyper, steps, checkpoints, sizes=None):
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    sizes = transformer_block_sizes() if sizes is None else sizes
    # weights and two gradient sets are generated on the device and read back for the oracle
    lib, D = dev.lib, dev.handle
    gpu = GpuRun(dev, rule, hyper, [np.empty(0, np.float32)] * 0)   # placeholder object, filled below
    gpu.sizes, gpu.n = sizes, len(sizes)
    gpu.w = [dev.alloc(4 * s) for s in sizes]
    gpu.state = {name: [dev.alloc(4 * s, zero=True) for s in sizes] for name in states_for(rule, hyper)}
    grads_dev = [[dev.alloc(4 * s) for s in sizes] for _ in range(2)]
    for k, s in enumerate(sizes):
        assert lib.gm_fill_normal_f32(D, gpu.w[k], s, 1000 + k, 0.0, 0.02) == 0
        for j in range(2):
            assert lib.gm_fill_normal_f32(D, grads_dev[j][k], s, 5000 + 1000 * j + k, 0.0, 1e-4) == 0
    gpu.byte_sizes = gpu.pkg.int_array([4 * s for s in sizes])
    gpu.c_w = gpu.pkg.handle_array(gpu.w)
    gpu.c_state = {k: gpu.pkg.handle_array(v) for k, v in gpu.state.items()}
    c_grads = [gpu.pkg.handle_array(g) for g in grads_dev]
    w_host = [dev.to_numpy(h, s) for h, s in zip(gpu.w, sizes)]
    g_host = [[dev.to_numpy(h, s) for h, s in zip(gs, sizes)] for gs in grads_dev]
    assert abs(float(np.std(w_host[0])) - 0.02) < 1e-3
    cpu = OracleRun(rule, hyper, w_host, nthreads=NTHREADS)
    del w_host
    try:
        for step in range(1, steps + 1):
            gpu.c_g = c_grads[step % 2]
            gpu.g = grads_dev[step % 2]
            gpu.launch()
            cpu.step(g_host[step % 2])
            if step in checkpoints:
                progress(f"config 5 list, {rule}: comparing after step {step}")
                for name, handles in [("w", gpu.w)] + sorted(gpu.state.items()):
                    ref = cpu.w if name == "w" else cpu.state[name]
                    for k, s in enumerate(sizes):
                        got = dev.to_numpy(handles[k], s)
                        assert np.array_equal(got.view(np.uint32), ref[k].view(np.uint32)), (rule, step, name, k)
    finally:
        for h in gpu.w + [x for hs in gpu.state.values() for x in hs] + grads_dev[0] + grads_dev[1]:
            dev.free(h)


def test_config5_adam_weight_decay_1b_params_20_steps():
    run_full_size("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4), 20, (1, 10, 20))


@pytest.mark.parametrize("rule,hyper", [
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=1e-4, nesterov=True)),
    ("rmsprop", dict(lr=1e-3, alpha=0.99, eps=1e-8, weight_decay=1e-4, momentum=0.9, centered=True)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=1e-4)),
    ("adadelta", dict(rho=0.9, eps=1e-6, weight_decay=1e-4)),
    ("nadam", dict(lr=2e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
], ids=lambda x: x if isinstance(x, str) else "")
def test_every_other_rule_over_the_1b_list(rule, hyper):
    """The other five kernels on the headline list's grid (3.9 million workgroups in two segments), weight decay
    on, the widest variant of each rule (Nesterov; RMSProp with momentum and centering: nine streams): three
    steps, compared after the last one."""
    run_full_size(rule, hyper, 3, (3,))


def test_tensors_of_the_largest_size_the_abi_can_name():
    """`sizes` are C ints in bytes, so the longest tensor a call can name has 2^29 - 1 elements (2^31 - 4 bytes, which
    the allocator rounds up to 2^31).  Two of them with a five-element tensor in between: every byte offset above
    2^31 inside the second large buffer, its last (odd) element and the tiny tensor's neighbours are the oracle's
    after two steps of Adam with weight decay."""
    top = 2 ** 29 - 1
    run_full_size("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4), 2, (2,),
                  sizes=[top, 5, top])


def test_adam_over_the_1b_list_through_the_optimizer_object():
    """The same list through the mirror of the Go `optimizer` package: state buffers from the pooled memory manager
    (800 of them, the large ones placed at their phases), Step on the caller's weight and gradient buffers, three
    steps, weights and both moments compared with the oracle."""
    from __graft_entry__ import load_package
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    pkg = load_package()
    lib, D = dev.lib, dev.handle
    lib.gmo_initialize_global_memory_manager(D)
    mm = lib.gmo_get_global_memory_manager()
    assert mm
    sizes = transformer_block_sizes()
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    opt = pkg.HostOptimizer("adam", [1e-3, 0.9, 0.999, 1e-8, 1e-4], [[s] for s in sizes], mm, D)
    assert opt.error is None, opt.error
    w = [dev.alloc(4 * s) for s in sizes]
    g = [dev.alloc(4 * s) for s in sizes]
    try:
        for k, s in enumerate(sizes):
            assert lib.gm_fill_normal_f32(D, w[k], s, 1000 + k, 0.0, 0.02) == 0
            assert lib.gm_fill_normal_f32(D, g[k], s, 5000 + k, 0.0, 1e-4) == 0
        big = max(range(len(sizes)), key=lambda k: sizes[k])
        assert opt.state_buffer("momentum", big) % (2 << 20) == 512 << 10
        assert opt.state_buffer("variance", big) % (2 << 20) == 1536 << 10
        w_host = [dev.to_numpy(h, s) for h, s in zip(w, sizes)]
        g_host = [dev.to_numpy(h, s) for h, s in zip(g, sizes)]
        cpu = OracleRun("adam", hyper, w_host, nthreads=NTHREADS)
        del w_host
        assert opt.SetWeightBuffers(w) is None
        for _ in range(3):
            assert opt.Step(g) is None
            cpu.step(g_host)
        assert opt.GetStepCount() == 3
        progress("config 5 list through the optimizer object: comparing after step 3")
        for name, ref, handle_of in (("w", cpu.w, lambda k: w[k]), ("m", cpu.state["m"], lambda k: opt.state_buffer("momentum", k)),
                                     ("v", cpu.state["v"], lambda k: opt.state_buffer("variance", k))):
            for k, s in enumerate(sizes):
                got = dev.to_numpy(handle_of(k), s)
                assert np.array_equal(got.view(np.uint32), ref[k].view(np.uint32)), (name, k)
    finally:
        opt.Cleanup()
        opt.free()
        for h in w + g:
            dev.free(h)


def test_one_pass_mixed_precision_over_the_1b_list_through_the_optimizer_object():
    """EnableMixedPrecision + EnablePingPong on the optimizer object over the same list: the second set of weights and
    moments from the pool, four StepAMP calls of which the second is dropped (a NaN in one gradient), the current
    set and the fp16 copy compared with the oracle."""
    import ctypes
    from __graft_entry__ import load_package
    from oracle_lib import oracle
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    pkg = load_package()
    lib, D = dev.lib, dev.handle
    lib.gmo_initialize_global_memory_manager(D)
    mm = lib.gmo_get_global_memory_manager()
    sizes = transformer_block_sizes()
    n, total = len(sizes), sum(sizes)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)
    opt = pkg.HostOptimizer("adam", [1e-3, 0.9, 0.999, 1e-8, 1e-4], [[s] for s in sizes], mm, D)
    assert opt.error is None, opt.error
    w = [dev.alloc(4 * s) for s in sizes]
    d_g16, d_w16 = dev.alloc(2 * total), dev.alloc(2 * total)
    g16 = [d_g16 + 2 * int(o) for o in offsets[:-1]]
    w16 = [d_w16 + 2 * int(o) for o in offsets[:-1]]
    try:
        for k, s in enumerate(sizes):
            assert lib.gm_fill_normal_f32(D, w[k], s, 1000 + k, 0.0, 0.02) == 0
            assert lib.convert_tensor_type(w[k], w16[k], pkg.int_array([s]), 1, 0, 2, D) == 0     # the copy starts as half(w)
        assert opt.SetWeightBuffers(w) is None
        assert opt.EnableMixedPrecision(65536.0, 2.0, 0.5, 2000) is None
        assert opt.EnablePingPong() is None
        w_host = [dev.to_numpy(h, s) for h, s in zip(w, sizes)]
        m_host = [np.zeros(s, np.float32) for s in sizes]
        v_host = [np.zeros(s, np.float32) for s in sizes]
        w16_host = [a.astype(np.float16).view(np.uint16) for a in w_host]
        st = oracle().amp_state(65536.0, 2.0, 0.5, 2000)
        words = np.empty((2 * total + 3) // 4, np.uint32)
        for step in range(4):
            assert lib.gm_fill_normal_f16(D, d_g16, total, 0xABC000 + step, 0.0, 1e-4, float(st.scale)) == 0
            if step == 1:
                bad = dev.from_numpy(np.array([0x7E00, 0], np.uint16))
                assert lib.copy_buffer_to_buffer_sync(bad, d_g16, 0, 2 * (int(offsets[33]) + 77), 2) == 0
                dev.free(bad)
            assert lib.copy_metal_buffer_to_int32_array(d_g16, words.ctypes.data_as(ctypes.c_void_p), words.size) == 0
            halves = words.view(np.uint16)
            skipped, err = opt.StepAMP(g16, w16)
            assert err is None, err
            want = oracle().adam_amp(w_host, [halves[offsets[k]:offsets[k + 1]] for k in range(n)], m_host, v_host, w16_host,
                                     state=st, nthreads=NTHREADS, **hyper)
            assert int(skipped) == want == (1 if step == 1 else 0)
        assert opt.GetStepCount() == 3 and opt.current_set() == 1
        progress("config 5 list, one-pass mixed precision through the optimizer object: comparing")
        for name, ref in (("weight", w_host), ("momentum", m_host), ("variance", v_host)):
            for k, s in enumerate(sizes):
                got = dev.to_numpy(opt.state_buffer(name, k), s)
                assert np.array_equal(got.view(np.uint32), ref[k].view(np.uint32)), (name, k)
        got16 = dev.to_numpy(d_w16, total, np.uint16)
        for k in range(n):
            assert np.array_equal(got16[offsets[k]:offsets[k + 1]], w16_host[k]), ("w16", k)
    finally:
        opt.Cleanup()
        opt.free()
        for h in w + [d_g16, d_w16]:
            dev.free(h)

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


def run_full_size(rule, hyper, steps, checkpoints):
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    sizes = transformer_block_sizes()
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

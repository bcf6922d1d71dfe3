"""GPU parity: libgometal_hip.so (through the C ABI) against the CPU oracle and the golden
vectors.  fp32 rules are required to be BIT-IDENTICAL to the oracle (the stated tolerance is
<= 2 ulp after 10 steps; the kernels evaluate the same IEEE operations in the same order, so
the tests hold them to 0 ulp and fail on any difference)."""
import json
import os

import numpy as np
import pytest

from harness import GpuRun, OracleRun, compare_snapshots, gpu_device
from workloads import cnn_sizes, ragged_sizes

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "optimizer_kat.json")) as f:
    KAT = json.load(f)

NTHREADS = min(16, os.cpu_count() or 1)


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


def f32(bits):
    return np.array(bits, dtype=np.uint32).view(np.float32).copy()


@pytest.mark.parametrize("case", KAT["cases"], ids=[c["name"] for c in KAT["cases"]])
def test_golden_vectors(dev, case):
    """Known-answer vectors (exact-rational evaluator), incl. the reference's own test inputs."""
    run = GpuRun(dev, case["rule"], case["hyper"], [f32(case["w0"])])
    run.step_count = case["first_step"] - 1
    try:
        for k, gbits in enumerate(case["grads"]):
            run.step([f32(gbits)])
            got = run.snapshot()
            for key in got:
                assert got[key][0].view(np.uint32).tolist() == case["expect"][k][key], (case["name"], k, key)
    finally:
        run.close()


def run_both(dev, rule, hyper, weights, grad_fn, steps, check_every=1, nthreads=NTHREADS):
    gpu = GpuRun(dev, rule, hyper, weights)
    cpu = OracleRun(rule, hyper, weights, nthreads=nthreads)
    try:
        for k in range(steps):
            grads = grad_fn(k)
            gpu.step(grads)
            cpu.step(grads)
            if (k + 1) % check_every == 0 or k == steps - 1:
                compare_snapshots(gpu.snapshot(), cpu.snapshot(), max_ulp=0, context=f"{rule} step {k + 1}")
    finally:
        gpu.close()


def test_config1_adam_flat_1m(dev):
    """One flat tensor of 1,048,576 params, N(0, 0.02); grads N(0, 1e-2); 10 steps, p/m/v after every step."""
    rng = np.random.default_rng(0x6D657461 + 1)
    n = 1 << 20
    w = [rng.normal(0, 0.02, n).astype(np.float32)]
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)
    run_both(dev, "adam", hyper, w, lambda k: [rng.normal(0, 1e-2, n).astype(np.float32)], steps=10)


@pytest.mark.parametrize("rule,hyper", [
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=False)),
    ("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)),
])
def test_config2_cnn_parameter_list(dev, rule, hyper):
    """16 tensors / 1,143,690 params, weights N(0, 0.02), grads N(0, 1e-3), 100 steps."""
    rng = np.random.default_rng(0x6D657461 + 2)
    sizes = cnn_sizes()
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    run_both(dev, rule, hyper, w, lambda k: [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes],
             steps=100, check_every=10)


CONFIG3 = [
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0, centered=False)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=0.0)),
    ("adadelta", dict(rho=0.9, eps=1e-6, weight_decay=0.0)),
    ("nadam", dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)),
]


@pytest.fixture(scope="module")
def config3_data():
    """25M params in 160 ragged tensors; a pool of 4 heavy-tailed gradient sets that the
    50 steps cycle through (N(0, 1e-3), a seeded 1% of elements x100)."""
    sizes = ragged_sizes()
    rng = np.random.default_rng(0x6D657461 + 30)
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    pool = []
    for _ in range(4):
        gs = []
        for n in sizes:
            g = rng.normal(0, 1e-3, n).astype(np.float32)
            g[rng.random(n) < 0.01] *= np.float32(100.0)
            gs.append(g)
        pool.append(gs)
    return sizes, w, pool


@pytest.mark.parametrize("rule,hyper", CONFIG3, ids=[c[0] for c in CONFIG3])
def test_config3_ragged_25m(dev, config3_data, rule, hyper):
    sizes, w, pool = config3_data
    run_both(dev, rule, hyper, w, lambda k: pool[k % len(pool)], steps=50, check_every=25)


@pytest.mark.parametrize("rule,hyper", [
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=1e-4, momentum=0.9, centered=True)),
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.9, centered=False)),
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0, centered=True)),
    ("sgd", dict(lr=0.01, momentum=0.0, weight_decay=5e-4, nesterov=False)),
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=5e-4, nesterov=True)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=1e-3)),
    ("adadelta", dict(rho=0.95, eps=1e-6, weight_decay=1e-3)),
    ("nadam", dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
    ("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
])
def test_variants_and_ragged_edges(dev, rule, hyper):
    """Every rule variant over sizes that exercise the vector body, the scalar tail, one-element
    tensors, an empty tensor, workgroup-slice boundaries (256 elements) and chunk boundaries
    (16384 elements)."""
    rng = np.random.default_rng(99)
    sizes = [1, 2, 3, 4, 5, 0, 63, 64, 65, 255, 256, 257, 1023, 1025, 4095, 4097, 16383, 16384, 16385, 65535, 65537,
             131072 + 7, 300001]
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    run_both(dev, rule, hyper, w, lambda k: [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes],
             steps=6, check_every=3, nthreads=1)


@pytest.mark.parametrize("rule,hyper", [
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=False)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=0.0)),
    ("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
])
def test_lists_of_many_tiny_tensors(dev, rule, hyper):
    """Hundreds of tensors of 1 to 700 elements (biases, normalisation scales): the planner then cuts the list
    into 256-element chunks, one descriptor per workgroup; with a few large tensors mixed in, into 1024."""
    rng = np.random.default_rng(41)
    for sizes in ([int(x) for x in rng.integers(1, 701, 400)],
                  [int(x) for x in rng.integers(64, 513, 300)] + [200_000] * 12):
        w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
        run_both(dev, rule, hyper, w, lambda k: [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes],
                 steps=4, check_every=2, nthreads=1)


SPECIALS = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-40, -3e-39, 1.17549435e-38,
                     3.4028235e38, -3.4028235e38, 1e-30, 1e30, 1.0, -1.0, 65504.0, 1e-8, 5e-324], dtype=np.float32)


@pytest.mark.parametrize("rule,hyper", [
    ("sgd", dict(lr=0.01, momentum=0.9, weight_decay=1e-4, nesterov=True)),
    ("adam", dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
    ("rmsprop", dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.9, centered=True)),
    ("adagrad", dict(lr=0.01, eps=1e-10, weight_decay=0.0)),
    ("adadelta", dict(rho=0.9, eps=1e-6, weight_decay=0.0)),
    ("nadam", dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)),
])
def test_special_values(dev, rule, hyper):
    """Every pairing of special weights and gradients (signed zeros, infinities, NaN, subnormals,
    the largest finite value): the GPU and the oracle agree on where NaNs appear and on every other
    bit -- subnormals are neither flushed on input nor on output, overflow goes to the same infinity."""
    w = np.repeat(SPECIALS, SPECIALS.size).astype(np.float32)
    g = np.tile(SPECIALS, SPECIALS.size).astype(np.float32)
    gpu, cpu = GpuRun(dev, rule, hyper, [w]), OracleRun(rule, hyper, [w])
    try:
        with np.errstate(all="ignore"):
            for _ in range(3):
                gpu.step([g])
                cpu.step([g])
        got, want = gpu.snapshot(), cpu.snapshot()
        for key in want:
            a, b = got[key][0], want[key][0]
            assert np.array_equal(np.isnan(a), np.isnan(b)), (rule, key, "NaN positions")
            ok = ~np.isnan(b)
            assert np.array_equal(a[ok].view(np.uint32), b[ok].view(np.uint32)), (rule, key)
    finally:
        gpu.close()


def random_case(rng):
    """A random rule, hyper-parameter set and tensor list (sizes from 0 to ~200k, log-uniform)."""
    rule = ["sgd", "adam", "rmsprop", "adagrad", "adadelta", "nadam"][int(rng.integers(0, 6))]
    f = lambda lo, hi: float(np.float32(10.0 ** rng.uniform(np.log10(lo), np.log10(hi))))
    wd = 0.0 if rng.random() < 0.4 else f(1e-6, 1e-1)
    if rule == "sgd":
        hyper = dict(lr=f(1e-4, 1.0), momentum=0.0 if rng.random() < 0.3 else float(np.float32(rng.uniform(0.1, 0.99))),
                     weight_decay=wd, nesterov=bool(rng.random() < 0.5))
    elif rule in ("adam", "nadam"):
        hyper = dict(lr=f(1e-5, 1e-1), beta1=float(np.float32(rng.uniform(0.5, 0.99))),
                     beta2=float(np.float32(rng.uniform(0.9, 0.9999))), eps=f(1e-10, 1e-4), weight_decay=wd)
    elif rule == "rmsprop":
        hyper = dict(lr=f(1e-4, 1e-1), alpha=float(np.float32(rng.uniform(0.8, 0.999))), eps=f(1e-10, 1e-4),
                     weight_decay=wd, momentum=0.0 if rng.random() < 0.5 else float(np.float32(rng.uniform(0.1, 0.95))),
                     centered=bool(rng.random() < 0.5))
    elif rule == "adagrad":
        hyper = dict(lr=f(1e-4, 1.0), eps=f(1e-12, 1e-6), weight_decay=wd)
    else:
        hyper = dict(rho=float(np.float32(rng.uniform(0.5, 0.99))), eps=f(1e-8, 1e-4), weight_decay=wd)
    count = int(rng.integers(1, 13))
    sizes = [0 if rng.random() < 0.05 else int(2.0 ** rng.uniform(0, 17.6)) for _ in range(count)]
    return rule, hyper, sizes


@pytest.mark.parametrize("seed", range(24))
def test_random_rules_hyperparameters_and_lists(dev, seed):
    """Randomised parity: rule, hyper-parameters, list shape, weight and gradient magnitudes all
    drawn from a seeded generator; 4 steps, every buffer compared bit for bit after each."""
    rng = np.random.default_rng(1000 + seed)
    rule, hyper, sizes = random_case(rng)
    wscale, gscale = 10.0 ** rng.uniform(-3, 1), 10.0 ** rng.uniform(-6, 1)
    w = [rng.normal(0, wscale, n).astype(np.float32) for n in sizes]
    print(f"seed {seed}: {rule} {hyper} sizes {sizes}", flush=True)
    with np.errstate(all="ignore"):
        run_both(dev, rule, hyper, w, lambda k: [rng.normal(0, gscale, n).astype(np.float32) for n in sizes],
                 steps=4, check_every=1, nthreads=1)

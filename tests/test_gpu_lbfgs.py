"""L-BFGS step on the GPU through the C ABI (execute_lbfgs_step_mpsgraph) against the CPU oracle
in its tree-order mode: bit-exact on every buffer, every rho and every alpha."""
import ctypes
import math
import sys

import numpy as np
import pytest

from harness import gpu_device
from lbfgs_cases import F, case_inputs, check_against_expected, load_cases, same_bits
from oracle_lib import oracle
from workloads import cnn_sizes, ragged_sizes
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()
TREE = 1


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


class LbfgsGpu:
    """Device copies of an L-BFGS state dictionary, stepped through the C ABI."""

    def __init__(self, dev, st, pooled=False):
        self.dev, self.pooled = dev, pooled
        self.sizes = [int(t.size) for t in st["w"]]
        self.n, self.m = len(self.sizes), len(st["s"])
        up = lambda a: dev.from_numpy(np.asarray(a, dtype=F)) if a.size else dev.alloc(4)
        self.w = [up(t) for t in st["w"]]
        self.old_g = [up(t) for t in st["old_g"]]
        self.dir = [up(t) for t in st["dir"]]
        self.g = [dev.alloc(max(4 * k, 4)) for k in self.sizes]
        self.s = [[up(t) for t in h] for h in st["s"]]
        self.y = [[up(t) for t in h] for h in st["y"]]
        self.rho = [dev.from_numpy(st["rho"][h:h + 1]) for h in range(self.m)]
        self.alpha = dev.from_numpy(st["alpha"])
        self.byte_sizes = pkg.int_array([4 * k for k in self.sizes])

    def handles(self):
        return [*self.w, *self.old_g, *self.dir, *self.g, *[b for h in self.s for b in h],
                *[b for h in self.y for b in h], *self.rho, self.alpha]

    def free(self):
        for h in self.handles():
            self.dev.free(h)

    def step(self, grads, count, index, initial_step, expect_rc=0):
        for h, g in zip(self.g, grads):
            if g.size:
                self.dev.upload(h, g)
        step = ctypes.c_float(-1.0)
        arr = pkg.handle_array
        args = [self.dev.handle, arr(self.w), arr(self.g), arr(self.old_g), arr(self.dir),
                arr([b for h in self.s for b in h]), arr([b for h in self.y for b in h]), arr(self.rho),
                self.alpha, self.n, self.byte_sizes, self.m, count, index, initial_step, 1e-4, 0.9, 20,
                1.0, 2.0]
        print(f"lbfgs step: sizes[:4]={self.sizes[:4]} n={self.n} m={self.m} count={count} index={index}",
              flush=True)
        if self.pooled:
            rc = self.dev.lib.execute_lbfgs_step_mpsgraph_pooled(*args, 0x2000, ctypes.byref(step))
        else:
            rc = self.dev.lib.execute_lbfgs_step_mpsgraph(*args, ctypes.byref(step))
        assert rc == expect_rc, (rc, self.dev.lib.gm_last_error())
        if rc == 0:
            assert step.value == np.float32(initial_step)
        return rc

    def download(self):
        d = self.dev
        get = lambda hs: [d.to_numpy(h, k) for h, k in zip(hs, self.sizes)]
        return {"w": get(self.w), "old_g": get(self.old_g), "dir": get(self.dir),
                "s": [get(h) for h in self.s], "y": [get(h) for h in self.y],
                "rho": np.concatenate([d.to_numpy(h, 1) for h in self.rho]),
                "alpha": d.to_numpy(self.alpha, self.m)}


def assert_same_state(got, want, where):
    for key in ("w", "old_g", "dir"):
        for i, (a, b) in enumerate(zip(got[key], want[key])):
            assert same_bits(a, b), (where, key, i)
    for key in ("s", "y"):
        for h in range(len(want[key])):
            for i, (a, b) in enumerate(zip(got[key][h], want[key][h])):
                assert same_bits(a, b), (where, key, h, i)
    assert same_bits(got["rho"], want["rho"]), (where, "rho", got["rho"], want["rho"])
    assert same_bits(got["alpha"], want["alpha"]), (where, "alpha", got["alpha"], want["alpha"])


@pytest.mark.parametrize("pooled", [False, True])
@pytest.mark.parametrize("case", load_cases(), ids=lambda c: c["name"])
def test_golden_vectors(dev, case, pooled):
    st, grads = case_inputs(case)
    run = LbfgsGpu(dev, st, pooled)
    m, count, index = case["history_size"], case["history_count"], case["history_index"]
    try:
        for k, g in enumerate(grads):
            run.step(g, count, index, case["initial_step"])
            check_against_expected(run.download(), case["expect"]["tree"][k], (case["name"], k))
            index, count = (index + 1) % m, min(count + 1, m)
    finally:
        run.free()


def seeded_state(rng, sizes, m, rho):
    r = lambda k, s: (rng.standard_normal(k) * s).astype(F)
    return {"w": [r(k, 0.5) for k in sizes], "old_g": [r(k, 1e-2) for k in sizes],
            "dir": [np.zeros(k, F) for k in sizes],
            "s": [[r(k, 1e-2) for k in sizes] for _ in range(m)],
            "y": [[r(k, 1e-2) for k in sizes] for _ in range(m)],
            "rho": np.asarray(rho, dtype=F), "alpha": r(m, 1.0)}


def clone(st):
    return {k: ([[t.copy() for t in h] for h in v] if k in ("s", "y") else
                [t.copy() for t in v] if isinstance(v, list) else v.copy()) for k, v in st.items()}


LISTS = {
    "cnn": cnn_sizes(),                                        # 16 tensors, 1.14M elements, tiny ones included
    "ragged": ragged_sizes(count=40, total=3_000_000, lo=1, hi=600_000, seed=5),   # > 1024 slices: 3 tree levels
    "edges": [1, 1023, 1024, 1025, 65535, 65536, 65537, 0, 3],
}


@pytest.mark.parametrize("name", list(LISTS))
@pytest.mark.parametrize("m,count,index,rho", [
    (3, 3, 1, [40.0, -7.5, 12.0]),            # full ring, wrapped
    (4, 2, 2, [3.0, 5e-11, 9.0, 9.0]),        # partial history with an invalid pair
    (1, 1, 0, [6.0]),
    (2, 0, 0, [0.0, 0.0]),                    # empty history
])
def test_step_matches_oracle(dev, name, m, count, index, rho):
    sizes = LISTS[name]
    rng = np.random.default_rng(len(sizes) * 1000 + m * 10 + count)
    st = seeded_state(rng, sizes, m, rho)
    ref = clone(st)
    run = LbfgsGpu(dev, st)
    try:
        for k in range(2):
            g = [(rng.standard_normal(n) * 1e-2).astype(F) for n in sizes]
            run.step(g, count, index, 0.5)
            rc, _ = oracle().lbfgs_step(ref, g, m, count, index, 0.5, TREE)
            assert rc == 0
            assert_same_state(run.download(), ref, (name, m, count, index, k))
            index, count = (index + 1) % m, min(count + 1, m)
    finally:
        run.free()


def test_optimizer_sequence_from_fresh_state(dev):
    # what optimizer/lbfgs.go drives: zeroed state, count and index advanced by the host
    sizes, m = cnn_sizes(), 3
    rng = np.random.default_rng(77)
    z = lambda: [np.zeros(k, F) for k in sizes]
    st = {"w": [rng.standard_normal(k).astype(F) for k in sizes], "old_g": z(), "dir": z(),
          "s": [z() for _ in range(m)], "y": [z() for _ in range(m)],
          "rho": np.zeros(m, F), "alpha": np.zeros(m, F)}
    ref = clone(st)
    run = LbfgsGpu(dev, st)
    count = index = 0
    try:
        for k in range(5):
            g = [(rng.standard_normal(n) * 1e-2).astype(F) for n in sizes]
            run.step(g, count, index, 1.0)
            assert oracle().lbfgs_step(ref, g, m, count, index, 1.0, TREE)[0] == 0
            index, count = (index + 1) % m, min(count + 1, m)
        got = run.download()
        assert_same_state(got, ref, "sequence")
        assert not got["rho"].any()
    finally:
        run.free()


def test_non_finite_gradient(dev):
    # inf - inf = NaN in y, NaN s.y fails the |s.y| > 1e-10 test, rho = 0 (bridge_optimizer.m:1304-1310)
    sizes, m = [300, 5], 2
    rng = np.random.default_rng(9)
    st = seeded_state(rng, sizes, m, [2.0, 3.0])
    ref = clone(st)
    g = [(rng.standard_normal(n) * 1e-2).astype(F) for n in sizes]
    g[0][17] = np.inf
    g[1][2] = np.nan
    run = LbfgsGpu(dev, st)
    try:
        run.step(g, 2, 0, 1.0)
        assert oracle().lbfgs_step(ref, g, m, 2, 0, 1.0, TREE)[0] == 0
        got = run.download()
        assert_same_state(got, ref, "non-finite")
        assert got["rho"][1] == 0.0
    finally:
        run.free()


@pytest.mark.parametrize("sizes", [[1], [1024], [1025], [70_000, 3], [2_500_000], [1 << 20, 1 << 20, 5]])
def test_dot_matches_oracle_tree_and_exact_sum(dev, sizes):
    rng = np.random.default_rng(sum(sizes) + 1)
    a = [rng.standard_normal(k).astype(F) for k in sizes]
    b = [rng.standard_normal(k).astype(F) for k in sizes]
    ha = [dev.from_numpy(t) for t in a]
    hb = [dev.from_numpy(t) for t in b]
    out = ctypes.c_float(0.0)
    try:
        rc = dev.lib.gm_lbfgs_dot(dev.handle, pkg.handle_array(ha), pkg.handle_array(hb), len(sizes),
                                  pkg.int_array([4 * k for k in sizes]), ctypes.byref(out))
        assert rc == 0, dev.lib.gm_last_error()
    finally:
        for h in ha + hb:
            dev.free(h)
    got = F(out.value)
    assert got.view(np.uint32) == oracle().lbfgs_dot(a, b, TREE).view(np.uint32)
    exact = math.fsum(float(x) for ta, tb in zip(a, b) for x in ta.astype(np.float64) * tb.astype(np.float64))
    assert abs(int(got.view(np.int32)) - int(F(exact).view(np.int32))) <= 1
    # and inside the error bound of the reference's running fp32 sum
    n = sum(sizes)
    mag = math.fsum(float(abs(x)) for ta, tb in zip(a, b) for x in ta.astype(np.float64) * tb.astype(np.float64))
    u = 2.0 ** -24
    ref_order = float(oracle().lbfgs_dot(a, b, 0))
    assert abs(float(got) - ref_order) <= 2 * (n + 1) * u / (1 - (n + 1) * u) * mag


def test_return_codes(dev):
    sizes, m = [100, 7], 2
    rng = np.random.default_rng(3)
    st = seeded_state(rng, sizes, m, [1.0, 1.0])
    run = LbfgsGpu(dev, st)
    g = [np.ones(k, F) for k in sizes]
    lib, arr = dev.lib, pkg.handle_array
    step = ctypes.c_float(0)
    flat_s, flat_y = [b for h in run.s for b in h], [b for h in run.y for b in h]

    def call(device=None, w=None, s=None, rho=None, alpha=None, count=1, index=0, msize=m, sizes_=None):
        return lib.execute_lbfgs_step_mpsgraph(
            dev.handle if device is None else device, arr(run.w if w is None else w), arr(run.g),
            arr(run.old_g), arr(run.dir), arr(flat_s if s is None else s), arr(flat_y),
            arr(run.rho if rho is None else rho), run.alpha if alpha is None else alpha, run.n,
            run.byte_sizes if sizes_ is None else sizes_, msize, count, index, 1.0, 1e-4, 0.9, 20, 0.0, 0.0,
            ctypes.byref(step))

    try:
        before = run.download()
        assert call(device=0) == -1                                   # bridge_optimizer.m:1005-1008
        assert call(count=3) == -5 and call(index=2) == -5 and call(count=-1) == -5 and call(msize=0) == -5
        assert call(w=[run.w[0], 0]) == -8 and b"nil" in lib.gm_last_error()
        assert call(s=[0] + flat_s[1:]) == -8
        assert call(rho=[run.rho[0], 0]) == -8
        assert call(alpha=0) == -8
        assert call(sizes_=pkg.int_array([4 * 100, 4 * 5000])) == -8 and b"shorter" in lib.gm_last_error()
        assert_same_state(run.download(), before, "failed calls write nothing")
        assert call() == 0
    finally:
        run.free()


def test_c3_size_list_full_recursion(dev):
    # 25M parameters in 160 ragged tensors, full history of 3: every pass at a realistic size
    sizes, m = ragged_sizes(), 3
    rng = np.random.default_rng(2024)
    st = seeded_state(rng, sizes, m, [25.0, -3.0, 8.0])
    ref = clone(st)
    g = [(rng.standard_normal(n) * 1e-2).astype(F) for n in sizes]
    run = LbfgsGpu(dev, st)
    try:
        run.step(g, 3, 2, 0.75)
        assert oracle().lbfgs_step(ref, g, m, 3, 2, 0.75, TREE)[0] == 0
        assert_same_state(run.download(), ref, "c3")
    finally:
        run.free()


def test_c4_size_list_two_valid_pairs(dev):
    # 125M parameters in 60 tensors: three tree levels per dot product, every pass at scale
    from workloads import amp_125m_sizes
    sizes, m = amp_125m_sizes(), 2
    rng = np.random.default_rng(125)
    r = lambda k, s: rng.standard_normal(k, dtype=F) * F(s)
    st = {"w": [r(k, 0.5) for k in sizes], "old_g": [r(k, 1e-2) for k in sizes],
          "dir": [np.zeros(k, F) for k in sizes],
          "s": [[r(k, 1e-2) for k in sizes] for _ in range(m)],
          "y": [[r(k, 1e-2) for k in sizes] for _ in range(m)],
          "rho": np.asarray([3e-4, -2e-4], dtype=F), "alpha": np.zeros(m, F)}
    g = [r(k, 1e-2) for k in sizes]
    run = LbfgsGpu(dev, st)
    try:
        run.step(g, 2, 0, 0.5)
        print("oracle step over 125M parameters", flush=True)
        assert oracle().lbfgs_step(st, g, m, 2, 0, 0.5, TREE)[0] == 0       # st is the reference from here on
        assert_same_state(run.download(), st, "c4")
        assert st["alpha"].all()
    finally:
        run.free()


def test_c5_size_dot_and_plain_step(dev):
    # 1,012,301,824 parameters in 400 tensors, data generated on the device: the dot product
    # against the oracle's tree (four levels), and the step with no valid pair against its closed form
    from workloads import transformer_block_sizes
    sizes = transformer_block_sizes()
    n, lib, D = len(sizes), dev.lib, dev.handle
    lists = {}
    for name, seed, std in (("w", 1, 0.02), ("g", 2, 1e-2), ("old_g", 3, 1e-2), ("dir", 4, 1.0), ("s", 5, 1e-2),
                            ("y", 6, 1e-2)):
        lists[name] = [dev.alloc(4 * k) for k in sizes]
        for i, k in enumerate(sizes):
            assert lib.gm_fill_normal_f32(D, lists[name][i], k, seed * 100000 + i, 0.0, std) == 0
    rho, alpha = dev.from_numpy(np.zeros(1, F)), dev.from_numpy(np.zeros(1, F))
    arr, bs = pkg.handle_array, pkg.int_array([4 * k for k in sizes])
    try:
        out = ctypes.c_float()
        print("dot product over 1.012B parameters", flush=True)
        assert lib.gm_lbfgs_dot(D, arr(lists["s"]), arr(lists["g"]), n, bs, ctypes.byref(out)) == 0
        a = [dev.to_numpy(h, k) for h, k in zip(lists["s"], sizes)]
        b = [dev.to_numpy(h, k) for h, k in zip(lists["g"], sizes)]
        print("oracle dot product", flush=True)
        assert F(out.value).view(np.uint32) == oracle().lbfgs_dot(a, b, TREE).view(np.uint32)
        del a
        w0 = [dev.to_numpy(lists["w"][i], sizes[i]) for i in (0, 2, 33, 399)]
        step = ctypes.c_float()
        # history_count 1 with rho = 0: the update pass from the gradient, which also writes y_prev and rho_prev
        assert lib.execute_lbfgs_step_mpsgraph(D, arr(lists["w"]), arr(lists["g"]), arr(lists["old_g"]),
                                               arr(lists["dir"]), arr(lists["s"]), arr(lists["y"]), arr([rho]),
                                               alpha, n, bs, 1, 1, 0, 0.25, 1e-4, 0.9, 20, 0.0, 0.0,
                                               ctypes.byref(step)) == 0
        for j, i in enumerate((0, 2, 33, 399)):
            k = sizes[i]
            assert same_bits(dev.to_numpy(lists["w"][i], k), w0[j] + F(0.25) * b[i]), i
            assert same_bits(dev.to_numpy(lists["dir"][i], k), b[i]), i
            assert same_bits(dev.to_numpy(lists["old_g"][i], k), b[i]), i
            assert same_bits(dev.to_numpy(lists["s"][i], k), F(0.25) * b[i]), i
            assert not dev.to_numpy(lists["y"][i], k).any(), i
        assert dev.to_numpy(rho, 1)[0] == 0.0 and dev.to_numpy(alpha, 1)[0] == 0.0
    finally:
        for hs in lists.values():
            for h in hs:
                dev.free(h)
        dev.free(rho)
        dev.free(alpha)


def test_dot_with_three_tree_levels(dev):
    # more than 1024 * 1024 slices (1.29e9 elements): a plain level, then the fused last two; the first tensor has
    # the largest size a C int in bytes can name (2^31 - 4), with a ragged last slice
    sizes = [2 ** 29 - 1, 450_000_000, 300_000_000]
    lib, D = dev.lib, dev.handle
    ha = [dev.alloc(4 * k) for k in sizes]
    hb = [dev.alloc(4 * k) for k in sizes]
    try:
        for i, k in enumerate(sizes):
            assert lib.gm_fill_normal_f32(D, ha[i], k, 900 + i, 0.0, 1.0) == 0
            assert lib.gm_fill_normal_f32(D, hb[i], k, 950 + i, 0.5, 1.0) == 0
        out = ctypes.c_float()
        print("dot product over 1.29e9 elements", flush=True)
        assert lib.gm_lbfgs_dot(D, pkg.handle_array(ha), pkg.handle_array(hb), 3, pkg.int_array([4 * k for k in sizes]),
                                ctypes.byref(out)) == 0
        a = [dev.to_numpy(h, k) for h, k in zip(ha, sizes)]
        b = [dev.to_numpy(h, k) for h, k in zip(hb, sizes)]
        print("oracle dot product", flush=True)
        want = oracle().lbfgs_dot(a, b, TREE)
        assert F(out.value).view(np.uint32) == want.view(np.uint32), (out.value, want)
    finally:
        for h in ha + hb:
            dev.free(h)


@pytest.mark.parametrize("seed", range(12))
def test_random_lists_histories_and_step_sizes(dev, seed):
    """Tensor lists, ring sizes, history counts / indices, rho values (valid, zero, just under the 1e-10
    threshold) and step sizes drawn from a seeded generator; three consecutive steps each, every buffer compared
    bit for bit with the oracle in tree order."""
    rng = np.random.default_rng(7000 + seed)
    nt = int(rng.integers(1, 12))
    sizes = [int(x) for x in np.exp(rng.uniform(0, np.log(300_000), nt)).astype(int)]
    if rng.random() < 0.5:
        sizes[int(rng.integers(0, nt))] = int(rng.choice([0, 1, 1023, 1024, 1025, 65536, 65537]))
    m = int(rng.integers(1, 6))
    count, index = int(rng.integers(0, m + 1)), int(rng.integers(0, m))
    rho = [float(rng.choice([0.0, 5e-11, rng.normal(0, 20)])) for _ in range(m)]
    st = seeded_state(rng, sizes, m, rho)
    ref = clone(st)
    run = LbfgsGpu(dev, st)
    try:
        for k in range(3):
            g = [(rng.standard_normal(n) * 1e-2).astype(F) for n in sizes]
            step = float(rng.choice([0.5, 1.0, 0.01]))
            run.step(g, count, index, step)
            rc, _ = oracle().lbfgs_step(ref, g, m, count, index, step, TREE)
            assert rc == 0
            assert_same_state(run.download(), ref, (seed, sizes, m, count, index, k))
            index, count = (index + 1) % m, min(count + 1, m)
    finally:
        run.free()


def recursion_float64(g, s, y, rho, count, index, perturb=None):
    """The two-loop recursion of the step (bridge_optimizer.m:1025-1213) in float64 with exact dot products,
    on flat vectors.  perturb = (k, delta) adds delta to the k-th dot product taken.  Returns the direction p,
    the alphas and, for every dot product, (value, sum of |a_i b_i|)."""
    m = len(s)
    q = -g.copy()
    alpha = np.zeros(count)
    dots = []

    def dot(a, b):
        k = len(dots)
        value = float(np.dot(a, b))
        dots.append((value, float(np.dot(np.abs(a), np.abs(b)))))
        return value + (perturb[1] if perturb and perturb[0] == k else 0.0)

    for j in range(count - 1, -1, -1):
        idx = (index - count + j + m) % m
        if abs(rho[idx]) < 1e-10:
            continue
        alpha[j] = rho[idx] * dot(s[idx], q)
        q = q - alpha[j] * y[idx]
    for j in range(count):
        idx = (index - count + j + m) % m
        if abs(rho[idx]) < 1e-10:
            continue
        beta = rho[idx] * dot(y[idx], q)
        q = q + (alpha[j] - beta) * s[idx]
    return -q, alpha, dots


def test_step_against_the_reference_summation_order_within_the_propagated_bound(dev):
    """The reference sums each dot product as a running fp32 sum in element order (bridge_optimizer.m:1100-1104);
    the library sums exact fp64 products in a fixed tree.  The two orders cannot agree bit for bit, so the GPU step
    is compared with the oracle run in the REFERENCE order under a stated bound: a running fp32 sum of n terms is
    within gamma_n * sum|a_i b_i| of the exact dot product (gamma_n = n u / (1 - n u), u = 2^-24), the tree within
    half an fp32 ulp.  That per-dot error is pushed through the recursion numerically (each dot product of a float64
    model of the recursion shifted by its own bound, one at a time, both signs) and the shifts of every alpha and
    every element of the direction are added up: twice that sum, plus a few ulps for the elementwise fp32 roundings,
    bounds the distance between the two runs.  The bound is tight enough to notice a missing term: it stays below
    2 % of the direction's largest element."""
    sizes, m, count, index = [70_000, 5, 4097, 1023, 30_000], 4, 3, 3
    rng = np.random.default_rng(77)
    r = lambda k, scale: (rng.standard_normal(k) * scale).astype(F)
    st = {"w": [r(k, 0.5) for k in sizes], "old_g": [r(k, 1e-2) for k in sizes], "dir": [np.zeros(k, F) for k in sizes],
          "s": [[r(k, 1e-2) for k in sizes] for _ in range(m)], "y": [[r(k, 1e-2) for k in sizes] for _ in range(m)],
          "rho": np.zeros(m, F), "alpha": np.zeros(m, F)}
    flat = lambda ts: np.concatenate([t.astype(np.float64) for t in ts])
    # rho_j = 1 / (s_j . y_j'), with y_j' = y_j + 3 s_j so that the curvature is positive and alpha is O(1)
    for h in range(m):
        st["y"][h] = [(yt + F(3.0) * st_).astype(F) for yt, st_ in zip(st["y"][h], st["s"][h])]
        st["rho"][h] = F(1.0 / np.dot(flat(st["s"][h]), flat(st["y"][h])))
    g = [r(k, 1e-2) for k in sizes]
    ref = clone(st)
    run = LbfgsGpu(dev, st)
    try:
        run.step(g, count, index, 0.5)
        got = run.download()
    finally:
        run.free()
    assert oracle().lbfgs_step(ref, g, m, count, index, 0.5, 0)[0] == 0          # 0: the reference's own order

    gf, sf, yf = flat(g), [flat(h) for h in st["s"]], [flat(h) for h in st["y"]]
    rho = st["rho"].astype(np.float64)
    p0, alpha0, dots = recursion_float64(gf, sf, yf, rho, count, index)
    assert len(dots) == 2 * count
    n, u = gf.size + len(sizes), 2.0 ** -24
    gamma = n * u / (1 - n * u)
    bound_p, bound_alpha = np.zeros_like(p0), np.zeros(count)
    for k, (value, magnitude) in enumerate(dots):
        e = gamma * magnitude + abs(value) * u             # running-sum bound, plus the final rounding of either order
        shift_p, shift_a = np.zeros_like(p0), np.zeros(count)
        for sign in (1.0, -1.0):
            p1, alpha1, _ = recursion_float64(gf, sf, yf, rho, count, index, perturb=(k, sign * e))
            shift_p, shift_a = np.maximum(shift_p, np.abs(p1 - p0)), np.maximum(shift_a, np.abs(alpha1 - alpha0))
        bound_p += shift_p
        bound_alpha += shift_a
    ulps = 32 * u
    slack_p = ulps * (np.abs(p0) + np.abs(gf) + sum(abs(a) * np.abs(yv) for a, yv in zip(alpha0, yf[:count])) +
                      sum((abs(a) + 1.0) * np.abs(sv) for a, sv in zip(alpha0, sf)))
    assert bound_p.max() < 0.02 * np.abs(p0).max(), "the bound must stay small against the direction itself"

    p_gpu, p_ref = flat(got["dir"]), flat(ref["dir"])
    assert not np.array_equal(p_gpu, p_ref), "the two summation orders are expected to differ in the last bits"
    assert np.all(np.abs(p_gpu - p_ref) <= 2 * bound_p + slack_p)
    assert np.all(np.abs(p_gpu - p0) <= bound_p + slack_p) and np.all(np.abs(p_ref - p0) <= bound_p + slack_p)
    a_gpu, a_ref = got["alpha"][:count].astype(np.float64), ref["alpha"][:count].astype(np.float64)
    assert np.all(np.abs(a_gpu - a_ref) <= 2 * bound_alpha + ulps * np.abs(alpha0))
    # the weights moved by step * p in both runs
    w_gpu, w_ref = flat(got["w"]), flat(ref["w"])
    assert np.all(np.abs(w_gpu - w_ref) <= 0.5 * (2 * bound_p + slack_p) + 4 * u * np.abs(w_ref))

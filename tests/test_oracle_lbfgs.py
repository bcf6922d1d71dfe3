"""CPU checks of the L-BFGS oracle (oracle/oracle_lbfgs.c): golden vectors from the independent
Python evaluator, closed forms, and the two dot-product orders against the exact sum."""
import math

import numpy as np
import pytest

from lbfgs_cases import (F, case_inputs, check_against_expected, load_cases, same_bits)
from oracle_lib import oracle

MODES = {"reference": 0, "tree": 1}


@pytest.mark.parametrize("mode", ["reference", "tree"])
@pytest.mark.parametrize("case", load_cases(), ids=lambda c: c["name"])
def test_golden(case, mode):
    o = oracle()
    st, grads = case_inputs(case)
    m, count, index = case["history_size"], case["history_count"], case["history_index"]
    for k, g in enumerate(grads):
        rc, step = o.lbfgs_step(st, g, m, count, index, case["initial_step"], MODES[mode])
        assert rc == 0 and step == case["initial_step"]
        check_against_expected(st, case["expect"][mode][k], (case["name"], mode, k))
        index = (index + 1) % m               # optimizer/lbfgs.go:287-290
        count = min(count + 1, m)


def fresh_state(rng, sizes, m):
    z = lambda: [np.zeros(k, F) for k in sizes]
    return {"w": [rng.standard_normal(k).astype(F) for k in sizes], "old_g": z(), "dir": z(),
            "s": [z() for _ in range(m)], "y": [z() for _ in range(m)],
            "rho": np.zeros(m, F), "alpha": np.zeros(m, F)}


@pytest.mark.parametrize("mode", [0, 1])
def test_empty_history_moves_weights_by_plus_step_times_gradient(mode):
    # q = -g, no recursion, p = -q = g, x += a * p  (bridge_optimizer.m:1025-1038, 1203-1240)
    rng = np.random.default_rng(1)
    sizes = [33, 1, 1500]
    st = fresh_state(rng, sizes, 3)
    w0 = [t.copy() for t in st["w"]]
    g = [rng.standard_normal(k).astype(F) for k in sizes]
    rc, step = oracle().lbfgs_step(st, g, 3, 0, 0, 0.25, mode)
    assert rc == 0 and step == 0.25
    for i in range(len(sizes)):
        assert same_bits(st["w"][i], w0[i] + F(0.25) * g[i])
        assert same_bits(st["dir"][i], g[i])
        assert same_bits(st["old_g"][i], g[i])
        assert same_bits(st["s"][0][i], F(0.25) * g[i])
        assert not st["s"][1][i].any() and not st["y"][0][i].any()


@pytest.mark.parametrize("mode", [0, 1])
def test_rho_written_by_the_step_is_always_zero(mode):
    # the old gradient is overwritten before y = g - old_g is formed (:1237-1238 before :1285-1288)
    rng = np.random.default_rng(2)
    sizes, m = [40, 9], 3
    st = fresh_state(rng, sizes, m)
    count = index = 0
    for _ in range(5):
        g = [rng.standard_normal(k).astype(F) for k in sizes]
        assert oracle().lbfgs_step(st, g, m, count, index, 1.0, mode)[0] == 0
        index, count = (index + 1) % m, min(count + 1, m)
        assert not st["rho"].any()
        for h in range(m):
            for t in st["y"][h]:
                assert not t.any()


def test_one_valid_pair_against_float64_formula():
    # direction with one history pair: q = -g; a = rho s.q; q -= a y; b = rho y.q; q += (a - b) s; p = -q
    rng = np.random.default_rng(3)
    n = 200
    st = fresh_state(rng, [n], 1)
    s = (rng.standard_normal(n) * 0.1).astype(F)
    y = (rng.standard_normal(n) * 0.1).astype(F)
    rho = F(1.0 / float(np.dot(s.astype(np.float64), y.astype(np.float64))))
    g = rng.standard_normal(n).astype(F)
    w0 = st["w"][0].copy()
    for mode in (0, 1):
        st["w"][0] = w0.copy()
        st["s"][0][0], st["y"][0][0], st["rho"][0] = s.copy(), y.copy(), rho
        assert oracle().lbfgs_step(st, [g], 1, 1, 0, 1.0, mode)[0] == 0
        s64, y64, g64, r64 = s.astype(np.float64), y.astype(np.float64), g.astype(np.float64), float(rho)
        q = -g64
        a = r64 * np.dot(s64, q)
        q = q - a * y64
        b = r64 * np.dot(y64, q)
        q = q + (a - b) * s64
        p = -q
        np.testing.assert_allclose(st["dir"][0], p, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(st["w"][0], w0.astype(np.float64) + p, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(float(st["alpha"][0]), a, rtol=1e-4)


def test_invalid_history_arguments():
    rng = np.random.default_rng(4)
    st = fresh_state(rng, [4], 2)
    g = [np.ones(4, F)]
    o = oracle()
    assert o.lbfgs_step(st, g, 2, 3, 0, 1.0, 0)[0] == -5
    assert o.lbfgs_step(st, g, 2, 0, 2, 1.0, 0)[0] == -5
    assert o.lbfgs_step(st, g, 2, -1, 0, 1.0, 0)[0] == -5


@pytest.mark.parametrize("sizes", [[1], [255], [1024], [1025], [5000, 3, 2048], [1 << 20, 77],
                                   [1100000]])
def test_tree_dot_is_within_one_ulp_of_the_exact_dot(sizes):
    # products of binary32 values are exact in binary64, math.fsum adds them exactly
    rng = np.random.default_rng(sum(sizes))
    a = [rng.standard_normal(k).astype(F) for k in sizes]
    b = [rng.standard_normal(k).astype(F) for k in sizes]
    exact = math.fsum(float(x) for ta, tb in zip(a, b)
                      for x in (ta.astype(np.float64) * tb.astype(np.float64)))
    got = oracle().lbfgs_dot(a, b, 1)
    assert abs(float(got) - exact) <= float(np.spacing(F(abs(exact)))) * 0.5000001 + 0.0 or \
        abs(int(got.view(np.uint32)) - int(F(exact).view(np.uint32))) <= 1


@pytest.mark.parametrize("per_tensor", [True, False])
def test_reference_order_dot_is_within_its_error_bound_of_the_exact_dot(per_tensor):
    # running fp32 sum of n terms: |error| <= gamma_n * sum |a_i b_i|
    rng = np.random.default_rng(7)
    sizes = [3000, 17, 900]
    a = [rng.standard_normal(k).astype(F) for k in sizes]
    b = [rng.standard_normal(k).astype(F) for k in sizes]
    prods = np.concatenate([ta.astype(np.float64) * tb.astype(np.float64) for ta, tb in zip(a, b)])
    exact, mag, n = math.fsum(prods), math.fsum(np.abs(prods)), prods.size
    u = 2.0 ** -24
    got = float(oracle().lbfgs_dot(a, b, 0, per_tensor))
    assert abs(got - exact) <= (n + 1) * u / (1 - (n + 1) * u) * mag
    # and the manual running sum reproduces it bit for bit
    total = F(0.0)
    for ta, tb in zip(a, b):
        acc = F(0.0) if per_tensor else total
        for x, yv in zip(ta, tb):
            acc = F(acc + F(x * yv))
        total = F(total + acc) if per_tensor else acc
    assert F(got).view(np.uint32) == total.view(np.uint32)


def test_tree_dot_levels_match_python_floats():
    # more than 1024 slices: three levels of the tree, restated with Python floats
    rng = np.random.default_rng(11)
    n = 1024 * 1030 + 5
    a = rng.standard_normal(n).astype(F)
    b = rng.standard_normal(n).astype(F)
    prods = a.astype(np.float64) * b.astype(np.float64)

    def node(v):
        lanes = np.zeros(256)
        for u in range(0, len(v), 256):           # lane l adds v[l], v[l+256], ... in that order
            part = v[u:u + 256]
            lanes[:len(part)] = lanes[:len(part)] + part
        while lanes.size > 1:
            lanes = lanes[0::2] + lanes[1::2]
        return lanes[0]

    level = np.array([node(prods[o:o + 1024]) for o in range(0, n, 1024)])
    while level.size > 1:
        level = np.array([node(level[o:o + 1024]) for o in range(0, level.size, 1024)])
    assert oracle().lbfgs_dot([a], [b], 1).view(np.uint32) == F(level[0]).view(np.uint32)

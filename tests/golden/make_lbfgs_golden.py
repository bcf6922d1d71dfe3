#!/usr/bin/env python3
"""Writes tests/golden/lbfgs_kat.json: known-answer vectors for the L-BFGS step
(cgo_bridge/bridge_optimizer.m:980-1321).

Two evaluators, neither sharing code with oracle/oracle_lbfgs.c or the HIP kernels,
must agree bit for bit on every case before the file is written:

  * numpy: element operations are float32 ufunc calls (one rounding each), the
    reference-order dot product is a Python loop over numpy float32 scalars, and the
    tree-order dot product runs on Python floats (binary64) with the product of two
    binary32 values formed exactly;
  * exact: every operation is carried out over the rationals (fractions.Fraction)
    and rounded to binary32 -- or, inside the tree, to binary64 -- by integer
    arithmetic (make_golden.round_to_format): "what IEEE-754 fixes" for the
    statement sequence.

The reference asserts no numerical output for this function, so the expected values
come from these evaluators; what they pin is the statement order of the reference's
loop nest (see the notes in oracle/oracle_lbfgs.c) and the two summation orders.

Run from the repo root:  python tests/golden/make_lbfgs_golden.py
"""
import hashlib
import json
import os

import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from make_golden import f32_bits, rf32, round_to_format  # noqa: E402  (exact rounding helpers)
F = np.float32
SLICE, LANES = 1024, 256


def node(values):
    lanes = []
    for l in range(LANES):
        acc = 0.0
        for i in range(l, min(len(values), SLICE), LANES):
            acc = acc + values[i]
        lanes.append(acc)
    while len(lanes) > 1:
        lanes = [lanes[i] + lanes[i + 1] for i in range(0, len(lanes), 2)]
    return lanes[0]


def dot_tree(a, b):
    level = []
    for ta, tb in zip(a, b):
        for off in range(0, len(ta), SLICE):
            prods = [float(x) * float(y) for x, y in zip(ta[off:off + SLICE], tb[off:off + SLICE])]
            level.append(node(prods))
    if not level:
        return F(0.0)
    while len(level) > 1:
        level = [node(level[i:i + SLICE]) for i in range(0, len(level), SLICE)]
    return F(level[0])


def dot_reference(a, b, per_tensor):
    total = F(0.0)
    for ta, tb in zip(a, b):
        if per_tensor:
            d = F(0.0)
            for x, y in zip(ta, tb):
                d = F(d + F(x * y))
            total = F(total + d)
        else:
            for x, y in zip(ta, tb):
                total = F(total + F(x * y))
    return total


def dot(a, b, mode, per_tensor):
    return dot_tree(a, b) if mode == "tree" else dot_reference(a, b, per_tensor)


def lbfgs_step(st, g, m, count, index, step, mode):
    """st: dict of lists of float32 arrays (w, old_g, dir, s[h], y[h]) plus rho, alpha arrays."""
    n = len(g)
    with np.errstate(all="ignore"):
        for i in range(n):
            st["dir"][i] = np.negative(g[i])
        for j in range(count - 1, -1, -1):
            idx = (index - count + j + m) % m
            rho = st["rho"][idx]
            if abs(float(rho)) < 1e-10:
                st["alpha"][j] = F(0.0)
                continue
            a = F(dot(st["s"][idx], st["dir"], mode, True) * rho)
            st["alpha"][j] = a
            for i in range(n):
                st["dir"][i] = np.subtract(st["dir"][i], np.multiply(a, st["y"][idx][i], dtype=F), dtype=F)
        for j in range(count):
            idx = (index - count + j + m) % m
            rho = st["rho"][idx]
            if abs(float(rho)) < 1e-10:
                continue
            beta = F(dot(st["y"][idx], st["dir"], mode, True) * rho)
            coeff = F(st["alpha"][j] - beta)
            for i in range(n):
                st["dir"][i] = np.add(st["dir"][i], np.multiply(coeff, st["s"][idx][i], dtype=F), dtype=F)
        for i in range(n):
            st["dir"][i] = np.negative(st["dir"][i])
        a = F(step)
        for i in range(n):
            st["w"][i] = np.add(st["w"][i], np.multiply(a, st["dir"][i], dtype=F), dtype=F)
            st["old_g"][i] = g[i].copy()
        for i in range(n):
            st["s"][index][i] = np.multiply(a, st["dir"][i], dtype=F)
        if count > 0:
            prev = (index - 1 + m) % m
            for i in range(n):
                st["y"][prev][i] = np.subtract(g[i], st["old_g"][i], dtype=F)
            sdy = dot(st["s"][prev], st["y"][prev], mode, False)
            st["rho"][prev] = F(1.0) / sdy if abs(float(sdy)) > 1e-10 else F(0.0)


# ----------------------------------------------------------------------------
# the exact evaluator (finite values only: the golden cases hold no inf / NaN)
# ----------------------------------------------------------------------------
def rf64(x):
    r = round_to_format(x, 52, -1022, 1023)
    assert not isinstance(r, str)
    return r


def exact_node(values):
    lanes = []
    for l in range(LANES):
        acc = Fraction(0)
        for i in range(l, min(len(values), SLICE), LANES):
            acc = rf64(acc + values[i])
        lanes.append(acc)
    while len(lanes) > 1:
        lanes = [rf64(lanes[i] + lanes[i + 1]) for i in range(0, len(lanes), 2)]
    return lanes[0]


def exact_dot(a, b, mode, per_tensor):
    if mode == "tree":
        level = []
        for ta, tb in zip(a, b):
            for off in range(0, len(ta), SLICE):
                level.append(exact_node([x * y for x, y in zip(ta[off:off + SLICE], tb[off:off + SLICE])]))
        if not level:
            return Fraction(0)
        while len(level) > 1:
            level = [exact_node(level[i:i + SLICE]) for i in range(0, len(level), SLICE)]
        return rf32(level[0])
    total = Fraction(0)
    for ta, tb in zip(a, b):
        if per_tensor:
            d = Fraction(0)
            for x, y in zip(ta, tb):
                d = rf32(d + rf32(x * y))
            total = rf32(total + d)
        else:
            for x, y in zip(ta, tb):
                total = rf32(total + rf32(x * y))
    return total


def exact_state(st):
    fr = lambda t: [Fraction(float(v)) for v in t]
    return {"w": [fr(t) for t in st["w"]], "old_g": [fr(t) for t in st["old_g"]], "dir": [fr(t) for t in st["dir"]],
            "s": [[fr(t) for t in h] for h in st["s"]], "y": [[fr(t) for t in h] for h in st["y"]],
            "rho": fr(st["rho"]), "alpha": fr(st["alpha"])}


def exact_step(st, g, m, count, index, step, mode):
    n = len(g)
    limit = Fraction(1, 10 ** 10)          # the double constant 1e-10 differs from 10^-10 by 4e-27; no rho comes that close
    st["dir"] = [[-x for x in t] for t in g]
    for j in range(count - 1, -1, -1):
        idx = (index - count + j + m) % m
        rho = st["rho"][idx]
        if abs(rho) < limit:
            st["alpha"][j] = Fraction(0)
            continue
        a = rf32(exact_dot(st["s"][idx], st["dir"], mode, True) * rho)
        st["alpha"][j] = a
        st["dir"] = [[rf32(x - rf32(a * y)) for x, y in zip(st["dir"][i], st["y"][idx][i])] for i in range(n)]
    for j in range(count):
        idx = (index - count + j + m) % m
        rho = st["rho"][idx]
        if abs(rho) < limit:
            continue
        beta = rf32(exact_dot(st["y"][idx], st["dir"], mode, True) * rho)
        coeff = rf32(st["alpha"][j] - beta)
        st["dir"] = [[rf32(x + rf32(coeff * sv)) for x, sv in zip(st["dir"][i], st["s"][idx][i])] for i in range(n)]
    st["dir"] = [[-x for x in t] for t in st["dir"]]
    a = Fraction(float(F(step)))
    st["w"] = [[rf32(w + rf32(a * p)) for w, p in zip(st["w"][i], st["dir"][i])] for i in range(n)]
    st["old_g"] = [list(t) for t in g]
    st["s"][index] = [[rf32(a * p) for p in st["dir"][i]] for i in range(n)]
    if count > 0:
        prev = (index - 1 + m) % m
        st["y"][prev] = [[rf32(x - o) for x, o in zip(g[i], st["old_g"][i])] for i in range(n)]
        sdy = exact_dot(st["s"][prev], st["y"][prev], mode, False)
        st["rho"][prev] = rf32(Fraction(1) / sdy) if abs(sdy) > limit else Fraction(0)


def exact_bits(t):
    # a zero result carries no sign here; the numpy evaluator's -0.0 (from -g with g = +0) never
    # occurs in the cases (gradients are non-zero) and x - x gives +0 in both
    return [f32_bits(v) for v in t]


def assert_same_as_exact(cur, ex, where):
    for key in ("w", "old_g", "dir"):
        for i, t in enumerate(cur[key]):
            assert bits(t) == exact_bits(ex[key][i]), (where, key, i)
    for key in ("s", "y"):
        for h, tensors in enumerate(cur[key]):
            for i, t in enumerate(tensors):
                assert bits(t) == exact_bits(ex[key][h][i]), (where, key, h, i)
    assert bits(cur["rho"]) == exact_bits(ex["rho"]), (where, "rho")
    assert bits(cur["alpha"]) == exact_bits(ex["alpha"]), (where, "alpha")


def formula_array(seed, n, scale):
    """Platform-independent pseudo-random float32 values: a 32-bit multiplicative hash of the
    element index mapped to [-scale/2, scale/2) in binary64, then rounded to binary32.  Used
    for the case too large to store element by element (the test regenerates the inputs)."""
    i = np.arange(n, dtype=np.uint64)
    h = ((i + np.uint64(seed)) * np.uint64(2654435761)) & np.uint64(0xFFFFFFFF)
    h ^= h >> np.uint64(15)
    h = (h * np.uint64(2246822519)) & np.uint64(0xFFFFFFFF)
    h ^= h >> np.uint64(13)
    return ((h.astype(np.float64) / 4294967296.0 - 0.5) * scale).astype(F)


def digest(st):
    """sha256 over every tensor of the state in a fixed order."""
    hsh = hashlib.sha256()
    for key in ("w", "old_g", "dir"):
        for t in st[key]:
            hsh.update(np.ascontiguousarray(t, dtype=F).tobytes())
    for key in ("s", "y"):
        for h in st[key]:
            for t in h:
                hsh.update(np.ascontiguousarray(t, dtype=F).tobytes())
    return hsh.hexdigest()


def bits(a):
    return np.asarray(a, dtype=F).view(np.uint32).tolist()


def snapshot(st):
    return {
        "w": [bits(t) for t in st["w"]], "old_g": [bits(t) for t in st["old_g"]],
        "dir": [bits(t) for t in st["dir"]],
        "s": [[bits(t) for t in h] for h in st["s"]], "y": [[bits(t) for t in h] for h in st["y"]],
        "rho": bits(st["rho"]), "alpha": bits(st["alpha"]),
    }


def clone(st):
    return {
        "w": [t.copy() for t in st["w"]], "old_g": [t.copy() for t in st["old_g"]],
        "dir": [t.copy() for t in st["dir"]],
        "s": [[t.copy() for t in h] for h in st["s"]], "y": [[t.copy() for t in h] for h in st["y"]],
        "rho": st["rho"].copy(), "alpha": st["alpha"].copy(),
    }


def build_inputs(rng, sizes, m, steps, seeded_history, rho_values, grad_scale, formula_seed):
    """Initial state and per-step gradients of a case.  With formula_seed the values come from
    formula_array in a fixed call order, so a test can rebuild them from the case's header."""
    counter = [0]

    def rand(nel, scale):
        if formula_seed is not None:
            counter[0] += 1
            return formula_array(formula_seed + 7919 * counter[0], nel, scale * 4.0)
        return (rng.standard_normal(nel) * scale).astype(F)

    st = {
        "w": [rand(k, 0.5) for k in sizes], "old_g": [np.zeros(k, F) for k in sizes],
        "dir": [np.zeros(k, F) for k in sizes],
        "s": [[np.zeros(k, F) for k in sizes] for _ in range(m)],
        "y": [[np.zeros(k, F) for k in sizes] for _ in range(m)],
        "rho": np.zeros(m, F), "alpha": np.zeros(m, F),
    }
    if seeded_history:
        for h in range(m):
            st["s"][h] = [rand(k, 1e-2) for k in sizes]
            st["y"][h] = [rand(k, 1e-2) for k in sizes]
        st["rho"] = np.asarray(rho_values, dtype=F)
        st["old_g"] = [rand(k, grad_scale) for k in sizes]
        st["alpha"] = rand(m, 1.0)           # stale values that the step must overwrite or ignore
    grads = [[rand(k, grad_scale) for k in sizes] for _ in range(steps)]
    return st, grads


def make_case(name, rng, sizes, m, count, index, steps, step_size, seeded_history, rho_values=None,
              grad_scale=1e-2, formula_seed=None):
    st, grads = build_inputs(rng, sizes, m, steps, seeded_history, rho_values, grad_scale, formula_seed)
    case = {"name": name, "sizes": sizes, "history_size": m, "history_count": count,
            "history_index": index, "initial_step": float(F(step_size)), "expect": {}}
    if formula_seed is None:
        case["init"] = snapshot(st)
        case["grads"] = [[bits(t) for t in g] for g in grads]
    else:
        case["formula_seed"] = formula_seed
        case["seeded_history"] = bool(seeded_history)
        case["rho_values"] = [float(x) for x in rho_values]
        case["grad_scale"] = grad_scale
        case["steps"] = steps
        case["init_digest"] = digest(st)
    for mode in ("reference", "tree"):
        cur = clone(st)
        ex = exact_state(st)
        c, hi = count, index
        out = []
        for k, g in enumerate(grads):
            lbfgs_step(cur, g, m, c, hi, step_size, mode)
            exact_step(ex, [[Fraction(float(v)) for v in t] for t in g], m, c, hi, step_size, mode)
            assert_same_as_exact(cur, ex, (name, mode, k))     # the two evaluators must agree exactly
            hi = (hi + 1) % m                      # optimizer/lbfgs.go:287-290
            c = min(c + 1, m)
            if formula_seed is None:
                out.append(snapshot(cur))
            else:
                out.append({"digest": digest(cur), "rho": bits(cur["rho"]), "alpha": bits(cur["alpha"])})
        case["expect"][mode] = out
    return case


def main():
    rng = np.random.default_rng(0x6C626667)
    cases = [
        # empty history: the weights move by +initial_step * g
        make_case("empty_history", rng, [5, 3], 3, 0, 0, 1, 1.0, False),
        # optimizer/lbfgs.go's own sequence from the constructor's state: every rho stays 0
        make_case("natural_sequence", rng, [7, 2, 9], 2, 0, 0, 4, 0.5, False),
        # caller-provided history, one invalid pair (|rho| < 1e-10) in the middle
        make_case("seeded_history", rng, [6, 11], 3, 3, 1, 2, 0.25, True, [37.5, 3e-11, -12.25]),
        make_case("seeded_partial", rng, [4, 4, 4], 4, 2, 2, 2, 1.0, True, [8.0, 2.5, 99.0, 99.0]),
        # one-slot history: the slot written in step 6 is the one y and rho are formed from
        make_case("history_of_one", rng, [10], 1, 1, 0, 2, 0.125, True, [4.0]),
        # more than one slice per tensor and a ragged tail: the two summation orders differ
        make_case("multi_slice", rng, [2300, 70, 1024], 2, 2, 0, 1, 1.0, True, [150.0, -75.0], grad_scale=1.0,
                  formula_seed=20240),
    ]
    differ = sum(c["expect"]["reference"][0]["alpha"] != c["expect"]["tree"][0]["alpha"] for c in cases)
    assert differ >= 1, "no case separates the two summation orders"
    path = os.path.join(HERE, "lbfgs_kat.json")
    with open(path, "w") as f:
        json.dump({"cases": cases}, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes;", differ, "cases separate the summation orders")


if __name__ == "__main__":
    main()

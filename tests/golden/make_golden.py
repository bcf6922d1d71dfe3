#!/usr/bin/env python3
"""Writes tests/golden/optimizer_kat.json: known-answer vectors for the six update
rules and the mixed-precision Adam step.

Two evaluators, neither sharing code with oracle/oracle.c or the HIP kernels:

  * ExactF32 -- every graph node is computed exactly over the rationals
    (fractions.Fraction) and then rounded to binary32 by integer arithmetic
    (round-to-nearest-even, gradual underflow).  Square roots are rounded
    correctly by comparing against the exact midpoint.  This is "what IEEE-754
    fixes" for the op chain in cgo_bridge/bridge_optimizer.m.
  * numpy float32 ufuncs -- each ufunc call rounds once.

The script asserts that both agree bit for bit on every case before writing
the file.  Inputs include the vectors the reference's own bridge tests feed
(cgo_bridge/optimizer_test.go:54-59: w_i = 0.1*(i+1), g_i = 0.01*(i+1), n = 16,
and the hyper-parameter sets at :83-96, :264-280, :437-447, :502-513, :568-581);
the reference asserts no outputs for them, so the outputs here come from the
evaluators.

Run from the repo root:  python tests/golden/make_golden.py
"""
import json
import os
import random
import struct
from decimal import Decimal, getcontext
from fractions import Fraction
from math import isqrt

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


# ----------------------------------------------------------------------------
# exact rounding to a binary floating-point format
# ----------------------------------------------------------------------------
def _floor_log2(x: Fraction) -> int:
    e = x.numerator.bit_length() - x.denominator.bit_length()
    if Fraction(2) ** e > x:
        e -= 1
    elif Fraction(2) ** (e + 1) <= x:
        e += 1
    assert Fraction(2) ** e <= x < Fraction(2) ** (e + 1)
    return e


def _round_half_even(x: Fraction) -> int:
    n = x.numerator // x.denominator
    rem = x - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    return n


def round_to_format(x: Fraction, mant_bits: int, emin: int, emax: int):
    """Nearest value of the format to x (ties to even).  Returns a Fraction, or
    the string 'inf' / '-inf' on overflow.  mant_bits excludes the hidden bit."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    ax = abs(x)
    e = _floor_log2(ax)
    ue = max(e, emin) - mant_bits
    n = _round_half_even(ax / Fraction(2) ** ue)
    r = n * Fraction(2) ** ue
    if r >= Fraction(2) ** (emax + 1):
        return "inf" if sign > 0 else "-inf"
    return sign * r


def rf32(x):
    r = round_to_format(x, 23, -126, 127)
    if isinstance(r, str):
        raise OverflowError("binary32 overflow in a golden case")
    return r


def sqrt_f32(x: Fraction) -> Fraction:
    """Correctly rounded binary32 square root of an exact rational."""
    assert x >= 0
    if x == 0:
        return Fraction(0)
    e = _floor_log2(x) // 2            # floor(log2(sqrt x))
    ue = max(e, -126) - 23
    y = x / Fraction(4) ** ue          # sqrt(x) / 2^ue = sqrt(y)
    n = isqrt(y.numerator // y.denominator)
    mid = Fraction(n * n + n) + Fraction(1, 4)   # (n + 1/2)^2
    if y > mid or (y == mid and (n & 1)):
        n += 1
    return n * Fraction(2) ** ue


def f32_bits(x: Fraction) -> int:
    f = float(x)                       # exact: x is a binary32 value
    assert Fraction(f) == x
    return struct.unpack("<I", struct.pack("<f", f))[0]


def bits_f32(b: int) -> Fraction:
    return Fraction(struct.unpack("<f", struct.pack("<I", b))[0])


def lit(v: float) -> Fraction:
    """A decimal literal as the float32 constant a C/Go compiler would make."""
    return Fraction(float(np.float32(v)))


class X:
    """Exact-rational binary32 arithmetic: one rounding per operation."""
    add = staticmethod(lambda a, b: rf32(a + b))
    sub = staticmethod(lambda a, b: rf32(a - b))
    mul = staticmethod(lambda a, b: rf32(a * b))
    div = staticmethod(lambda a, b: rf32(a / b))
    sqrt = staticmethod(sqrt_f32)
    neg = staticmethod(lambda a: -a)


class N:
    """numpy float32 ufunc chain."""
    add = staticmethod(lambda a, b: np.add(a, b, dtype=np.float32))
    sub = staticmethod(lambda a, b: np.subtract(a, b, dtype=np.float32))
    mul = staticmethod(lambda a, b: np.multiply(a, b, dtype=np.float32))
    div = staticmethod(lambda a, b: np.divide(a, b, dtype=np.float32))
    sqrt = staticmethod(lambda a: np.sqrt(a, dtype=np.float32))
    neg = staticmethod(lambda a: np.negative(a))


# ----------------------------------------------------------------------------
# host scalars, correctly rounded (bridge_optimizer.m:398-399, :2066)
# ----------------------------------------------------------------------------
def pow_int_f32(base: Fraction, t: int) -> Fraction:
    return rf32(base ** t)


def pow_real_f32(base: Fraction, y: Fraction) -> Fraction:
    getcontext().prec = 80
    b = Decimal(base.numerator) / Decimal(base.denominator)
    yy = Decimal(y.numerator) / Decimal(y.denominator)
    r = (yy * b.ln()).exp()
    return rf32(Fraction(r))


def bias_corrections(beta1, beta2, t):
    one = Fraction(1)
    return rf32(one - pow_int_f32(beta1, t)), rf32(one - pow_int_f32(beta2, t))


def nadam_mu_next(beta1, t):
    exponent = rf32(Fraction(t + 1) * lit(0.004))
    decay = pow_real_f32(lit(0.96), exponent)
    half_decay = rf32(lit(0.5) * decay)
    one_minus = rf32(Fraction(1) - half_decay)
    return rf32(beta1 * one_minus)


# ----------------------------------------------------------------------------
# the update rules, written once over an arithmetic backend A (X or N)
# element-wise on python scalars (X) or numpy arrays (N)
# ----------------------------------------------------------------------------
def sgd(A, w, g, m, h):
    if h["weight_decay"] > 0:
        g = A.add(g, A.mul(w, h["weight_decay"]))
    if h["momentum"] > 0 and m is not None:
        m2 = A.add(A.mul(m, h["momentum"]), g)
        if h["nesterov"]:
            upd = A.mul(h["lr"], A.add(A.mul(h["momentum"], m2), g))
        else:
            upd = A.mul(h["lr"], m2)
        return A.sub(w, upd), m2
    return A.sub(w, A.mul(h["lr"], g)), m


def adam(A, w, g, m, v, h, bc1, bc2):
    m2 = A.add(A.mul(m, h["beta1"]), A.mul(g, h["omb1"]))
    v2 = A.add(A.mul(v, h["beta2"]), A.mul(A.mul(g, g), h["omb2"]))
    m_hat = A.div(m2, bc1)
    v_hat = A.div(v2, bc2)
    den = A.add(A.sqrt(v_hat), h["eps"])
    upd = A.div(m_hat, den)
    if h["weight_decay"] > 0:
        upd = A.add(upd, A.mul(w, h["weight_decay"]))
    return A.sub(w, A.mul(upd, h["lr"])), m2, v2


def rmsprop(A, w, g, s, b, ga, h):
    s2 = A.add(A.mul(s, h["alpha"]), A.mul(A.mul(g, g), h["oma"]))
    if h["centered"]:
        ga = A.add(A.mul(ga, h["alpha"]), A.mul(g, h["oma"]))
        den = A.sqrt(A.add(A.sub(s2, A.mul(ga, ga)), h["eps"]))
    else:
        den = A.sqrt(A.add(s2, h["eps"]))
    upd = A.div(g, den)
    if h["momentum"] > 0:
        b = A.add(A.mul(b, h["momentum"]), upd)
        upd = b
    if h["weight_decay"] > 0:
        upd = A.add(upd, A.mul(w, h["weight_decay"]))
    return A.sub(w, A.mul(upd, h["lr"])), s2, b, ga


def adagrad(A, w, g, s, h):
    if h["weight_decay"] > 0:
        g = A.add(g, A.mul(w, h["weight_decay"]))
    s2 = A.add(s, A.mul(g, g))
    den = A.add(A.sqrt(s2), h["eps"])
    alr = A.div(h["lr"], den)
    return A.sub(w, A.mul(alr, g)), s2


def adadelta(A, w, g, s, a, h):
    if h["weight_decay"] > 0:
        g = A.add(g, A.mul(w, h["weight_decay"]))
    s2 = A.add(A.mul(s, h["rho"]), A.mul(A.mul(g, g), h["omr"]))
    rms_g = A.sqrt(A.add(s2, h["eps"]))
    rms_u = A.sqrt(A.add(a, h["eps"]))
    d = A.mul(A.div(rms_u, rms_g), g)
    nd = A.neg(d)
    w2 = A.add(w, nd)
    a2 = A.add(A.mul(a, h["rho"]), A.mul(A.mul(nd, nd), h["omr"]))
    return w2, s2, a2


def nadam(A, w, g, m, v, h, bc1, bc2, mu, one_minus_mu):
    m2 = A.add(A.mul(m, h["beta1"]), A.mul(g, h["omb1"]))
    v2 = A.add(A.mul(v, h["beta2"]), A.mul(A.mul(g, g), h["omb2"]))
    v_hat = A.div(v2, bc2)
    m_hat = A.div(m2, bc1)
    g_hat = A.div(g, bc1)
    m_bar = A.add(A.mul(m_hat, mu), A.mul(g_hat, one_minus_mu))
    den = A.add(A.sqrt(v_hat), h["eps"])
    upd = A.div(m_bar, den)
    if h["weight_decay"] > 0:
        upd = A.add(upd, A.mul(w, h["weight_decay"]))
    return A.sub(w, A.mul(upd, h["lr"])), m2, v2


# ----------------------------------------------------------------------------
# case runner: evaluates a case with both backends and checks they agree
# ----------------------------------------------------------------------------
STATE_NAMES = {
    "sgd": ["m"], "adam": ["m", "v"], "rmsprop": ["s", "b", "ga"],
    "adagrad": ["s"], "adadelta": ["s", "a"], "nadam": ["m", "v"],
}


def derive(rule, hp):
    """Hyper-parameters as exact binary32 rationals plus the host-side
    derived constants (1 - beta etc., computed in binary32 like the host does)."""
    h = {k: (lit(v) if isinstance(v, float) else v) for k, v in hp.items()}
    one = Fraction(1)
    if rule in ("adam", "nadam"):
        h["omb1"] = rf32(one - h["beta1"])
        h["omb2"] = rf32(one - h["beta2"])
    if rule == "rmsprop":
        h["oma"] = rf32(one - h["alpha"])
    if rule == "adadelta":
        h["omr"] = rf32(one - h["rho"])
    return h


def to_np(h):
    return {k: (np.float32(float(v)) if isinstance(v, Fraction) else v) for k, v in h.items()}


def run_case(name, rule, hp, w0, grads, steps, first_step=1):
    """w0: list of Fractions; grads: list (len steps) of lists of Fractions."""
    n = len(w0)
    h = derive(rule, hp)
    hn = to_np(h)
    zero = [Fraction(0)] * n
    st = {k: list(zero) for k in STATE_NAMES[rule]}
    if rule == "sgd" and not hp["momentum"] > 0:
        st = {}
    w = list(w0)
    wn = np.array([float(x) for x in w0], dtype=np.float32)
    stn = {k: np.zeros(n, dtype=np.float32) for k in st}
    out_steps = []
    scalars = []
    for k in range(steps):
        t = first_step + k
        g = grads[k]
        gn = np.array([float(x) for x in g], dtype=np.float32)
        sc = {}
        if rule in ("adam", "nadam"):
            bc1, bc2 = bias_corrections(h["beta1"], h["beta2"], t)
            sc = {"bc1": f32_bits(bc1), "bc2": f32_bits(bc2)}
        if rule == "nadam":
            mu = nadam_mu_next(h["beta1"], t)
            omm = rf32(Fraction(1) - mu)
            sc["mu_next"] = f32_bits(mu)
        # exact evaluator, element by element
        for i in range(n):
            if rule == "sgd":
                w[i], m2 = sgd(X, w[i], g[i], st["m"][i] if st else None, h)
                if st:
                    st["m"][i] = m2
            elif rule == "adam":
                w[i], st["m"][i], st["v"][i] = adam(X, w[i], g[i], st["m"][i], st["v"][i], h, bc1, bc2)
            elif rule == "rmsprop":
                w[i], st["s"][i], st["b"][i], st["ga"][i] = rmsprop(
                    X, w[i], g[i], st["s"][i], st["b"][i], st["ga"][i], h)
            elif rule == "adagrad":
                w[i], st["s"][i] = adagrad(X, w[i], g[i], st["s"][i], h)
            elif rule == "adadelta":
                w[i], st["s"][i], st["a"][i] = adadelta(X, w[i], g[i], st["s"][i], st["a"][i], h)
            elif rule == "nadam":
                w[i], st["m"][i], st["v"][i] = nadam(X, w[i], g[i], st["m"][i], st["v"][i], h,
                                                     bc1, bc2, mu, omm)
        # numpy evaluator, whole arrays
        with np.errstate(all="ignore"):
            if rule == "sgd":
                wn, m2 = sgd(N, wn, gn, stn["m"] if stn else None, hn)
                if stn:
                    stn["m"] = m2
            elif rule == "adam":
                wn, stn["m"], stn["v"] = adam(N, wn, gn, stn["m"], stn["v"], hn,
                                              np.float32(float(bc1)), np.float32(float(bc2)))
            elif rule == "rmsprop":
                wn, stn["s"], stn["b"], stn["ga"] = rmsprop(N, wn, gn, stn["s"], stn["b"], stn["ga"], hn)
            elif rule == "adagrad":
                wn, stn["s"] = adagrad(N, wn, gn, stn["s"], hn)
            elif rule == "adadelta":
                wn, stn["s"], stn["a"] = adadelta(N, wn, gn, stn["s"], stn["a"], hn)
            elif rule == "nadam":
                wn, stn["m"], stn["v"] = nadam(N, wn, gn, stn["m"], stn["v"], hn,
                                               np.float32(float(bc1)), np.float32(float(bc2)),
                                               np.float32(float(mu)), np.float32(float(omm)))
        # the two evaluators must agree exactly
        rec = {"w": [f32_bits(x) for x in w]}
        assert rec["w"] == wn.view(np.uint32).tolist(), (name, "w", k)
        for key in st:
            rec[key] = [f32_bits(x) for x in st[key]]
            assert rec[key] == stn[key].view(np.uint32).tolist(), (name, key, k)
        out_steps.append(rec)
        scalars.append(sc)
    return {
        "name": name, "rule": rule, "hyper": hp, "n": n, "first_step": first_step,
        "w0": [f32_bits(x) for x in w0],
        "grads": [[f32_bits(x) for x in g] for g in grads],
        "scalars": scalars, "expect": out_steps,
    }


def ref_inputs(n=16):
    """cgo_bridge/optimizer_test.go:54-59 (Go evaluates both products in float32)."""
    w = [rf32(lit(0.1) * Fraction(i + 1)) for i in range(n)]
    g = [rf32(lit(0.01) * Fraction(i + 1)) for i in range(n)]
    return w, g


def rand_f32(rng, lo_exp, hi_exp):
    e = rng.uniform(lo_exp, hi_exp)
    v = np.float32(rng.choice([-1.0, 1.0]) * rng.uniform(1.0, 2.0) * 2.0 ** e)
    return Fraction(float(v))


# ----------------------------------------------------------------------------
# mixed-precision Adam: brute-force state machine over exact arithmetic
# ----------------------------------------------------------------------------
def f16_value(bits: int):
    sign = -1 if bits & 0x8000 else 1
    exp = (bits >> 10) & 0x1F
    man = bits & 0x3FF
    if exp == 0x1F:
        return None                      # inf / NaN
    if exp == 0:
        return sign * Fraction(man, 1 << 24)
    return sign * Fraction((1 << 10) | man) * Fraction(2) ** (exp - 25)


def f16_bits_from_value(x: Fraction) -> int:
    r = round_to_format(x, 10, -14, 15)
    if isinstance(r, str):
        return 0x7C00 if r == "inf" else 0xFC00
    sign = 0x8000 if x < 0 else 0        # zero results keep the sign of x (w' != 0 in cases)
    ar = abs(r)
    if ar == 0:
        return sign
    e = _floor_log2(ar)
    if e < -14:
        return sign | int(ar * (1 << 24))
    man = int(ar / Fraction(2) ** (e - 10)) - (1 << 10)
    return sign | ((e + 15) << 10) | man


F32_OVERFLOW = Fraction(2 ** 128 - 2 ** 103)      # values from here up round to +inf (ties to even)
F32_MIN_NORMAL = Fraction(1, 2 ** 126)


def run_amp_case(name, hp, amp, w0, g16_steps):
    """g16_steps: list of steps; each step is a list of tensors; each tensor a list of half bits."""
    h = derive("adam", hp)
    scale = lit(amp["init_scale"])
    growth = lit(amp["growth_factor"])
    backoff = lit(amp["backoff_factor"])
    interval = amp["growth_interval"]
    tracker = 0
    step_count = 0
    w = [list(t) for t in w0]
    m = [[Fraction(0)] * len(t) for t in w0]
    v = [[Fraction(0)] * len(t) for t in w0]
    w16 = [[0] * len(t) for t in w0]
    trace = []
    for g16 in g16_steps:
        found = any(f16_value(b) is None for t in g16 for b in t)
        if found:
            if rf32(scale * backoff) >= F32_MIN_NORMAL:      # the scale stays a normal, finite number
                scale = rf32(scale * backoff)
            tracker = 0
        else:
            step_count += 1
            bc1, bc2 = bias_corrections(h["beta1"], h["beta2"], step_count)
            inv = rf32(Fraction(1) / scale)
            for ti, t in enumerate(g16):
                for i, b in enumerate(t):
                    g = rf32(f16_value(b) * inv)
                    w[ti][i], m[ti][i], v[ti][i] = adam(X, w[ti][i], g, m[ti][i], v[ti][i], h, bc1, bc2)
                    w16[ti][i] = f16_bits_from_value(w[ti][i])
            tracker += 1
            if tracker == interval:
                if scale * growth < F32_OVERFLOW:                # the product rounds to a finite binary32
                    scale = rf32(scale * growth)
                tracker = 0
        trace.append({
            "skipped": int(found), "scale": f32_bits(scale), "growth_tracker": tracker,
            "step_count": step_count,
            "w": [[f32_bits(x) for x in t] for t in w],
            "m": [[f32_bits(x) for x in t] for t in m],
            "v": [[f32_bits(x) for x in t] for t in v],
            "w16": [list(t) for t in w16],
        })
    return {"name": name, "hyper": hp, "amp": amp,
            "w0": [[f32_bits(x) for x in t] for t in w0],
            "g16": g16_steps, "expect": trace}


def main():
    rng = random.Random(0x6D657461)
    cases = []
    w, g = ref_inputs()

    # the reference's own bridge-test inputs, five steps with the same gradient
    cases.append(run_case("ref_adam", "adam",
                          dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0001),
                          w, [g] * 5, 5))
    cases.append(run_case("ref_sgd_momentum", "sgd",
                          dict(lr=0.01, momentum=0.9, weight_decay=0.001, nesterov=False),
                          w, [g] * 5, 5))
    cases.append(run_case("ref_rmsprop", "rmsprop",
                          dict(lr=0.001, alpha=0.99, eps=1e-8, weight_decay=0.0001, momentum=0.0,
                               centered=False),
                          w, [g] * 5, 5))
    cases.append(run_case("ref_adagrad", "adagrad",
                          dict(lr=0.01, eps=1e-8, weight_decay=0.001), w, [g] * 5, 5))
    cases.append(run_case("ref_adadelta", "adadelta",
                          dict(rho=0.95, eps=1e-8, weight_decay=0.001), w, [g] * 5, 5))
    cases.append(run_case("ref_nadam", "nadam",
                          dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0001),
                          w, [g] * 5, 5))

    # the benchmark configurations' hyper-parameters, mixed signs and magnitudes, fresh gradient per step
    n = 24
    wr = [rand_f32(rng, -8, 1) for _ in range(n)]

    def grads(steps, lo, hi):
        return [[rand_f32(rng, lo, hi) for _ in range(n)] for _ in range(steps)]

    cases.append(run_case("adam_default_nodecay", "adam",
                          dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0),
                          wr, grads(6, -12, -4), 6))
    cases.append(run_case("adam_late_steps", "adam",
                          dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0001),
                          wr, grads(3, -12, -4), 3, first_step=1998))
    cases.append(run_case("sgd_vanilla", "sgd",
                          dict(lr=0.01, momentum=0.0, weight_decay=0.0, nesterov=False),
                          wr, grads(3, -12, -4), 3))
    cases.append(run_case("sgd_vanilla_decay", "sgd",
                          dict(lr=0.01, momentum=0.0, weight_decay=0.0005, nesterov=False),
                          wr, grads(3, -12, -4), 3))
    cases.append(run_case("sgd_nesterov", "sgd",
                          dict(lr=0.01, momentum=0.9, weight_decay=0.0, nesterov=True),
                          wr, grads(4, -12, -4), 4))
    cases.append(run_case("rmsprop_config3", "rmsprop",
                          dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0,
                               centered=False),
                          wr, grads(4, -14, -3), 4))
    cases.append(run_case("rmsprop_momentum_centered", "rmsprop",
                          dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0001, momentum=0.9,
                               centered=True),
                          wr, grads(4, -14, -3), 4))
    cases.append(run_case("adagrad_config3", "adagrad",
                          dict(lr=0.01, eps=1e-10, weight_decay=0.0), wr, grads(4, -14, -3), 4))
    cases.append(run_case("adadelta_config3", "adadelta",
                          dict(rho=0.9, eps=1e-6, weight_decay=0.0), wr, grads(4, -14, -3), 4))
    cases.append(run_case("nadam_config3", "nadam",
                          dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0),
                          wr, grads(4, -14, -3), 4))
    # extreme magnitudes: products underflow into the binary32 subnormal range
    wide = [rand_f32(rng, -30, 12) for _ in range(n)]
    cases.append(run_case("adam_wide_range", "adam",
                          dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0001),
                          wide, grads(3, -70, 10), 3))
    cases.append(run_case("adadelta_wide_range", "adadelta",
                          dict(rho=0.9, eps=1e-6, weight_decay=0.0), wide, grads(3, -60, 10), 3))

    # host scalars over a range of steps
    b1, b2 = lit(0.9), lit(0.999)
    scalar_table = []
    for t in list(range(1, 41)) + [100, 500, 1000, 1999, 2000, 2001, 3000, 4999, 5000]:
        bc1, bc2 = bias_corrections(b1, b2, t)
        scalar_table.append({"step": t, "bc1": f32_bits(bc1), "bc2": f32_bits(bc2),
                             "mu_next": f32_bits(nadam_mu_next(b1, t))})

    # mixed-precision Adam: 3 tensors, 14 steps, interval 4, overflow injected on steps 3, 4, 9
    sizes = [5, 8, 3]
    amp = dict(init_scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=4)
    hp = dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0001)
    w0 = [[rand_f32(rng, -6, 0) for _ in range(s)] for s in sizes]
    g16_steps = []
    inject = {3: (1, 2, 0x7C00), 4: (0, 0, 0xFC00), 9: (2, 1, 0x7E01)}
    for k in range(14):
        step = []
        for s in sizes:
            t = []
            for _ in range(s):
                # finite half: random sign, exponent field 1..29, random mantissa
                t.append((rng.getrandbits(1) << 15) | (rng.randint(1, 29) << 10) | rng.getrandbits(10))
            step.append(t)
        if k in inject:
            ti, i, b = inject[k]
            step[ti][i] = b
        g16_steps.append(step)
    amp_case = run_amp_case("amp_adam_small", hp, amp, w0, g16_steps)

    out = {"format": "uint32 values are IEEE binary32 bit patterns; g16/w16 are binary16 bit patterns",
           "cases": cases, "scalar_table": {"beta1": 0.9, "beta2": 0.999, "rows": scalar_table},
           "amp_cases": [amp_case]}
    path = os.path.join(HERE, "optimizer_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes;", len(cases), "cases")


if __name__ == "__main__":
    main()

"""Properties of the CPU oracle that the mathematics fixes (closed forms, invariants, library
casts): a dropped term, a wrong sign or a misplaced epsilon fails one of them."""
import ctypes

import numpy as np
import pytest

from oracle_lib import oracle

RNG = np.random.default_rng(2024)
N = 4096


def rand(scale, n=N):
    return (RNG.standard_normal(n) * scale).astype(np.float32)


def test_fp16_widening_matches_numpy_exhaustively():
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle().f16_to_f32(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp16_narrowing_matches_numpy():
    o = oracle()
    halves = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16).astype(np.float32)
    finite = np.sort(halves[np.isfinite(halves)].astype(np.float64))
    mids = ((finite[:-1] + finite[1:]) / 2).astype(np.float32)
    x = np.concatenate([halves[np.isfinite(halves)], mids, np.nextafter(mids, np.float32(np.inf)),
                        np.nextafter(mids, np.float32(-np.inf)),
                        np.array([65504.0, 65519.99, 65520.0, 1e10, -1e10, np.inf, -np.inf, 0.0, -0.0,
                                  5.9604645e-8, 2.9802322e-8, 2.9802325e-8, 1e-40], np.float32),
                        rand(1.0, 100000) * np.float32(10.0) ** RNG.integers(-9, 6, 100000).astype(np.float32)])
    x = x.astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(o.f32_to_f16(x), want)
    nan = o.f32_to_f16(np.array([np.nan], np.float32)).view(np.float16)
    assert np.isnan(nan[0])


def test_adam_first_step_closed_form():
    """t = 1, m = v = 0, wd = 0: m' = (1-b1) g, v' = (1-b2) g^2 and w' = w - lr * sign(g) for |g| >> eps."""
    w, g = rand(0.02), rand(1e-2)
    g[np.abs(g) < 1e-4] = np.float32(1e-3)
    w0 = w.copy()
    m, v = np.zeros(N, np.float32), np.zeros(N, np.float32)
    oracle().adam(w, g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    assert np.array_equal(m, g * (np.float32(1) - np.float32(0.9)))
    assert np.array_equal(v, (g * g) * (np.float32(1) - np.float32(0.999)))
    np.testing.assert_allclose(w0 - w, 1e-3 * np.sign(g), rtol=2e-4)


def test_adam_against_float64_formula_and_decay_order():
    """Ten steps against a float64 evaluation of the same formula; weight decay enters after the
    adaptive term and before the lr multiply, on the pre-update weight."""
    o = oracle()
    # the hyper-parameters as the binary32 constants the host passes, evaluated in float64
    lr, b1, b2, eps, wd = (float(np.float32(x)) for x in (1e-3, 0.9, 0.999, 1e-8, 1e-2))
    w, m, v = rand(0.5), np.zeros(N, np.float32), np.zeros(N, np.float32)
    w64, m64, v64 = w.astype(np.float64), np.zeros(N), np.zeros(N)
    for t in range(1, 11):
        g = rand(1e-2)
        o.adam(w, g, m, v, lr, b1, b2, eps, wd, t)
        g64 = g.astype(np.float64)
        m64 = b1 * m64 + (1 - b1) * g64
        v64 = b2 * v64 + (1 - b2) * g64 * g64
        upd = (m64 / (1 - b1 ** t)) / (np.sqrt(v64 / (1 - b2 ** t)) + eps) + wd * w64
        w64 = w64 - lr * upd
    np.testing.assert_allclose(w, w64, rtol=0, atol=2e-6)
    np.testing.assert_allclose(m, m64, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(v, v64, rtol=1e-5, atol=1e-12)
    # a decay applied to the gradient instead (the L2-into-grad variant) would differ visibly
    w2, m2, v2 = rand(0.5), np.zeros(N, np.float32), np.zeros(N, np.float32)
    g = np.zeros(N, np.float32)
    w2_0 = w2.copy()
    o.adam(w2, g, m2, v2, lr, b1, b2, eps, wd, 1)
    assert np.all(m2 == 0) and np.all(v2 == 0)                 # moments never see the decay
    np.testing.assert_allclose(w2, w2_0 * (1 - lr * wd), rtol=1e-6)   # zero gradient: w moves only by decay


def test_adam_wd_zero_matches_torch_loosely():
    """With wd = 0 torch.optim.Adam has the same epsilon placement; rounding order differs."""
    torch = pytest.importorskip("torch")
    w, m, v = rand(0.5, 512), np.zeros(512, np.float32), np.zeros(512, np.float32)
    p = torch.tensor(w.copy(), requires_grad=True)
    opt = torch.optim.Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
    for t in range(1, 6):
        g = rand(1e-2, 512)
        oracle().adam(w, g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0.0, t)
        p.grad = torch.tensor(g)
        opt.step()
    np.testing.assert_allclose(w, p.detach().numpy(), rtol=1e-5, atol=1e-7)


def test_sgd_closed_forms():
    o = oracle()
    w, g = rand(0.1), rand(1e-2)
    w0 = w.copy()
    o.sgd(w, g, None, 0.01, 0.0, 0.0, False)
    assert np.array_equal(w, w0 - np.float32(0.01) * g)            # vanilla: w - lr g
    # momentum: first step m = g, w = w - lr g; second step m = mu m + g
    w, m = w0.copy(), np.zeros(N, np.float32)
    o.sgd(w, g, m, 0.01, 0.9, 0.0, False)
    assert np.array_equal(m, g) and np.array_equal(w, w0 - np.float32(0.01) * g)
    o.sgd(w, g, m, 0.01, 0.9, 0.0, False)
    assert np.array_equal(m, g * np.float32(0.9) + g)
    # Nesterov: upd = lr (mu m' + g); L2 decay goes into the gradient before the momentum
    w, m = w0.copy(), np.zeros(N, np.float32)
    o.sgd(w, g, m, 0.01, 0.9, 0.1, True)
    g2 = g + w0 * np.float32(0.1)
    assert np.array_equal(m, g2)
    assert np.array_equal(w, w0 - np.float32(0.01) * (np.float32(0.9) * g2 + g2))


def test_adagrad_closed_form_and_monotone_state():
    o = oracle()
    w, g, s = rand(0.1), rand(1e-2), np.zeros(N, np.float32)
    w0 = w.copy()
    o.adagrad(w, g, s, 0.01, 1e-10, 0.0)
    assert np.array_equal(s, g * g)
    # first step: w - (lr / (|g| + eps)) g, with the quotient formed before the product
    want = w0 - (np.float32(0.01) / (np.sqrt(g * g) + np.float32(1e-10))) * g
    assert np.array_equal(w, want)
    prev = s.copy()
    for _ in range(5):
        o.adagrad(w, rand(1e-2), s, 0.01, 1e-10, 0.0)
        assert np.all(s >= prev)
        prev = s.copy()


def test_adadelta_first_step_closed_form():
    o = oracle()
    rho, eps = np.float32(0.9), np.float32(1e-6)
    w, g, s, a = rand(0.1), rand(1e-2), np.zeros(N, np.float32), np.zeros(N, np.float32)
    w0 = w.copy()
    o.adadelta(w, g, s, a, 0.9, 1e-6, 0.0)
    s1 = (g * g) * (np.float32(1) - rho)
    d = (np.sqrt(eps) / np.sqrt(s1 + eps)) * g
    assert np.array_equal(s, s1)
    assert np.array_equal(w, w0 - d)
    assert np.array_equal(a, (d * d) * (np.float32(1) - rho))
    assert np.all(a >= 0) and np.all(s >= 0)


def test_rmsprop_epsilon_inside_the_root_and_variants():
    o = oracle()
    w, g, s = rand(0.1), rand(1e-2), np.zeros(N, np.float32)
    w0 = w.copy()
    o.rmsprop(w, g, s, None, None, 0.01, 0.99, 1e-8, 0.0, 0.0, False)
    s1 = (g * g) * (np.float32(1) - np.float32(0.99))
    assert np.array_equal(s, s1)
    assert np.array_equal(w, w0 - (g / np.sqrt(s1 + np.float32(1e-8))) * np.float32(0.01))
    # zero gradient: the root is sqrt(eps), never a division by zero
    wz, sz = w0.copy(), np.zeros(N, np.float32)
    o.rmsprop(wz, np.zeros(N, np.float32), sz, None, None, 0.01, 0.99, 1e-8, 0.0, 0.0, False)
    assert np.array_equal(wz, w0)
    # momentum and centered states are persisted
    w, s, b, ga = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.float32)
    o.rmsprop(w, g, s, b, ga, 0.01, 0.99, 1e-8, 0.0, 0.9, True)
    ga1 = g * (np.float32(1) - np.float32(0.99))
    assert np.array_equal(ga, ga1)
    u = g / np.sqrt((s1 - ga1 * ga1) + np.float32(1e-8))
    assert np.array_equal(b, u) and np.array_equal(w, w0 - u * np.float32(0.01))


def test_nadam_against_float64_formula():
    o = oracle()
    lr, b1, b2, eps = (float(np.float32(x)) for x in (0.002, 0.9, 0.999, 1e-8))
    w, m, v = rand(0.5), np.zeros(N, np.float32), np.zeros(N, np.float32)
    w64, m64, v64 = w.astype(np.float64), np.zeros(N), np.zeros(N)
    for t in range(1, 8):
        g = rand(1e-2)
        o.nadam(w, g, m, v, lr, b1, b2, eps, 0.0, t)
        g64 = g.astype(np.float64)
        mu = b1 * (1 - 0.5 * 0.96 ** ((t + 1) * 0.004))
        m64 = b1 * m64 + (1 - b1) * g64
        v64 = b2 * v64 + (1 - b2) * g64 * g64
        bc1, bc2 = 1 - b1 ** t, 1 - b2 ** t
        mbar = mu * m64 / bc1 + (1 - mu) * g64 / bc1
        w64 = w64 - lr * mbar / (np.sqrt(v64 / bc2) + eps)
    np.testing.assert_allclose(w, w64, rtol=0, atol=3e-6)


def test_threaded_oracle_equals_scalar_oracle():
    o = oracle()
    n = 100003
    w, g = rand(0.02, n), rand(1e-2, n)
    a = [w.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)]
    b = [w.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)]
    for t in (1, 2, 3):
        o.adam(a[0], g, a[1], a[2], 1e-3, 0.9, 0.999, 1e-8, 1e-4, t, nthreads=1)
        o.adam(b[0], g, b[1], b[2], 1e-3, 0.9, 0.999, 1e-8, 1e-4, t, nthreads=8)
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))


def amp_reference_sequence(flags, init_scale, growth, backoff, interval):
    """Brute-force state machine in pure Python over a list of overflow flags."""
    scale, tracker, steps, out = np.float32(init_scale), 0, 0, []
    for f in flags:
        with np.errstate(over="ignore", under="ignore"):
            if f:
                lower = np.float32(scale * np.float32(backoff))
                scale, tracker = (lower if lower >= np.finfo(np.float32).tiny else scale), 0
            else:
                steps += 1
                tracker += 1
                if tracker == interval:
                    higher = np.float32(scale * np.float32(growth))
                    scale, tracker = (higher if np.isfinite(higher) else scale), 0
        out.append((int(f), float(scale), tracker, steps))
    return out


def test_amp_skip_and_scale_sequence_against_brute_force():
    o = oracle()
    rng = np.random.default_rng(7)
    sizes = [33, 7, 128]
    flags = rng.random(400) < 0.08
    st = o.amp_state(65536.0, 2.0, 0.5, 5)
    w = [rand(0.1, n) for n in sizes]
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    w16 = [np.zeros(n, np.uint16) for n in sizes]
    want = amp_reference_sequence(flags, 65536.0, 2.0, 0.5, 5)
    for k, f in enumerate(flags):
        # clipped so that only the injected elements overflow (the scale itself grows without bound here)
        g16 = [np.clip(rng.standard_normal(n) * 1e-4 * st.scale, -6e4, 6e4).astype(np.float16).view(np.uint16)
               for n in sizes]
        if f:
            t = int(rng.integers(0, len(sizes)))
            g16[t][int(rng.integers(0, sizes[t]))] = [0x7C00, 0xFC00, 0x7E00][k % 3]
        before = [a.copy() for a in w + m + v] + [a.copy() for a in w16]
        skipped = o.adam_amp(w, g16, m, v, w16, 1e-3, 0.9, 0.999, 1e-8, 0.0, st)
        assert (skipped, float(np.float32(st.scale)), st.growth_tracker, st.step_count) == want[k], k
        if skipped:                      # a skipped step leaves every buffer byte-identical
            for x, y in zip(before, w + m + v + w16):
                assert np.array_equal(x.view(np.uint8), y.view(np.uint8))
        else:
            for a, h in zip(w, w16):
                assert np.array_equal(h, a.astype(np.float16).view(np.uint16))


def test_amp_scale_stays_finite_and_normal():
    """Zero gradients never overflow, so the scale grows at every interval: it must stop at the largest
    finite power of two instead of reaching +inf (where inf * backoff = inf would hold it for good), and
    a run of overflows must stop at the smallest normal number instead of reaching zero.
    Perturbation tried: the two range checks removed from oracle.c -> this test fails at step 3 / 4."""
    o = oracle()
    n = [8]
    w, m, v, w16 = [rand(0.1, 8)], [np.zeros(8, np.float32)], [np.zeros(8, np.float32)], [np.zeros(8, np.uint16)]
    st = o.amp_state(2.0 ** 125, 2.0, 0.5, 1)
    zero = [np.zeros(8, np.uint16)]
    scales = []
    for _ in range(5):
        assert o.adam_amp(w, zero, m, v, w16, 1e-3, 0.9, 0.999, 1e-8, 0.0, st) == 0
        scales.append(float(st.scale))
    assert scales == [2.0 ** 126, 2.0 ** 127, 2.0 ** 127, 2.0 ** 127, 2.0 ** 127]
    assert [s for _, s, _, _ in amp_reference_sequence([0] * 5, 2.0 ** 125, 2.0, 0.5, 1)] == scales
    assert np.all(np.isfinite(w[0]))
    st = o.amp_state(2.0 ** -124, 2.0, 0.5, 1000)
    bad = [np.full(8, 0x7C00, np.uint16)]
    scales = []
    for _ in range(5):
        assert o.adam_amp(w, bad, m, v, w16, 1e-3, 0.9, 0.999, 1e-8, 0.0, st) == 1
        scales.append(float(st.scale))
    assert scales == [2.0 ** -125, 2.0 ** -126, 2.0 ** -126, 2.0 ** -126, 2.0 ** -126]
    assert [s for _, s, _, _ in amp_reference_sequence([1] * 5, 2.0 ** -124, 2.0, 0.5, 1000)] == scales


def test_fast_forms_of_the_fp16_conversions_equal_the_reference_forms_everywhere():
    """The bulk loops convert through inlined fast paths; over all 2^32 binary32 patterns and all 2^16
    binary16 patterns they return what gm_oracle_f32_to_f16 / gm_oracle_f16_to_f32 return (which are pinned
    against numpy exhaustively / on boundary sets in tests/test_oracle_golden.py)."""
    o = oracle()
    threads = min(8, __import__("os").cpu_count() or 1)
    assert o.lib.gm_oracle_f16_fast_mismatches(0, 1 << 32, 0, threads) == 0
    assert o.lib.gm_oracle_f16_fast_mismatches(0, 1 << 16, 1, 1) == 0


def test_vector_form_of_the_mixed_precision_step_equals_the_scalar_form():
    """Hosts with AVX2 + F16C run the applied mixed-precision step eight lanes at a time.  Both forms over
    the same inputs (every fp16 pattern as a gradient, inf and NaN included; weights and moments with random
    bit patterns, subnormals, zeros, negative second moments) must agree in every bit of w, m, v and w16 (a NaN
    result counts as equal to any NaN: payload propagation depends on operand order)."""
    o = oracle()
    rng = np.random.default_rng(99)
    n = 1 << 18
    g16 = np.tile(np.arange(1 << 16, dtype=np.uint16), n >> 16)
    rng.shuffle(g16)
    for case in range(4):
        if case == 0:        # ordinary training data
            w, m, v = rand(0.02, n), rand(1e-3, n), np.abs(rand(1e-6, n))
        elif case == 1:      # anything at all
            w, m, v = (rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32) for _ in range(3))
        elif case == 2:      # tiny values: subnormal moments and weights, underflowing fp16 copies
            w, m, v = rand(1e-6, n), rand(1e-39, n), np.abs(rand(1e-42, n))
        else:                # weights around the fp16 limits
            w, m, v = rand(40000.0, n), rand(1e-3, n), np.abs(rand(1e-6, n))
        for wd in (0.0, 1e-4):
            bad = o.lib.gm_oracle_amp_vector_mismatches(
                np.ascontiguousarray(w).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                g16.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)),
                np.ascontiguousarray(m).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                np.ascontiguousarray(v).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                n, 1e-3, 0.9, 0.999, 1e-8, wd, 0.1, 0.001, 1.0 / 65536.0)
            if bad == 2 ** 64 - 1:
                pytest.skip("this host has no AVX2 + F16C: the scalar form is the only one")
            assert bad == 0, (case, wd, bad)


# ---- pins that separate neighbouring formulas (each docstring names the perturbation of oracle.c it was
# ---- checked against: the test fails with that one line changed and passes with the line as it is)
F = np.float32


def nadam_mu_float64(beta1, t):
    """bridge_optimizer.m:2066 in float64: beta1 * (1 - 0.5 * 0.96^((t + 1) * 0.004))."""
    return float(F(beta1)) * (1.0 - 0.5 * 0.96 ** ((t + 1) * 0.004))


def test_nadam_momentum_schedule_is_taken_at_t_plus_one():
    """mu(t + 1), not mu(t): the two differ by 8e-5 relative, a thousand times the tolerance used here.
    Perturbation tried: `(float)(step + 1)` -> `(float)step` in gm_oracle_nadam_mu_next: fails at every t."""
    o = oracle()
    for t in (1, 2, 10, 250, 2500, 5000):
        got = float(o.nadam_mu_next(0.9, t))
        assert abs(got - nadam_mu_float64(0.9, t)) <= 2e-7 * abs(got), t
        assert abs(got - float(F(0.9)) * (1.0 - 0.5 * 0.96 ** (t * 0.004))) > 1e-5 * abs(got), t
    # and the schedule really moves between steps 1 and 250 (a constant mu would pass the check above at one t)
    assert float(o.nadam_mu_next(0.9, 250)) - float(o.nadam_mu_next(0.9, 1)) > 0.9 * 0.5 * 0.035


def nadam_first_step_float32(w, g, lr, b1, b2, eps, wd, mu):
    """t = 1, m = v = 0: every operation of bridge_optimizer.m:2114-2198 as one numpy float32 operation."""
    lr, b1, b2, eps, wd, mu = (F(x) for x in (lr, b1, b2, eps, wd, mu))
    one = F(1.0)
    bc1, bc2 = one - b1, one - b2                       # 1 - beta^1
    m = g * (one - b1)                                  # :2117-2120 with m = 0 (0 * beta1 + x = x exactly)
    v = (g * g) * (one - b2)                            # :2125-2134
    v_hat, m_hat, g_hat = v / bc2, m / bc1, g / bc1     # :2139-2148
    m_bar = m_hat * mu + g_hat * (one - mu)             # :2158-2164
    den = np.sqrt(v_hat) + eps                          # :2170-2171  epsilon OUTSIDE the root
    upd = m_bar / den                                   # :2176
    if wd > 0:
        upd = upd + w * wd                              # :2181-2190  decay after the adaptive term, on the old weight
    return w - upd * lr, m, v                           # :2193-2198


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_nadam_first_step_closed_form_bit_exact(wd):
    """First step against a chain of numpy float32 operations, with and without weight decay, on gradients
    spread over twelve decades (so that v_hat ranges from far below eps^2 to far above).
    Perturbations tried, each failing this test: eps moved inside the root (`sqrtf(v_hat + eps)`), `g_term`
    dropped from m_bar, decay added to the gradient instead of the update."""
    o = oracle()
    w = rand(0.5)
    g = (rand(1.0) * F(10.0) ** RNG.integers(-10, 2, N).astype(F)).astype(F)
    w0 = w.copy()
    m, v = np.zeros(N, F), np.zeros(N, F)
    o.nadam(w, g, m, v, 0.002, 0.9, 0.999, 1e-8, wd, 1)
    want_w, want_m, want_v = nadam_first_step_float32(w0, g, 0.002, 0.9, 0.999, 1e-8, wd, o.nadam_mu_next(0.9, 1))
    assert np.array_equal(m.view(np.uint32), want_m.view(np.uint32))
    assert np.array_equal(v.view(np.uint32), want_v.view(np.uint32))
    assert np.array_equal(w.view(np.uint32), want_w.view(np.uint32))


def test_epsilon_placement_where_it_decides_the_result():
    """Gradients of 1e-8, where sqrt(v_hat) equals eps: with eps outside the root the denominator is 2e-8,
    with eps inside it would be 1e-4, a factor of 5000 in the step.  Adam and NAdam put eps outside
    (bridge_optimizer.m:519-521, :2170-2171); RMSProp puts it inside (:827-830).
    Perturbations tried: Adam `sqrtf(v_hat) + eps` -> `sqrtf(v_hat + eps)`, the same for NAdam, and RMSProp
    `sqrtf(s_eps)` -> `sqrtf(si) + eps`: each fails its assertion below."""
    o = oracle()
    g = np.full(N, 1e-8, F)
    g[::2] *= F(-1)
    # Adam, t = 1: m_hat = g, v_hat = g^2  ->  step = lr * g / (|g| + eps) = lr / 2
    w, m, v = np.zeros(N, F), np.zeros(N, F), np.zeros(N, F)
    o.adam(w, g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    np.testing.assert_allclose(np.abs(w), 0.5e-3, rtol=1e-5)
    # NAdam, t = 1: m_bar = (mu + 10 (1 - mu)) g
    w, m, v = np.zeros(N, F), np.zeros(N, F), np.zeros(N, F)
    o.nadam(w, g, m, v, 0.002, 0.9, 0.999, 1e-8, 0.0, 1)
    mu = nadam_mu_float64(0.9, 1)
    np.testing.assert_allclose(np.abs(w), 0.002 * (mu + 10 * (1 - mu)) / 2, rtol=1e-4)
    # RMSProp: s = 0.01 g^2 = 1e-18, root = sqrt(1e-18 + 1e-8) ~ 1e-4  ->  step = lr * g / 1e-4 = 1e-6
    w, s = np.zeros(N, F), np.zeros(N, F)
    o.rmsprop(w, g, s, None, None, 0.01, 0.99, 1e-8, 0.0, 0.0, False)
    np.testing.assert_allclose(np.abs(w), 0.01 * 1e-8 / 1e-4, rtol=1e-4)


def test_adadelta_second_step_uses_the_previous_update_average():
    """Two steps as numpy float32 chains: the step-2 numerator is sqrt(E[dx^2] + eps) with the average as it
    stood BEFORE step 2 (bridge_optimizer.m:1807-1810 reads the buffer, :1832-1841 writes it afterwards).
    Only visible from the second step on (the first starts from zero either way).
    Perturbations tried: the update average advanced before rms_u is formed (which no first-step test can
    see), and rho used in place of (1 - rho) in the update average: both fail here."""
    o = oracle()
    rho, eps, one = F(0.9), F(1e-6), F(1.0)
    w, s, a = rand(0.1), np.zeros(N, F), np.zeros(N, F)
    ws, ss, as_ = w.copy(), s.copy(), a.copy()
    for step in range(2):
        g = rand(1e-2)
        o.adadelta(w, g, s, a, 0.9, 1e-6, 0.0)
        s_new = ss * rho + (g * g) * (one - rho)
        d = (np.sqrt(as_ + eps) / np.sqrt(s_new + eps)) * g          # as_ is the OLD average
        neg_d = -d
        ws = ws + neg_d
        as_ = as_ * rho + (neg_d * neg_d) * (one - rho)
        ss = s_new
        for got, want, name in ((w, ws, "w"), (s, ss, "s"), (a, as_, "a")):
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (step, name)
    assert np.all(a > 0)


def test_decay_order_for_every_rule_on_a_zero_gradient():
    """With g = 0 a rule that adds the decay to the UPDATE (Adam, NAdam, RMSProp: bridge_optimizer.m:531-540,
    :2181-2190, :857-866) moves w by exactly lr * (w * wd) and leaves every state at zero; a rule that adds it
    to the GRADIENT (SGD, AdaGrad, AdaDelta: :219-228, :1480-1488, :1773-1781) feeds it through its state.
    Perturbations tried: RMSProp and NAdam decay moved in front of the state update (`gi = gi + decay`): their
    state assertions fail; AdaGrad decay moved behind the adaptive term: its state assertion fails."""
    o = oracle()
    lr, wd = F(0.01), F(0.1)
    zero = np.zeros(N, F)
    w0 = rand(0.5)
    moved = w0 - (w0 * wd) * lr
    # decay on the update
    w, m, v = w0.copy(), zero.copy(), zero.copy()
    o.adam(w, zero, m, v, 0.01, 0.9, 0.999, 1e-8, 0.1, 1)
    assert np.array_equal(w, moved) and not m.any() and not v.any()
    w, m, v = w0.copy(), zero.copy(), zero.copy()
    o.nadam(w, zero, m, v, 0.01, 0.9, 0.999, 1e-8, 0.1, 1)
    assert np.array_equal(w, moved) and not m.any() and not v.any()
    w, s = w0.copy(), zero.copy()
    o.rmsprop(w, zero, s, None, None, 0.01, 0.99, 1e-8, 0.1, 0.0, False)
    assert np.array_equal(w, moved) and not s.any()
    # decay into the gradient
    gd = w0 * wd
    w, s = w0.copy(), zero.copy()
    o.adagrad(w, zero, s, 0.01, 1e-10, 0.1)
    assert np.array_equal(s, gd * gd)
    assert np.array_equal(w, w0 - (lr / (np.sqrt(gd * gd) + F(1e-10))) * gd)
    w, s, a = w0.copy(), zero.copy(), zero.copy()
    o.adadelta(w, zero, s, a, 0.9, 1e-6, 0.1)
    assert np.array_equal(s, (gd * gd) * (F(1.0) - F(0.9)))
    w, m = w0.copy(), zero.copy()
    o.sgd(w, zero, m, 0.01, 0.9, 0.1, False)
    assert np.array_equal(m, gd) and np.array_equal(w, w0 - lr * gd)


def test_rmsprop_second_step_with_decay_bit_exact():
    """Two plain RMSProp steps with weight decay as numpy float32 chains (bridge_optimizer.m:782-874): the
    running average multiplies the OLD state by alpha and the new square by (1 - alpha); the decay joins the
    update after the division.  Perturbation tried: alpha and (1 - alpha) swapped: fails at step 1."""
    o = oracle()
    alpha, eps, lr, wd, one = F(0.99), F(1e-8), F(0.01), F(1e-2), F(1.0)
    w, s = rand(0.5), np.zeros(N, F)
    ws, ss = w.copy(), s.copy()
    for step in range(2):
        g = rand(1e-2)
        o.rmsprop(w, g, s, None, None, 0.01, 0.99, 1e-8, 1e-2, 0.0, False)
        ss = ss * alpha + (g * g) * (one - alpha)
        upd = g / np.sqrt(ss + eps) + ws * wd
        ws = ws - upd * lr
        assert np.array_equal(s.view(np.uint32), ss.view(np.uint32)), step
        assert np.array_equal(w.view(np.uint32), ws.view(np.uint32)), step

"""Each pin in test_oracle_properties.py is shown to bite: oracle.c is rebuilt with ONE plausible mistake (a term
dropped, epsilon on the other side of the root, the decay folded in at the wrong place, a schedule taken at the wrong
step, two coefficients swapped, a bound removed) and the pin that is meant to catch it must then fail.  Unperturbed,
the same pins pass (they are part of this suite).  The perturbed builds live in a temporary folder; the pins run in a
child process that loads them through GM_ORACLE_SO."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
PINS = os.path.join(ROOT, "tests", "test_oracle_properties.py")

# (name, text in oracle.c, what it becomes, -k expression of the pins that must fail)
CASES = [
    ("NAdam momentum schedule taken at t instead of t + 1",
     "float exponent = (float)(step + 1) * 0.004f;", "float exponent = (float)(step) * 0.004f;",
     "test_nadam_momentum_schedule_is_taken_at_t_plus_one"),
    ("NAdam epsilon inside the root",
     "        float root = sqrtf(v_hat);              /* :2170 */\n        float den = root + eps;                 /* :2171 */",
     "        float root = sqrtf(v_hat + eps);\n        float den = root;",
     "test_nadam_first_step_closed_form_bit_exact or test_epsilon_placement"),
    ("NAdam gradient term dropped from the look-ahead",
     "float m_bar = m_term + g_term;          /* :2164 */", "float m_bar = m_term; (void)g_term;",
     "test_nadam_first_step_closed_form_bit_exact"),
    ("NAdam decay folded into the gradient",
     "        float gi = g[i];\n        float m_scaled = m[i] * beta1;          /* :2114 */",
     "        float gi = g[i] + (weight_decay > 0.0f ? w[i] * weight_decay : 0.0f);\n        float m_scaled = m[i] * beta1;",
     "test_nadam_first_step_closed_form_bit_exact or test_decay_order"),
    ("Adam epsilon inside the root",
     "    float root = sqrtf(v_hat);                 /* :519 */\n    float den = root + eps;                    /* :521 */",
     "    float root = sqrtf(v_hat + eps);\n    float den = root;",
     "test_epsilon_placement"),
    ("RMSProp epsilon outside the root",
     "            float s_eps = si + eps;\n            den = sqrtf(s_eps);", "            den = sqrtf(si) + eps;",
     "test_epsilon_placement or test_rmsprop_epsilon_inside"),
    ("AdaDelta numerator fed by the updated average",
     "        float a_eps = ai + eps;                /* :1807 */",
     "        ai = ai * rho + (gi * gi) * omr; float a_eps = ai + eps;",
     "test_adadelta_second_step"),
    ("AdaDelta rho and 1 - rho swapped in the update average",
     "        float d_sq_scaled = d_sq * omr;        /* :1838 */", "        float d_sq_scaled = d_sq * rho;",
     "test_adadelta_second_step"),
    ("RMSProp decay folded into the gradient",
     "        float gi = g[i];\n        float g_sq = gi * gi;                  /* :782 */",
     "        float gi = g[i] + (weight_decay > 0.0f ? w[i] * weight_decay : 0.0f);\n        float g_sq = gi * gi;",
     "test_decay_order"),
    ("AdaGrad decay dropped from the gradient",
     "            gi = gi + decay;\n        }\n        float g_sq = gi * gi;                  /* :1492 */",
     "            (void)decay;\n        }\n        float g_sq = gi * gi;",
     "test_decay_order"),
    ("RMSProp alpha and 1 - alpha swapped",
     "        float s_scaled = s[i] * alpha;         /* :785 */\n        float g_sq_scaled = g_sq * oma;        /* :788 */",
     "        float s_scaled = s[i] * oma;\n        float g_sq_scaled = g_sq * alpha;",
     "test_rmsprop_second_step_with_decay_bit_exact"),
    ("SGD Nesterov look-ahead built from the old momentum",
     "                float t1 = momentum * mi;", "                float t1 = momentum * m[i];",
     "test_sgd_closed_forms"),
    ("SGD momentum with dampening",
     "            float mi = scaled + gi;          /* :248 */", "            float mi = scaled + gi * (1.0f - momentum);",
     "test_sgd_closed_forms"),
    ("SGD decay applied to the weight instead of the gradient",
     "            float decay = wi * weight_decay;\n            gi = gi + decay;\n        }\n        if (use_momentum) {",
     "            wi = wi - lr * wi * weight_decay;\n        }\n        if (use_momentum) {",
     "test_sgd_closed_forms or test_decay_order"),
    ("Adam second-moment bias correction dropped",
     "    float v_hat = vi / bc2;                    /* :514 */", "    float v_hat = vi; (void)bc2;",
     "test_adam_first_step_closed_form or test_adam_against_float64_formula_and_decay_order"),
    ("Adam beta1 and 1 - beta1 swapped",
     "    float m_scaled = *m * beta1;               /* :484 */\n    float g_scaled = g * one_minus_beta1;      /* :487 */",
     "    float m_scaled = *m * one_minus_beta1;\n    float g_scaled = g * beta1;",
     "test_adam_first_step_closed_form"),
    ("Adam decay folded into the gradient",
     "    float m_scaled = *m * beta1;               /* :484 */",
     "    if (weight_decay > 0.0f) g = g + wi * weight_decay;\n    float m_scaled = *m * beta1;",
     "test_adam_against_float64_formula_and_decay_order or test_decay_order"),
    ("Adam decay scaled by nothing (applied after the learning rate)",
     "    float scaled = upd * lr;                   /* :543 */\n    *w = wi - scaled;                          /* :548 */",
     "    float scaled = (upd - (weight_decay > 0.0f ? wi * weight_decay : 0.0f)) * lr;\n    *w = wi - scaled - (weight_decay > 0.0f ? wi * weight_decay : 0.0f);",
     "test_adam_against_float64_formula_and_decay_order or test_decay_order"),
    ("AdaGrad epsilon inside the root",
     "        float root = sqrtf(si);                /* :1501 */\n        float den = root + eps;                /* :1503 */",
     "        float root = sqrtf(si + eps);\n        float den = root;",
     "test_adagrad_closed_form_and_monotone_state or test_epsilon_placement"),
    ("AdaGrad product formed before the quotient",
     "        float alr = lr / den;                  /* :1506 */\n        float upd = alr * gi;                  /* :1512 */",
     "        float alr = lr * gi;\n        float upd = alr / den;",
     "test_adagrad_closed_form_and_monotone_state"),
    ("AdaDelta epsilon outside the roots",
     "        float s_eps = si + eps;                /* :1800 */\n        float rms_g = sqrtf(s_eps);            /* :1803 */",
     "        float s_eps = si;\n        float rms_g = sqrtf(s_eps) + eps;",
     "test_adadelta_first_step_closed_form"),
    ("mixed precision: clean-step counter not reset by a dropped step",
     "        st->growth_tracker = 0;\n        return 1;", "        return 1;",
     "test_amp_skip_and_scale_sequence_against_brute_force"),
    ("mixed precision: a dropped step advances the step count",
     "        st->growth_tracker = 0;\n        return 1;", "        st->growth_tracker = 0;\n        st->step_count += 1;\n        return 1;",
     "test_amp_skip_and_scale_sequence_against_brute_force"),
    ("mixed precision: growth one step late",
     "    if (st->growth_tracker == st->growth_interval) {", "    if (st->growth_tracker > st->growth_interval) {",
     "test_amp_skip_and_scale_sequence_against_brute_force"),
    ("mixed precision: NaN gradients not treated as overflow",
     "            local |= ((g[i] & 0x7C00u) == 0x7C00u);", "            local |= ((g[i] & 0x7FFFu) == 0x7C00u);",
     "test_amp_skip_and_scale_sequence_against_brute_force"),
    ("mixed precision: no backoff on a dropped step",
     "        if (next >= FLT_MIN) st->scale = next;        /* the scale stays a normal number */", "        (void)next;",
     "test_amp_skip_and_scale_sequence_against_brute_force"),
    ("loss-scale growth unbounded",
     "        if (next <= FLT_MAX) st->scale = next;", "        st->scale = next;",
     "test_amp_scale_stays_finite"),
]


def run_case(case, folder, source="oracle.c", pin_file=PINS):
    name, old, new, pins = case
    src = open(os.path.join(ORACLE_DIR, source)).read()
    if src.count(old) != 1:
        return name, f"the line to perturb was not found exactly once in {source}"
    os.makedirs(folder, exist_ok=True)
    files = {f: os.path.join(ORACLE_DIR, f) for f in ("oracle.c", "oracle_lbfgs.c")}
    files[source] = os.path.join(folder, source)
    with open(files[source], "w") as f:
        f.write(src.replace(old, new))
    so = os.path.join(folder, "liboracle.so")
    build = subprocess.run(["gcc", "-O2", "-std=c11", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-w",
                            "-I", ORACLE_DIR, "-shared", "-o", so, files["oracle.c"], files["oracle_lbfgs.c"], "-lm"],
                           capture_output=True, text=True)
    if build.returncode != 0:
        return name, "the perturbed oracle did not build: " + build.stderr[-500:]
    r = subprocess.run([sys.executable, "-m", "pytest", pin_file, "-q", "-x", "-k", pins, "-p", "no:cacheprovider"],
                       env=dict(os.environ, GM_ORACLE_SO=so), capture_output=True, text=True)
    if r.returncode == 0:
        return name, f"NOT caught by: {pins}"
    if " failed" not in r.stdout:
        return name, "the pins did not run to a failure: " + (r.stdout + r.stderr)[-500:]
    return name, None


def test_every_perturbation_of_the_oracle_fails_its_pin(tmp_path):
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(lambda ic: run_case(ic[1], str(tmp_path / f"case{ic[0]}")), enumerate(CASES)))
    problems = [f"{name}: {why}" for name, why in results if why]
    assert not problems, "\n".join(problems)


LBFGS_PINS = os.path.join(ROOT, "tests", "test_oracle_lbfgs.py")
LBFGS_CASES = [
    ("recursion started from +g", "dir[i][k] = -g[i][k];", "dir[i][k] = g[i][k];", "test"),
    ("first loop adds alpha y", "dir[i][k] = dir[i][k] - alpha_j * yj[i][k];", "dir[i][k] = dir[i][k] + alpha_j * yj[i][k];", "test"),
    ("second loop uses alpha + beta", "const float coeff = alpha[j] - beta;", "const float coeff = alpha[j] + beta;", "test"),
    ("direction not negated after the recursion", "dir[i][k] = -dir[i][k];", "dir[i][k] = dir[i][k];", "test"),
    ("old gradient kept until after y is formed", "        memcpy(old_g[i], g[i], n[i] * sizeof(float));\n    }",
     "    }", "test"),
    ("history walked newest-last in the first loop",
     "    for (int j = history_count - 1; j >= 0; j--) {\n        const int idx = (history_index - history_count + j + history_size) % history_size;",
     "    for (int j = history_count - 1; j >= 0; j--) {\n        const int idx = (history_index - 1 - j + history_size) % history_size;",
     "test"),
    ("current step stored into the previous slot", "    const int cur = history_index;",
     "    const int cur = (history_index - 1 + history_size) % history_size;", "test"),
]


def test_every_perturbation_of_the_lbfgs_oracle_fails_its_pins(tmp_path):
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(lambda ic: run_case(ic[1], str(tmp_path / f"case{ic[0]}"), "oracle_lbfgs.c", LBFGS_PINS),
                                enumerate(LBFGS_CASES)))
    problems = [f"{name}: {why}" for name, why in results if why]
    assert not problems, "\n".join(problems)

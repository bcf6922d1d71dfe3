"""ctypes binding of oracle/liboracle.so (the CPU checker) for the tests, the smoke
check and the bench's cpu_baseline leg.  Never imported by the shipped package."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
# GM_ORACLE_SO points the tests at another build of the checker: how a deliberately perturbed oracle.c is
# shown to fail the pins in tests/test_oracle_properties.py
ORACLE_SO = os.environ.get("GM_ORACLE_SO") or os.path.join(ORACLE_DIR, "liboracle.so")

c_float_p = ctypes.POINTER(ctypes.c_float)
c_u16_p = ctypes.POINTER(ctypes.c_uint16)


class AmpState(ctypes.Structure):
    _fields_ = [("scale", ctypes.c_float), ("growth_tracker", ctypes.c_int32),
                ("growth_factor", ctypes.c_float), ("backoff_factor", ctypes.c_float),
                ("growth_interval", ctypes.c_int32), ("step_count", ctypes.c_uint64)]


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, "liboracle.so"])


def _fp(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(c_float_p)


def _hp(a):
    assert a.dtype == np.uint16 and a.flags.c_contiguous
    return a.ctypes.data_as(c_u16_p)


class Oracle:
    def __init__(self):
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        L = self.lib = ctypes.CDLL(ORACLE_SO)
        f, i, sz = ctypes.c_float, ctypes.c_int, ctypes.c_size_t
        L.gm_oracle_bias_corrections.argtypes = [f, f, i, c_float_p, c_float_p]
        L.gm_oracle_bias_corrections.restype = None
        L.gm_oracle_nadam_mu_next.argtypes = [f, i]
        L.gm_oracle_nadam_mu_next.restype = f
        L.gm_oracle_sgd_step.argtypes = [c_float_p, c_float_p, c_float_p, sz, f, f, f, i, i]
        L.gm_oracle_adam_step.argtypes = [c_float_p] * 4 + [sz, f, f, f, f, f, i, i]
        L.gm_oracle_rmsprop_step.argtypes = [c_float_p] * 5 + [sz, f, f, f, f, f, i, i]
        L.gm_oracle_adagrad_step.argtypes = [c_float_p] * 3 + [sz, f, f, f, i]
        L.gm_oracle_adadelta_step.argtypes = [c_float_p] * 4 + [sz, f, f, f, i]
        L.gm_oracle_nadam_step.argtypes = [c_float_p] * 4 + [sz, f, f, f, f, f, i, i]
        for fn in (L.gm_oracle_sgd_step, L.gm_oracle_adam_step, L.gm_oracle_rmsprop_step,
                   L.gm_oracle_adagrad_step, L.gm_oracle_adadelta_step, L.gm_oracle_nadam_step):
            fn.restype = None
        pp = ctypes.POINTER(c_float_p)
        L.gm_oracle_lbfgs_dot.argtypes = [pp, pp, ctypes.POINTER(sz), i, i, i]
        L.gm_oracle_lbfgs_dot.restype = f
        L.gm_oracle_lbfgs_step.argtypes = [pp] * 6 + [c_float_p, c_float_p, ctypes.POINTER(sz),
                                                      i, i, i, i, f, i, c_float_p]
        L.gm_oracle_lbfgs_step.restype = i
        L.gm_oracle_f32_to_f16.argtypes = [f]
        L.gm_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.gm_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.gm_oracle_f16_to_f32.restype = f
        L.gm_oracle_f16_fast_mismatches.argtypes = [ctypes.c_uint64, ctypes.c_uint64, i, i]
        L.gm_oracle_f16_fast_mismatches.restype = ctypes.c_uint64
        L.gm_oracle_amp_vector_mismatches.argtypes = [c_float_p, c_u16_p, c_float_p, c_float_p, sz] + [f] * 8
        L.gm_oracle_amp_vector_mismatches.restype = ctypes.c_uint64
        L.gm_oracle_convert_f32_to_f16.argtypes = [c_float_p, c_u16_p, sz, i]
        L.gm_oracle_convert_f32_to_f16.restype = None
        L.gm_oracle_convert_f16_to_f32.argtypes = [c_u16_p, c_float_p, sz, i]
        L.gm_oracle_convert_f16_to_f32.restype = None
        pp_f = ctypes.POINTER(c_float_p)
        pp_h = ctypes.POINTER(c_u16_p)
        L.gm_oracle_amp_found_inf.argtypes = [pp_h, ctypes.POINTER(sz), i, i]
        L.gm_oracle_amp_found_inf.restype = i
        L.gm_oracle_adam_amp_step.argtypes = [pp_f, pp_h, pp_f, pp_f, pp_h, ctypes.POINTER(sz), i,
                                              f, f, f, f, f, ctypes.POINTER(AmpState), i]
        L.gm_oracle_adam_amp_step.restype = i

    # ---- scalars ----
    def bias_corrections(self, beta1, beta2, step):
        a, b = ctypes.c_float(), ctypes.c_float()
        self.lib.gm_oracle_bias_corrections(beta1, beta2, step, ctypes.byref(a), ctypes.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def nadam_mu_next(self, beta1, step):
        return np.float32(self.lib.gm_oracle_nadam_mu_next(beta1, step))

    # ---- one tensor, in place ----
    def sgd(self, w, g, m, lr, momentum, weight_decay, nesterov, nthreads=1):
        self.lib.gm_oracle_sgd_step(_fp(w), _fp(g), _fp(m), w.size, lr, momentum, weight_decay,
                                    int(bool(nesterov)), nthreads)

    def adam(self, w, g, m, v, lr, beta1, beta2, eps, weight_decay, step, nthreads=1):
        self.lib.gm_oracle_adam_step(_fp(w), _fp(g), _fp(m), _fp(v), w.size, lr, beta1, beta2, eps,
                                     weight_decay, step, nthreads)

    def rmsprop(self, w, g, s, mom, gavg, lr, alpha, eps, weight_decay, momentum, centered, nthreads=1):
        self.lib.gm_oracle_rmsprop_step(_fp(w), _fp(g), _fp(s), _fp(mom), _fp(gavg), w.size, lr, alpha,
                                        eps, weight_decay, momentum, int(bool(centered)), nthreads)

    def adagrad(self, w, g, s, lr, eps, weight_decay, nthreads=1):
        self.lib.gm_oracle_adagrad_step(_fp(w), _fp(g), _fp(s), w.size, lr, eps, weight_decay, nthreads)

    def adadelta(self, w, g, s, a, rho, eps, weight_decay, nthreads=1):
        self.lib.gm_oracle_adadelta_step(_fp(w), _fp(g), _fp(s), _fp(a), w.size, rho, eps,
                                         weight_decay, nthreads)

    def nadam(self, w, g, m, v, lr, beta1, beta2, eps, weight_decay, step, nthreads=1):
        self.lib.gm_oracle_nadam_step(_fp(w), _fp(g), _fp(m), _fp(v), w.size, lr, beta1, beta2, eps,
                                      weight_decay, step, nthreads)

    # ---- L-BFGS ----
    DOT_REFERENCE, DOT_TREE = 0, 1

    def lbfgs_dot(self, a, b, mode, per_tensor=True):
        """a, b: lists of float32 arrays."""
        k = len(a)
        P = (c_float_p * k)
        sizes = (ctypes.c_size_t * k)(*[t.size for t in a])
        return np.float32(self.lib.gm_oracle_lbfgs_dot(P(*[_fp(t) for t in a]), P(*[_fp(t) for t in b]),
                                                       sizes, k, mode, 1 if per_tensor else 0))

    def lbfgs_step(self, st, g, history_size, history_count, history_index, initial_step, mode):
        """st: dict with lists of float32 arrays w, old_g, dir, s[h][i], y[h][i] and float32
        arrays rho, alpha (history_size each); updated in place.  Returns (code, step_size)."""
        k = len(g)
        P = (c_float_p * k)
        PH = (c_float_p * (k * history_size))
        sizes = (ctypes.c_size_t * k)(*[t.size for t in g])
        step = np.zeros(1, dtype=np.float32)
        rc = self.lib.gm_oracle_lbfgs_step(
            P(*[_fp(t) for t in st["w"]]), P(*[_fp(t) for t in g]), P(*[_fp(t) for t in st["old_g"]]),
            P(*[_fp(t) for t in st["dir"]]),
            PH(*[_fp(t) for h in st["s"] for t in h]), PH(*[_fp(t) for h in st["y"] for t in h]),
            _fp(st["rho"]), _fp(st["alpha"]), sizes, k, history_size, history_count, history_index,
            initial_step, mode, _fp(step))
        return rc, float(step[0])

    # ---- casts ----
    def f32_to_f16(self, src, nthreads=1):
        dst = np.empty(src.shape, dtype=np.uint16)
        self.lib.gm_oracle_convert_f32_to_f16(_fp(src), _hp(dst), src.size, nthreads)
        return dst

    def f16_to_f32(self, src, nthreads=1):
        dst = np.empty(src.shape, dtype=np.float32)
        self.lib.gm_oracle_convert_f16_to_f32(_hp(src), _fp(dst), src.size, nthreads)
        return dst

    # ---- mixed precision ----
    @staticmethod
    def amp_state(init_scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=2000):
        return AmpState(init_scale, 0, growth_factor, backoff_factor, growth_interval, 0)

    def adam_amp(self, w, g16, m, v, w16, lr, beta1, beta2, eps, weight_decay, state, nthreads=1):
        """Lists of numpy arrays (fp32 w/m/v, uint16 g16/w16), updated in place.
        Returns 1 if the step was skipped."""
        k = len(w)
        F = (c_float_p * k)
        H = (c_u16_p * k)
        sizes = (ctypes.c_size_t * k)(*[a.size for a in w])
        return self.lib.gm_oracle_adam_amp_step(
            F(*[_fp(a) for a in w]), H(*[_hp(a) for a in g16]), F(*[_fp(a) for a in m]),
            F(*[_fp(a) for a in v]), H(*[_hp(a) for a in w16]), sizes, k,
            lr, beta1, beta2, eps, weight_decay, ctypes.byref(state), nthreads)


_ORACLE = None


def oracle():
    global _ORACLE
    if _ORACLE is None:
        _ORACLE = Oracle()
    return _ORACLE

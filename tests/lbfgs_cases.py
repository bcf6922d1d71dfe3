"""Loads tests/golden/lbfgs_kat.json into numpy state dictionaries (shared by the CPU test of
the oracle and the GPU parity test)."""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
F = np.float32


def _arr(bits):
    return np.asarray(bits, dtype=np.uint32).view(F).copy()


def load_cases():
    with open(os.path.join(HERE, "golden", "lbfgs_kat.json")) as f:
        return json.load(f)["cases"]


def state_from_snapshot(snap):
    return {
        "w": [_arr(t) for t in snap["w"]], "old_g": [_arr(t) for t in snap["old_g"]],
        "dir": [_arr(t) for t in snap["dir"]],
        "s": [[_arr(t) for t in h] for h in snap["s"]], "y": [[_arr(t) for t in h] for h in snap["y"]],
        "rho": _arr(snap["rho"]), "alpha": _arr(snap["alpha"]),
    }


def state_digest(st):
    hsh = hashlib.sha256()
    for key in ("w", "old_g", "dir"):
        for t in st[key]:
            hsh.update(np.ascontiguousarray(t, dtype=F).tobytes())
    for key in ("s", "y"):
        for h in st[key]:
            for t in h:
                hsh.update(np.ascontiguousarray(t, dtype=F).tobytes())
    return hsh.hexdigest()


def case_inputs(case):
    """(initial state, list of per-step gradient lists) of a golden case."""
    if "formula_seed" not in case:
        return state_from_snapshot(case["init"]), [[_arr(t) for t in g] for g in case["grads"]]
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import make_lbfgs_golden as gen       # only its input formula; the expected values are in the JSON
    st, grads = gen.build_inputs(None, case["sizes"], case["history_size"], case["steps"],
                                 case["seeded_history"], case["rho_values"], case["grad_scale"],
                                 case["formula_seed"])
    assert state_digest(st) == case["init_digest"]
    return st, grads


def same_bits(a, b):
    """Bitwise equality of float32 arrays, any NaN equal to any NaN."""
    a = np.asarray(a, dtype=F)
    b = np.asarray(b, dtype=F)
    if a.shape != b.shape:
        return False
    both_nan = np.isnan(a) & np.isnan(b)
    return bool(np.all((a.view(np.uint32) == b.view(np.uint32)) | both_nan))


def check_against_expected(st, expect, where):
    if "digest" in expect:
        assert state_digest(st) == expect["digest"], where
    else:
        for key in ("w", "old_g", "dir"):
            for i, t in enumerate(st[key]):
                assert same_bits(t, _arr(expect[key][i])), (where, key, i)
        for key in ("s", "y"):
            for h, tensors in enumerate(st[key]):
                for i, t in enumerate(tensors):
                    assert same_bits(t, _arr(expect[key][h][i])), (where, key, h, i)
    assert same_bits(st["rho"], _arr(expect["rho"])), (where, "rho")
    assert same_bits(st["alpha"], _arr(expect["alpha"])), (where, "alpha")

"""The C-ABI library loads without a GPU and exports every symbol the headers declare."""
import ctypes
import glob
import os
import re

from __graft_entry__ import load_package

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text):
            name = m.group(1)
            if name not in ("defined", "sizeof", "__attribute__"):
                names.add(name)
    return names


def test_library_exports_every_declared_symbol():
    pkg = load_package()
    lib = pkg.load_library()
    names = declared_symbols()
    assert len(names) >= 35
    for name in sorted(names):
        assert hasattr(lib, name), f"{name} is declared in include/ but not exported"
    # and the ctypes view covers the whole header
    missing = names - set(pkg.ABI) - getattr(pkg, "HOST_ABI_NAMES", set())
    assert not missing, missing


def test_nil_device_is_rejected_before_anything_else():
    """Device 0 -> -1 from every step entry point (cgo_bridge/bridge_optimizer.m:175-178, 376-380),
    without touching the GPU."""
    pkg = load_package()
    lib = pkg.load_library()
    one = pkg.handle_array([0x1000])
    size = pkg.int_array([64])
    assert lib.execute_sgd_step_mpsgraph(0, one, one, one, 1, size, 0.01, 0.9, 0.0, 0, 1) == -1
    assert lib.execute_adam_step_mpsgraph(0, one, one, one, one, 1, size, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1) == -1
    assert lib.execute_adam_step_mpsgraph_pooled(0, one, one, one, one, 1, size, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0x2000) == -1
    assert lib.execute_adam_step_mpsgraph_pooled(0x1000, one, one, one, one, 1, size, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0) == -15
    assert lib.execute_rmsprop_step_mpsgraph(0, one, one, one, one, one, 1, size, 0.01, 0.99, 1e-8, 0.0, 0.0, False, 1) == -1
    assert lib.execute_adagrad_step_mpsgraph(0, one, one, one, 1, size, 0.01, 1e-10, 0.0) == -1
    assert lib.execute_adadelta_step_mpsgraph(0, one, one, one, one, 1, size, 0.9, 1e-6, 0.0) == -1
    assert lib.execute_nadam_step_mpsgraph(0, one, one, one, one, 1, size, 0.002, 0.9, 0.999, 1e-8, 0.0, 1) == -1
    assert lib.zero_metal_buffer(0, 0x1000, 64) == -1
    assert lib.zero_metal_buffer(0x1000, 0, 64) == -1
    assert lib.create_command_queue(0) == 0
    assert lib.allocate_metal_buffer(0, 64, 1) == 0
    assert lib.allocate_metal_buffer(0x1000, 0, 1) == 0
    assert lib.gm_synchronize(0) == -1


def test_copy_argument_checks_need_no_gpu():
    """bridge_memory.m:193-196, 223-226, 263-266, 327-339, 507-515."""
    pkg = load_package()
    lib = pkg.load_library()
    buf = (ctypes.c_float * 4)()
    assert lib.copy_float32_array_to_metal_buffer(0, buf, 4) == -1
    assert lib.copy_float32_array_to_metal_buffer(0x1000, None, 4) == -1
    assert lib.copy_float32_array_to_metal_buffer(0x1000, buf, 0) == -1
    assert lib.copy_metal_buffer_to_float32_array(0, buf, 4) == -1
    assert lib.copy_metal_buffer_to_float32_array(0x1000, buf, -1) == -1
    assert lib.copy_data_to_metal_buffer(0x1000, buf, 0) == -1
    shape = pkg.int_array([4])
    assert lib.convert_tensor_type(0, 0x1000, shape, 1, 0, 2, 0x1000) == -1
    assert lib.convert_tensor_type(0x1000, 0x1000, None, 1, 0, 2, 0x1000) == -1
    assert lib.convert_tensor_type(0x1000, 0x1000, shape, 0, 0, 2, 0x1000) == -1
    assert lib.convert_tensor_type(0x1000, 0x1000, shape, 1, 0, 2, 0) == -2
    assert lib.convert_tensor_type(0x1000, 0x1000, shape, 1, 0, 0, 0x1000) == -3
    assert lib.convert_tensor_type(0x1000, 0x1000, shape, 1, 1, 2, 0x1000) == -3
    assert lib.copy_buffer_to_buffer_sync(0, 0x1000, 0, 0, 4) == -1
    assert lib.copy_buffer_to_buffer_sync(0x1000, 0x1000, 0, 0, 0) == -2
    assert lib.copy_buffer_to_buffer_sync(0x1000, 0x1000, -4, 0, 4) == -2


def test_host_scalars_match_oracle():
    import numpy as np
    from oracle_lib import oracle
    pkg = load_package()
    lib = pkg.load_library()
    o = oracle()
    for t in list(range(1, 200)) + [1999, 2000, 4999, 5000, 100000]:
        a, b = ctypes.c_float(), ctypes.c_float()
        lib.gm_bias_corrections(0.9, 0.999, t, ctypes.byref(a), ctypes.byref(b))
        bc1, bc2 = o.bias_corrections(0.9, 0.999, t)
        assert np.float32(a.value) == bc1 and np.float32(b.value) == bc2, t
        assert np.float32(lib.gm_nadam_mu_next(0.9, t)) == o.nadam_mu_next(0.9, t), t


def test_headers_are_valid_c11(tmp_path):
    """cgo compiles the preamble as C: both headers must parse with a C compiler, warnings as errors."""
    import subprocess
    src = tmp_path / "abi_check.c"
    src.write_text('#include "gometal_hip.h"\n#include "gometal_optimizer.h"\n'
                   "uintptr_t (*const probe_a)(void) = create_metal_device;\n"
                   "int (*const probe_b)(uintptr_t, const uintptr_t *, int) = gmo_step;\n"
                   "int main(void) { return 0; }\n")
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src)])


def test_lbfgs_nil_device_and_history_checks_need_no_gpu():
    pkg = load_package()
    lib = pkg.load_library()
    one = pkg.handle_array([0x1000])
    size = pkg.int_array([64])
    step = ctypes.c_float(-1.0)
    args = (one, one, one, one, one, one, one, 0x1000, 1, size, 1, 0, 0, 1.0, 1e-4, 0.9, 20, 0.0, 0.0)
    assert lib.execute_lbfgs_step_mpsgraph(0, *args, ctypes.byref(step)) == -1      # bridge_optimizer.m:1005-1009
    assert lib.execute_lbfgs_step_mpsgraph_pooled(0, *args, 0x2000, ctypes.byref(step)) == -1
    assert step.value == -1.0


def test_prototypes_equal_the_references_cgo_preamble():
    """Return and parameter types of every function the reference's cgo preamble also declares
    (tests/golden/reference_prototypes.json, extracted from cgo_bridge/bridge.go) are the same in
    include/gometal_hip.h: the Go wrappers would compile against this header unchanged."""
    import json
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
    import make_reference_prototypes as gen
    with open(os.path.join(ROOT, "tests", "golden", "reference_prototypes.json")) as f:
        ref = json.load(f)["prototypes"]
    mine = gen.header_prototypes()
    assert len(ref) == 26
    for name, proto in ref.items():
        assert mine[name] == proto, (name, mine[name], proto)

"""Host-side mirror of the Go `optimizer` and `memory` packages: the behaviour the reference's
own GPU-less tests pin (mock optimizers, helper tables, pool maths), driven through
include/gometal_optimizer.h.  No GPU is needed: nothing here reaches a kernel."""
import json
import math

import numpy as np
import pytest

from __graft_entry__ import load_package

pkg = load_package()
lib = pkg.load_library()
MOCK_DEVICE = 0x1000      # memory.CreateMockDevice, memory/manager.go:322-326
MOCK_QUEUE = 0x2000


def f32(x):
    return float(np.float32(x))


@pytest.fixture
def mm():
    h = lib.gmo_memory_manager_new(MOCK_DEVICE)
    yield h
    lib.gmo_memory_manager_free(h)


def new(kind, config, shapes, mm, device=MOCK_DEVICE):
    return pkg.HostOptimizer(kind, config, shapes, mm, device)


# ---- config defaults: adam_test.go:129-153, sgd_test.go:13-38, rmsprop.go:54-63, adagrad.go:42-48,
# ---- adadelta.go:43-49, nadam.go:47-55
@pytest.mark.parametrize("kind,expected", [
    ("sgd", [0.01, 0.0, 0.0, 0.0]),
    ("adam", [0.001, 0.9, 0.999, 1e-8, 0.0]),
    ("rmsprop", [0.01, 0.99, 1e-8, 0.0, 0.0, 0.0]),
    ("adagrad", [0.01, 1e-10, 0.0]),
    ("adadelta", [0.95, 1e-6, 0.0]),
    ("nadam", [0.002, 0.9, 0.999, 1e-8, 0.0]),
])
def test_default_configs(kind, expected):
    import ctypes
    cfg = (ctypes.c_float * 6)()
    n = lib.gmo_default_config(pkg.KINDS[kind], cfg)
    assert n == len(expected)
    assert [cfg[k] for k in range(n)] == [f32(v) for v in expected]


# ---- constructor validation, in the order and with the strings of the Go constructors
def test_constructor_argument_errors(mm):
    for kind, cfg in [("sgd", [0.01, 0, 0, 0]), ("adam", [1e-3, .9, .999, 1e-8, 0]),
                      ("rmsprop", [.01, .99, 1e-8, 0, 0, 0]), ("adagrad", [.01, 1e-10, 0]),
                      ("adadelta", [.95, 1e-6, 0]), ("nadam", [.002, .9, .999, 1e-8, 0])]:
        assert new(kind, cfg, [[4]], 0).error == "memory manager cannot be nil"
        assert new(kind, cfg, [[4]], mm, device=0).error == "device cannot be nil"
        assert new(kind, cfg, [], mm).error == "no weight shapes provided"


def test_sgd_validation_messages(mm):                       # sgd.go:77-88
    assert new("sgd", [-0.01, 0, 0, 0], [[4]], mm).error == "learning rate cannot be negative: -0.010000"
    assert new("sgd", [0.01, -0.5, 0, 0], [[4]], mm).error == "momentum cannot be negative: -0.500000"
    assert new("sgd", [0.01, 1.5, 0, 0], [[4]], mm).error == "momentum cannot be greater than 1.0: 1.500000"
    assert new("sgd", [0.01, 0, -1, 0], [[4]], mm).error == "weight decay cannot be negative: -1.000000"


def test_adadelta_and_nadam_validation_messages(mm):        # adadelta.go:70-72, nadam.go:77-91
    assert new("adadelta", [0.0, 1e-6, 0], [[4]], mm).error == "rho must be in range (0, 1), got 0.000000"
    assert new("adadelta", [1.0, 1e-6, 0], [[4]], mm).error == "rho must be in range (0, 1), got 1.000000"
    assert new("nadam", [0.0, .9, .999, 1e-8, 0], [[4]], mm).error == "learning rate must be positive, got 0.000000"
    assert new("nadam", [.002, 1.0, .999, 1e-8, 0], [[4]], mm).error == "beta1 must be in [0, 1), got 1.000000"
    assert new("nadam", [.002, .9, -0.1, 1e-8, 0], [[4]], mm).error == "beta2 must be in [0, 1), got -0.100000"
    assert new("nadam", [.002, .9, .999, 0.0, 0], [[4]], mm).error == "epsilon must be positive, got 0.000000e+00"
    assert new("nadam", [.002, .9, .999, 1e-8, -1], [[4]], mm).error == "weight decay must be non-negative, got -1.000000"


@pytest.fixture
def vanilla_sgd(mm):
    """SGD without momentum allocates nothing, so it can be built without a GPU
    (the reference's MockSGDOptimizer, sgd_test.go)."""
    opt = new("sgd", [0.01, 0.0, 0.0, 0], [[10, 5], [5]], mm)
    assert opt.error is None
    yield opt
    opt.free()


def test_set_weight_buffers_length_check(vanilla_sgd):      # sgd.go:151-158
    assert vanilla_sgd.SetWeightBuffers([0x1000]) == "expected 2 weight buffers, got 1"
    assert vanilla_sgd.SetWeightBuffers([0x1000, 0x2000]) is None


def test_step_errors_and_step_count(vanilla_sgd):           # sgd_test.go:694-720
    vanilla_sgd.SetWeightBuffers([0x1000, 0x2000])
    err = vanilla_sgd.Step([0x1000])
    assert err == "gradient buffers length (1) doesn't match weight buffers length (2)"
    assert vanilla_sgd.GetStepCount() == 0
    # right count, but no GPU behind the mock device: the native step fails, the count stays incremented
    err = vanilla_sgd.Step([0x1000, 0x2000])
    if err is not None:
        assert err.startswith("SGD step execution failed: SGD step execution failed with error code: ")
    assert vanilla_sgd.GetStepCount() == 1


def test_set_command_pool_and_learning_rate(vanilla_sgd):   # adam_test.go:257-279, sgd.go:191-199
    assert lib.gmo_uses_pooling(vanilla_sgd.handle) == 0
    vanilla_sgd.SetCommandPool(MOCK_QUEUE)
    assert lib.gmo_uses_pooling(vanilla_sgd.handle) == 1
    vanilla_sgd.SetCommandPool(0)
    assert lib.gmo_uses_pooling(vanilla_sgd.handle) == 0
    vanilla_sgd.UpdateLearningRate(0.5)
    assert vanilla_sgd.field("LearningRate") == 0.5


def test_get_state_structure_without_buffers(vanilla_sgd):  # sgd.go:229-256
    text, err = vanilla_sgd.GetStateJSON()
    assert err is None
    st = json.loads(text)
    assert st["type"] == "SGD" and st["state_data"] == []
    assert set(st["parameters"]) == {"learning_rate", "momentum", "weight_decay", "nesterov", "step_count"}
    assert st["parameters"]["nesterov"] is False and st["parameters"]["step_count"] == 0
    assert np.float32(st["parameters"]["learning_rate"]) == np.float32(0.01)


def test_load_state_validation_and_tolerance(vanilla_sgd):  # adam_test.go:339-454 restated for SGD
    sgd = vanilla_sgd
    assert sgd.LoadStateJSON(json.dumps({"type": "InvalidType", "parameters": {}, "state_data": []})) == \
        "state type mismatch: expected SGD, got InvalidType"
    ok = {"type": "SGD", "parameters": {"learning_rate": 0.002, "momentum": 0.85, "weight_decay": 0.005,
                                        "nesterov": True, "step_count": 10}, "state_data": []}
    assert sgd.LoadStateJSON(json.dumps(ok)) is None
    assert sgd.field("LearningRate") == f32(0.002) and sgd.field("Momentum") == f32(0.85)
    assert sgd.field("WeightDecay") == f32(0.005) and sgd.field("Nesterov") == 1.0
    assert sgd.GetStepCount() == 10
    # missing parameters leave the fields alone
    assert sgd.LoadStateJSON(json.dumps({"type": "SGD", "parameters": {"learning_rate": 0.003}})) is None
    assert sgd.field("LearningRate") == f32(0.003) and sgd.field("Momentum") == f32(0.85)
    # wrong types are ignored, not errors
    assert sgd.LoadStateJSON(json.dumps({"type": "SGD", "parameters": {"learning_rate": "not_a_number",
                                                                      "momentum": 0.9}})) is None
    assert sgd.field("LearningRate") == f32(0.003) and sgd.field("Momentum") == f32(0.9)
    # a momentum tensor for an optimizer that has no momentum buffers (sgd.go:281-283)
    bad = {"type": "SGD", "parameters": {}, "state_data": [
        {"name": "momentum_0", "shape": [50], "data": [0.0] * 50, "state_type": "momentum"}]}
    assert sgd.LoadStateJSON(json.dumps(bad)) == "momentum buffer 0 not allocated"
    bad["state_data"][0]["name"] = "momentum_7"
    assert sgd.LoadStateJSON(json.dumps(bad)) == "invalid buffer index in tensor name: momentum_7"
    assert sgd.LoadStateJSON("{not json") .startswith("invalid optimizer state JSON")


def test_cleanup_clears_lists(vanilla_sgd):                 # sgd.go:212-226
    vanilla_sgd.Cleanup()
    assert vanilla_sgd.SetWeightBuffers([0x1000, 0x2000]) == "expected 0 weight buffers, got 2"


# ---- helper tables
@pytest.mark.parametrize("name,expected", [                  # state_helpers_test.go:316-365
    ("momentum_0", 0), ("variance_5", 5), ("squared_grad_avg_10", 10), ("momentum", -1),
    ("momentum_abc", -1), ("", -1), ("_", -1), ("momentum_buffer_5", 5), ("momentum_-1", -1),
    ("momentum_999", 999)])
def test_extract_buffer_index(name, expected):
    assert lib.gmo_extract_buffer_index(name.encode()) == expected


@pytest.mark.parametrize("shape,expected", [                 # state_helpers_test.go:212-246
    ([], 1), ([10], 10), ([10, 20], 200), ([5, 10, 20], 1000), ([2, 3, 4, 5], 120), ([1], 1), ([0], 0)])
def test_calculate_tensor_size(shape, expected):
    assert lib.gmo_calculate_tensor_size(pkg.int_array(shape) if shape else None, len(shape)) == expected


# ---- package memory
@pytest.mark.parametrize("requested,expected", [(100, 1024), (1024, 1024), (5000, 16384),
                                                (100000000, 100000000)])   # memory_test.go:219-227
def test_find_pool_size(mm, requested, expected):
    assert lib.gmo_find_pool_size(mm, requested) == expected


@pytest.mark.parametrize("size,expected", [(1024, 100), (4096, 100), (16384, 50), (65536, 50), (262144, 20),
                                           (1048576, 20), (4194304, 20), (16777216, 20), (67108864, 15)])
def test_reference_pool_caps_table(size, expected):           # memory_test.go:242-255
    assert lib.gmo_reference_max_pool_size(size) == expected
    # the cap in force is never below the reference's, and a 1B-parameter Adam state fits
    assert lib.gmo_calculate_max_pool_size(size) >= expected


def test_pool_caps_hold_transformer_sized_state():
    """28 tensors of 64 MB need 56 state buffers for Adam; the reference's cap of 15 refuses them."""
    assert lib.gmo_reference_max_pool_size(67108864) < 56 <= lib.gmo_calculate_max_pool_size(67108864)
    lib.gmo_set_pool_byte_budget(10 * 67108864)
    try:
        assert lib.gmo_calculate_max_pool_size(67108864) == 15      # budget below the reference cap: the cap wins
        lib.gmo_set_pool_byte_budget(100 * 67108864)
        assert lib.gmo_calculate_max_pool_size(67108864) == 100
    finally:
        lib.gmo_set_pool_byte_budget(128 << 30)


def test_allocate_without_global_manager_or_gpu_returns_nil(mm):   # manager.go:289-296
    # no global manager yet in this process (or no GPU behind it): AllocateBuffer signals failure by nil
    assert lib.gmo_allocate_buffer(mm, 1024) == 0 or lib.create_metal_device() != 0
    lib.gmo_release_buffer(mm, 0)      # nil is ignored


def normalize(doc):
    """The library's decoder followed by its encoder (no optimizer object, no GPU)."""
    import ctypes
    text = doc if isinstance(doc, str) else json.dumps(doc)
    p = lib.gmo_state_json_normalize(text.encode())
    if not p:
        return None, lib.gmo_last_error().decode()
    out = ctypes.string_at(p).decode()
    lib.gmo_free_string(p)
    return out, None


def test_optimizer_state_json_round_trip_is_exact():
    """Every float32 value the encoder writes decodes to the same bits, in this library's decoder and in
    Python's: 5000 random values over the whole exponent range, the extremes, signed zero, subnormals."""
    rng = np.random.default_rng(5)
    bits = np.concatenate([rng.integers(0, 1 << 32, 5000, dtype=np.uint64).astype(np.uint32),
                           np.array([0x00000000, 0x80000000, 0x00000001, 0x807FFFFF, 0x00800000, 0x7F7FFFFF,
                                     0xFF7FFFFF, 0x3F800000, 0x33D6BF95], np.uint32)])
    vals = bits.view(np.float32)
    vals = vals[np.isfinite(vals)]
    doc = {"type": "Adam", "parameters": {"learning_rate": 0.001, "step_count": 7},
           "state_data": [{"name": "momentum_0", "shape": [int(vals.size)],
                           "data": [float(v) for v in vals], "state_type": "momentum"}]}
    once, err = normalize(doc)
    assert err is None
    twice, err = normalize(once)
    assert err is None and twice == once                                   # a fixed point after one pass
    # ("-0" is an integer to Python's decoder, which would drop the sign: read every number as a float)
    back = np.array(json.loads(once, parse_int=float)["state_data"][0]["data"], np.float64).astype(np.float32)
    assert np.array_equal(back.view(np.uint32), vals.view(np.uint32))


def test_optimizer_state_json_shape_and_field_handling():
    """What Go's encoding/json would do with the same documents (optimizer/interface.go:47-51,
    checkpoints/checkpoint.go:81-86): key order of the parameter map, numbers as float64, unknown fields
    ignored, missing fields left empty, non-finite data not representable."""
    out, err = normalize({"type": "SGD", "parameters": {"z": 1, "a": 2.5, "m": True, "s": "x"}, "state_data": [],
                          "something_else": [1, 2, 3]})
    assert err is None
    assert out == '{"type":"SGD","parameters":{"a":2.5,"m":true,"s":"x","z":1},"state_data":[]}'
    out, err = normalize({"type": "RMSProp"})
    assert err is None and json.loads(out) == {"type": "RMSProp", "parameters": {}, "state_data": []}
    out, err = normalize('{"type":"Adam","parameters":{},"state_data":[{"name":"v_1","shape":[2],'
                         '"data":[1.5,null],"state_type":"variance"}]}')
    assert err is None                                      # "the JSON null value has no effect": the element stays 0
    assert json.loads(out)["state_data"][0]["data"] == [1.5, 0]
    out, err = normalize('{"type":"A","state_data":[{"name":"x","shape":[1],"data":[1],"state_type":"s"}],'
                         '"type":"B","state_data":[]}')
    assert err is None and json.loads(out) == {"type": "B", "parameters": {}, "state_data": []}   # last key wins
    for broken in ("", "{", '{"type":5}', '{"type":"Adam","parameters":[1]}', '{"type":"Adam","state_data":[{"shape":"x"}]}',
                   '{"type":"Adam"} trailing'):
        out, err = normalize(broken)
        assert out is None and err.startswith("invalid optimizer state JSON"), (broken, out, err)


def test_optimizer_state_json_numbers_follow_the_json_grammar():
    """Numbers are JSON numbers and nothing else: what strtod would also take (nan, inf, hex, a leading
    plus, a bare leading or trailing point) is refused, and so are values beyond the target type's
    range, as in encoding/json ("cannot unmarshal number 1e400 into Go value of type float64",
    "... number 1e39 into Go struct field .data of type float32", "... number 1.5 into ... of type int")."""
    param = '{"type":"Adam","parameters":{"a":%s},"state_data":[]}'
    for good in ("0", "-0", "12", "-1.5", "1e5", "1E-5", "0.5e+3", "1.7976931348623157e308", "4.9e-324"):
        out, err = normalize(param % good)
        assert err is None, (good, err)
    for bad in ("nan", "NaN", "-inf", "inf", "Infinity", "0x10", "+1", "01", "1.", ".5", "1e", "1e+", "--1", "1e400",
                "-1e400"):
        out, err = normalize(param % bad)
        assert out is None and err.startswith("invalid optimizer state JSON"), (bad, out)
    tensor = '{"type":"Adam","parameters":{},"state_data":[{"name":"m_0","shape":[%s],"data":[%s],"state_type":"m"}]}'
    for shape, data, ok in (("2", "1,2", True), ("2", "3.4028234e38,-3.4028234e38", True), ("1", "1e39", False),
                            ("1", "-1e39", False), ("1", "3.5e38", False), ("1.5", "1", False), ("1e10", "1", False),
                            ("-3", "1", True), ("null", "null", True)):
        out, err = normalize(tensor % (shape, data))
        assert (err is None) == ok, (shape, data, err)
    # a parameter of null is a nil interface value: present in no typed lookup, absent after re-encoding
    out, err = normalize(param % "null")
    assert err is None and json.loads(out)["parameters"] == {}
    # counts outside the uint64 range saturate (Go leaves the conversion implementation-defined)
    assert lib.gmo_extract_uint64_param(b'{"step_count":-5}', b"step_count", 7) == 0
    assert lib.gmo_extract_uint64_param(b'{"step_count":1e300}', b"step_count", 7) == 2 ** 64 - 1
    assert lib.gmo_extract_uint64_param(b'{"step_count":41}', b"step_count", 7) == 41


# ---- memory.Tensor helpers
@pytest.mark.parametrize("shape,dtype,expected", [          # memory_test.go:94-122
    ([], 0, 0), ([1], 0, 4), ([10], 0, 40), ([3, 4], 0, 48), ([2, 3, 4], 0, 96), ([10], 1, 40), ([10], 2, 20),
    ([10], 3, 10), ([10], 99, -1)])
def test_calculate_size(shape, dtype, expected):
    assert lib.gmo_calculate_size(pkg.int_array(shape) if shape else None, len(shape), dtype) == expected


def test_new_tensor_without_global_manager_or_gpu_fails_cleanly():
    if lib.gmo_get_global_memory_manager() == 0:
        assert lib.gmo_tensor_new(pkg.int_array([4]), 1, 0, 1) == 0
        assert lib.gmo_last_error().decode().startswith("failed to allocate buffer: ")


def test_precomputed_gradient_step_argument_errors(vanilla_sgd):   # engine/training_engine.go:108-124
    one = pkg.handle_array([0])
    assert lib.gmo_execute_step_with_precomputed_gradients(vanilla_sgd.handle, one, 1, one, 0) == -1
    assert lib.gmo_last_error().decode() == "weight tensors (1) and gradient tensors (0) count mismatch"
    two = pkg.handle_array([0, 0])
    assert lib.gmo_execute_step_with_precomputed_gradients(vanilla_sgd.handle, two, 2, two, 2) == -1
    assert lib.gmo_last_error().decode() == "weight tensor 0 is nil"
    assert lib.gmo_execute_step_with_precomputed_gradients(0, two, 2, two, 2) == -1
    assert lib.gmo_last_error().decode() == "Adam optimizer not initialized"


def test_optimizer_state_inside_a_reference_checkpoint_document(vanilla_sgd):
    """checkpoints/checkpoint.go:38-52: the optimizer state travels under "optimizer_state" of the
    JSON checkpoint (pretty-printed by saveJSON, :146-147).  Reading one back and writing one."""
    doc = json.dumps({
        "model_spec": {"layers": [{"name": "fc1", "type": 0, "params": {"a": [1, {"b": "}"}]}}]},
        "weights": [{"name": "fc1.weight", "shape": [2, 2], "data": [1.0, 2.0, 3.0, 4.0], "layer": "fc1", "type": "weight"}],
        "training_state": {"epoch": 3, "step": 42, "learning_rate": 0.01, "best_loss": 0.5, "best_accuracy": 0.9,
                           "total_steps": 42},
        "optimizer_state": {"type": "SGD", "parameters": {"learning_rate": 0.25, "momentum": 0.0, "nesterov": False,
                                                          "step_count": 42, "weight_decay": 0.125},
                            "state_data": []},
        "metadata": {"version": "1.0.0", "framework": "go-metal", "created_at": "2025-01-01T00:00:00Z"}}, indent=2)
    assert vanilla_sgd.LoadCheckpointJSON(doc) is None
    assert vanilla_sgd.field("LearningRate") == 0.25 and vanilla_sgd.field("WeightDecay") == 0.125
    assert vanilla_sgd.GetStepCount() == 42
    text, err = vanilla_sgd.GetCheckpointJSON()
    assert err is None
    out = json.loads(text)
    assert list(out) == ["model_spec", "weights", "training_state", "optimizer_state", "metadata"]
    assert out["optimizer_state"]["type"] == "SGD" and out["optimizer_state"]["parameters"]["step_count"] == 42
    assert out["metadata"]["framework"] == "go-metal"
    assert vanilla_sgd.LoadCheckpointJSON(json.dumps({"weights": [], "metadata": {}})) == "checkpoint has no optimizer state"
    assert vanilla_sgd.LoadCheckpointJSON(json.dumps({"optimizer_state": None})) == "checkpoint has no optimizer state"


# ---- learning-rate schedules (training/scheduler.go)
def test_lr_schedulers_follow_the_reference_formulas(vanilla_sgd):
    mk = lib.gmo_scheduler_new
    step = mk(0, 30, 0.1, 0.0, None)
    assert lib.gmo_scheduler_name(step) == b"StepLR"
    assert [lib.gmo_scheduler_get_lr(step, e, 0, 0.1) for e in (0, 29, 30, 65)] == \
        [0.1, 0.1, 0.1 * math.pow(0.1, 1.0), 0.1 * math.pow(0.1, 2.0)]
    bad = mk(0, -5, 7.0, 0.0, None)                       # invalid arguments fall back to 30 / 0.1 (scheduler.go:26-31)
    assert lib.gmo_scheduler_get_lr(bad, 30, 0, 1.0) == 0.1
    expo = mk(1, 0, 0.95, 0.0, None)
    assert lib.gmo_scheduler_get_lr(expo, 10, 0, 0.01) == 0.01 * math.pow(0.95, 10.0)
    cos = mk(2, 100, 1e-5, 0.0, None)
    assert lib.gmo_scheduler_get_lr(cos, 0, 0, 0.1) == 0.1
    assert lib.gmo_scheduler_get_lr(cos, 50, 0, 0.1) == 1e-5 + (0.1 - 1e-5) * (1 + math.cos(math.pi * 50 / 100)) / 2
    assert lib.gmo_scheduler_get_lr(cos, 100, 0, 0.1) == 1e-5 and lib.gmo_scheduler_get_lr(cos, 500, 0, 0.1) == 1e-5
    plateau = mk(3, 2, 0.5, 1e-4, b"min")
    assert lib.gmo_scheduler_name(plateau) == b"ReduceLROnPlateau"
    assert lib.gmo_scheduler_get_lr(plateau, 0, 0, 0.1) == 0.1          # not initialised yet: base LR
    seq = [lib.gmo_scheduler_plateau_step(plateau, m, 0.1) for m in (1.0, 0.9, 0.95, 0.95, 0.95, 0.5, 0.6, 0.6)]
    assert seq == [0.1, 0.1, 0.1, 0.05, 0.05, 0.05, 0.05, 0.025]
    assert lib.gmo_scheduler_get_lr(plateau, 9, 0, 0.1) == 0.025
    const = mk(4, 0, 0.0, 0.0, None)
    assert lib.gmo_scheduler_name(const) == b"ConstantLR" and lib.gmo_scheduler_get_lr(const, 7, 3, 0.3) == 0.3
    assert math.isnan(lib.gmo_scheduler_plateau_step(const, 1.0, 0.1))
    # fan-out to the optimizer (engine/model_engine.go:2332-2390): the float32 of the scheduled rate
    assert lib.gmo_scheduler_apply(expo, vanilla_sgd.handle, 3, 0, 0.01) == 0.01 * math.pow(0.95, 3.0)
    assert vanilla_sgd.field("LearningRate") == f32(0.01 * math.pow(0.95, 3.0))
    for h in (step, bad, expo, cos, plateau, const):
        lib.gmo_scheduler_free(h)


def test_lr_schedulers_reference_tables():
    """The known answers of the reference's own tests, with its tolerances (training/scheduler_test.go:8-108)."""
    mk = lib.gmo_scheduler_new
    step = mk(0, 2, 0.1, 0.0, None)                                   # TestStepLRScheduler
    for epoch, want in [(0, 0.1), (1, 0.1), (2, 0.01), (3, 0.01), (4, 0.001), (5, 0.001), (6, 0.0001)]:
        assert abs(lib.gmo_scheduler_get_lr(step, epoch, 0, 0.1) - want) <= 1e-8
    expo = mk(1, 0, 0.9, 0.0, None)                                   # TestExponentialLRScheduler
    for epoch, want in [(0, 0.1), (1, 0.09), (2, 0.081), (3, 0.0729), (4, 0.06561), (5, 0.059049)]:
        assert abs(lib.gmo_scheduler_get_lr(expo, epoch, 0, 0.1) - want) <= 1e-8
    cos = mk(2, 5, 0.0001, 0.0, None)                                 # TestCosineAnnealingLRScheduler
    for epoch, want in [(0, 0.01), (5, 0.0001), (2, 0.006580)]:
        assert abs(lib.gmo_scheduler_get_lr(cos, epoch, 0, 0.01) - want) <= 1e-6
    assert lib.gmo_scheduler_get_lr(cos, 10, 0, 0.01) == 0.0001
    plateau = mk(3, 2, 0.5, 0.01, b"min")                             # TestReduceLROnPlateauScheduler
    lr = lib.gmo_scheduler_plateau_step(plateau, 1.0, 0.1)
    assert lr == 0.1
    lr = lib.gmo_scheduler_plateau_step(plateau, 0.98, lr)
    assert lr == 0.1
    lr = lib.gmo_scheduler_plateau_step(plateau, 0.99, lr)
    assert lr == 0.1
    lr = lib.gmo_scheduler_plateau_step(plateau, 0.99, lr)
    assert lr == 0.05
    names = [(mk(0, 10, 0.1, 0.0, None), b"StepLR"), (mk(1, 0, 0.9, 0.0, None), b"ExponentialLR"),
             (mk(2, 10, 0.0, 0.0, None), b"CosineAnnealingLR"), (mk(3, 5, 0.5, 0.01, b"min"), b"ReduceLROnPlateau")]
    for h, want in names:                                             # TestSchedulerNames (:111-128)
        assert lib.gmo_scheduler_name(h) == want
    for h in [step, expo, cos, plateau] + [h for h, _ in names]:
        lib.gmo_scheduler_free(h)


# ---- optimizer/lbfgs.go without a GPU: lbfgs_test.go:11-32, 131-162 and the Go error strings ----
def test_lbfgs_default_config_and_constructor_errors(mm):
    cfg = pkg.HostLBFGS.default_config()
    assert cfg == (10, f32(1e-4), 20, f32(1e-4), f32(0.9), 1.0)
    assert pkg.HostLBFGS(cfg, [[10, 5]], 0, MOCK_DEVICE).error == "memory manager cannot be nil"
    assert pkg.HostLBFGS(cfg, [[10, 5]], mm, 0).error == "device cannot be nil"
    assert pkg.HostLBFGS(cfg, [], mm, MOCK_DEVICE).error == "no weight shapes provided"
    assert pkg.HostLBFGS((0,) + cfg[1:], [[10, 5]], mm, MOCK_DEVICE).error == \
        "history size must be positive, got 0"
    # without a GPU behind the manager the first allocation fails and everything is released
    opt = pkg.HostLBFGS(cfg, [[10, 5]], mm, MOCK_DEVICE)
    if lib.create_metal_device() == 0:
        assert opt.error == "failed to allocate s vector buffer for history 0, weight 0"
    else:
        opt.Cleanup()
        opt.free()


def test_nil_object_handles_are_errors_not_crashes():
    import ctypes
    assert lib.gmo_step(0, None, 0) == -1 and lib.gmo_last_error() == b"object handle is nil"
    assert lib.gmo_set_weight_buffers(0, None, 0) == -1
    assert lib.gmo_get_step_count(0) == 0
    assert lib.gmo_get_state_json(0) is None
    assert lib.gmo_load_state_json(0, b"{}") == -1
    assert math.isnan(lib.gmo_get_field(0, b"LearningRate"))
    assert lib.gmo_state_buffer(0, b"momentum", 0) == 0
    lib.gmo_cleanup(0)
    lib.gmo_update_learning_rate(0, 0.1)
    lib.gmo_optimizer_free(0)
    assert lib.gmo_lbfgs_step(0, None, 0, 1.0) == -1
    assert lib.gmo_lbfgs_get_step(0) == 0
    lib.gmo_lbfgs_cleanup(0)
    lib.gmo_lbfgs_free(0)
    assert lib.gmo_tensor_size(0) == -1 and lib.gmo_tensor_buffer(0) == 0
    assert lib.gmo_tensor_copy_from(0, 0) == -1
    lib.gmo_tensor_release(0)
    assert math.isnan(lib.gmo_scheduler_get_lr(0, 1, 1, 0.1))
    sched = lib.gmo_scheduler_new(0, 10, 0.5, 0.0, None)
    assert lib.gmo_scheduler_apply(sched, 0, 10, 0, 0.1) == pytest.approx(0.05)     # no optimizer to fan out to
    lib.gmo_scheduler_free(sched)


@pytest.mark.parametrize("x,y,expected", [(5.0, 0.0, 1.0), (5.0, 1.0, 5.0), (3.0, 2.0, 9.0), (2.0, 3.0, 8.0),
                                          (-2.0, 2.0, 4.0), (1.5, 2.0, 2.25)])
def test_pow_helper(x, y, expected):                        # adam_test.go:282-308
    assert lib.gmo_pow(x, y) == expected


def test_a_cpp_exception_stops_at_the_c_boundary(mm):
    """A standard-library exception inside an entry point (here: a negative dimension count, which makes the
    shape vector's constructor throw std::length_error) must come back as the entry point's failure value with
    the reason in gmo_last_error(), not unwind into the caller's C, Go or Python frames."""
    import ctypes
    cfg = (ctypes.c_float * 6)(0.01, 0, 0, 0, 0, 0)
    dims = (ctypes.c_int * 1)(4)
    ndims = (ctypes.c_int * 1)(-1)
    h = lib.gmo_optimizer_new(pkg.KINDS["sgd"], cfg, dims, ndims, 1, mm, MOCK_DEVICE)
    assert h == 0
    assert lib.gmo_last_error().decode().startswith("exception: ")
    # the library is still usable afterwards
    ndims[0] = 1
    h = lib.gmo_optimizer_new(pkg.KINDS["sgd"], cfg, dims, ndims, 1, mm, MOCK_DEVICE)
    assert h != 0
    lib.gmo_optimizer_free(h)


# ---- optimizer/state_helpers_test.go restated: the tables of the reference's own tests
@pytest.mark.parametrize("params,key,default,expected", [        # state_helpers_test.go:11-57
    ({"learning_rate": 0.01}, "learning_rate", 0.001, 0.01),
    ({"beta1": 0.9}, "learning_rate", 0.001, 0.001),
    ({"learning_rate": "0.01"}, "learning_rate", 0.001, 0.001),
    ({"learning_rate": 0.0}, "learning_rate", 0.001, 0.0),
])
def test_extract_float32_param(params, key, default, expected):
    got = lib.gmo_extract_float32_param(json.dumps(params).encode(), key.encode(), default)
    assert got == f32(expected)


@pytest.mark.parametrize("params,key,default,expected", [        # state_helpers_test.go:60-106
    ({"centered": True}, "centered", False, True),
    ({"nesterov": True}, "centered", False, False),
    ({"centered": "true"}, "centered", False, False),
    ({"centered": False}, "centered", True, False),
])
def test_extract_bool_param(params, key, default, expected):
    assert lib.gmo_extract_bool_param(json.dumps(params).encode(), key.encode(), int(default)) == int(expected)


@pytest.mark.parametrize("params,key,default,expected", [        # state_helpers_test.go:109-163
    ({"step_count": 100.0}, "step_count", 0, 100),
    ({"learning_rate": 0.01}, "step_count", 0, 0),
    ({"step_count": "100"}, "step_count", 0, 0),
    ({"step_count": 0.0}, "step_count", 5, 0),
    ({"step_count": 10.7}, "step_count", 0, 10),
])
def test_extract_uint64_param(params, key, default, expected):
    assert lib.gmo_extract_uint64_param(json.dumps(params).encode(), key.encode(), default) == expected


def test_extract_and_restore_buffer_state_messages():            # state_helpers_test.go:165-204
    import ctypes
    assert lib.gmo_extract_buffer_state(0, 64, b"test_buffer", b"momentum", None, 0) == 0     # nil: no tensor, no error
    data = (ctypes.c_float * 2)(1.0, 2.0)
    assert lib.gmo_restore_buffer_state(0, data, 2, 8, b"test_buffer") == -1
    assert lib.gmo_last_error().decode() == "test_buffer buffer is nil"
    assert lib.gmo_restore_buffer_state(MOCK_DEVICE, data, 2, 16, b"test_buffer") == -1
    assert lib.gmo_last_error().decode() == "data size mismatch for test_buffer: expected 4 elements, got 2"


@pytest.mark.parametrize("optimizer_type,state_type,ok", [       # state_helpers_test.go:260-308
    ("Adam", "Adam", True), ("Adam", "SGD", False), ("Adam", "", False), ("", "Adam", False)])
def test_validate_state_type(optimizer_type, state_type, ok):
    rc = lib.gmo_validate_state_type(optimizer_type.encode(), state_type.encode())
    assert (rc == 0) == ok
    if not ok:                                                    # interface.go:81
        assert lib.gmo_last_error().decode() == f"state type mismatch: expected {optimizer_type}, got {state_type}"

"""The host-side mirror of the Go `optimizer` / `memory` packages on the GPU: construction through
the pooled MemoryManager, Step against the oracle, GetState / LoadState checkpoint round trips
(resume-then-continue equals the uninterrupted run bit for bit), Cleanup, StepAMP."""
import json

import numpy as np
import pytest

from harness import OracleRun, gpu_device, states_for
from oracle_lib import oracle
from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
pkg = load_package()

CASES = [
    ("sgd", [0.01, 0.9, 1e-4, 1], dict(lr=0.01, momentum=0.9, weight_decay=1e-4, nesterov=True)),
    ("sgd", [0.01, 0.0, 0.0, 0], dict(lr=0.01, momentum=0.0, weight_decay=0.0, nesterov=False)),
    ("adam", [1e-3, 0.9, 0.999, 1e-8, 1e-4], dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)),
    ("rmsprop", [0.01, 0.99, 1e-8, 0.0, 0.0, 0],
     dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=0.0, momentum=0.0, centered=False)),
    ("rmsprop", [0.01, 0.99, 1e-8, 1e-4, 0.9, 1],
     dict(lr=0.01, alpha=0.99, eps=1e-8, weight_decay=1e-4, momentum=0.9, centered=True)),
    ("adagrad", [0.01, 1e-10, 1e-3], dict(lr=0.01, eps=1e-10, weight_decay=1e-3)),
    ("adadelta", [0.9, 1e-6, 0.0], dict(rho=0.9, eps=1e-6, weight_decay=0.0)),
    ("nadam", [0.002, 0.9, 0.999, 1e-8, 0.0], dict(lr=0.002, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)),
]
SHAPES = [[32, 3, 3, 3], [32], [300, 17], [1], [70000]]
STATE_TYPE = {"m": "momentum", "v": "variance", "s": "squared_grad_avg", "b": "momentum", "ga": "gradient_avg",
              "a": "squared_update_avg"}


@pytest.fixture(scope="module")
def env():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    dev.lib.gmo_initialize_global_memory_manager(dev.handle)
    mm = dev.lib.gmo_get_global_memory_manager()
    assert mm
    return dev, mm


def make(env, kind, cfg):
    dev, mm = env
    opt = pkg.HostOptimizer(kind, cfg, SHAPES, mm, dev.handle)
    assert opt.error is None, opt.error
    dev.lib.gmo_set_log_progress(opt.handle, 0)
    return opt


def read_states(dev, opt, kind, hyper, sizes):
    out = {}
    for name in states_for(kind, hyper):
        out[name] = [dev.to_numpy(opt.state_buffer(STATE_TYPE[name], k), n) for k, n in enumerate(sizes)]
    return out


@pytest.mark.parametrize("kind,cfg,hyper", CASES, ids=[f"{c[0]}-{i}" for i, c in enumerate(CASES)])
def test_step_checkpoint_resume(env, kind, cfg, hyper):
    dev, mm = env
    rng = np.random.default_rng(31)
    sizes = [int(np.prod(s)) for s in SHAPES]
    w0 = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    grads = [[rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes] for _ in range(8)]
    opt = make(env, kind, cfg)
    weights = [dev.from_numpy(w) for w in w0]
    gbufs = [dev.alloc(4 * n) for n in sizes]
    assert opt.SetWeightBuffers(weights) is None
    cpu = OracleRun(kind, hyper, w0)

    def step(o, k):
        for h, g in zip(gbufs, grads[k]):
            dev.upload(h, g)
        assert o.Step(gbufs) is None

    def check(o, wbufs):
        for k, n in enumerate(sizes):
            assert np.array_equal(dev.to_numpy(wbufs[k], n).view(np.uint32), cpu.w[k].view(np.uint32))
        got = read_states(dev, o, kind, hyper, sizes)
        for name, arrays in got.items():
            for k in range(len(sizes)):
                assert np.array_equal(arrays[k].view(np.uint32), cpu.state[name][k].view(np.uint32)), (name, k)

    for k in range(5):
        step(opt, k)
        cpu.step(grads[k])
    assert opt.GetStepCount() == 5
    check(opt, weights)

    # checkpoint: GetState -> JSON -> a fresh optimizer -> LoadState, weights copied
    text, err = opt.GetStateJSON()
    assert err is None
    st = json.loads(text)
    assert st["type"] == {"sgd": "SGD", "adam": "Adam", "rmsprop": "RMSProp", "adagrad": "AdaGrad",
                          "adadelta": "AdaDelta", "nadam": "Nadam"}[kind]
    assert st["parameters"]["step_count"] == 5
    names = [t["name"] for t in st["state_data"]]
    expected = [f"{STATE_TYPE[s]}_{k}" for s in states_for(kind, hyper) for k in range(len(sizes))]
    assert names == expected
    assert all(t["shape"] == [len(t["data"])] for t in st["state_data"])

    resumed = make(env, kind, cfg)
    weights2 = [dev.from_numpy(dev.to_numpy(h, n)) for h, n in zip(weights, sizes)]
    assert resumed.SetWeightBuffers(weights2) is None
    assert resumed.LoadStateJSON(text) is None
    assert resumed.GetStepCount() == 5
    for k in range(5, 8):
        step(opt, k)
        for h, g in zip(gbufs, grads[k]):
            dev.upload(h, g)
        assert resumed.Step(gbufs) is None
        cpu.step(grads[k])
    check(opt, weights)
    check(resumed, weights2)

    # a tensor of the wrong length is refused with the reference's message (state_helpers.go:41-42)
    if st["state_data"]:
        st["state_data"][0]["data"] = st["state_data"][0]["data"][:-1]
        first = st["state_data"][0]["name"]
        assert resumed.LoadStateJSON(json.dumps(st)) == \
            f"data size mismatch for {first}: expected {sizes[0]} elements, got {sizes[0] - 1}"

    for o in (opt, resumed):
        o.Cleanup()
        o.free()
    for h in weights + weights2 + gbufs:
        dev.free(h)


def pool_allocated(dev, mm, tier):
    import ctypes
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    if dev.lib.gmo_pool_stats(mm, tier, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) != 0:
        return 0, 0
    return a.value, b.value


def test_pool_reuses_released_state_buffers(env):
    """Cleanup returns the state buffers to their size tier; the next optimizer draws them from
    the pool (no new device allocation) and finds them zeroed."""
    dev, mm = env
    tiers = sorted({dev.lib.gmo_find_pool_size(mm, 4 * int(np.prod(s))) for s in SHAPES})
    opt = make(env, "adam", CASES[2][1])
    opt.Cleanup()
    opt.free()
    before = {t: pool_allocated(dev, mm, t) for t in tiers}
    again = make(env, "adam", CASES[2][1])
    after = {t: pool_allocated(dev, mm, t) for t in tiers}
    for t in tiers:
        assert after[t][1] == before[t][1], "a pooled buffer was available, yet a new one was allocated"
        assert after[t][0] < before[t][0]
    for k, shape in enumerate(SHAPES):
        n = int(np.prod(shape))
        assert not dev.to_numpy(again.state_buffer("momentum", k), n).any()
        assert not dev.to_numpy(again.state_buffer("variance", k), n).any()
    again.Cleanup()
    again.free()


def test_large_state_exceeds_reference_pool_cap(env):
    """Twenty 64 MB-tier state tensors for Adam = 40 buffers of one pool; the reference's cap is 15."""
    dev, mm = env
    shapes = [[4096, 4096]] * 20
    opt = pkg.HostOptimizer("adam", CASES[2][1], shapes, mm, dev.handle)
    assert opt.error is None, opt.error
    import ctypes
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert dev.lib.gmo_pool_stats(mm, 67108864, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) == 0
    assert b.value >= 40 and c.value >= 40
    opt.Cleanup()
    opt.free()


def test_step_amp_through_the_mirror(env):
    dev, mm = env
    rng = np.random.default_rng(8)
    sizes = [int(np.prod(s)) for s in SHAPES]
    cfg, hyper = CASES[2][1], CASES[2][2]
    opt = make(env, "adam", cfg)
    skipped, err = opt.StepAMP([0] * len(sizes))
    assert err == "mixed precision is not enabled: call EnableMixedPrecision first"
    assert opt.EnableMixedPrecision(65536.0, 2.0, 0.5, 3) is None
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    w16 = [np.zeros(n, np.uint16) for n in sizes]
    dw = [dev.from_numpy(a) for a in w]
    dw16 = [dev.alloc(2 * n + 2, zero=True) for n in sizes]
    dg = [dev.alloc(2 * n + 2) for n in sizes]
    assert opt.SetWeightBuffers(dw) is None
    st = oracle().amp_state(65536.0, 2.0, 0.5, 3)
    for k in range(9):
        g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
        if k in (2, 6):
            g16[4][100] = 0x7C00
        for h, g in zip(dg, g16):
            dev.upload(h, g)
        skipped, err = opt.StepAMP(dg, dw16)
        assert err is None
        want = oracle().adam_amp(w, g16, m, v, w16, state=st, **hyper)
        assert skipped == bool(want)
        assert opt.GetStepCount() == st.step_count
        assert dev.lib.gmo_loss_scale(opt.handle) == float(np.float32(st.scale))
        assert dev.lib.gmo_growth_tracker(opt.handle) == st.growth_tracker
    for k, n in enumerate(sizes):
        assert np.array_equal(dev.to_numpy(dw[k], n).view(np.uint32), w[k].view(np.uint32))
        assert np.array_equal(dev.to_numpy(dw16[k], n, np.uint16), w16[k])
    # the loss-scale state travels with the checkpoint
    text, err = opt.GetStateJSON()
    params = json.loads(text)["parameters"]
    assert params["loss_scale"] == float(np.float32(st.scale)) and params["growth_tracker"] == st.growth_tracker
    opt.Cleanup()
    opt.free()
    for h in dw + dw16 + dg:
        dev.free(h)


def test_step_amp_async_through_the_mirror(env):
    """StepAMPAsync mixed with Step and StepAMP: the device keeps the step count while steps are
    pending, and every host-side reader of StepCount catches up first."""
    dev, mm = env
    rng = np.random.default_rng(18)
    sizes = [int(np.prod(s)) for s in SHAPES]
    cfg, hyper = CASES[2][1], CASES[2][2]
    opt = make(env, "adam", cfg)
    assert opt.StepAMPAsync([0] * len(sizes)) == "mixed precision is not enabled: call EnableMixedPrecision first"
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    dw = [dev.from_numpy(a) for a in w]
    dw16 = [dev.alloc(2 * n + 2, zero=True) for n in sizes]
    dg32 = [dev.alloc(4 * n) for n in sizes]
    dg = [dev.alloc(2 * n + 2) for n in sizes]
    assert opt.SetWeightBuffers(dw) is None
    ref = OracleRun("adam", hyper, w)
    # two plain fp32 steps first: StepCount = 2 before mixed precision starts
    for _ in range(2):
        g = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
        for h, a in zip(dg32, g):
            dev.upload(h, a)
        assert opt.Step(dg32) is None
        ref.step(g)
    assert opt.EnableMixedPrecision(4096.0, 2.0, 0.5, 2) is None
    st = oracle().amp_state(4096.0, 2.0, 0.5, 2)
    st.step_count = 2
    m, v = ref.state["m"], ref.state["v"]
    w16 = [np.zeros(n, np.uint16) for n in sizes]
    skipped_want = 0
    for k in range(7):
        g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
        if k in (1, 4):
            g16[2][7] = 0xFC00
        for h, g in zip(dg, g16):
            dev.upload(h, g)
        assert opt.StepAMPAsync(dg, dw16) is None
        skipped_want += oracle().adam_amp(ref.w, g16, m, v, w16, state=st, **hyper)
    assert opt.GetStepCount() == st.step_count == 7          # 2 + 7 - 2 dropped; the call waits for the steps
    skipped, err = opt.SyncAMP()
    assert err is None and skipped == skipped_want == 2
    assert dev.lib.gmo_loss_scale(opt.handle) == float(np.float32(st.scale))
    assert dev.lib.gmo_growth_tracker(opt.handle) == st.growth_tracker
    # a synchronous mixed-precision step and a plain step continue from there
    g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
    for h, g in zip(dg, g16):
        dev.upload(h, g)
    skipped, err = opt.StepAMP(dg, dw16)
    assert err is None and not skipped
    oracle().adam_amp(ref.w, g16, m, v, w16, state=st, **hyper)
    ref.step_count = st.step_count
    g = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
    for h, a in zip(dg32, g):
        dev.upload(h, a)
    assert opt.Step(dg32) is None
    ref.step(g)
    assert opt.GetStepCount() == ref.step_count == 9
    # and one more asynchronous step after the plain one (the host pushes its count to the device)
    st.step_count = 9
    g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
    for h, gg in zip(dg, g16):
        dev.upload(h, gg)
    assert opt.StepAMPAsync(dg, dw16) is None
    oracle().adam_amp(ref.w, g16, m, v, w16, state=st, **hyper)
    text, err = opt.GetStateJSON()                            # catches up before reading
    assert err is None and json.loads(text)["parameters"]["step_count"] == 10
    for k, n in enumerate(sizes):
        assert np.array_equal(dev.to_numpy(dw[k], n).view(np.uint32), ref.w[k].view(np.uint32)), k
        assert np.array_equal(dev.to_numpy(dw16[k], n, np.uint16), w16[k]), k
        assert np.array_equal(dev.to_numpy(opt.state_buffer("momentum", k), n).view(np.uint32), m[k].view(np.uint32))
    opt.Cleanup()
    opt.free()
    for h in dw + dw16 + dg + dg32:
        dev.free(h)


def test_enabling_mixed_precision_again_keeps_the_current_ping_pong_set(env):
    """EnableMixedPrecision called a second time (another initial scale, say) replaces the loss-scale state on the
    device.  After an odd number of applied ping-pong steps the shadow set is the current one: the new state must
    be told, or the next step would read the stale set A and overwrite the real weights in B."""
    dev, mm = env
    rng = np.random.default_rng(23)
    sizes = [int(np.prod(s)) for s in SHAPES]
    cfg, hyper = CASES[2][1], CASES[2][2]
    for applied_before in (1, 2):
        opt = make(env, "adam", cfg)
        w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
        dw = [dev.from_numpy(a) for a in w]
        w16 = [a.astype(np.float16).view(np.uint16) for a in w]
        dw16 = [dev.from_numpy(h) for h in w16]
        dg = [dev.alloc(2 * n + 2) for n in sizes]
        m = [np.zeros(n, np.float32) for n in sizes]
        v = [np.zeros(n, np.float32) for n in sizes]
        assert opt.SetWeightBuffers(dw) is None
        assert opt.EnableMixedPrecision(4096.0, 2.0, 0.5, 100) is None and opt.EnablePingPong() is None
        st = oracle().amp_state(4096.0, 2.0, 0.5, 100)

        def step(use_async):
            g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
            for h, g in zip(dg, g16):
                dev.upload(h, g)
            if use_async:
                assert opt.StepAMPAsync(dg, dw16) is None
            else:
                assert opt.StepAMP(dg, dw16) == (False, None)
            assert oracle().adam_amp(w, g16, m, v, w16, state=st, **hyper) == 0

        for k in range(applied_before):
            step(use_async=(k == applied_before - 1))          # the last one still in flight when the state is replaced
        # a new loss-scale state with another scale; the oracle's state is replaced the same way
        assert opt.EnableMixedPrecision(1024.0, 2.0, 0.5, 7) is None
        assert opt.current_set() == applied_before % 2 and opt.GetStepCount() == applied_before
        st2 = oracle().amp_state(1024.0, 2.0, 0.5, 7)
        st2.step_count = st.step_count
        st = st2
        for k in range(3):
            step(use_async=False)
        assert opt.current_set() == (applied_before + 3) % 2 and opt.GetStepCount() == applied_before + 3
        for k, n in enumerate(sizes):
            for name, host in (("weight", w), ("momentum", m), ("variance", v)):
                assert np.array_equal(dev.to_numpy(opt.state_buffer(name, k), n).view(np.uint32), host[k].view(np.uint32)), (applied_before, name, k)
            assert np.array_equal(dev.to_numpy(dw16[k], n, np.uint16), w16[k]), (applied_before, k)
        opt.Cleanup()
        opt.free()
        for h in dw + dw16 + dg:
            dev.free(h)


def test_ping_pong_mixed_precision_through_the_mirror(env):
    """EnablePingPong: StepAMP / StepAMPAsync run the one-pass step over two sets of weights and moments.  The
    current weights (state_buffer "weight"), the moments GetState reads, the fp16 copy and every counter follow
    the oracle through synchronous steps, dropped steps, asynchronous steps, a plain fp32 step and a checkpoint
    round trip into a second ping-pong optimizer; Cleanup returns the shadow buffers to the pool."""
    dev, mm = env
    rng = np.random.default_rng(19)
    sizes = [int(np.prod(s)) for s in SHAPES]
    cfg, hyper = CASES[2][1], CASES[2][2]
    opt = make(env, "adam", cfg)
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    dw = [dev.from_numpy(a) for a in w]
    w16 = [a.astype(np.float16).view(np.uint16) for a in w]
    dw16 = [dev.from_numpy(h) for h in w16]                      # the fp16 copy starts as half of the weights
    dg = [dev.alloc(2 * n + 2) for n in sizes]
    dg32 = [dev.alloc(4 * n) for n in sizes]
    assert opt.EnablePingPong() == "mixed precision is not enabled: call EnableMixedPrecision first"
    assert opt.SetWeightBuffers(dw) is None
    assert opt.EnableMixedPrecision(4096.0, 2.0, 0.5, 3) is None
    tier = dev.lib.gmo_find_pool_size(mm, 4 * sizes[4])
    before_alloc = pool_allocated(dev, mm, tier)
    assert opt.EnablePingPong() is None and opt.current_set() == 0
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    st = oracle().amp_state(4096.0, 2.0, 0.5, 3)

    def grads(inject):
        g16 = [(rng.normal(0, 1e-4, n) * st.scale).astype(np.float16).view(np.uint16) for n in sizes]
        if inject:
            g16[4][100] = 0x7C00
        for h, g in zip(dg, g16):
            dev.upload(h, g)
        return g16

    def check(o, context):
        for k, n in enumerate(sizes):
            assert np.array_equal(dev.to_numpy(o.state_buffer("weight", k), n).view(np.uint32), w[k].view(np.uint32)), (context, k)
            assert np.array_equal(dev.to_numpy(o.state_buffer("momentum", k), n).view(np.uint32), m[k].view(np.uint32)), (context, k)
            assert np.array_equal(dev.to_numpy(o.state_buffer("variance", k), n).view(np.uint32), v[k].view(np.uint32)), (context, k)
            assert np.array_equal(dev.to_numpy(dw16[k], n, np.uint16), w16[k]), (context, k)

    applied = 0
    for k in range(6):                                           # synchronous steps, two of them dropped
        g16 = grads(k in (0, 3))
        skipped, err = opt.StepAMP(dg, dw16)
        assert err is None
        want = oracle().adam_amp(w, g16, m, v, w16, state=st, **hyper)
        applied += 0 if want else 1
        assert skipped == bool(want) and opt.current_set() == applied % 2
        assert opt.GetStepCount() == st.step_count
    check(opt, "synchronous")
    assert (opt.state_buffer("weight", 0) == dw[0]) == (applied % 2 == 0)     # the caller's own buffers or the shadows
    for k in range(5):                                           # asynchronous steps, one dropped
        g16 = grads(k == 2)
        assert opt.StepAMPAsync(dg, dw16) is None
        want = oracle().adam_amp(w, g16, m, v, w16, state=st, **hyper)
        applied += 0 if want else 1
        dev.synchronize()                                        # (the gradient buffers are reused)
    assert opt.current_set() == applied % 2 and opt.GetStepCount() == st.step_count
    check(opt, "asynchronous")
    # a plain fp32 step updates the current set in place
    g = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
    for h, a in zip(dg32, g):
        dev.upload(h, a)
    assert opt.Step(dg32) is None
    for k in range(len(sizes)):
        oracle().adam(w[k], g[k], m[k], v[k], step=int(st.step_count) + 1, **hyper)
    st.step_count += 1
    for k, n in enumerate(sizes):
        assert np.array_equal(dev.to_numpy(opt.state_buffer("weight", k), n).view(np.uint32), w[k].view(np.uint32))
    # checkpoint into a second ping-pong optimizer whose current set is its own set A
    text, err = opt.GetStateJSON()
    assert err is None
    resumed = make(env, "adam", cfg)
    dw2 = [dev.from_numpy(a) for a in w]
    assert resumed.SetWeightBuffers(dw2) is None
    assert resumed.EnableMixedPrecision(4096.0, 2.0, 0.5, 3) is None and resumed.EnablePingPong() is None
    assert resumed.LoadStateJSON(text) is None
    for h, a in zip(dw16, w):                                    # the fp16 copy of the restored weights
        dev.upload(h, a.astype(np.float16).view(np.uint16))
    w16 = [a.astype(np.float16).view(np.uint16) for a in w]
    for k in range(3):
        g16 = grads(k == 1)
        skipped, err = resumed.StepAMP(dg, dw16)
        assert err is None
        assert skipped == bool(oracle().adam_amp(w, g16, m, v, w16, state=st, **hyper))
    assert resumed.GetStepCount() == st.step_count
    check(resumed, "resumed")
    for o in (opt, resumed):
        o.Cleanup()
        o.free()
    assert pool_allocated(dev, mm, tier)[0] >= before_alloc[0] + 2      # shadow buffers of that tier are back in the pool
    for h in dw + dw2 + dw16 + dg + dg32:
        dev.free(h)

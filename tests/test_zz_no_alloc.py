"""The allocation-free Adam step (execute_adam_step_noalloc) against execute_adam_step_mpsgraph.

Both entry points run the same update kernel; what differs is the chunk table (a __device__ array
written by a kernel from kernel-argument records, against an uploaded, cached table).  The results
must be bit-identical, also on a second call with a smaller list, which finds the previous call's
descriptors still in the table.  Collected last on purpose (file name)."""
import ctypes

import numpy as np
import pytest

from harness import gpu_device
from workloads import ragged_sizes

pytestmark = pytest.mark.gpu

HYPER = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-4)


def _device():
    dev = gpu_device()
    if dev is None:
        pytest.fail("libgometal_hip.so or the GPU is missing: the allocation-free step has no fallback")
    return dev


class _List:
    """One parameter list on the device: weights, gradients, m, v, uploaded from host arrays."""

    def __init__(self, dev, pkg, w, g):
        self.dev, self.sizes = dev, [a.size for a in w]
        self.w = [dev.from_numpy(a) for a in w]
        self.g = [dev.from_numpy(a) for a in g]
        self.m = [dev.alloc(max(4 * n, 4), zero=True) for n in self.sizes]
        self.v = [dev.alloc(max(4 * n, 4), zero=True) for n in self.sizes]
        self.c = [pkg.handle_array(x) for x in (self.w, self.g, self.m, self.v)]
        self.bs = pkg.int_array([4 * n for n in self.sizes])

    def step(self, fn, t):
        rc = fn(self.dev.handle, *self.c, len(self.sizes), self.bs, HYPER["lr"], HYPER["beta1"], HYPER["beta2"],
                HYPER["eps"], HYPER["weight_decay"], t)
        assert rc == 0, (rc, self.dev.lib.gm_last_error())

    def snapshot(self):
        return [[self.dev.to_numpy(h, n) for h, n in zip(hs, self.sizes)] for hs in (self.w, self.m, self.v)]

    def close(self):
        for h in self.w + self.g + self.m + self.v:
            self.dev.free(h)


def _compare(dev, pkg, sizes, seed, steps):
    rng = np.random.default_rng(seed)
    w = [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes]
    g = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    ref, new = _List(dev, pkg, w, g), _List(dev, pkg, w, g)
    try:
        for t in range(1, steps + 1):
            print(f"no-alloc parity: {len(sizes)} tensors, {sum(sizes)} params, step {t}", flush=True)
            ref.step(dev.lib.execute_adam_step_mpsgraph, t)
            new.step(dev.lib.execute_adam_step_noalloc, t)
        want, got = ref.snapshot(), new.snapshot()
        for name, a, b in zip("wmv", want, got):
            for k, (x, y) in enumerate(zip(a, b)):
                assert np.array_equal(x.view(np.uint32), y.view(np.uint32)), (name, k, sizes[k])
        # the step did something
        assert any(not np.array_equal(x, y) for x, y in zip(w, got[0]) if x.size)
    finally:
        ref.close()
        new.close()


def test_no_alloc_matches_the_caching_entry_point_twice_in_a_row():
    from __graft_entry__ import load_package
    pkg = load_package()
    dev = _device()
    # 1. 203 tensors (four table-kernel launches), ragged sizes with edge cases: empty tensors, one
    #    element, around the 256-lane slice and around the chunk sizes the planner may pick
    big = ragged_sizes(count=160, total=6_000_000, lo=64, hi=1 << 20, seed=11)
    edges = [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 16383, 16384, 16385,
             65535, 65536, 65537, 0, 3, 5, 7, 300_001]
    extra = [17] * 17
    _compare(dev, pkg, big[:80] + edges + big[80:] + extra, seed=21, steps=3)
    # 2. right after it, a smaller list: the table still holds the first call's descriptors
    _compare(dev, pkg, [70_000, 5, 4096, 0, 33_333], seed=22, steps=2)


def test_no_alloc_leaves_the_plan_cache_counters_untouched():
    """The library's own counters of chunk tables laid out and table slots allocated do not move over five
    allocation-free steps: the step goes round the plan cache.  (That the call makes no hipMalloc at all is read
    off its source, which has none on its path; this test watches the cache only.)"""
    from __graft_entry__ import load_package
    pkg = load_package()
    dev = _device()
    lib = dev.lib
    rng = np.random.default_rng(5)
    sizes = [1000, 70_000, 64]
    lst = _List(dev, pkg, [rng.normal(0, 0.02, n).astype(np.float32) for n in sizes],
                [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes])
    try:
        builds, tables = ctypes.c_uint64(), ctypes.c_uint64()
        assert lib.gm_plan_cache_stats(dev.handle, ctypes.byref(builds), ctypes.byref(tables), None) == 0
        before = (builds.value, tables.value)
        for t in range(1, 6):
            lst.step(lib.execute_adam_step_noalloc, t)
        assert lib.gm_plan_cache_stats(dev.handle, ctypes.byref(builds), ctypes.byref(tables), None) == 0
        assert (builds.value, tables.value) == before
    finally:
        lst.close()


def test_no_alloc_rejects_lists_beyond_its_table_before_touching_anything():
    from __graft_entry__ import load_package
    pkg = load_package()
    dev = _device()
    lib = dev.lib
    # 48 tensors of 2^29 - 1 elements: 393k chunks of 65536, twelve times the table.  The handles are
    # placeholders; the call must fail in validation, before any launch.
    n = 48
    fake = pkg.handle_array([0x7000_0000_0000 + 0x1_0000_0000 * k for k in range(n)])
    bs = pkg.int_array([(2 ** 31 - 4)] * n)
    rc = lib.execute_adam_step_noalloc(dev.handle, fake, fake, fake, fake, n, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    assert rc == -17
    assert b"32768" in lib.gm_last_error()
    # more tensors than the entry point takes
    n = 4097
    fake = pkg.handle_array([0x7000_0000_0000 + 4096 * k for k in range(n)])
    bs = pkg.int_array([64] * n)
    rc = lib.execute_adam_step_noalloc(dev.handle, fake, fake, fake, fake, n, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1)
    assert rc == -17 and b"4096" in lib.gm_last_error()
    # the usual codes are kept
    assert lib.execute_adam_step_noalloc(0, fake, fake, fake, fake, 1, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1) == -1
    nil = pkg.handle_array([0])
    one = pkg.handle_array([0x7000_0000_0000])
    assert lib.execute_adam_step_noalloc(dev.handle, one, one, nil, one, 1, bs, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1) == -4

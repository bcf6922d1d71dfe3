"""Buffer primitives of the C ABI on the GPU.  The first three tests restate the reference's
exact-equality device tests (cgo_bridge/bridge_test.go:188-276, advanced_test.go:53-98)."""
import ctypes

import numpy as np
import pytest

from harness import gpu_device
from oracle_lib import oracle

pytestmark = pytest.mark.gpu
vp = ctypes.c_void_p


@pytest.fixture(scope="module")
def dev():
    d = gpu_device()
    if d is None:
        pytest.fail("libgometal_hip.so is missing or no GPU is usable: GPU tests cannot run")
    return d


def test_float32_round_trip(dev):                      # bridge_test.go:188-229
    data = (np.arange(64, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    buf = dev.alloc(256)
    assert dev.lib.copy_float32_array_to_metal_buffer(buf, data.ctypes.data_as(vp), 64) == 0
    out = np.empty(64, np.float32)
    assert dev.lib.copy_metal_buffer_to_float32_array(buf, out.ctypes.data_as(vp), 64) == 0
    assert np.array_equal(out.view(np.uint32), data.view(np.uint32))
    dev.free(buf)


def test_zero_buffer(dev):                             # bridge_test.go:232-276
    data = np.arange(1, 33, dtype=np.float32)
    buf = dev.alloc(128)
    dev.upload(buf, data)
    assert dev.lib.zero_metal_buffer(dev.handle, buf, 128) == 0
    assert np.all(dev.to_numpy(buf, 32).view(np.uint32) == 0)
    dev.free(buf)


def test_buffer_to_buffer_sync_copy(dev):              # advanced_test.go:53-98
    data = (np.arange(64, dtype=np.float32) * np.float32(0.5)).astype(np.float32)
    src, dst = dev.alloc(256), dev.alloc(256)
    dev.upload(src, data)
    assert dev.lib.copy_buffer_to_buffer_sync(src, dst, 0, 0, 256) == 0
    assert np.array_equal(dev.to_numpy(dst, 64), data)
    # offsets, and the range checks of bridge_memory.m:523-537
    assert dev.lib.copy_buffer_to_buffer_sync(src, dst, 16, 32, 64) == 0
    got = dev.to_numpy(dst, 64)
    assert np.array_equal(got[8:24], data[4:20]) and np.array_equal(got[:8], data[:8])
    assert dev.lib.copy_buffer_to_buffer_sync(src, dst, 200, 0, 64) == -4
    assert dev.lib.copy_buffer_to_buffer_sync(src, dst, 0, 200, 64) == -5
    dev.free(src)
    dev.free(dst)


@pytest.mark.parametrize("n", [1, 3, 5, 7, 255, 4097])
def test_odd_sizes_and_canaries(dev, n):
    """Zeroing and copying n floats must not touch the floats around them."""
    total = n + 64
    canary = np.full(total, np.float32(-123.5))
    buf = dev.alloc(4 * total)
    dev.upload(buf, canary)
    assert dev.lib.zero_metal_buffer(dev.handle, buf, 4 * n) == 0
    got = dev.to_numpy(buf, total)
    assert np.all(got[:n] == 0) and np.all(got[n:] == np.float32(-123.5))
    dev.free(buf)


def test_allocation_length_is_rounded_to_16(dev):      # bridge_memory.m:28
    for size, want in [(1, 16), (16, 16), (17, 32), (1000, 1008)]:
        h = dev.lib.allocate_metal_buffer(dev.handle, size, 1)
        assert h != 0 and h % 256 == 0
        assert dev.lib.gm_buffer_length(h) == want
        dev.lib.deallocate_metal_buffer(h)
        assert dev.lib.gm_buffer_length(h) == 0


def test_large_buffer_round_trip(dev):
    """A 2^28-byte buffer: copy helpers hold up beyond small test sizes."""
    n = (1 << 28) // 4
    rng = np.random.default_rng(3)
    data = rng.standard_normal(n, dtype=np.float32)
    buf = dev.alloc(4 * n)
    dev.upload(buf, data)
    assert np.array_equal(dev.to_numpy(buf, n), data)
    dev.free(buf)


@pytest.mark.parametrize("nbytes", [(8 << 20) - 4, 8 << 20, (8 << 20) + 4, (24 << 20) + 12, (37 << 20) + 4092])
def test_host_copies_around_the_staging_threshold(dev, nbytes):
    """Copies of 8 MiB and more travel through pinned staging slots on two lanes (4 MiB slots, the range
    split at a page boundary): sizes either side of the threshold, and ranges that end inside a slot, must
    arrive exactly, inside a larger buffer whose other bytes stay untouched."""
    n = nbytes // 4
    pad = 1024
    rng = np.random.default_rng(nbytes)
    data = rng.integers(0, 1 << 32, n, dtype=np.uint32)
    whole = np.full(n + 2 * pad, 0xDEADBEEF, np.uint32)
    buf = dev.from_numpy(whole)
    view = buf + 4 * pad
    assert dev.lib.copy_data_to_metal_buffer(view, data.ctypes.data_as(vp), nbytes) == 0
    got = dev.to_numpy(buf, n + 2 * pad, np.uint32)
    assert np.all(got[:pad] == 0xDEADBEEF) and np.all(got[-pad:] == 0xDEADBEEF)
    assert np.array_equal(got[pad:-pad], data)
    back = np.zeros(n + 8, np.uint32)
    assert dev.lib.copy_metal_buffer_to_int32_array(view, back.ctypes.data_as(vp), n) == 0
    assert np.array_equal(back[:n], data) and np.all(back[n:] == 0)
    dev.free(buf)


def test_two_threads_copy_large_buffers_at_once(dev):
    """The staging lanes are shared: concurrent large copies from two threads take turns and both arrive."""
    import threading
    n = (16 << 20) // 4
    data = [np.random.default_rng(k).integers(0, 1 << 32, n, dtype=np.uint32) for k in range(2)]
    bufs = [dev.alloc(4 * n) for _ in range(2)]
    out = [np.zeros(n, np.uint32) for _ in range(2)]
    errors = []

    def work(k):
        for _ in range(3):
            if dev.lib.copy_data_to_metal_buffer(bufs[k], data[k].ctypes.data_as(vp), 4 * n) != 0:
                errors.append(("in", k))
            if dev.lib.copy_metal_buffer_to_int32_array(bufs[k], out[k].ctypes.data_as(vp), n) != 0:
                errors.append(("out", k))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    for k in range(2):
        assert np.array_equal(out[k], data[k])
        dev.free(bufs[k])


def all_half_patterns():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_convert_f16_to_f32_exhaustive(dev):
    """Every binary16 pattern: the device widening equals the oracle's (NaNs compared as NaN)."""
    h = all_half_patterns()
    src = dev.from_numpy(h)
    dst = dev.alloc(4 * h.size)
    shape = (ctypes.c_int * 1)(h.size)
    assert dev.lib.convert_tensor_type(src, dst, shape, 1, 2, 0, dev.handle) == 0
    got = dev.to_numpy(dst, h.size)
    want = oracle().f16_to_f32(h)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    dev.free(src)
    dev.free(dst)


def test_convert_f32_to_f16_boundaries_and_random(dev):
    """Round-to-nearest-even narrowing: every half value, the midpoints between neighbouring halves
    (ties), values one ulp either side of them, the overflow edge, subnormals, and random floats."""
    o = oracle()
    halves = o.f16_to_f32(all_half_patterns())
    finite = np.sort(halves[np.isfinite(halves)].astype(np.float64))
    mids = ((finite[:-1] + finite[1:]) / 2).astype(np.float32)
    cases = [halves[np.isfinite(halves)], mids, np.nextafter(mids, np.float32(np.inf)),
             np.nextafter(mids, np.float32(-np.inf)),
             np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e10, -65520.0, np.inf, -np.inf,
                       5.9604645e-8, 2.9802322e-8, 2.9802325e-8, 1e-10, 0.0, -0.0, 1.0e-40], np.float32),
             np.random.default_rng(11).standard_normal(200000).astype(np.float32) *
             np.float32(10.0) ** np.random.default_rng(12).integers(-9, 6, 200000).astype(np.float32)]
    x = np.concatenate(cases).astype(np.float32)
    src = dev.from_numpy(x)
    dst = dev.alloc(2 * x.size + 16)
    shape = (ctypes.c_int * 2)(1, x.size)
    assert dev.lib.convert_tensor_type(src, dst, shape, 2, 0, 2, dev.handle) == 0
    got = dev.to_numpy(dst, x.size, np.uint16)
    want = o.f32_to_f16(x)
    assert np.array_equal(got, want)
    # the unsupported pairs of the reference (bridge_memory.m:413-416)
    assert dev.lib.convert_tensor_type(src, dst, shape, 2, 0, 0, dev.handle) == -3
    dev.free(src)
    dev.free(dst)


def test_fill_normal_is_reproducible_and_sane(dev):
    n = 1 << 20
    a, b = dev.alloc(4 * n), dev.alloc(4 * n)
    assert dev.lib.gm_fill_normal_f32(dev.handle, a, n, 42, 0.5, 2.0) == 0
    assert dev.lib.gm_fill_normal_f32(dev.handle, b, n, 42, 0.5, 2.0) == 0
    xa, xb = dev.to_numpy(a, n), dev.to_numpy(b, n)
    assert np.array_equal(xa, xb)
    assert abs(xa.mean() - 0.5) < 0.02 and abs(xa.std() - 2.0) < 0.02 and np.all(np.isfinite(xa))
    dev.free(a)
    dev.free(b)


def test_offset_views_take_the_unaligned_paths(dev):
    """A handle is a device address, so a caller may pass base + offset: zeroing and the casts
    must not assume 16-byte alignment, and must leave the bytes around the view alone."""
    o = oracle()
    n = 1000
    x = (np.random.default_rng(5).standard_normal(n + 8) * 3).astype(np.float32)
    src = dev.from_numpy(x)
    dst16 = dev.from_numpy(np.full(n + 16, 0x1234, np.uint16))
    shape = (ctypes.c_int * 1)(n - 3)
    # fp32 view starting 4 bytes in, fp16 view starting 2 bytes in
    assert dev.lib.convert_tensor_type(src + 4, dst16 + 2, shape, 1, 0, 2, dev.handle) == 0
    got = dev.to_numpy(dst16, n + 16, np.uint16)
    assert np.array_equal(got[1:n - 2], o.f32_to_f16(x[1:n - 2]))
    assert got[0] == 0x1234 and np.all(got[n - 2:] == 0x1234)
    # and back, into an fp32 view that is 4 bytes off
    back = dev.from_numpy(np.full(n + 8, -7.0, np.float32))
    assert dev.lib.convert_tensor_type(dst16 + 2, back + 4, shape, 1, 2, 0, dev.handle) == 0
    got32 = dev.to_numpy(back, n + 8)
    assert np.array_equal(got32[1:n - 2].view(np.uint32), o.f16_to_f32(got[1:n - 2]).view(np.uint32))
    assert got32[0] == -7.0 and np.all(got32[n - 2:] == -7.0)
    # zero 37 bytes starting 5 bytes in
    raw = dev.from_numpy(np.full(64, 0xAB, np.uint8))
    assert dev.lib.zero_metal_buffer(dev.handle, raw + 5, 37) == 0
    b = dev.to_numpy(raw, 64, np.uint8)
    assert np.all(b[:5] == 0xAB) and np.all(b[5:42] == 0) and np.all(b[42:] == 0xAB)
    for h in (src, dst16, back, raw):
        dev.free(h)


@pytest.mark.parametrize("src_off,dst_off,size", [
    (0, 0, 4096), (0, 0, 4099), (16, 48, 1000), (16, 48, 7),          # 16-byte aligned: the library's copy kernel
    (4, 8, 4096), (1, 3, 333), (16, 5, 64),                            # unaligned: the runtime's copy
    (0, 0, 16 * 64 * 3 + 5), (32, 16, 16 * 64),                        # several workgroups, exact multiple
])
def test_buffer_to_buffer_copy_offsets_sizes_and_canaries(dev, src_off, dst_off, size):
    """Every (offset, size) class of copy_buffer_to_buffer_sync moves exactly the bytes asked for."""
    total = 8192
    rng = np.random.default_rng(size)
    a = rng.integers(0, 256, total, dtype=np.uint8)
    b = rng.integers(0, 256, total, dtype=np.uint8)
    src, dst = dev.from_numpy(a), dev.from_numpy(b)
    assert dev.lib.copy_buffer_to_buffer_sync(src, dst, src_off, dst_off, size) == 0
    want = b.copy()
    want[dst_off:dst_off + size] = a[src_off:src_off + size]
    assert np.array_equal(dev.to_numpy(dst, total, np.uint8), want)
    assert np.array_equal(dev.to_numpy(src, total, np.uint8), a)
    dev.free(src)
    dev.free(dst)


def test_buffer_to_buffer_copy_inside_one_buffer(dev):
    """Disjoint ranges of one buffer copy exactly; overlapping ranges go to the runtime's copy and at
    least return without error (their result is unspecified in the reference as well)."""
    a = np.random.default_rng(11).integers(0, 256, 4096, dtype=np.uint8)
    buf = dev.from_numpy(a)
    assert dev.lib.copy_buffer_to_buffer_sync(buf, buf, 0, 2048, 1024) == 0
    want = a.copy()
    want[2048:3072] = a[:1024]
    assert np.array_equal(dev.to_numpy(buf, 4096, np.uint8), want)
    assert dev.lib.copy_buffer_to_buffer_sync(buf, buf, 0, 16, 1024) == 0
    dev.free(buf)


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 63, 64, 255, 256, 257, 1027, 65537])
def test_convert_lengths_around_the_group_and_workgroup_sizes(dev, n):
    """Conversions work in 4-element groups, 64 lanes to a workgroup, with the last n % 4 elements apart:
    every length class, with canaries behind the destination."""
    o = oracle()
    x = (np.random.default_rng(n).standard_normal(n) * 100).astype(np.float32)
    src = dev.from_numpy(x)
    half = dev.from_numpy(np.full(n + 8, 0x5555, np.uint16))
    shape = (ctypes.c_int * 1)(n)
    assert dev.lib.convert_tensor_type(src, half, shape, 1, 0, 2, dev.handle) == 0
    got = dev.to_numpy(half, n + 8, np.uint16)
    want = o.f32_to_f16(x)
    assert np.array_equal(got[:n], want) and np.all(got[n:] == 0x5555)
    back = dev.from_numpy(np.full(n + 4, -3.0, np.float32))
    assert dev.lib.convert_tensor_type(half, back, shape, 1, 2, 0, dev.handle) == 0
    got32 = dev.to_numpy(back, n + 4)
    assert np.array_equal(got32[:n].view(np.uint32), o.f16_to_f32(want).view(np.uint32))
    assert np.all(got32[n:] == -3.0)
    for h in (src, half, back):
        dev.free(h)


def test_ranges_beyond_an_allocation_are_refused(dev):
    """The reference trusts its callers here; an overrun on a GPU is a fault, so buffers of this
    library are checked against their recorded length."""
    buf = dev.alloc(64)
    small = dev.alloc(16)
    host = np.zeros(64, np.float32)
    assert dev.lib.copy_float32_array_to_metal_buffer(buf, host.ctypes.data_as(vp), 17) == -3
    assert dev.lib.copy_data_to_metal_buffer(buf, host.ctypes.data_as(vp), 65) == -3
    assert dev.lib.copy_metal_buffer_to_float32_array(buf, host.ctypes.data_as(vp), 17) == -3
    assert b"exceeds" in dev.lib.gm_last_error()
    assert dev.lib.copy_float32_array_to_metal_buffer(buf, host.ctypes.data_as(vp), 16) == 0
    shape = (ctypes.c_int * 1)(16)
    assert dev.lib.convert_tensor_type(buf, small, shape, 1, 0, 2, dev.handle) == -5     # 32 bytes into 16
    assert dev.lib.convert_tensor_type(small, buf, shape, 1, 2, 0, dev.handle) == -5     # 32 bytes out of 16
    shape8 = (ctypes.c_int * 1)(8)
    assert dev.lib.convert_tensor_type(buf, small, shape8, 1, 0, 2, dev.handle) == 0
    assert dev.lib.zero_metal_buffer(dev.handle, buf, 65) == -5
    dev.free(buf)
    dev.free(small)

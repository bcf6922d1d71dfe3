"""Tensor lists of the five benchmark configurations (product configuration: bench.py measures them, the parity tests step them)."""
import numpy as np

# config 2: conv [oc, ic, k, k] + bias, BatchNorm gamma / beta, dense [in, out] + bias
CNN_SHAPES = [
    (32, 3, 3, 3), (32,), (64, 32, 3, 3), (64,), (128, 64, 3, 3), (128,),
    (32,), (32,), (64,), (64,), (128,), (128,),
    (8192, 128), (128,), (128, 10), (10,),
]


def cnn_sizes():
    sizes = [int(np.prod(s)) for s in CNN_SHAPES]
    assert sum(sizes) == 1_143_690
    return sizes


def ragged_sizes(count=160, total=25_000_000, lo=64, hi=4 * 1024 * 1024, seed=0x6D657461 + 3):
    """config 3: `count` sizes, log-uniform in [lo, hi], rescaled so they sum to `total`."""
    rng = np.random.default_rng(seed)
    raw = np.exp(rng.uniform(np.log(lo), np.log(hi), count))
    sizes = np.maximum(lo, np.floor(raw * (total / raw.sum()))).astype(np.int64)
    sizes = np.minimum(sizes, hi)
    diff = total - int(sizes.sum())
    for idx in np.argsort(-sizes):      # put the rounding remainder where there is room
        room = hi - sizes[idx] if diff > 0 else sizes[idx] - lo
        take = int(np.sign(diff) * min(abs(diff), room))
        sizes[idx] += take
        diff -= take
        if diff == 0:
            break
    assert int(sizes.sum()) == total and sizes.min() >= lo and sizes.max() <= hi
    return [int(s) for s in sizes]


def amp_125m_sizes():
    """config 4: 60 tensors, 125,000,000 params."""
    sizes = [2_097_152] * 50 + [2_014_240] * 10
    assert sum(sizes) == 125_000_000
    return sizes


def transformer_block_sizes():
    """config 5: 400 tensors, 1,012,301,824 params:
    12 x (2 x [4096,4096], 1 x [4096,11008], 30 x [4096]) then 4 x [4096,4096]."""
    sizes = []
    for _ in range(12):
        sizes += [4096 * 4096] * 2 + [4096 * 11008] + [4096] * 30
    sizes += [4096 * 4096] * 4
    assert len(sizes) == 400 and sum(sizes) == 1_012_301_824
    return sizes


def two_segment_sizes():
    """A list the planner cuts into two segments: one 120M-element tensor keeps 65536-element chunks within
    the 5 % idle limit, and 80 small tensors in the middle of the list would idle about 20k workgroups of that
    size, more than the 16384 that earn them a segment with a smaller chunk."""
    small = [1, 255, 256, 257, 1023, 1025, 4095, 4097, 5, 300, 77, 2049] * 7
    small = small[:80]
    return small[:40] + [120_000_001] + small[40:]

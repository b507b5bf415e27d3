"""Seeded synthetic tensors for the test and benchmark harnesses.

A counter-based SplitMix64 stream in pure integer arithmetic: the same seed gives
the same bytes on every machine and numpy version."""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, count, offset=0):
    idx = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def fill_u8(shape, seed, lo=0, hi=255):
    count = int(np.prod(shape))
    r = splitmix64(seed, count) >> np.uint64(11)
    return (np.uint64(lo) + r % np.uint64(hi - lo + 1)).astype(np.uint8).reshape(shape)


def fill_i32(shape, seed, lo, hi):
    count = int(np.prod(shape))
    r = (splitmix64(seed, count) >> np.uint64(11)) % np.uint64(hi - lo + 1)
    return (r.astype(np.int64) + lo).astype(np.int32).reshape(shape)


def fill_normal_field(shape, seed):
    """int64 values close to N(0, 65535): a 12-term Irwin-Hall sum of 16-bit uniforms, centred (what float weights
    drawn from a normal distribution look like before a quantizer sees them, in integer arithmetic)"""
    count = int(np.prod(shape))
    r = splitmix64(seed, count * 3).reshape(count, 3)
    total = np.zeros(count, np.int64)
    for sh in (0, 16, 32, 48):
        total += ((r >> np.uint64(sh)) & np.uint64(0xFFFF)).astype(np.int64).sum(axis=1)
    return (total - 6 * 65535).reshape(shape)


def fill_u8_normal(shape, seed, mean, sd):
    """clip(round(N(mean, sd)), 0, 255): a 12-term Irwin-Hall sum of 16-bit uniforms in integer arithmetic."""
    count = int(np.prod(shape))
    r = splitmix64(seed, count * 3).reshape(count, 3)
    total = np.zeros(count, np.int64)
    for sh in (0, 16, 32, 48):
        total += ((r >> np.uint64(sh)) & np.uint64(0xFFFF)).astype(np.int64).sum(axis=1)
    num = np.int64(sd) * (total - 6 * 65535)
    dev = np.where(num >= 0, (num + 32768) // 65536, -((-num + 32768) // 65536))
    return np.clip(mean + dev, 0, 255).astype(np.uint8).reshape(shape)

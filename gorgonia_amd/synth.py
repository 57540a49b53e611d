"""Seeded synthetic inputs for the benchmark configurations and the parity
tests.  The reference's own initialisers are seeded from the wall clock
(weights.go:270-511) and cannot be reproduced, so every tensor here comes from
a counter-based SplitMix64 stream: element i of a tensor with seed s is a pure
function of (s, i).  Values are handed to the engine as data (the reference's
WithValue path, node.go:135)."""
from __future__ import annotations

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(seed, n, offset=0):
    with np.errstate(over="ignore"):
        i = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed) * np.uint64(0xD1342543DE82EF95) + i * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform01(seed, shape):
    """float32 in [0, 1) with 24 random mantissa bits."""
    n = int(np.prod(shape))
    u = (_splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    return u.reshape(shape)


def uniform(seed, shape, lo, hi):
    return (uniform01(seed, shape) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)


def normal(seed, shape, mean=0.0, std=1.0):
    """Box-Muller on two SplitMix64 streams, evaluated in float64, rounded once."""
    n = int(np.prod(shape))
    u1 = ((_splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0 ** -53
    u2 = (_splitmix64(seed ^ 0x5DEECE66D, n) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * std + mean).astype(np.float32).reshape(shape)


def glorot_uniform(seed, shape, gain=1.0):
    """U(+-gain*sqrt(6/(fan_in+fan_out))) (formula of weights.go:397-427)."""
    fan_in, fan_out = _fans(shape)
    lim = gain * np.sqrt(6.0 / (fan_in + fan_out))
    return uniform(seed, shape, -lim, lim)


def he_normal(seed, shape, gain=np.sqrt(2.0)):
    """N(0, gain/sqrt(fan_in)) (formula of weights.go:455-479)."""
    fan_in, _ = _fans(shape)
    return normal(seed, shape, 0.0, gain / np.sqrt(fan_in))


def _fans(shape):
    if len(shape) == 2:
        return shape[0], shape[1]
    if len(shape) == 4:  # (F, C, kh, kw)
        rf = shape[2] * shape[3]
        return shape[1] * rf, shape[0] * rf
    n = int(np.prod(shape))
    return n, n

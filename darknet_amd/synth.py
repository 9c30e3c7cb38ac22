"""Seeded synthetic tensors for the darknet forward path.

The reference seeds nothing (its ``main`` never calls ``srand``, examples/darknet.c:400-420)
and initialises convolution weights with ``rand_normal`` (src/convolutional_layer.c:205-209),
so every harness in this repository writes weights, batch-norm statistics and inputs itself.
The generator is counter based (a splitmix64 finaliser over ``seed + index``), so element *i* of
a stream depends only on ``(seed, i)``: the same bytes come out on every machine, for any
chunking, without carrying generator state between the CPU checker and the GPU library.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def uniform01(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """``n`` float32 values uniform on [0, 1) with 24 random bits each."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = _mix(np.uint64(seed) * np.uint64(0xD1342543DE82EF95) + idx * _GOLDEN)
    return ((z >> np.uint64(40)).astype(np.float32)) * np.float32(1.0 / (1 << 24))


def uniform(seed: int, n: int, lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    """``n`` float32 values uniform on [lo, hi)."""
    u = uniform01(seed, n)
    return (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float32)


def conv_weights(seed: int, n: int, c_per_group: int, size: int, he_scale: bool = True) -> np.ndarray:
    """Weights ``[n][c/groups][size][size]`` = uniform(-1,1) * sqrt(2/(size*size*c/groups)).

    This is the initialisation the benchmark configurations ask for; it is the commented-out
    ``rand_uniform`` variant of src/convolutional_layer.c:204-208, not the ``rand_normal`` one the
    reference actually runs.
    """
    count = n * c_per_group * size * size
    w = uniform(seed, count)
    if he_scale:
        w = w * np.float32(np.sqrt(2.0 / (size * size * c_per_group)))
    return w.astype(np.float32)


def bn_identity(n: int):
    """(biases, scales, rolling_mean, rolling_variance) = (0, 1, 0, 1) as float32 vectors."""
    return (np.zeros(n, np.float32), np.ones(n, np.float32),
            np.zeros(n, np.float32), np.ones(n, np.float32))


def bn_random(seed: int, n: int):
    """Non-trivial batch-norm vectors, so that a dropped term in the fused tail shows up."""
    biases = uniform(seed + 11, n, -0.5, 0.5)
    scales = uniform(seed + 12, n, 0.5, 1.5)
    mean = uniform(seed + 13, n, -0.3, 0.3)
    var = uniform(seed + 14, n, 0.25, 2.0)
    return biases, scales, mean, var

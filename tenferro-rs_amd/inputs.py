"""Seeded, order-independent synthetic inputs for the five benchmark configurations.

Element i (row-major logical index) of tensor `tensor_id` under `seed` is a pure function of
(seed, tensor_id, i): h = splitmix64(seed ^ (tensor_id << 48) + i).  Generated once on the host in
float64 and rounded once to the target dtype, so the CPU baseline and the GPU run see identical bits.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(x):
    """Vectorised SplitMix64 finaliser over uint64 (wrap-around arithmetic)."""
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = x
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def _hash(seed, tensor_id, n, stream=0):
    with np.errstate(over="ignore"):
        base = np.uint64(seed) ^ (np.uint64(tensor_id) << np.uint64(48)) ^ (np.uint64(stream) << np.uint64(40))
        return splitmix64(base + np.arange(n, dtype=np.uint64))


def _unit(h):
    """uint64 hash -> float64 in [0, 1) from the top 53 bits."""
    return (h >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform(seed, tensor_id, shape, dtype=np.float64):
    """iid uniform[-1, 1)."""
    n = int(np.prod(shape))
    return (_unit(_hash(seed, tensor_id, n)) * 2.0 - 1.0).astype(dtype).reshape(shape)


def normal(seed, tensor_id, shape, dtype=np.float64, sigma=1.0, stream=0):
    """iid N(0, sigma^2) by Box-Muller on two counter streams, computed in float64."""
    n = int(np.prod(shape))
    u1 = 1.0 - _unit(_hash(seed, tensor_id, n, stream=2 * stream + 1))      # (0, 1]
    u2 = _unit(_hash(seed, tensor_id, n, stream=2 * stream + 2))
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * z).astype(dtype).reshape(shape)


def complex_normal(seed, tensor_id, shape, sigma=1.0, dtype=np.complex128):
    """real and imaginary parts iid N(0, sigma^2)."""
    re = normal(seed, tensor_id, shape, np.float64, sigma, stream=0)
    im = normal(seed, tensor_id, shape, np.float64, sigma, stream=1)
    return (re + 1j * im).astype(dtype)


def draw_block_dims(seed, n_blocks, choices=tuple(range(64, 1025, 64))):
    """(i, j, k) per block, each drawn independently and uniformly from `choices`."""
    h = _hash(seed, 0xB10C, 3 * n_blocks)
    idx = (h % np.uint64(len(choices))).astype(np.int64).reshape(n_blocks, 3)
    return [tuple(int(choices[c]) for c in row) for row in idx]

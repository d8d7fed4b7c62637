"""Input builders shared by the oracle tests and the GPU parity tests."""
import numpy as np


def rule(shape, step):
    """Tensor [1,1,H,W] filled with x + y*step + 1 (the reference self-test's pattern)."""
    h, w = shape
    y, x = np.mgrid[0:h, 0:w]
    return (x + y * step + 1).astype(np.float32).reshape(1, 1, h, w)


def batch(a, n=10):
    """The reference self-test repeats one sample over a batch of 10."""
    return np.ascontiguousarray(np.broadcast_to(a, (n,) + a.shape[1:]))


def rng_uniform(seed, *shape, lo=-1.0, hi=1.0):
    return np.random.default_rng(seed).uniform(lo, hi, size=shape).astype(np.float32)


def rng_normal(seed, *shape, std=1.0):
    return (np.random.default_rng(seed).standard_normal(size=shape) * std).astype(np.float32)

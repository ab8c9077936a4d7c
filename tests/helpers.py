"""Shared input builders for the CPU and GPU tests (numpy only)."""
import numpy as np

QB = 32


def rand_codes(rng, shape, sparse=0.0):
    q = rng.integers(-127, 128, size=shape, dtype=np.int64).astype(np.int8)
    if sparse:
        q[rng.random(shape) < sparse] = 0
    return q


def rand_scales(rng, shape, lo=-12, hi=-2, f16=True):
    """Positive scales spread over several binades; f16-representable if asked."""
    s = rng.uniform(1.0, 2.0, size=shape) * np.exp2(rng.integers(lo, hi, size=shape))
    s = s.astype(np.float32)
    if f16:
        s = s.astype(np.float16).astype(np.float32)
    return s


def block_view(x, b=QB):
    R, C = x.shape
    return x.reshape(R // b, b, C // b, b).transpose(0, 2, 1, 3)


def block_amax(x, b=QB):
    return np.abs(block_view(x, b)).max(axis=(2, 3))


def expand_scales(s, b=QB):
    return np.repeat(np.repeat(s, b, axis=0), b, axis=1)

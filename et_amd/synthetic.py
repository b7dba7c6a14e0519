"""Seeded synthetic operands: one generator and one rounding to half, shared by
the benchmark, the smoke check and the tests, so that all of them (and the CPU
oracle they are compared with) see the same bits."""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def randn_h(r, shape, std=1.0):
    """N(0, std) drawn in float64, rounded to half once"""
    return (r.standard_normal(shape) * std).astype(np.float16)

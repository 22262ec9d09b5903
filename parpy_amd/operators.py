"""CPU meaning of the operators usable inside a @jit function.

Running the un-jitted Python function with these gives the sequential
semantics (python/parpy/operators.py:1-75 of the reference): NumPy math,
two-argument max/min = np.maximum/np.minimum, casts = int()/float(),
`gpu` a null context and `label` a no-op.
"""
from builtins import abs
from numpy import cos, exp, inf, log, sin, sqrt, tanh
from numpy import arctan2 as atan2
import numpy as np
import contextlib

gpu = contextlib.nullcontext()


def min(x, y=None, axis=None):
    if y is None:
        return np.min(x) if axis is None else np.min(x, axis=axis)
    assert axis is None
    return np.minimum(x, y)


def max(x, y=None, axis=None):
    if y is None:
        return np.max(x) if axis is None else np.max(x, axis=axis)
    assert axis is None
    return np.maximum(x, y)


def sum(x, axis=None):
    return np.sum(x) if axis is None else np.sum(x, axis=axis)


def prod(x, axis=None):
    return np.prod(x) if axis is None else np.prod(x, axis=axis)


def float16(x):
    return float(x)


def float32(x):
    return float(x)


def float64(x):
    return float(x)


def int8(x):
    return int(x)


def int16(x):
    return int(x)


def int32(x):
    return int(x)


def int64(x):
    return int(x)


def uint8(x):
    return int(x)


def uint16(x):
    return int(x)


def uint32(x):
    return int(x)


def uint64(x):
    return int(x)


def label(x):
    assert x is not None, "parpy.label expects one argument"

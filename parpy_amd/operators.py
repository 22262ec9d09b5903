"""What the operators usable inside a @jit function mean on the CPU.

Calling the undecorated Python function with these gives the sequential semantics of the program
(python/parpy/operators.py:1-75 of the reference): math functions are NumPy's, a reduction takes one array
(optionally an axis), `max`/`min` of two values are element-wise, a cast yields a Python number, `gpu` is a
context that does nothing and `label` only checks that it was given a name.
"""
import contextlib
from builtins import abs   # noqa: F401  (re-exported: `parpy.operators.abs` is the builtin)

import numpy as np
from numpy import cos, exp, inf, log, sin, sqrt, tanh   # noqa: F401
from numpy import arctan2 as atan2                      # noqa: F401

gpu = contextlib.nullcontext()


def _reduction(whole, pairwise=None):
    """Reduction over an array, or -- for max and min -- the element-wise form when given two operands."""
    def op(x, y=None, axis=None):
        if y is not None:
            assert axis is None
            return pairwise(x, y)
        return whole(x) if axis is None else whole(x, axis=axis)

    def op1(x, axis=None):
        return whole(x) if axis is None else whole(x, axis=axis)
    chosen = op if pairwise is not None else op1
    chosen.__name__ = chosen.__qualname__ = whole.__name__
    return chosen


min = _reduction(np.min, np.minimum)
max = _reduction(np.max, np.maximum)
sum = _reduction(np.sum)
prod = _reduction(np.prod)

# casts: the width only matters on the device; on the CPU the value becomes a Python float or int.  Every
# cast is a function object of its own, because the front end recognises operators by identity.
def _cast(name, to):
    def cast(x):
        return to(x)
    cast.__name__ = cast.__qualname__ = name
    return cast


for _name in ("float16", "float32", "float64"):
    globals()[_name] = _cast(_name, float)
for _name in ("int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64"):
    globals()[_name] = _cast(_name, int)
del _name


def label(x):
    assert x is not None, "parpy.label expects one argument"

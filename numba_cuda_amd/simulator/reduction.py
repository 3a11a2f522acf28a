"""cuda.reduce in the CPU mode: a strict left fold through the Python callable, one
call per element, `init` used as given (numba_cuda/numba/cuda/simulator/reduction.py:7-19)."""

from functools import reduce as _fold


def Reduce(func, reference_order=None):
    """`reference_order` (this package's own argument of the GPU mode's Reduce) is accepted and
    has nothing to choose here: the fold has one order."""
    def reduce_wrapper(seq, res=None, init=0):
        value = _fold(func, seq, init)
        if res is None:
            return value
        res[0] = value
        return None

    return reduce_wrapper


reduce = Reduce

"""Literal lock-step SIMT emulation of the reference's reduction kernels.

Test infrastructure.  Where oracle.c states the *derived* association order of
numba_cuda/numba/cuda/kernels/reduction.py in closed form, this module walks the
kernel text itself: a shared-memory array per block, threadIdx/blockIdx vectors,
one numpy statement per line of device code, every statement applied to all
threads at once (which is what the barriers in the kernel guarantee).  The two
are compared bit for bit on float32 data, where any difference in association
shows up in the rounding.
"""

import numpy as np

WARPSIZE = 32
NUMWARPS = 4
BLOCKSIZE = WARPSIZE * NUMWARPS


def _ops(dtype):
    def add(a, b):
        with np.errstate(over="ignore"):
            return (a + b).astype(dtype, copy=False)

    def mul(a, b):
        with np.errstate(over="ignore"):
            return (a * b).astype(dtype, copy=False)

    def vmax(a, b):
        return np.where(b > a, b, a)

    def vmin(a, b):
        return np.where(b < a, b, a)

    return {"add": add, "mul": mul, "max": vmax, "min": vmin}


def _inner_warp_reduction(op, sm, tid, value):
    """reduction.py:22-41.  sm: [grid, 4, 33]; tid: active thread ids of the
    block; value: [grid, len(tid)]."""
    warpid, laneid = tid // WARPSIZE, tid % WARPSIZE
    sm[:, warpid, laneid] = value
    width = WARPSIZE // 2
    while width:
        act = laneid < width
        w, l = warpid[act], laneid[act]
        old = sm[:, w, l]
        sm[:, w, l] = op(old, sm[:, w, l + width])
        width //= 2


def _full_block(op, arr, partials, sm, grid):
    """reduction.py:43-97, blockDim.x == 128."""
    tid = np.arange(BLOCKSIZE)
    blkid = np.arange(grid)[:, None]
    start = tid[None, :] + BLOCKSIZE * blkid          # [grid, 128]
    stop = arr.size
    step = BLOCKSIZE * grid
    tmp = arr[start]
    i = start + step
    while (i < stop).any():
        m = i < stop
        nxt = op(tmp, arr[np.where(m, i, 0)])
        tmp = np.where(m, nxt, tmp)
        i = i + step
    _inner_warp_reduction(op, sm, tid, tmp)
    # :91-97
    t2 = np.arange(2)
    sm[:, t2, 0] = op(sm[:, t2, 0], sm[:, t2 + 2, 0])
    partials[:grid] = op(sm[:, 0, 0], sm[:, 1, 0])


def _partial_block(op, arr, partials, sm, blksz):
    """reduction.py:99-141, one block of blksz == arr.size < 128 threads."""
    size = arr.size
    tid = np.arange(blksz)
    warpid, laneid = tid // WARPSIZE, tid % WARPSIZE
    value = arr[tid]
    sm[0, warpid, laneid] = value
    full = (warpid + 1) * WARPSIZE < size
    if full.any():
        _inner_warp_reduction(op, sm[:1], tid[full], value[full][None, :])
    for w in np.unique(warpid[~full]):
        base = w * WARPSIZE
        for i in range(1, size - base):
            sm[0, w, 0] = op(sm[0, w, 0], sm[0, w, i])
    num_active_warps = (blksz + WARPSIZE - 1) // WARPSIZE
    result = sm[0, 0, 0]
    for i in range(1, num_active_warps):
        result = op(result, sm[0, i, 0])
    partials[0] = result


def _launch(op, grid, block, arr, partials, init, use_init, dtype):
    """reduction.py:143-166"""
    sm = np.zeros((grid, NUMWARPS, WARPSIZE + 1), dtype)
    if block == BLOCKSIZE:
        _full_block(op, arr, partials, sm, grid)
    else:
        assert grid == 1
        _partial_block(op, arr, partials, sm, block)
    if use_init:
        partials[0] = op(partials[0], init)


def reduce(opname, arr, init=0):
    """Reduce.__call__, reduction.py:194-265."""
    arr = np.ascontiguousarray(arr)
    dtype = arr.dtype
    op = _ops(dtype)[opname]
    init = dtype.type(init)
    if arr.size < 1:
        return init
    size_full = (arr.size // BLOCKSIZE) * BLOCKSIZE
    size_partial = arr.size - size_full
    full_blockct = min(size_full // BLOCKSIZE, WARPSIZE * 2)
    partials_size = full_blockct + (1 if size_partial else 0)
    partials = np.zeros(partials_size, dtype)
    if size_full:
        _launch(op, full_blockct, BLOCKSIZE, arr[:size_full], partials[:full_blockct],
                init, True, dtype)
    if size_partial:
        _launch(op, 1, size_partial, arr[size_full:], partials[full_blockct:],
                init, not full_blockct, dtype)
    if partials.size > 1:
        _launch(op, 1, partials_size, partials, partials, init, False, dtype)
    return partials[0]

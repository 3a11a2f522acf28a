"""Device memory shared between two processes on one GPU (reference:
tests/cudapy/test_ipc.py:86-170: the same arrays, slices and three ways of passing the
handle; the second process is a spawned worker)."""

import concurrent.futures
import multiprocessing as mp
import os
import pickle
import sys

import numpy as np
import pytest

import numba_cuda_amd as cuda
from tests import ipc_children

pytestmark = pytest.mark.gpu

TIMEOUT = 150          # the first call also starts the worker and loads the libraries there
INDICES = (None, slice(3, None), slice(3, 8), slice(None, 8))


def _say(*what):
    print("[ipc]", *what, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def worker():
    exe = concurrent.futures.ProcessPoolExecutor(max_workers=1, mp_context=mp.get_context("spawn"))
    try:
        yield exe
    finally:
        exe.shutdown()


class _Foreign:
    def __init__(self, arr):
        self._arr = arr
        self.__cuda_array_interface__ = arr.__cuda_array_interface__


def _source(index, foreign):
    arr = np.arange(10, dtype=np.intp)
    devarr = cuda.to_device(arr)
    if index is not None:
        devarr = devarr[index]
    if foreign:
        devarr = cuda.as_cuda_array(_Foreign(devarr))
    return devarr, devarr.copy_to_host()


def test_raw_handle_bytes(worker):
    _say("raw handle")
    arr = np.arange(10, dtype=np.intp)
    devarr = cuda.to_device(arr)
    ipch = cuda.current_context().get_ipc_handle(devarr.gpu_data)
    fut = worker.submit(ipc_children.read_raw_handle, ipch.handle.reserved, ipch.size, parent_pid=os.getpid())
    np.testing.assert_array_equal(fut.result(timeout=TIMEOUT), arr)


@pytest.mark.parametrize("foreign", [False, True])
@pytest.mark.parametrize("index", INDICES, ids=str)
def test_pickled_handle(worker, index, foreign):
    _say("pickled handle", index, foreign)
    devarr, expect = _source(index, foreign)
    ctx = cuda.current_context()
    ipch = ctx.get_ipc_handle(devarr.gpu_data)
    recon = pickle.loads(pickle.dumps(ipch))
    assert recon.base is None and recon.size == ipch.size
    assert recon.handle.reserved == ipch.handle.reserved
    with pytest.raises(ValueError, match="opening IpcHandle from original process"):
        ipch.open(ctx)
    fut = worker.submit(ipc_children.read_pickled_handle, ipch, parent_pid=os.getpid())
    np.testing.assert_array_equal(fut.result(timeout=TIMEOUT), expect)


@pytest.mark.parametrize("foreign", [False, True])
@pytest.mark.parametrize("index", INDICES, ids=str)
def test_array_handle(worker, index, foreign):
    _say("array handle", index, foreign)
    devarr, expect = _source(index, foreign)
    fut = worker.submit(ipc_children.read_array_handle, devarr.get_ipc_handle(), parent_pid=os.getpid())
    np.testing.assert_array_equal(fut.result(timeout=TIMEOUT), expect)


def test_staged_open_on_every_device(worker):
    """tests/cudapy/test_ipc.py:212-233: the importer copies through the exporting device."""
    _say("staged")
    arr = np.arange(10, dtype=np.intp)
    devarr = cuda.to_device(arr)
    ipch = cuda.current_context().get_ipc_handle(devarr.gpu_data)
    for device_num in range(len(cuda.gpus)):
        fut = worker.submit(ipc_children.read_staged, ipch, device_num, parent_pid=os.getpid())
        np.testing.assert_array_equal(fut.result(timeout=TIMEOUT), arr)
    np.testing.assert_array_equal(devarr.copy_to_host(), arr)       # the child only wrote to its copy


def test_the_other_process_computes_on_and_writes_to_the_shared_array(worker):
    _say("compute in the other process")
    rng = np.random.default_rng(5)
    a = rng.integers(-8, 8, size=(300, 500)).astype(np.float32)     # sums exactly in float32
    devarr = cuda.to_device(a)
    fut = worker.submit(ipc_children.reduce_transpose_and_write, devarr.get_ipc_handle(), parent_pid=os.getpid())
    total, flipped = fut.result(timeout=TIMEOUT)
    assert total == float(a.sum(dtype=np.float64))
    np.testing.assert_array_equal(flipped, a.T)
    back = devarr.copy_to_host()
    assert (back[0] == -1.0).all()
    np.testing.assert_array_equal(back[1:], a[1:])


def test_pooled_memory_can_be_shared(worker):
    """Blocks of the caching pool are allocations of their own."""
    _say("pooled memory")
    from numba_cuda_amd.pool import PoolMemoryManager
    ctx = cuda.current_context()
    original = ctx.memory_manager
    ctx.memory_manager = PoolMemoryManager(context=ctx)
    try:
        cuda.current_context()                  # initialises the new manager
        arr = np.arange(1000, dtype=np.intp)
        devarr = cuda.to_device(arr)[100:]
        fut = worker.submit(ipc_children.read_array_handle, devarr.get_ipc_handle(), parent_pid=os.getpid())
        np.testing.assert_array_equal(fut.result(timeout=TIMEOUT), arr[100:])
        del devarr
    finally:
        ctx.memory_manager.reset()              # hands the idle blocks back to the driver
        ctx.memory_manager = original
        cuda.current_context()

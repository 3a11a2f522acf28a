"""Deferred deallocation as the reference's suite pins it
(numba_cuda/numba/cuda/tests/cudadrv/test_deallocations.py), restated with the lines
each case follows.  Run on the fake library and on the GPU."""
import contextlib
import gc
import io
import sys

import numpy as np
import pytest

from numba_cuda_amd.core import config
from numba_cuda_amd.cudadrv import driver


def _is_fake():
    return type(driver.driver.lib).__name__ == "FakeLib"


def _queue_of_the_default_manager(cuda):
    """These cases count device frees that wait in the default manager's queue; a pooling
    manager takes blocks back at once and never queues them."""
    mm = cuda.current_context().memory_manager
    if type(mm) is not driver.NumbaCUDAMemoryManager:
        pytest.skip("device frees do not wait in a queue under %s" % type(mm).__name__)


def pending_byte_threshold(cuda):
    # :31-58
    _queue_of_the_default_manager(cuda)
    ctx = cuda.current_context()
    deallocs = ctx.memory_manager.deallocations
    deallocs.clear()
    assert len(deallocs) == 0
    total = ctx.get_memory_info().total
    max_pending = 10**6
    old = config.CUDA_DEALLOCS_RATIO
    try:
        config.CUDA_DEALLOCS_RATIO = max_pending / total
        assert abs(deallocs.byte_budget - max_pending) <= 1
        cuda.to_device(np.ones(max_pending // 2, dtype=np.int8))
        gc.collect()
        assert len(deallocs) == 1
        cuda.to_device(np.ones(deallocs.byte_budget - deallocs.pending_bytes, dtype=np.int8))
        gc.collect()
        assert len(deallocs) == 2
        cuda.to_device(np.ones(1, dtype=np.int8))
        gc.collect()
        assert len(deallocs) == 0
    finally:
        config.CUDA_DEALLOCS_RATIO = old


def defer_cleanup_blocks(cuda):
    # :60-100
    _queue_of_the_default_manager(cuda)
    h = np.arange(5)
    for depth in (1, 2):
        d1 = cuda.to_device(h)
        deallocs = cuda.current_context().memory_manager.deallocations
        deallocs.clear()
        assert len(deallocs) == 0
        with contextlib.ExitStack() as stack:
            for _ in range(depth):
                stack.enter_context(cuda.defer_cleanup())
            d2 = cuda.to_device(h)
            del d1
            gc.collect()
            assert len(deallocs) == 1
            del d2
            gc.collect()
            assert len(deallocs) == 2
            deallocs.clear()
            assert len(deallocs) == 2          # nothing is freed while deferred
        deallocs.clear()
        assert len(deallocs) == 0


def defer_cleanup_survives_an_exception(cuda):
    # :102-128
    _queue_of_the_default_manager(cuda)
    h = np.arange(5)
    d1 = cuda.to_device(h)
    deallocs = cuda.current_context().memory_manager.deallocations
    deallocs.clear()

    class CustomError(Exception):
        pass

    with pytest.raises(CustomError):
        with cuda.defer_cleanup():
            d2 = cuda.to_device(h)
            del d2
            gc.collect()
            assert len(deallocs) == 1
            deallocs.clear()
            assert len(deallocs) == 1
            raise CustomError
    deallocs.clear()
    assert len(deallocs) == 0
    del d1
    gc.collect()
    assert len(deallocs) == 1
    deallocs.clear()
    assert len(deallocs) == 0


@contextlib.contextmanager
def _nothing_on_stderr(ctx):
    old, sys.stderr = sys.stderr, io.StringIO()
    try:
        yield
        gc.collect()
        ctx.deallocations.clear()
        ctx.memory_manager.deallocations.clear()
        text = sys.stderr.getvalue()
    finally:
        sys.stderr = old
    assert not text, text


def deleting_resources_is_silent(cuda):
    # :130-172
    ctx = cuda.current_context()
    makers = (ctx.create_stream, ctx.create_event, lambda: ctx.memhostalloc(32),
              lambda: ctx.memhostalloc(32, mapped=True), lambda: ctx.memalloc(32), lambda: ctx.memallocmanaged(32))
    for make in makers:
        obj = make()
        with _nothing_on_stderr(ctx):
            del obj


def pin_and_map_context_managers(cuda):
    # :174-222 (page-locking existing memory is refused on the GPU machines used here)
    if not _is_fake():
        return
    ctx = cuda.current_context()
    ctx.deallocations.clear()
    for manager in (cuda.pinned, cuda.mapped):
        class Boom(Exception):
            pass

        arr = np.zeros(1)
        with _nothing_on_stderr(ctx):
            with manager(arr):
                pass
            with manager(arr):
                pass
            with cuda.defer_cleanup():
                with manager(arr):
                    pass
                with manager(arr):
                    pass
            try:
                with manager(arr):
                    raise Boom
            except Boom:
                with manager(arr):
                    pass


ALL = [pending_byte_threshold, defer_cleanup_blocks, defer_cleanup_survives_an_exception,
       deleting_resources_is_silent, pin_and_map_context_managers]

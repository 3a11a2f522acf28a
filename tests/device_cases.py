"""Device selection, reset and the gpus list as the reference's suite pins them
(numba_cuda/numba/cuda/tests/cudadrv/test_select_device.py, test_reset_device.py,
test_context_stack.py, test_cuda_auto_context.py), restated with the lines each case
follows; what needs a second GPU or CUDA's context stack has no counterpart.  Run on
the fake library and on the GPU."""
import numbers
import threading
from queue import Queue

import numpy as np

from numba_cuda_amd.cudadrv import driver


def _in_threads(body, count):
    errors = Queue()

    def runner():
        try:
            body()
        except Exception as e:      # noqa: BLE001 - reported to the caller
            errors.put(e)

    for _ in range(count):
        t = threading.Thread(target=runner)
        t.start()
        t.join()
    found = []
    while not errors.empty():
        found.append(errors.get())
    assert found == []


def select_device_in_fresh_threads(cuda):
    # test_select_device.py:9-36
    def body():
        cuda.select_device(0)
        st = cuda.stream()
        d = cuda.to_device(np.arange(100), stream=st)
        st.synchronize()
        del d
        del st
        cuda.synchronize()

    _in_threads(body, 10)


def select_and_close_repeatedly(cuda):
    # test_reset_device.py:10-33
    def body():
        for _ in range(2):
            for d in range(driver.driver.get_device_count()):
                cuda.select_device(d)
                cuda.close()

    _in_threads(body, 1)
    cuda.select_device(0)


def gpus_list_and_memory_info(cuda):
    # test_context_stack.py:11-44, test_cuda_auto_context.py:8-19
    assert len(cuda.gpus) > 0 and len(list(cuda.gpus)) > 0
    for dev in cuda.list_devices():
        with cuda.gpus[dev.id]:
            assert cuda.gpus.current.id == dev.id
    mem = cuda.current_context().get_memory_info()
    assert isinstance(mem.free, numbers.Number) and mem.free == mem[0]
    assert isinstance(mem.total, numbers.Number) and mem.total == mem[1]
    assert mem.free <= mem.total
    a = np.arange(10, dtype=np.float32)
    back = np.empty_like(a)
    cuda.to_device(a).copy_to_host(back)
    assert np.allclose(a, back)


def active_context_and_push_pop(cuda):
    # test_context_stack.py:48-68 (the active context of a fresh thread is empty; after a device is
    # selected it names that device) and cudadrv/driver.py:1161-1175 (push / pop in LIFO order)
    seen = {}

    def fresh_thread():
        with driver.driver.get_active_context() as ac:
            seen["devnum"], seen["truth"] = ac.devnum, bool(ac)

    _in_threads(fresh_thread, 1)
    assert seen == {"devnum": None, "truth": False}
    cuda.select_device(0)
    with driver.driver.get_active_context() as ac:
        assert ac.devnum == 0 and ac.context_handle is not None and ac
    ctx = cuda.current_context()
    assert driver.driver.pop_active_context() is None       # nothing was pushed on this thread
    ctx.push()
    ctx.push()
    with driver.driver.get_active_context() as ac:
        assert ac.devnum == 0
    ctx.pop()
    ctx.pop()
    try:
        ctx.pop()
    except AssertionError:
        pass
    else:
        raise AssertionError("pop of a context that is not on the stack must fail")
    d = cuda.to_device(np.arange(4))
    assert d.copy_to_host().tolist() == [0, 1, 2, 3]


def auto_device_helper(cuda):
    # api.py:522-523
    host = np.arange(5.0)
    dev, fresh = cuda._auto_device(host)
    assert fresh and dev.copy_to_host().tolist() == host.tolist()
    again, fresh = cuda._auto_device(dev)
    assert again is dev and not fresh


def driver_and_runtime_versions(cuda):
    # cudadrv/driver.py:410-418, 2732-2736; cudadrv/runtime.py:15-33; device_init.py:128-143
    from numba_cuda_amd.cudadrv import runtime
    major, minor = driver.get_version()
    assert major >= 6 and 0 <= minor < 100
    assert runtime.get_version() == cuda.runtime.get_version() and runtime.get_version()[0] >= 6
    assert cuda.is_supported_version() is True


ALL = [select_device_in_fresh_threads, select_and_close_repeatedly, gpus_list_and_memory_info,
       active_context_and_push_pop, auto_device_helper, driver_and_runtime_versions]

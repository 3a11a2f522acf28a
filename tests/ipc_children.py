"""What the second process does in tests/test_gpu_ipc.py (run by a spawned worker, so
these must be importable functions).  torch goes first for the reason given in
tests/conftest.py: both processes must use the same HIP runtime."""

import os

try:
    import torch  # noqa: F401
except ImportError:
    pass

import numpy as np

import numba_cuda_amd as cuda


def read_raw_handle(handle_bytes, size, parent_pid):
    assert os.getpid() != parent_pid
    dtype = np.dtype(np.intp)
    with cuda.open_ipc_array(handle_bytes, shape=size // dtype.itemsize, dtype=dtype) as darr:
        return darr.copy_to_host()


def read_pickled_handle(handle, parent_pid):
    assert os.getpid() != parent_pid
    dtype = np.dtype(np.intp)
    darr = handle.open_array(cuda.current_context(), shape=handle.size // dtype.itemsize, dtype=dtype)
    arr = darr.copy_to_host()
    handle.close()
    return arr


def read_array_handle(ipcarr, parent_pid):
    assert os.getpid() != parent_pid
    with ipcarr as darr:
        arr = darr.copy_to_host()
        try:
            with ipcarr:
                pass
        except ValueError as e:
            assert "IpcHandle is already opened" in str(e)
        else:
            raise AssertionError("a second open must fail")
    return arr


def reduce_transpose_and_write(ipcarr, parent_pid):
    """Compute on the shared memory from this process and write into it."""
    assert os.getpid() != parent_pid
    with ipcarr as darr:
        total = cuda.reduce(lambda a, b: a + b)(darr.reshape(darr.size))
        flipped = cuda.kernels.transpose.transpose(darr).copy_to_host()
        darr[0, :] = -1.0
        cuda.synchronize()
    return float(total), flipped


def read_staged(handle, device_num, parent_pid):
    """The reference's staged case (tests/cudapy/test_ipc.py:177-191): a copy of the shared
    memory made through the exporting device; writes to the copy stay in this process."""
    assert os.getpid() != parent_pid
    with cuda.gpus[device_num]:
        ctx = cuda.devices.get_context()
        copy = handle.open_staged(ctx)
        count = handle.size // np.dtype(np.intp).itemsize
        host = np.zeros(count, dtype=np.intp)
        cuda.driver.device_to_host(host, copy, size=handle.size)
        cuda.driver.device_memset(copy, 0xFF, handle.size)      # must not reach the exporter
        cuda.synchronize()
        handle.close()
    return host

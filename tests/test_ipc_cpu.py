"""IPC handles, host logic: what travels, the bookkeeping of open / close and the
error messages (reference: tests/cudapy/test_ipc.py:86-170, cudadrv/driver.py:1408-1603).
The fake library's "other process" is this process, so a rebuilt handle can be opened
here; on a GPU that needs a second process (tests/test_gpu_ipc.py)."""

import pickle

import numpy as np
import pytest

import numba_cuda_amd as cuda
from numba_cuda_amd.cudadrv import driver as drv

INDICES = (None, slice(3, None), slice(3, 8), slice(None, 8))     # the reference's variants


class _Foreign:
    """An object that only offers the CUDA Array Interface."""

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


@pytest.mark.parametrize("foreign", [False, True])
@pytest.mark.parametrize("index", INDICES, ids=str)
def test_handle_pickles_and_opens(fake_gpu, index, foreign):
    devarr, expect = _source(index, foreign)
    ctx = cuda.current_context()
    ipch = ctx.get_ipc_handle(devarr.gpu_data)
    assert isinstance(ipch, cuda.IpcHandle) and ipch.base is not None
    assert ipch.size == expect.nbytes
    assert ipch.offset == (index.start or 0) * 8 if index is not None else ipch.offset == 0
    assert ipch.source_info == ctx.device.get_device_identity()
    assert len(ipch.handle.reserved) == 64
    with pytest.raises(ValueError, match="opening IpcHandle from original process"):
        ipch.open(ctx)

    recon = pickle.loads(pickle.dumps(ipch))
    assert recon.base is None and recon.size == ipch.size and recon.offset == ipch.offset
    assert recon.handle.reserved == ipch.handle.reserved and recon.source_info == ipch.source_info

    dtype = np.dtype(np.intp)
    darr = recon.open_array(ctx, shape=recon.size // dtype.itemsize, dtype=dtype)
    np.testing.assert_array_equal(darr.copy_to_host(), expect)
    with pytest.raises(ValueError, match="IpcHandle is already opened"):
        recon.open(ctx)
    recon.close()
    assert [c[0] for c in fake_gpu.calls if c[0].startswith("ipc_")] == ["ipc_get_handle", "ipc_open", "ipc_close"]
    with pytest.raises(ValueError, match="IpcHandle not opened"):
        recon.close()


@pytest.mark.parametrize("foreign", [False, True])
@pytest.mark.parametrize("index", INDICES, ids=str)
def test_array_handle(fake_gpu, index, foreign):
    devarr, expect = _source(index, foreign)
    ipcarr = pickle.loads(pickle.dumps(devarr.get_ipc_handle()))
    with ipcarr as darr:
        assert darr.shape == expect.shape and darr.dtype == expect.dtype
        np.testing.assert_array_equal(darr.copy_to_host(), expect)
        with pytest.raises(ValueError, match="IpcHandle is already opened"):
            with ipcarr:
                pass
    with ipcarr as darr:                       # closed by the block above: can be opened again
        np.testing.assert_array_equal(darr.copy_to_host(), expect)


def test_two_dimensional_array_keeps_its_layout(fake_gpu):
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    d = cuda.to_device(a)[1:, ::2]
    with pickle.loads(pickle.dumps(d.get_ipc_handle())) as shared:
        assert shared.shape == (3, 3) and shared.strides == d.strides
        np.testing.assert_array_equal(shared.copy_to_host(), a[1:, ::2])


@pytest.mark.parametrize("spell", [bytes, tuple, list])
def test_open_ipc_array_takes_raw_bytes(fake_gpu, spell):
    arr = np.arange(10, dtype=np.intp)
    devarr = cuda.to_device(arr)
    ipch = cuda.current_context().get_ipc_handle(devarr.gpu_data)
    raw = spell(ipch.handle.reserved)
    with cuda.open_ipc_array(raw, shape=ipch.size // 8, dtype=np.intp) as darr:
        np.testing.assert_array_equal(darr.copy_to_host(), arr)
    with cuda.open_ipc_array(raw, shape=4, dtype=np.intp, offset=3 * 8) as darr:
        np.testing.assert_array_equal(darr.copy_to_host(), arr[3:7])
    assert fake_gpu.ipc_open == []
    with pytest.raises(ValueError, match="64 bytes"):
        with cuda.open_ipc_array(b"short", shape=1, dtype=np.intp):
            pass


def test_large_allocations_are_refused(fake_gpu, monkeypatch):
    devarr = cuda.to_device(np.arange(10, dtype=np.intp))
    base = devarr.gpu_data.handle
    monkeypatch.setattr(drv, "device_extents", lambda mem: (base, base + (2 << 30)))
    with pytest.raises(ValueError, match="2 GiB or more cannot be shared"):
        devarr.get_ipc_handle()
    big = drv.IpcHandle(None, drv.IpcMemHandle(bytes(64)), size=2 << 30)
    with pytest.raises(ValueError, match="2 GiB or more cannot be shared"):
        big.open(cuda.current_context())
    with pytest.raises(ValueError, match="IpcHandle not opened"):   # the failed open left nothing behind
        big.close()


def test_other_cases(fake_gpu, monkeypatch):
    ctx = cuda.current_context()
    devarr = cuda.to_device(np.arange(4.0))
    ipch = ctx.get_ipc_handle(devarr.gpu_data)
    assert ipch.can_access_peer(ctx)
    anonymous = drv.IpcHandle(None, ipch.handle, ipch.size)
    with pytest.raises(RuntimeError, match="IPC handle doesn't have source info"):
        anonymous.can_access_peer(ctx)
    with pytest.raises(RuntimeError, match="IPC handle doesn't have source info"):
        anonymous.open_staged(ctx)
    elsewhere = pickle.loads(pickle.dumps(ipch))
    elsewhere.source_info = {"pci_domain_id": 9, "pci_bus_id": 9, "pci_device_id": 9}
    with pytest.raises(RuntimeError, match="No device of .* is found"):
        elsewhere.open(ctx)
    # staged: a copy through the exporting device (here the same one), owned by the caller
    with pytest.raises(ValueError, match="opening IpcHandle from original process"):
        ipch.open_staged(ctx)
    imported = pickle.loads(pickle.dumps(ipch))
    copy = imported.open_staged(ctx)
    got = np.zeros(4)
    drv.device_to_host(got, copy, got.nbytes)
    np.testing.assert_array_equal(got, np.arange(4.0))
    assert copy.device_pointer_value != devarr.gpu_data.device_pointer_value
    with pytest.raises(ValueError, match="IpcHandle is already opened"):
        imported.open_staged(ctx)
    imported.close()                                  # nothing to unmap; the copy lives on
    with pytest.raises(ValueError, match="IpcHandle not opened"):
        imported.close()
    monkeypatch.setattr(drv.sys, "platform", "win32")
    with pytest.raises(OSError, match="OS does not support CUDA IPC"):
        ctx.get_ipc_handle(devarr.gpu_data)


def test_plugins_can_reuse_the_default_implementation(fake_gpu):
    """An External Memory Management plugin built on hipMalloc gets get_ipc_handle()
    from the mixin (reference: driver.py:861-878)."""
    from tests.test_plumbing_cpu import _RecordingManager

    class WithIpc(cuda.GetIpcHandleMixin, _RecordingManager):
        def memalloc(self, size):
            return drv.NumbaCUDAMemoryManager.memalloc(self, size)

    cuda.set_memory_manager(WithIpc)
    try:
        d = cuda.to_device(np.arange(6, dtype=np.int32))
        h = d[2:].get_ipc_handle()
        assert h._ipc_handle.offset == 8 and h._ipc_handle.size == 16
    finally:
        drv._memory_manager = None

"""DeviceRecord and structured device arrays as the reference's suite pins them
(numba_cuda/numba/cuda/tests/cudadrv/test_cuda_devicerecord.py), restated with the
lines each case follows (numba type objects, :52-54, have no counterpart here).  Run
on the fake library and on the GPU."""
import numpy as np

from numba_cuda_amd.cudadrv.devicearray import DeviceRecord, auto_device, from_record_like

N_CHARS = 5
recordtype = np.dtype([("a", np.float64), ("b", np.int32), ("c", np.complex64), ("d", (np.str_, N_CHARS))],
                      align=True)
recordwitharray = np.dtype([("g", np.int32), ("h", np.float32, 2)], align=True)
recwithmat = np.dtype([("i", np.int32), ("j", np.float32, (3, 3))])
recwithrecwithmat = np.dtype([("x", np.int32), ("y", recwithmat)])


def _check(reference, rec):
    # :44-51
    assert rec.shape == () and rec.strides == ()
    assert rec.dtype == reference.dtype and rec.alloc_size == reference.dtype.itemsize
    assert rec.gpu_data is not None
    assert rec.device_ctypes_pointer.value not in (0, None)


def single_records(cuda):
    # :33-110, once with np.void and once with np.record host values
    dtype = np.dtype([("a", np.int32), ("b", np.float32)], align=True)
    for ctor in (np.zeros, np.recarray):
        hostz = ctor(1, dtype)[0]
        hostnz = ctor(1, dtype)[0]
        hostz["a"], hostz["b"] = 0, 0.0
        hostnz["a"], hostnz["b"] = 10, 11.0
        dev = DeviceRecord(dtype)
        _check(hostz.copy(), dev)
        dev.copy_to_device(hostz.copy())
        back = hostnz.copy()
        dev.copy_to_host(back)
        np.testing.assert_equal(hostz, back)
        dev.copy_to_device(hostnz.copy())
        back = hostz.copy()
        dev.copy_to_host(back)
        np.testing.assert_equal(back, hostnz)
        like = from_record_like(hostz.copy())
        _check(hostz, like)
        like2 = from_record_like(like)
        _check(like, like2)
        assert like.gpu_data != like2.gpu_data
        auto, created = auto_device(hostnz.copy())
        _check(hostnz, auto)
        assert created
        back = hostz.copy()
        auto.copy_to_host(back)
        np.testing.assert_equal(back, hostnz)


def structured_arrays(cuda):
    # :121-176
    ary = cuda.device_array(3, dtype=recordtype)
    for i in range(ary.size):
        x = i + 1
        ary[i]["a"] = x / 2
        ary[i]["b"] = x
        ary[i]["c"] = x * 1j
        ary[i]["d"] = str(x) * N_CHARS
    for i in range(ary.size):
        x = i + 1
        assert ary[i]["a"] == x / 2 and ary[i]["b"] == x and ary[i]["c"] == x * 1j
        assert ary[i]["d"] == str(x) * N_CHARS
    rec = cuda.device_array(1, dtype=recordwitharray)[0]
    rec["g"] = 2
    rec["h"][0] = 3.0
    rec["h"][1] = 4.0
    assert rec["g"] == 2 and rec["h"][0] == 3.0 and rec["h"][1] == 4.0
    rec = cuda.device_array(1, dtype=recwithmat)[0]
    mat = np.array([[5.0, 10.0, 15.0], [20.0, 25.0, 30.0], [35.0, 40.0, 45.0]], dtype=np.float32)
    rec["j"][:] = mat
    np.testing.assert_equal(rec["j"], mat)
    d = cuda.to_device(np.zeros(1, dtype=recwithrecwithmat))
    d[0]["y"]["i"] = 1
    assert d[0]["y"]["i"] == 1
    d[0]["y"]["j"][0, 0] = 2.0
    assert d[0]["y"]["j"][0, 0] == 2.0


ALL = [single_records, structured_arrays]

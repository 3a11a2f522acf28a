"""Contiguity queries, ravel and reshape as the reference's suite pins them
(numba_cuda/numba/cuda/tests/cudadrv/test_array_attr.py), restated with the lines each
case follows.  Run on the fake library and on the GPU."""
import numpy as np
import pytest


def contiguity_queries(cuda):
    # :10-47
    for shape in ((2, 5), (2, 5, 2), (2, 5, 2, 3)):
        c = np.arange(int(np.prod(shape))).reshape(shape)
        f = np.asfortranarray(c)
        dc, df = cuda.to_device(c), cuda.to_device(f)
        assert dc.is_c_contiguous() and not df.is_c_contiguous()
        assert not dc.is_f_contiguous() and df.is_f_contiguous()


def _same(expect, got):
    assert expect.dtype == got.dtype and expect.shape == got.shape and np.array_equal(expect, got)


def ravel(cuda):
    # :49-60
    h = np.arange(60)
    d = cuda.to_device(h)
    for order in "CFA":
        flat = d.ravel(order=order)
        assert flat is not d
        _same(h.ravel(order=order), flat.copy_to_host())
    # :76-95, :111-121
    shaped = h.reshape(2, 5, 2, 3)
    for host, orders in ((shaped, "CA"), (np.asfortranarray(shaped), "FA")):
        for order in orders:
            d = cuda.to_device(host)
            flat = d.ravel(order=order)
            assert flat is not d and flat.ndim == 1
            _same(host.ravel(order=order), flat.copy_to_host())
    _same(shaped.ravel(), cuda.to_device(shaped).ravel().copy_to_host())
    # :62-74, :97-109, :123-135: strided views share the base address and cannot be flattened
    for host, key in ((h, (slice(None, None, 2),)), (shaped, (slice(None, None, 2),) * 4),
                      (np.asfortranarray(shaped), (slice(None, None, 2),) * 4)):
        d = cuda.to_device(host)
        view = d[key]
        assert d.__cuda_array_interface__["data"][0] == view.__cuda_array_interface__["data"][0]
        with pytest.raises(NotImplementedError):
            view.ravel()


def reshape(cuda):
    # :137-153
    h = np.arange(10)
    d = cuda.to_device(h)
    _same(h.reshape(2, 5), d.reshape(2, 5).copy_to_host())
    _same(h.reshape(2, 5, order="F"), d.reshape(2, 5, order="F").copy_to_host())


ALL = [contiguity_queries, ravel, reshape]

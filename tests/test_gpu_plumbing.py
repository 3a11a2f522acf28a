"""Device-array plumbing on the real library and GPU."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from tests import plumbing_cases


@pytest.mark.parametrize("case", plumbing_cases.ALL, ids=lambda f: f.__name__)
def test_plumbing(case):
    print(case.__name__, flush=True)
    case(cuda)


def test_memset_and_views_of_raw_memory():
    d = cuda.device_array(64, np.uint8)
    d.gpu_data.memset(0xAB)
    assert (d.copy_to_host() == 0xAB).all()
    cuda.cudadrv.driver.device_memset(d, 1, 16)
    assert d.copy_to_host().tolist() == [1] * 16 + [0xAB] * 48
    lo, hi = cuda.cudadrv.driver.device_extents(d)
    assert lo <= d.device_ctypes_pointer.value < hi
    assert cuda.cudadrv.driver.device_memory_size(d.gpu_data) == 64


def test_mapped_array_is_device_addressable():
    m = cuda.mapped_array(1000, dtype=np.float32)
    m[:] = np.arange(1000, dtype=np.float32)
    got = cuda.reduce(lambda a, b: a + b)(m)
    assert got == np.arange(1000, dtype=np.float32).sum()


def test_cuda_array_interface_with_torch_tensors():
    """Zero-copy import of a PyTorch-ROCm tensor, checked against torch itself."""
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    t = torch.arange(1 << 20, dtype=torch.float32, device="cuda").reshape(1024, 1024)
    torch.cuda.synchronize()
    assert cuda.is_cuda_array(t)
    d = cuda.as_cuda_array(t)
    assert d.shape == (1024, 1024) and d.device_ctypes_pointer.value == t.data_ptr()
    got = cuda.reduce(lambda a, b: a + b)(d.reshape(-1))
    assert got == float(t.sum().item())
    tt = d.T
    back = torch.as_tensor(tt, device="cuda")
    assert torch.equal(back, t.t().contiguous())
    with pytest.raises(TypeError):
        cuda.as_cuda_array(np.zeros(3))

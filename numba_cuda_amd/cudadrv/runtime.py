"""Version of the HIP runtime the library is linked against, under the names user code
knows from the reference (numba/cuda/cudadrv/runtime.py:13-33, where they report the CUDA
toolkit).  The numbers come from the GPU library (`nbh_hip_versions`); no device is needed."""

from . import driver as _driver

# major versions of ROCm whose HIP runtime the kernels are built and tested with
SUPPORTED_TOOLKIT_MAJOR_VERSIONS = (6, 7)


class Runtime:
    """`cuda.runtime`: what runs underneath."""

    tested_majors = frozenset(SUPPORTED_TOOLKIT_MAJOR_VERSIONS)

    def get_version(self):
        _, of_runtime = _driver.driver.hip_versions()
        return of_runtime                      # (major, minor)

    def is_supported_version(self):
        major, _minor = self.get_version()
        return major in self.tested_majors


runtime = Runtime()
get_version = runtime.get_version

"""The runtime's version, under the names of the reference's
numba/cuda/cudadrv/runtime.py:13-33 (there: the CUDA toolkit's version; here: the HIP
runtime's, asked of the library)."""

from .driver import driver

# ROCm releases this package's kernels are built and tested with
SUPPORTED_TOOLKIT_MAJOR_VERSIONS = (6, 7)


class Runtime:
    def get_version(self):
        """(major, minor) of the HIP runtime."""
        return driver.hip_versions()[1]

    def is_supported_version(self):
        """Whether the HIP runtime is a version this package is tested with."""
        return self.get_version()[0] in SUPPORTED_TOOLKIT_MAJOR_VERSIONS


runtime = Runtime()


def get_version():
    """The runtime's version as (major, minor)."""
    return runtime.get_version()

"""Intent wrappers for host arrays handed to device operations (reference:
numba_cuda/numba/cuda/args.py:15-88): `In` copies to the device before,
`Out` copies back after, `InOut` does both."""

from numba_cuda_amd.cudadrv import devicearray


class ArgHint:
    def __init__(self, value):
        self.value = value

    def to_device(self, retr, stream=0):
        """-> device object for the operation; appends write-back callbacks to `retr`."""
        raise NotImplementedError


class In(ArgHint):
    def to_device(self, retr, stream=0):
        devary, _ = devicearray.auto_device(self.value, stream=stream)
        return devary


class Out(ArgHint):
    def to_device(self, retr, stream=0):
        devary, conv = devicearray.auto_device(self.value, copy=False, stream=stream)
        if conv:
            retr.append(lambda: devary.copy_to_host(self.value, stream=stream))
        return devary


class InOut(ArgHint):
    def to_device(self, retr, stream=0):
        devary, conv = devicearray.auto_device(self.value, stream=stream)
        if conv:
            retr.append(lambda: devary.copy_to_host(self.value, stream=stream))
        return devary


def wrap_arg(value, default=InOut):
    return value if isinstance(value, ArgHint) else default(value)


__all__ = ["In", "Out", "InOut", "ArgHint", "wrap_arg"]

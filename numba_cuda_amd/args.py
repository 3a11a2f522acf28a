"""Intent wrappers for host arrays handed to device operations (reference:
numba_cuda/numba/cuda/args.py:15-88): `In` copies to the device before the
operation, `Out` copies back after it, `InOut` does both.  Objects that already
live on the device pass through untouched whatever the wrapper."""

from numba_cuda_amd.cudadrv import devicearray


class ArgHint:
    """A value together with the direction(s) its data has to travel.  The two class
    flags are all a subclass sets."""

    copy_in = True      # host -> device before the operation
    copy_out = True     # device -> host after it

    def __init__(self, value):
        self.value = value

    def to_device(self, retr, stream=0):
        """-> the device object to operate on.  When a device copy had to be made and
        results are to come back, a callable doing that copy is appended to `retr`
        for the caller to run after the operation."""
        on_device, was_copied = devicearray.auto_device(self.value, copy=self.copy_in, stream=stream)
        if was_copied and self.copy_out:
            host = self.value

            def write_back():
                on_device.copy_to_host(host, stream=stream)

            retr.append(write_back)
        return on_device


class In(ArgHint):
    copy_out = False


class Out(ArgHint):
    copy_in = False


class InOut(ArgHint):
    pass


def wrap_arg(value, default=InOut):
    """`value` itself if it already says which way it goes, else `default(value)`."""
    if isinstance(value, ArgHint):
        return value
    return default(value)


__all__ = ["In", "Out", "InOut", "ArgHint", "wrap_arg"]

"""In / Out / InOut in the CPU mode (numba_cuda/numba/cuda/simulator/args.py): the same
three intents as on the GPU, over NumPy-backed arrays."""

from numba_cuda_amd.simulator import hostarray


class ArgHint:
    copy_in = True
    copy_out = True

    def __init__(self, value):
        self.value = value

    def to_device(self, retr, stream=0):
        on_device, was_copied = hostarray.auto_device(self.value, copy=self.copy_in, stream=stream)
        if was_copied and self.copy_out:
            host = self.value
            retr.append(lambda: on_device.copy_to_host(host, stream=stream))
        return on_device


class In(ArgHint):
    copy_out = False


class Out(ArgHint):
    copy_in = False


class InOut(ArgHint):
    pass


def wrap_arg(value, default=InOut):
    return value if isinstance(value, ArgHint) else default(value)

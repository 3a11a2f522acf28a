"""Streams, events, devices and contexts of the CPU mode: everything runs at once on the
calling thread, so these keep the interface and do nothing
(numba_cuda/numba/cuda/simulator/api.py:28-120, simulator/cudadrv/devices.py)."""

from contextlib import contextmanager


class Stream:
    handle = None

    @contextmanager
    def auto_synchronize(self):
        yield

    def synchronize(self):
        pass

    def __int__(self):
        return 0


stream = Stream
default_stream = Stream
legacy_default_stream = Stream
per_thread_default_stream = Stream


def external_stream(ptr):
    raise RuntimeError("External streams are unsupported in the simulator")


class Event:
    def record(self, stream=0):
        pass

    def wait(self, stream=0):
        pass

    def synchronize(self):
        pass

    def query(self):
        return True

    def elapsed_time(self, event):
        """Kept for the interface; nothing is timed."""
        return -1.0


def event(timing=True):
    return Event()


def event_elapsed_time(start, end):
    return start.elapsed_time(end)


def synchronize():
    pass


class FakeDevice:
    id = 0
    name = "SIMULATOR"
    compute_capability = (5, 0)
    uuid = "GPU-00000000-0000-0000-0000-000000000000"

    def reset(self):
        pass


class FakeContext:
    """The one context of the one simulated device."""

    def __init__(self, device):
        self.device = device

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False

    def reset(self):
        pass

    def synchronize(self):
        pass

    def get_memory_info(self):
        import collections
        import psutil
        mem = psutil.virtual_memory()
        return collections.namedtuple("MemoryInfo", "free,total")(mem.available, mem.total)

    def __str__(self):
        return "<Managed Device 0>"


class _DeviceList:
    def __init__(self):
        self.lst = (FakeContext(FakeDevice()),)
        self.closed = False

    def __getitem__(self, index):
        if not isinstance(index, int) or index != 0:
            raise AssertionError("Only a single device supported by the simulator")
        return self.lst[0]

    def __iter__(self):
        return iter(self.lst)

    def __len__(self):
        return 1

    def __str__(self):
        return ", ".join(str(d) for d in self.lst)

    @property
    def current(self):
        return None if self.closed else self.lst[0]


gpus = _DeviceList()


def list_devices():
    return gpus


def get_context(devnum=0):
    return gpus[devnum]


current_context = get_context


def require_context(fn):
    return fn


def select_device(dev=0):
    assert dev == 0, "Only a single device supported by the simulator"
    return gpus[0].device


def get_current_device():
    return gpus[0].device


def close():
    gpus.closed = True


def reset():
    gpus[0].reset()
    gpus.closed = False


def detect():
    print("Found 1 CUDA devices")
    print("id %d    %20s %40s" % (0, "SIMULATOR", "[SUPPORTED]"))
    print("%40s: 5.0" % "compute capability")
    return True


def is_available():
    return True


def cuda_error():
    return None


def is_supported_version():
    return True


def is_float16_supported():
    return True


def is_bfloat16_supported():
    return False


@contextmanager
def defer_cleanup():
    yield


def profile_start():
    pass


def profile_stop():
    pass


@contextmanager
def profiling():
    yield

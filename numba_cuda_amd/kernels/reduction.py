"""`Reduce`: full reduction of a 1-d array with a binary operator.

Drop-in for numba_cuda/numba/cuda/kernels/reduction.py:169-265.  The reference
JIT-compiles the Python functor into a three-launch tree reduction.  Here the functor is
first *recognised*: a + b, a * b, max(a, b), min(a, b), and a & b, a | b, a ^ b on
integers have hand-written HIP kernels, and a single launch of nbh_reduce does the work.
Element types on that path: the integers, booleans, float16 (accumulated in float16, as
the reference's JIT does), float32, float64, complex64 and complex128.

Any other functor is translated (kernels/functor.py: run on recording stand-ins, typed
with the JIT's rules, written out as C++) and compiled for the device at run time, once
per functor and element type; nbh_reduce_custom then runs it in one launch.  Element
types there: integers, booleans and the real floating-point types.  What cannot be
translated raises NotImplementedError - there is no host fallback.
"""

import operator

import numpy as np

from numba_cuda_amd import _lib
from numba_cuda_amd.core import config as _config
from numba_cuda_amd.cudadrv import devicearray, devices
from numba_cuda_amd.cudadrv import driver as _driver
from numba_cuda_amd.kernels import functor as _functor


class _Sym:
    """Operand stand-in that records which operator the functor applies."""

    def __init__(self, name, log):
        self.name, self.log = name, log

    def _binary(self, opname, other, swapped=False):
        if not isinstance(other, _Sym):
            raise _Unrecognised("operand mixed with a constant")
        lhs, rhs = (other, self) if swapped else (self, other)
        self.log.append((opname, lhs.name, rhs.name))
        return _Sym("(%s %s %s)" % (lhs.name, opname, rhs.name), self.log)

    def __add__(self, o):
        return self._binary("add", o)

    def __radd__(self, o):
        return self._binary("add", o, True)

    def __mul__(self, o):
        return self._binary("mul", o)

    def __rmul__(self, o):
        return self._binary("mul", o, True)

    def __and__(self, o):
        return self._binary("and", o)

    def __rand__(self, o):
        return self._binary("and", o, True)

    def __or__(self, o):
        return self._binary("or", o)

    def __ror__(self, o):
        return self._binary("or", o, True)

    def __xor__(self, o):
        return self._binary("xor", o)

    def __rxor__(self, o):
        return self._binary("xor", o, True)

    def _compare(self, opname, other):
        if not isinstance(other, _Sym):
            raise _Unrecognised("operand compared with a constant")
        return _Cond(opname, self.name, other.name, self.log)

    def __gt__(self, o):
        return self._compare("gt", o)

    def __lt__(self, o):
        return self._compare("lt", o)

    def __ge__(self, o):
        return self._compare("ge", o)

    def __le__(self, o):
        return self._compare("le", o)

    def __bool__(self):
        raise _Unrecognised("truth value of an operand")


class _Cond:
    """Result of comparing two stand-ins; its truth value is scripted."""

    def __init__(self, opname, lhs, rhs, log):
        self.key = (opname, lhs, rhs)
        self.log = log

    def __bool__(self):
        self.log.append(("cmp",) + self.key)
        return self.log.answer


class _Log(list):
    answer = True


class _Unrecognised(Exception):
    pass


_DIRECT = {operator.add: "add", operator.mul: "mul", max: "max", min: "min",
           np.add: "add", np.multiply: "mul",
           operator.and_: "and", operator.or_: "or", operator.xor: "xor",
           np.bitwise_and: "and", np.bitwise_or: "or", np.bitwise_xor: "xor"}
_ARITHMETIC = ("add", "mul", "and", "or", "xor")


def _trace(functor, answer):
    log = _Log()
    log.answer = answer
    out = functor(_Sym("a", log), _Sym("b", log))
    if not isinstance(out, _Sym):
        raise _Unrecognised("functor did not return one of its operands or their sum/product")
    return out.name, list(log)


def classify_functor(functor, detail=None):
    """-> "add" | "mul" | "max" | "min" | "and" | "or" | "xor", or NotImplementedError.
    `detail`, a dict, receives "kernel_form": False when the functor is a max / min whose
    comparison treats NaN and equal operands (signed zeros) differently from the kernels'
    own `b if b > a else a` / `b if b < a else a`, which is what max(a, b) / min(a, b) do.

    The functor is run on two recording stand-ins.  `a + b` / `a * b` show up as
    one arithmetic event.  `max(a, b)` / `min(a, b)` and the equivalent
    conditional expressions show up as one comparison whose scripted outcome
    decides which operand comes back; running with both outcomes tells max from
    min.  The verdict is then confirmed on real numbers."""
    try:
        if functor in _DIRECT:
            return _DIRECT[functor]
    except TypeError:
        pass
    verdict = None
    try:
        name_t, log_t = _trace(functor, True)
        name_f, log_f = _trace(functor, False)
        if len(log_t) == 1 and log_t == log_f and log_t[0][0] in _ARITHMETIC:
            if {log_t[0][1], log_t[0][2]} == {"a", "b"}:
                verdict = log_t[0][0]
        elif (len(log_t) == 1 and len(log_f) == 1 and log_t[0][0] == "cmp" and log_t == log_f
              and {name_t, name_f} == {"a", "b"}):
            _, cmp_op, lhs, rhs = log_t[0]
            if {lhs, rhs} == {"a", "b"}:
                # when "lhs <cmp_op> rhs" holds the functor returns name_t
                greater_wins = (cmp_op in ("gt", "ge")) == (name_t == lhs)
                verdict = "max" if greater_wins else "min"
                # the kernels: a strict comparison that, when it holds, picks the LATER operand
                if detail is not None:
                    detail["kernel_form"] = cmp_op in ("gt", "lt") and name_t == "b"
    except _Unrecognised:
        verdict = None
    except Exception:
        verdict = None
    if verdict is not None:
        probes = {"add": 8, "mul": 15, "max": 5, "min": 3, "and": 1, "or": 7, "xor": 6}
        try:
            ok = functor(3, 5) == probes[verdict] and functor(5, 3) == probes[verdict]
        except Exception:
            ok = False
        if ok:
            return verdict
    raise NotImplementedError(
        "Reduce supports the binary operators a + b, a * b, max(a, b), min(a, b) and, for integers, "
        "a & b, a | b, a ^ b; "
        "%r was not recognised as one of them" % (functor,))


class Reduce:
    """Reduction object for a binary function; the recognised operator is cached
    in the object and per functor."""

    _cache = {}

    def __init__(self, functor, reference_order=None):
        """`functor`: the binary operation, e.g. ``lambda a, b: a + b``.

        `reference_order` (not in the reference): True applies the operator to the same pairs
        of values, in the same order, as the reference's kernels do, so that floating-point
        sums and products - and what max / min make of NaN and signed zeros - come out bit for
        bit as the reference computes them (about 5 TB/s instead of 7); False uses this
        library's own order (within 2 n eps sum|x| of it); None takes the setting of
        NUMBA_CUDA_REDUCE_REFERENCE_ORDER (default 0).  Integer and boolean results of the
        operators with kernels of their own are the same either way.  A translated functor
        (any other operation) is applied in the reference's order too: its result then is the
        reference's also where the operation is not associative."""
        self._functor = functor
        if reference_order is None:
            reference_order = bool(_config.CUDA_REDUCE_REFERENCE_ORDER)
        self._ordered = bool(reference_order)
        self._kernel_form = True
        self._twin = None
        try:
            self._op, self._kernel_form = self._cache[functor]
        except (KeyError, TypeError):
            try:
                detail = {}
                self._op = classify_functor(functor, detail)
                self._kernel_form = detail.get("kernel_form", True)
            except NotImplementedError:
                # not one of the operators with kernels of their own: translate it
                try:
                    self._op = _functor.trace(functor)
                except NotImplementedError as why:
                    raise NotImplementedError(
                        "Reduce could not translate %r for the device: %s.  Translated are arithmetic, "
                        "comparisons, conditionals and math functions of the two operands." % (functor, why)) from None
            try:
                self._cache[functor] = (self._op, self._kernel_form)
            except TypeError:
                pass
        self._custom = not isinstance(self._op, str)
        # cases the native passage does not take
        self._native_off = self._custom or self._ordered or not self._kernel_form
        self._opcode = None if self._custom else _lib.OP_CODES[self._op]
        self._codes = {}    # dtype -> (operator code, element code), filled once the pairing is checked
                            # (translated functors: dtype -> handle of the compiled operation)

    def _codes_for(self, dtype):
        """(operator code, element code) nbh_reduce is called with for arrays of `dtype`."""
        opcode = self._opcode
        if dtype == _BOOL:
            # One byte holding 0 or 1, reduced by the uint8 kernels.  and / or / xor / max /
            # min of such bytes are again 0 or 1.  `a + b` and `a * b` are typed int64 by
            # the reference's JIT and converted back with `!= 0` wherever the kernels store
            # them into their boolean arrays (kernels/reduction.py:32-37, :96), which makes
            # the sum "any is true" and the product "all are true": the or / and kernels.
            if self._op == "add":
                opcode = _lib.OP_CODES["or"]
            elif self._op == "mul":
                opcode = _lib.OP_CODES["and"]
            return opcode, _DTYPE_CODE[np.dtype(np.uint8)]
        code = _DTYPE_CODE.get(dtype)
        if code is None:
            raise NotImplementedError("Reduce does not support dtype %s" % dtype)
        if dtype.kind == "c" and self._op in ("max", "min"):
            # the reference fails the same way, at compile time: complex numbers are not ordered
            raise TypeError("max / min are not defined for %s" % dtype)
        if dtype.kind not in "iu" and self._op in ("and", "or", "xor"):
            # the reference fails at compile time too: no bitwise operators on floating point
            raise TypeError("bitwise %s is not defined for %s" % (self._op, dtype))
        return opcode, code

    def __call__(self, arr, size=None, res=None, init=0, stream=0):
        """Full reduction of `arr`.

        arr    : 1-d host or device array
        size   : reduce only the first `size` items
        res    : device array; the result goes into its first item and nothing is
                 copied to the host (the call is then fully asynchronous)
        init   : initial value, converted to arr.dtype
        stream : stream to work on (0: the default stream)
        Returns the result as a NumPy scalar, or None when `res` is given.
        """
        # This is the whole per-call cost of small reductions (a 256 KiB row takes the
        # device 3 us).  The plain case with `res=` goes from the array objects to the
        # launch in native code (arrays this path has seen before carry their address,
        # length, stride and dtype as `_rk`); everything else, and whatever that call
        # declines, takes the path below: plain attribute reads, dictionary look-ups and
        # one native call.
        if res is not None and size is None and not self._native_off:
            rc = _reduce_into(self._codes, arr, res, init, stream, _thread_state, _Stream, _INT_INIT,
                              _driver.driver.lib)
            if rc is None:
                return None
            if rc is not NotImplemented:
                _driver.driver.check("nbh_reduce", rc)
        if arr.ndim != 1:
            raise TypeError("only support 1D array")
        if size is not None:
            arr = arr[:size]
        dtype = arr.dtype
        n = arr.size
        if n < 1:
            return dtype.type(init)          # `res` is left untouched, as in the reference
        if self._custom:
            return self._call_translated(arr, dtype, n, res, init, stream)
        if not self._kernel_form and dtype.kind == "f":
            # a max / min spelled with another comparison than the kernels': the same for
            # integers, not for NaN and signed zeros - floating point takes the translated functor
            twin = self._twin
            if twin is None:
                twin = self._twin = Reduce.__new__(Reduce)
                twin.__dict__.update(self.__dict__)
                twin._op, twin._custom, twin._codes = _functor.trace(self._functor), True, {}
            return twin._call_translated(arr, dtype, n, res, init, stream)

        codes = self._codes.get(dtype)
        if codes is None:
            codes = self._codes[dtype] = self._codes_for(dtype)

        ctx = getattr(_thread_state, "ctx", None)       # devices.get_context() without the calls
        if ctx is None or not ctx.prepared:
            ctx = devices.get_context()
        try:
            in_ptr = arr.gpu_data.device_pointer
        except AttributeError:
            if not _driver.is_device_memory(arr):
                # host input: implicit transfer, as a kernel argument would get
                arr, _ = devicearray.auto_device(arr, stream=stream)
            in_ptr = arr.device_ctypes_pointer.value

        hstream = stream._h if stream.__class__ is _Stream else _driver._stream_handle(stream)
        scratch = ctx._scratch.get(hstream)
        if scratch is None or hstream == _PER_THREAD:
            scratch = ctx.reduce_scratch(hstream)
        init_ptr = _INT_INIT.get((dtype, init)) if init.__class__ is int else None
        if init_ptr is None:
            init_ptr = _init_buffer(dtype, init)
        lib = _driver.driver.lib
        try:
            entry = lib._reduce_entry
        except AttributeError:
            entry = lib._reduce_entry = _entry_address(lib)
        reduce_fn = lib.nbh_reduce
        if self._ordered:                    # the reference's association: its own entry point
            entry, reduce_fn = 0, lib.nbh_reduce_ordered

        if res is not None:
            _check_result_array(res, dtype)
            try:
                out_ptr = res.gpu_data.device_pointer
            except AttributeError:
                out_ptr = res.device_ctypes_pointer.value
            if entry:
                if size is None:
                    # what the native passage needs to know about the two arrays next time
                    try:
                        arr._rk = (in_ptr, n, arr.strides[0], dtype)
                        if res.ndim == 1 and res.size >= 1:
                            res._rk = (out_ptr, res.size, res.strides[0], res.dtype)
                    except AttributeError:
                        pass
                rc = _call_reduce(entry, codes[0], codes[1], in_ptr, n, arr.strides[0], init_ptr, out_ptr,
                                  scratch[0], scratch[1], hstream)
            else:
                rc = reduce_fn(codes[0], codes[1], in_ptr, n, arr.strides[0], init_ptr, out_ptr,
                               scratch[0], scratch[1], hstream or None)
            if rc:
                _driver.driver.check("nbh_reduce", rc)
            return None
        # The value is wanted on the host: the kernel writes it into a cell of host
        # memory the device can address (taken for this call alone, so that calls from
        # other threads or on other streams cannot land in it), the host waits for the
        # stream and reads the cell - no copy back.
        cell = ctx.take_result_cell()
        try:
            rc = reduce_fn(codes[0], codes[1], in_ptr, n, arr.strides[0], init_ptr, cell[0],
                           scratch[0], scratch[1], hstream or None)
            if rc:
                _driver.driver.check("nbh_reduce", rc)
            _driver.driver.nbh_stream_synchronize(hstream or None)
            return cell[1][:dtype.itemsize].view(dtype)[0]
        finally:
            ctx.give_back_result_cell(cell)


    def _call_translated(self, arr, dtype, n, res, init, stream):
        """The same call for a functor that was translated and compiled at run time."""
        ctx = devices.get_context()              # also loads the library on the first call
        handle = self._codes.get(dtype)
        if handle is None:
            handle = self._codes[dtype] = compile_translated(self._op, dtype)
        if not _driver.is_device_memory(arr):
            arr, _ = devicearray.auto_device(arr, stream=stream)
        in_ptr = arr.device_ctypes_pointer.value
        hstream = _driver._stream_handle(stream)
        scratch = ctx.reduce_scratch(hstream)
        init_ptr = _init_buffer(dtype, init)
        lib = _driver.driver.lib
        launch, name = lib.nbh_reduce_custom, "nbh_reduce_custom"
        if self._ordered:                        # the reference's association: its own entry point
            launch, name = lib.nbh_reduce_custom_ordered, "nbh_reduce_custom_ordered"
        if res is not None:
            _check_result_array(res, dtype)
            rc = launch(handle, in_ptr, n, arr.strides[0], init_ptr, res.device_ctypes_pointer.value,
                        scratch[0], scratch[1], hstream or None)
            if rc:
                _driver.driver.check(name, rc)
            return None
        cell = ctx.take_result_cell()
        try:
            rc = launch(handle, in_ptr, n, arr.strides[0], init_ptr, cell[0],
                        scratch[0], scratch[1], hstream or None)
            if rc:
                _driver.driver.check(name, rc)
            _driver.driver.nbh_stream_synchronize(hstream or None)
            return cell[1][:dtype.itemsize].view(dtype)[0]
        finally:
            ctx.give_back_result_cell(cell)


def _check_result_array(res, dtype):
    """The reference stores the result with res[:1].copy_to_device(partials[:1])
    (kernels/reduction.py:259-262): `res` must hold the dtype and its first slice exactly
    one item."""
    if res.dtype != dtype:
        raise TypeError("res has dtype %s, expected %s" % (res.dtype, dtype))
    if res.ndim == 0:
        raise IndexError("too many indices for array: res is 0-dimensional")
    head = (min(1, res.shape[0]),) + tuple(res.shape[1:])
    items = 1
    for extent in head:
        items *= extent
    if items != 1:
        raise ValueError("incompatible shape: %s vs. (1,)" % (head,))


# (body, element code) -> handle from nbh_reduce_compile, kept for the life of the process
_COMPILED = {}


def compile_translated(expr, dtype):
    """Handle of the compiled operation for an expression tree and an element type
    (what Reduce._compile, kernels/reduction.py:182-190, is in the reference)."""
    import ctypes
    body = _functor.body_for(expr, dtype)
    code = _DTYPE_CODE[np.dtype(np.uint8)] if dtype == _BOOL else _DTYPE_CODE.get(dtype)
    if code is None:
        raise NotImplementedError("Reduce with a general functor does not support dtype %s" % dtype)
    key = (body, code)
    handle = _COMPILED.get(key)
    if handle is None:
        lib = _driver.driver.lib
        out = ctypes.c_void_p()
        log = ctypes.create_string_buffer(8192)
        rc = lib.nbh_reduce_compile(code, body.encode(), ctypes.byref(out), log, len(log))
        if rc:
            raise RuntimeError("compiling the functor for %s failed (error %d)\n%s\n-- generated code --\n%s"
                               % (dtype, rc, log.value.decode(errors="replace"), body))
        handle = _COMPILED[key] = out.value
    return handle


_Stream = _driver.Stream
_PER_THREAD = _driver.HIP_STREAM_PER_THREAD
_thread_state = devices._runtime._tls
_call_reduce = _driver._hostbuf.call_reduce
_reduce_into = getattr(_driver._hostbuf, "reduce_into", lambda *args: NotImplemented)   # absent from an older build

def _entry_address(lib):
    """Address of the library's nbh_reduce (nbh_reduce_queued with launching threads) for
    call_reduce and reduce_into, kept on the library object (0: not a native function, e.g. a
    test double - call it the ordinary way)."""
    import ctypes
    try:
        if _config.CUDA_REDUCE_LAUNCH_THREADS and not lib.nbh_launch_threads(1):
            lib._launch_threads = True
            _stop_threads_at_exit(lib)
            return ctypes.cast(lib.nbh_reduce_queued, ctypes.c_void_p).value or 0
        return ctypes.cast(lib.nbh_reduce, ctypes.c_void_p).value or 0
    except (TypeError, ctypes.ArgumentError, AttributeError):
        return 0


def launch_threads(enable=True):
    """Hand the kernel launches of `Reduce(...)(arr, res=..., stream=s)` on streams made with
    `cuda.stream()` to a launching thread per stream (True), or make them on the calling
    thread again (False, the default; `NUMBA_CUDA_REDUCE_LAUNCH_THREADS=1` starts with True).
    Not in the reference.  The runtime's launch path takes 2.4 - 3.0 us per launch on one host
    thread and runs side by side from several, so a loop of small reductions over a few
    streams gets through about twice as fast.  Everything this package does with such a
    stream afterwards (copies, events, synchronize, other kernels) first waits until the
    queued launches are in the stream, so results and ordering are those of the default mode.
    Code outside the package that was handed the stream (`__cuda_array_interface__` consumers,
    external-stream wrappers) cannot know about the queue: `stream.synchronize()` first."""
    import ctypes
    devices.get_context()                    # loads the library on the first call
    lib = _driver.driver.lib
    try:
        entry = lib.nbh_reduce_queued if enable else lib.nbh_reduce
        rc = lib.nbh_launch_threads(1 if enable else 0)
    except AttributeError:
        raise NotImplementedError("this build of the library has no launching threads") from None
    if rc:
        _driver.driver.check("nbh_launch_threads", rc)
    lib._launch_threads = bool(enable)
    if enable:
        _stop_threads_at_exit(lib)
    try:
        lib._reduce_entry = ctypes.cast(entry, ctypes.c_void_p).value or 0
    except (TypeError, ctypes.ArgumentError):
        lib._reduce_entry = 0


def _stop_threads_at_exit(lib):
    """The launching threads must be idle and joined before the interpreter and the GPU runtime
    shut down (exit hooks run in reverse order of registration: this one, registered after the
    library was loaded, runs before the runtime's own)."""
    if getattr(lib, "_stop_hook", False):
        return
    import atexit

    def stop():
        try:
            lib.nbh_launch_threads(-1)
        except Exception:       # noqa: BLE001 - nothing to report to at exit
            pass

    atexit.register(stop)
    lib._stop_hook = True


_DTYPE_CODE = {np.dtype(name): code for name, code in _lib.DTYPE_CODES.items()}
_BOOL = np.dtype(np.bool_)

# host copies of `init` values, one element each, kept alive for the process:
# (dtype, bytes of the value) -> (array, address).  nbh_reduce reads the value during the call.
_INIT_CACHE = {}


# (dtype, int value) -> address: the common case (`init=0`) without building an array first
_INT_INIT = {}


def _init_buffer(dtype, init):
    """Address of a host copy of `init` converted to `dtype`.  The copies are kept for
    the life of the process, found again by the bit pattern of the converted value
    (so that 0.0 and -0.0, which compare equal, stay apart)."""
    buf = np.array([dtype.type(init)], dtype=dtype)
    key = (dtype, buf.tobytes())
    kept = _INIT_CACHE.get(key)
    if kept is None:
        if len(_INIT_CACHE) < 4096:
            kept = _INIT_CACHE[key] = (buf, buf.ctypes.data)
        else:
            _KEEPALIVE.append(buf)
            if len(_KEEPALIVE) > 64:
                del _KEEPALIVE[:32]
            return buf.ctypes.data
    if init.__class__ is int and len(_INT_INIT) < 4096:
        _INT_INIT[dtype, init] = kept[1]
    return kept[1]


_KEEPALIVE = []


reduce = Reduce

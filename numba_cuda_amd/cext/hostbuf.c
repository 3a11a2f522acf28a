/* _hostbuf: the two pieces of host-side plumbing that need the CPython C API.
 *
 *   HostBuffer   base class for Python objects that stand for a run of host memory
 *                (page-locked, device-mapped or managed allocations).  A subclass
 *                instance says where its bytes are through two attributes, `_bufptr_`
 *                (address) and `_buflen_` (length), and is then usable wherever the
 *                buffer protocol is: np.ndarray(..., buffer=mem), memoryview(mem).
 *                The exported buffer keeps the instance alive.
 *   address(obj, writable)  address of the first byte of any buffer-protocol object
 *   extents(obj)            half-open byte range [lo, hi) its items occupy, strides of
 *                           either sign, empty when any extent is zero
 *   extents_of(shape, strides, itemsize)  the same from a description, relative to 0
 *   reduce_into(codes, arr, res, init, stream, ...)  Reduce.__call__ with `res=` for the plain
 *                           case, from the array objects to the launch (described at the function)
 *   call_reduce(entry, op, dtype, in, n, stride, init, out, scratch, scratch_bytes, stream)
 *                           calls the library's nbh_reduce through its address, all
 *                           arguments plain integers: the launch path of Reduce.__call__
 *                           without the per-argument conversions of a ctypes call
 *
 * Counterpart of numba_cuda/numba/cuda/cext/mviewbuf.c:48-70 (address), :76-135 and
 * :138-209 (extents), :212-363 (the buffer-exporting type).
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

/* ---- byte range of a strided block ------------------------------------------------ */

static void span(const Py_ssize_t *shape, const Py_ssize_t *strides, int ndim, Py_ssize_t itemsize,
                 Py_ssize_t origin, Py_ssize_t *lo_out, Py_ssize_t *hi_out)
{
    Py_ssize_t lo = origin, hi = origin;
    for (int k = 0; k < ndim; ++k) {
        if (shape[k] == 0) { /* no items at all */
            *lo_out = *hi_out = origin;
            return;
        }
        const Py_ssize_t reach = strides[k] * (shape[k] - 1);
        if (reach > 0)
            hi += reach;
        else
            lo += reach;
    }
    *lo_out = lo;
    *hi_out = hi + itemsize;
}

static int attr_as_ssize(PyObject *obj, const char *name, Py_ssize_t *out)
{
    PyObject *v = PyObject_GetAttrString(obj, name);
    if (!v)
        return -1;
    /* addresses above 2^63 do not occur in user space; accept any integer-like object */
    PyObject *as_int = PyNumber_Index(v);
    Py_DECREF(v);
    if (!as_int)
        return -1;
    *out = (Py_ssize_t)PyLong_AsUnsignedLongLongMask(as_int);
    Py_DECREF(as_int);
    return PyErr_Occurred() ? -1 : 0;
}

/* ---- HostBuffer ------------------------------------------------------------------------ */

static int hostbuffer_getbuffer(PyObject *self, Py_buffer *view, int flags)
{
    Py_ssize_t ptr = 0, len = 0;
    if (attr_as_ssize(self, "_bufptr_", &ptr) || attr_as_ssize(self, "_buflen_", &len))
        return -1;
    if (len < 0 || (len > 0 && ptr == 0)) {
        PyErr_SetString(PyExc_BufferError, "HostBuffer: _bufptr_ / _buflen_ do not describe memory");
        return -1;
    }
    /* one-dimensional, writable bytes; FillInfo takes the reference that keeps self alive */
    return PyBuffer_FillInfo(view, self, (void *)ptr, len, 0, flags);
}

static PyBufferProcs hostbuffer_as_buffer = {.bf_getbuffer = hostbuffer_getbuffer, .bf_releasebuffer = NULL};

static PyTypeObject HostBufferType = {
    PyVarObject_HEAD_INIT(NULL, 0)
    .tp_name = "numba_cuda_amd._hostbuf.HostBuffer",
    .tp_basicsize = sizeof(PyObject),
    .tp_flags = Py_TPFLAGS_DEFAULT | Py_TPFLAGS_BASETYPE,
    .tp_doc = "Base class: exports [_bufptr_, _bufptr_ + _buflen_) through the buffer protocol.",
    .tp_as_buffer = &hostbuffer_as_buffer,
    .tp_new = PyType_GenericNew,
};

/* ---- module functions ------------------------------------------------------------------- */

static PyObject *hb_address(PyObject *mod, PyObject *args)
{
    PyObject *obj;
    int writable = 1;
    if (!PyArg_ParseTuple(args, "O|p", &obj, &writable))
        return NULL;
    Py_buffer b;
    if (PyObject_GetBuffer(obj, &b, writable ? PyBUF_WRITABLE | PyBUF_RECORDS : PyBUF_RECORDS_RO) < 0)
        return NULL;
    PyObject *ret = PyLong_FromVoidPtr(b.buf);
    PyBuffer_Release(&b);
    return ret;
}

static PyObject *hb_extents(PyObject *mod, PyObject *obj)
{
    Py_buffer b;
    if (PyObject_GetBuffer(obj, &b, PyBUF_RECORDS_RO) < 0)
        return NULL;
    Py_ssize_t lo, hi;
    if (b.ndim == 0 || !b.shape) {
        lo = (Py_ssize_t)b.buf;
        hi = lo + (b.ndim == 0 ? b.itemsize : b.len);
    } else if (!b.strides) {
        PyBuffer_Release(&b);
        PyErr_SetString(PyExc_ValueError, "buffer strides is not defined");
        return NULL;
    } else {
        span(b.shape, b.strides, b.ndim, b.itemsize, (Py_ssize_t)b.buf, &lo, &hi);
    }
    PyBuffer_Release(&b);
    return Py_BuildValue("nn", lo, hi);
}

static int fill_from_sequence(PyObject *seq, Py_ssize_t *dst, Py_ssize_t n, const char *what)
{
    PyObject *fast = PySequence_Fast(seq, what);
    if (!fast)
        return -1;
    if (PySequence_Fast_GET_SIZE(fast) != n) {
        Py_DECREF(fast);
        PyErr_SetString(PyExc_ValueError, "shape and strides differ in length");
        return -1;
    }
    for (Py_ssize_t k = 0; k < n; ++k) {
        dst[k] = PyNumber_AsSsize_t(PySequence_Fast_GET_ITEM(fast, k), PyExc_OverflowError);
        if (dst[k] == -1 && PyErr_Occurred()) {
            Py_DECREF(fast);
            return -1;
        }
    }
    Py_DECREF(fast);
    return 0;
}

static PyObject *hb_extents_of(PyObject *mod, PyObject *args)
{
    PyObject *shape, *strides;
    Py_ssize_t itemsize;
    if (!PyArg_ParseTuple(args, "OOn", &shape, &strides, &itemsize))
        return NULL;
    if (itemsize <= 0) {
        PyErr_SetString(PyExc_ValueError, "itemsize must be positive");
        return NULL;
    }
    const Py_ssize_t n = PySequence_Size(shape);
    if (n < 0)
        return NULL;
    enum { kMaxDims = 64 };
    if (n > kMaxDims) {
        PyErr_SetString(PyExc_ValueError, "too many dimensions");
        return NULL;
    }
    Py_ssize_t dims[kMaxDims], steps[kMaxDims];
    if (fill_from_sequence(shape, dims, n, "shape is not a sequence") ||
        fill_from_sequence(strides, steps, n, "strides is not a sequence"))
        return NULL;
    Py_ssize_t lo, hi;
    span(dims, steps, (int)n, itemsize, 0, &lo, &hi);
    return Py_BuildValue("nn", lo, hi);
}

/* ---- the reduction launch, called thousands of times a second ------------------------ */

typedef int (*nbh_reduce_fn)(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init,
                             void *out, void *scratch, size_t scratch_bytes, void *stream);

static int as_word(PyObject *o, unsigned long long *out)
{
    /* addresses and sizes arrive as non-negative Python ints, None stands for 0 */
    if (o == Py_None) {
        *out = 0;
        return 0;
    }
    unsigned long long v = PyLong_AsUnsignedLongLong(o);
    if (v == (unsigned long long)-1 && PyErr_Occurred())
        return -1;
    *out = v;
    return 0;
}

static PyObject *hb_call_reduce(PyObject *mod, PyObject *const *args, Py_ssize_t nargs)
{
    if (nargs != 11) {
        PyErr_SetString(PyExc_TypeError, "call_reduce takes 11 arguments");
        return NULL;
    }
    unsigned long long entry, in, init, out, scratch, scratch_bytes, stream;
    if (as_word(args[0], &entry) || as_word(args[3], &in) || as_word(args[6], &init) || as_word(args[7], &out) ||
        as_word(args[8], &scratch) || as_word(args[9], &scratch_bytes) || as_word(args[10], &stream))
        return NULL;
    const long op = PyLong_AsLong(args[1]), dtype = PyLong_AsLong(args[2]);
    const long long n = PyLong_AsLongLong(args[4]), stride = PyLong_AsLongLong(args[5]);
    if (PyErr_Occurred())
        return NULL;
    if (!entry) {
        PyErr_SetString(PyExc_ValueError, "call_reduce: null entry point");
        return NULL;
    }
    int status;
    Py_BEGIN_ALLOW_THREADS
    status = ((nbh_reduce_fn)(uintptr_t)entry)((int)op, (int)dtype, (const void *)(uintptr_t)in, (int64_t)n,
                                               (int64_t)stride, (const void *)(uintptr_t)init,
                                               (void *)(uintptr_t)out, (void *)(uintptr_t)scratch,
                                               (size_t)scratch_bytes, (void *)(uintptr_t)stream);
    Py_END_ALLOW_THREADS
    return PyLong_FromLong(status);
}

/* reduce_into(codes, arr, res, init, stream, thread_state, stream_type, init_cache, lib)
 *
 * The whole of Reduce.__call__(arr, res=res, init=init, stream=stream) for the plain case, so
 * that a small reduction costs the host little more than the launch itself: both arrays carry
 * a cached description `_rk` = (address, items, stride in bytes, dtype) that the Python path
 * stores on its first visit, `codes` maps the dtype to (operator code, element code), the
 * calling thread's context holds the scratch buffer per stream handle, `init_cache` maps
 * (dtype, int) to the address of the converted initial value, `lib` is the loaded library
 * object with the address of nbh_reduce in `_reduce_entry`.  Anything out of the ordinary -
 * no description yet, dtypes that are not the same object, an empty array, a stream that is
 * not a Stream of ours, the per-thread default stream, no scratch buffer yet, an initial value
 * that is not a cached int - returns NotImplemented and the Python path does the call (and
 * raises what there is to raise).  Returns None after a launch, or the error status as int. */
static PyObject *str_rk, *str_handle, *str_ctx, *str_prepared, *str_scratch, *str_entry;

static PyObject *hb_reduce_into(PyObject *mod, PyObject *const *args, Py_ssize_t nargs)
{
    if (nargs != 9) {
        PyErr_SetString(PyExc_TypeError, "reduce_into takes 9 arguments");
        return NULL;
    }
    PyObject *codes = args[0], *arr = args[1], *res = args[2], *init = args[3], *stream = args[4];
    PyObject *tls = args[5], *stream_type = args[6], *init_cache = args[7];
    PyObject *rk = NULL, *rr = NULL, *handle = NULL, *ctx = NULL, *flag = NULL, *table = NULL, *key = NULL;
    PyObject *entry_obj = NULL;
    PyObject *result = NULL;  /* NULL at `out` without an exception set: NotImplemented */

    if (!PyDict_CheckExact(codes) || !PyDict_CheckExact(init_cache) || !PyLong_CheckExact(init) ||
        (PyObject *)Py_TYPE(stream) != stream_type)
        goto out;
    rk = PyObject_GetAttr(arr, str_rk);
    if (!rk)
        goto out;
    rr = PyObject_GetAttr(res, str_rk);
    if (!rr)
        goto out;
    if (!PyTuple_CheckExact(rk) || PyTuple_GET_SIZE(rk) != 4 || !PyTuple_CheckExact(rr) || PyTuple_GET_SIZE(rr) != 4)
        goto out;
    PyObject *dtype = PyTuple_GET_ITEM(rk, 3);
    if (PyTuple_GET_ITEM(rr, 3) != dtype)
        goto out;
    PyObject *pair = PyDict_GetItemWithError(codes, dtype);  /* borrowed */
    if (!pair || !PyTuple_CheckExact(pair) || PyTuple_GET_SIZE(pair) != 2)
        goto out;
    handle = PyObject_GetAttr(stream, str_handle);
    if (!handle || !PyLong_CheckExact(handle))
        goto out;
    ctx = PyObject_GetAttr(tls, str_ctx);
    if (!ctx || ctx == Py_None)
        goto out;
    flag = PyObject_GetAttr(ctx, str_prepared);
    if (flag != Py_True)
        goto out;
    table = PyObject_GetAttr(ctx, str_scratch);
    if (!table || !PyDict_CheckExact(table))
        goto out;
    PyObject *scratch = PyDict_GetItemWithError(table, handle);  /* borrowed */
    if (!scratch || !PyTuple_CheckExact(scratch) || PyTuple_GET_SIZE(scratch) < 2)
        goto out;
    key = PyTuple_Pack(2, dtype, init);
    if (!key)
        goto out;
    PyObject *init_addr = PyDict_GetItemWithError(init_cache, key);  /* borrowed */
    if (!init_addr)
        goto out;
    {
        unsigned long long entry, in, init_ptr, dst, scr, scr_bytes, hstream;
        entry_obj = PyObject_GetAttr(args[8], str_entry);
        if (!entry_obj)
            goto out;
        if (as_word(entry_obj, &entry) || as_word(PyTuple_GET_ITEM(rk, 0), &in) || as_word(init_addr, &init_ptr) ||
            as_word(PyTuple_GET_ITEM(rr, 0), &dst) || as_word(PyTuple_GET_ITEM(scratch, 0), &scr) ||
            as_word(PyTuple_GET_ITEM(scratch, 1), &scr_bytes) || as_word(handle, &hstream))
            goto out;
        const long op = PyLong_AsLong(PyTuple_GET_ITEM(pair, 0)), code = PyLong_AsLong(PyTuple_GET_ITEM(pair, 1));
        const long long n = PyLong_AsLongLong(PyTuple_GET_ITEM(rk, 1));
        const long long stride = PyLong_AsLongLong(PyTuple_GET_ITEM(rk, 2));
        const long long room = PyLong_AsLongLong(PyTuple_GET_ITEM(rr, 1));
        /* the per-thread default stream keeps its scratch per host thread: Python's business */
        if (PyErr_Occurred() || !entry || n < 1 || room < 1 || hstream == 2)
            goto out;
        int status;
        Py_BEGIN_ALLOW_THREADS
        status = ((nbh_reduce_fn)(uintptr_t)entry)((int)op, (int)code, (const void *)(uintptr_t)in, (int64_t)n,
                                                   (int64_t)stride, (const void *)(uintptr_t)init_ptr,
                                                   (void *)(uintptr_t)dst, (void *)(uintptr_t)scr, (size_t)scr_bytes,
                                                   (void *)(uintptr_t)hstream);
        Py_END_ALLOW_THREADS
        if (status == 0) {
            result = Py_None;
            Py_INCREF(result);
        } else {
            result = PyLong_FromLong(status);
        }
    }
out:
    Py_XDECREF(rk);
    Py_XDECREF(rr);
    Py_XDECREF(handle);
    Py_XDECREF(ctx);
    Py_XDECREF(flag);
    Py_XDECREF(table);
    Py_XDECREF(key);
    Py_XDECREF(entry_obj);
    if (result)
        return result;
    PyErr_Clear();  /* a missing attribute or the like: the Python path will say what is wrong */
    Py_RETURN_NOTIMPLEMENTED;
}

static PyMethodDef hb_methods[] = {
    {"reduce_into", (PyCFunction)(void (*)(void))hb_reduce_into, METH_FASTCALL,
     "reduce_into(codes, arr, res, init, stream, thread_state, stream_type, init_cache, lib) -> None | status | NotImplemented"},
    {"call_reduce", (PyCFunction)(void (*)(void))hb_call_reduce, METH_FASTCALL,
     "call_reduce(entry, op, dtype, in, n, stride, init, out, scratch, scratch_bytes, stream) -> status"},
    {"address", hb_address, METH_VARARGS, "address(obj, writable=True) -> int"},
    {"extents", hb_extents, METH_O, "extents(obj) -> (lo, hi)"},
    {"extents_of", hb_extents_of, METH_VARARGS, "extents_of(shape, strides, itemsize) -> (lo, hi)"},
    {NULL, NULL, 0, NULL},
};

static struct PyModuleDef hb_module = {
    PyModuleDef_HEAD_INIT, .m_name = "_hostbuf", .m_doc = NULL, .m_size = -1, .m_methods = hb_methods,
};

PyMODINIT_FUNC PyInit__hostbuf(void)
{
    if (PyType_Ready(&HostBufferType) < 0)
        return NULL;
    PyObject *m = PyModule_Create(&hb_module);
    if (!m)
        return NULL;
    str_rk = PyUnicode_InternFromString("_rk");
    str_handle = PyUnicode_InternFromString("_h");
    str_ctx = PyUnicode_InternFromString("ctx");
    str_prepared = PyUnicode_InternFromString("prepared");
    str_scratch = PyUnicode_InternFromString("_scratch");
    str_entry = PyUnicode_InternFromString("_reduce_entry");
    if (!str_rk || !str_handle || !str_ctx || !str_prepared || !str_scratch || !str_entry) {
        Py_DECREF(m);
        return NULL;
    }
    Py_INCREF(&HostBufferType);
    if (PyModule_AddObject(m, "HostBuffer", (PyObject *)&HostBufferType) < 0) {
        Py_DECREF(&HostBufferType);
        Py_DECREF(m);
        return NULL;
    }
    return m;
}

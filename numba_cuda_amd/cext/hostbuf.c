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

static PyMethodDef hb_methods[] = {
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
    Py_INCREF(&HostBufferType);
    if (PyModule_AddObject(m, "HostBuffer", (PyObject *)&HostBufferType) < 0) {
        Py_DECREF(&HostBufferType);
        Py_DECREF(m);
        return NULL;
    }
    return m;
}

/*
 * nbhip.h - C ABI of libnbhip.so: the MI355X (gfx950) back end of the numba-cuda
 * data-parallel array library (reduce / transpose / xoroshiro128+ and the device
 * memory, stream and event plumbing underneath them).
 *
 * The reference has no C boundary for this path: its Python layer reaches the
 * CUDA driver through cuda.bindings and JIT-compiles its kernels.  Each entry
 * point below names the reference interface it stands in for; paths are relative
 * to numba_cuda/numba/cuda/ in NVIDIA/numba-cuda 0.30.4.
 *
 * Conventions
 *   - every function returns a hipError_t as int; 0 is success; nothing throws
 *   - all pointers are plain host or device addresses, sizes are in bytes unless
 *     stated otherwise, strides are in bytes and may be negative
 *   - nbh_stream_t is a hipStream_t; NULL is the legacy default stream
 *   - the library never frees or reallocates caller memory; lifetimes of buffers
 *     passed to asynchronous calls are the caller's to keep
 *   - functions are re-entrant; the current device is per host thread
 */
#ifndef NBHIP_H
#define NBHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *nbh_stream_t;
typedef void *nbh_event_t;

#define NBH_VERSION 1

/* element types understood by nbh_reduce */
enum nbh_dtype {
    NBH_I8 = 0, NBH_I16 = 1, NBH_I32 = 2, NBH_I64 = 3,
    NBH_U8 = 4, NBH_U16 = 5, NBH_U32 = 6, NBH_U64 = 7,
    NBH_F32 = 8, NBH_F64 = 9,
    NBH_C64 = 10, NBH_C128 = 11,   /* complex: pairs (re, im) of float32 / float64; ADD and MUL only */
    NBH_F16 = 12,                  /* IEEE binary16; accumulated in binary16, one rounding per operation */
    NBH_DTYPE_COUNT = 13
};

/* binary operators understood by nbh_reduce.  Semantics are those the reference's
 * JIT gives the Python functor (cpython/builtins.py:224-269):
 *   ADD a + b, MUL a * b      native arithmetic, integers wrap modulo 2^bits; complex
 *                             products are (ac - bd) + (ad + bc)i, each operation rounded
 *   MAX b if b > a else a,  MIN b if b < a else a
 *   AND a & b, OR a | b, XOR a ^ b     integer element types only */
enum nbh_op { NBH_ADD = 0, NBH_MUL = 1, NBH_MAX = 2, NBH_MIN = 3, NBH_AND = 4, NBH_OR = 5, NBH_XOR = 6,
              NBH_OP_COUNT = 7 };

/* ---- library / device ---------------------------------------------------- */

int nbh_version(void);
/* cudadrv/driver.py:410-418 Driver.get_version, cudadrv/runtime.py:15-24 Runtime.get_version:
 * the versions of the HIP driver and runtime as HIP encodes them, major * 10 000 000 +
 * minor * 100 000 + patch.  Needs no device. */
int nbh_hip_versions(int *driver_version, int *runtime_version);

/* cudadrv/driver.py:245-419 Driver (error checking): name / text of an error code */
const char *nbh_error_name(int code);
const char *nbh_error_string(int code);

/* cudadrv/driver.py:385-388 get_device_count */
int nbh_device_count(int *count);
/* cudadrv/devices.py:101-187 _Runtime (per-thread current context) */
int nbh_set_device(int dev);
int nbh_get_device(int *dev);
/* cudadrv/driver.py:470-587 Device: name, attributes looked up by the CUDA
 * attribute name without its CU_DEVICE_ATTRIBUTE_ prefix (:509-517), e.g.
 * "MAX_THREADS_PER_BLOCK", "MULTIPROCESSOR_COUNT", "WARP_SIZE".  Unknown names
 * return hipErrorInvalidValue. */
int nbh_device_name(int dev, char *buf, int buflen);
int nbh_device_attr(int dev, const char *name, int *value);
/* cudadrv/driver.py:1095-1097 Context.get_memory_info */
int nbh_mem_info(size_t *free_bytes, size_t *total_bytes);
/* cudadrv/driver.py:1282-1283 Context.synchronize */
int nbh_device_synchronize(void);

/* ---- memory --------------------------------------------------------------- */

/* cudadrv/driver.py:891-902 NumbaCUDAMemoryManager.memalloc (cuMemAlloc) and the
 * cuMemFree its finalizer queues (:1316-1325) */
int nbh_malloc(void **dptr, size_t nbytes);
int nbh_free(void *dptr);
/* cudadrv/driver.py:819-838 memallocmanaged (cuMemAllocManaged): memory addressable
 * from the host and the device at the same address; attach_global != 0 ->
 * attached to every stream, 0 -> host-attached.  Release with nbh_free. */
int nbh_malloc_managed(void **ptr, size_t nbytes, int attach_global);
/* A caching allocator behind the external-memory-manager interface
 * (cudadrv/driver.py:592-703 BaseCUDAMemoryManager; the reference ships none and
 * points to RMM's pool for this): nbh_pool_malloc hands out a block of the current
 * device, nbh_pool_free takes it back WITHOUT freeing it.  A block is handed out again
 * only after the work that had been submitted, through this library, to any stream
 * before the free has completed (events, no host-side wait).  nbh_pool_trim returns
 * every idle block to the driver; nbh_pool_stats reports bytes idle / handed out and
 * how many requests were served from the pool (hits) or by hipMalloc (misses). */
int nbh_pool_malloc(void **dptr, size_t nbytes);
int nbh_pool_free(void *dptr);
int nbh_pool_trim(void);
int nbh_pool_stats(size_t *idle_bytes, size_t *live_bytes, uint64_t *hits, uint64_t *misses);
/* cudadrv/driver.py:747-779 memhostalloc (cuMemHostAlloc / cuMemFreeHost).
 * flags: bit 0 portable, bit 1 device-mapped, bit 2 write-combined */
int nbh_host_alloc(void **hptr, size_t nbytes, unsigned flags);
int nbh_host_free(void *hptr);
/* cudadrv/driver.py:781-817 mempin (cuMemHostRegister / cuMemHostUnregister) */
int nbh_host_register(void *hptr, size_t nbytes, unsigned flags);
int nbh_host_unregister(void *hptr);
/* cudadrv/driver.py:1735-1770 MappedMemory (cuMemHostGetDevicePointer) */
int nbh_host_get_device_pointer(void **dptr, void *hptr);
/* cudadrv/driver.py:2496-2506 device_extents (cuMemGetAddressRange) */
int nbh_mem_address_range(void **base, size_t *size, void *dptr);

/* cudadrv/driver.py:861-878 GetIpcHandleMixin.get_ipc_handle (cuIpcGetMemHandle),
 * :1408-1440 _CudaIpcImpl.open / close (cuIpcOpenMemHandle / cuIpcCloseMemHandle).
 * `handle` is NBH_IPC_HANDLE_BYTES opaque bytes, valid in other processes on the same
 * machine; `dptr` must be the start of an allocation.  nbh_ipc_open takes the number
 * of bytes the importer will use.  Allocations of 2 GiB or more are refused
 * (hipErrorNotSupported). */
#define NBH_IPC_HANDLE_BYTES 64
int nbh_ipc_get_handle(void *handle, void *dptr);
int nbh_ipc_open(void **dptr, const void *handle, size_t nbytes);
int nbh_ipc_close(void *dptr);

/* cudadrv/driver.py:2625-2670 host_to_device / device_to_host / device_to_device:
 * stream == NULL selects the synchronous copy, any other stream the asynchronous
 * one, exactly as the reference picks cuMemcpyXtoY vs cuMemcpyXtoYAsync */
int nbh_memcpy_h2d(void *dst, const void *src, size_t nbytes, nbh_stream_t stream);
int nbh_memcpy_d2h(void *dst, const void *src, size_t nbytes, nbh_stream_t stream);
int nbh_memcpy_d2d(void *dst, const void *src, size_t nbytes, nbh_stream_t stream);
/* cudadrv/driver.py:2673-2704 device_memset (cuMemsetD8 / cuMemsetD8Async) */
int nbh_memset8(void *dst, int byte, size_t nbytes, nbh_stream_t stream);

/* ---- streams and events --------------------------------------------------- */

/* cudadrv/driver.py:1244-1271 Context.create_stream (default flags: the stream
 * synchronises with the legacy default stream), :1890-2017 Stream */
int nbh_stream_create(nbh_stream_t *stream);
int nbh_stream_destroy(nbh_stream_t stream);
int nbh_stream_synchronize(nbh_stream_t stream);
int nbh_stream_query(nbh_stream_t stream);
/* cudadrv/driver.py:1937-1973 Stream.add_callback (cuStreamAddCallback): `fn(user)`
 * runs on a runtime thread once all work queued on `stream` so far has finished.
 * No library call may be made from inside `fn`. */
typedef void (*nbh_host_fn)(void *user);
int nbh_stream_add_callback(nbh_stream_t stream, nbh_host_fn fn, void *user);
/* cudadrv/driver.py:1273-1280 Context.create_event, :2037-2095 Event */
int nbh_event_create(nbh_event_t *event, int timing);
int nbh_event_destroy(nbh_event_t event);
int nbh_event_record(nbh_event_t event, nbh_stream_t stream);
int nbh_event_synchronize(nbh_event_t event);
int nbh_event_query(nbh_event_t event);
int nbh_stream_wait_event(nbh_stream_t stream, nbh_event_t event);
int nbh_event_elapsed_ms(float *ms, nbh_event_t start, nbh_event_t stop);

/* ---- reduction ------------------------------------------------------------ */

/* Size of the scratch buffer nbh_reduce needs.  The caller allocates it in device
 * memory, clears it to zero ONCE, and may then reuse it for any number of calls
 * that do not overlap in time (one buffer per stream).  The library leaves it in
 * the cleared state after every call. */
size_t nbh_reduce_scratch_bytes(void);

/* kernels/reduction.py:194-265 Reduce.__call__ together with the kernels it
 * launches (:15-166).  Computes
 *     out[0] = init (op) in[0] (op) in[1] (op) ... (op) in[n-1]
 * for n >= 1 elements of `dtype` in device memory, `in_stride` bytes apart (a
 * multiple of the element size, any sign; the element size itself selects the
 * 128-bit streaming path), in one launch and fully asynchronously on `stream`.
 * `init` points to one element of `dtype` in HOST memory (read before the call
 * returns); `out` is one element in DEVICE memory (what `res[:1]` is in the
 * reference).  The association order differs from the reference's (integer
 * results are identical; floating-point sums agree within rounding,
 * |err| <= 2 n eps sum|x|), and is the same on every run. */
int nbh_reduce(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
               void *scratch, size_t scratch_bytes, nbh_stream_t stream);

/* The same reduction with the reference's association, operation for operation:
 * kernels/reduction.py:194-265 Reduce.__call__ launching gpu_reduce_block_strided (:143-166:
 * device_reduce_full_block :43-97, inner_warp_reduction :22-41, device_reduce_partial_block
 * :99-141) over the full blocks, the remainder and the partials.  For float16, float32,
 * float64 and the complex types the result has the bits a run of the reference's kernels
 * produces (sums and products round in the same places; max / min treat NaN and signed zeros
 * alike); integers and booleans go to nbh_reduce, whose result is the same in any order.
 * Arguments, scratch buffer and asynchrony as for nbh_reduce; one launch. */
int nbh_reduce_ordered(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                       void *scratch, size_t scratch_bytes, nbh_stream_t stream);

/* Launching threads for loops of small reductions (no counterpart in the reference, whose
 * Reduce.__call__ pays a kernel launch and an allocation on the calling thread,
 * kernels/reduction.py:242-258).  The runtime's launch path costs 2.4 - 3.0 us per launch on
 * one host thread and runs side by side from several.  After nbh_launch_threads(1),
 * nbh_reduce_queued - same arguments and result as nbh_reduce; `init` is copied before the
 * call returns - hands the launch to a thread that belongs to `stream` (made on first use,
 * one per stream: the launches of a stream keep the order of the calls) and returns 0.
 *   - Every entry point of this library that is given that stream first waits until its
 *     queue has been launched; entry points that concern the whole device (a default stream,
 *     synchronous copies, nbh_free, nbh_pool_free, nbh_device_synchronize ...) wait for all
 *     queues.  Code OUTSIDE the library that was handed the stream does not: call
 *     nbh_stream_synchronize first.  That is why the mode is off unless asked for.
 *   - A launch that fails on the launching thread is reported by the next
 *     nbh_stream_synchronize of the stream.
 *   - The default streams (0, legacy, per-thread), and every call while the mode is off, go
 *     straight to nbh_reduce.  nbh_launch_threads(0) waits for all queues and switches the
 *     mode off; the threads sleep until their streams are destroyed.  nbh_launch_threads(-1)
 *     does the same and then joins every thread: for the end of a process, before the GPU
 *     runtime's own exit handlers run.  A forked child starts with the mode off and no queues.
 *   - nbh_launch_threads_wait(stream) waits until what has been queued for `stream` (0: for
 *     every stream) is in its stream, without waiting for the device.
 *   - nbh_stream_pin_direct(stream): the stream's handle is about to be used by code outside
 *     the library.  What is queued for it is launched, and from then on its reductions are
 *     launched on the calling thread whatever the mode (until the stream is destroyed). */
int nbh_launch_threads(int enable);
int nbh_launch_threads_wait(nbh_stream_t stream);
int nbh_stream_pin_direct(nbh_stream_t stream);
int nbh_reduce_queued(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                      void *scratch, size_t scratch_bytes, nbh_stream_t stream);

/* nbh_reduce for callers that cannot allocate device memory: code under stream (graph)
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference (whose Reduce.__call__ allocates its partials on every call,
 * kernels/reduction.py:242).  Same arguments, kernels and results as nbh_reduce, minus
 * the scratch buffer: ticket and partials live in a 33 KiB array that is part of the
 * library's code object, one copy per device, held until the process ends.  The call
 * makes no hipMalloc / hipFree / hipHostMalloc and no allocating library call (host side:
 * one map node the first time a stream is seen while the pooling manager is in use).
 * The address of the array is looked up on the first call on each device: make that call
 * outside stream capture.
 *   - n above NBH_REDUCE_NOALLOC_MAX_ITEMS is refused with hipErrorInvalidValue before
 *     anything is launched
 *   - every call on a device shares that device's array: calls that overlap in time would
 *     race.  A call on another stream than the previous call's, made while that call's
 *     kernel has not finished, is refused with hipErrorNotReady (an event query, no wait);
 *     calls on one stream, and calls involving the null stream, are ordered by the stream.
 *     Under stream capture the check is left out (nothing runs then): replays of graphs
 *     that hold such calls must not overlap.  Callers that need overlap bring one scratch
 *     buffer per stream to nbh_reduce instead
 *   - a call that fails after its launch marks the array; the next call clears the ticket
 *     with a one-workgroup kernel on its stream before it starts
 *   - the array starts zeroed and each call leaves its ticket at zero again; the partials
 *     keep the last call's values and are overwritten before they are read */
#define NBH_REDUCE_NOALLOC_MAX_ITEMS ((int64_t)1 << 36)
int nbh_reduce_noalloc(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init,
                       void *out, nbh_stream_t stream);

/* Reductions with a binary operation supplied as source text.  Stands where the
 * reference's JIT compiles an arbitrary Python functor for the reduction kernels
 * (kernels/reduction.py:15-20, :175-192 Reduce._compile).
 *
 * nbh_reduce_compile builds, with the HIP run-time compiler (libhiprtc.so, loaded on
 * first use), the kernels for
 *     __device__ T nbh_op(T a, T b) { <body> }
 * where T is the C type of `dtype` (NBH_I8 .. NBH_F64, NBH_F16; NBH_C64 / NBH_C128 as
 * nbh_c64 / nbh_c128, structs {re, im} of float / double) and `body` is C++ that returns
 * the combined value.  Available to the body: the HIP device math functions, nbh_i64 /
 * nbh_u64 (64-bit integer types), nbh_floordiv(x, y) and nbh_mod(x, y) with Python's
 * rounding for nbh_i64, nbh_u64, float and double, nbh_ipow(x, e), and for the complex
 * types + - * / == != as the reference's JIT lowers them (numba/cuda/cpython/numbers.py:
 * 1091-1221), nbh_cabs(z), nbh_conj(z) and nbh_cplx_from<float | double>(x) for conversions.  Needs no device.  On failure the compiler's messages are in `log`
 * (NUL-terminated, cut to log_bytes) and the result is hipErrorInvalidSource (300), or
 * hipErrorSharedObjectInitFailed (303) when the compiler library is absent.
 * `*op` stays valid until nbh_reduce_op_free(op); it may be used from any thread and on
 * any device (each device loads its module at its first call). */
int nbh_reduce_compile(int dtype, const char *body, void **op, char *log, size_t log_bytes);
int nbh_reduce_op_dtype(const void *op);
int nbh_reduce_op_free(void *op);

/* out[0] = nbh_op(... nbh_op(nbh_op(in[0], in[1]), in[2]) ..., init) in SOME order of
 * association: every element and `init` enter exactly once, n applications for n
 * elements, so the result equals the reference's (kernels/reduction.py:194-265) for every
 * operation that is associative and commutative - the same condition the reference's own
 * tree imposes.  Arguments as for nbh_reduce (`scratch` is the same buffer, used the same
 * way: the ticket is handed back at zero).  One launch on `stream`, fully asynchronous. */
int nbh_reduce_custom(void *op, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                      void *scratch, size_t scratch_bytes, nbh_stream_t stream);

/* The same reduction with every application of nbh_op on the same pair of values, in the
 * same order, as a run of the reference's kernels (kernels/reduction.py:22-166 launched as
 * in :233-258): the result then has the reference's bits also for operations that are not
 * associative or whose rounding depends on the order.  Same arguments, one launch. */
int nbh_reduce_custom_ordered(void *op, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                              void *scratch, size_t scratch_bytes, nbh_stream_t stream);

/* ---- transpose ------------------------------------------------------------ */

/* kernels/transpose.py:10-65 transpose(a, b): out[j, i] = in[i, j] for a
 * rows x cols input of items of `itemsize` bytes; all four strides are in bytes
 * and arbitrary (views), any itemsize >= 1 (records).  The input and output
 * regions must not overlap. */
int nbh_transpose(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_stride0,
                  int64_t in_stride1, int64_t out_stride0, int64_t out_stride1, int64_t itemsize,
                  nbh_stream_t stream);

/* ---- strided assignment ---------------------------------------------------- */

#define NBH_ASSIGN_MAX_NDIM 8

/* cudadrv/devicearray.py:534-575 _assign_kernel and :741-790 _do_setitem (the
 * device side of `darr[key] = value`): dst[i0..ik] = src[i0..ik] for every index
 * of `shape` (ndim <= NBH_ASSIGN_MAX_NDIM), items of `itemsize` bytes, byte
 * strides arbitrary on both sides; a source stride of 0 broadcasts that axis.
 * Contiguous-to-contiguous assignments run as a flat 128-bit copy.  Source and
 * destination must not overlap. */
int nbh_assign(void *dst, const void *src, int ndim, const int64_t *shape, const int64_t *dst_strides,
               const int64_t *src_strides, int64_t itemsize, nbh_stream_t stream);
/* The same assignment with ONE item as the right-hand side, passed by value (`value`
 * points to `itemsize` bytes in HOST memory, read before the call returns; itemsize 1,
 * 2, 4, 8 or 16): `darr[key] = scalar` without a device-side source. */
int nbh_fill(void *dst, int ndim, const int64_t *shape, const int64_t *dst_strides, int64_t itemsize,
             const void *value, nbh_stream_t stream);

/* ---- xoroshiro128+ -------------------------------------------------------- */

/* random.py:241-282 init_xoroshiro128p_states (the sequential CPU jump chain plus
 * the host-to-device copy): states[i] = jump^(subsequence_start + i)(seed state),
 * computed on the device.  `states` is n records {uint64 s0; uint64 s1} (:47-50). */
int nbh_xoro_init_states(void *states, int64_t n, uint64_t seed, uint64_t subsequence_start,
                         nbh_stream_t stream);

/* random.py:159-238 xoroshiro128p_{uniform,normal}_float{32,64} applied in bulk
 * with the layout of the reference's test kernels (tests/cudapy/test_random.py
 * :29-52): generator t draws `count` values into out[t*count + i], i ascending,
 * and its state is advanced in place (by `count` steps for uniforms, 2*count for
 * normals). */
int nbh_xoro_uniform_f32(void *states, int64_t nstates, float *out, int64_t count, nbh_stream_t stream);
int nbh_xoro_uniform_f64(void *states, int64_t nstates, double *out, int64_t count, nbh_stream_t stream);
int nbh_xoro_normal_f32(void *states, int64_t nstates, float *out, int64_t count, nbh_stream_t stream);
int nbh_xoro_normal_f64(void *states, int64_t nstates, double *out, int64_t count, nbh_stream_t stream);

/* random.py:96-238 the per-generator functions xoroshiro128p_next / _jump /
 * _uniform_float32 / _uniform_float64 / _normal_float32 / _normal_float64 applied to ONE
 * generator of a device-resident state array (the reference's simulator lets host code
 * call them on the array create_xoroshiro128p_states returned).  `state` points to the
 * generator's 16-byte record in device memory and is advanced in place; the value goes
 * to `out`, 8-byte aligned memory the device can address (uint64 for NEXT, float /
 * double for the draws; unused and may be NULL for JUMP).  Same bits as the bulk calls. */
enum nbh_xoro_kind { NBH_XORO_NEXT = 0, NBH_XORO_JUMP = 1, NBH_XORO_UNIFORM_F32 = 2, NBH_XORO_UNIFORM_F64 = 3,
                     NBH_XORO_NORMAL_F32 = 4, NBH_XORO_NORMAL_F64 = 5 };
int nbh_xoro_one(void *state, int kind, void *out, nbh_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* NBHIP_H */

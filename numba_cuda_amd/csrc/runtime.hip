// Device, memory, stream and event entry points of libnbhip.so: thin, checked
// passages to the HIP runtime.  The Python layer owns every lifetime.
#include "common.h"


#include <string.h>

#include <atomic>

extern "C" {

int nbh_version(void) { return NBH_VERSION; }

int nbh_hip_versions(int *driver_version, int *runtime_version)
{
    if (!driver_version || !runtime_version)
        return (int)hipErrorInvalidValue;
    hipError_t e = hipDriverGetVersion(driver_version);
    if (e == hipSuccess)
        e = hipRuntimeGetVersion(runtime_version);
    return (int)e;
}

const char *nbh_error_name(int code) { return hipGetErrorName((hipError_t)code); }
const char *nbh_error_string(int code) { return hipGetErrorString((hipError_t)code); }

int nbh_device_count(int *count)
{
    if (!count)
        return (int)hipErrorInvalidValue;
    hipError_t e = hipGetDeviceCount(count);
    if (e == hipErrorNoDevice) {  // a machine without a GPU has zero devices
        *count = 0;
        (void)hipGetLastError();
        return (int)hipSuccess;
    }
    return (int)e;
}

int nbh_set_device(int dev) { return (int)hipSetDevice(dev); }
int nbh_get_device(int *dev) { return (int)hipGetDevice(dev); }

int nbh_device_name(int dev, char *buf, int buflen)
{
    if (!buf || buflen <= 0)
        return (int)hipErrorInvalidValue;
    return (int)hipDeviceGetName(buf, buflen, dev);
}

namespace {
struct AttrName {
    const char *name;
    hipDeviceAttribute_t attr;
};
// CUDA attribute names the reference exposes as Device.<NAME>, mapped to HIP.
const AttrName kAttrs[] = {
    {"MAX_THREADS_PER_BLOCK", hipDeviceAttributeMaxThreadsPerBlock},
    {"MAX_BLOCK_DIM_X", hipDeviceAttributeMaxBlockDimX},
    {"MAX_BLOCK_DIM_Y", hipDeviceAttributeMaxBlockDimY},
    {"MAX_BLOCK_DIM_Z", hipDeviceAttributeMaxBlockDimZ},
    {"MAX_GRID_DIM_X", hipDeviceAttributeMaxGridDimX},
    {"MAX_GRID_DIM_Y", hipDeviceAttributeMaxGridDimY},
    {"MAX_GRID_DIM_Z", hipDeviceAttributeMaxGridDimZ},
    {"MAX_SHARED_MEMORY_PER_BLOCK", hipDeviceAttributeMaxSharedMemoryPerBlock},
    {"MAX_SHARED_MEMORY_PER_MULTIPROCESSOR", hipDeviceAttributeMaxSharedMemoryPerMultiprocessor},
    {"TOTAL_CONSTANT_MEMORY", hipDeviceAttributeTotalConstantMemory},
    {"WARP_SIZE", hipDeviceAttributeWarpSize},
    {"MAX_REGISTERS_PER_BLOCK", hipDeviceAttributeMaxRegistersPerBlock},
    {"CLOCK_RATE", hipDeviceAttributeClockRate},
    {"MEMORY_CLOCK_RATE", hipDeviceAttributeMemoryClockRate},
    {"GLOBAL_MEMORY_BUS_WIDTH", hipDeviceAttributeMemoryBusWidth},
    {"MULTIPROCESSOR_COUNT", hipDeviceAttributeMultiprocessorCount},
    {"MAX_THREADS_PER_MULTIPROCESSOR", hipDeviceAttributeMaxThreadsPerMultiProcessor},
    {"L2_CACHE_SIZE", hipDeviceAttributeL2CacheSize},
    {"COMPUTE_CAPABILITY_MAJOR", hipDeviceAttributeComputeCapabilityMajor},
    {"COMPUTE_CAPABILITY_MINOR", hipDeviceAttributeComputeCapabilityMinor},
    {"COMPUTE_MODE", hipDeviceAttributeComputeMode},
    {"CONCURRENT_KERNELS", hipDeviceAttributeConcurrentKernels},
    {"ECC_ENABLED", hipDeviceAttributeEccEnabled},
    {"INTEGRATED", hipDeviceAttributeIntegrated},
    {"KERNEL_EXEC_TIMEOUT", hipDeviceAttributeKernelExecTimeout},
    {"CAN_MAP_HOST_MEMORY", hipDeviceAttributeCanMapHostMemory},
    {"PCI_BUS_ID", hipDeviceAttributePciBusId},
    {"PCI_DEVICE_ID", hipDeviceAttributePciDeviceId},
    {"PCI_DOMAIN_ID", hipDeviceAttributePciDomainID},
    {"MANAGED_MEMORY", hipDeviceAttributeManagedMemory},
    {"CONCURRENT_MANAGED_ACCESS", hipDeviceAttributeConcurrentManagedAccess},
    {"PAGEABLE_MEMORY_ACCESS", hipDeviceAttributePageableMemoryAccess},
    {"COOPERATIVE_LAUNCH", hipDeviceAttributeCooperativeLaunch},
    {"ASYNC_ENGINE_COUNT", hipDeviceAttributeAsyncEngineCount},
    {"UNIFIED_ADDRESSING", hipDeviceAttributeUnifiedAddressing},
    {"MAX_PITCH", hipDeviceAttributeMaxPitch},
    {"TEXTURE_ALIGNMENT", hipDeviceAttributeTextureAlignment},
};
}  // namespace

int nbh_device_attr(int dev, const char *name, int *value)
{
    if (!name || !value)
        return (int)hipErrorInvalidValue;
    for (const AttrName &a : kAttrs)
        if (strcmp(a.name, name) == 0)
            return (int)hipDeviceGetAttribute(value, a.attr, dev);
    return (int)hipErrorInvalidValue;
}

int nbh_mem_info(size_t *free_bytes, size_t *total_bytes) { return (int)hipMemGetInfo(free_bytes, total_bytes); }
int nbh_device_synchronize(void)
{
    nbh_queue_drain_all();
    return (int)hipDeviceSynchronize();
}

// ---- memory ----------------------------------------------------------------

int nbh_malloc(void **dptr, size_t nbytes)
{
    if (!dptr)
        return (int)hipErrorInvalidValue;
    return (int)hipMalloc(dptr, nbytes);
}
int nbh_free(void *dptr)
{
    nbh_queue_drain_all();  // a queued launch may still name this memory
    return (int)hipFree(dptr);
}
int nbh_malloc_managed(void **ptr, size_t nbytes, int attach_global)
{
    if (!ptr)
        return (int)hipErrorInvalidValue;
    return (int)hipMallocManaged(ptr, nbytes, attach_global ? hipMemAttachGlobal : hipMemAttachHost);
}

int nbh_host_alloc(void **hptr, size_t nbytes, unsigned flags)
{
    if (!hptr)
        return (int)hipErrorInvalidValue;
    unsigned f = hipHostMallocDefault;
    if (flags & 1u)
        f |= hipHostMallocPortable;
    if (flags & 2u)
        f |= hipHostMallocMapped;
    if (flags & 4u)
        f |= hipHostMallocWriteCombined;
    return (int)hipHostMalloc(hptr, nbytes, f);
}
int nbh_host_free(void *hptr)
{
    nbh_queue_drain_all();
    return (int)hipHostFree(hptr);
}

int nbh_host_register(void *hptr, size_t nbytes, unsigned flags)
{
    unsigned f = hipHostRegisterDefault;
    if (flags & 1u)
        f |= hipHostRegisterPortable;
    if (flags & 2u)
        f |= hipHostRegisterMapped;
    return (int)hipHostRegister(hptr, nbytes, f);
}
int nbh_host_unregister(void *hptr)
{
    nbh_queue_drain_all();
    return (int)hipHostUnregister(hptr);
}
int nbh_host_get_device_pointer(void **dptr, void *hptr) { return (int)hipHostGetDevicePointer(dptr, hptr, 0); }

int nbh_mem_address_range(void **base, size_t *size, void *dptr)
{
    hipDeviceptr_t b = nullptr;
    size_t n = 0;
    NBH_TRY(hipMemGetAddressRange(&b, &n, (hipDeviceptr_t)dptr));
    if (base)
        *base = (void *)b;
    if (size)
        *size = n;
    return 0;
}

// ---- sharing an allocation with another process ---------------------------------------
// Handles are hipIpcMemHandle_t, 64 opaque bytes.  Opening an allocation of 2 GiB or more
// has been seen not to return on MI355X hosts, so such allocations are refused on both
// sides (the exporter knows the size of the allocation, the importer only the size the
// caller asks for).
static_assert(sizeof(hipIpcMemHandle_t) == NBH_IPC_HANDLE_BYTES, "handle size");
static constexpr size_t kIpcLimit = (size_t)2 << 30;

int nbh_ipc_get_handle(void *handle, void *dptr)
{
    if (!handle || !dptr)
        return (int)hipErrorInvalidValue;
    hipDeviceptr_t base = nullptr;
    size_t n = 0;
    NBH_TRY(hipMemGetAddressRange(&base, &n, (hipDeviceptr_t)dptr));
    if ((void *)base != dptr)
        return (int)hipErrorInvalidValue;  // handles name whole allocations
    if (n >= kIpcLimit)
        return (int)hipErrorNotSupported;
    hipIpcMemHandle_t h;
    NBH_TRY(hipIpcGetMemHandle(&h, dptr));
    memcpy(handle, &h, sizeof h);
    return 0;
}

int nbh_ipc_open(void **dptr, const void *handle, size_t nbytes)
{
    if (!dptr || !handle)
        return (int)hipErrorInvalidValue;
    if (nbytes >= kIpcLimit)
        return (int)hipErrorNotSupported;
    hipIpcMemHandle_t h;
    memcpy(&h, handle, sizeof h);
    return (int)hipIpcOpenMemHandle(dptr, h, hipIpcMemLazyEnablePeerAccess);
}

int nbh_ipc_close(void *dptr)
{
    nbh_queue_drain_all();
    return (int)hipIpcCloseMemHandle(dptr);
}

static int copy(void *dst, const void *src, size_t nbytes, hipMemcpyKind kind, nbh_stream_t stream)
{
    if (nbytes == 0)
        return 0;
    nbh_stream_report report(nbh_hip_stream(stream));
    if (stream)
        return (int)hipMemcpyAsync(dst, src, nbytes, kind, nbh_hip_stream(stream));
    return (int)hipMemcpy(dst, src, nbytes, kind);
}
// Large copies of pageable memory are pipelined through page-locked buffers by the
// library itself (with or without a stream: a copy of pageable memory cannot outlive
// the call either way).
int nbh_memcpy_h2d(void *dst, const void *src, size_t nbytes, nbh_stream_t stream)
{
    nbh_stream_report report(nbh_hip_stream(stream));
    const int rc = nbh_staged_h2d(dst, src, nbytes, nbh_hip_stream(stream));
    if (rc >= 0)
        return rc;
    return copy(dst, src, nbytes, hipMemcpyHostToDevice, stream);
}
int nbh_memcpy_d2h(void *dst, const void *src, size_t nbytes, nbh_stream_t stream)
{
    nbh_stream_report report(nbh_hip_stream(stream));
    const int rc = nbh_staged_d2h(dst, src, nbytes, nbh_hip_stream(stream));
    if (rc >= 0)
        return rc;
    return copy(dst, src, nbytes, hipMemcpyDeviceToHost, stream);
}
// Plain device memory of the current device?  (Not host-mapped or managed memory,
// not another device's, not a pointer HIP has never seen.)
static bool local_device_memory(const void *p)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess)
        return false;
    return attr.type == hipMemoryTypeDevice && attr.device == dev;
}

// Large copies inside one device run on the library's own copy kernel: 6.3 TB/s
// against 5.2 TB/s for hipMemcpyDtoD (MI355X, 1 GiB).  Everything else is hipMemcpy's.
int nbh_memcpy_d2d(void *dst, const void *src, size_t nbytes, nbh_stream_t stream)
{
    constexpr size_t kOwnKernelFrom = (size_t)1 << 20;
    if (nbytes >= kOwnKernelFrom && local_device_memory(dst) && local_device_memory(src)) {
        hipStream_t s = nbh_hip_stream(stream);
        int rc = nbh_flat_copy(dst, src, (int64_t)nbytes, s);
        if (rc || stream)
            return rc;
        return (int)hipStreamSynchronize(s);  // no stream given: the caller expects a finished copy
    }
    return copy(dst, src, nbytes, hipMemcpyDeviceToDevice, stream);
}
int nbh_memset8(void *dst, int byte, size_t nbytes, nbh_stream_t stream)
{
    if (nbytes == 0)
        return 0;
    nbh_stream_report report(nbh_hip_stream(stream));
    if (stream)
        return (int)hipMemsetAsync(dst, byte, nbytes, nbh_hip_stream(stream));
    return (int)hipMemset(dst, byte, nbytes);
}

// ---- streams and events ------------------------------------------------------

int nbh_stream_create(nbh_stream_t *stream)
{
    if (!stream)
        return (int)hipErrorInvalidValue;
    hipStream_t s = nullptr;
    NBH_TRY(hipStreamCreateWithFlags(&s, hipStreamDefault));
    *stream = (nbh_stream_t)s;
    return 0;
}
int nbh_stream_destroy(nbh_stream_t stream)
{
    nbh_queue_forget(stream);
    nbh_pool_forget_stream(nbh_hip_stream(stream));
    return (int)hipStreamDestroy(nbh_hip_stream(stream));
}
int nbh_stream_synchronize(nbh_stream_t stream)
{
    const int rc = (int)hipStreamSynchronize(nbh_hip_stream(stream));
    const int queued = nbh_queue_take_status(stream);  // a launch that a launching thread could not make
    return rc ? rc : queued;
}
int nbh_stream_query(nbh_stream_t stream) { return (int)hipStreamQuery(nbh_hip_stream(stream)); }

int nbh_stream_add_callback(nbh_stream_t stream, nbh_host_fn fn, void *user)
{
    if (!fn)
        return (int)hipErrorInvalidValue;
    return (int)hipLaunchHostFunc(nbh_hip_stream(stream), fn, user);
}

int nbh_event_create(nbh_event_t *event, int timing)
{
    if (!event)
        return (int)hipErrorInvalidValue;
    hipEvent_t e = nullptr;
    NBH_TRY(hipEventCreateWithFlags(&e, timing ? hipEventDefault : hipEventDisableTiming));
    *event = (nbh_event_t)e;
    return 0;
}
int nbh_event_destroy(nbh_event_t event) { return (int)hipEventDestroy((hipEvent_t)event); }
int nbh_event_record(nbh_event_t event, nbh_stream_t stream)
{
    return (int)hipEventRecord((hipEvent_t)event, nbh_hip_stream(stream));
}
int nbh_event_synchronize(nbh_event_t event) { return (int)hipEventSynchronize((hipEvent_t)event); }
int nbh_event_query(nbh_event_t event) { return (int)hipEventQuery((hipEvent_t)event); }
int nbh_stream_wait_event(nbh_stream_t stream, nbh_event_t event)
{
    return (int)hipStreamWaitEvent(nbh_hip_stream(stream), (hipEvent_t)event, 0);
}
int nbh_event_elapsed_ms(float *ms, nbh_event_t start, nbh_event_t stop)
{
    return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}

}  // extern "C"

// ---- shared helper -----------------------------------------------------------

int nbh_cu_count()
{
    constexpr int kMaxDev = 64;
    static std::atomic<int> cache[kMaxDev];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev)
        return 256;
    int v = cache[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            v = 256;
        cache[dev].store(v, std::memory_order_relaxed);
    }
    return v;
}

// nbh_reduce_compile / nbh_reduce_custom: reductions with a binary operation that the
// caller supplies as source text, compiled for the device at run time.
//
// The reference turns ANY Python functor into device code with its JIT
// (kernels/reduction.py:175-192).  The seven operators that matter most have hand-written
// kernels (reduce.hip); every other functor arrives here as the body of
//
//     __device__ T nbh_op(T a, T b) { <body> }
//
// (the Python layer writes it from the functor, with the reference's typing rules spelled
// out as casts), is compiled once per (body, element type) with the HIP run-time compiler
// and kept as a code object; a module is loaded from it on each device that uses it.
//
// The operation has no known identity element, so nothing may be padded: every lane
// carries a "have" flag next to its accumulator, an input element enters the fold exactly
// once, and n elements plus `init` cost exactly n applications, as in the reference (which
// matters for operations like a + b + 1).  The order of association is this library's, not
// the reference's: like the reference, the result is only defined for operations that are
// associative and commutative.
//
// Two launches: `nbh_custom_partials` leaves one partial (and its flag) per workgroup in
// the scratch buffer, `nbh_custom_finish` (one workgroup) folds those, applies `init` and
// writes `out`.  The partial slots are those of nbh_reduce's scratch buffer; the ticket in
// its header is not touched, so one buffer serves both kinds of calls on a stream.
#include <dlfcn.h>
#include <hip/hiprtc.h>

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kMaxGrid = 2048;            // 8 workgroups per compute unit on a 256-CU part
constexpr size_t kHeaderBytes = 256;      // nbh_reduce's ticket lives here
constexpr size_t kFlagsOffset = kHeaderBytes + sizeof(uint64_t) * kMaxGrid;
constexpr size_t kNeededBytes = kFlagsOffset + sizeof(uint32_t) * kMaxGrid;
constexpr int kMaxDevices = 64;

// ---- the run-time compiler, loaded on first use ---------------------------------------
struct Rtc {
    decltype(&hiprtcCreateProgram) create = nullptr;
    decltype(&hiprtcCompileProgram) compile = nullptr;
    decltype(&hiprtcGetProgramLogSize) log_size = nullptr;
    decltype(&hiprtcGetProgramLog) log = nullptr;
    decltype(&hiprtcGetCodeSize) code_size = nullptr;
    decltype(&hiprtcGetCode) code = nullptr;
    decltype(&hiprtcDestroyProgram) destroy = nullptr;
    bool ok = false;
};

const Rtc &rtc()
{
    static Rtc r = [] {
        Rtc t;
        void *h = nullptr;
        for (const char *name : {"libhiprtc.so", "libhiprtc.so.7", "/opt/rocm/lib/libhiprtc.so"}) {
            h = dlopen(name, RTLD_NOW | RTLD_LOCAL);
            if (h)
                break;
        }
        if (!h)
            return t;
#define NBH_SYM(field, name) t.field = reinterpret_cast<decltype(t.field)>(dlsym(h, name))
        NBH_SYM(create, "hiprtcCreateProgram");
        NBH_SYM(compile, "hiprtcCompileProgram");
        NBH_SYM(log_size, "hiprtcGetProgramLogSize");
        NBH_SYM(log, "hiprtcGetProgramLog");
        NBH_SYM(code_size, "hiprtcGetCodeSize");
        NBH_SYM(code, "hiprtcGetCode");
        NBH_SYM(destroy, "hiprtcDestroyProgram");
#undef NBH_SYM
        t.ok = t.create && t.compile && t.log_size && t.log && t.code_size && t.code && t.destroy;
        return t;
    }();
    return r;
}

const char *type_name(int dtype, size_t *elem)
{
    switch (dtype) {
    case NBH_I8: *elem = 1; return "signed char";
    case NBH_I16: *elem = 2; return "short";
    case NBH_I32: *elem = 4; return "int";
    case NBH_I64: *elem = 8; return "long long";
    case NBH_U8: *elem = 1; return "unsigned char";
    case NBH_U16: *elem = 2; return "unsigned short";
    case NBH_U32: *elem = 4; return "unsigned int";
    case NBH_U64: *elem = 8; return "unsigned long long";
    case NBH_F32: *elem = 4; return "float";
    case NBH_F64: *elem = 8; return "double";
    case NBH_F16: *elem = 2; return "_Float16";
    default: return nullptr;
    }
}

// Device source: `typedef <type> T;` goes in front, the caller's body replaces @BODY@.
const char kSource[] = R"NBHSRC(
typedef long long nbh_i64;
typedef unsigned long long nbh_u64;
typedef unsigned int nbh_u32x4 __attribute__((ext_vector_type(4)));

// Python's // and % (round towards minus infinity, the remainder takes the divisor's
// sign); a zero divisor gives 0 instead of raising
__device__ __forceinline__ nbh_i64 nbh_floordiv(nbh_i64 a, nbh_i64 b)
{
    if (b == 0) return 0;
    if (b == -1) return (nbh_i64)(0ull - (nbh_u64)a);
    const nbh_i64 q = a / b;
    return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
}
__device__ __forceinline__ nbh_i64 nbh_mod(nbh_i64 a, nbh_i64 b)
{
    if (b == 0 || b == -1) return 0;
    const nbh_i64 r = a % b;
    return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r;
}
__device__ __forceinline__ nbh_u64 nbh_floordiv(nbh_u64 a, nbh_u64 b) { return b ? a / b : 0ull; }
__device__ __forceinline__ nbh_u64 nbh_mod(nbh_u64 a, nbh_u64 b) { return b ? a % b : 0ull; }
__device__ __forceinline__ double nbh_floordiv(double a, double b) { return floor(a / b); }
__device__ __forceinline__ float nbh_floordiv(float a, float b) { return floorf(a / b); }
__device__ __forceinline__ double nbh_mod(double a, double b)
{
    const double r = fmod(a, b);
    return (r != 0.0 && ((r < 0.0) != (b < 0.0))) ? r + b : r;
}
__device__ __forceinline__ float nbh_mod(float a, float b)
{
    const float r = fmodf(a, b);
    return (r != 0.0f && ((r < 0.0f) != (b < 0.0f))) ? r + b : r;
}
// integer power with a non-negative exponent, wrapping like the multiplications it stands for
__device__ __forceinline__ nbh_i64 nbh_ipow(nbh_i64 x, nbh_i64 e)
{
    nbh_u64 r = 1, m = (nbh_u64)x;
    for (nbh_u64 k = e > 0 ? (nbh_u64)e : 0ull; k; k >>= 1) {
        if (k & 1) r *= m;
        m *= m;
    }
    return (nbh_i64)r;
}

__device__ __forceinline__ T nbh_op(T a, T b)
{
@BODY@
}
// (everything above this line is also valid host C++ once __device__ and __forceinline__
// are defined away: the translation of functors is checked that way without a device)

constexpr int kItems = 16 / (int)sizeof(T);     // elements per 16-byte packet
union nbh_packet { nbh_u32x4 raw; T item[kItems]; };
union nbh_slot { nbh_u64 word; T value; };

__device__ __forceinline__ nbh_u64 nbh_word_of(T v)
{
    nbh_slot s;
    s.word = 0;
    s.value = v;
    return s.word;
}
__device__ __forceinline__ T nbh_value_of(nbh_u64 w)
{
    nbh_slot s;
    s.word = w;
    return s.value;
}
__device__ __forceinline__ void nbh_take(T &acc, bool &have, T v)
{
    acc = have ? nbh_op(acc, v) : v;
    have = true;
}
__device__ __forceinline__ T nbh_fold_packet(const nbh_u32x4 raw)
{
    nbh_packet p;
    p.raw = raw;
    T v = p.item[0];
#pragma unroll
    for (int j = 1; j < kItems; ++j)
        v = nbh_op(v, p.item[j]);
    return v;
}

// Lane 0 of the wavefront, then thread 0 of the workgroup, ends up with every item that
// any thread holds, each taken once.
__device__ __forceinline__ void nbh_fold_workgroup(T &acc, bool &have)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const nbh_u64 theirs = __shfl_down(nbh_word_of(acc), off, 64);
        const int they_have = __shfl_down((int)have, off, 64);
        if (lane + off < 64 && they_have)
            nbh_take(acc, have, nbh_value_of(theirs));
    }
    __shared__ nbh_u64 wave_value[4];
    __shared__ int wave_has[4];
    if (lane == 0) {
        wave_value[wave] = nbh_word_of(acc);
        wave_has[wave] = (int)have;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int waves = (int)(blockDim.x + 63) >> 6;
        for (int w = 1; w < waves; ++w)
            if (wave_has[w])
                nbh_take(acc, have, nbh_value_of(wave_value[w]));
    }
}

// packets > 0: `in` is contiguous and 16-byte aligned; the first `packets` packets are read
// whole, the fewer than kItems items after them one by one.  packets == 0: items
// `stride` bytes apart.
extern "C" __global__ __launch_bounds__(256) void nbh_custom_partials(const char *__restrict__ in, long long n,
                                                                     long long stride, long long packets,
                                                                     nbh_u64 *__restrict__ part_value,
                                                                     unsigned *__restrict__ part_has)
{
    const long long me = blockIdx.x * 256ll + threadIdx.x, step = gridDim.x * 256ll;
    T acc = T();
    bool have = false;
    if (packets > 0) {
        const nbh_u32x4 *__restrict__ p = reinterpret_cast<const nbh_u32x4 *>(in);
        long long k = me;
        if (k < packets) {
            acc = nbh_fold_packet(__builtin_nontemporal_load(p + k));
            have = true;
            k += step;
        }
        for (; k + 3 * step < packets; k += 4 * step) {
            const nbh_u32x4 r0 = __builtin_nontemporal_load(p + k);
            const nbh_u32x4 r1 = __builtin_nontemporal_load(p + k + step);
            const nbh_u32x4 r2 = __builtin_nontemporal_load(p + k + 2 * step);
            const nbh_u32x4 r3 = __builtin_nontemporal_load(p + k + 3 * step);
            const T v01 = nbh_op(nbh_fold_packet(r0), nbh_fold_packet(r1));
            const T v23 = nbh_op(nbh_fold_packet(r2), nbh_fold_packet(r3));
            acc = nbh_op(acc, nbh_op(v01, v23));
        }
        for (; k < packets; k += step)
            acc = nbh_op(acc, nbh_fold_packet(__builtin_nontemporal_load(p + k)));
        const long long t = packets * kItems + me;
        if (t < n)
            nbh_take(acc, have, reinterpret_cast<const T *>(in)[t]);
    } else {
        for (long long i = me; i < n; i += step)
            nbh_take(acc, have, *reinterpret_cast<const T *>(in + i * stride));
    }
    nbh_fold_workgroup(acc, have);
    if (threadIdx.x == 0) {
        part_value[blockIdx.x] = nbh_word_of(acc);
        part_has[blockIdx.x] = have ? 1u : 0u;
    }
}

extern "C" __global__ __launch_bounds__(256) void nbh_custom_finish(const nbh_u64 *__restrict__ part_value,
                                                                   const unsigned *__restrict__ part_has, int count,
                                                                   T init, T *__restrict__ out)
{
    T acc = T();
    bool have = false;
    for (int k = threadIdx.x; k < count; k += 256)
        if (part_has[k])
            nbh_take(acc, have, nbh_value_of(part_value[k]));
    nbh_fold_workgroup(acc, have);
    if (threadIdx.x == 0)
        out[0] = have ? nbh_op(acc, init) : init;
}
)NBHSRC";

struct CustomOp {
    int dtype = 0;
    size_t elem = 0;
    std::vector<char> code;
    std::mutex lock;
    struct Loaded {
        hipModule_t module = nullptr;
        hipFunction_t partials = nullptr, finish = nullptr;
    } on_device[kMaxDevices];
};

void put_log(char *log, size_t log_bytes, const std::string &text)
{
    if (!log || log_bytes == 0)
        return;
    const size_t n = text.size() < log_bytes - 1 ? text.size() : log_bytes - 1;
    memcpy(log, text.data(), n);
    log[n] = 0;
}

int functions_for(CustomOp *op, CustomOp::Loaded **out)
{
    int dev = 0;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> hold(op->lock);
    CustomOp::Loaded &slot = op->on_device[dev];
    if (!slot.finish) {
        hipModule_t m = nullptr;
        NBH_TRY(hipModuleLoadData(&m, op->code.data()));
        hipFunction_t f1 = nullptr, f2 = nullptr;
        hipError_t e = hipModuleGetFunction(&f1, m, "nbh_custom_partials");
        if (e == hipSuccess)
            e = hipModuleGetFunction(&f2, m, "nbh_custom_finish");
        if (e != hipSuccess) {
            (void)hipModuleUnload(m);
            return (int)e;
        }
        slot.module = m;
        slot.partials = f1;
        slot.finish = f2;
    }
    *out = &slot;
    return 0;
}

}  // namespace

extern "C" int nbh_reduce_compile(int dtype, const char *body, void **op_out, char *log, size_t log_bytes)
{
    put_log(log, log_bytes, "");
    size_t elem = 0;
    const char *type = type_name(dtype, &elem);
    if (!type || !body || !op_out)
        return (int)hipErrorInvalidValue;
    const Rtc &r = rtc();
    if (!r.ok) {
        put_log(log, log_bytes, "the HIP run-time compiler (libhiprtc.so) could not be loaded");
        return (int)hipErrorSharedObjectInitFailed;
    }
    std::string source = std::string("typedef ") + type + " T;\n" + kSource;
    const size_t at = source.find("@BODY@");
    source.replace(at, 6, body);

    hiprtcProgram prog = nullptr;
    if (r.create(&prog, source.c_str(), "nbh_reduce_custom.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        return (int)hipErrorInvalidSource;
    // the same code generation choices as the rest of the library: no contraction of a * b + c
    // (the reference compiles without it), no packed float32 instructions
    const char *options[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
                             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult built = r.compile(prog, (int)(sizeof(options) / sizeof(options[0])), options);
    size_t log_len = 0;
    if (r.log_size(prog, &log_len) == HIPRTC_SUCCESS && log_len > 1) {
        std::string text(log_len, '\0');
        if (r.log(prog, &text[0]) == HIPRTC_SUCCESS)
            put_log(log, log_bytes, text.c_str());
    }
    if (built != HIPRTC_SUCCESS) {
        r.destroy(&prog);
        return (int)hipErrorInvalidSource;
    }
    CustomOp *op = new CustomOp;
    op->dtype = dtype;
    op->elem = elem;
    size_t bytes = 0;
    if (r.code_size(prog, &bytes) != HIPRTC_SUCCESS || bytes == 0) {
        r.destroy(&prog);
        delete op;
        return (int)hipErrorInvalidSource;
    }
    op->code.resize(bytes);
    const hiprtcResult got = r.code(prog, op->code.data());
    r.destroy(&prog);
    if (got != HIPRTC_SUCCESS) {
        delete op;
        return (int)hipErrorInvalidSource;
    }
    *op_out = op;
    return 0;
}

extern "C" int nbh_reduce_op_dtype(const void *op)
{
    return op ? static_cast<const CustomOp *>(op)->dtype : -1;
}

extern "C" int nbh_reduce_op_free(void *handle)
{
    CustomOp *op = static_cast<CustomOp *>(handle);
    if (!op)
        return 0;
    int before = 0;
    const bool have_device = hipGetDevice(&before) == hipSuccess;
    for (int d = 0; d < kMaxDevices; ++d)
        if (op->on_device[d].module && hipSetDevice(d) == hipSuccess)
            (void)hipModuleUnload(op->on_device[d].module);
    if (have_device)
        (void)hipSetDevice(before);
    delete op;
    return 0;
}

extern "C" int nbh_reduce_custom(void *handle, const void *in, int64_t n, int64_t in_stride, const void *init,
                                 void *out, void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    CustomOp *op = static_cast<CustomOp *>(handle);
    if (!op || !in || !init || !out || !scratch || n < 1 || scratch_bytes < kNeededBytes ||
        ((uintptr_t)scratch) % 8 != 0 || in_stride % (int64_t)op->elem != 0)
        return (int)hipErrorInvalidValue;
    CustomOp::Loaded *fn = nullptr;
    const int rc = functions_for(op, &fn);
    if (rc)
        return rc;
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);

    const int64_t items = 16 / (int64_t)op->elem;
    long long packets = 0;
    if (in_stride == (int64_t)op->elem && ((uintptr_t)in) % 16 == 0)
        packets = n / items;
    const int64_t threads = packets > 0 ? packets : n;
    int64_t grid = (threads + kBlock - 1) / kBlock;
    if (grid > kMaxGrid)
        grid = kMaxGrid;
    if (grid < 1)
        grid = 1;

    const char *in_arg = static_cast<const char *>(in);
    long long n_arg = n, stride_arg = in_stride;
    uint64_t *part_value = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kHeaderBytes);
    unsigned *part_has = reinterpret_cast<unsigned *>(static_cast<char *>(scratch) + kFlagsOffset);
    void *args1[] = {&in_arg, &n_arg, &stride_arg, &packets, &part_value, &part_has};
    NBH_TRY(hipModuleLaunchKernel(fn->partials, (unsigned)grid, 1, 1, kBlock, 1, 1, 0, s, args1, nullptr));

    int count = (int)grid;
    // `init` travels as a kernel argument: the launch copies the element it points to
    void *args2[] = {&part_value, &part_has, &count, const_cast<void *>(init), &out};
    NBH_TRY(hipModuleLaunchKernel(fn->finish, 1, 1, 1, kBlock, 1, 1, 0, s, args2, nullptr));
    return 0;
}

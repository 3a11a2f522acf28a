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
// One launch of `nbh_custom_reduce`, shaped like nbh_reduce's kernel: 512-thread workgroups,
// two per compute unit, each streaming one contiguous slice (large inputs: 16 KiB pieces
// dealt out round robin); one partial per workgroup in
// the scratch buffer; the workgroup that draws the last ticket folds the partials, applies
// `init` and writes `out`.  Ticket and partial slots are those of nbh_reduce's scratch
// buffer, used the same way (the ticket is handed back at zero), so one buffer serves both
// kinds of calls on a stream.
#include <dlfcn.h>
#include <hip/hiprtc.h>

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

namespace {

constexpr int kBlock = 512;               // threads per workgroup; the device source says the same
constexpr int kUnroll = 4;
constexpr int64_t kPiecePackets = 2 * kBlock;  // a dealt piece; the device source says the same
constexpr int kGridPerCU = 2;
constexpr int kMaxGrid = 4096;            // partial slots in nbh_reduce's scratch buffer
constexpr size_t kHeaderBytes = 256;      // the ticket lives here
constexpr size_t kNeededBytes = kHeaderBytes + sizeof(uint64_t) * kMaxGrid;
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
    case NBH_C64: *elem = 8; return "nbh_c64";
    case NBH_C128: *elem = 16; return "nbh_c128";
    default: return nullptr;
    }
}

// Device source: the element type replaces @T@, the caller's body replaces @BODY@.
const char kSource[] = R"NBHSRC(
typedef long long nbh_i64;
typedef unsigned long long nbh_u64;
typedef unsigned int nbh_u32x4 __attribute__((ext_vector_type(4)));

// Complex numbers as the reference's JIT computes with them (numba/cuda/cpython/numbers.py:
// :1091-1120 sums and differences part by part, :1123-1146 the product as (ac - bd) + (ad + bc)i
// with every product and sum rounded once, :1149-1179 the quotient by CPython's algorithm,
// :1200-1221 equality, :1224-1233 abs as hypot).  An aggregate: it lives in unions with raw words.
template <typename R> struct nbh_cplx { R re, im; };
typedef nbh_cplx<float> nbh_c64;
typedef nbh_cplx<double> nbh_c128;
typedef @T@ T;

template <typename R> __device__ __forceinline__ nbh_cplx<R> operator+(nbh_cplx<R> x, nbh_cplx<R> y)
{
    return {x.re + y.re, x.im + y.im};
}
template <typename R> __device__ __forceinline__ nbh_cplx<R> operator-(nbh_cplx<R> x, nbh_cplx<R> y)
{
    return {x.re - y.re, x.im - y.im};
}
template <typename R> __device__ __forceinline__ nbh_cplx<R> operator-(nbh_cplx<R> x) { return {-x.re, -x.im}; }
template <typename R> __device__ __forceinline__ nbh_cplx<R> operator*(nbh_cplx<R> x, nbh_cplx<R> y)
{
    const R ac = x.re * y.re, bd = x.im * y.im, ad = x.re * y.im, bc = x.im * y.re;
    return {ac - bd, ad + bc};
}
// a zero divisor raises ZeroDivisionError in Python; here it gives NaN + NaN i
template <typename R> __device__ __forceinline__ nbh_cplx<R> operator/(nbh_cplx<R> x, nbh_cplx<R> y)
{
    const R nan = (R)__builtin_nan("");
    const R abs_re = y.re < 0 ? -y.re : y.re, abs_im = y.im < 0 ? -y.im : y.im;
    if (abs_re >= abs_im) {
        if (y.re == 0)
            return {nan, nan};
        const R ratio = y.im / y.re, denom = y.re + y.im * ratio;
        return {(x.re + x.im * ratio) / denom, (x.im - x.re * ratio) / denom};
    }
    if (y.im == 0)
        return {nan, nan};
    const R ratio = y.re / y.im, denom = y.re * ratio + y.im;
    return {(x.re * ratio + x.im) / denom, (x.im * ratio - x.re) / denom};
}
template <typename R> __device__ __forceinline__ bool operator==(nbh_cplx<R> x, nbh_cplx<R> y)
{
    return x.re == y.re && x.im == y.im;
}
template <typename R> __device__ __forceinline__ bool operator!=(nbh_cplx<R> x, nbh_cplx<R> y)
{
    return x.re != y.re || x.im != y.im;
}
__device__ __forceinline__ float nbh_cabs(nbh_c64 z) { return hypotf(z.re, z.im); }
__device__ __forceinline__ double nbh_cabs(nbh_c128 z) { return hypot(z.re, z.im); }
template <typename R> __device__ __forceinline__ nbh_cplx<R> nbh_conj(nbh_cplx<R> z) { return {z.re, -z.im}; }
// conversions into a complex type: from a real number (imaginary part 0) or the other complex type
template <typename R, typename X> __device__ __forceinline__ nbh_cplx<R> nbh_cplx_from(X x) { return {(R)x, (R)0}; }
template <typename R, typename Q> __device__ __forceinline__ nbh_cplx<R> nbh_cplx_from(nbh_cplx<Q> z)
{
    return {(R)z.re, (R)z.im};
}

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
constexpr int kThreads = 512, kWaves = 8, kUnroll = 4;
constexpr long long kPiece = 2 * kThreads;      // packets per dealt piece
union nbh_packet { nbh_u32x4 raw; T item[kItems]; };
// a value as the 64-bit words it travels in (shuffles, the partials in the scratch buffer)
constexpr int kSlotWords = ((int)sizeof(T) + 7) / 8;
union nbh_image { nbh_u64 w[kSlotWords]; T value; };

__device__ __forceinline__ nbh_image nbh_image_of(T v)
{
    nbh_image s;
#pragma unroll
    for (int k = 0; k < kSlotWords; ++k)
        s.w[k] = 0;
    s.value = v;
    return s;
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

// Thread 0 of the workgroup ends up with every item that any thread holds, each taken
// once, in an order that depends on nothing but the thread indices.
__device__ __forceinline__ void nbh_fold_workgroup(T &acc, bool &have)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const nbh_image mine = nbh_image_of(acc);
        nbh_image theirs;
#pragma unroll
        for (int k = 0; k < kSlotWords; ++k)
            theirs.w[k] = __shfl_down(mine.w[k], off, 64);
        const int they_have = __shfl_down((int)have, off, 64);
        if (lane + off < 64 && they_have)
            nbh_take(acc, have, theirs.value);
    }
    __shared__ T wave_value[kWaves];
    __shared__ int wave_has[kWaves];
    __syncthreads();  // the slots may still be read from a previous fold
    if (lane == 0) {
        wave_value[wave] = acc;
        wave_has[wave] = (int)have;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kWaves; ++w)
            if (wave_has[w])
                nbh_take(acc, have, wave_value[w]);
    }
}

// One launch.  Every workgroup owns a contiguous, non-empty slice of the input and streams
// it with kUnroll 16-byte non-temporal loads in flight per lane; it leaves one partial; the
// workgroup that draws the last ticket folds the partials in index order, applies `init`
// and writes `out`.  Partials are put in place with an agent-scope atomic exchange whose
// result is awaited before the ticket is drawn (the protocol of nbh_reduce, for the same
// reason: the L2 caches of the XCDs are not coherent with one another, agent-scope
// atomics are carried out where all of them look).
// packed != 0: items [head, head + units * kItems) are `units` aligned packets; the `head`
// items in front and the fewer than kItems behind are taken by single lanes of workgroup 0.
// packed == 2: large inputs, read piece by piece instead of slice by slice (see there).
// packed == 0: `units` items, `stride` bytes apart.
extern "C" __global__ __launch_bounds__(512) void nbh_custom_reduce(const char *__restrict__ in, long long n,
                                                                   long long head, long long units,
                                                                   long long stride, int packed, T init,
                                                                   T *__restrict__ out,
                                                                   nbh_u64 *__restrict__ partials,
                                                                   unsigned *__restrict__ ticket)
{
    __shared__ bool last_block;
    const int tid = threadIdx.x;
    const long long per = (units + gridDim.x - 1) / gridDim.x;
    const long long begin = (long long)blockIdx.x * per;
    long long end = begin + per;
    if (end > units)
        end = units;
    T acc = T();
    bool have = false;
    long long i = begin + tid;
    if (packed == 2) {
        // pieces of 2 * kThreads packets dealt out round robin (piece q of a round to the
        // workgroup whose XCD comes q / (grid / 8)-th): the workgroups read one moving
        // window; the caller sees to it that each of them gets two pieces or more
        const nbh_u32x4 *__restrict__ p = reinterpret_cast<const nbh_u32x4 *>(in + head * (long long)sizeof(T));
        const long long grid = gridDim.x, pieces = units / kPiece;
        const long long first = grid % 8 == 0 ? (long long)(blockIdx.x % 8) * (grid / 8) + blockIdx.x / 8
                                              : (long long)blockIdx.x;
        const nbh_u32x4 *__restrict__ q = p + first * kPiece + tid;
        nbh_u32x4 c0 = __builtin_nontemporal_load(q), c1 = __builtin_nontemporal_load(q + kThreads);
        q += grid * kPiece;
        nbh_u32x4 n0 = __builtin_nontemporal_load(q), n1 = __builtin_nontemporal_load(q + kThreads);
        acc = nbh_op(nbh_fold_packet(c0), nbh_fold_packet(c1));
        have = true;
        c0 = n0;
        c1 = n1;
        for (long long c = first + 2 * grid; c < pieces; c += grid) {
            q += grid * kPiece;
            n0 = __builtin_nontemporal_load(q);
            n1 = __builtin_nontemporal_load(q + kThreads);
            acc = nbh_op(acc, nbh_op(nbh_fold_packet(c0), nbh_fold_packet(c1)));
            c0 = n0;
            c1 = n1;
            __syncthreads();  // the wavefronts ask for a piece together, as one run of 16 KiB
        }
        acc = nbh_op(acc, nbh_op(nbh_fold_packet(c0), nbh_fold_packet(c1)));
        if (blockIdx.x == gridDim.x - 1)  // less than a piece of whole packets is left over
            for (long long k = pieces * kPiece + tid; k < units; k += kThreads)
                acc = nbh_op(acc, nbh_fold_packet(__builtin_nontemporal_load(p + k)));
        if (blockIdx.x == 0) {
            const T *__restrict__ items = reinterpret_cast<const T *>(in);
            const long long tail_begin = head + units * kItems;
            if (tid < head)
                nbh_take(acc, have, items[tid]);
            else if (tail_begin + (tid - head) < n)
                nbh_take(acc, have, items[tail_begin + (tid - head)]);
        }
    } else if (packed) {
        const nbh_u32x4 *__restrict__ p = reinterpret_cast<const nbh_u32x4 *>(in + head * (long long)sizeof(T));
        if (i < end) {
            acc = nbh_fold_packet(__builtin_nontemporal_load(p + i));
            have = true;
            i += kThreads;
        }
        for (; i + (kUnroll - 1) * kThreads < end; i += kUnroll * kThreads) {
            const nbh_u32x4 r0 = __builtin_nontemporal_load(p + i);
            const nbh_u32x4 r1 = __builtin_nontemporal_load(p + i + kThreads);
            const nbh_u32x4 r2 = __builtin_nontemporal_load(p + i + 2 * kThreads);
            const nbh_u32x4 r3 = __builtin_nontemporal_load(p + i + 3 * kThreads);
            const T v01 = nbh_op(nbh_fold_packet(r0), nbh_fold_packet(r1));
            const T v23 = nbh_op(nbh_fold_packet(r2), nbh_fold_packet(r3));
            acc = nbh_op(acc, nbh_op(v01, v23));
        }
        for (; i < end; i += kThreads)
            acc = nbh_op(acc, nbh_fold_packet(__builtin_nontemporal_load(p + i)));
        if (blockIdx.x == 0) {
            const T *__restrict__ items = reinterpret_cast<const T *>(in);
            const long long tail_begin = head + units * kItems;
            if (tid < head)
                nbh_take(acc, have, items[tid]);
            else if (tail_begin + (tid - head) < n)
                nbh_take(acc, have, items[tail_begin + (tid - head)]);
        }
    } else {
        if (i < end) {
            acc = *reinterpret_cast<const T *>(in + i * stride);
            have = true;
            i += kThreads;
        }
        for (; i + (kUnroll - 1) * kThreads < end; i += kUnroll * kThreads) {
            const T v0 = *reinterpret_cast<const T *>(in + i * stride);
            const T v1 = *reinterpret_cast<const T *>(in + (i + kThreads) * stride);
            const T v2 = *reinterpret_cast<const T *>(in + (i + 2 * kThreads) * stride);
            const T v3 = *reinterpret_cast<const T *>(in + (i + 3 * kThreads) * stride);
            acc = nbh_op(acc, nbh_op(nbh_op(v0, v1), nbh_op(v2, v3)));
        }
        for (; i < end; i += kThreads)
            acc = nbh_op(acc, *reinterpret_cast<const T *>(in + i * stride));
    }
    nbh_fold_workgroup(acc, have);  // thread 0 has the slice's value: the slice is not empty

    if (gridDim.x == 1) {
        if (tid == 0)
            out[0] = nbh_op(acc, init);
        return;
    }
    if (tid == 0) {
        const nbh_image img = nbh_image_of(acc);
        nbh_u64 before[kSlotWords];
#pragma unroll
        for (int k = 0; k < kSlotWords; ++k)
            before[k] = __hip_atomic_exchange(&partials[(long long)blockIdx.x * kSlotWords + k], img.w[k],
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int k = 0; k < kSlotWords; ++k)
            asm volatile("" ::"v"(before[k]) : "memory");  // wait until the exchanges have been carried out
        const unsigned t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_block = (t == gridDim.x - 1);
        if (last_block)
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (!last_block)
        return;
    have = false;
    for (int k = tid; k < (int)gridDim.x; k += kThreads) {
        nbh_image img;
#pragma unroll
        for (int w = 0; w < kSlotWords; ++w)
            img.w[w] = __hip_atomic_load(&partials[(long long)k * kSlotWords + w], __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
        nbh_take(acc, have, img.value);
    }
    nbh_fold_workgroup(acc, have);
    if (tid == 0) {
        out[0] = nbh_op(acc, init);
        // leave the scratch buffer as the caller handed it over
        __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- the reference's order of association ---------------------------------------------
// nbh_custom_reduce_ordered: every application of the operation on the same pair of values,
// in the same order, as a run of the reference's kernels (kernels/reduction.py:22-166 launched
// as in :233-258) - for operations that are not associative, or whose rounding depends on the
// order.  With F = n rounded down to a multiple of 128 and G = min(F / 128, 64) blocks of 128
// threads, thread g < S = 128 G folds a[g], a[g + S], ... below F from left to right (:70-78);
// a warp of 32 is the tree (l, l + 16), (l, l + 8) ... (:22-41); a block is (w0 op w2) op
// (w1 op w3) (:88-97); block 0 takes `init` in (:163-164); the n - F values behind and the
// partials go through the one-block routine (:99-141, :256-258).
// One workgroup per warp of the reference: 32 chains whose items lie side by side in every
// row of S items.  All 512 lanes load rows of 32 items into one of two LDS buffers, a batch
// at a time, the next batch travelling while lanes 0 - 31 fold the parked one down their
// chains.  The buffers hold the rows of a chain side by side, so that a chain reads eight of
// its items with one or two wide LDS reads, and a batch is 512 rows of 4-byte items (2^28
// float32 with a - b: 382 us with one 4-byte read per row and batches of 128 rows, 354 us
// now; 8- and 16-byte items stay within 3 %); the row pitch, eight bytes more than a batch,
// spreads the scattered stores of a wavefront over the banks.  Warp results are published like the partials above; the workgroup that draws the
// last ticket does the small rest the way the reference's kernels do.
constexpr int kRefWarp = 32, kRefBlock = 128, kRefMaxGrid = 64;
constexpr int kOrdRows = (2048 / (int)sizeof(T)) > 512 ? 512 : (2048 / (int)sizeof(T));  // rows parked per batch
constexpr int kOrdLoads = kOrdRows * kRefWarp / kThreads;                                // loads per lane and batch
constexpr int kOrdPitch = kOrdRows + (sizeof(T) < 8 ? 8 / (int)sizeof(T) : 1);           // items per chain and buffer

// the reference's one-block routine (:99-141) over m <= 128 values, by one thread: a full warp
// that is not the last is a tree, the last warp a left fold, and so are the warps
__device__ T nbh_ref_one_block(const T *v, int m)
{
    const int nw = (m + kRefWarp - 1) / kRefWarp;
    T result = v[0];
    for (int w = 0; w < nw; ++w) {
        T wres;
        if ((w + 1) * kRefWarp < m) {
            T t[kRefWarp];
            for (int l = 0; l < kRefWarp; ++l)
                t[l] = v[w * kRefWarp + l];
            for (int width = kRefWarp / 2; width; width /= 2)
                for (int l = 0; l < width; ++l)
                    t[l] = nbh_op(t[l], t[l + width]);
            wres = t[0];
        } else {
            wres = v[w * kRefWarp];
            for (int i = 1; i < m - w * kRefWarp; ++i)
                wres = nbh_op(wres, v[w * kRefWarp + i]);
        }
        result = w == 0 ? wres : nbh_op(result, wres);
    }
    return result;
}

extern "C" __global__ __launch_bounds__(512) void nbh_custom_reduce_ordered(const char *__restrict__ in, long long n,
                                                                           long long stride, T init,
                                                                           T *__restrict__ out,
                                                                           nbh_u64 *__restrict__ partials,
                                                                           unsigned *__restrict__ ticket)
{
    __shared__ __attribute__((aligned(16))) T cols[2][kRefWarp][kOrdPitch];
    __shared__ T small[kRefBlock + 1 + kRefMaxGrid + 1];
    __shared__ bool last_block;
    const int tid = threadIdx.x;
    const long long full = (n / kRefBlock) * kRefBlock;
    long long ref_grid = full / kRefBlock;
    if (ref_grid > kRefMaxGrid)
        ref_grid = kRefMaxGrid;
    const long long S = ref_grid * kRefBlock;      // chains; 0 when n < 128
    const int warps = (int)(S / kRefWarp);         // = workgroups with chains

    if ((int)blockIdx.x < warps) {
        // each XCD (workgroups are dealt to the eight in turn) takes a run of neighbouring
        // warps: a contiguous piece of every row
        int warp = (int)blockIdx.x;
        if (warps % 8 == 0)
            warp = (warp % 8) * (warps / 8) + warp / 8;
        const long long c0 = (long long)warp * kRefWarp;
        const long long nrows = (full - c0 + S - 1) / S;   // items per chain, the same for the 32 of a warp
        const int chain = tid % kRefWarp, row0 = tid / kRefWarp;
        constexpr int kRowStep = kThreads / kRefWarp;
        T held[kOrdLoads];
        auto fetch = [&](long long first_row) {     // rows behind the last repeat the last: parked, never folded
#pragma unroll
            for (int k = 0; k < kOrdLoads; ++k) {
                long long r = first_row + row0 + k * kRowStep;
                r = r < nrows ? r : nrows - 1;
                held[k] = *reinterpret_cast<const T *>(in + (r * S + c0 + chain) * stride);
            }
        };
        T acc = T();
        const long long nb = (nrows + kOrdRows - 1) / kOrdRows;
        fetch(0);
        for (long long b = 0; b < nb; ++b) {
            const int buf = (int)(b & 1);
#pragma unroll
            for (int k = 0; k < kOrdLoads; ++k)
                cols[buf][chain][row0 + k * kRowStep] = held[k];
            // one barrier per batch: whoever parks into a buffer next has passed the barrier
            // that the folding lanes reached after reading it
            __syncthreads();
            if (b + 1 < nb)
                fetch((b + 1) * kOrdRows);
            if (tid < kRefWarp) {
                const long long left = nrows - b * kOrdRows;
                const int count = (int)(left < kOrdRows ? left : kOrdRows);
                const T *__restrict__ mine = cols[buf][tid];
                int r = 0;
                if (b == 0) {                       // a chain starts with its first value ...
                    acc = mine[0];
                    for (r = 1; r < 8 && r < count; ++r)   // ... and goes on in steps of eight items, aligned
                        acc = nbh_op(acc, mine[r]);
                }
                struct alignas(8) Eight { T v[8]; };         // a chain starts on an 8-byte boundary, eight items apart stay on one
                if (r + 8 <= count) {
                    Eight cur = *reinterpret_cast<const Eight *>(mine + r);
                    for (; r + 16 <= count; r += 8) {
                        const Eight next = *reinterpret_cast<const Eight *>(mine + r + 8);
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            acc = nbh_op(acc, cur.v[j]);
                        cur = next;
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        acc = nbh_op(acc, cur.v[j]);
                    r += 8;
                }
                for (; r < count; ++r)
                    acc = nbh_op(acc, mine[r]);
            }
        }
        if (tid < 64) {                             // the first wavefront, whole: the shuffles need its lanes
#pragma unroll
            for (int width = kRefWarp / 2; width; width /= 2) {
                const nbh_image mine = nbh_image_of(acc);
                nbh_image theirs;
#pragma unroll
                for (int w = 0; w < kSlotWords; ++w)
                    theirs.w[w] = __shfl_down(mine.w[w], width, 64);
                if (tid < width)
                    acc = nbh_op(acc, theirs.value);
            }
            if (tid == 0) {
                const nbh_image img = nbh_image_of(acc);
                nbh_u64 before[kSlotWords];
#pragma unroll
                for (int w = 0; w < kSlotWords; ++w)
                    before[w] = __hip_atomic_exchange(&partials[(long long)warp * kSlotWords + w], img.w[w],
                                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int w = 0; w < kSlotWords; ++w)
                    asm volatile("" ::"v"(before[w]) : "memory");  // carried out before the ticket is drawn
            }
        }
        __syncthreads();
    }
    if (gridDim.x > 1) {
        if (tid == 0) {
            const unsigned t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_block = (t == gridDim.x - 1);
            if (last_block)
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        __syncthreads();
        if (!last_block)
            return;
    }

    // the small rest: small[0 .. 127] the values behind `full`, small[129 ...] one value per block
    const int m_tail = (int)(n - full);
    T *tail = small, *part = small + kRefBlock + 1;
    if (tid < m_tail)
        tail[tid] = *reinterpret_cast<const T *>(in + (full + tid) * stride);
    if (tid < (int)ref_grid) {                      // block = (w0 op w2) op (w1 op w3)
        T w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            nbh_image img;
#pragma unroll
            for (int k = 0; k < kSlotWords; ++k)
                img.w[k] = __hip_atomic_load(&partials[((long long)tid * 4 + q) * kSlotWords + k], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
            w[q] = img.value;
        }
        part[tid] = nbh_op(nbh_op(w[0], w[2]), nbh_op(w[1], w[3]));
    }
    __syncthreads();
    if (tid == 0) {
        int np = (int)ref_grid;
        if (ref_grid)
            part[0] = nbh_op(part[0], init);
        if (m_tail) {
            part[np] = nbh_ref_one_block(tail, m_tail);
            if (!ref_grid)
                part[0] = nbh_op(part[0], init);
            ++np;
        }
        out[0] = np > 1 ? nbh_ref_one_block(part, np) : part[0];
        if (gridDim.x > 1)
            __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
)NBHSRC";

struct CustomOp {
    int dtype = 0;
    size_t elem = 0;
    std::vector<char> code;
    std::mutex lock;
    struct Loaded {
        hipModule_t module = nullptr;
        hipFunction_t reduce = nullptr, ordered = nullptr;
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
    if (!slot.reduce) {
        hipModule_t m = nullptr;
        NBH_TRY(hipModuleLoadData(&m, op->code.data()));
        hipFunction_t f = nullptr, g = nullptr;
        hipError_t e = hipModuleGetFunction(&f, m, "nbh_custom_reduce");
        if (e == hipSuccess)
            e = hipModuleGetFunction(&g, m, "nbh_custom_reduce_ordered");
        if (e != hipSuccess) {
            (void)hipModuleUnload(m);
            return (int)e;
        }
        slot.module = m;
        slot.reduce = f;
        slot.ordered = g;
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
    std::string source = kSource;
    source.replace(source.find("@T@"), 3, type);
    source.replace(source.find("@BODY@"), 6, body);

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
    const uintptr_t addr = (uintptr_t)in;
    if (addr % op->elem != 0 || ((uintptr_t)out) % op->elem != 0)
        return (int)hipErrorInvalidValue;
    const int packed = (in_stride == (int64_t)op->elem || n == 1) ? 1 : 0;
    long long head = 0, units = n;  // units: packets when packed, items otherwise
    if (packed) {
        head = (long long)(((16 - (addr % 16)) % 16) / op->elem);
        if (head > n)
            head = n;
        units = (n - head) / items;
    }
    // as many workgroups as nbh_reduce would start, then no more than have a slice each
    const int64_t per_block = (int64_t)kBlock * kUnroll;
    int64_t grid = (units + per_block - 1) / per_block;
    if (grid < 32) {
        grid = (units + kBlock - 1) / kBlock;
        if (grid > 32)
            grid = 32;
    }
    int64_t cap = (int64_t)nbh_cu_count() * kGridPerCU;
    if (cap > kMaxGrid)
        cap = kMaxGrid;
    if (grid > cap)
        grid = cap;
    if (grid < 1)
        grid = 1;
    if (units > 0) {
        const int64_t per = (units + grid - 1) / grid;
        grid = (units + per - 1) / per;  // every workgroup's slice holds at least one unit
    }

    const char *in_arg = static_cast<const char *>(in);
    long long n_arg = n, stride_arg = in_stride;
    // from sixteen pieces per workgroup on, the pieces are dealt out (as in nbh_reduce)
    int packed_arg = (packed && units / kPiecePackets >= 16 * grid) ? 2 : packed;
    uint64_t *partials = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kHeaderBytes);
    unsigned *ticket = reinterpret_cast<unsigned *>(scratch);
    // `init` travels as a kernel argument: the launch copies the element it points to
    void *args[] = {&in_arg, &n_arg, &head, &units, &stride_arg, &packed_arg, const_cast<void *>(init),
                    &out, &partials, &ticket};
    NBH_TRY(hipModuleLaunchKernel(fn->reduce, (unsigned)grid, 1, 1, kBlock, 1, 1, 0, s, args, nullptr));
    return 0;
}

extern "C" int nbh_reduce_custom_ordered(void *handle, const void *in, int64_t n, int64_t in_stride, const void *init,
                                         void *out, void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    CustomOp *op = static_cast<CustomOp *>(handle);
    if (!op || !in || !init || !out || !scratch || n < 1 || scratch_bytes < kNeededBytes ||
        ((uintptr_t)scratch) % 8 != 0 || in_stride % (int64_t)op->elem != 0)
        return (int)hipErrorInvalidValue;
    if (((uintptr_t)in) % op->elem != 0 || ((uintptr_t)out) % op->elem != 0)
        return (int)hipErrorInvalidValue;
    CustomOp::Loaded *fn = nullptr;
    const int rc = functions_for(op, &fn);
    if (rc)
        return rc;
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);

    // one workgroup per warp of the reference's launch (at most 64 blocks of four warps)
    int64_t ref_grid = n / 128;
    if (ref_grid > 64)
        ref_grid = 64;
    const int64_t grid = ref_grid ? ref_grid * 4 : 1;
    const char *in_arg = static_cast<const char *>(in);
    long long n_arg = n, stride_arg = in_stride;
    uint64_t *partials = reinterpret_cast<uint64_t *>(static_cast<char *>(scratch) + kHeaderBytes);
    unsigned *ticket = reinterpret_cast<unsigned *>(scratch);
    void *args[] = {&in_arg, &n_arg, &stride_arg, const_cast<void *>(init), &out, &partials, &ticket};
    NBH_TRY(hipModuleLaunchKernel(fn->ordered, (unsigned)grid, 1, 1, kBlock, 1, 1, 0, s, args, nullptr));
    return 0;
}

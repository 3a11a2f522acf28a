// nbh_assign: dst[i0, ..., ik] = src[i0, ..., ik] over an n-d index space, with
// arbitrary byte strides on both sides (a zero source stride broadcasts).
//
// The host first squeezes the index space: axes of length 1 vanish and neighbouring
// axes that are laid out back to back on both sides fuse.  What is left decides
// the kernel:
//   * one axis with unit stride on both sides -> a flat copy: one wavefront per
//     workgroup and one 16-byte packet per lane (1 KiB per workgroup), non-temporal on
//     both sides; packets start at the first 128-byte line of the destination, the bytes
//     in front of it and behind the last packet are done chunk by chunk.  Measured on
//     MI355X, 2^28 float32, TB/s: a fixed grid looping grid-stride with cached
//     accesses 4.80, non-temporal 5.03, a fixed grid looping over contiguous slices
//     5.5, one workgroup of 256 lanes per 16 KiB 6.3, per 4 KiB 6.6, one wavefront per
//     1 KiB 6.7 (hipMemcpyDtoD: 5.2)
//   * two axes, the inner one with unit stride on both sides (a block of a pitched
//     matrix, `d[10:1000, 20:4000] = s`) -> every row is a run of bytes moved in 16-byte
//     packets that need only the alignment the rows have; a workgroup is TY rows x TX
//     lanes, TX sized to the row length, so short rows do not idle lanes.  Measured,
//     16384 x 16000 float32 out of a 16384-wide matrix: 2.6 TB/s with one lane per item,
//     6.2 TB/s this way (5.4 when rows start off the 16-byte grid)
//   * anything else -> one lane per chunk of an item, innermost axis fastest; an inner
//     axis with unit strides is re-cut into the widest chunks its rows are aligned to
//
// nbh_fill: dst[...] = value for one item of 1, 2, 4, 8 or 16 bytes passed by value -
// what `darr[key] = scalar` needs, without the device allocation and host-to-device
// copy that a source array would cost (60 -> 15 us for one element) and at the speed of
// a pure write for a whole array.
//
// HBM roofline of the flat copy: bytes read + bytes written = 2 * n * itemsize.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxDims = NBH_ASSIGN_MAX_NDIM;

struct alignas(16) Chunk16 {
    uint32_t w[4];
};
template <int G> struct ChunkOf;
template <> struct ChunkOf<1> { using type = uint8_t; };
template <> struct ChunkOf<2> { using type = uint16_t; };
template <> struct ChunkOf<4> { using type = uint32_t; };
template <> struct ChunkOf<8> { using type = uint64_t; };
template <> struct ChunkOf<16> { using type = Chunk16; };

typedef nbh_u32x4 u32x4;

// Streaming kernels do best here with the smallest workgroups: one wavefront, one 16-byte
// packet per lane, 1 KiB per workgroup, in launch order (2^28 float32 copied, TB/s: 256 lanes x 4
// packets 6.1-6.3, 256 x 2 6.0, 256 x 1 6.6, 64 x 1 6.7-6.8; filled: 256 x 16 4.9, x 4 5.9, x 1 6.6,
// 64 x 1 4.8).
constexpr int kFlatThreads = 64;

template <int G>
__global__ __launch_bounds__(kFlatThreads) void copy_flat(char *__restrict__ dst, const char *__restrict__ src,
                                                          int64_t nbytes, int64_t head)
{
    const int64_t npack = (nbytes - head) / 16;
    const char *__restrict__ from = src + head;  // packets: G-aligned here,
    char *__restrict__ to = dst + head;           // 128-byte aligned here
    const int64_t p = (int64_t)blockIdx.x * kFlatThreads + threadIdx.x;
    if (p < npack)
        nbh_store16<16, true>(to + p * 16, nbh_load16<G, true>(from + p * 16));

    if (blockIdx.x == 0) {  // fewer than 128 + 16 bytes in all
        using C = typename ChunkOf<G>::type;
        for (int64_t b = (int64_t)threadIdx.x * G; b < head; b += (int64_t)kFlatThreads * G)
            *reinterpret_cast<C *>(dst + b) = *reinterpret_cast<const C *>(src + b);
        for (int64_t b = head + npack * 16 + (int64_t)threadIdx.x * G; b < nbytes; b += (int64_t)kFlatThreads * G)
            *reinterpret_cast<C *>(dst + b) = *reinterpret_cast<const C *>(src + b);
    }
}

// Rows of `run` bytes, `rows` of them, row r at dst + r * dst_pitch / src + r * src_pitch.
// tx_log2: lanes along a row per workgroup = 1 << tx_log2; segs: workgroups along a row.
constexpr int kRowsInFlight = 1;  // packets per lane (16384 x 16000 float32 block: 4 -> 6.2 TB/s, 2 -> 6.0, 1 -> 6.6)

template <int G, bool NT>
__global__ __launch_bounds__(kThreads) void copy_rows(char *__restrict__ dst, const char *__restrict__ src,
                                                      int64_t rows, int64_t run, int64_t dst_pitch,
                                                      int64_t src_pitch, int tx_log2, int64_t segs)
{
    constexpr int kInFlight = kRowsInFlight;
    const int tx_count = 1 << tx_log2;
    const int tx = threadIdx.x & (tx_count - 1), ty = threadIdx.x >> tx_log2;
    const int64_t seg = (int64_t)blockIdx.x % segs;
    const int64_t row = ((int64_t)blockIdx.x / segs) * (kThreads >> tx_log2) + ty;
    if (row >= rows)
        return;
    const char *__restrict__ from = src + row * src_pitch;
    char *__restrict__ to = dst + row * dst_pitch;
    const int64_t npack = run / 16;
    const int64_t p0 = seg * ((int64_t)tx_count * kInFlight) + tx;
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
        const int64_t p = p0 + (int64_t)u * tx_count;
        if (p < npack)
            v[u] = nbh_load16<G, NT>(from + p * 16);
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
        const int64_t p = p0 + (int64_t)u * tx_count;
        if (p < npack)
            nbh_store16<G, NT>(to + p * 16, v[u]);
    }
    if (seg == segs - 1) {  // fewer than 16 bytes behind the last packet
        using C = typename ChunkOf<G>::type;
        for (int64_t b = npack * 16 + (int64_t)tx * G; b < run; b += (int64_t)tx_count * G)
            *reinterpret_cast<C *>(to + b) = *reinterpret_cast<const C *>(from + b);
    }
}

struct Dims {
    int nd;
    int64_t shape[kMaxDims];
    int64_t dst_stride[kMaxDims];
    int64_t src_stride[kMaxDims];
};

template <int G>
__global__ __launch_bounds__(kThreads) void copy_strided(char *__restrict__ dst, const char *__restrict__ src,
                                                         Dims d, int64_t chunks, int64_t total)
{
    using C = typename ChunkOf<G>::type;
    const int64_t step = (int64_t)gridDim.x * kThreads;
    for (int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x; id < total; id += step) {
        int64_t rest = id / chunks;
        int64_t doff = (id % chunks) * G, soff = doff;
        for (int k = d.nd - 1; k >= 0; --k) {
            const int64_t i = rest % d.shape[k];
            rest /= d.shape[k];
            doff += i * d.dst_stride[k];
            soff += i * d.src_stride[k];
        }
        *reinterpret_cast<C *>(dst + doff) = *reinterpret_cast<const C *>(src + soff);
    }
}

// ---- filling with one value -------------------------------------------------------------
// `pattern` is the item repeated to 16 bytes (item sizes 1, 2, 4, 8, 16), rotated so that
// it is right at every 16-byte boundary of the destination.

// (a pure write is limited by the rate at which workgroups start before one wavefront per
// workgroup pays: four wavefronts, one packet per lane, 4 KiB per workgroup)
template <int G>
__global__ __launch_bounds__(kThreads) void fill_flat(char *__restrict__ dst, int64_t nbytes, int64_t head,
                                                          u32x4 pattern, u32x4 unrotated)
{
    const int64_t npack = (nbytes - head) / 16;
    char *__restrict__ to = dst + head;  // 128-byte aligned
    // Consecutive workgroups start on different XCDs (workgroup b on XCD b % 8).  Within every
    // whole group of 512 workgroups XCD k writes pieces 64 k ... 64 k + 63, 256 KiB in a row,
    // instead of every eighth piece (a pure write of 4 GiB: 6.5 - 6.8 -> 7.0 TB/s; runs of 2 to
    // 16 pieces are slower than no runs at all, down to 5.7 TB/s at 8).
    int64_t piece = blockIdx.x;
    if (piece < (int64_t)(gridDim.x / 512) * 512) {
        const int64_t r = piece % 512;
        piece += (r % 8) * 64 + r / 8 - r;
    }
    const int64_t p = piece * kThreads + threadIdx.x;
    if (p < npack)
        nbh_store16<16, true>(to + p * 16, pattern);
    if (blockIdx.x == 0) {  // in front of the first line and behind the last packet
        using C = typename ChunkOf<G>::type;
        union {
            u32x4 v;
            C c[16 / G];
        } a, b;
        a.v = unrotated;  // bytes of dst[0:16]
        b.v = pattern;    // bytes of dst[head + 16 k : ...]
        for (int64_t off = (int64_t)threadIdx.x * G; off < head; off += (int64_t)kThreads * G)
            *reinterpret_cast<C *>(dst + off) = a.c[(off % 16) / G];
        const int64_t tail = head + npack * 16;
        for (int64_t off = tail + (int64_t)threadIdx.x * G; off < nbytes; off += (int64_t)kThreads * G)
            *reinterpret_cast<C *>(dst + off) = b.c[((off - head) % 16) / G];
    }
}

// One lane per G-byte chunk of one item, innermost axis fastest.
template <int G>
__global__ __launch_bounds__(kThreads) void fill_strided(char *__restrict__ dst, Dims d, int64_t chunks,
                                                         int64_t total, u32x4 item16)
{
    using C = typename ChunkOf<G>::type;
    union {
        u32x4 v;
        C c[16 / G];
    } value;
    value.v = item16;  // the item itself in the first `chunks` chunks
    const int64_t step = (int64_t)gridDim.x * kThreads;
    for (int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x; id < total; id += step) {
        int64_t rest = id / chunks;
        const int64_t u = id % chunks;
        int64_t off = u * G;
        for (int k = d.nd - 1; k >= 0; --k) {
            off += (rest % d.shape[k]) * d.dst_stride[k];
            rest /= d.shape[k];
        }
        *reinterpret_cast<C *>(dst + off) = value.c[u];
    }
}

inline int64_t low_bit(uint64_t x) { return (int64_t)(x & (~x + 1)); }

template <int G> int launch_flat(void *dst, const void *src, int64_t nbytes, hipStream_t s)
{
    // bytes in front of the destination's first 128-byte line (a multiple of G)
    int64_t head = (int64_t)((128 - (uintptr_t)dst % 128) % 128);
    if (head > nbytes)
        head = nbytes;
    int64_t grid = ((nbytes - head) / 16 + kFlatThreads - 1) / kFlatThreads;
    if (grid < 1)
        grid = 1;
    if (grid > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((copy_flat<G>), dim3((unsigned)grid), dim3(kFlatThreads), 0, s, (char *)dst, (const char *)src,
                       nbytes, head);
    return nbh_launch_status();
}

template <int G>
int launch_rows(void *dst, const void *src, int64_t rows, int64_t run, int64_t dst_pitch, int64_t src_pitch,
                hipStream_t s)
{
    const int64_t npack = run / 16;
    int tx_log2 = 0;
    while (tx_log2 < 8 && (1 << tx_log2) < npack)
        ++tx_log2;
    const int64_t per_seg = (int64_t)(1 << tx_log2) * kRowsInFlight;
    int64_t segs = (npack + per_seg - 1) / per_seg;
    if (segs < 1)
        segs = 1;
    const int64_t ty_count = kThreads >> tx_log2;
    const int64_t grid = segs * ((rows + ty_count - 1) / ty_count);
    if (grid > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    // past the caches only when every row starts and ends on a 128-byte line
    const uint64_t mix = (uint64_t)(uintptr_t)dst | (uint64_t)(uintptr_t)src | (uint64_t)dst_pitch |
                         (uint64_t)src_pitch | (uint64_t)run;
    if (mix % 128 == 0)
        hipLaunchKernelGGL((copy_rows<G, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, (char *)dst,
                           (const char *)src, rows, run, dst_pitch, src_pitch, tx_log2, segs);
    else
        hipLaunchKernelGGL((copy_rows<G, false>), dim3((unsigned)grid), dim3(kThreads), 0, s, (char *)dst,
                           (const char *)src, rows, run, dst_pitch, src_pitch, tx_log2, segs);
    return nbh_launch_status();
}

template <int G>
int launch_strided(void *dst, const void *src, const Dims &d, int64_t itemsize, int64_t items, hipStream_t s)
{
    const int64_t chunks = itemsize / G;
    const int64_t total = items * chunks;
    int64_t grid = (total + kThreads - 1) / kThreads;
    const int64_t cap = (int64_t)nbh_cu_count() * 32;
    if (grid > cap)
        grid = cap;
    hipLaunchKernelGGL((copy_strided<G>), dim3((unsigned)grid), dim3(kThreads), 0, s, (char *)dst,
                       (const char *)src, d, chunks, total);
    return nbh_launch_status();
}

template <int G> int launch_fill_flat(void *dst, int64_t nbytes, int64_t itemsize, const unsigned char *item, hipStream_t s)
{
    int64_t head = (int64_t)((128 - (uintptr_t)dst % 128) % 128);
    if (head > nbytes)
        head = nbytes;
    union {
        u32x4 v;
        unsigned char b[16];
    } plain, rotated;
    for (int k = 0; k < 16; ++k) {
        plain.b[k] = item[k % itemsize];
        rotated.b[k] = item[(head + k) % itemsize];
    }
    int64_t grid = ((nbytes - head) / 16 + kThreads - 1) / kThreads;
    if (grid < 1)
        grid = 1;
    if (grid > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((fill_flat<G>), dim3((unsigned)grid), dim3(kThreads), 0, s, (char *)dst, nbytes, head,
                       rotated.v, plain.v);
    return nbh_launch_status();
}

template <int G>
int launch_fill_strided(void *dst, const Dims &d, int64_t itemsize, int64_t items, const unsigned char *item,
                        hipStream_t s)
{
    union {
        u32x4 v;
        unsigned char b[16];
    } value = {};
    for (int k = 0; k < itemsize; ++k)
        value.b[k] = item[k];
    const int64_t chunks = itemsize / G;
    const int64_t total = items * chunks;
    int64_t grid = (total + kThreads - 1) / kThreads;
    const int64_t cap = (int64_t)nbh_cu_count() * 32;
    if (grid > cap)
        grid = cap;
    hipLaunchKernelGGL((fill_strided<G>), dim3((unsigned)grid), dim3(kThreads), 0, s, (char *)dst, d, chunks, total,
                       value.v);
    return nbh_launch_status();
}

}  // namespace

int nbh_flat_copy(void *dst, const void *src, int64_t nbytes, hipStream_t stream)
{
    nbh_stream_report report(stream);
    const uint64_t mix = (uint64_t)(uintptr_t)dst | (uint64_t)(uintptr_t)src | (uint64_t)nbytes | 16u;
    switch (low_bit(mix)) {
    case 1: return launch_flat<1>(dst, src, nbytes, stream);
    case 2: return launch_flat<2>(dst, src, nbytes, stream);
    case 4: return launch_flat<4>(dst, src, nbytes, stream);
    case 8: return launch_flat<8>(dst, src, nbytes, stream);
    default: return launch_flat<16>(dst, src, nbytes, stream);
    }
}

extern "C" int nbh_fill(void *dst, int ndim, const int64_t *shape, const int64_t *dst_strides, int64_t itemsize,
                        const void *value, nbh_stream_t stream)
{
    const bool size_ok = itemsize == 1 || itemsize == 2 || itemsize == 4 || itemsize == 8 || itemsize == 16;
    if (ndim < 0 || ndim > kMaxDims || !size_ok || !value || (ndim > 0 && (!shape || !dst_strides)))
        return (int)hipErrorInvalidValue;
    int64_t items = 1;
    for (int k = 0; k < ndim; ++k) {
        if (shape[k] < 0)
            return (int)hipErrorInvalidValue;
        items *= shape[k];
    }
    if (items == 0)
        return 0;
    if (!dst)
        return (int)hipErrorInvalidValue;
    Dims d;
    d.nd = 0;
    for (int k = 0; k < ndim; ++k) {  // drop unit axes, fuse axes that continue each other
        if (shape[k] == 1)
            continue;
        if (d.nd > 0 && d.dst_stride[d.nd - 1] == dst_strides[k] * shape[k]) {
            d.shape[d.nd - 1] *= shape[k];
            d.dst_stride[d.nd - 1] = dst_strides[k];
        } else {
            d.shape[d.nd] = shape[k];
            d.dst_stride[d.nd] = dst_strides[k];
            d.src_stride[d.nd] = 0;
            ++d.nd;
        }
    }
    for (int k = d.nd; k < kMaxDims; ++k) {
        d.shape[k] = 1;
        d.dst_stride[k] = d.src_stride[k] = 0;
    }
    uint64_t mix = (uint64_t)itemsize | (uint64_t)(uintptr_t)dst | 16u;
    for (int k = 0; k < d.nd; ++k)
        mix |= (uint64_t)d.dst_stride[k];
    const int64_t g = low_bit(mix);
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);
    const unsigned char *item = static_cast<const unsigned char *>(value);
    const bool flat = d.nd == 0 || (d.nd == 1 && d.dst_stride[0] == itemsize);
    if (flat) {
        const int64_t nbytes = items * itemsize;
        switch (g) {
        case 1: return launch_fill_flat<1>(dst, nbytes, itemsize, item, s);
        case 2: return launch_fill_flat<2>(dst, nbytes, itemsize, item, s);
        case 4: return launch_fill_flat<4>(dst, nbytes, itemsize, item, s);
        case 8: return launch_fill_flat<8>(dst, nbytes, itemsize, item, s);
        default: return launch_fill_flat<16>(dst, nbytes, itemsize, item, s);
        }
    }
    switch (g) {
    case 1: return launch_fill_strided<1>(dst, d, itemsize, items, item, s);
    case 2: return launch_fill_strided<2>(dst, d, itemsize, items, item, s);
    case 4: return launch_fill_strided<4>(dst, d, itemsize, items, item, s);
    case 8: return launch_fill_strided<8>(dst, d, itemsize, items, item, s);
    default: return launch_fill_strided<16>(dst, d, itemsize, items, item, s);
    }
}

extern "C" int nbh_assign(void *dst, const void *src, int ndim, const int64_t *shape, const int64_t *dst_strides,
                          const int64_t *src_strides, int64_t itemsize, nbh_stream_t stream)
{
    if (ndim < 0 || ndim > kMaxDims || itemsize < 1 || (ndim > 0 && (!shape || !dst_strides || !src_strides)))
        return (int)hipErrorInvalidValue;
    int64_t items = 1;
    for (int k = 0; k < ndim; ++k) {
        if (shape[k] < 0)
            return (int)hipErrorInvalidValue;
        items *= shape[k];
    }
    if (items == 0)
        return 0;
    if (!dst || !src)
        return (int)hipErrorInvalidValue;

    // squeeze: drop unit axes, fuse axes that continue each other on both sides
    Dims d;
    d.nd = 0;
    for (int k = 0; k < ndim; ++k) {
        if (shape[k] == 1)
            continue;
        if (d.nd > 0 && d.dst_stride[d.nd - 1] == dst_strides[k] * shape[k] &&
            d.src_stride[d.nd - 1] == src_strides[k] * shape[k]) {
            d.shape[d.nd - 1] *= shape[k];
            d.dst_stride[d.nd - 1] = dst_strides[k];
            d.src_stride[d.nd - 1] = src_strides[k];
        } else {
            d.shape[d.nd] = shape[k];
            d.dst_stride[d.nd] = dst_strides[k];
            d.src_stride[d.nd] = src_strides[k];
            ++d.nd;
        }
    }
    for (int k = d.nd; k < kMaxDims; ++k) {
        d.shape[k] = 1;
        d.dst_stride[k] = d.src_stride[k] = 0;
    }

    uint64_t mix = (uint64_t)itemsize | (uint64_t)(uintptr_t)dst | (uint64_t)(uintptr_t)src | 16u;
    for (int k = 0; k < d.nd; ++k)
        mix |= (uint64_t)d.dst_stride[k] | (uint64_t)d.src_stride[k];
    const int64_t g = low_bit(mix);
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);

    const bool flat = d.nd == 0 || (d.nd == 1 && d.dst_stride[0] == itemsize && d.src_stride[0] == itemsize);
    if (flat) {
        const int64_t nbytes = items * itemsize;
        switch (g) {
        case 1: return launch_flat<1>(dst, src, nbytes, s);
        case 2: return launch_flat<2>(dst, src, nbytes, s);
        case 4: return launch_flat<4>(dst, src, nbytes, s);
        case 8: return launch_flat<8>(dst, src, nbytes, s);
        default: return launch_flat<16>(dst, src, nbytes, s);
        }
    }
    // inner axis with unit strides: a run of bytes, whatever the items are
    if (d.nd >= 2 && d.dst_stride[d.nd - 1] == itemsize && d.src_stride[d.nd - 1] == itemsize) {
        const int64_t run = d.shape[d.nd - 1] * itemsize;
        uint64_t rmix = (uint64_t)run | (uint64_t)(uintptr_t)dst | (uint64_t)(uintptr_t)src | 16u;
        for (int k = 0; k + 1 < d.nd; ++k)
            rmix |= (uint64_t)d.dst_stride[k] | (uint64_t)d.src_stride[k];
        const int64_t rg = low_bit(rmix);
        if (d.nd == 2) {
            const int64_t rows = d.shape[0], dp = d.dst_stride[0], sp = d.src_stride[0];
            switch (rg) {
            case 1: return launch_rows<1>(dst, src, rows, run, dp, sp, s);
            case 2: return launch_rows<2>(dst, src, rows, run, dp, sp, s);
            case 4: return launch_rows<4>(dst, src, rows, run, dp, sp, s);
            case 8: return launch_rows<8>(dst, src, rows, run, dp, sp, s);
            default: return launch_rows<16>(dst, src, rows, run, dp, sp, s);
            }
        }
        // more axes: same lanes-per-chunk kernel, but with chunks as wide as the rows allow
        d.shape[d.nd - 1] = run / rg;
        d.dst_stride[d.nd - 1] = d.src_stride[d.nd - 1] = rg;
        const int64_t chunks_total = items * itemsize / rg;
        switch (rg) {
        case 1: return launch_strided<1>(dst, src, d, 1, chunks_total, s);
        case 2: return launch_strided<2>(dst, src, d, 2, chunks_total, s);
        case 4: return launch_strided<4>(dst, src, d, 4, chunks_total, s);
        case 8: return launch_strided<8>(dst, src, d, 8, chunks_total, s);
        default: return launch_strided<16>(dst, src, d, 16, chunks_total, s);
        }
    }
    switch (g) {
    case 1: return launch_strided<1>(dst, src, d, itemsize, items, s);
    case 2: return launch_strided<2>(dst, src, d, itemsize, items, s);
    case 4: return launch_strided<4>(dst, src, d, itemsize, items, s);
    case 8: return launch_strided<8>(dst, src, d, itemsize, items, s);
    default: return launch_strided<16>(dst, src, d, itemsize, items, s);
    }
}

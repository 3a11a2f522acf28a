// nbh_transpose: out[j, i] = in[i, j] for items of any size and any byte strides.
//
// Two kernels:
//   * tiled  - item size 1, 2, 4, 8 or 16 bytes with unit inner stride on both
//              sides (row strides free).  A workgroup moves one tile whose rows
//              are 256 bytes long on the input side and on the output side: it
//              reads the tile with 128-bit loads along input rows, parks it in
//              LDS (row pitch padded by one item against bank conflicts), and
//              writes it with 128-bit stores along output rows.  Ragged edge
//              tiles fall back to per-item accesses only for the vectors that
//              stick out.
//   * strided - everything else (records such as 28-byte items, element strides,
//              negative strides): one lane per (item, chunk) with the output
//              index fastest, so writes stay as dense as the layout allows.
//
// HBM roofline: every item is read once and written once, 2*rows*cols*itemsize.
#include "common.h"

namespace {

constexpr int kThreads = 256;

struct alignas(16) Item16 {
    uint32_t w[4];
};
template <int E> struct ItemOf;
template <> struct ItemOf<1> { using type = uint8_t; };
template <> struct ItemOf<2> { using type = uint16_t; };
template <> struct ItemOf<4> { using type = uint32_t; };
template <> struct ItemOf<8> { using type = uint64_t; };
template <> struct ItemOf<16> { using type = Item16; };

// A 16-byte packet of items that is only guaranteed the alignment of one item.
// Global memory accepts such accesses; the compiler still emits one dwordx4.
template <int E> struct __attribute__((packed, aligned(E))) Packet {
    typename ItemOf<E>::type item[16 / E];
};

// Tile edge in items: 256-byte rows on both sides, capped so the tile fits LDS
// comfortably for the narrow item sizes.
template <int E> struct TileOf {
    static constexpr int edge = (E == 1) ? 128 : (256 / E);
};

template <int E>
__global__ __launch_bounds__(kThreads) void transpose_tiled(const char *__restrict__ in, char *__restrict__ out,
                                                             int64_t rows, int64_t cols, int64_t in_s0,
                                                             int64_t out_s0, int64_t tiles_c)
{
    using Item = typename ItemOf<E>::type;
    using Pack = Packet<E>;
    constexpr int V = 16 / E;            // items per 128-bit access
    constexpr int T = TileOf<E>::edge;   // tile is T x T items
    constexpr int PPR = T / V;           // packets per tile row
    __shared__ Item tile[T][T + 1];

    const int tid = threadIdx.x;
    const int64_t tile_r = (int64_t)blockIdx.x / tiles_c;
    const int64_t tile_c = (int64_t)blockIdx.x % tiles_c;
    const int64_t r0 = tile_r * T;
    const int64_t c0 = tile_c * T;

    // in[r0 + r, c0 + p*V ... + V)  ->  tile[r][p*V ...]
#pragma unroll 4
    for (int idx = tid; idx < T * PPR; idx += kThreads) {
        const int r = idx / PPR;
        const int p = idx % PPR;
        const int64_t gr = r0 + r;
        const int64_t gc = c0 + (int64_t)p * V;
        if (gr < rows) {
            const char *src = in + gr * in_s0 + gc * E;
            if (gc + V <= cols) {
                Pack v = *reinterpret_cast<const Pack *>(src);
#pragma unroll
                for (int j = 0; j < V; ++j)
                    tile[r][p * V + j] = v.item[j];
            } else {
                for (int j = 0; j < V; ++j)
                    if (gc + j < cols)
                        tile[r][p * V + j] = *reinterpret_cast<const Item *>(src + (int64_t)j * E);
            }
        }
    }
    __syncthreads();

    // tile[p*V ...][c]  ->  out[c0 + c, r0 + p*V ... + V)
#pragma unroll 4
    for (int idx = tid; idx < T * PPR; idx += kThreads) {
        const int c = idx / PPR;
        const int p = idx % PPR;
        const int64_t gc = c0 + c;              // output row
        const int64_t gr = r0 + (int64_t)p * V;  // first output column
        if (gc < cols) {
            char *dst = out + gc * out_s0 + gr * E;
            if (gr + V <= rows) {
                Pack v;
#pragma unroll
                for (int j = 0; j < V; ++j)
                    v.item[j] = tile[p * V + j][c];
                *reinterpret_cast<Pack *>(dst) = v;
            } else {
                for (int j = 0; j < V; ++j)
                    if (gr + j < rows)
                        *reinterpret_cast<Item *>(dst + (int64_t)j * E) = tile[p * V + j][c];
            }
        }
    }
}

// One lane per G-byte chunk of one item; chunk index fastest, then the output's
// inner index, then its outer index.
template <int G>
__global__ __launch_bounds__(kThreads) void transpose_strided(const char *__restrict__ in, char *__restrict__ out,
                                                               int64_t rows, int64_t cols, int64_t in_s0,
                                                               int64_t in_s1, int64_t out_s0, int64_t out_s1,
                                                               int64_t chunks, int64_t total)
{
    using Chunk = typename ItemOf<G>::type;
    const int64_t step = (int64_t)gridDim.x * kThreads;
    for (int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x; id < total; id += step) {
        const int64_t u = id % chunks;
        const int64_t e = id / chunks;
        const int64_t i = e % rows;  // input row    = output column
        const int64_t j = e / rows;  // input column = output row
        const Chunk v = *reinterpret_cast<const Chunk *>(in + i * in_s0 + j * in_s1 + u * G);
        *reinterpret_cast<Chunk *>(out + j * out_s0 + i * out_s1 + u * G) = v;
    }
}

template <int E>
int launch_tiled(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
                 hipStream_t stream)
{
    constexpr int T = TileOf<E>::edge;
    const int64_t tiles_r = (rows + T - 1) / T;
    const int64_t tiles_c = (cols + T - 1) / T;
    const int64_t tiles = tiles_r * tiles_c;
    if (tiles > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((transpose_tiled<E>), dim3((unsigned)tiles), dim3(kThreads), 0, stream, (const char *)in,
                       (char *)out, rows, cols, in_s0, out_s0, tiles_c);
    return nbh_launch_status();
}

template <int G>
int launch_strided(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t in_s1,
                   int64_t out_s0, int64_t out_s1, int64_t itemsize, hipStream_t stream)
{
    const int64_t chunks = itemsize / G;
    const int64_t total = rows * cols * chunks;
    int64_t grid = (total + kThreads - 1) / kThreads;
    const int64_t cap = (int64_t)nbh_cu_count() * 32;
    if (grid > cap)
        grid = cap;
    hipLaunchKernelGGL((transpose_strided<G>), dim3((unsigned)grid), dim3(kThreads), 0, stream, (const char *)in,
                       (char *)out, rows, cols, in_s0, in_s1, out_s0, out_s1, chunks, total);
    return nbh_launch_status();
}

inline int64_t low_bit(uint64_t x) { return (int64_t)(x & (~x + 1)); }

}  // namespace

extern "C" int nbh_transpose(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t in_s1,
                             int64_t out_s0, int64_t out_s1, int64_t itemsize, nbh_stream_t stream)
{
    if (rows < 0 || cols < 0 || itemsize < 1)
        return (int)hipErrorInvalidValue;
    if (rows == 0 || cols == 0)
        return 0;
    if (!in || !out)
        return (int)hipErrorInvalidValue;
    hipStream_t s = nbh_hip_stream(stream);

    // largest power of two (<= 16) that divides the item size, every stride and
    // both base addresses: the widest access that is aligned everywhere
    uint64_t mix = (uint64_t)itemsize | (uint64_t)in_s0 | (uint64_t)in_s1 | (uint64_t)out_s0 | (uint64_t)out_s1 |
                   (uint64_t)(uintptr_t)in | (uint64_t)(uintptr_t)out | 16u;
    const int64_t g = low_bit(mix);

    const bool unit_inner = in_s1 == itemsize && out_s1 == itemsize && in_s0 > 0 && out_s0 > 0;
    if (unit_inner && g == itemsize) {  // item size is a power of two <= 16 and items are aligned
        switch (itemsize) {
        case 1: return launch_tiled<1>(in, out, rows, cols, in_s0, out_s0, s);
        case 2: return launch_tiled<2>(in, out, rows, cols, in_s0, out_s0, s);
        case 4: return launch_tiled<4>(in, out, rows, cols, in_s0, out_s0, s);
        case 8: return launch_tiled<8>(in, out, rows, cols, in_s0, out_s0, s);
        case 16: return launch_tiled<16>(in, out, rows, cols, in_s0, out_s0, s);
        default: break;
        }
    }
    switch (g) {
    case 1: return launch_strided<1>(in, out, rows, cols, in_s0, in_s1, out_s0, out_s1, itemsize, s);
    case 2: return launch_strided<2>(in, out, rows, cols, in_s0, in_s1, out_s0, out_s1, itemsize, s);
    case 4: return launch_strided<4>(in, out, rows, cols, in_s0, in_s1, out_s0, out_s1, itemsize, s);
    case 8: return launch_strided<8>(in, out, rows, cols, in_s0, in_s1, out_s0, out_s1, itemsize, s);
    default: return launch_strided<16>(in, out, rows, cols, in_s0, in_s1, out_s0, out_s1, itemsize, s);
    }
}

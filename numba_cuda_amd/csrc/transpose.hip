// nbh_transpose: out[j, i] = in[i, j] for items of any size and any byte strides.
//
// Four kernels:
//   * packets - item size 1, 2, 4, 8 or 16 bytes with unit inner stride on both
//               sides (row strides free).  Every lane moves V x V items, V = 16 /
//               itemsize: it loads one 16-byte packet from each of V consecutive
//               input rows, transposes the V x V block in registers, and stores one
//               packet to each of V consecutive output rows.  The 64 lanes of a
//               wavefront form an 8 x 8 grid, so each load and each store
//               instruction covers eight whole 128-byte lines: no LDS, no barrier.
//               A workgroup covers a tall tile (many input rows, few columns) and
//               consecutive workgroups walk DOWN the input, i.e. ALONG the output
//               rows: what is in flight at any time writes long contiguous runs.
//               Measured on MI355X (float32 16384^2): square 64x64 tiles in
//               column-fastest order 4.5 TB/s whether staged through LDS or
//               registers; row-fastest order 5.4 TB/s; 256 x 64 tiles with
//               non-temporal loads and stores 6.0 TB/s; 256 x 32 tiles with at most
//               three workgroups per compute unit 6.1 TB/s.  A tile that tall would
//               need tens of KiB of LDS per workgroup; in registers it needs none.
//               Where the time goes (float32 16384^2, 256 x 32 tiles): the loads alone
//               take 156 us, the stores alone 168 us, both patterns issued side by
//               side 360 us whether or not the stores depend on the loads - reads and
//               writes mixed cost this memory more than their sum unless both streams
//               are perfectly linear (a flat copy of the same bytes: 320 us).
//               Non-temporal access only pays when every row starts on a 128-byte
//               line (16384-wide float32: 6.0 vs 5.4 TB/s); when rows straddle
//               lines it is far worse than cached access (16388-wide: 2.3 vs
//               4.2 TB/s) because neighbouring packets no longer meet in L2, so the
//               kernel is instantiated both ways and the host picks by alignment.
//   * sheared - the same item sizes when output rows do not start on 128-byte lines
//               (described at the kernel).
//   * records - any other item size up to 512 bytes with unit inner stride: tiles
//               through LDS in chunks of the widest aligned power of two.
//   * strided - everything else (element strides, negative strides, huge items): one
//               lane per (item, chunk) with the output index fastest, so writes stay
//               as dense as the layout allows.
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

// Sixteen bytes as one vector: loaded / stored with one instruction at any
// item-aligned address (nbh_load16 / nbh_store16).
typedef nbh_u32x4 u32x4;

// Shape of the workgroup tile per item size: WR x WC wavefronts, REP wavefront
// tiles stacked along the rows per wavefront.  A wavefront tile is 8V x 8V items.
// (2-byte items, int16 8192 x 32768, us: 256 x 64 as below 186; 512 x 64 with eight wavefronts
// 190, with four and REP = 2 200; 128 x 64 with REP = 2 196; 256 x 128 206; 128 x 128 222;
// 128 x 256 193.)
template <int E> struct ShapeOf;
template <> struct ShapeOf<1> { static constexpr int WR = 4, WC = 1, REP = 1; };   // 512 x 128
template <> struct ShapeOf<2> { static constexpr int WR = 4, WC = 1, REP = 1; };   // 256 x 64
template <> struct ShapeOf<4> { static constexpr int WR = 4, WC = 1, REP = 2; };   // 256 x 32
template <> struct ShapeOf<8> { static constexpr int WR = 2, WC = 2, REP = 4; };   // 128 x 32
template <> struct ShapeOf<16> { static constexpr int WR = 2, WC = 2, REP = 4; };  //  64 x 16

template <int E, bool GUARD, bool NT>
__device__ __forceinline__ void move_block(const char *__restrict__ in, char *__restrict__ out, int64_t rows,
                                           int64_t cols, int64_t in_s0, int64_t out_s0, int64_t r0, int64_t c0)
{
    // lane's V x V block has its top-left item at in[r0, c0]
    using Item = typename ItemOf<E>::type;
    constexpr int V = 16 / E;
    union Block {
        u32x4 pk[V];
        Item it[V][V];
    };
    Block a, b;
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const char *src = in + (r0 + j) * in_s0 + c0 * E;
        if (!GUARD || (r0 + j < rows && c0 + V <= cols)) {
            a.pk[j] = nbh_load16<E, NT>(src);
        } else if (r0 + j < rows) {
            for (int k = 0; k < V; ++k)
                if (c0 + k < cols)
                    a.it[j][k] = *reinterpret_cast<const Item *>(src + (int64_t)k * E);
        }
    }
#pragma unroll
    for (int i = 0; i < V; ++i)
#pragma unroll
        for (int j = 0; j < V; ++j)
            b.it[i][j] = a.it[j][i];
#pragma unroll
    for (int i = 0; i < V; ++i) {
        char *dst = out + (c0 + i) * out_s0 + r0 * E;
        if (!GUARD || (c0 + i < cols && r0 + V <= rows)) {
            nbh_store16<E, NT>(dst, b.pk[i]);
        } else if (c0 + i < cols) {
            for (int k = 0; k < V; ++k)
                if (r0 + k < rows)
                    *reinterpret_cast<Item *>(dst + (int64_t)k * E) = b.it[i][k];
        }
    }
}

template <int E, bool NT, typename Shape = ShapeOf<E>>
__global__ __launch_bounds__(64 * Shape::WR * Shape::WC) void transpose_packets(
    const char *__restrict__ in, char *__restrict__ out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
    int64_t tiles_r, bool diagonal)
{
    constexpr int V = 16 / E;
    constexpr int WT = 8 * V;  // wavefront tile edge, in items
    constexpr int WR = Shape::WR, WC = Shape::WC, REP = Shape::REP;
    constexpr int TR = WT * WR * REP, TC = WT * WC;

    // consecutive workgroups go down the input rows = along the output rows
    int64_t tile_c = (int64_t)blockIdx.x / tiles_r;
    const int64_t tile_r = (int64_t)blockIdx.x % tiles_r;
    if (diagonal) {
        // Output rows exactly 32 KiB apart, input rows a power of two of at most that: the
        // workgroups that run together (consecutive ones, going down the input rows) each take
        // the next column band as well, so that they write to different output rows.
        // Measured, us, bands in order (two passes for 2-byte items) -> diagonal, with the two
        // pitches in KiB: int16 16384^2 (32/32) 211 -> 190, 16384 x 8192 (16/32) 104 -> 96,
        // 16384 x 4096 (8/32) 52.8 -> 48.1; float32 8192^2 (32/32) 97.7 -> 93.3, 8192 x 4096
        // (16/32) 49.3 -> 47.4; float64 4096^2 (32/32) 47.1 -> 44.9.  No other pair of pitches
        // gains on every shape tried: output rows 64 KiB apart lose 4 - 9 % with input rows
        // as far apart (float32 16384^2 352 -> 385) and win or lose with shorter ones (float32
        // 16384 x 8192 205 -> 191, int16 32768 x 16384 370 -> 402); pitches that are no
        // powers of two lose (float32 16000^2 353 -> 423, 12000 x 8192 141 -> 151).
        tile_c = (tile_c + tile_r) % ((int64_t)gridDim.x / tiles_r);
    } else if (E == 2) {
        // 2-byte items: the column bands are walked in two passes, even bands first, then odd
        // ones, so that bands side by side are not in flight together.  Measured, bands in
        // order -> two passes, us: 8192 x 32768 191.3 -> 188.1, 32768 x 8192 216.8 -> 209.9,
        // 16384^2 214.9 -> 211.6, 8192^2 51.1 -> 49.3.  (4- and 8-byte items: 8192^2 float32
        // 96.3 -> 93.0, 12288^2 220.9 -> 213.8, but 16384^2 353 -> 364 and float64
        // 8192 x 16384 353 -> 373: no rule that holds there, so they keep the plain order.)
        const int64_t tiles_c = (int64_t)gridDim.x / tiles_r, half = (tiles_c + 1) / 2;
        tile_c = tile_c < half ? tile_c * 2 : (tile_c - half) * 2 + 1;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wr = wave / WC, wc = wave % WC;
    const int cx = lane & 7, ry = lane >> 3;
    const int64_t r_base = tile_r * TR + (int64_t)wr * (WT * REP) + ry * V;
    const int64_t c0 = tile_c * TC + (int64_t)wc * WT + cx * V;

    const bool inside = (tile_r + 1) * TR <= rows && (tile_c + 1) * TC <= cols;
    if (inside) {
#pragma unroll
        for (int q = 0; q < REP; ++q)
            move_block<E, false, NT>(in, out, rows, cols, in_s0, out_s0, r_base + q * WT, c0);
    } else {
        for (int q = 0; q < REP; ++q)
            if (r_base + q * WT < rows && c0 < cols)
                move_block<E, true, NT>(in, out, rows, cols, in_s0, out_s0, r_base + q * WT, c0);
    }
}

// Output rows that do not start on a 128-byte line.  With the packet kernel every
// 128-byte piece a wavefront stores would straddle two lines (measured: float32,
// 16388 rows, 4.1 TB/s against 5.4 TB/s when only the INPUT rows straddle).  Here a
// workgroup walks down a strip of the input, TR rows at a time, through a ring of
// RING = TR + S rows in LDS, and for every output row c it writes the items r in
// [lo(c), hi(c)), both ends rounded down to the nearest r at which output row c crosses
// a SECTOR boundary (S items).  Eight lanes write one line as eight aligned 16-byte
// packets, non-temporally, so every store instruction covers whole lines except where
// a tile's part of an output row begins or ends inside a line: there the lanes outside
// [lo, hi) stay idle and the rest of the line comes from the tile above or below.  What
// lies below hi(c) stays in the ring for the next step, so nothing is read twice except
// the S rows above the start of a strip.  Sectors of 32 bytes are what the memory takes
// as whole writes; with whole lines as the unit (S = items per line) every tile reads
// the 16 float64 rows above it a second time - 14 % more input traffic for a 112-row
// tile, against 3 % with 4-row sectors.  The ring's row pitch (TC + PAD items) spreads
// the column reads of one store instruction over the banks.
// Measured: float64 12345 x 6789 4.0 -> 5.1 TB/s, float32 16388 x 16384 4.1 -> 5.0.
// One-byte items stay with the packet kernel: gathering 16 single bytes from the ring
// per store costs more than the straddling does (2.5 against 3.2 TB/s).
// Shape of the ring kernel.  RING (a power of two) rows of TC columns, THREADS lanes,
// STEPS steps of TR = RING - SECTOR / E rows per workgroup.
template <int E_, int RING_, int TC_, int PAD_, int THREADS_, int STEPS_, int SECTOR_ = 128> struct RingCfg {
    static constexpr int E = E_, RING = RING_, TC = TC_, PAD = PAD_, THREADS = THREADS_, STEPS = STEPS_;
    static constexpr int SECTOR = SECTOR_ < E_ * 2 ? E_ * 2 : SECTOR_;  // at least two items: 16-byte items
};
// Measured on MI355X (TB/s of algorithmic traffic, ring 64 rows x 8 steps -> these shapes):
// float64 12345 x 6789 5.07 -> 5.44, float32 16388 x 16384 5.10 -> 5.75, 16385^2 5.09 -> 5.32,
// int16 8193 x 32769 4.40 -> 5.04, 16-byte items 8193^2 5.18 -> 5.86.  Tall tiles win (long
// runs of every output row are written by one workgroup at one time) and so do short
// strips: with one step per workgroup there are more, shorter workgroups in flight and
// the rows above a strip, read a second time, cost less than the lost overlap did.
// 2-byte items: 256 x 64 in two steps with 256 threads -> one step with 512
// threads and the unguarded interior path: 8193 x 32769 214 -> 206 us, 30001 x 7001 195 -> 183.
// 8-byte items, float64 12345 x 6789: ring 256 x 32 (half the rows read twice, half the workgroups per
// compute unit) 234 -> 253 us, ring 128 x 64 with 512 threads 234 -> 243 us: 128 x 32 stays.
template <int E> struct ShearOf;
template <> struct ShearOf<2> { using type = RingCfg<2, 256, 64, 8, 512, 1>; };
template <> struct ShearOf<4> { using type = RingCfg<4, 256, 64, 4, 512, 1>; };
template <> struct ShearOf<8> { using type = RingCfg<8, 128, 32, 4, 256, 1>; };
template <> struct ShearOf<16> { using type = RingCfg<16, 64, 32, 1, 256, 1>; };

constexpr int kOrderPlain = 0, kOrderByXcd = 1, kOrderPadded = 2;

template <typename Cfg>
__global__ __launch_bounds__(Cfg::THREADS) void transpose_sheared(const char *__restrict__ in, char *__restrict__ out,
                                                                   int64_t rows, int64_t cols, int64_t in_s0,
                                                                   int64_t out_s0, int64_t strips_r, int order, bool lean)
{
    constexpr int E = Cfg::E;
    using Item = typename ItemOf<E>::type;
    constexpr int V = 16 / E;    // items per packet
    constexpr int L = 128 / E;   // items per cache line
    constexpr int S = Cfg::SECTOR / E;  // items per sector: where a tile's part of an output row begins and ends
    constexpr int RING = Cfg::RING, TC = Cfg::TC, kThr = Cfg::THREADS;
    constexpr int TR = RING - S;
    constexpr int PPR = TC / V;     // packets per tile row
    constexpr int NL = RING / L + 1;  // lines of one output row a step can touch, at most
    static_assert((RING & (RING - 1)) == 0 && TR > 0 && S % V == 0 && L % S == 0 && RING % L == 0, "ring depth");
    __shared__ Item ring[RING][TC + Cfg::PAD];

    const int tid = threadIdx.x;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  When a
    // tile row is no wider than a line and input rows straddle lines, neighbouring
    // column bands fetch the same lines: give each XCD a contiguous share of the bands
    // so that they meet in one L2 (float32 16385^2: 4.6 -> 5.1 TB/s).
    int64_t logical = blockIdx.x;
    if (order == kOrderByXcd) {
        const int64_t per = (int64_t)gridDim.x / 8;
        if (logical < per * 8)
            logical = (logical % 8) * per + logical / 8;
    }
    // kOrderPadded: the strips of a column band are counted up to a multiple of 8, and XCD x
    // (workgroup index mod 8) walks down the x-th run of neighbouring strips of every band.
    // Tiles side by side (same strip, neighbouring bands) then run on the same XCD, strips_pad / 8
    // dispatches apart: the line of every input row that straddles their common edge is
    // fetched from memory once and found in that XCD's L2 the second time.  So are the S rows
    // above a tile, which the tile above, eight workgroups earlier on the same XCD, reads as its
    // last ones.  The order in which the chip walks through the matrix stays what it was.
    // (float64 12345 x 6789: fetched bytes 1.62 x the input in plain order, 1.15 x with the
    // strips dealt to the XCDs one by one, 1.01 x with the runs - at the same 233 - 235 us, the
    // kernel is not short of bandwidth; 8193^2 188 -> 184 us, 20001 x 5003 290 -> 288.  The surplus
    // workgroups leave at once.)
    const int64_t strips_pad = order == kOrderPadded ? (strips_r + 7) / 8 * 8 : strips_r;
    const int64_t tile_c = logical / strips_pad;
    int64_t strip = logical % strips_pad;
    if (order == kOrderPadded)
        strip = (strip % 8) * (strips_pad / 8) + strip / 8;
    if (strip >= strips_r)
        return;
    const int64_t C0 = tile_c * TC;
    const int64_t strip_begin = strip * (int64_t)(Cfg::STEPS * TR);
    int64_t strip_end = strip_begin + (int64_t)Cfg::STEPS * TR;
    const bool last_strip = strip == strips_r - 1;
    if (last_strip)
        strip_end = rows;

    // A step's rows travel global -> registers -> ring, so that the loads of the next
    // step are already in flight while this step's rows are being written out.
    constexpr int NP = (RING * PPR + kThr - 1) / kThr;  // packets per thread, at most
    union Pack {
        u32x4 pk;
        Item it[V];
    };
    Pack held[NP];

    // Tiles of a one-step configuration that lie wholly inside the matrix (`lean`: the host
    // asks for this path where it was measured to win): nothing needs a guard, so
    // the tile and the S rows above it arrive with ONE round of loads (the general path
    // below waits for those rows before it asks for the rest), and every thread then writes
    // its 16-byte piece of every line of one output row, 128 bytes apart, all read from
    // LDS before the first store.  Measured with whole lines as the sector, general path ->
    // this one: float64 12345 x 6789 246 -> 234 us (with the padded order), float32 16100^2
    // 391 -> 369, 12345 x 13578 259 -> 239.  With input
    // rows ON the grid it is slower for 4- and 8-byte items (float32 16388 x 16384 374 -> 391,
    // float64 4099 x 20000 229 -> 243) and for 16-byte items always (8193^2 366 -> 401):
    // those keep the general path.  2-byte items gain either way (8193 x 32769 214 -> 206,
    // 10001 x 12001 88 -> 75, input rows on the grid 8193 x 32768 206 -> 205).
    // One workgroup per tile, here for a few microseconds, is also what keeps the memory busy:
    // the same path as a loop in as many resident workgroups as the chip holds, each asking
    // for its next tile's loads while it reads the ring and stores, was slower on every shape
    // (float64 12345 x 6789 234 -> 266 us, float32 16100^2 366 -> 429, int16 8193 x 32769
    // 210 -> 279): a workgroup that ends frees its place while its stores are still on their way.
    // Nor is it the way into LDS that costs: the tile loaded straight into LDS (eight
    // global_load_lds_dwordx4 per lane into unpadded 256-byte rows, the packets of a row permuted by
    // the row number so that the column reads stay free of bank conflicts; no registers held, no
    // LDS write instructions) runs float64 12345 x 6789 in 236.6 us against 235.0, and 4099 x 20000,
    // 8193^2, 20001 x 5003 within 0.3 % of this path.
    if constexpr (Cfg::STEPS == 1 && E < 16) {
        if (lean && strip_begin >= S && strip_begin + TR < rows && C0 + TC <= cols) {
            constexpr int RPS = kThr / PPR;      // tile rows one round of the workgroup loads
            constexpr int NPF = RING * PPR / kThr;
            constexpr int NLF = (RING + L - 2 * S + L - 1) / L;  // line slots of one output row
            static_assert(RING * PPR % kThr == 0 && kThr % PPR == 0, "whole rounds of loads");
            static_assert(kThr / 8 == TC, "eight lanes per output row");
            const int64_t A = strip_begin - S;
            const int lr0 = tid / PPR, pc = tid % PPR;
            const char *src = in + (A + lr0) * in_s0 + (C0 + (int64_t)pc * V) * E;
            u32x4 got[NPF];
#pragma unroll
            for (int k = 0; k < NPF; ++k)
                got[k] = nbh_load16<E, false>(src + (int64_t)k * RPS * in_s0);
#pragma unroll
            for (int k = 0; k < NPF; ++k)  // tile row t sits in ring row t: one step, no wrap
                *reinterpret_cast<u32x4 *>(&ring[lr0 + k * RPS][pc * V]) = got[k];
            __syncthreads();
            const int lc = tid >> 3, sub = tid & 7;
            char *row = out + (C0 + lc) * out_s0;
            const int phase = (int)(((uintptr_t)row % 128) / E);
            // this tile's part of the output row: [lo, lo + TR), lo in (strip_begin - S, strip_begin]
            const int lo_t = S - (int)((phase + strip_begin) % S);   // tile row of item lo, in [1, S]
            const int first_t = lo_t - (int)((phase + A + lo_t) % L); // tile row at which lo's line begins (may be < 0)
            Pack p[NLF];
#pragma unroll
            for (int i = 0; i < NLF; ++i) {
                const int d = first_t + i * L + sub * V;  // tile row of this lane's first item
                if (d >= lo_t && d < lo_t + TR) {
#pragma unroll
                    for (int j = 0; j < V; ++j)
                        p[i].it[j] = ring[d + j][lc];
                }
            }
            char *dst = row + (A + first_t + sub * V) * E;  // 16-byte aligned: first_t starts a line
#pragma unroll
            for (int i = 0; i < NLF; ++i) {
                const int d = first_t + i * L + sub * V;
                if (d >= lo_t && d < lo_t + TR)
                    __builtin_nontemporal_store(p[i].pk, reinterpret_cast<u32x4 *>(dst + i * 128));
            }
            return;
        }
    }

    auto fetch = [&](int64_t from, int64_t to) {  // rows [from, to) -> held
        const int count = (int)(to - from) * PPR;
#pragma unroll
        for (int k = 0; k < NP; ++k) {
            const int idx = tid + k * kThr;
            if (idx >= count)
                break;
            const int64_t gr = from + idx / PPR;
            const int64_t gc = C0 + (int64_t)(idx % PPR) * V;
            if (gr < 0 || gc >= cols)
                continue;
            const char *src = in + gr * in_s0 + gc * E;
            if (gc + V <= cols) {
                held[k].pk = nbh_load16<E, false>(src);
            } else {
                for (int j = 0; j < V; ++j)
                    if (gc + j < cols)
                        held[k].it[j] = *reinterpret_cast<const Item *>(src + (int64_t)j * E);
            }
        }
    };
    auto park = [&](int64_t from, int64_t to) {  // held -> ring (columns beyond the edge carry junk, never stored)
        const int count = (int)(to - from) * PPR;
#pragma unroll
        for (int k = 0; k < NP; ++k) {
            const int idx = tid + k * kThr;
            if (idx >= count)
                break;
            const int64_t gr = from + idx / PPR;
            if (gr < 0)
                continue;
            Item *dst = &ring[gr & (RING - 1)][(idx % PPR) * V];
#pragma unroll
            for (int j = 0; j < V; ++j)
                dst[j] = held[k].it[j];
        }
    };

    fetch(strip_begin - S, strip_begin);  // what the first step needs from above
    park(strip_begin - S, strip_begin);
    int64_t R0 = strip_begin;
    int64_t step_end = (R0 + TR < strip_end) ? R0 + TR : strip_end;
    fetch(R0, step_end);
    while (R0 < strip_end) {
        park(R0, step_end);
        __syncthreads();
        const int64_t next = step_end;
        const int64_t next_end = (next + TR < strip_end) ? next + TR : strip_end;
        if (next < strip_end)
            fetch(next, next_end);
        // eight lanes per 128-byte line of output; a pass of the workgroup covers
        // kThr / 8 lines, neighbouring output rows first
        for (int w = tid >> 3; w < TC * NL; w += kThr / 8) {
            const int lc = w % TC, k = w / TC;
            const int64_t c = C0 + lc;
            if (c >= cols)
                continue;
            char *row = out + c * out_s0;
            const int64_t phase = (int64_t)(((uintptr_t)row % 128) / E);  // line offset of item 0, in items
            // this step's part of the output row: [lo, hi), both on sector boundaries of the row
            const int64_t lo = (R0 == 0) ? 0 : R0 - (phase + R0) % S;
            const int64_t hi = (step_end == rows) ? rows : step_end - (phase + step_end) % S;
            const int64_t line = lo - (phase + lo) % L + (int64_t)k * L;  // first item of this line (below 0 in row 0's first line)
            if (line >= hi)
                continue;
            const int64_t r = line + (tid & 7) * V;
            Pack p;
            if (r >= lo && r + V <= hi) {
#pragma unroll
                for (int j = 0; j < V; ++j)
                    p.it[j] = ring[(r + j) & (RING - 1)][lc];
                u32x4 *dst = reinterpret_cast<u32x4 *>(row + r * E);  // 16-byte aligned: the line is
                __builtin_nontemporal_store(p.pk, dst);
            } else {  // where the matrix begins or ends inside a packet
                for (int j = 0; j < V; ++j)
                    if (r + j >= lo && r + j < hi)
                        *reinterpret_cast<Item *>(row + (r + j) * E) = ring[(r + j) & (RING - 1)][lc];
            }
        }
        __syncthreads();  // the next step overwrites rows that were just read
        R0 = next;
        step_end = next_end;
    }
}

// Items of any other size (records, 12-byte strings, 16-byte items that are only
// 8-byte aligned ...) with unit inner stride on both sides: a T x T tile of items goes
// through LDS in chunks of G bytes, G being the widest power of two that divides the
// item size, the row strides and both base addresses.  Consecutive lanes read
// consecutive chunks of an input row segment (T * itemsize contiguous bytes) and
// write consecutive chunks of an output row segment, whatever the item size; the
// divisions by the two run lengths are multiplications by precomputed reciprocals
// (exact for operands below 2^16).  Measured, 8192^2 items of 12 bytes: 4.2 TB/s,
// against 1.6 TB/s with one lane per chunk straight from global memory, where every
// 4-byte read of a wavefront comes from a different input row.
struct RecordShape {
    int32_t itemsize, tile, chunks_per_run, pitch;  // run = tile * itemsize bytes
    uint32_t inv_chunks_per_run, inv_itemsize;      // floor(2^32 / d) + 1
};

// W = 16 when WIDE (both bases and both row strides are multiples of 16, and so is
// a run): global memory is then moved 16 bytes per lane although items can only be
// picked out of the tile G bytes at a time.  Index arithmetic, not memory, bounds this
// kernel, so the fewer chunks the better (28-byte items: 2.9 -> 4.3 TB/s, 3-byte
// items 1.2 -> 1.9); with 8-byte pieces it no longer pays (24-byte items: 5.0 -> 4.4)
// and is not used.
template <int G, bool WIDE>
__global__ __launch_bounds__(kThreads) void transpose_records(const char *__restrict__ in, char *__restrict__ out,
                                                               int64_t rows, int64_t cols, int64_t in_s0,
                                                               int64_t out_s0, int64_t tiles_r, RecordShape sh)
{
    using Piece = typename ItemOf<G>::type;
    constexpr int W = WIDE ? 16 : G;
    constexpr int NP = W / G;  // pieces per chunk
    union Chunk {
        Piece piece[NP];
        typename ItemOf<W>::type whole;
    };
    extern __shared__ __attribute__((aligned(16))) char record_tile[];
    const int64_t tile_c = (int64_t)blockIdx.x / tiles_r;  // consecutive workgroups go along the output rows
    const int64_t tile_r = (int64_t)blockIdx.x % tiles_r;
    const int64_t R0 = tile_r * sh.tile, C0 = tile_c * sh.tile;
    const int nrows = (int)((rows - R0 < sh.tile) ? rows - R0 : sh.tile);
    const int ncols = (int)((cols - C0 < sh.tile) ? cols - C0 : sh.tile);
    const int total = sh.tile * sh.chunks_per_run;

    const char *src = in + R0 * in_s0 + C0 * sh.itemsize;
    const int in_run = ncols * sh.itemsize;  // bytes of one input row inside the tile
    for (int idx = threadIdx.x; idx < total; idx += kThreads) {
        const int r = (int)__umulhi((uint32_t)idx, sh.inv_chunks_per_run);
        const int b = (idx - r * sh.chunks_per_run) * W;
        if (r >= nrows || b >= in_run)
            continue;
        const char *g = src + (int64_t)r * in_s0 + b;
        char *l = record_tile + r * sh.pitch + b;
        if (b + W <= in_run) {
            *reinterpret_cast<typename ItemOf<W>::type *>(l) = *reinterpret_cast<const typename ItemOf<W>::type *>(g);
        } else {  // the run ends inside this chunk (last columns of the matrix)
            for (int k = 0; b + k * G < in_run; ++k)
                reinterpret_cast<Piece *>(l)[k] = reinterpret_cast<const Piece *>(g)[k];
        }
    }
    __syncthreads();
    char *dst = out + C0 * out_s0 + R0 * sh.itemsize;
    const int out_run = nrows * sh.itemsize;  // bytes of one output row inside the tile
    for (int idx = threadIdx.x; idx < total; idx += kThreads) {
        const int c = (int)__umulhi((uint32_t)idx, sh.inv_chunks_per_run);
        const int b = (idx - c * sh.chunks_per_run) * W;
        if (c >= ncols || b >= out_run)
            continue;
        int r = (int)__umulhi((uint32_t)b, sh.inv_itemsize);
        int within = b - r * sh.itemsize;
        const char *l = record_tile + c * sh.itemsize;
        char *g = dst + (int64_t)c * out_s0 + b;
        Chunk v;
#pragma unroll
        for (int k = 0; k < NP; ++k) {
            if (b + k * G < out_run)
                v.piece[k] = *reinterpret_cast<const Piece *>(l + r * sh.pitch + within);
            within += G;
            if (within >= sh.itemsize) {
                within -= sh.itemsize;
                ++r;
            }
        }
        if (b + W <= out_run) {
            *reinterpret_cast<typename ItemOf<W>::type *>(g) = v.whole;
        } else {
            for (int k = 0; b + k * G < out_run; ++k)
                reinterpret_cast<Piece *>(g)[k] = v.piece[k];
        }
    }
}

// One lane per G-byte chunk of one item; chunk index fastest, then the output's
// inner index, then its outer index.
template <int G>
__global__ __launch_bounds__(kThreads) void transpose_strided(const char *__restrict__ in, char *__restrict__ out,
                                                               int64_t rows, int64_t in_s0, int64_t in_s1,
                                                               int64_t out_s0, int64_t out_s1, int64_t chunks,
                                                               int64_t total)
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

template <int E, typename Shape = ShapeOf<E>>
int launch_packets(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
                   hipStream_t stream)
{
    constexpr int WT = 8 * (16 / E);
    constexpr int TR = WT * Shape::WR * Shape::REP, TC = WT * Shape::WC;
    const int64_t tiles_r = (rows + TR - 1) / TR;
    const int64_t tiles_c = (cols + TC - 1) / TC;
    const int64_t tiles = tiles_r * tiles_c;
    if (tiles > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    // stream past the caches only if every row of both arrays starts on a 128-byte line
    const uint64_t mix = (uint64_t)(uintptr_t)in | (uint64_t)(uintptr_t)out | (uint64_t)in_s0 | (uint64_t)out_s0;
    const dim3 grid((unsigned)tiles), block(64 * Shape::WR * Shape::WC);
    // Large matrices run with fewer workgroups per compute unit than would fit: what the chip
    // has in flight then covers a narrower window of both matrices, which the memory takes
    // better.  The kernel uses no LDS; asking for a third of a compute unit's LDS per
    // workgroup is the throttle (at most three workgroups per compute unit).  Measured, us,
    // free -> throttled: float32 16384^2 365 -> 353, 16000^2 363 -> 348, 8192 x 32768 372 ->
    // 358; float64 8192 x 16384 355 -> 345, 4096 x 32768 357 -> 340; int16 32768^2 766 -> 720,
    // 20000 x 20032 369 -> 347.  Below the thresholds it loses (float32 8192^2 96 -> 107,
    // float64 8192^2 186 -> 195); 1- and 16-byte items never gain.
    const double moved = 2.0 * (double)rows * (double)cols * E;
    const double threshold = E == 4 ? 0.75 * (1u << 30) : 1.5 * (1u << 30);
    const unsigned throttle = ((E == 2 || E == 4 || E == 8) && moved >= threshold) ? 54000u : 0u;
    // the order in which the workgroups take the tiles, by the two pitches (measurements at the kernel)
    const bool diagonal = (E == 2 || E == 4 || E == 8) && out_s0 == 32768 && in_s0 > 0 && in_s0 <= 32768 &&
                          (in_s0 & (in_s0 - 1)) == 0;
    if (mix % 128 == 0)
        hipLaunchKernelGGL((transpose_packets<E, true, Shape>), grid, block, throttle, stream, (const char *)in,
                           (char *)out, rows, cols, in_s0, out_s0, tiles_r, diagonal);
    else
        hipLaunchKernelGGL((transpose_packets<E, false, Shape>), grid, block, throttle, stream, (const char *)in,
                           (char *)out, rows, cols, in_s0, out_s0, tiles_r, diagonal);
    return nbh_launch_status();
}

template <typename Cfg>
int launch_sheared_cfg(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
                       hipStream_t stream)
{
    constexpr int E = Cfg::E;
    constexpr int TR = Cfg::RING - Cfg::SECTOR / E;
    const int64_t strips_r = (rows + (int64_t)Cfg::STEPS * TR - 1) / ((int64_t)Cfg::STEPS * TR);
    const int64_t tiles_c = (cols + Cfg::TC - 1) / Cfg::TC;
    const bool ragged_in = (((uint64_t)(uintptr_t)in | (uint64_t)in_s0) % 128) != 0;
    int order = kOrderPlain;
    if (ragged_in && Cfg::TC * E <= 128)
        order = kOrderByXcd;
    else if (ragged_in && Cfg::STEPS == 1 && E < 16)
        order = kOrderPadded;
    const int64_t strips_grid = order == kOrderPadded ? (strips_r + 7) / 8 * 8 : strips_r;
    const int64_t blocks = strips_grid * tiles_c;
    if (blocks > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    const bool lean = Cfg::STEPS == 1 && (E == 2 || (order == kOrderPadded && E < 16));
    hipLaunchKernelGGL((transpose_sheared<Cfg>), dim3((unsigned)blocks), dim3(Cfg::THREADS), 0, stream,
                       (const char *)in, (char *)out, rows, cols, in_s0, out_s0, strips_r, order, lean);
    return nbh_launch_status();
}

template <int E>
int launch_sheared(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
                   hipStream_t stream)
{
    return launch_sheared_cfg<typename ShearOf<E>::type>(in, out, rows, cols, in_s0, out_s0, stream);
}

template <int G>
int launch_records(const void *in, void *out, int64_t rows, int64_t cols, int64_t in_s0, int64_t out_s0,
                   int64_t itemsize, hipStream_t stream)
{
    RecordShape sh;
    sh.itemsize = (int32_t)itemsize;
    sh.tile = itemsize <= 32 ? 32 : itemsize <= 128 ? 16 : 8;  // about 32 KiB of LDS at most
    const int run = sh.tile * sh.itemsize;
    const uint64_t mix = (uint64_t)(uintptr_t)in | (uint64_t)(uintptr_t)out | (uint64_t)in_s0 | (uint64_t)out_s0 |
                         (uint64_t)run;
    const bool wide = G <= 4 && mix % 16 == 0;
    const int w = wide ? 16 : G;
    sh.chunks_per_run = run / w;
    sh.pitch = run + 16;
    sh.inv_chunks_per_run = (uint32_t)(0x100000000ull / (uint32_t)sh.chunks_per_run) + 1u;
    sh.inv_itemsize = (uint32_t)(0x100000000ull / (uint32_t)sh.itemsize) + 1u;
    const int64_t tiles_r = (rows + sh.tile - 1) / sh.tile;
    const int64_t tiles_c = (cols + sh.tile - 1) / sh.tile;
    const int64_t tiles = tiles_r * tiles_c;
    if (tiles > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    const size_t lds = (size_t)sh.tile * sh.pitch;
    const dim3 grid((unsigned)tiles), block(kThreads);
    if (wide)
        hipLaunchKernelGGL((transpose_records<G, (G <= 4)>), grid, block, lds, stream, (const char *)in, (char *)out,
                           rows, cols, in_s0, out_s0, tiles_r, sh);
    else
        hipLaunchKernelGGL((transpose_records<G, false>), grid, block, lds, stream, (const char *)in, (char *)out,
                           rows, cols, in_s0, out_s0, tiles_r, sh);
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
                       (char *)out, rows, in_s0, in_s1, out_s0, out_s1, chunks, total);
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
    nbh_stream_report report(s);

    // largest power of two (<= 16) that divides the item size, every stride and
    // both base addresses: the widest access that is aligned everywhere
    uint64_t mix = (uint64_t)itemsize | (uint64_t)in_s0 | (uint64_t)in_s1 | (uint64_t)out_s0 | (uint64_t)out_s1 |
                   (uint64_t)(uintptr_t)in | (uint64_t)(uintptr_t)out | 16u;
    const int64_t g = low_bit(mix);

    const bool unit_inner = in_s1 == itemsize && out_s1 == itemsize && in_s0 > 0 && out_s0 > 0;
    if (unit_inner && g == itemsize) {  // item size is a power of two <= 16 and items are aligned
        // output rows off the 128-byte grid and long enough for the shear to pay
        const bool ragged_out = (((uint64_t)(uintptr_t)out | (uint64_t)out_s0) % 128) != 0 && rows * itemsize >= 512 &&
                                itemsize > 1;
        if (ragged_out) {
            switch (itemsize) {
            case 2: return launch_sheared<2>(in, out, rows, cols, in_s0, out_s0, s);
            case 4: return launch_sheared<4>(in, out, rows, cols, in_s0, out_s0, s);
            case 8: return launch_sheared<8>(in, out, rows, cols, in_s0, out_s0, s);
            case 16: return launch_sheared<16>(in, out, rows, cols, in_s0, out_s0, s);
            default: break;
            }
        }
        switch (itemsize) {
        case 1: return launch_packets<1>(in, out, rows, cols, in_s0, out_s0, s);
        case 2: return launch_packets<2>(in, out, rows, cols, in_s0, out_s0, s);
        case 4: return launch_packets<4>(in, out, rows, cols, in_s0, out_s0, s);
        case 8: return launch_packets<8>(in, out, rows, cols, in_s0, out_s0, s);
        case 16: return launch_packets<16>(in, out, rows, cols, in_s0, out_s0, s);
        default: break;
        }
    }
    if (unit_inner && itemsize <= 512) {
        switch (g) {
        case 1: return launch_records<1>(in, out, rows, cols, in_s0, out_s0, itemsize, s);
        case 2: return launch_records<2>(in, out, rows, cols, in_s0, out_s0, itemsize, s);
        case 4: return launch_records<4>(in, out, rows, cols, in_s0, out_s0, itemsize, s);
        case 8: return launch_records<8>(in, out, rows, cols, in_s0, out_s0, itemsize, s);
        default: return launch_records<16>(in, out, rows, cols, in_s0, out_s0, itemsize, s);
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

// nbh_reduce: single-launch, deterministic tree reduction for gfx950 (wave64).
//
// Shape of the computation
//   * the input is read once with 128-bit loads; the few elements in front of the
//     first 16-byte boundary and behind the last whole vector are picked up by
//     single lanes of workgroup 0
//   * inputs from 128 MiB on are cut into pieces of 16 KiB that are dealt out to the
//     workgroups (8 wavefronts, two workgroups per compute unit) round robin, so that at
//     any moment all of them read one window of a few MiB that moves through the input:
//     piece p of a round goes to the workgroup whose XCD comes p / (grid / 8)-th, which
//     gives every XCD one run of consecutive pieces per round; a workgroup has the loads
//     of its next piece in flight while it adds the current one (non-temporal 16-byte
//     loads, four per lane in flight) and meets at a barrier after every piece, so that a
//     piece is asked for as one run.  2^28 float32: 153.6 us with one contiguous slice per
//     workgroup, 149.1 us dealt - the memory serves one moving front better than 512
//     separate streams.  (Many short-lived workgroups that read a piece each come to
//     143 us, but each needs a partial and a ticket: 12 ns per workgroup with all tickets
//     on one address, and no cheaper with the tickets spread out.)
//   * smaller inputs are cut into one contiguous slice per workgroup instead, kUnroll
//     independent 16-byte loads in flight per lane
//   * lanes fold into per-lane accumulators, a wavefront folds with four DPP
//     steps inside each row of 16 lanes plus three scalar combines of the four row
//     totals, the workgroup folds its wavefront totals through LDS
//   * each workgroup publishes one partial; the workgroup that draws the last
//     ticket folds the partials in index order, applies `init` and writes `out`.
//     Which workgroup finishes does not change the association, so results are
//     identical from run to run.
//
// Publishing a partial.  An agent-scope release (what __threadfence() or a
// release RMW would emit) writes back the whole L2 of the XCD; measured on MI355X
// that costs about 90 us per 2048 workgroups on a 160 us kernel.  It is also more
// than is needed: the only datum to publish is the partial itself.  So the partial
// is put in place with an agent-scope atomic EXCHANGE - a read-modify-write is carried
// out where every XCD looks, and its result comes back from there - the wavefront
// waits for that result, and only then takes its ticket with a relaxed agent-scope
// atomic add.
// THE INVARIANT THIS RESTS ON: on gfx942 / gfx950 the L2 caches of the eight XCDs are not
// coherent with one another; agent-scope atomics are issued with the sc1 bit, which sends
// them past the XCD's own L2 to the one place all XCDs share (LLVM's AMDGPU memory model
// for gfx942 lowers every agent-scope atomicrmw and atomic load to an sc1 access for this
// reason).  A returning atomic's result is produced there, after the new value is in
// place, so (a) once the result is back the partial can be seen by an sc1 load from any
// XCD, and (b) the finisher's sc1 loads cannot be served from a stale private L2.  What the
// documentation does NOT promise is any order between two atomics to DIFFERENT addresses
// that are merely issued one after the other - hence the wait for the result in between.
// In the language-level memory model the relaxed accesses still form a race on the
// partials; NBH_REDUCE_RELEASE_PUBLISH=1 builds the release/acquire protocol instead.  (A written-through atomic store followed by a wait for its
// acknowledgement is not enough: the acknowledgement does not mean that the value is
// where other XCDs read it.  With tickets and partials in different pages a ticket was
// seen to overtake its partial, one wrong sum in some 10^4 closings; the exchange costs
// 0.4 us on a 154 us kernel.)  The finishing workgroup invalidates its caches once
// (agent-scope acquire fence) and reads the partials with agent-scope atomic loads.
// Few, large workgroups keep the tickets, which all hit one address, off the critical
// path: atomics on one address - or on neighbouring addresses, which share a memory
// channel - take about 6 ns each, one after the other (one workgroup per 16 KiB with
// tickets 4 bytes apart: 557 us for 2^28 float32; tickets 4 KiB apart: 180 us).
//
// HBM roofline: n * itemsize bytes are read once; nothing else of size is moved.
#include "common.h"

#include <atomic>
#include <limits>
#include <mutex>
#include <type_traits>

namespace {

constexpr int kBlock = 512;
constexpr int kWaves = kBlock / 64;
constexpr int kMaxGrid = 4096;
constexpr size_t kHeaderBytes = 256;  // ticket counter, padded to its own cache lines
constexpr size_t kScratchBytes = kHeaderBytes + sizeof(uint64_t) * kMaxGrid;
constexpr int kGridPerCU = 2;
constexpr int kUnroll = 4;
constexpr int kDeal = 2;                                // 16-byte loads per lane and dealt piece
constexpr int64_t kPieceVecs = (int64_t)kBlock * kDeal;  // 16 KiB
// Build with -DNBH_REDUCE_RELEASE_PUBLISH=1 to publish partials the slow, by-the-book way
// (see "Publishing a partial" above): the reference point when the fast protocol is in doubt.
#ifndef NBH_REDUCE_RELEASE_PUBLISH
#define NBH_REDUCE_RELEASE_PUBLISH 0
#endif
constexpr bool kReleasePublish = NBH_REDUCE_RELEASE_PUBLISH != 0;

// ---- complex elements -------------------------------------------------------------
// An aggregate (it lives in unions with raw packets).  Multiplication is the plain
// formula (ac - bd) + (ad + bc)i, four products and two sums each rounded once, which
// is what the reference's JIT emits for `a * b` on complex operands.
template <typename R> struct Cplx {
    R re, im;
};
template <typename R> __device__ __forceinline__ Cplx<R> operator+(Cplx<R> a, Cplx<R> b)
{
    return {a.re + b.re, a.im + b.im};
}
template <typename R> __device__ __forceinline__ Cplx<R> operator*(Cplx<R> a, Cplx<R> b)
{
    return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
template <typename T> struct IsCplx : std::false_type {};
template <typename R> struct IsCplx<Cplx<R>> : std::true_type {};
// float16 elements: the accumulator is a half too, every operation rounds to binary16
// (what the reference's JIT emits for `a + b` on float16 operands)
using Half = _Float16;
// real floating point, binary16 included
template <typename T> struct IsReal : std::integral_constant<bool, std::is_floating_point<T>::value || std::is_same<T, Half>::value> {};
// real or complex floating point: the accumulator is the element type itself
template <typename T> struct IsInexact : std::integral_constant<bool, IsReal<T>::value || IsCplx<T>::value> {};

// ---- operators -----------------------------------------------------------------
struct OpAdd {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a + b; }
};
struct OpMul {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a * b; }
};
struct OpMax {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return b > a ? b : a; }
};
struct OpMin {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return b < a ? b : a; }
};
// bitwise functors, integers only
struct OpAnd {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a & b; }
};
struct OpOr {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a | b; }
};
struct OpXor {
    template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a ^ b; }
};
template <typename Op> struct IsBitwise : std::integral_constant<bool, std::is_same<Op, OpAnd>::value || std::is_same<Op, OpOr>::value || std::is_same<Op, OpXor>::value> {};

// Accumulator type.  Sums and products of integers are carried in an unsigned
// type at least 32 bits wide: arithmetic modulo 2^32 / 2^64 truncates to the same
// element value as arithmetic modulo 2^bits, and unsigned wrap-around is defined.
// Comparisons keep the signedness of the element type.
template <typename T, typename Op> struct AccOf {
    static constexpr bool arith = std::is_same<Op, OpAdd>::value || std::is_same<Op, OpMul>::value || IsBitwise<Op>::value;
    using wide_int = typename std::conditional<
        sizeof(T) == 8, typename std::conditional<arith || std::is_unsigned<T>::value, uint64_t, int64_t>::type,
        typename std::conditional<arith || std::is_unsigned<T>::value, uint32_t, int32_t>::type>::type;
    using type = typename std::conditional<IsInexact<T>::value, T, wide_int>::type;
};

template <typename T, typename Op> __device__ __forceinline__ typename AccOf<T, Op>::type identity_of()
{
    using A = typename AccOf<T, Op>::type;
    if constexpr (IsCplx<T>::value)
        return A{std::is_same<Op, OpMul>::value ? 1 : 0, 0};
    else if constexpr (std::is_same<Op, OpAdd>::value || std::is_same<Op, OpOr>::value || std::is_same<Op, OpXor>::value)
        return A(0);
    else if constexpr (std::is_same<Op, OpAnd>::value)
        return (A) ~(A)0;
    else if constexpr (std::is_same<Op, OpMul>::value)
        return A(1);
    else if constexpr (IsReal<T>::value)
        return std::is_same<Op, OpMax>::value ? A(-__builtin_huge_valf()) : A(__builtin_huge_valf());
    else if constexpr (std::is_same<Op, OpMax>::value)
        return A(std::numeric_limits<T>::lowest());
    else
        return A(std::numeric_limits<T>::max());
}

// ---- wavefront / workgroup folding -----------------------------------------------
template <int CTRL> __device__ __forceinline__ uint32_t dpp_move(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}

template <typename A, int CTRL> __device__ __forceinline__ A dpp(A v)
{
    if constexpr (sizeof(A) == 2) {
        uint16_t b = __builtin_bit_cast(uint16_t, v);
        return __builtin_bit_cast(A, (uint16_t)dpp_move<CTRL>(b));
    } else if constexpr (sizeof(A) == 4) {
        uint32_t b = __builtin_bit_cast(uint32_t, v);
        return __builtin_bit_cast(A, dpp_move<CTRL>(b));
    } else if constexpr (sizeof(A) == 8) {
        uint64_t b = __builtin_bit_cast(uint64_t, v);
        uint32_t lo = dpp_move<CTRL>((uint32_t)b);
        uint32_t hi = dpp_move<CTRL>((uint32_t)(b >> 32));
        return __builtin_bit_cast(A, ((uint64_t)hi << 32) | lo);
    } else {
        static_assert(sizeof(A) == 16, "accumulators are 2, 4, 8 or 16 bytes");
        nbh_u32x4 b = __builtin_bit_cast(nbh_u32x4, v);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            b[k] = dpp_move<CTRL>(b[k]);
        return __builtin_bit_cast(A, b);
    }
}

template <typename A> __device__ __forceinline__ A read_lane(A v, int lane)
{
    if constexpr (sizeof(A) == 2) {
        uint16_t b = __builtin_bit_cast(uint16_t, v);
        return __builtin_bit_cast(A, (uint16_t)__builtin_amdgcn_readlane((int)b, lane));
    } else if constexpr (sizeof(A) == 4) {
        uint32_t b = __builtin_bit_cast(uint32_t, v);
        return __builtin_bit_cast(A, (uint32_t)__builtin_amdgcn_readlane((int)b, lane));
    } else if constexpr (sizeof(A) == 8) {
        uint64_t b = __builtin_bit_cast(uint64_t, v);
        uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, lane);
        uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), lane);
        return __builtin_bit_cast(A, ((uint64_t)hi << 32) | lo);
    } else {
        nbh_u32x4 b = __builtin_bit_cast(nbh_u32x4, v);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            b[k] = (uint32_t)__builtin_amdgcn_readlane((int)b[k], lane);
        return __builtin_bit_cast(A, b);
    }
}

// Total of the 64 lanes, returned in every lane.
template <typename A, typename Op> __device__ __forceinline__ A wave_fold(A v)
{
    v = Op::apply(v, dpp<A, 0xB1>(v));   // quad_perm [1,0,3,2]: lane ^ 1
    v = Op::apply(v, dpp<A, 0x4E>(v));   // quad_perm [2,3,0,1]: lane ^ 2
    v = Op::apply(v, dpp<A, 0x141>(v));  // row_half_mirror: the other quad of 8
    v = Op::apply(v, dpp<A, 0x140>(v));  // row_mirror: the other half of 16
    A r0 = read_lane(v, 0), r1 = read_lane(v, 16), r2 = read_lane(v, 32), r3 = read_lane(v, 48);
    return Op::apply(Op::apply(r0, r1), Op::apply(r2, r3));
}

// Total of the workgroup, returned in every thread.  One LDS slot per wavefront.
template <typename A, typename Op> __device__ __forceinline__ A block_fold(A v, A *lds)
{
    A w = wave_fold<A, Op>(v);
    __syncthreads();  // slots may still be read from a previous fold
    if ((threadIdx.x & 63) == 0)
        lds[threadIdx.x >> 6] = w;
    __syncthreads();
    static_assert(kWaves == 8, "combine below assumes eight wavefronts");
    return Op::apply(Op::apply(Op::apply(lds[0], lds[1]), Op::apply(lds[2], lds[3])),
                     Op::apply(Op::apply(lds[4], lds[5]), Op::apply(lds[6], lds[7])));
}

// A partial is published as kWords words of type Word (16-byte accumulators as two
// 8-byte words; each word is one atomic store, the ticket is drawn after all of them
// have been acknowledged).
template <typename A> struct WordsOf {
    using Word = typename std::conditional<sizeof(A) <= 4, uint32_t, uint64_t>::type;
    static constexpr int kWords = sizeof(A) <= 4 ? 1 : (int)(sizeof(A) / sizeof(Word));
    struct Image {
        Word w[kWords];
    };
    static __device__ __forceinline__ Image pack(A v)
    {
        if constexpr (sizeof(A) == 2) {  // a half travels in the low 16 bits of a word
            Image img;
            img.w[0] = __builtin_bit_cast(uint16_t, v);
            return img;
        } else {
            return __builtin_bit_cast(Image, v);
        }
    }
    static __device__ __forceinline__ A unpack(Image img)
    {
        if constexpr (sizeof(A) == 2)
            return __builtin_bit_cast(A, (uint16_t)img.w[0]);
        else
            return __builtin_bit_cast(A, img);
    }
};

// ---- the kernel ------------------------------------------------------------------
// STRIDED: the items are `stride` bytes apart (any sign) instead of packed; they are
// then read one by one, `nvec` counts items and `head` is 0.
// pieces > 0 (packed only): the first pieces * kPieceVecs vectors are dealt out piece by
// piece, the vectors behind them go to the last workgroup; pieces == 0: one slice each.
template <typename T, typename Op, bool STRIDED>
__global__ __launch_bounds__(kBlock) void reduce_kernel(const T *__restrict__ in, int64_t n, int64_t head,
                                                        int64_t nvec, int64_t pieces, int64_t stride, T init,
                                                        T *__restrict__ out,
                                                        uint64_t *__restrict__ partials_raw,
                                                        unsigned *__restrict__ ticket)
{
    using A = typename AccOf<T, Op>::type;
    using Word = typename WordsOf<A>::Word;
    using Image = typename WordsOf<A>::Image;
    constexpr int kWords = WordsOf<A>::kWords;
    constexpr int V = 16 / (int)sizeof(T);
    union VecT {  // one 16-byte packet of V elements
        nbh_u32x4 raw;
        T item[V];
    };

    __shared__ A lds[kWaves];
    __shared__ bool last_block;

    const int tid = threadIdx.x;
    A acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j)
        acc[j] = identity_of<T, Op>();

    // contiguous slice of vectors owned by this workgroup
    const nbh_u32x4 *__restrict__ vin = reinterpret_cast<const nbh_u32x4 *>(in + head);
    const int64_t per = (nvec + gridDim.x - 1) / gridDim.x;
    const int64_t begin = (int64_t)blockIdx.x * per;
    int64_t end = begin + per;
    if (end > nvec)
        end = nvec;

    int64_t i = begin + tid;
    if constexpr (STRIDED) {
        const char *__restrict__ bytes = reinterpret_cast<const char *>(in);
        for (; i + (kUnroll - 1) * kBlock < end; i += kUnroll * kBlock) {
            T v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                v[u] = *reinterpret_cast<const T *>(bytes + (i + u * kBlock) * stride);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                acc[u % V] = Op::apply(acc[u % V], (A)v[u]);
        }
        for (; i < end; i += kBlock)
            acc[0] = Op::apply(acc[0], (A) * reinterpret_cast<const T *>(bytes + i * stride));
    } else if (pieces > 0) {
        const int64_t grid = gridDim.x;
        const int64_t first = grid % 8 == 0 ? (int64_t)(blockIdx.x % 8) * (grid / 8) + blockIdx.x / 8
                                            : (int64_t)blockIdx.x;
        if (first < pieces) {
            const nbh_u32x4 *__restrict__ p = vin + first * kPieceVecs + tid;
            VecT cur[kDeal], nxt[kDeal];
#pragma unroll
            for (int u = 0; u < kDeal; ++u)
                cur[u].raw = __builtin_nontemporal_load(&p[u * kBlock]);
            // every pass fetches without a condition: the waits of the adds can then count
            // the loads of the next piece as still outstanding
            for (int64_t c = first + grid; c < pieces; c += grid) {
                p += grid * kPieceVecs;
#pragma unroll
                for (int u = 0; u < kDeal; ++u)
                    nxt[u].raw = __builtin_nontemporal_load(&p[u * kBlock]);
#pragma unroll
                for (int u = 0; u < kDeal; ++u)
#pragma unroll
                    for (int j = 0; j < V; ++j)
                        acc[j] = Op::apply(acc[j], (A)cur[u].item[j]);
#pragma unroll
                for (int u = 0; u < kDeal; ++u)
                    cur[u] = nxt[u];
                // keeps the eight wavefronts together, so that a piece is asked for as one
                // run of 16 KiB (2^28 float32: 150.4 -> 148.2 us)
                __syncthreads();
            }
#pragma unroll
            for (int u = 0; u < kDeal; ++u)
#pragma unroll
                for (int j = 0; j < V; ++j)
                    acc[j] = Op::apply(acc[j], (A)cur[u].item[j]);
        }
        if (blockIdx.x == gridDim.x - 1)  // fewer than one piece of whole vectors is left over
            for (int64_t k = pieces * kPieceVecs + tid; k < nvec; k += kBlock) {
                VecT v;
                v.raw = __builtin_nontemporal_load(&vin[k]);
#pragma unroll
                for (int j = 0; j < V; ++j)
                    acc[j] = Op::apply(acc[j], (A)v.item[j]);
            }
    } else {
        for (; i + (kUnroll - 1) * kBlock < end; i += kUnroll * kBlock) {
            VecT v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                v[u].raw = __builtin_nontemporal_load(&vin[i + u * kBlock]);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int j = 0; j < V; ++j)
                    acc[j] = Op::apply(acc[j], (A)v[u].item[j]);
        }
        for (; i < end; i += kBlock) {
            VecT v;
            v.raw = __builtin_nontemporal_load(&vin[i]);
#pragma unroll
            for (int j = 0; j < V; ++j)
                acc[j] = Op::apply(acc[j], (A)v.item[j]);
        }
    }
    if constexpr (!STRIDED) {
        // elements outside the aligned body: fewer than 2 V, one per lane of workgroup 0
        if (blockIdx.x == 0) {
            const int64_t tail_begin = head + nvec * V;
            if (tid < head)
                acc[0] = Op::apply(acc[0], (A)in[tid]);
            else if (tail_begin + (tid - head) < n)
                acc[0] = Op::apply(acc[0], (A)in[tail_begin + (tid - head)]);
        }
    }

    A mine = acc[0];
#pragma unroll
    for (int j = 1; j < V; ++j)
        mine = Op::apply(mine, acc[j]);
    A total = block_fold<A, Op>(mine, lds);

    if (gridDim.x == 1) {
        if (tid == 0)
            out[0] = (T)Op::apply(total, (A)init);
        return;
    }

    Word *partials = reinterpret_cast<Word *>(partials_raw);
    if (tid == 0) {
        const Image img = WordsOf<A>::pack(total);
        unsigned t;
        if constexpr (kReleasePublish) {
            // the textbook protocol: ordinary stores, then a ticket drawn with release
            // semantics at agent scope (writes this XCD's L2 back before the ticket moves)
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                partials[(int64_t)blockIdx.x * kWords + w] = img.w[w];
            t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            Word before[kWords];
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                before[w] = __hip_atomic_exchange(&partials[(int64_t)blockIdx.x * kWords + w], img.w[w],
                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the results of the exchanges come from where every XCD looks: once they are
            // back, the partial is in place and the ticket may be drawn
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                asm volatile("" ::"v"(before[w]) : "memory");
            t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        last_block = (t == gridDim.x - 1);
        if (last_block)  // every partial has been published: drop stale cache lines once
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (!last_block)
        return;

    A fin = identity_of<T, Op>();
    for (int k = tid; k < (int)gridDim.x; k += kBlock) {
        Image img;
#pragma unroll
        for (int w = 0; w < kWords; ++w)
            img.w[w] = __hip_atomic_load(&partials[(int64_t)k * kWords + w], __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
        fin = Op::apply(fin, WordsOf<A>::unpack(img));
    }
    fin = block_fold<A, Op>(fin, lds);
    if (tid == 0) {
        out[0] = (T)Op::apply(fin, (A)init);
        // leave the scratch buffer as the caller handed it over
        __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- the reference's order of association ------------------------------------------------
// nbh_reduce_ordered: the same reduction with every operation applied to the same pair of
// values, in the same order, as a run of the reference's kernels (kernels/reduction.py:22-166
// launched as in :233-258), so that floating-point results come out bit for bit - sums,
// products, and what max / min make of NaN and signed zeros.
//
// The reference's order: with F = n rounded down to a multiple of 128 and G = min(F / 128, 64)
// blocks of 128 threads, thread g < S = 128 G folds a[g], a[g + S], a[g + 2 S], ... below F
// from left to right (:70-78); each warp of 32 runs the tree (l, l+16), (l, l+8) ... (l, l+1)
// (:22-41); a block is (w0 op w2) op (w1 op w3) (:88-97); block 0 takes `init` in (:163-164);
// the n - F values behind go through the one-block routine (:99-141: a full warp is a tree,
// the last warp a left fold, the warps a left fold) and so do the partials (:256-258).
//
// At most 8192 chains, each strictly sequential - but every 32 consecutive chains read one
// contiguous piece of 32 items from every "row" of S items, so a workgroup owns one of the
// reference's warps: eight wavefronts load rows of that piece, 16 bytes per lane, two batches
// of eight rounds in flight, and park them in LDS; 32 lanes of a ninth wavefront do nothing
// but add down the parked rows, one chain each.  That wavefront is what the kernel waits for
// (cycle counters around its phases: busy 95 % of the time, the loading wavefronts waiting at
// the barrier half of theirs): 32 768 rows per chain at about 1.4 instructions per row, and a
// wavefront on its own issues an instruction every 2.5 - 3 ns on this part whatever the
// instructions depend on (one wavefront alone in a loop of additions: 4.0 ns per dependent
// addition, 2.9 - 3.1 ns per independent one; the same chain loop alone in a kernel: 3.9 ns
// per row).  One launch: warp results
// are published like the partials of reduce_kernel, the workgroup that draws the last
// ticket does the small rest the way the reference's kernels do.
constexpr int kOrdLoaders = 512;                 // lanes that load and park
constexpr int kOrdThreads = kOrdLoaders + 64;    // and one more wavefront that runs the chains
constexpr int kOrdRounds = 8;      // 16-byte loads in flight per lane
constexpr int kRefWarp = 32, kRefBlock = 128, kRefMaxGrid = 64;

// value of lane `lane + delta` (wave64 lanes; delta < 32)
template <typename A> __device__ __forceinline__ A lane_below(A v, int delta)
{
    constexpr int kDwords = (int)((sizeof(A) + 3) / 4);
    union {
        A a;
        uint32_t w[kDwords];
    } u;
    u.w[kDwords - 1] = 0;
    u.a = v;
#pragma unroll
    for (int k = 0; k < kDwords; ++k)
        u.w[k] = (uint32_t)__shfl_down((int)u.w[k], delta, 64);
    return u.a;
}

// the reference's one-block routine (:99-141) over m < 128 values, by one thread
template <typename A, typename Op> __device__ A ref_one_block(const A *v, int m)
{
    const int nw = (m + kRefWarp - 1) / kRefWarp;
    A result{};
    for (int w = 0; w < nw; ++w) {
        A wres;
        if ((w + 1) * kRefWarp < m) {
            A t[kRefWarp];
            for (int l = 0; l < kRefWarp; ++l)
                t[l] = v[w * kRefWarp + l];
            for (int width = kRefWarp / 2; width; width /= 2)
                for (int l = 0; l < width; ++l)
                    t[l] = Op::apply(t[l], t[l + width]);
            wres = t[0];
        } else {
            wres = v[w * kRefWarp];
            for (int i = 1; i < m - w * kRefWarp; ++i)
                wres = Op::apply(wres, v[w * kRefWarp + i]);
        }
        result = w == 0 ? wres : Op::apply(result, wres);
    }
    return result;
}

template <typename T, typename Op, bool PACKED>
__global__ __launch_bounds__(kOrdThreads) void reduce_ordered_kernel(const T *__restrict__ in, int64_t n,
                                                                     int64_t stride, T init, T *__restrict__ out,
                                                                     uint64_t *__restrict__ partials_raw,
                                                                     unsigned *__restrict__ ticket)
{
    using A = typename AccOf<T, Op>::type;
    using Word = typename WordsOf<A>::Word;
    using Image = typename WordsOf<A>::Image;
    constexpr int kWords = WordsOf<A>::kWords;
    constexpr int E = (int)sizeof(T);
    constexpr int V = 16 / E;                      // items per 16-byte packet
    constexpr int LPR = kRefWarp / V;              // lanes that load one row piece of 32 items
    constexpr int RPP = kOrdLoaders / LPR;         // rows per round of the loading lanes
    constexpr int kBatch = RPP * kOrdRounds;       // rows parked in LDS at a time
    // items per chain and buffer (the rows of a chain lie side by side).  Two more than a
    // power of two: the scattered stores of a wavefront that parks its packets then fall
    // on every LDS bank equally, and a pair of rows can still be read as one aligned piece
    constexpr int kPitch = kBatch + 2;
    // two buffers: the chains take one in while the next batch is parked in the other
    __shared__ __attribute__((aligned(16))) T cols[2][kRefWarp][kPitch];
    __shared__ A small[kRefBlock + 1 + kRefMaxGrid + 1];
    __shared__ bool last_block;

    const int tid = threadIdx.x;
    const int64_t full = (n / kRefBlock) * kRefBlock;
    int64_t ref_grid = full / kRefBlock;
    if (ref_grid > kRefMaxGrid)
        ref_grid = kRefMaxGrid;
    const int64_t S = ref_grid * kRefBlock;        // chains; 0 when n < 128
    const int warps = (int)(S / kRefWarp);         // = workgroups doing chains
    const char *bytes = reinterpret_cast<const char *>(in);

    if ((int)blockIdx.x < warps) {
        // Workgroups are dealt to the eight XCDs in turn, and a workgroup reads the same 128
        // bytes of every row: with warp w on workgroup w an XCD would see addresses that agree
        // in bits 7 - 9, a fraction of its L2 channels.  Each XCD takes a run of neighbouring
        // warps instead: a contiguous 4 KiB of every row.
        int warp = (int)blockIdx.x;
        if (warps % 8 == 0)
            warp = (warp % 8) * (warps / 8) + warp / 8;
        const int64_t c0 = (int64_t)warp * kRefWarp;                    // first chain of this warp
        const int64_t nrows = (full - c0 + S - 1) / S;                   // items per chain
        const bool loader = tid < kOrdLoaders;     // wavefronts 0..7; wavefront 8 runs the chains
        const int lane = tid - kOrdLoaders;         // of the chain wavefront
        const int my_row = tid / LPR, my_piece = tid % LPR;
        A acc{};
        union Pack {
            nbh_u32x4 raw;
            T item[V];
        };
        Pack held[2][kOrdRounds];                   // two batches on their way at any time
        // Every round loads, without a branch around it (rows behind the last are replaced by
        // the last: their copies are parked and never added): eight independent loads per lane
        // that the hardware can have in flight together.
        auto fetch = [&](Pack *into, int64_t first_row) {
            if constexpr (PACKED) {
#pragma unroll
                for (int k = 0; k < kOrdRounds; ++k) {
                    int64_t r = first_row + k * RPP + my_row;
                    r = r < nrows ? r : nrows - 1;
                    into[k].raw = nbh_load16<E, true>(in + (r * S + c0 + my_piece * V));
                }
            } else {
#pragma unroll
                for (int k = 0; k < kOrdRounds; ++k) {
                    int64_t r = first_row + k * RPP + my_row;
                    r = r < nrows ? r : nrows - 1;
                    const int64_t item = r * S + c0 + my_piece * V;
#pragma unroll
                    for (int j = 0; j < V; ++j)
                        into[k].item[j] = *reinterpret_cast<const T *>(bytes + (item + j) * stride);
                }
            }
        };
        auto park = [&](const Pack *from, int buf) {  // lane (row, piece) holds V neighbouring chains' items of one row
#pragma unroll
            for (int k = 0; k < kOrdRounds; ++k)
#pragma unroll
                for (int j = 0; j < V; ++j)
                    cols[buf][my_piece * V + j][k * RPP + my_row] = from[k].item[j];
        };
        auto chains = [&](int buf, int64_t base) {
            if (lane >= 0 && lane < kRefWarp) {
                const T *__restrict__ mine = cols[buf][lane];
                const int count = (int)((nrows - base < kBatch) ? nrows - base : kBatch);
                int r = 0;
                if (base == 0) {                    // a chain starts with its first value, not with an identity
                    acc = (A)mine[0];
                    r = 1;
                }
                if (r < count && (r & 1)) {
                    acc = Op::apply(acc, (A)mine[r]);
                    ++r;
                }
                struct alignas(2 * sizeof(T)) Two {
                    T item[2];
                };
                const Two *__restrict__ pairs = reinterpret_cast<const Two *>(mine);
                // two sets of registers take turns: while one is added up, the other is on its
                // way from LDS (32 dwords a set, whatever the element size)
                constexpr int U = (32 / E) < 1 ? 1 : (32 / E);   // pairs of rows per set
                constexpr int G = 2 * U;                          // rows per set
                auto read = [&](Two *into, int at) {     // `at` is even and not negative
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        into[u] = pairs[((unsigned)at >> 1) + u];
                };
                auto add_up = [&](const Two *from) {
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        acc = Op::apply(acc, (A)from[u].item[0]);
                        acc = Op::apply(acc, (A)from[u].item[1]);
                    }
                };
                // Four register sets take turns: the reads of a set are issued three sets (48 rows of
                // float32) before its rows are added.  A set of reads comes back after some 70 ns, about
                // what the sixteen dependent additions of a set take: with one set ahead the chain
                // waits for the LDS between any two sets (196 -> 193 us for 2^28 float32, 190 us with the fixed trip count for whole batches below; the steady
                // loop is 77 % of the chain wavefront's time, the first and last sets of a batch the
                // rest).  2-byte items keep two sets: their conversions need the registers.  No read
                // in the steady loop is conditional, so every set stays in the registers it was read into.
                if constexpr (E != 2) {
                    // a whole batch in the middle of a chain, which is what all but the first and the
                    // last of a chain's batches are: nothing depends on `count`, the trip count is fixed
                    const bool whole = base != 0 && count == kBatch;
                    if (r + 3 * G <= count) {
                        Two s0[U], s1[U], s2[U], s3[U];
                        const Two *__restrict__ p = pairs + ((unsigned)r >> 1);   // rows r ...: sets lie U pairs apart
                        auto ahead = [&](Two *into, int set) {
#pragma unroll
                            for (int u = 0; u < U; ++u)
                                into[u] = p[set * U + u];
                        };
                        ahead(s0, 0);
                        ahead(s1, 1);
                        ahead(s2, 2);
                        // One step: ask for the set three ahead, wait until all reads but the twelve
                        // youngest (three sets of four 16-byte reads) have come back - that is the set
                        // whose turn it is - and add it up.  The explicit wait stands for the four
                        // the compiler would place, one in front of each read's first use; the barriers
                        // keep its scheduler from gathering the reads of several sets in one place,
                        // which puts them right in front of their first use again.
                        // s_waitcnt immediate: vmcnt 63 and expcnt 7 (no wait), lgkmcnt 12
#define NBH_CHAIN_STEP(NEXT, SET, CUR)                \
    ahead(NEXT, SET);                                  \
    __builtin_amdgcn_sched_barrier(0);                 \
    __builtin_amdgcn_s_waitcnt(0xCC7F);                \
    __builtin_amdgcn_sched_barrier(0);                 \
    add_up(CUR);                                       \
    __builtin_amdgcn_sched_barrier(0);
                        if (whole) {
                            static_assert(kBatch % (4 * G) == 0 && kBatch >= 8 * G, "whole rounds of four sets");
#pragma unroll 1
                            for (int round = 0; round < kBatch / (4 * G) - 1; ++round) {
                                NBH_CHAIN_STEP(s3, 3, s0)
                                NBH_CHAIN_STEP(s0, 4, s1)
                                NBH_CHAIN_STEP(s1, 5, s2)
                                NBH_CHAIN_STEP(s2, 6, s3)
                                p += 4 * U;
                            }
                            ahead(s3, 3);
                            add_up(s0);
                            add_up(s1);
                            add_up(s2);
                            add_up(s3);
                            return;
                        }
                        while (r + 7 * G <= count) {
                            NBH_CHAIN_STEP(s3, 3, s0)
                            NBH_CHAIN_STEP(s0, 4, s1)
                            NBH_CHAIN_STEP(s1, 5, s2)
                            NBH_CHAIN_STEP(s2, 6, s3)
                            r += 4 * G;
                            p += 4 * U;
                        }
#undef NBH_CHAIN_STEP
                        const bool fourth = r + 4 * G <= count;
                        if (fourth)
                            ahead(s3, 3);
                        add_up(s0);
                        add_up(s1);
                        add_up(s2);
                        r += 3 * G;
                        if (fourth) {
                            add_up(s3);
                            r += G;
                        }
                    }
                }
                if (r + G <= count) {                // what is left of whole sets: two sets taking turns
                    Two one[U], other[U];
                    read(one, r);
                    while (r + 3 * G <= count) {
                        read(other, r + G);
                        add_up(one);
                        read(one, r + 2 * G);
                        add_up(other);
                        r += 2 * G;
                    }
                    if (r + 2 * G <= count) {
                        read(other, r + G);
                        add_up(one);
                        add_up(other);
                        r += 2 * G;
                    } else {
                        add_up(one);
                        r += G;
                    }
                }
                for (; r < count; ++r)
                    acc = Op::apply(acc, (A)mine[r]);
            }
        };
        // Two batches are on their way at any time, one per set of registers: a batch is parked
        // as soon as it has arrived (the younger one still travelling), the batch after next is
        // asked for into the registers just emptied, and the chains take the parked batch in
        // meanwhile.  One barrier per batch: whoever parks into a buffer has passed the barrier
        // the chains reached after reading it.  The loading wavefronts and the chain wavefront
        // each run a loop of their own with the same number of barriers (a wavefront is one or the
        // other as a whole): the registers that hold batches on their way and the ones the chains
        // read ahead into are then never live together, which one common loop would make them.
        const int64_t nb = (nrows + kBatch - 1) / kBatch;
        if (loader) {
            fetch(held[0], 0);
            fetch(held[1], kBatch);                 // rows behind the last repeat the last: harmless
            int64_t b = 0;
            for (; b + 1 < nb; b += 2) {
                park(held[0], 0);
                __syncthreads();
                if (b + 2 < nb)
                    fetch(held[0], (b + 2) * kBatch);
                park(held[1], 1);
                __syncthreads();
                if (b + 3 < nb)
                    fetch(held[1], (b + 3) * kBatch);
            }
            if (b < nb) {
                park(held[0], 0);
                __syncthreads();
            }
        } else {
            int64_t b = 0;
            for (; b + 1 < nb; b += 2) {
                __syncthreads();
                chains(0, b * kBatch);
                __syncthreads();
                chains(1, (b + 1) * kBatch);
            }
            if (b < nb) {
                __syncthreads();
                chains(0, b * kBatch);
            }
        }
        if (!loader) {                              // the chain wavefront, whole: the shuffles need its lanes
#pragma unroll
            for (int width = kRefWarp / 2; width; width /= 2) {
                const A other = lane_below(acc, width);
                if (lane < width)
                    acc = Op::apply(acc, other);
            }
            if (lane == 0) {
                Word *partials = reinterpret_cast<Word *>(partials_raw);
                const Image img = WordsOf<A>::pack(acc);
                Word before[kWords];
#pragma unroll
                for (int w = 0; w < kWords; ++w)
                    before[w] = __hip_atomic_exchange(&partials[(int64_t)warp * kWords + w], img.w[w],
                                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int w = 0; w < kWords; ++w)
                    asm volatile("" ::"v"(before[w]) : "memory");  // carried out before anyone goes on
            }
        }
        __syncthreads();                            // the warp's result is published: the ticket may be drawn
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

    // the small rest, laid out as small[0 .. 127]: the values behind `full`, small[128 ...]: the partials
    const int m_tail = (int)(n - full);
    A *tail = small, *part = small + kRefBlock + 1;
    if (tid < m_tail)
        tail[tid] = (A) * reinterpret_cast<const T *>(bytes + (full + tid) * stride);
    if (tid < (int)ref_grid) {                      // block = (w0 op w2) op (w1 op w3)
        const Word *partials = reinterpret_cast<const Word *>(partials_raw);
        A w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            Image img;
#pragma unroll
            for (int k = 0; k < kWords; ++k)
                img.w[k] = __hip_atomic_load(&partials[((int64_t)tid * 4 + q) * kWords + k], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
            w[q] = WordsOf<A>::unpack(img);
        }
        part[tid] = Op::apply(Op::apply(w[0], w[2]), Op::apply(w[1], w[3]));
    }
    __syncthreads();
    if (tid == 0) {
        int np = (int)ref_grid;
        if (ref_grid)
            part[0] = Op::apply(part[0], (A)init);
        if (m_tail) {
            part[np] = ref_one_block<A, Op>(tail, m_tail);
            if (!ref_grid)
                part[0] = Op::apply(part[0], (A)init);
            ++np;
        }
        const A result = np > 1 ? ref_one_block<A, Op>(part, np) : part[0];
        out[0] = (T)result;
        if (gridDim.x > 1)
            __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename T, typename Op>
int launch_ordered(const void *in, int64_t n, int64_t stride, const void *init, void *out, void *scratch,
                   hipStream_t stream)
{
    const uintptr_t addr = (uintptr_t)in;
    if (addr % sizeof(T) != 0 || ((uintptr_t)out) % sizeof(T) != 0 || stride % (int64_t)sizeof(T) != 0)
        return (int)hipErrorInvalidValue;
    int64_t ref_grid = n / kRefBlock;
    if (ref_grid > kRefMaxGrid)
        ref_grid = kRefMaxGrid;
    const int64_t grid = ref_grid ? ref_grid * (kRefBlock / kRefWarp) : 1;  // one workgroup per reference warp
    T init_value;
    __builtin_memcpy(&init_value, init, sizeof(T));
    unsigned *ticket = reinterpret_cast<unsigned *>(scratch);
    uint64_t *partials = reinterpret_cast<uint64_t *>((char *)scratch + kHeaderBytes);
    if (stride == (int64_t)sizeof(T) || n == 1)
        hipLaunchKernelGGL((reduce_ordered_kernel<T, Op, true>), dim3((unsigned)grid), dim3(kOrdThreads), 0, stream,
                           (const T *)in, n, (int64_t)sizeof(T), init_value, (T *)out, partials, ticket);
    else
        hipLaunchKernelGGL((reduce_ordered_kernel<T, Op, false>), dim3((unsigned)grid), dim3(kOrdThreads), 0, stream,
                           (const T *)in, n, stride, init_value, (T *)out, partials, ticket);
    return nbh_launch_status();
}

template <typename T> int launch_ordered_op(int op, const void *in, int64_t n, int64_t stride, const void *init,
                                            void *out, void *scratch, hipStream_t s)
{
    switch (op) {
    case NBH_ADD: return launch_ordered<T, OpAdd>(in, n, stride, init, out, scratch, s);
    case NBH_MUL: return launch_ordered<T, OpMul>(in, n, stride, init, out, scratch, s);
    default: break;
    }
    if constexpr (!IsCplx<T>::value) {
        switch (op) {
        case NBH_MAX: return launch_ordered<T, OpMax>(in, n, stride, init, out, scratch, s);
        case NBH_MIN: return launch_ordered<T, OpMin>(in, n, stride, init, out, scratch, s);
        default: break;
        }
    }
    return (int)hipErrorInvalidValue;
}

template <typename T, typename Op>
int launch(const void *in, int64_t n, int64_t stride, const void *init, void *out, void *scratch,
           hipStream_t stream)
{
    constexpr int V = 16 / (int)sizeof(T);
    const uintptr_t addr = (uintptr_t)in;
    if (addr % sizeof(T) != 0 || ((uintptr_t)out) % sizeof(T) != 0 || stride % (int64_t)sizeof(T) != 0)
        return (int)hipErrorInvalidValue;
    const bool strided = stride != (int64_t)sizeof(T) && n > 1;
    int64_t head = 0, units = n;  // units: vectors when packed, items when strided
    if (!strided) {
        head = (int64_t)(((16 - (addr % 16)) % 16) / sizeof(T));
        if (head > n)
            head = n;
        units = (n - head) / V;
    }

    const int64_t per_block = (int64_t)kBlock * kUnroll;
    int64_t grid = (units + per_block - 1) / per_block;
    // Small inputs are latency, not bandwidth: spread them over up to 32 workgroups with
    // one load per lane (256 KiB: 4.1 -> 3.8 us, against 2.4 - 2.7 us for an empty kernel).
    if (grid < 32) {
        grid = (units + kBlock - 1) / kBlock;
        if (grid > 32)
            grid = 32;
    }
    int64_t cap = (int64_t)nbh_cu_count() * kGridPerCU;
    constexpr int64_t kSlots = (int64_t)kMaxGrid * 8 / (sizeof(T) > 8 ? 16 : 8);  // partials that fit the scratch
    if (cap > kSlots)
        cap = kSlots;
    if (grid > cap)
        grid = cap;
    if (grid < 1)
        grid = 1;

    // dealt pieces from sixteen per workgroup on (128 MiB on 256 compute units: 2 % faster than
    // slices there, 3 % at 1 GiB, 13 - 17 % where the length is no multiple of anything; at
    // 64 MiB slices are still 1.5 % ahead), slices below
    int64_t pieces = strided ? 0 : units / kPieceVecs;
    if (pieces < 16 * grid)
        pieces = 0;

    T init_value;
    __builtin_memcpy(&init_value, init, sizeof(T));
    unsigned *ticket = reinterpret_cast<unsigned *>(scratch);
    uint64_t *partials = reinterpret_cast<uint64_t *>((char *)scratch + kHeaderBytes);
    if (strided)
        hipLaunchKernelGGL((reduce_kernel<T, Op, true>), dim3((unsigned)grid), dim3(kBlock), 0, stream,
                           (const T *)in, n, head, units, pieces, stride, init_value, (T *)out, partials, ticket);
    else
        hipLaunchKernelGGL((reduce_kernel<T, Op, false>), dim3((unsigned)grid), dim3(kBlock), 0, stream,
                           (const T *)in, n, head, units, pieces, stride, init_value, (T *)out, partials, ticket);
    return nbh_launch_status();
}

template <typename T>
int launch_op(int op, const void *in, int64_t n, int64_t stride, const void *init, void *out, void *scratch,
              hipStream_t s)
{
    switch (op) {
    case NBH_ADD: return launch<T, OpAdd>(in, n, stride, init, out, scratch, s);
    case NBH_MUL: return launch<T, OpMul>(in, n, stride, init, out, scratch, s);
    case NBH_MAX: return launch<T, OpMax>(in, n, stride, init, out, scratch, s);
    case NBH_MIN: return launch<T, OpMin>(in, n, stride, init, out, scratch, s);
    default: break;
    }
    if constexpr (std::is_integral<T>::value) {
        switch (op) {
        case NBH_AND: return launch<T, OpAnd>(in, n, stride, init, out, scratch, s);
        case NBH_OR: return launch<T, OpOr>(in, n, stride, init, out, scratch, s);
        case NBH_XOR: return launch<T, OpXor>(in, n, stride, init, out, scratch, s);
        default: break;
        }
    }
    return (int)hipErrorInvalidValue;
}

// complex elements: sums and products only (there is no order to take a maximum by)
template <typename T>
int launch_op_complex(int op, const void *in, int64_t n, int64_t stride, const void *init, void *out,
                      void *scratch, hipStream_t s)
{
    switch (op) {
    case NBH_ADD: return launch<T, OpAdd>(in, n, stride, init, out, scratch, s);
    case NBH_MUL: return launch<T, OpMul>(in, n, stride, init, out, scratch, s);
    default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace

extern "C" {

size_t nbh_reduce_scratch_bytes(void) { return kScratchBytes; }

int nbh_reduce(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
               void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    if (!in || !init || !out || !scratch || n < 1 || scratch_bytes < kScratchBytes ||
        ((uintptr_t)scratch) % 8 != 0)
        return (int)hipErrorInvalidValue;
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);
    switch (dtype) {
    case NBH_I8: return launch_op<int8_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_I16: return launch_op<int16_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_I32: return launch_op<int32_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_I64: return launch_op<int64_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_U8: return launch_op<uint8_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_U16: return launch_op<uint16_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_U32: return launch_op<uint32_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_U64: return launch_op<uint64_t>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_F32: return launch_op<float>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_F64: return launch_op<double>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_F16: return launch_op<Half>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_C64: return launch_op_complex<Cplx<float>>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_C128: return launch_op_complex<Cplx<double>>(op, in, n, in_stride, init, out, scratch, s);
    default: return (int)hipErrorInvalidValue;
    }
}

int nbh_reduce_ordered(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                       void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    if (!in || !init || !out || !scratch || n < 1 || scratch_bytes < kScratchBytes ||
        ((uintptr_t)scratch) % 8 != 0)
        return (int)hipErrorInvalidValue;
    hipStream_t s = nbh_hip_stream(stream);
    nbh_stream_report report(s);
    switch (dtype) {
    case NBH_F32: return launch_ordered_op<float>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_F64: return launch_ordered_op<double>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_F16: return launch_ordered_op<Half>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_C64: return launch_ordered_op<Cplx<float>>(op, in, n, in_stride, init, out, scratch, s);
    case NBH_C128: return launch_ordered_op<Cplx<double>>(op, in, n, in_stride, init, out, scratch, s);
    default:
        // integers and booleans: every order of association gives the same bits
        return nbh_reduce(op, dtype, in, n, in_stride, init, out, scratch, scratch_bytes, stream);
    }
}

}  // extern "C"

// ---- the same reduction for callers that cannot allocate ------------------------------
// Ticket and partials live in an array inside the code object: every device the library
// runs on holds its own copy, at its own address, from the moment the code object is
// loaded there until the process ends.  The array's name is a host-side stand-in; the
// address kernels can use is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

constexpr int kMaxDevices = 64;

// What the host knows about one device's copy of `scratch`.
struct StaticScratch {
    std::atomic<void *> address{nullptr};  // device address of `scratch`
    hipEvent_t done = nullptr;             // recorded after the latest call's kernel
    hipStream_t last = nullptr;            // the stream of that call
    bool have_last = false;
    bool dirty = false;                    // a call failed after its launch: the ticket may not be back at zero
    std::mutex mu;                         // the four fields above
};
StaticScratch g_static[kMaxDevices];
std::mutex g_static_mu;

// The current device's entry, its array looked up and its event made on first use.
int static_scratch(StaticScratch **out)
{
    int dev = -1;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return (int)hipErrorInvalidDevice;
    StaticScratch &st = g_static[dev];
    if (!st.address.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_static_mu);
        if (!st.address.load(std::memory_order_relaxed)) {
            void *p = nullptr;
            NBH_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            if (!p)
                return (int)hipErrorInvalidSymbol;
            NBH_TRY(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
            // the array is zero when the code object is loaded, and every reduction hands
            // the ticket back at zero: nothing to clear here
            st.address.store(p, std::memory_order_release);
        }
    }
    *out = &st;
    return 0;
}

__global__ void clear_header_kernel(unsigned *header)
{
    header[threadIdx.x] = 0u;
}

bool is_null_stream(hipStream_t s) { return s == nullptr || s == hipStreamLegacy; }

}  // namespace

extern "C" int nbh_reduce_noalloc(int op, int dtype, const void *in, int64_t n, int64_t in_stride,
                                  const void *init, void *out, nbh_stream_t stream)
{
    if (n > NBH_REDUCE_NOALLOC_MAX_ITEMS)
        return (int)hipErrorInvalidValue;  // stated limit of this entry point; nothing is launched
    StaticScratch *st = nullptr;
    if (int rc = static_scratch(&st))
        return rc;
    void *ptr = st->address.load(std::memory_order_relaxed);
    hipStream_t s = nbh_hip_stream(stream);
    // Under stream capture nothing runs now: the graph's own edges order the replays, and
    // event queries are not allowed, so the bookkeeping below is left out.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = !is_null_stream(s) && s != hipStreamPerThread &&
                           hipStreamIsCapturing(s, &capture) == hipSuccess && capture == hipStreamCaptureStatusActive;
    if (capturing)
        return nbh_reduce(op, dtype, in, n, in_stride, init, out, ptr, kScratchBytes, stream);
    std::lock_guard<std::mutex> hold(st->mu);
    // Calls on one stream run one after the other; the null stream waits for the others and
    // they for it.  A call on ANOTHER stream while the previous call's kernel has not finished
    // would share the ticket and the partials with it: refused instead of giving wrong results.
    if (st->have_last && st->last != s && !is_null_stream(s) && !is_null_stream(st->last)) {
        const hipError_t state = hipEventQuery(st->done);
        if (state != hipSuccess)
            return (int)state;  // hipErrorNotReady: still running
    }
    if (st->dirty) {  // a failed call may have left tickets drawn: start from zero again (no allocation: one launch)
        hipLaunchKernelGGL(clear_header_kernel, dim3(1), dim3(kHeaderBytes / sizeof(unsigned)), 0, s, (unsigned *)ptr);
        if (int rc = nbh_launch_status())
            return rc;
        st->dirty = false;
    }
    const int rc = nbh_reduce(op, dtype, in, n, in_stride, init, out, ptr, kScratchBytes, stream);
    if (rc) {
        st->dirty = true;
        return rc;
    }
    if (hipEventRecord(st->done, s) == hipSuccess) {
        st->last = s;
        st->have_last = true;
    }
    return 0;
}

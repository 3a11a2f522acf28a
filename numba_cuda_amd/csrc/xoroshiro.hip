// xoroshiro128+ (2016 constants 55/14/36) on gfx950: parallel state initialisation
// and bulk uniform / normal draws.
//
// State initialisation.  The reference builds states[i] = jump^i(states[0]) as one
// sequential chain on the CPU.  `next` is linear over GF(2), so `jump` (2^64 steps)
// is a 128x128 bit matrix J; the host tabulates J^(2^k), k = 0..63, once per
// process.  A wavefront owns 4096 consecutive states: lane l starts at
// J^(first + l) * s and keeps stepping by J^64, so every step of the wavefront
// writes 64 consecutive states (1 KiB).  Three kinds of matrix-vector product:
//   * J^first (bits >= 12 of the index, the same vector in every lane): the 64
//     lanes split the 128 columns between them and XOR-reduce across the
//     wavefront - about 40 instructions per product instead of 1150;
//   * J^l, l < 64 (the same vector in every lane, a different matrix per lane): byte
//     tables of all 64 matrices in global memory, laid out [position][byte][lane], so that
//     each of the sixteen look-ups of a wavefront is one 1 KiB run (4 MiB per device);
//   * the J^64 step (a different vector per lane): byte tables in LDS, sixteen look-ups
//     of 16 bytes per step (64 KiB per 1024-thread workgroup);
// The number of steps a wavefront makes is chosen at launch: small arrays are spread over
// many wavefronts of few steps (a single step needs no table in LDS at all).
//
// Draws.  Each lane owns one generator whose 128-bit state stays in registers.
// The reference's layout out[t*count + i] gives every lane its own run of `count`
// values, so values are parked in LDS for a round and written back with the run
// index fastest: every store instruction of a wavefront covers whole 128-byte lines.
// The Box-Muller normals take their logarithm and cosine from boxmuller_math.h.
//
// HBM roofline: out bytes written + 2 * 16 bytes of state per generator.
#include "common.h"
#include "boxmuller_math.h"

#include <mutex>
#include <type_traits>

namespace {

// ---- host side: the jump matrices ---------------------------------------------

struct U128 {
    uint64_t s0, s1;
};

inline uint64_t rotl_h(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

inline void next_h(U128 &s)
{
    uint64_t a = s.s0, b = s.s1 ^ s.s0;
    s.s0 = rotl_h(a, 55) ^ b ^ (b << 14);
    s.s1 = rotl_h(b, 36);
}

inline U128 jump_h(U128 s)
{
    const uint64_t poly[2] = {0xBEAC0467EBA5FACBull, 0xD86B048B86AA9922ull};
    U128 acc = {0, 0};
    for (int w = 0; w < 2; ++w)
        for (int b = 0; b < 64; ++b) {
            if ((poly[w] >> b) & 1) {
                acc.s0 ^= s.s0;
                acc.s1 ^= s.s1;
            }
            next_h(s);
        }
    return acc;
}

constexpr int kPowers = 64;
// table[k][c] = column c of J^(2^k): the image of the state with only bit c set
// (bits 0..63 live in s0, bits 64..127 in s1).
struct JumpTable {
    U128 col[kPowers][128];
    // lut8[p][v]: XOR of columns 8p+b of J^64 over the set bits b of v
    U128 lut8[16][256];
    // lane8[p][v][l]: XOR of columns 8p+b of J^l over the set bits b of v, l = 0 .. 63 (4 MiB):
    // J^l applied to a vector is the XOR of sixteen entries, and when the 64 lanes of a wavefront
    // hold the SAME vector, lane l wanting J^l of it, entry (p, v) of all lanes is one 1 KiB run
    U128 lane8[16][256][64];
};
constexpr int kLutEntries = 16 * 256;

inline U128 apply_h(const U128 *m, U128 v)
{
    U128 r = {0, 0};
    for (int b = 0; b < 64; ++b) {
        if ((v.s0 >> b) & 1) {
            r.s0 ^= m[b].s0;
            r.s1 ^= m[b].s1;
        }
        if ((v.s1 >> b) & 1) {
            r.s0 ^= m[64 + b].s0;
            r.s1 ^= m[64 + b].s1;
        }
    }
    return r;
}

const JumpTable &jump_table()
{
    static JumpTable *table = nullptr;
    static std::once_flag once;
    std::call_once(once, [] {
        JumpTable *t = new JumpTable;
        for (int c = 0; c < 128; ++c) {
            U128 e = {c < 64 ? (1ull << c) : 0, c < 64 ? 0 : (1ull << (c - 64))};
            t->col[0][c] = jump_h(e);
        }
        for (int k = 1; k < kPowers; ++k)  // square: column c of M*M is M applied to column c of M
            for (int c = 0; c < 128; ++c)
                t->col[k][c] = apply_h(t->col[k - 1], t->col[k - 1][c]);
        // the columns of J^l, l = 0 .. 63, one power after the other, and their byte tables
        {
            U128 power[128];
            for (int c = 0; c < 128; ++c)
                power[c] = U128{c < 64 ? (1ull << c) : 0, c < 64 ? 0 : (1ull << (c - 64))};
            for (int l = 0; l < 64; ++l) {
                for (int p = 0; p < 16; ++p) {
                    t->lane8[p][0][l] = U128{0, 0};
                    for (int v = 1; v < 256; ++v) {
                        const U128 rest = t->lane8[p][v & (v - 1)][l], col = power[8 * p + __builtin_ctz(v)];
                        t->lane8[p][v][l] = U128{rest.s0 ^ col.s0, rest.s1 ^ col.s1};
                    }
                }
                for (int c = 0; c < 128; ++c)
                    power[c] = apply_h(t->col[0], power[c]);
            }
        }
        for (int p = 0; p < 16; ++p)
            for (int v = 0; v < 256; ++v) {
                U128 x = {0, 0};
                for (int b = 0; b < 8; ++b)
                    if ((v >> b) & 1) {
                        x.s0 ^= t->col[6][8 * p + b].s0;
                        x.s1 ^= t->col[6][8 * p + b].s1;
                    }
                t->lut8[p][v] = x;
            }
        table = t;
    });
    return *table;
}

// Device copy of the table, one per device, made on first use and kept for the
// life of the process (4.2 MiB: matrix columns and lookup tables).
int device_table(const U128 **out)
{
    constexpr int kMaxDev = 64;
    static const U128 *cache[kMaxDev] = {};
    static std::mutex mu;
    int dev = 0;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDev)
        return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (!cache[dev]) {
        const JumpTable &t = jump_table();
        void *d = nullptr;
        NBH_TRY(hipMalloc(&d, sizeof(JumpTable)));
        hipError_t e = hipMemcpy(d, &t, sizeof(JumpTable), hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(d);
            return (int)e;
        }
        cache[dev] = (const U128 *)d;
    }
    *out = cache[dev];
    return 0;
}

// Device copy of the logarithm table of the normal generators (3 KiB), one per
// device, made on first use and kept for the life of the process.
int device_log_table(const bm::LogTable **out)
{
    constexpr int kMaxDev = 64;
    static const bm::LogTable *cache[kMaxDev] = {};
    static std::mutex mu;
    int dev = 0;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDev)
        return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (!cache[dev]) {
        bm::LogTable host;
        bm::build_log_table(host);
        void *d = nullptr;
        NBH_TRY(hipMalloc(&d, sizeof(bm::LogTable)));
        hipError_t e = hipMemcpy(d, &host, sizeof(bm::LogTable), hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(d);
            return (int)e;
        }
        cache[dev] = (const bm::LogTable *)d;
    }
    *out = cache[dev];
    return 0;
}

// ---- device side ------------------------------------------------------------------

// The generator step on 32-bit halves: the 64-bit rotations are funnel shifts of register
// pairs (v_alignbit_b32), two instructions each; the plain shift is one 64-bit shift
// instruction (shl64 below).
__device__ __forceinline__ uint32_t funnel(uint32_t hi, uint32_t lo, int right)
{
    return __builtin_amdgcn_alignbit(hi, lo, right);  // bits [right, right + 32) of hi:lo
}

// Shifts of a register pair by a constant in ONE instruction.  Left to itself the compiler
// splits them into a funnel shift and a 32-bit shift.
template <int N> __device__ __forceinline__ uint64_t shl64(uint64_t x)
{
    uint64_t r;
    asm("v_lshlrev_b64 %0, %1, %2" : "=v"(r) : "n"(N), "v"(x));
    return r;
}
template <int N> __device__ __forceinline__ uint64_t shr64(uint64_t x)
{
    uint64_t r;
    asm("v_lshrrev_b64 %0, %1, %2" : "=v"(r) : "n"(N), "v"(x));
    return r;
}

__device__ __forceinline__ uint64_t next_d(uint64_t &s0, uint64_t &s1)
{
    const uint64_t r = s0 + s1;
    const uint32_t a_lo = (uint32_t)s0, a_hi = (uint32_t)(s0 >> 32);
    const uint32_t t_lo = a_lo ^ (uint32_t)s1, t_hi = a_hi ^ (uint32_t)(s1 >> 32);
    // rotl(s0, 55): swap halves, then rotate left by 23
    const uint32_t r55_hi = funnel(a_lo, a_hi, 9), r55_lo = funnel(a_hi, a_lo, 9);
    // t << 14: one 64-bit shift costs what one v_alignbit_b32 does (1.8 ns per wavefront and
    // SIMD), a funnel for the high word plus a 32-bit shift for the low one 2.9 ns
    const uint64_t sh = shl64<14>(((uint64_t)t_hi << 32) | t_lo);
    const uint32_t sh_hi = (uint32_t)(sh >> 32), sh_lo = (uint32_t)sh;
    // rotl(t, 36): swap halves, then rotate left by 4
    const uint32_t r36_hi = funnel(t_lo, t_hi, 28), r36_lo = funnel(t_hi, t_lo, 28);
    // a ^ b ^ c in one instruction (truth table 0x96); the compiler does not form it itself
    // (the builtin returns int: without the casts the low word would be sign-extended)
    const uint32_t n_hi = (uint32_t)__builtin_amdgcn_bitop3_b32(r55_hi, t_hi, sh_hi, 0x96);
    const uint32_t n_lo = (uint32_t)__builtin_amdgcn_bitop3_b32(r55_lo, t_lo, sh_lo, 0x96);
    s0 = ((uint64_t)n_hi << 32) | n_lo;
    s1 = ((uint64_t)r36_hi << 32) | r36_lo;
    return r;
}

constexpr int kInitSteps = 64;  // consecutive 64-state groups produced by one wavefront, at most

// XOR of a value over the 64 lanes, returned in every lane.
__device__ __forceinline__ uint32_t wave_xor32(uint32_t v)
{
    v ^= (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0xB1, 0xF, 0xF, false);   // lane ^ 1
    v ^= (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x4E, 0xF, 0xF, false);   // lane ^ 2
    v ^= (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x141, 0xF, 0xF, false);  // other quad of 8
    v ^= (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x140, 0xF, 0xF, false);  // other half of 16
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 0) ^ (uint32_t)__builtin_amdgcn_readlane((int)v, 16) ^
           (uint32_t)__builtin_amdgcn_readlane((int)v, 32) ^ (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
}
__device__ __forceinline__ uint64_t wave_xor64(uint64_t v)
{
    return ((uint64_t)wave_xor32((uint32_t)(v >> 32)) << 32) | wave_xor32((uint32_t)v);
}

// r = M * (s0, s1) when every lane holds the SAME vector: lane l contributes
// columns l and 64 + l, the wavefront XORs the contributions together.
__device__ __forceinline__ void apply_shared(const U128 *__restrict__ m, int lane, uint64_t &s0, uint64_t &s1)
{
    const U128 ca = m[lane], cb = m[64 + lane];
    const uint64_t ma = 0 - ((s0 >> lane) & 1), mb = 0 - ((s1 >> lane) & 1);
    const uint64_t p0 = (ca.s0 & ma) ^ (cb.s0 & mb);
    const uint64_t p1 = (ca.s1 & ma) ^ (cb.s1 & mb);
    s0 = wave_xor64(p0);
    s1 = wave_xor64(p1);
}

typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));

constexpr int kTabBlock = 1024;

// One application of J^64 to every lane's own state, 16 look-ups of 8 bits each, WITHOUT bank
// conflicts.  A wavefront's lanes hold unrelated states, so look-ups into one table hit random
// banks: measured, 61 % of the LDS's active cycles were conflict stalls.  The banks repeat
// every 256 bytes and a 128-bit read takes four of them, so the tables are laid out
// [value][position]: row v (256 bytes) holds the 16 entries that value v selects, position p
// in banks 4p .. 4p+3.  In look-up round t lane l takes position p = t XOR (l mod 16): over
// the 16 rounds every lane visits every position, and in any one round the 16 lanes of a row
// of the wavefront read 16 different positions - 16 different groups of banks, whatever the
// values.  Which byte of the state a lane needs in round t then depends on the lane; the state
// is permuted once per step so that round t finds its byte in a fixed place: byte i of word j
// of the permuted state is byte i ^ (l & 3) of word j ^ ((l >> 2) & 3) of the state - the words
// 0 <-> 2, 1 <-> 3 by conditional moves, the rest by one two-source v_perm_b32 per word.
// The address of round t is (value << 8) | ((t ^ l) << 4): the low byte never changes, so each
// round keeps its address register and a step only moves the value into byte 1 of it
// (one sub-dword move per look-up instead of an extraction and a merge).
struct LaneOrder {
    uint32_t select;   // v_perm selector for (other word, this word): byte and word exchange in one
    bool swap2;        // exchange words 0 <-> 2, 1 <-> 3 of the 128-bit state
    uint32_t at[16];   // address of round t within the table: byte 0 = (t ^ l16) << 4, byte 1 = the value
};

__device__ __forceinline__ LaneOrder lane_order(int lane)
{
    const uint32_t l16 = (uint32_t)lane & 15u;
    LaneOrder o;
    // selector bytes 0 - 3 pick from the second source, 4 - 7 from the first
    o.select = (0x03020100u ^ ((l16 & 3u) * 0x01010101u)) | ((l16 & 4u) ? 0x04040404u : 0u);
    o.swap2 = (l16 & 8u) != 0;
#pragma unroll
    for (int t = 0; t < 16; ++t)
        o.at[t] = (l16 << 4) ^ (uint32_t)(t << 4);
    return o;
}

// byte K of `w` into byte 1 of `at`, the other bytes of `at` kept
template <int K> __device__ __forceinline__ void put_row(uint32_t &at, uint32_t w)
{
    if constexpr (K == 0)
        asm("v_mov_b32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_0" : "+v"(at) : "v"(w));
    else if constexpr (K == 1)
        asm("v_mov_b32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1" : "+v"(at) : "v"(w));
    else if constexpr (K == 2)
        asm("v_mov_b32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_2" : "+v"(at) : "v"(w));
    else
        asm("v_mov_b32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3" : "+v"(at) : "v"(w));
}

__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c)
{
    return (uint32_t)__builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
}

// lut8: the J^64 table in LDS as [256 values][16 positions] of 16-byte entries
template <int T> __device__ __forceinline__ void put_rows(LaneOrder &o, const uint32_t (&r)[4])
{
    if constexpr (T < 16) {
        put_row<(T & 3)>(o.at[T], r[T >> 2]);
        put_rows<T + 1>(o, r);
    }
}

__device__ __forceinline__ void apply_lut8_spread(const unsigned char *__restrict__ lut8, LaneOrder &o,
                                                  uint64_t &s0, uint64_t &s1)
{
    const uint32_t d0 = (uint32_t)s0, d1 = (uint32_t)(s0 >> 32), d2 = (uint32_t)s1, d3 = (uint32_t)(s1 >> 32);
    const uint32_t f0 = o.swap2 ? d2 : d0, f1 = o.swap2 ? d3 : d1, f2 = o.swap2 ? d0 : d2, f3 = o.swap2 ? d1 : d3;
    uint32_t r[4];
    r[0] = __builtin_amdgcn_perm(f1, f0, o.select);
    r[1] = __builtin_amdgcn_perm(f0, f1, o.select);
    r[2] = __builtin_amdgcn_perm(f3, f2, o.select);
    r[3] = __builtin_amdgcn_perm(f2, f3, o.select);
    put_rows<0>(o, r);
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    u32x4_t got[16];
#pragma unroll
    for (int t = 0; t < 16; ++t)
        got[t] = *reinterpret_cast<const u32x4_t *>(lut8 + o.at[t]);
    uint32_t acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        uint32_t a = xor3(got[0][c], got[1][c], got[2][c]);
        a = xor3(a, got[3][c], got[4][c]);
        a = xor3(a, got[5][c], got[6][c]);
        a = xor3(a, got[7][c], got[8][c]);
        a = xor3(a, got[9][c], got[10][c]);
        a = xor3(a, got[11][c], got[12][c]);
        a = xor3(a, got[13][c], got[14][c]);
        acc[c] = a ^ got[15][c];
    }
    s0 = ((uint64_t)acc[1] << 32) | acc[0];
    s1 = ((uint64_t)acc[3] << 32) | acc[2];
}

__global__ __launch_bounds__(kTabBlock) void init_states_tables_kernel(uint64_t *__restrict__ states, int64_t n,
                                                                       uint64_t b0, uint64_t b1,
                                                                       const U128 *__restrict__ table,
                                                                       const u64x2_t *__restrict__ lut_global,
                                                                       const u64x2_t *__restrict__ lane_global,
                                                                       int steps)
{
    // `steps` groups of 64 consecutive states per wavefront (1 .. kInitSteps, the host's choice:
    // small arrays are spread over many wavefronts of few steps).  64 KiB: the byte tables of
    // J^64, transposed to [256 values][16 positions]; not needed for a single step.
    __shared__ u64x2_t lut[kLutEntries];
    if (steps > 1)
        for (int i = threadIdx.x; i < kLutEntries; i += kTabBlock)
            lut[(i & 255) * 16 + (i >> 8)] = lut_global[i];  // lut8[p][value] in global memory

    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kTabBlock / 64) + (threadIdx.x >> 6);
    const int64_t first = wave * (64 * (int64_t)steps);
    uint64_t s0 = b0, s1 = b1;
    if (first < n) {
        const uint64_t hi = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(first >> 6)) |
                            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(first >> 38)) << 32);
        for (int k = 6; k < kPowers; ++k)
            if ((hi >> (k - 6)) & 1)
                apply_shared(table + (size_t)k * 128, lane, s0, s1);
        // J^lane: every lane still holds the same vector, so byte p of it picks, for all lanes
        // at once, one 1 KiB run of the table [position][byte][lane]: sixteen coalesced loads
        // and their XOR, where six conditional 128 x 128 products through 4-bit tables in LDS
        // cost 1200 vector instructions and 48 KiB of LDS (2^24 states: 77.4 -> 71.8 us per launch)
        const uint64_t u0 = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s0) |
                            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(s0 >> 32)) << 32);
        const uint64_t u1 = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s1) |
                            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(s1 >> 32)) << 32);
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
        u32x4_t part[16];
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const int byte = (int)(((p < 8 ? u0 : u1) >> (8 * (p & 7))) & 255);
            part[p] = *reinterpret_cast<const u32x4_t *>(lane_global + ((size_t)(p * 256 + byte) * 64 + lane));
        }
        uint32_t acc[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t a = xor3(part[0][c], part[1][c], part[2][c]);
            a = xor3(a, part[3][c], part[4][c]);
            a = xor3(a, part[5][c], part[6][c]);
            a = xor3(a, part[7][c], part[8][c]);
            a = xor3(a, part[9][c], part[10][c]);
            a = xor3(a, part[11][c], part[12][c]);
            a = xor3(a, part[13][c], part[14][c]);
            acc[c] = a ^ part[15][c];
        }
        s0 = ((uint64_t)acc[1] << 32) | acc[0];
        s1 = ((uint64_t)acc[3] << 32) | acc[2];
    }
    __syncthreads();
    if (first >= n)
        return;
    const unsigned char *__restrict__ step = reinterpret_cast<const unsigned char *>(lut);  // J^64
    LaneOrder order = lane_order(lane);
    if (first + 64 * (int64_t)steps <= n) {  // a whole run: nothing to test on the way
        u64x2_t *dst = reinterpret_cast<u64x2_t *>(states + 2 * (first + lane));
#pragma unroll 1
        for (int g = 0; g < steps - 1; ++g) {
            const u64x2_t v = {s0, s1};
            dst[(int64_t)g * 64] = v;
            apply_lut8_spread(step, order, s0, s1);
        }
        const u64x2_t v = {s0, s1};
        dst[(int64_t)(steps - 1) * 64] = v;
        return;
    }
    for (int g = 0; g < steps; ++g) {
        if (first + (int64_t)g * 64 >= n)
            break;
        const int64_t idx = first + (int64_t)g * 64 + lane;
        if (idx < n) {
            u64x2_t v = {s0, s1};
            *reinterpret_cast<u64x2_t *>(states + 2 * idx) = v;
        }
        if (g + 1 < steps)
            apply_lut8_spread(step, order, s0, s1);
    }
}

// ---- draws -------------------------------------------------------------------------

// (x >> 11) * 2^-53 without integer-to-double conversions.  With m = x >> 11 =
// hi * 2^32 + lo (hi < 2^21), the doubles whose bit patterns are
//   {0x41E00000, hi} = 2^31 + hi * 2^-21      and      {0x3FE00000, lo} = 2^-1 + lo * 2^-53
// carry the two halves in their mantissas; (first - (2^31 + 2^-1)) + second is
// m * 2^-53, and both additions are exact (every intermediate is a multiple of
// 2^-53 below 1 in magnitude).
// The two halves of m are made by two 32-bit instructions, each writing the low word of its
// double directly (one 64-bit shift would leave them in a register pair, to be moved apart).
__device__ __forceinline__ double unit_double(uint64_t x)
{
    const uint32_t x_lo = (uint32_t)x, x_hi = (uint32_t)(x >> 32);
    const uint32_t m_hi = x_hi >> 11, m_lo = funnel(x_hi, x_lo, 11);
    const double a = __hiloint2double((int)0x41E00000, (int)m_hi);
    const double b = __hiloint2double((int)0x3FE00000, (int)m_lo);
    return (a - 2147483648.5) + b;
}

struct UniformF32 {
    using value_type = float;
    static constexpr bool kHeavy = false;
    template <typename Tab = const bm::LogTable *>
    static __device__ __forceinline__ float draw(uint64_t &s0, uint64_t &s1, Tab = Tab())
    {
        // the exact value in double, then one rounding to float
        return (float)unit_double(next_d(s0, s1));
    }
};
struct UniformF64 {
    using value_type = double;
    static constexpr bool kHeavy = false;
    template <typename Tab = const bm::LogTable *>
    static __device__ __forceinline__ double draw(uint64_t &s0, uint64_t &s1, Tab = Tab())
    {
        return unit_double(next_d(s0, s1));
    }
};
// Box-Muller, cosine branch.  The float32 variant works in float32 throughout;
// log and cos are evaluated in double and rounded once, which is the closest
// available stand-in for correctly rounded float32 routines.
struct NormalF32 {
    using value_type = float;
    static constexpr bool kHeavy = true;
    template <typename Tab> static __device__ __forceinline__ float draw(uint64_t &s0, uint64_t &s1, Tab tab)
    {
        const float u1 = UniformF32::draw(s0, s1);
        const float u2 = UniformF32::draw(s0, s1);
        const float two_pi = 6.283185307179586f;
        const float lg2 = bm::bm_log2x_f32_rounded(u1, tab);  // 2 log(u1), exactly twice the float32 logarithm
        const float r = sqrtf(-lg2);
        const float c = (float)bm::bm_cos_2pi((double)(two_pi * u2), tab);
        return r * c;
    }
};
// The float64 variant still draws float32 uniforms and takes the logarithm of a
// float32 (so its result is a float32); the square root and cosine are float64.
struct NormalF64 {
    using value_type = double;
    static constexpr bool kHeavy = true;
    template <typename Tab> static __device__ __forceinline__ double draw(uint64_t &s0, uint64_t &s1, Tab tab)
    {
        const float u1 = UniformF32::draw(s0, s1);
        const float u2 = UniformF32::draw(s0, s1);
        const double two_pi = 6.283185307179586;
        const float lg2 = bm::bm_log2x_f32_rounded(u1, tab);  // 2 log(u1), exactly twice the float32 logarithm
        // (-sqrt(-2 log u1)) * (-cos(2 pi u2)): both factors negated, which costs nothing, where
        // negating 2 log(u1) for the square root would cost an instruction
        const double neg_r = bm::bm_neg_sqrt_of_neg((double)lg2);
        const double neg_c = bm::bm_cos_2pi<true>(two_pi * (double)u2, tab);
        return neg_r * neg_c;
    }
};

constexpr int kFillBlock = 256;

// Output packets of 16 bytes are only guaranteed the alignment of one value (runs
// start at t*count, which need not be a multiple of four values): nbh_store16.
typedef nbh_u32x4 u32x4;

// Each wavefront works on its own 64 generators and its own slice of LDS, so
// wavefronts never wait for one another.  A round is 128 bytes per generator: the
// lane draws them into registers, parks them in its LDS row with 128-bit writes
// (row pitch 144 bytes keeps those conflict-free), and the wavefront then reads
// the rows back eight lanes per row and stores 16 bytes per lane, so one store
// instruction covers eight whole 128-byte lines.  Within a wavefront LDS accesses
// execute in program order; the wavefront-scope fences only keep the compiler
// from moving them across the hand-over.
// NT: non-temporal stores, chosen by the host when every run starts on a 128-byte line
// (they are slower than cached stores when the packets of a wavefront straddle lines:
// 31 float64 per generator 3.6 ms against 2.0 ms).  Runs off the lines that are longer
// than a line and a half go to fill_ring_kernel below (2^24 generators x 100 float64:
// 5.1 ms here, 2.55 ms there); shorter ones and the compute-bound normal draws stay here.
template <typename Gen, bool NT, int LINES>
__global__ __launch_bounds__(kFillBlock) void fill_kernel(uint64_t *__restrict__ states, int64_t n,
                                                          typename Gen::value_type *__restrict__ out,
                                                          int64_t count, const bm::LogTable *__restrict__ log_table)
{
    using VT = typename Gen::value_type;
    constexpr int CHUNK = 128 / (int)sizeof(VT);  // values per line
    constexpr int ROUND = LINES * CHUNK;          // values per generator per round
    constexpr int PER = 16 / (int)sizeof(VT);     // values per 16-byte packet
    constexpr int PITCH = ROUND + PER;            // 144-byte rows (272 with two lines)
    constexpr int LPR = 8 * LINES;                // lanes (packets) per row of a round
    constexpr int RPI = 64 / LPR;                 // rows per store instruction
    __shared__ __attribute__((aligned(16))) VT park_all[kFillBlock / 64][64][PITCH];

    // the normal generators look their logarithm up in a 3 KiB table: into LDS first
    __shared__ typename std::conditional<Gen::kHeavy, bm::LogTable, char>::type tab_store;
    // typed as an LDS pointer: the table look-ups are then LDS instructions with 32-bit addresses
    typedef const __attribute__((address_space(3))) bm::LogTable *LdsTable;
    const LdsTable tab = (LdsTable)reinterpret_cast<const bm::LogTable *>(&tab_store);
    if (Gen::kHeavy) {
        const double *src = reinterpret_cast<const double *>(log_table);
        double *dst = reinterpret_cast<double *>(&tab_store);
        for (int k = threadIdx.x; k < (int)(sizeof(bm::LogTable) / sizeof(double)); k += kFillBlock)
            dst[k] = src[k];
        __syncthreads();
    }

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    VT(*park)[PITCH] = park_all[wave];
    const int64_t t0 = ((int64_t)blockIdx.x * (kFillBlock / 64) + wave) * 64;  // first generator of this wavefront
    if (t0 >= n)
        return;
    const int64_t t = t0 + lane;
    const bool live = t < n;
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    uint64_t s0 = 0, s1 = 0;
    if (live) {
        u64x2 v = *reinterpret_cast<const u64x2 *>(states + 2 * t);
        s0 = v.x;
        s1 = v.y;
    }
    const int lanes_here = (n - t0 > 64) ? 64 : (int)(n - t0);  // generators this wavefront really has
    VT *__restrict__ base = out + t0 * count;
    const int sub = lane % LPR;  // which packet of a row this lane stores
    const int row = lane / LPR;  // which of the rows of a store instruction

    for (int64_t i0 = 0; i0 < count; i0 += ROUND) {
        const int m = (int)((count - i0 < ROUND) ? (count - i0) : ROUND);
        if (m % CHUNK == 0 && !Gen::kHeavy) {
            if (live) {
#pragma unroll
                for (int h = 0; h < LINES; ++h) {
                    if (h * CHUNK >= m)  // the last round of a run may be short of lines
                        break;
                    union {
                        VT val[CHUNK];
                        u32x4 pk[8];
                    } mine;
#pragma unroll
                    for (int j = 0; j < CHUNK; ++j)
                        mine.val[j] = Gen::draw(s0, s1, (const bm::LogTable *)nullptr);
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        *reinterpret_cast<u32x4 *>(&park[lane][h * CHUNK + k * PER]) = mine.pk[k];
                }
            }
        } else if (live) {
            // transcendental-heavy draws stay in a loop, two to a turn: unrolling sixteen
            // inlined log/cos bodies only thrashes the instruction cache
            int j = 0;
#pragma unroll 1
            for (; j + 1 < m; j += 2) {  // two values per 16-byte write where the value is 8 bytes
                VT two[2];
                two[0] = Gen::draw(s0, s1, tab);
                two[1] = Gen::draw(s0, s1, tab);
                park[lane][j] = two[0];
                park[lane][j + 1] = two[1];
            }
            if (j < m)
                park[lane][j] = Gen::draw(s0, s1, tab);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (m == ROUND) {
#pragma unroll
            for (int k = 0; k < LPR; ++k) {
                const int l = k * RPI + row;
                if (l < lanes_here) {
                    u32x4 v = *reinterpret_cast<const u32x4 *>(&park[l][sub * PER]);
                    nbh_store16<(int)sizeof(VT), NT>(base + (int64_t)l * count + i0 + sub * PER, v);
                }
            }
        } else if (LINES > 1 && m % CHUNK == 0) {
            // a last round of fewer whole lines: line by line, eight rows per instruction
            for (int h = 0; h * CHUNK < m; ++h) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int l = k * 8 + (lane >> 3);
                    if (l < lanes_here) {
                        const int col = h * CHUNK + (lane & 7) * PER;
                        u32x4 v = *reinterpret_cast<const u32x4 *>(&park[l][col]);
                        nbh_store16<(int)sizeof(VT), NT>(base + (int64_t)l * count + i0 + col, v);
                    }
                }
            }
        } else if (m % PER == 0) {
            // a short round of whole packets: the lanes form rows x packets with the row
            // length rounded up to a power of two, so no lane needs a division
            const int packets = m / PER;
            int shift = 0;
            while ((1 << shift) < packets)
                ++shift;
            const int q = lane & ((1 << shift) - 1);
            if (q < packets)
                for (int l = lane >> shift; l < lanes_here; l += 64 >> shift) {
                    u32x4 v = *reinterpret_cast<const u32x4 *>(&park[l][q * PER]);
                    nbh_store16<(int)sizeof(VT), false>(base + (int64_t)l * count + i0 + q * PER, v);
                }
        } else {
            // a ragged round: the same arrangement value by value
            int shift = 0;
            while ((1 << shift) < m)
                ++shift;
            const int j = lane & ((1 << shift) - 1);
            if (j < m)
                for (int l = lane >> shift; l < lanes_here; l += 64 >> shift)
                    base[(int64_t)l * count + i0 + j] = park[l][j];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (live) {
        u64x2 v = {s0, s1};
        *reinterpret_cast<u64x2 *>(states + 2 * t) = v;
    }
}

// Runs of whole 256-byte pieces on 128-byte lines, cheap generators.  The kernel above parks a
// round of every lane in LDS - 17 KB per wavefront with two lines per round, which leaves room
// for two wavefronts per SIMD, too few to keep the vector ALU busy while some of them wait for
// their stores.  Here a lane draws its 256 bytes into REGISTERS, and the wavefront hands them
// over sixteen generators at a time through 4 KB of LDS: the sixteen lanes of a quarter park
// their runs, all 64 lanes read them back as (generator, packet) and store - four store
// instructions of 1 KiB, each over four whole runs, so a wavefront still writes its 16 KiB as
// one piece.  Occupancy is then bounded by registers (four wavefronts per SIMD), and which XCD
// writes what starts to matter: with each XCD writing 256 KiB in a row (`runs` workgroups)
// 2^24 generators x 64 float32 take 710 - 728 us against 770 with every eighth workgroup's 64 KiB
// and 745 - 757 for the kernel above (where the order makes no difference).  Alone, the stores
// of this pattern take 675 us (805 without the runs) and the generation 587 us.
// Consecutive workgroups are started on different XCDs (workgroup b on XCD b % 8).  Within
// every whole group of 8 * runs consecutive workgroups this hands XCD k the pieces k * runs ...
// k * runs + runs - 1, so that an XCD writes `runs` workgroups' worth in a row; the workgroups
// past the last whole group keep their own piece.
__device__ __forceinline__ int64_t piece_of_block(int64_t block, int64_t grid, int runs)
{
    const int64_t span = 8 * (int64_t)runs;
    if (runs <= 1 || block >= grid / span * span)
        return block;
    const int64_t r = block % span;
    return block - r + (r % 8) * runs + r / 8;
}
template <typename Gen>
__global__ __launch_bounds__(kFillBlock) void fill_regs_kernel(uint64_t *__restrict__ states, int64_t n,
                                                               typename Gen::value_type *__restrict__ out,
                                                               int64_t count, int runs)
{
    static_assert(!Gen::kHeavy, "for the generators that are bound by their stores");
    using VT = typename Gen::value_type;
    constexpr int PER = 16 / (int)sizeof(VT);     // values per 16-byte packet
    constexpr int ROUND = 256 / (int)sizeof(VT);  // values per generator and round
    constexpr int PK = ROUND / PER;               // packets per generator and round: 16
    constexpr int PITCH = ROUND + PER;            // 272-byte rows
    __shared__ __attribute__((aligned(16))) VT park_all[kFillBlock / 64][16][PITCH];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    VT(*park)[PITCH] = park_all[wave];
    const int64_t t0 = (piece_of_block(blockIdx.x, gridDim.x, runs) * (kFillBlock / 64) + wave) * 64;
    if (t0 >= n)
        return;
    const int64_t t = t0 + lane;
    const bool live = t < n;
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    uint64_t s0 = 0, s1 = 0;
    if (live) {
        u64x2 v = *reinterpret_cast<const u64x2 *>(states + 2 * t);
        s0 = v.x;
        s1 = v.y;
    }
    const int lanes_here = (n - t0 > 64) ? 64 : (int)(n - t0);
    VT *__restrict__ base = out + t0 * count;
    const int quarter = lane >> 4, packet = lane & 15;

    for (int64_t i0 = 0; i0 < count; i0 += ROUND) {   // count is a multiple of ROUND (the host's check)
        union {
            VT val[ROUND];
            u32x4 pk[PK];
        } mine;
#pragma unroll
        for (int j = 0; j < ROUND; ++j)
            mine.val[j] = Gen::draw(s0, s1, (const bm::LogTable *)nullptr);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (quarter == q) {
#pragma unroll
                for (int k = 0; k < PK; ++k)
                    *reinterpret_cast<u32x4 *>(&park[lane & 15][k * PER]) = mine.pk[k];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 4 * i + quarter;          // a store instruction covers rows 4 i ... 4 i + 3
                const int gen = 16 * q + row;
                if (gen < lanes_here) {
                    u32x4 v = *reinterpret_cast<const u32x4 *>(&park[row][packet * PER]);
                    nbh_store16<(int)sizeof(VT), true>(base + (int64_t)gen * count + i0 + packet * PER, v);
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
    if (live) {
        u64x2 v = {s0, s1};
        *reinterpret_cast<u64x2 *>(states + 2 * t) = v;
    }
}

// Runs that do not start on 128-byte lines (count * itemsize not a multiple of 128, or
// an unaligned array) and are longer than a line.  Cutting the rounds where the runs
// start makes every store of the kernel above straddle two lines.  Here the rounds of
// the STORES follow the lines of the output instead, while generation still proceeds
// 128 bytes per generator at a time: each lane parks its values in a ring of two
// rounds, value i in column (i + skew) mod ring, where skew is the distance of the
// run's start from the line below it.  After generation round r the columns of line r
// are complete for every generator (the last `skew` values of the round wait in the
// other half for line r+1), they start on a packet boundary of the ring whatever the
// skew, and the wavefront stores them as whole, aligned, non-temporal 16-byte packets,
// eight generators' lines per instruction.
// The line in which one run ends is the line in which the next begins.  Each lane keeps
// its first round in registers and, before the last lines are stored, adds the head of
// its run to the ring of the generator before it, so that line too leaves as one whole
// line; only the first line of a wavefront's first run and the last line of its last
// run are stored value by value.  One more store-only round flushes the tails.
// Requires count >= one round (the first round is drawn in the unrolled path).
template <typename Gen>
__global__ __launch_bounds__(kFillBlock) void fill_ring_kernel(uint64_t *__restrict__ states, int64_t n,
                                                               typename Gen::value_type *__restrict__ out,
                                                               int64_t count)
{
    static_assert(!Gen::kHeavy, "compute-bound generators gain nothing here and lose occupancy");
    using VT = typename Gen::value_type;
    constexpr int ROUND = 128 / (int)sizeof(VT);
    constexpr int PER = 16 / (int)sizeof(VT);
    constexpr int RING = 2 * ROUND;
    constexpr int PITCH = RING + PER;  // 272-byte rows
    __shared__ __attribute__((aligned(16))) VT ring_all[kFillBlock / 64][64][PITCH];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    VT(*ring)[PITCH] = ring_all[wave];
    const int64_t t0 = ((int64_t)blockIdx.x * (kFillBlock / 64) + wave) * 64;
    if (t0 >= n)
        return;
    const int64_t t = t0 + lane;
    const bool live = t < n;
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    uint64_t s0 = 0, s1 = 0;
    if (live) {
        u64x2 v = *reinterpret_cast<const u64x2 *>(states + 2 * t);
        s0 = v.x;
        s1 = v.y;
    }
    const int lanes_here = (n - t0 > 64) ? 64 : (int)(n - t0);
    VT *__restrict__ base = out + t0 * count;
    const int sub = lane & 7;
    const int row = lane >> 3;
    // position of generator l's run in values, modulo a line: (first + l * count) mod ROUND
    const uint32_t first = (uint32_t)((uintptr_t)base / sizeof(VT));
    const uint32_t step = (uint32_t)count;
    const int my_skew = (int)((first + (uint32_t)lane * step) & (ROUND - 1));
    const int64_t gen_rounds = (count + ROUND - 1) / ROUND;
    // largest power of two (up to a packet) that divides the start of every run
    const uint32_t both = (uint32_t)((uintptr_t)out / sizeof(VT)) | step;
    const int grain = (both & 1) ? 1 : (both & 2) ? 2 : 4;
    VT head[ROUND];  // this lane's first round
#pragma unroll
    for (int j = 0; j < ROUND; ++j)
        head[j] = VT(0);

    for (int64_t r = 0; r <= gen_rounds; ++r) {
        const int64_t i0 = r * ROUND;
        const int half = (int)(r & 1) * ROUND;  // i0 mod RING
        if (r < gen_rounds) {
            const int m = (int)((count - i0 < ROUND) ? (count - i0) : ROUND);
            const int col0 = half + my_skew;
            if (m == ROUND) {
                if (live) {
                    union {
                        VT val[ROUND];
                        u32x4 pk[8];
                        uint64_t pr[16];
                    } mine;
#pragma unroll
                    for (int j = 0; j < ROUND; ++j)
                        mine.val[j] = Gen::draw(s0, s1, (const bm::LogTable *)nullptr);
                    // every skew of the launch is a multiple of `grain` values: park in
                    // pieces of that size (they neither straddle the wrap nor lose alignment)
                    if (grain >= PER) {
#pragma unroll
                        for (int k = 0; k < 8; ++k)
                            *reinterpret_cast<u32x4 *>(&ring[lane][(col0 + k * PER) & (RING - 1)]) = mine.pk[k];
                    } else if (sizeof(VT) == 4 && grain >= 2) {
#pragma unroll
                        for (int k = 0; k < 16; ++k)
                            *reinterpret_cast<uint64_t *>(&ring[lane][(col0 + 2 * k) & (RING - 1)]) = mine.pr[k];
                    } else {
#pragma unroll
                        for (int j = 0; j < ROUND; ++j)
                            ring[lane][(col0 + j) & (RING - 1)] = mine.val[j];
                    }
                    if (r == 0) {
#pragma unroll
                        for (int j = 0; j < ROUND; ++j)
                            head[j] = mine.val[j];
                    }
                }
            } else if (live) {
                // the last, short round: four draws at a time so that the conversion of
                // one overlaps the state update of the next
                int j = 0;
#pragma unroll 1
                for (; j + 4 <= m; j += 4) {
                    VT four[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        four[e] = Gen::draw(s0, s1, (const bm::LogTable *)nullptr);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        ring[lane][(col0 + j + e) & (RING - 1)] = four[e];
                }
#pragma unroll 1
                for (; j < m; ++j)
                    ring[lane][(col0 + j) & (RING - 1)] = Gen::draw(s0, s1, (const bm::LogTable *)nullptr);
            }
            if (r == gen_rounds - 1 && live && lane > 0 && my_skew > 0) {
                // the run before this one ends `my_skew` values into its last line: the
                // rest of that line is the head of this run
                const int skew_before = (int)((first + (uint32_t)(lane - 1) * step) & (ROUND - 1));
                const int64_t last_line = (count + skew_before - my_skew) / ROUND;
                const int at = (int)(last_line & 1) * ROUND + my_skew;
#pragma unroll
                for (int j = 0; j < ROUND; ++j)
                    if (j < ROUND - my_skew)
                        ring[lane - 1][at + j] = head[j];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // line r of every run: ring columns [half, half + ROUND), values from i0 - skew on
        const int col = half + sub * PER;
        if (r >= 1 && i0 + ROUND <= count) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int l = k * 8 + row;
                if (l < lanes_here) {
                    const int skew = (int)((first + (uint32_t)l * step) & (ROUND - 1));
                    u32x4 v = *reinterpret_cast<const u32x4 *>(&ring[l][col]);
                    nbh_store16<16, true>(base + (int64_t)l * count + (i0 - skew + sub * PER), v);
                }
            }
        } else {
            // first and last lines: whole packets first, all eight rows in flight at once
            bool partial = false;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int l = k * 8 + row;
                const int skew = (int)((first + (uint32_t)l * step) & (ROUND - 1));
                const int64_t line_lo = i0 - skew;  // value index of the line's first column
                // not past the end of the run; a first line shared with the run before is
                // stored from that run's ring; the head of the next run completes a last line
                const bool mine = l < lanes_here && line_lo < count && !(line_lo < 0 && l > 0);
                const int64_t limit = (l + 1 < lanes_here) ? line_lo + ROUND : count;
                const int64_t lo = line_lo + sub * PER;
                const bool whole = lo >= 0 && lo + PER <= limit;
                u32x4 v = *reinterpret_cast<const u32x4 *>(&ring[l & 63][col]);
                if (mine && whole)
                    nbh_store16<16, true>(base + (int64_t)l * count + lo, v);
                partial |= mine && !whole;
            }
            if (partial) {
                // the first line of the wavefront's first run, the last line of its last
#pragma unroll 1
                for (int k = 0; k < 8; ++k) {
                    const int l = k * 8 + row;
                    const int skew = (int)((first + (uint32_t)l * step) & (ROUND - 1));
                    const int64_t line_lo = i0 - skew;
                    if (l >= lanes_here || line_lo >= count || (line_lo < 0 && l > 0))
                        continue;
                    const int64_t limit = (l + 1 < lanes_here) ? line_lo + ROUND : count;
                    const int64_t lo = line_lo + sub * PER;
                    if (lo >= 0 && lo + PER <= limit)
                        continue;
                    for (int e = 0; e < PER; ++e)
                        if (lo + e >= 0 && lo + e < limit)
                            base[(int64_t)l * count + lo + e] = ring[l][col + e];
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (live) {
        u64x2 v = {s0, s1};
        *reinterpret_cast<u64x2 *>(states + 2 * t) = v;
    }
}

// runs from this many bytes on go through the ring when they are not on lines
constexpr int64_t kRingFromBytes = 192;

template <typename Gen, bool HEAVY = Gen::kHeavy>
struct RingLaunch {
    static void go(dim3 grid, hipStream_t s, uint64_t *states, int64_t n, typename Gen::value_type *out,
                   int64_t count)
    {
        hipLaunchKernelGGL((fill_ring_kernel<Gen>), grid, dim3(kFillBlock), 0, s, states, n, out, count);
    }
};
template <typename Gen>
struct RingLaunch<Gen, true> {
    static void go(dim3, hipStream_t, uint64_t *, int64_t, typename Gen::value_type *, int64_t) {}
};

template <typename Gen, bool Heavy = Gen::kHeavy>
struct FillRegs {
    static void go(dim3 grid, hipStream_t s, uint64_t *states, int64_t n, typename Gen::value_type *out, int64_t count,
                   int runs)
    {
        hipLaunchKernelGGL((fill_regs_kernel<Gen>), grid, dim3(kFillBlock), 0, s, states, n, out, count, runs);
    }
};
template <typename Gen>
struct FillRegs<Gen, true> {
    static void go(dim3, hipStream_t, uint64_t *, int64_t, typename Gen::value_type *, int64_t, int) {}
};

template <typename Gen>
int launch_fill(void *states, int64_t n, void *out, int64_t count, nbh_stream_t stream)
{
    if (n < 0 || count < 0)
        return (int)hipErrorInvalidValue;
    if (n == 0 || count == 0)
        return 0;
    if (!states || !out || ((uintptr_t)states) % 16 != 0 ||
        ((uintptr_t)out) % sizeof(typename Gen::value_type) != 0)
        return (int)hipErrorInvalidValue;
    const int64_t grid = (n + kFillBlock - 1) / kFillBlock;
    if (grid > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    const bm::LogTable *log_table = nullptr;
    if (Gen::kHeavy) {
        int rc = device_log_table(&log_table);
        if (rc)
            return rc;
    }
    nbh_stream_report report(nbh_hip_stream(stream));
    using VT = typename Gen::value_type;
    const bool on_lines = ((uintptr_t)out % 128 == 0) && ((uint64_t)count * sizeof(VT)) % 128 == 0;
    // Lines per generator and round (measured, 2^24 generators, uniform draws): two lines
    // beat one from 256-byte runs on (64 float32: 839 -> 754 us); four lines need 135 KB of
    // LDS per workgroup, one workgroup per CU, which float32 generation only forgives when the
    // runs are long (4 KiB on: 15.3 -> 12.9 ms at 1024 float32), float64 also at 512 B and 1 KiB.
    const uint64_t run_bytes = (uint64_t)count * sizeof(VT);
    const bool four = run_bytes >= 4096 || (sizeof(VT) == 8 && (run_bytes == 512 || run_bytes == 1024));
    const int lines = Gen::kHeavy ? 1 : four ? 4 : run_bytes >= 256 ? 2 : 1;
    if (on_lines && lines == 4)
        hipLaunchKernelGGL((fill_kernel<Gen, true, 4>), dim3((unsigned)grid), dim3(kFillBlock), 0,
                           nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count, log_table);
    else if (on_lines && lines == 2 && (run_bytes == 256 || run_bytes == 512)) {
        // (measured, 2^22 generators, this kernel against the one above: 64 float32 194 -> 183 us,
        // 128 float32 436 -> 422, 32 float64 194 -> 183, 64 float64 the same; longer runs lose:
        // 192 float32 576 -> 598, 256 float32 780 -> 802)
        // a workgroup writes kFillBlock runs in a row; XCDs take turns after 256 KiB
        int runs = 1;
        while ((uint64_t)runs * kFillBlock * run_bytes < (256u << 10))
            runs *= 2;
        FillRegs<Gen>::go(dim3((unsigned)grid), nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count, runs);
    }
    else if (on_lines && lines == 2)
        hipLaunchKernelGGL((fill_kernel<Gen, true, 2>), dim3((unsigned)grid), dim3(kFillBlock), 0,
                           nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count, log_table);
    else if (on_lines)
        hipLaunchKernelGGL((fill_kernel<Gen, true, 1>), dim3((unsigned)grid), dim3(kFillBlock), 0,
                           nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count, log_table);
    else if (!Gen::kHeavy && count * (int64_t)sizeof(VT) >= kRingFromBytes)
        RingLaunch<Gen>::go(dim3((unsigned)grid), nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count);
    else
        hipLaunchKernelGGL((fill_kernel<Gen, false, 1>), dim3((unsigned)grid), dim3(kFillBlock), 0,
                           nbh_hip_stream(stream), (uint64_t *)states, n, (VT *)out, count, log_table);
    return nbh_launch_status();
}

// ---- one generator at a time --------------------------------------------------------
// What the per-generator functions of the Python layer run when the states live on the
// device: one lane, the same draw routines as the bulk kernels (hence the same bits).
__global__ __launch_bounds__(64) void one_generator_kernel(uint64_t *__restrict__ state, int kind,
                                                           void *__restrict__ out,
                                                           const bm::LogTable *__restrict__ log_table)
{
    if (threadIdx.x != 0)
        return;
    uint64_t s0 = state[0], s1 = state[1];
    switch (kind) {
    case NBH_XORO_NEXT:
        *static_cast<uint64_t *>(out) = next_d(s0, s1);
        break;
    case NBH_XORO_JUMP: {
        // random.py:118-142: XOR together the states reached after k steps for every set
        // bit k of the 128-bit jump polynomial (= 2^64 steps)
        const uint64_t poly[2] = {0xBEAC0467EBA5FACBull, 0xD86B048B86AA9922ull};
        uint64_t j0 = 0, j1 = 0;
        for (int w = 0; w < 2; ++w)
            for (int b = 0; b < 64; ++b) {
                if ((poly[w] >> b) & 1) {
                    j0 ^= s0;
                    j1 ^= s1;
                }
                (void)next_d(s0, s1);
            }
        s0 = j0;
        s1 = j1;
        break;
    }
    case NBH_XORO_UNIFORM_F32:
        *static_cast<float *>(out) = UniformF32::draw(s0, s1);
        break;
    case NBH_XORO_UNIFORM_F64:
        *static_cast<double *>(out) = UniformF64::draw(s0, s1);
        break;
    case NBH_XORO_NORMAL_F32:
        *static_cast<float *>(out) = NormalF32::draw(s0, s1, log_table);
        break;
    default:
        *static_cast<double *>(out) = NormalF64::draw(s0, s1, log_table);
        break;
    }
    state[0] = s0;
    state[1] = s1;
}

}  // namespace

extern "C" {

int nbh_xoro_one(void *state, int kind, void *out, nbh_stream_t stream)
{
    if (!state || ((uintptr_t)state) % 16 != 0 || kind < NBH_XORO_NEXT || kind > NBH_XORO_NORMAL_F64)
        return (int)hipErrorInvalidValue;
    if (kind != NBH_XORO_JUMP && (!out || ((uintptr_t)out) % 8 != 0))
        return (int)hipErrorInvalidValue;
    const bm::LogTable *log_table = nullptr;
    if (kind == NBH_XORO_NORMAL_F32 || kind == NBH_XORO_NORMAL_F64)
        if (int rc = device_log_table(&log_table))
            return rc;
    hipLaunchKernelGGL(one_generator_kernel, dim3(1), dim3(64), 0, nbh_hip_stream(stream), (uint64_t *)state, kind,
                       out, log_table);
    const int rc = nbh_launch_status();
    nbh_stream_report report(nbh_hip_stream(stream));
    return rc;
}

int nbh_xoro_init_states(void *states, int64_t n, uint64_t seed, uint64_t subsequence_start, nbh_stream_t stream)
{
    if (n < 0)
        return (int)hipErrorInvalidValue;
    if (n == 0)
        return 0;
    if (!states || ((uintptr_t)states) % 16 != 0)
        return (int)hipErrorInvalidValue;
    // SplitMix64 step; the same word seeds both halves
    uint64_t z = seed + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    U128 base = {z, z};
    // advance to the first subsequence on the host: at most 64 matrix products
    const JumpTable &t = jump_table();
    for (int k = 0; k < kPowers; ++k)
        if ((subsequence_start >> k) & 1)
            base = apply_h(t.col[k], base);
    const U128 *dtable = nullptr;
    int rc = device_table(&dtable);
    if (rc)
        return rc;
    hipStream_t hs = nbh_hip_stream(stream);
    nbh_stream_report report(hs);
    // Steps per wavefront: as few as leave every SIMD of the device four wavefronts, 64 from 2^24
    // states on (one workgroup of 16 wavefronts per compute unit and 65536 states then).
    // Measured per launch, 64 steps whatever the size (and, below 2^18 states, masked XORs over
    // the 128 columns instead of tables) -> this choice: 2^12 states 201 -> 7.7 us, 2^16 208 ->
    // 10.1, 2^18 40 -> 12.5, 2^20 42 -> 17.5, 2^22 47 -> 27, 2^23 49 -> 37, 2^24 the same.
    const int64_t wavefronts_wanted = (int64_t)nbh_cu_count() * (kTabBlock / 64);
    int64_t steps = (n + 64 * wavefronts_wanted - 1) / (64 * wavefronts_wanted);
    steps = steps < 1 ? 1 : steps > kInitSteps ? kInitSteps : steps;
    const int64_t per_block = (int64_t)(kTabBlock / 64) * 64 * steps;
    const int64_t grid = (n + per_block - 1) / per_block;
    if (grid > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    const u64x2_t *lut = reinterpret_cast<const u64x2_t *>(dtable + (size_t)kPowers * 128);
    const u64x2_t *lanes = lut + kLutEntries;
    hipLaunchKernelGGL(init_states_tables_kernel, dim3((unsigned)grid), dim3(kTabBlock), 0, hs, (uint64_t *)states,
                       n, base.s0, base.s1, dtable, lut, lanes, (int)steps);
    return nbh_launch_status();
}

int nbh_xoro_uniform_f32(void *states, int64_t nstates, float *out, int64_t count, nbh_stream_t stream)
{
    return launch_fill<UniformF32>(states, nstates, out, count, stream);
}
int nbh_xoro_uniform_f64(void *states, int64_t nstates, double *out, int64_t count, nbh_stream_t stream)
{
    return launch_fill<UniformF64>(states, nstates, out, count, stream);
}
int nbh_xoro_normal_f32(void *states, int64_t nstates, float *out, int64_t count, nbh_stream_t stream)
{
    return launch_fill<NormalF32>(states, nstates, out, count, stream);
}
int nbh_xoro_normal_f64(void *states, int64_t nstates, double *out, int64_t count, nbh_stream_t stream)
{
    return launch_fill<NormalF64>(states, nstates, out, count, stream);
}

}  // extern "C"

/*
 * CPU restatement of the numba-cuda data-parallel array library, in plain C.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
 * compared against and the CPU baseline that the benchmark times.  Nothing in
 * the shipped package links, loads or calls it.
 *
 * Every function names the reference source it restates (paths relative to
 * numba_cuda/numba/cuda/ in NVIDIA/numba-cuda 0.30.4).
 *
 * Parity status of each group:
 *   xoroshiro128+ state/next/jump/uniform : pinned (SplitMix64 published vectors,
 *       jump == next^(2^64) by GF(2) matrix power, big-int twin, closed forms)
 *   reduce tree order                     : pinned against a literal lock-step
 *       SIMT emulation (oracle/reduce_simt.py) and closed forms n(n+1)/2, n!
 *   float16 arithmetic (software binary16): pinned against NumPy's float16 on every
 *       bit pattern, and the float16 folds / trees against NumPy float16 folds and
 *       the lock-step emulation run in float16
 *   transpose                             : pinned against numpy's a.T
 *   Box-Muller normals                    : parity unpinned at bit level.  The
 *       reference evaluates log/cos in NVIDIA libdevice, whose result bits no
 *       file in the reference records; this restatement follows the reference's
 *       precision mix with correctly rounded libm calls.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, no fast-math).
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* xoroshiro128+ (2016 constants 55/14/36) and SplitMix64 seeding             */
/* ------------------------------------------------------------------------- */

/* random.py:62-85  init_xoroshiro128p_state: one SplitMix64 step, the same
 * word is stored into both halves of the state. */
void orc_xoro_seed_state(uint64_t seed, uint64_t *s)
{
    uint64_t z = seed + UINT64_C(0x9E3779B97F4A7C15);
    z = (z ^ (z >> 30)) * UINT64_C(0xBF58476D1CE4E5B9);
    z = (z ^ (z >> 27)) * UINT64_C(0x94D049BB133111EB);
    z = z ^ (z >> 31);
    s[0] = z;
    s[1] = z;
}

/* random.py:88-93 */
static inline uint64_t rotl64(uint64_t x, unsigned k)
{
    return (x << k) | (x >> (64u - k));
}

/* random.py:96-115  xoroshiro128p_next */
uint64_t orc_xoro_next(uint64_t *s)
{
    uint64_t s0 = s[0];
    uint64_t s1 = s[1];
    uint64_t result = s0 + s1;
    s1 ^= s0;
    s[0] = rotl64(s0, 55) ^ s1 ^ (s1 << 14);
    s[1] = rotl64(s1, 36);
    return result;
}

/* random.py:118-142  xoroshiro128p_jump: advance by 2^64 steps */
void orc_xoro_jump(uint64_t *s)
{
    static const uint64_t poly[2] = {UINT64_C(0xBEAC0467EBA5FACB),
                                     UINT64_C(0xD86B048B86AA9922)};
    uint64_t a0 = 0, a1 = 0;
    for (int w = 0; w < 2; ++w) {
        for (int b = 0; b < 64; ++b) {
            if (poly[w] & (UINT64_C(1) << b)) {
                a0 ^= s[0];
                a1 ^= s[1];
            }
            (void)orc_xoro_next(s);
        }
    }
    s[0] = a0;
    s[1] = a1;
}

/* random.py:241-257  init_xoroshiro128p_states_cpu: sequential jump chain.
 * states is n records of {s0, s1}. */
void orc_xoro_init_states(uint64_t *states, int64_t n, uint64_t seed,
                          uint64_t subsequence_start)
{
    if (n < 1)
        return;
    orc_xoro_seed_state(seed, states);
    for (uint64_t k = 0; k < subsequence_start; ++k)
        orc_xoro_jump(states);
    for (int64_t i = 1; i < n; ++i) {
        states[2 * i] = states[2 * i - 2];
        states[2 * i + 1] = states[2 * i - 1];
        orc_xoro_jump(states + 2 * i);
    }
}

/* random.py:145-149 */
double orc_u64_to_unit_f64(uint64_t x)
{
    return (double)(x >> 11) * (1.0 / 9007199254740992.0);
}

/* random.py:152-156: a single double->float rounding of the value above */
float orc_u64_to_unit_f32(uint64_t x)
{
    return (float)orc_u64_to_unit_f64(x);
}

/* random.py:159-184 */
float orc_xoro_uniform_f32(uint64_t *s) { return orc_u64_to_unit_f32(orc_xoro_next(s)); }
double orc_xoro_uniform_f64(uint64_t *s) { return orc_u64_to_unit_f64(orc_xoro_next(s)); }

/* random.py:187-213  xoroshiro128p_normal_float32.  Every operation is carried
 * out in float32 in the compiled reference (cudamath.py:41-58 types
 * math.log/cos/sqrt(float32) -> float32; mathimpl.py:36-43 lowers them to
 * logf/cosf/sqrtf).  Each libm call below is evaluated in double and rounded
 * once, i.e. a correctly rounded stand-in for the float32 routine. */
float orc_xoro_normal_f32(uint64_t *s)
{
    const float two_pi = (float)(2.0 * 3.14159265358979323846);
    float u1 = orc_xoro_uniform_f32(s);
    float u2 = orc_xoro_uniform_f32(s);
    float lg = (float)log((double)u1);
    float arg = -2.0f * lg;
    float r = (float)sqrt((double)arg);
    float ang = two_pi * u2;
    float c = (float)cos((double)ang);
    return r * c;
}

/* random.py:216-238  xoroshiro128p_normal_float64.  The two uniforms are still
 * float32; log is taken on a float32 argument and therefore returns float32,
 * which is then promoted; sqrt and cos are float64. */
double orc_xoro_normal_f64(uint64_t *s)
{
    const double two_pi = 2.0 * 3.14159265358979323846;
    float u1 = orc_xoro_uniform_f32(s);
    float u2 = orc_xoro_uniform_f32(s);
    float lg = (float)log((double)u1);
    double r = sqrt(-2.0 * (double)lg);
    double c = cos(two_pi * (double)u2);
    return r * c;
}

/* Bulk draws with the layout of the reference's own test kernels
 * (tests/cudapy/test_random.py:29-52): out[tid * count + i], states advanced
 * in place. */
void orc_xoro_fill_uniform_f32(uint64_t *states, int64_t n, float *out, int64_t count)
{
    for (int64_t t = 0; t < n; ++t)
        for (int64_t i = 0; i < count; ++i)
            out[t * count + i] = orc_xoro_uniform_f32(states + 2 * t);
}
void orc_xoro_fill_uniform_f64(uint64_t *states, int64_t n, double *out, int64_t count)
{
    for (int64_t t = 0; t < n; ++t)
        for (int64_t i = 0; i < count; ++i)
            out[t * count + i] = orc_xoro_uniform_f64(states + 2 * t);
}
void orc_xoro_fill_normal_f32(uint64_t *states, int64_t n, float *out, int64_t count)
{
    for (int64_t t = 0; t < n; ++t)
        for (int64_t i = 0; i < count; ++i)
            out[t * count + i] = orc_xoro_normal_f32(states + 2 * t);
}
void orc_xoro_fill_normal_f64(uint64_t *states, int64_t n, double *out, int64_t count)
{
    for (int64_t t = 0; t < n; ++t)
        for (int64_t i = 0; i < count; ++i)
            out[t * count + i] = orc_xoro_normal_f64(states + 2 * t);
}

/* ------------------------------------------------------------------------- */
/* Reduction                                                                  */
/* ------------------------------------------------------------------------- */

/* Operator semantics under the reference's JIT (cpython/builtins.py:224-269):
 *   a + b, a * b : native arithmetic of the dtype; integers wrap
 *   max(a, b)    : b if b > a else a
 *   min(a, b)    : b if b < a else a
 * Integer add/mul go through uint64_t so that wrap-around is defined and the
 * narrow types are not promoted to a signed int that could overflow.
 */
#define OP_ADD_I(T, U, a, b) ((T)(U)((uint64_t)(U)(a) + (uint64_t)(U)(b)))
#define OP_MUL_I(T, U, a, b) ((T)(U)((uint64_t)(U)(a) * (uint64_t)(U)(b)))
#define OP_ADD_F(T, U, a, b) ((T)((a) + (b)))
#define OP_MUL_F(T, U, a, b) ((T)((a) * (b)))
/* bitwise functors (`a & b`, `a | b`, `a ^ b`) on integers: two's complement, like the
 * reference's LLVM and/or/xor on the element type */
#define OP_AND_I(T, U, a, b) ((T)(U)((U)(a) & (U)(b)))
#define OP_OR_I(T, U, a, b) ((T)(U)((U)(a) | (U)(b)))
#define OP_XOR_I(T, U, a, b) ((T)(U)((U)(a) ^ (U)(b)))
#define OP_MAX(T, U, a, b) (((b) > (a)) ? (b) : (a))
#define OP_MIN(T, U, a, b) (((b) < (a)) ? (b) : (a))

#define WARP 32
#define NWARPS 4
#define BLOCK (WARP * NWARPS)
#define MAXGRID (2 * WARP)

/*
 * DEFINE_REDUCE(name, T, U, OP) emits
 *
 *   orc_fold_<name>: simulator/reduction.py:7-19 - strict left fold
 *       functools.reduce(op, seq, init)
 *
 *   orc_tree_<name>: kernels/reduction.py:194-265 with the device functions at
 *       :22-166, evaluated in exactly the association order a CUDA run uses:
 *       - full launch  (:43-97, :233-248): grid = min(n/128, 64) blocks of 128
 *         lanes; lane g folds a[g], a[g+S], ... left to right (S = 128*grid);
 *         each 32-lane warp runs the shared-memory tree (l, l+16), (l, l+8),
 *         (l, l+4), (l, l+2), (l, l+1) (:22-41); block = (w0 op w2) op (w1 op w3);
 *         block 0 then folds in init (:163-164)
 *       - tail launch  (:99-141, :250-254): one block over the last n%128
 *         values; init folded here only when there was no full launch
 *       - finish launch (:256-258): the same one-block routine over the partials
 */
#define DEFINE_REDUCE(name, T, U, OP)                                          \
    void orc_fold_##name(const T *a, int64_t n, const T *init, T *out)         \
    {                                                                          \
        T acc = *init;                                                         \
        for (int64_t i = 0; i < n; ++i)                                        \
            acc = OP(T, U, acc, a[i]);                                         \
        *out = acc;                                                            \
    }                                                                          \
    /* :22-41 one fully populated warp, values v[0..31] */                     \
    static T warp_tree_##name(T *v)                                            \
    {                                                                          \
        for (int width = WARP / 2; width; width /= 2)                          \
            for (int l = 0; l < width; ++l)                                    \
                v[l] = OP(T, U, v[l], v[l + width]);                           \
        return v[0];                                                           \
    }                                                                          \
    /* :99-141 one block of m < 128 lanes */                                   \
    static T one_block_##name(const T *a, int m)                               \
    {                                                                          \
        T wres[NWARPS] = {0};                                                  \
        int nw = (m + WARP - 1) / WARP;                                        \
        for (int w = 0; w < nw; ++w) {                                         \
            if ((w + 1) * WARP < m) {                                          \
                T v[WARP];                                                     \
                memcpy(v, a + w * WARP, sizeof v);                             \
                wres[w] = warp_tree_##name(v);                                 \
            } else {                                                           \
                T acc = a[w * WARP];                                           \
                for (int i = 1; i < m - w * WARP; ++i)                         \
                    acc = OP(T, U, acc, a[w * WARP + i]);                      \
                wres[w] = acc;                                                 \
            }                                                                  \
        }                                                                      \
        T r = wres[0];                                                         \
        for (int w = 1; w < nw; ++w)                                           \
            r = OP(T, U, r, wres[w]);                                          \
        return r;                                                              \
    }                                                                          \
    void orc_tree_##name(const T *a, int64_t n, const T *init, T *out)         \
    {                                                                          \
        if (n < 1) {                                                           \
            *out = *init;                                                      \
            return;                                                            \
        }                                                                      \
        int64_t size_full = (n / BLOCK) * BLOCK;                               \
        int m_tail = (int)(n - size_full);                                     \
        int64_t grid = size_full / BLOCK;                                      \
        if (grid > MAXGRID)                                                    \
            grid = MAXGRID;                                                    \
        T partials[MAXGRID + 1];                                               \
        int np = (int)grid + (m_tail ? 1 : 0);                                 \
        int64_t S = BLOCK * grid;                                              \
        for (int64_t blk = 0; blk < grid; ++blk) {                             \
            T wres[NWARPS];                                                    \
            for (int w = 0; w < NWARPS; ++w) {                                 \
                T v[WARP];                                                     \
                for (int l = 0; l < WARP; ++l) {                               \
                    int64_t g = blk * BLOCK + w * WARP + l;                    \
                    T acc = a[g];                                              \
                    for (int64_t i = g + S; i < size_full; i += S)             \
                        acc = OP(T, U, acc, a[i]);                             \
                    v[l] = acc;                                                \
                }                                                              \
                wres[w] = warp_tree_##name(v);                                 \
            }                                                                  \
            T lo = OP(T, U, wres[0], wres[2]);                                 \
            T hi = OP(T, U, wres[1], wres[3]);                                 \
            partials[blk] = OP(T, U, lo, hi);                                  \
        }                                                                      \
        if (grid)                                                              \
            partials[0] = OP(T, U, partials[0], *init);                        \
        if (m_tail) {                                                          \
            partials[grid] = one_block_##name(a + size_full, m_tail);          \
            if (!grid)                                                         \
                partials[0] = OP(T, U, partials[0], *init);                    \
        }                                                                      \
        if (np > 1)                                                            \
            partials[0] = one_block_##name(partials, np);                      \
        *out = partials[0];                                                    \
    }

#define DEFINE_REDUCE_INT(sfx, T, U)                   \
    DEFINE_REDUCE(add_##sfx, T, U, OP_ADD_I)           \
    DEFINE_REDUCE(mul_##sfx, T, U, OP_MUL_I)           \
    DEFINE_REDUCE(max_##sfx, T, U, OP_MAX)             \
    DEFINE_REDUCE(min_##sfx, T, U, OP_MIN)             \
    DEFINE_REDUCE(and_##sfx, T, U, OP_AND_I)           \
    DEFINE_REDUCE(or_##sfx, T, U, OP_OR_I)             \
    DEFINE_REDUCE(xor_##sfx, T, U, OP_XOR_I)
#define DEFINE_REDUCE_FLT(sfx, T)                      \
    DEFINE_REDUCE(add_##sfx, T, T, OP_ADD_F)           \
    DEFINE_REDUCE(mul_##sfx, T, T, OP_MUL_F)           \
    DEFINE_REDUCE(max_##sfx, T, T, OP_MAX)             \
    DEFINE_REDUCE(min_##sfx, T, T, OP_MIN)

DEFINE_REDUCE_INT(i8, int8_t, uint8_t)
DEFINE_REDUCE_INT(i16, int16_t, uint16_t)
DEFINE_REDUCE_INT(i32, int32_t, uint32_t)
DEFINE_REDUCE_INT(i64, int64_t, uint64_t)
DEFINE_REDUCE_INT(u8, uint8_t, uint8_t)
DEFINE_REDUCE_INT(u16, uint16_t, uint16_t)
DEFINE_REDUCE_INT(u32, uint32_t, uint32_t)
DEFINE_REDUCE_INT(u64, uint64_t, uint64_t)
DEFINE_REDUCE_FLT(f32, float)
DEFINE_REDUCE_FLT(f64, double)

/* Complex elements: `a + b` componentwise, `a * b` by the plain formula
 * (ac - bd) + (ad + bc)i with every product and sum rounded once - what the
 * reference's JIT emits for complex operands (no special-value recovery, no fused
 * operations in this restatement; the compiled reference may contract to FMA, which
 * is why complex PRODUCTS are compared with a tolerance).  No max / min. */
typedef struct { float re, im; } orc_c64;
typedef struct { double re, im; } orc_c128;
static inline orc_c64 c64_add(orc_c64 a, orc_c64 b) { orc_c64 r = {a.re + b.re, a.im + b.im}; return r; }
static inline orc_c128 c128_add(orc_c128 a, orc_c128 b) { orc_c128 r = {a.re + b.re, a.im + b.im}; return r; }
static inline orc_c64 c64_mul(orc_c64 a, orc_c64 b)
{
    orc_c64 r = {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
    return r;
}
static inline orc_c128 c128_mul(orc_c128 a, orc_c128 b)
{
    orc_c128 r = {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
    return r;
}
#define OP_ADD_C64(T, U, a, b) c64_add(a, b)
#define OP_MUL_C64(T, U, a, b) c64_mul(a, b)
#define OP_ADD_C128(T, U, a, b) c128_add(a, b)
#define OP_MUL_C128(T, U, a, b) c128_mul(a, b)
DEFINE_REDUCE(add_c64, orc_c64, orc_c64, OP_ADD_C64)
DEFINE_REDUCE(mul_c64, orc_c64, orc_c64, OP_MUL_C64)
DEFINE_REDUCE(add_c128, orc_c128, orc_c128, OP_ADD_C128)
DEFINE_REDUCE(mul_c128, orc_c128, orc_c128, OP_MUL_C128)

/* float16 elements.  The reference's JIT lowers `a + b`, `a * b` on float16 operands to
 * the GPU's native half-precision add / mul (one IEEE rounding to binary16 per
 * operation) and max / min to comparisons of the two halves, so the accumulator is a
 * half all the way (kernels/reduction.py:78-81: `tmp = reduce_op(tmp, arr[i])` keeps
 * the element type).  Restated in software: a half is carried as its 16 bits; the sum
 * and the product of two halves are exact in double (at most 40 and 22 significant
 * bits), so one round-to-nearest-even from double to half is the one rounding.
 *   parity of orc_f16_from_double / orc_f16_to_double: pinned against NumPy's float16
 *   conversions on all 65536 bit patterns and on random doubles (tests/).  */
typedef uint16_t orc_f16;

double orc_f16_to_double(orc_f16 h)
{
    const int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
    double v;
    if (e == 31)
        v = m ? NAN : INFINITY;
    else if (e == 0)
        v = ldexp((double)m, -24);              /* subnormal: m * 2^-24 */
    else
        v = ldexp((double)(1024 + m), e - 25);  /* (1 + m/1024) * 2^(e-15) */
    return sign ? -v : v;
}

orc_f16 orc_f16_from_double(double x)
{
    const orc_f16 sign = signbit(x) ? 0x8000u : 0u;
    const double a = fabs(x);
    if (isnan(x))
        return (orc_f16)(sign | 0x7e00u);
    if (a >= 65520.0)                           /* halfway between 65504 and 2^16 rounds to even: infinity */
        return (orc_f16)(sign | 0x7c00u);
    if (a < 0x1p-14) {
        /* subnormal range: units of 2^-24; 1024 units is the smallest normal, whose
         * bit pattern is exactly 1024 */
        return (orc_f16)(sign | (orc_f16)nearbyint(ldexp(a, 24)));
    }
    int ex;
    (void)frexp(a, &ex);                        /* a = f * 2^ex, f in [0.5, 1) */
    int e = ex - 1;                             /* a in [2^e, 2^(e+1)) */
    double r = nearbyint(ldexp(a, 10 - e));     /* in [1024, 2048], ties to even */
    if (r == 2048.0) {
        r = 1024.0;
        e += 1;
    }
    return (orc_f16)(sign | (orc_f16)((e + 15) << 10) | (orc_f16)((int)r - 1024));
}

static inline orc_f16 f16_add(orc_f16 a, orc_f16 b)
{
    return orc_f16_from_double(orc_f16_to_double(a) + orc_f16_to_double(b));
}
static inline orc_f16 f16_mul(orc_f16 a, orc_f16 b)
{
    return orc_f16_from_double(orc_f16_to_double(a) * orc_f16_to_double(b));
}
#define OP_ADD_H(T, U, a, b) f16_add(a, b)
#define OP_MUL_H(T, U, a, b) f16_mul(a, b)
#define OP_MAX_H(T, U, a, b) ((orc_f16_to_double(b) > orc_f16_to_double(a)) ? (b) : (a))
#define OP_MIN_H(T, U, a, b) ((orc_f16_to_double(b) < orc_f16_to_double(a)) ? (b) : (a))
DEFINE_REDUCE(add_f16, orc_f16, orc_f16, OP_ADD_H)
DEFINE_REDUCE(mul_f16, orc_f16, orc_f16, OP_MUL_H)
DEFINE_REDUCE(max_f16, orc_f16, orc_f16, OP_MAX_H)
DEFINE_REDUCE(min_f16, orc_f16, orc_f16, OP_MIN_H)

/* Boolean elements under `a + b` and `a * b`.  The JIT types bool + bool and
 * bool * bool as int64, and every store into the kernels' boolean arrays (shared
 * partials :32-37, `partials[blkid]` :96, the result) converts back with `!= 0`; the
 * per-thread accumulator of the strided loop (:78-81) is unified to int64 and holds a
 * count (a product of 0/1 values) that cannot wrap.  Whatever the association, the
 * result is therefore "any element or init is true" for +, "all are true" for *,
 * as a boolean.  One byte per element, 0 or 1. */
#define OP_ADD_B(T, U, a, b) ((T)((((int64_t)((a) != 0)) + ((int64_t)((b) != 0))) != 0))
#define OP_MUL_B(T, U, a, b) ((T)((((int64_t)((a) != 0)) * ((int64_t)((b) != 0))) != 0))
DEFINE_REDUCE(add_b1, uint8_t, uint8_t, OP_ADD_B)
DEFINE_REDUCE(mul_b1, uint8_t, uint8_t, OP_MUL_B)

/* Association-free yardsticks for the floating-point tolerance
 * |err| <= 2 n eps sum|x|: the sum and the sum of magnitudes accumulated in
 * long double with Neumaier compensation. */
static void neumaier(long double x, long double *s, long double *c)
{
    long double t = *s + x;
    if (fabsl(*s) >= fabsl(x))
        *c += (*s - t) + x;
    else
        *c += (x - t) + *s;
    *s = t;
}
void orc_sum_exact_f32(const float *a, int64_t n, double *sum, double *sum_abs)
{
    long double s = 0, c = 0, sa = 0, ca = 0;
    for (int64_t i = 0; i < n; ++i) {
        neumaier(a[i], &s, &c);
        neumaier(fabsl((long double)a[i]), &sa, &ca);
    }
    *sum = (double)(s + c);
    *sum_abs = (double)(sa + ca);
}
void orc_sum_exact_f64(const double *a, int64_t n, double *sum, double *sum_abs)
{
    long double s = 0, c = 0, sa = 0, ca = 0;
    for (int64_t i = 0; i < n; ++i) {
        neumaier(a[i], &s, &c);
        neumaier(fabsl((long double)a[i]), &sa, &ca);
    }
    *sum = (double)(s + c);
    *sum_abs = (double)(sa + ca);
}

/* ------------------------------------------------------------------------- */
/* Transpose                                                                  */
/* ------------------------------------------------------------------------- */

/* kernels/transpose.py:10-65: out[j, i] = in[i, j] for a 2-D array of any item
 * size and any (byte) strides on either side.  rows/cols are the shape of the
 * input. */
void orc_transpose(const char *in, char *out, int64_t rows, int64_t cols,
                   int64_t in_s0, int64_t in_s1, int64_t out_s0, int64_t out_s1,
                   int64_t itemsize)
{
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t j = 0; j < cols; ++j)
            memcpy(out + j * out_s0 + i * out_s1, in + i * in_s0 + j * in_s1,
                   (size_t)itemsize);
}

/* ------------------------------------------------------------------------- */
/* Extent of a strided buffer                                                 */
/* ------------------------------------------------------------------------- */

/* cext/mviewbuf.c:76-135 get_extents with ptr = 0: half-open byte range
 * [start, end) touched by an array of the given shape and byte strides; the
 * range is empty when any dimension is 0. */
void orc_extents(const int64_t *shape, const int64_t *strides, int ndim,
                 int64_t itemsize, int64_t *start, int64_t *end)
{
    int64_t lo = 0, hi = 0;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 0) {
            *start = 0;
            *end = 0;
            return;
        }
        if (strides[d] > 0)
            hi += strides[d] * (shape[d] - 1);
        else if (strides[d] < 0)
            lo += strides[d] * (shape[d] - 1);
    }
    *start = lo;
    *end = hi + itemsize;
}

// The two transcendental steps of Box-Muller, specialised to the arguments the
// generators produce:
//
//   bm_log_f32(u)  natural logarithm of a float32 in (0, 1] (any positive normal
//                  float32 works), evaluated in double to within 0.52 units in the last
//                  place (4.5 for u between 1/2 and 1, where terms cancel) - its callers
//                  round it to float32, and for EVERY float32 in [2^-53, 1] (all a
//                  generator can produce besides 0) that float32 is the one the correctly
//                  rounded double logarithm rounds to; u == 0 gives -infinity.
//   bm_cos_2pi(x)  cosine of a double in [0, 6.2832], i.e. of 2*pi*u, within one unit
//                  in the last place of double.
//   bm_neg_sqrt_of_neg(w)  -sqrt(-w) for the range that occurs, w = 2 log(u).
//
// The general-purpose library routines spend most of their time on cases that
// cannot occur here (subnormals, huge arguments, Payne-Hanek reduction): on
// MI355X they cost 650 us (log) and 460 us (cos) per 2^28 normals against 150 us for
// the square root and 530 us for everything else including the stores.
//
// Both functions are plain C++ so that a host build can sweep them against a
// long-double reference; BM_FN is the only thing that differs between the builds.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

#ifdef __HIPCC__
#define BM_FN __host__ __device__ __forceinline__
#else
#define BM_FN inline
#endif

namespace bm {

// a * b + c in one instruction whose addend may be a constant in a scalar register.  Left to
// itself the compiler keeps some addends of a Horner chain in vector registers and copies
// them before every accumulating multiply-add: one more vector instruction per step.
BM_FN double fma_const(double a, double b, double c)
{
#ifdef __HIP_DEVICE_COMPILE__
    double d;
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "s"(c));
    return d;
#else
    return __builtin_fma(a, b, c);
#endif
}

// ---- logarithm -------------------------------------------------------------------
// u = 2^e * m with m in [sqrt(1/2), sqrt(2)).  The 2^23 mantissa patterns of m are cut
// into 128 runs of 2^16; run j has a centre c_j (1.0 for the run that contains 1.0)
// and the table holds q_j = RN(1 / c_j) and t_j = -log(q_j) as a double-double, so that
//     log(m) = t_j + log1p(r),  r = m * q_j - 1  (|r| <= 2^-8)
// holds exactly.  t_hi keeps 42 fractional bits: e * ln2_hi + t_hi is then exact.  (The table
// words are stored doubled, for the evaluation of 2 log(u) below.)
// Nothing is carried in two parts beyond that: a compensated evaluation (r as a sum of
// two doubles, error-free addition of the leading terms) is good to 0.513 units in the
// last place at 20 double-precision operations; the 12 below lose up to 4.5 where u is
// just below 1, and a sweep over all 444 596 224 possible arguments
// (tests/boxmuller_math_check.cpp) shows that no float32 rounding moves.  (One table word per run instead of two, or ln 2 in one
// piece, moves one of them.)
// (The table also carries the two coefficient sets of the cosine, see below: it is the
// one block of constants the generators keep in LDS.)
struct LogTable {
    double q[128];
    double t_hi[128];
    double t_lo[128];
    double trig[2][6];  // [0]: C6..C1 (cosine kernel), [1]: S6..S1 (sine kernel)
};
constexpr uint32_t kSqrtHalfBits = 0x3f3504f3u;  // float32 bits of sqrt(1/2)

inline float bm_bits_to_float(uint32_t b)
{
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

// Host side: fill the table (long double carries 64 bits, the table needs ~100
// between t_hi and t_lo, which the split provides: t_hi is exact by construction).
inline void build_log_table(LogTable &t)
{
    for (int j = 0; j < 128; ++j) {
        const uint32_t first = kSqrtHalfBits + ((uint32_t)j << 16), last = first + 0xffffu;
        const double lo = (double)bm_bits_to_float(first), hi = (double)bm_bits_to_float(last);
        const double c = (lo <= 1.0 && 1.0 <= hi) ? 1.0 : 0.5 * (lo + hi);
        const double q = 1.0 / c;
        const long double full = -logl((long double)q);
        const double hi_part = (double)(std::floor((double)full * 0x1p42) * 0x1p-42);
        t.q[j] = q;
        t.t_hi[j] = 2.0 * hi_part;  // the table serves 2 log(u), see log2x_positive_f32
        t.t_lo[j] = 2.0 * (double)(full - (long double)hi_part);
    }
    const double c[6] = {-0x1.8fae9be8838d4p-37, 0x1.1ee9ebdb4b1c4p-29, -0x1.27e4f809c52adp-22,
                         0x1.a01a019cb159p-16,   -0x1.6c16c16c15177p-10, 0x1.555555555554cp-5};
    const double sn[6] = {0x1.5d93a5acfd57cp-33,  -0x1.ae5e68a2b9cebp-26, 0x1.71de357b1fe7dp-19,
                          -0x1.a01a019c161d5p-13, 0x1.111111110f8a6p-7,   -0x1.5555555555549p-3};
    for (int k = 0; k < 6; ++k) {
        t.trig[0][k] = c[k];
        t.trig[1][k] = sn[k];
    }
}

// `Tab` in the functions below: a pointer to a LogTable - `const LogTable *`, or on the device
// one that carries the LDS address space, so that the look-ups are LDS instructions with
// 32-bit addresses.
// Returns 2 log(u): the generators want -2 log(u), the doubling is exact in every step (table
// words, coefficients and ln 2 carry the factor), and the sign is a source modifier where the
// value is used - one multiplication less than doubling the rounded logarithm.
template <typename Tab> BM_FN double log2x_positive_f32(float u, Tab tab)
{
    uint32_t bits;
#ifdef __HIP_DEVICE_COMPILE__
    bits = __float_as_uint(u);
#else
    std::memcpy(&bits, &u, 4);
#endif
    const uint32_t ix = bits - kSqrtHalfBits;
    const int e = (int32_t)ix >> 23;
    const uint32_t j = (ix >> 16) & 127u;
    const uint32_t mbits = (ix & 0x007fffffu) + kSqrtHalfBits;
    float mf;
#ifdef __HIP_DEVICE_COMPILE__
    mf = __uint_as_float(mbits);
#else
    std::memcpy(&mf, &mbits, 4);
#endif
    const double m = (double)mf, fe = (double)e;
    // r = RN(m * q_j - 1): one rounding, relative to r itself
    const double r = __builtin_fma(m, tab->q[j], -1.0);
    // 2 (log1p(r) - r), |r| <= 2^-8: the r^7 / 7 term is below 2^-58
    double p = fma_const(r, -2.0 / 6.0, 2.0 / 5.0);
    p = fma_const(r, p, -2.0 / 4.0);
    p = fma_const(r, p, 2.0 / 3.0);
    p = __builtin_fma(r, p, -1.0);
    const double ln2_hi = 2.0 * 0x1.62e42feep-1;       // 32 bits of ln 2, doubled
    const double ln2_lo = 2.0 * 0x1.a39ef35793c76p-33; // ln 2 - ln2_hi, doubled
    const double hi = __builtin_fma(fe, ln2_hi, tab->t_hi[j]);  // exact
    const double lo = __builtin_fma(r * r, p, __builtin_fma(fe, ln2_lo, tab->t_lo[j]));
    return hi + __builtin_fma(r, 2.0, lo);             // the small terms first
}

template <typename Tab> BM_FN double bm_log_f32(float u, Tab tab)
{
    const double v = 0.5 * log2x_positive_f32(u, tab);
    return (u == 0.0f) ? -HUGE_VAL : v;
}

// What the generators use: 2 log(u) rounded to float32, which is twice the float32 the logarithm
// rounds to.  The case u == 0 is sorted out after the rounding, on one 32-bit word instead of two.
template <typename Tab> BM_FN float bm_log2x_f32_rounded(float u, Tab tab)
{
    const float v = (float)log2x_positive_f32(u, tab);
    return (u == 0.0f) ? -HUGE_VALF : v;
}
template <typename Tab> BM_FN float bm_log_f32_rounded(float u, Tab tab)
{
    return 0.5f * bm_log2x_f32_rounded(u, tab);
}

// ---- cosine ------------------------------------------------------------------------
// x = n * pi/2 + (y0 + y1), n = 0..4, |y0| <= pi/4 (+ a rounding's worth), with pi/2
// carried to 119 bits in three pieces so that y0 + y1 is good to 2^-65 relative even
// for x = RN(pi/2), where everything but 6e-17 cancels.  y0 is the difference rounded once and y1
// what it lacks: below 2^-53 of y0 except where the difference cancels, and small against y0 there
// too, which is all the two formulas below ask of the pair (a y0 that also absorbs the third piece,
// as a general-purpose reduction makes it, costs four more operations and changes nothing the
// sweeps see).  On [-pi/4, pi/4], with
// z = y0^2 (coefficients S1..S6, C1..C6: the minimax sets of fdlibm's __kernel_sin /
// __kernel_cos),
//     sin(y0 + y1) = y0 + [ y0 z  (S1 + z (S2 + ... z S6)) + y1 (1 - z/2) ]
//     cos(y0 + y1) = w  + [ z^2   (C1 + z (C2 + ... z C6)) + ((1 - w) - z/2) - y0 y1 ],  w = 1 - z/2
// have the same shape, base + fma(factor, Horner(z), tail).  Double-precision
// instructions are what bounds the generators, so ONE Horner chain runs: the quadrant
// picks factor, tail and base per lane (32-bit selects) and the row of the coefficient
// table (loads from LDS on the device, which cost the vector ALU nothing).
// NEGATED: the cosine with its sign flipped, at no cost (the quadrant's sign bit is an added constant).
template <bool NEGATED = false, typename Tab> BM_FN double bm_cos_2pi(double x, Tab tab)
{
    const double inv_pio2 = 0x1.45f306dc9c883p-1;
    const double pio2_1 = 0x1.921fb544p+0;             // first 33 bits of pi/2
    const double pio2_2 = 0x1.0b4611a6p-34;            // next 33 bits
    const double pio2_2t = 0x1.3198a2e037073p-69;      // pi/2 - pio2_1 - pio2_2
    // x * 2/pi rounded to an integer in one fused operation: added to 1.5 * 2^52 the product loses
    // its fraction (to nearest, ties to even), and the integer stands in the low word of the sum
    const double shifted = __builtin_fma(x, inv_pio2, 0x1.8p52);
    const double fn = shifted - 0x1.8p52;
#ifdef __HIP_DEVICE_COMPILE__
    const int n = __double2loint(shifted);
#else
    int64_t shifted_bits;
    std::memcpy(&shifted_bits, &shifted, 8);
    const int n = (int)(uint32_t)shifted_bits;
#endif
    const double t = __builtin_fma(-fn, pio2_1, x);    // exact: fn * pio2_1 has 36 bits
    const double y0 = __builtin_fma(-fn, pio2_2, t);   // fn * pio2_2 is exact too: one rounding, of t - fn * pio2_2
    // what that rounding lost (t - y0 is exact and so is the fused operation), less the third piece
    const double y1 = __builtin_fma(-fn, pio2_2t, __builtin_fma(-fn, pio2_2, t - y0));

    const bool odd = (n & 1) != 0;                     // odd quadrant: -+sin, even: +-cos
    auto k = &tab->trig[n & 1][0];                     // S6..S1 : C6..C1
#ifdef __HIP_DEVICE_COMPILE__
    // the row's address as ONE value: the six loads then differ in their offset fields only
    // (otherwise the compiler hoists "table + 16" and "table + 32" and adds the row to each)
    asm("" : "+v"(k));
#endif
    const double z = y0 * y0;
    const double wc = __builtin_fma(-0.5, z, 1.0);     // 1 - z/2, one rounding (z/2 is exact)
    double q = __builtin_fma(z, k[0], k[1]);
    q = __builtin_fma(z, q, k[2]);
    q = __builtin_fma(z, q, k[3]);
    q = __builtin_fma(z, q, k[4]);
    q = __builtin_fma(z, q, k[5]);
    const double factor = z * (odd ? y0 : z);
    const double tail_sin = y1 * wc;
    // (1 - wc) - z/2: what the rounding of wc lost; 1 - wc is exact, so this is too
    const double tail_cos = __builtin_fma(-y0, y1, __builtin_fma(-0.5, z, 1.0 - wc));
    const double tail = odd ? tail_sin : tail_cos;
    const double base = odd ? y0 : wc;
    const double pick = base + __builtin_fma(factor, q, tail);
    // cos(n*pi/2 + y): n&3 = 0: cos y, 1: -sin y, 2: -cos y, 3: sin y
#ifdef __HIP_DEVICE_COMPILE__
    // bit 1 of n + 1 moved onto the sign bit and xor-ed in: a shift-and-add and one
    // three-input bit operation, hi ^ (sign & 0x80000000)
    const uint32_t sign = ((uint32_t)n << 30) + (NEGATED ? 0xC0000000u : 0x40000000u);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_bitop3_b32(__double2hiint(pick), sign, 0x80000000u, 0x78);
    return __hiloint2double((int)hi, __double2loint(pick));
#else
    return ((((n + 1) & 2) != 0) != NEGATED) ? -pick : pick;
#endif
}

// Square root of -2 log(u): zero, +infinity or a double in [2^-22, 210] - never
// subnormal, so the range scaling the general routine wraps around the same steps (two
// ldexp, a compare, two selects) is left out.  Reciprocal square root estimate, one
// coupled Newton step on (g, h) ~ (sqrt a, 1 / (2 sqrt a)), one correction of g: the
// estimate is good to 2^-26 or so, the coupled step squares that, and the correction -
// the residual a - g^2 is exact in the fused operation - leaves an error near 2^-100 before
// the one rounding.  (A second correction, as the general routine has it, changes none of
// the float64 normals over all 260 million values the first uniform can take.  Leaving h
// as the estimate gave it would save an operation and leave an error near 2^-77: enough to
// move the last bit of some thirty of those values.)
// Zero and infinity, where the estimate is infinite or zero, are told by one class test.
// The argument comes negated, w = 2 log(u) <= 0, and the root goes out negated: -sqrt(-w), and w
// itself where that is a zero or -infinity.  Every negation below is an operand modifier of an
// instruction that is there anyway; the caller multiplies by the negated cosine.
BM_FN double bm_neg_sqrt_of_neg(double w)
{
#ifdef __HIP_DEVICE_COMPILE__
    const double y = __builtin_amdgcn_rsq(-w);
    double g = -w * y;
    double h = 0.5 * y;
    const double r = __builtin_fma(-h, g, 0.5);
    g = __builtin_fma(g, r, g);
    h = __builtin_fma(h, r, h);
    const double d = __builtin_fma(-g, g, -w);
    const double neg_g = __builtin_fma(-d, h, -g);
    constexpr int kZeroOrMinusInfinity = 0x020 | 0x040 | 0x004;  // -0, +0, -infinity
    return __builtin_amdgcn_class(w, kZeroOrMinusInfinity) ? w : neg_g;
#else
    return (w == 0.0) ? w : -std::sqrt(-w);
#endif
}

}  // namespace bm

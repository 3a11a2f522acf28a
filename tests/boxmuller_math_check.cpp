// Host-side sweep of numba_cuda_amd/csrc/boxmuller_math.h against long double.
// Prints, per case, the largest error in units of the last place of the double
// result and the number of inputs whose rounding to float32 differs from the
// rounding of the long-double value.  Built and run by tests/test_boxmuller_math.py.
#include "boxmuller_math.h"
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

static double ulp_of(long double want)
{
    int e;
    frexpl(want, &e);                    // want = f * 2^e, f in [0.5, 1)
    return (double)ldexpl(1.0L, e - 53);
}

int main(int argc, char **argv)
{
    const uint32_t stride = argc > 1 ? (uint32_t)atoi(argv[1]) : 1;   // 1 = every mantissa
    bm::LogTable tab;
    bm::build_log_table(tab);

    // logarithm: every float32 of the binades [2^-k, 2^-k+1), k = 1..3, 24, 53, and 1.0
    const int binades[] = {1, 2, 3, 24, 53};
    for (int k : binades) {
        double worst = 0;
        long flips = 0, count = 0;
        for (uint32_t mant = 0; mant < (1u << 23); mant += stride) {
            const uint32_t bits = ((uint32_t)(127 - k) << 23) | mant;
            const float u = bm::bm_bits_to_float(bits);
            const double got = bm::bm_log_f32(u, &tab);
            const long double want = logl((long double)u);
            const double err = (double)fabsl((long double)got - want) / ulp_of(want);
            if (err > worst)
                worst = err;
            flips += ((float)got != (float)want);
            ++count;
        }
        printf("log binade 2^-%d: n=%ld worst_ulp=%.4f float_flips=%ld\n", k, count, worst, flips);
    }
    {
        const double one = bm::bm_log_f32(1.0f, &tab), zero = bm::bm_log_f32(0.0f, &tab);
        printf("log edge: log(1)=%g signbit=%d log(0)=%g\n", one, (int)std::signbit(one), zero);
        const float one_f = bm::bm_log_f32_rounded(1.0f, &tab), zero_f = bm::bm_log_f32_rounded(0.0f, &tab);
        printf("log edge, rounded: log(1)=%g signbit=%d log(0)=%g\n", (double)one_f, (int)std::signbit(one_f),
               (double)zero_f);
    }

    // logarithm, what its callers use: the float32 it rounds to, for every float32 a generator
    // can produce besides zero - exponents -53 ... -1, every mantissa (second argument "all";
    // eight threads, two seconds).  The yardstick is the exact logarithm rounded to double and
    // then to float32.  (Rounding the exact logarithm to float32 in one step differs for one
    // argument of them all, 0x1.827a74p-7, whose logarithm -0x1.1c2b1efffffffb1p+2 rounds to a
    // double that lies exactly between two float32.)
    if (argc > 2 && std::strcmp(argv[2], "all") == 0) {
        std::atomic<long> flips{0}, count{0};
        std::atomic<int> next{1};
        std::vector<std::thread> workers;
        for (int t = 0; t < 8; ++t)
            workers.emplace_back([&] {
                for (;;) {
                    const int k = next.fetch_add(1);
                    if (k > 53)
                        break;
                    long f = 0;
                    for (uint32_t mant = 0; mant < (1u << 23); ++mant) {
                        const float u = bm::bm_bits_to_float(((uint32_t)(127 - k) << 23) | mant);
                        // rounded twice, to double and then to float32, as the callers do and as the
                        // CPU restatement of the generators does
                        f += bm::bm_log_f32_rounded(u, &tab) != (float)(double)logl((long double)u);
                    }
                    flips += f;
                    count += 1 << 23;
                }
            });
        for (auto &w : workers)
            w.join();
        printf("log every float32 of [2^-53, 1): n=%ld float_flips=%ld\n", count.load(), flips.load());

        // cosine of the float32 variant, the same way: the angle is RN32(RN32(2 pi) * u), the
        // cosine is taken in double and rounded to float32; every u in [2^-53, 1)
        std::atomic<long> cflips{0}, ccount{0};
        next = 1;
        workers.clear();
        for (int t = 0; t < 8; ++t)
            workers.emplace_back([&] {
                for (;;) {
                    const int k = next.fetch_add(1);
                    if (k > 53)
                        break;
                    long f = 0;
                    for (uint32_t mant = 0; mant < (1u << 23); ++mant) {
                        const float u = bm::bm_bits_to_float(((uint32_t)(127 - k) << 23) | mant);
                        const double x = (double)(6.283185307179586f * u);
                        f += (float)bm::bm_cos_2pi(x, &tab) != (float)(double)cosl((long double)x);
                    }
                    cflips += f;
                    ccount += 1 << 23;
                }
            });
        for (auto &w : workers)
            w.join();
        printf("cos f32 every float32 of [2^-53, 1): n=%ld float_flips=%ld\n", ccount.load(), cflips.load());
    }

    // cosine: x = RN(RN(2 pi) * u) for u = k / 2^24 (float64 variant) and
    // x = (double)(RN32(RN32(2 pi) * u)) (float32 variant), every k
    for (int variant = 0; variant < 2; ++variant) {
        double worst = 0;
        long flips = 0, count = 0;
        for (uint32_t k = 0; k <= (1u << 24); k += stride) {
            const float u = (float)k * 0x1p-24f;
            const double x = variant == 0 ? 6.283185307179586 * (double)u : (double)(6.283185307179586f * u);
            const double got = bm::bm_cos_2pi(x, &tab);
            const long double want = cosl((long double)x);
            const double err = (double)fabsl((long double)got - want) / ulp_of(want);
            if (err > worst)
                worst = err;
            flips += ((float)got != (float)want);
            ++count;
        }
        printf("cos variant %s: n=%ld worst_ulp=%.4f float_flips=%ld\n", variant ? "f32" : "f64", count, worst, flips);
    }
    // small arguments of the f64 variant: u below 2^-24 (the uniform can be as small as 2^-53)
    {
        double worst = 0;
        for (int e = 25; e <= 53; ++e)
            for (uint32_t mant = 0; mant < (1u << 23); mant += 4099 * stride) {
                const float u = bm::bm_bits_to_float(((uint32_t)(127 - e) << 23) | mant);
                const double x = 6.283185307179586 * (double)u;
                const long double want = cosl((long double)x);
                const double err = (double)fabsl((long double)bm::bm_cos_2pi(x, &tab) - want) / ulp_of(want);
                if (err > worst)
                    worst = err;
            }
        printf("cos tiny arguments: worst_ulp=%.4f\n", worst);
    }
    return 0;
}

// CPU build of the SFloat / DFloat function cores of cumo_amd/csrc/ew_ops.h, for
// tests/test_nmath_vectors.py. Every step of those algorithms is an IEEE operation (fused
// multiply-adds included) except the device's reciprocal and reciprocal square root estimates,
// which the algorithms refine by a Newton step to 2^-44 and for which the exact quotient and
// root stand in here: this program computes what the device computes up to that.
//
//   float_cores_check vectors <file>   reads "name type n" blocks of arguments (hex bit
//                                      patterns), prints the results as hex bit patterns
//   float_cores_check pow <n>          n random (base, exponent) pairs through the SFloat power's arithmetic against
//                                      (float)glibc pow; prints pairs tried, mismatches and the largest difference in ulps
//   float_cores_check dsweep <n>       n random doubles through each DFloat core that works on pairs of doubles (tanh sinh
//                                      cosh erfc log1p asinh acosh atanh) against the long double function; prints, per
//                                      function, arguments tried, the largest error in ulps and where it was
//   float_cores_check dpow <n>         n random (base, exponent) pairs through the DFloat power's arithmetic against powl
//   float_cores_check halves <stride>  every stride-th float through the SFloat power by whole numbers of halves against (float)glibc pow
//   float_cores_check two <n>          n random pairs through the SFloat atan2 and hypot against (float)glibc in double
//   float_cores_check sweep <stride>   every stride-th float bit pattern through each SFloat
//                                      core against (float)glibc((double)x); prints, per
//                                      function, patterns tried, mismatches and the largest
//                                      difference in ulps
#define CUMO_HIP_HOST_CHECK 1
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
static inline int __double2hiint(double d) { uint64_t u; std::memcpy(&u, &d, 8); return (int)(uint32_t)(u >> 32); }
static inline int __double2loint(double d) { uint64_t u; std::memcpy(&u, &d, 8); return (int)(uint32_t)u; }
static inline double __hiloint2double(int hi, int lo) { uint64_t u = ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo; double d; std::memcpy(&d, &u, 8); return d; }
static inline long long __double_as_longlong(double d) { long long u; std::memcpy(&u, &d, 8); return u; }
static inline double __longlong_as_double(long long u) { double d; std::memcpy(&d, &u, 8); return d; }
static inline int __float_as_int(float f) { int u; std::memcpy(&u, &f, 4); return u; }
static inline float __int_as_float(int u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline unsigned __float_as_uint(float f) { unsigned u; std::memcpy(&u, &f, 4); return u; }
static inline float __uint_as_float(unsigned u) { float f; std::memcpy(&f, &u, 4); return f; }

#include "../cumo_amd/csrc/ew_ops.h"

using namespace cumo_hip;

static double sinc_ref(double x) { return x == 0 ? 1.0 : std::sin(x) / x; }
typedef float (*F32)(float);
typedef double (*F64)(double);
struct Core32 { const char* name; F32 f; F64 ref; };
static const Core32 kCores32[] = {
    {"exp", exp_float_rounded_once, exp},     {"log", log_float_rounded_once<0>, log},   {"log2", log_float_rounded_once<2>, log2},
    {"log10", log_float_rounded_once<10>, log10}, {"log1p", log1p_float_rounded_once, log1p}, {"tanh", tanh_float_rounded_once, tanh},
    {"sinh", sinh_float_rounded_once, sinh},  {"cosh", cosh_float_rounded_once, cosh},   {"expm1", expm1_float_rounded_once, expm1},
    {"asinh", asinh_float_rounded_once, asinh}, {"acosh", acosh_float_rounded_once, acosh}, {"atanh", atanh_float_rounded_once, atanh},
    {"sin", trig_float_rounded_once<0>, sin}, {"cos", trig_float_rounded_once<1>, cos}, {"tan", trig_float_rounded_once<2>, tan},
    {"atan", atan_float_rounded_once, atan},  {"erf", erf_float_rounded_once, erf},
    {"asin", asin_acos_float_rounded_once<false>, asin}, {"acos", asin_acos_float_rounded_once<true>, acos},
    {"erfc", erfc_float_rounded_once, erfc},  {"sinc", sinc_float_rounded_once, sinc_ref},
};
struct Core64 { const char* name; F64 f; };
static const Core64 kCores64[] = {{"log", log_double<0>}, {"log2", log_double<2>}, {"log10", log_double<10>},
                                  {"tanh", tanh_double}, {"sinh", sinh_double}, {"cosh", cosh_double}, {"erfc", erfc_double},
                                  {"log1p", log1p_double}, {"asinh", asinh_double}, {"acosh", acosh_double}, {"atanh", atanh_double}};

static int64_t ordered(float f) { int32_t i; std::memcpy(&i, &f, 4); return i < 0 ? (int64_t)INT32_MIN - i : i; }

int main(int argc, char** argv) {
    if (argc >= 3 && std::strcmp(argv[1], "sweep") == 0) {
        const uint32_t stride = (uint32_t)std::strtoul(argv[2], nullptr, 10);
        for (const Core32& c : kCores32) {
            uint64_t tried = 0, bad = 0;
            int64_t worst = 0;
            for (uint64_t b = 0; b < (1ull << 32); b += stride) {
                uint32_t u = (uint32_t)b;
                float x; std::memcpy(&x, &u, 4);
                const float got = c.f(x), want = (float)c.ref((double)x);
                ++tried;
                if (got != got && want != want) continue;
                uint32_t gu, wu; std::memcpy(&gu, &got, 4); std::memcpy(&wu, &want, 4);
                if (gu == wu) continue;
                if (got != got || want != want) { ++bad; worst = 1 << 30; continue; }
                if (got == want) { ++bad; if (worst < 1) worst = 1; continue; }  // +0 against -0
                int64_t d = ordered(got) - ordered(want);
                if (d < 0) d = -d;
                ++bad;
                if (d > worst) worst = d;
            }
            std::printf("%s %llu %llu %lld\n", c.name, (unsigned long long)tried, (unsigned long long)bad, (long long)worst);
        }
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "dsweep") == 0) {
        // n random doubles per DFloat core (magnitudes spread evenly over the exponents from 2^-40 up to the function's
        // range, both signs, then arguments next to the ends of the ranges) against the long double function, whose
        // own error is 2^-11 ulp of a double; prints, per function, arguments tried and the largest error in ulps
        const uint64_t n = std::strtoull(argv[2], nullptr, 10);
        struct CoreL { const char* name; F64 f; long double (*ref)(long double); double top; };
        const CoreL cores[] = {{"tanh", tanh_double, tanhl, 40.0}, {"sinh", sinh_double, sinhl, 710.4}, {"cosh", cosh_double, coshl, 710.4},
                               {"erfc", erfc_double, erfcl, 26.5}, {"log1p", log1p_double, log1pl, 1e300}, {"asinh", asinh_double, asinhl, 1e300},
                               {"acosh", acosh_double, acoshl, 1e300}, {"atanh", atanh_double, atanhl, 1.0}};
        for (const CoreL& c : cores) {
            uint64_t state = 0x9e3779b97f4a7c15ull;
            auto next = [&state]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
            double worst = 0.0, worst_x = 0.0;
            for (uint64_t it = 0; it < n; ++it) {
                const uint64_t a = next(), b = next();
                double x;
                if (it % 4 != 3 || c.top > 1e10) {
                    const double lo_e = -40.0, hi_e = std::log2(c.top);
                    const double e = lo_e + (hi_e - lo_e) * (double)(a >> 11) * 0x1p-53;
                    x = std::exp2(e) * (1.0 + (double)(b >> 12) * 0x1p-52 * 1e-3);
                } else {
                    x = c.top * (double)(a >> 11) * 0x1p-53;   // evenly over the range: mostly large arguments
                }
                if (x > c.top) x = c.top;
                const bool is = std::strcmp(c.name, "acosh") == 0;
                if (is) x = 1.0 + x;                                     // 1 + 2^-40 ... : the domain of acosh
                else if (std::strcmp(c.name, "atanh") == 0) { if (x >= 1.0) x = 1.0 - 0x1p-53 * (double)(1 + (a & 0xffff)); }
                else if (std::strcmp(c.name, "log1p") == 0 && (b & 1) && x >= 1.0) x = 1.0 - 0x1p-53 * (double)(1 + (a & 0xffff));
                if ((b & 1) && !is) x = -x;
                const double got = c.f(x);
                const long double want = c.ref((long double)x);
                int ex;
                std::frexp((double)want, &ex);
                const long double ulp = std::ldexp(1.0L, ex - 53);
                const double err = (double)(fabsl((long double)got - want) / ulp);
                if (err > worst) { worst = err; worst_x = x; }
            }
            std::printf("%s %llu %.4f %a\n", c.name, (unsigned long long)n, worst, worst_x);
        }
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "two") == 0) {
        // n random pairs of floats through the SFloat atan2 (finite arguments that are not zero: the others are the
        // library's) and hypot (every argument) against (float)glibc((double)., (double).): magnitudes spread over every
        // float exponent, over neighbouring exponents (where the quotient's reduction changes form), and special values
        // for hypot; prints, per function, pairs tried, mismatches and the largest difference in ulps
        const uint64_t n = std::strtoull(argv[2], nullptr, 10);
        for (int which = 0; which < 3; ++which) {
            uint64_t state = 0x9e3779b97f4a7c15ull, tried = 0, bad = 0;
            int64_t worst = 0;
            auto next = [&state]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
            const uint32_t special[] = {0u, 0x80000000u, 0x7f800000u, 0xff800000u, 0x7fc00000u, 1u, 0x007fffffu, 0x7f7fffffu, 0x3f800000u};
            for (uint64_t it = 0; it < n; ++it) {
                const uint64_t a = next(), b = next();
                uint32_t ux = (uint32_t)a, uy = (uint32_t)b;
                if (it % 2 == 1) {
                    // exponents within two of each other
                    const uint32_t ex = (ux >> 23) & 0xffu;
                    const uint32_t ey = (uint32_t)((int)ex + (int)((b >> 40) % 5) - 2) & 0xffu;
                    uy = (uy & 0x807fffffu) | (ey << 23);
                }
                if (which == 1 && it % 97 == 0) ux = special[(a >> 33) % 9];
                if (which == 1 && it % 89 == 0) uy = special[(b >> 33) % 9];
                float x, y; std::memcpy(&x, &ux, 4); std::memcpy(&y, &uy, 4);
                float got, want;
                if (which == 0) {
                    if (atan2_is_rare(y, x)) continue;
                    got = atan2_fast(y, x);
                    want = (float)std::atan2((double)y, (double)x);
                } else if (which == 2) {
                    // (quotients of every size up to the limit: the divisor's exponent up to 29 below the dividend's)
                    if (it % 2 == 0) {
                        const uint32_t ex = (ux >> 23) & 0xffu;
                        const uint32_t ey = (uint32_t)((int)ex - (int)((b >> 40) % 31)) & 0xffu;
                        uy = (uy & 0x807fffffu) | (ey << 23);
                        std::memcpy(&y, &uy, 4);
                    }
                    if (it % 5 == 0) { y = (float)(1 + (b >> 50) % 7); x = y * (float)(int)((a >> 40) % 100000) + ((it % 10 == 0) ? 0.0f : y * 0x1p-20f); }
                    if (fmod_is_rare(x, y)) continue;
                    got = fmod_fast(x, y);
                    want = std::fmod(x, y);
                } else {
                    got = hypot_float_rounded_once(x, y);
                    want = (float)std::hypot((double)x, (double)y);
                }
                ++tried;
                if (got != got && want != want) continue;
                uint32_t gu, wu; std::memcpy(&gu, &got, 4); std::memcpy(&wu, &want, 4);
                if (gu == wu) continue;
                ++bad;
                if (got != got || want != want) { worst = 1 << 30; continue; }
                int64_t d = ordered(got) - ordered(want);
                if (d < 0) d = -d;
                if (d > worst) worst = d;
            }
            std::printf("%s %llu %llu %lld\n", which == 0 ? "atan2" : (which == 1 ? "hypot" : "fmod"), (unsigned long long)tried, (unsigned long long)bad, (long long)worst);
        }
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "dpow") == 0) {
        // n random (base, exponent) pairs through the DFloat power's arithmetic against the long double function: bases
        // over every positive normal double with exponents that spread the results over the double range and past
        // both of its ends, bases next to 1 with exponents up to 2^40, and everyday pairs; prints pairs tried and the
        // largest error in ulps (of a normal result: a subnormal one is rounded twice, by the arithmetic and by ldexp)
        const uint64_t n = std::strtoull(argv[2], nullptr, 10);
        uint64_t state = 0x9e3779b97f4a7c15ull;
        auto next = [&state]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
        double worst = 0.0, worst_x = 0.0, worst_y = 0.0, worst_sub = 0.0;
        uint64_t wrong_ends = 0;
        for (uint64_t it = 0; it < n; ++it) {
            const uint64_t a = next(), b = next();
            double x, y;
            const double u = (double)(b >> 11) * 0x1p-53;   // [0, 1)
            if (it % 3 == 0) {
                uint64_t bits = 0x0010000000000000ull + a % (0x7ff0000000000000ull - 0x0010000000000000ull);
                std::memcpy(&x, &bits, 8);
                const double lg = std::log2(x);
                const double target = (2.0 * u - 1.0) * 1090.0;
                y = lg != 0.0 ? target / lg : u * 1000.0;
            } else if (it % 3 == 1) {
                const double d = std::exp2(-1.0 - 50.0 * (double)(a >> 11) * 0x1p-53);   // distance from 1: 2^-51 .. 2^-1
                x = (a & 1) ? 1.0 + d : 1.0 - d;
                const double lg = std::log2(x);
                y = (2.0 * u - 1.0) * 1090.0 / lg;
                if (!(std::fabs(y) < 0x1p40)) y = (2.0 * u - 1.0) * 0x1p40;
            } else {
                x = 0.01 + 100.0 * (double)(a >> 11) * 0x1p-53;
                y = (2.0 * u - 1.0) * 20.0;
            }
            if (pow_double_is_rare(x, y)) continue;
            const double got = pow_double_fast(x, y);
            const long double want = powl((long double)x, (long double)y);
            if (want > 1.7976931348623157e308L * (1.0L + 0x1p-54L) || want < 0x1p-1076L) {
                // past the ends: infinity above; zero (or the smallest subnormal next to the boundary) below
                if (want > 1.7976931348623157e308L ? got != INFINITY : got > 4.9406564584124654e-324) ++wrong_ends;
                continue;
            }
            int ex;
            std::frexp((double)want, &ex);
            const bool sub = ex < -1021;
            const long double ulp = std::ldexp(1.0L, sub ? -1074 : ex - 53);
            const double err = (double)(fabsl((long double)got - want) / ulp);
            if (sub) { if (err > worst_sub) worst_sub = err; }
            else if (err > worst) { worst = err; worst_x = x; worst_y = y; }
        }
        std::printf("pow %llu %.4f %.4f %llu %a %a\n", (unsigned long long)n, worst, worst_sub, (unsigned long long)wrong_ends, worst_x, worst_y);
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "dhalves") == 0) {
        // n random bases between 2^-100 and 2^100 through the DFloat power for every exponent that is a whole number of
        // halves up to 8 either way, against powl; prints, per exponent, bases tried and the largest error in ulps
        const uint64_t n = std::strtoull(argv[2], nullptr, 10);
        for (int twice = -16; twice <= 16; ++twice) {
            if (twice == 0) continue;
            uint64_t state = 0x9e3779b97f4a7c15ull;
            auto next = [&state]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
            double worst = 0.0;
            for (uint64_t it = 0; it < n; ++it) {
                const uint64_t a = next(), b = next();
                const double e = (it % 2) ? 200.0 * (double)(a >> 11) * 0x1p-53 - 100.0 : 4.0 * (double)(a >> 11) * 0x1p-53 - 2.0;
                double x = std::exp2(std::floor(e)) * (1.0 + (double)(b >> 12) * 0x1p-52);
                if (pow_halves_double_is_rare(x)) continue;
                const double got = twice < 0 ? pow_halves_double_fast<true>(x, twice) : pow_halves_double_fast<false>(x, twice);
                const long double want = powl((long double)x, 0.5L * twice);
                int ex;
                std::frexp((double)want, &ex);
                const double err = (double)(fabsl((long double)got - want) / std::ldexp(1.0L, ex - 53));
                if (err > worst) worst = err;
            }
            std::printf("%g %llu %.4f\n", 0.5 * twice, (unsigned long long)n, worst);
        }
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "halves") == 0) {
        // every stride-th float bit pattern through the SFloat power for exponents that are whole numbers of halves
        // against (float)glibc pow in double; prints, per exponent, patterns tried, mismatches and the largest difference in ulps
        const uint32_t stride = (uint32_t)std::strtoul(argv[2], nullptr, 10);
        const int twices[] = {0, 1, -1, 2, -2, 3, -3, 4, -4, 5, -5, 6, 7, 15, -15, 20, 32, 33, -33, 63, 64, -64};
        for (int twice : twices) {
            OpPowHalves<true> down;
            OpPowHalves<false> up;
            down.twice = up.twice = twice;
            const double y = 0.5 * twice;
            uint64_t tried = 0, bad = 0;
            int64_t worst = 0;
            for (uint64_t b = 0; b < (1ull << 32); b += stride) {
                uint32_t u = (uint32_t)b;
                float x; std::memcpy(&x, &u, 4);
                float got = 0.0f;
                if (twice < 0) down(x, 0.0f, got);
                else up(x, 0.0f, got);
                const float want = (float)std::pow((double)x, y);
                ++tried;
                if (got != got && want != want) continue;
                uint32_t gu, wu; std::memcpy(&gu, &got, 4); std::memcpy(&wu, &want, 4);
                if (gu == wu) continue;
                ++bad;
                if (got != got || want != want) { worst = 1 << 30; continue; }
                if (got == want) { if (worst < 1) worst = 1; continue; }  // +0 against -0
                int64_t d = ordered(got) - ordered(want);
                if (d < 0) d = -d;
                if (d > worst) worst = d;
            }
            std::printf("%g %llu %llu %lld\n", y, (unsigned long long)tried, (unsigned long long)bad, (long long)worst);
        }
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "pow") == 0) {
        // n random (base, exponent) pairs: bases over every positive float, exponents spread so that results span the
        // float range (and beyond), then bases next to 1 with large exponents; against (float)pow((double)x, (double)y)
        const uint64_t n = std::strtoull(argv[2], nullptr, 10);
        uint64_t state = 0x9e3779b97f4a7c15ull, tried = 0, bad = 0;
        int64_t worst = 0;
        auto next = [&state]() { state ^= state << 13; state ^= state >> 7; state ^= state << 17; return state; };
        for (uint64_t it = 0; it < n; ++it) {
            const uint64_t a = next(), b = next();
            float x, y;
            if (it % 3 == 0) {
                uint32_t u = (uint32_t)(a % 0x7f800000u); if (u == 0) u = 1; std::memcpy(&x, &u, 4);
                const double lg = std::log2((double)x);
                const double target = ((double)(b % 2000001) / 1000000.0 - 1.0) * 155.0;   // wanted log2 of the result
                y = (float)(lg != 0.0 ? target / lg : (double)(b % 1000));
            } else if (it % 3 == 1) {
                x = 1.0f + ((float)(int64_t)(a % 4000001) - 2000000.0f) * 1.0e-7f * (float)((a >> 32) % 100 + 1);
                y = ((float)(int64_t)(b % 2000001) - 1000000.0f) * (float)((b >> 40) % 1000 + 1) * 1.0e-4f;
            } else {
                x = (float)(a % 1000003) / 1000.0f + 1.0e-3f;
                y = ((float)(int64_t)(b % 200001) - 100000.0f) / 5000.0f;
            }
            if (pow_is_rare(x, y)) continue;
            const float got = pow_fast(x, y), want = (float)std::pow((double)x, (double)y);
            ++tried;
            uint32_t gu, wu; std::memcpy(&gu, &got, 4); std::memcpy(&wu, &want, 4);
            if (gu == wu) continue;
            ++bad;
            int64_t d = (got != got || want != want) ? (1 << 30) : ordered(got) - ordered(want);
            if (d < 0) d = -d;
            if (d > worst) worst = d;
        }
        std::printf("pow %llu %llu %lld\n", (unsigned long long)tried, (unsigned long long)bad, (long long)worst);
        return 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "vectors") == 0) {
        FILE* f = std::fopen(argv[2], "r");
        if (!f) return 2;
        char name[32], type[8];
        unsigned long n;
        while (std::fscanf(f, "%31s %7s %lu", name, type, &n) == 3) {
            std::printf("%s %s %lu\n", name, type, n);
            const bool is32 = std::strcmp(type, "f32") == 0;
            F32 f32 = nullptr; F64 f64 = nullptr;
            if (is32) { for (const Core32& c : kCores32) if (std::strcmp(c.name, name) == 0) f32 = c.f; }
            else { for (const Core64& c : kCores64) if (std::strcmp(c.name, name) == 0) f64 = c.f; }
            for (unsigned long i = 0; i < n; ++i) {
                unsigned long long bits;
                if (std::fscanf(f, "%llx", &bits) != 1) return 3;
                if (is32) {
                    uint32_t u = (uint32_t)bits; float x; std::memcpy(&x, &u, 4);
                    float y = f32 ? f32(x) : NAN; std::memcpy(&u, &y, 4);
                    std::printf("%x\n", u);
                } else {
                    uint64_t u = bits; double x; std::memcpy(&x, &u, 8);
                    double y = f64 ? f64(x) : NAN; std::memcpy(&u, &y, 8);
                    std::printf("%llx\n", (unsigned long long)u);
                }
            }
        }
        std::fclose(f);
        return 0;
    }
    std::fprintf(stderr, "usage: float_cores_check sweep <stride> | vectors <file>\n");
    return 1;
}

// expf evaluated the way the C library on the CPU path evaluates it, so that GPU and CPU
// agree bit for bit on every exp() that feeds an int8 quantiser or a softmax.
//
// The reference calls f32::exp (emit.rs:384, 688-699, 833-840), which on Linux is glibc's
// expf: the table-driven double-precision algorithm of ARM's optimized-routines
// (x*N/ln2 = k + r, 2^(k/N) from a 32-entry table, cubic in r, all in binary64, one final
// rounding to binary32).  glibc selects an FMA build of it on CPUs with FMA; `kFma` follows
// that build, the other branch the plain one.  The two differ only in binary64 rounding and
// give the same binary32 result except when the exact value is within ~1e-16 relative of a
// rounding boundary.
#pragma once

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define FH_HD __host__ __device__
#else
#define FH_HD
#endif

namespace fh {

namespace expf_detail {
FH_HD inline uint64_t tab(int i) {
    // asuint64(2^(i/32)) - (i << 47), i = 0..31
    constexpr uint64_t T[32] = {
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};
    return T[i];
}
FH_HD inline double u64_as_double(uint64_t u) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __longlong_as_double((long long)u);
#else
    double d; memcpy(&d, &u, 8); return d;
#endif
}
FH_HD inline uint64_t double_as_u64(double d) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint64_t)__double_as_longlong(d);
#else
    uint64_t u; memcpy(&u, &d, 8); return u;
#endif
}
}  // namespace expf_detail

// `lookup(i)` returns tab(i): a kernel that keeps a copy of the table close by (LDS) passes its own.
template <bool kFma, typename Lookup>
FH_HD inline float expf_ref_with(float x, Lookup lookup) {
    using namespace expf_detail;
    constexpr double N = 32.0;
    constexpr double InvLn2N = 0x1.71547652b82fep+0 * N;
    constexpr double Shift = 0x1.8p+52;
    constexpr double C0 = 0x1.c6af84b912394p-5 / N / N / N;
    constexpr double C1 = 0x1.ebfce50fac4f3p-3 / N / N;
    constexpr double C2 = 0x1.62e42ff0c52d6p-1 / N;
    if (x != x) return x + x;
    if (x > 0x1.62e42ep6f) return INFINITY;       // > log(2^128)
    if (x < -0x1.9fe368p6f) return 0.0f;          // < log(2^-150); also -inf
    const double xd = (double)x;
    double z = InvLn2N * xd;
    double kd = z + Shift;
    const uint64_t ki = double_as_u64(kd);
    kd -= Shift;
    const double r = z - kd;
    uint64_t t = lookup((int)(ki & 31));
    t += ki << 47;
    const double s = u64_as_double(t);
    double y;
    if (kFma) {
        z = fma(C0, r, C1);
        const double r2 = r * r;
        y = fma(C2, r, 1.0);
        y = fma(z, r2, y);
    } else {
        z = C0 * r + C1;
        const double r2 = r * r;
        y = C2 * r + 1.0;
        y = z * r2 + y;
    }
    y = y * s;
    return (float)y;
}

namespace expf_detail {
struct TabLookup { FH_HD uint64_t operator()(int i) const { return tab(i); } };
}  // namespace expf_detail

template <bool kFma>
FH_HD inline float expf_ref(float x) { return expf_ref_with<kFma>(x, expf_detail::TabLookup{}); }

}  // namespace fh

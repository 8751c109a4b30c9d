// Goldilocks field p = 2^64 - 2^32 + 1 for gfx950 wavefronts.
//
// The VALU has no 64-bit multiplier, so a product is built from four 32x32->64
// partial products (v_mad_u64_u32) and reduced with the two identities
//     2^64 = 2^32 - 1   and   2^96 = -1   (mod p).
// Canonical-in / canonical-out; for arbitrary 64-bit inputs add/sub/mul return the
// same word the reference device functions return
// (prover/kernels/goldilocks.cuh:28-81), so elementwise results agree bit for bit
// even on non-canonical operands.
//
// The same header compiles for the host (VI_HD empty) so that the kernels' index
// logic and arithmetic can be exercised by a CPU build in the test-suite.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define VI_HD __host__ __device__ __forceinline__
#else
#define VI_HD inline
#endif

// Fence for the instruction scheduler (device code only): keeps it from hoisting a
// whole phase's loads above the arithmetic of the previous one, which costs more
// live registers than the latency it hides.
#if defined(__HIP_DEVICE_COMPILE__)
#define VI_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#else
#define VI_SCHED_FENCE() ((void)0)
#endif

typedef uint64_t u64;
typedef uint32_t u32;
typedef int64_t i64;

namespace gl {

constexpr u64 P = 0xFFFFFFFF00000001ull;
constexpr u64 EPS = 0xFFFFFFFFull;   // 2^32 - 1 = 2^64 mod p

VI_HD u64 add(u64 a, u64 b) {
    u64 s = a + b;
    if (s < a) s += EPS;             // wrapped past 2^64: add 2^64 mod p
    if (s >= P) s -= P;
    return s;
}

VI_HD u64 sub(u64 a, u64 b) {
    u64 d = a - b;
    if (a < b) d -= EPS;             // borrowed 2^64: take 2^64 mod p back out
    return d;
}

VI_HD u64 neg(u64 a) { return a == 0 ? 0 : P - a; }

// Sum of two CANONICAL values (cheaper than add(): the wrap past 2^64 and the
// overshoot past p take the same correction, + (2^32 - 1) mod 2^64, so one select
// serves both).  Not for arbitrary words: with both operands >= p it can be wrong.
VI_HD u64 addc(u64 a, u64 b) {
    u64 s = a + b;
    u64 r = s + EPS;
    return ((s < a) | (r < s)) ? r : s;
}

// x mod p for an arbitrary 64-bit word
VI_HD u64 canon(u64 x) {
    u64 r = x + EPS;
    return (r < x) ? r : x;
}

// (hi:lo) -> [0, p).  hi = hh*2^32 + hl  =>  value = lo - hh + hl*(2^32 - 1).
VI_HD u64 reduce128(u64 lo, u64 hi) {
    u32 hh = (u32)(hi >> 32), hl = (u32)hi;
    u64 t0 = lo - hh;
    if (lo < hh) t0 -= EPS;
    u64 t1 = ((u64)hl << 32) - hl;   // hl * (2^32 - 1), no multiplier needed
    u64 r = t0 + t1;
    if (r < t0) r += EPS;
    if (r >= P) r -= P;
    return r;
}

// (hi:lo) -> some 64-bit word congruent to it (not necessarily below p): reduce128 without
// its last conditional subtraction.  Good enough as an operand of mul / mul_wide.
VI_HD u64 reduce128_lazy(u64 lo, u64 hi) {
    u32 hh = (u32)(hi >> 32), hl = (u32)hi;
    u64 t0 = lo - hh;
    if (lo < hh) t0 -= EPS;
    u64 t1 = ((u64)hl << 32) - hl;
    u64 r = t0 + t1;
    if (r < t0) r += EPS;
    return r;
}

// 64x64 -> 128 from 32-bit halves; every line is one v_mad_u64_u32 (the addends
// cannot overflow: (2^32-1)^2 + 2*(2^32-1) < 2^64).
VI_HD void mul_wide(u64 a, u64 b, u64 &lo, u64 &hi) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u64 p00 = (u64)a0 * b0;
    u64 p01 = (u64)a0 * b1 + (p00 >> 32);
    u64 p10 = (u64)a1 * b0 + (u32)p01;
    u64 p11 = (u64)a1 * b1 + (p01 >> 32) + (p10 >> 32);
    lo = (p10 << 32) | (u32)p00;
    hi = p11;
}

VI_HD u64 mul(u64 a, u64 b) {
    u64 lo, hi;
    mul_wide(a, b, lo, hi);
    return reduce128(lo, hi);
}

// product as a non-canonical word (see reduce128_lazy): for chains of multiplications
VI_HD u64 mul_lazy(u64 a, u64 b) {
    u64 lo, hi;
    mul_wide(a, b, lo, hi);
    return reduce128_lazy(lo, hi);
}

VI_HD u64 pow(u64 base, u64 e) {
    u64 r = 1;
    while (e) {
        if (e & 1) r = mul(r, base);
        base = mul(base, base);
        e >>= 1;
    }
    return r;
}

VI_HD u64 sqr_n(u64 x, int n) {
    for (int i = 0; i < n; ++i) x = mul(x, x);
    return x;
}

// x^(p-2) by a fixed addition chain: p - 2 = (2^31 - 1) * 2^33 + (2^32 - 1), and x^(2^k - 1)
// doubles its k with k squarings and one product.  64 squarings + 10 products instead of the
// 63 + 62 of square-and-multiply; 0 -> 0 like the Fermat power.
VI_HD u64 inv(u64 x) {
    u64 a2 = mul(sqr_n(x, 1), x);            // 2^2 - 1
    u64 a4 = mul(sqr_n(a2, 2), a2);
    u64 a8 = mul(sqr_n(a4, 4), a4);
    u64 a16 = mul(sqr_n(a8, 8), a8);
    u64 a24 = mul(sqr_n(a16, 8), a8);
    u64 a28 = mul(sqr_n(a24, 4), a4);
    u64 a30 = mul(sqr_n(a28, 2), a2);
    u64 a31 = mul(sqr_n(a30, 1), x);         // 2^31 - 1
    u64 a32 = mul(sqr_n(a31, 1), x);         // 2^32 - 1
    return mul(sqr_n(a31, 33), a32);
}

// canonical x times 2^s for 0 <= s < 96, as shifts: the 64-bit value moved left by
// s bits occupies at most three 32-bit limbs L[q..q+2] (s = 32q + r) of
//   L0 + L1*phi + L2*phi^2 + L3*phi^3 + L4*phi^4,  phi = 2^32,
// and phi^2 = phi - 1, phi^3 = -1, phi^4 = -phi fold it back to two limbs.
VI_HD u64 mul_pow2(u64 x, u32 s) {
    u32 q = s >> 5, r = s & 31;
    u32 x0 = (u32)x, x1 = (u32)(x >> 32);
    u32 m0 = x0 << r;
    u32 m1 = r ? ((x1 << r) | (x0 >> (32 - r))) : x1;
    u32 m2 = r ? (x1 >> (32 - r)) : 0;
    if (q == 0) return reduce128(((u64)m1 << 32) | m0, (u64)m2);            // m0 + m1 phi + m2 phi^2
    if (q == 1) return reduce128((u64)m0 << 32, ((u64)m2 << 32) | m1);      // m0 phi + m1 phi^2 + m2 phi^3
    // q == 2: m0 phi^2 + m1 phi^3 + m2 phi^4 = (m0 - m2) phi - (m0 + m1)
    u64 pos = (u64)m0 << 32;                       // m0 * phi            < p
    u64 negv = (u64)m2 << 32;                      // m2 * phi            < p
    u64 small = (u64)m0 + (u64)m1;                 // < 2^33              < p
    return sub(sub(pos, negv), small);
}

}  // namespace gl

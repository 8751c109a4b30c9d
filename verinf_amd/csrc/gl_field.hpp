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

#include <type_traits>

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

#if defined(__HIP_DEVICE_COMPILE__)
// Hand-scheduled gfx950 sequences.  Written from 64-bit C++ the compiler spends a 64-bit compare (two issue
// slots) and two selects on every carry test and builds register pairs with moves: 29 VALU instructions (42
// issue slots) for a product, 7 (11) for a modular sum.  On 32-bit halves with explicit carries the same
// functions are 19 (24), 6 and 5.  On this chip a VALU instruction that reads a carry or mask needs two
// wait states after the VALU instruction that wrote it; inside an asm block the assembler does not add
// them, so every such pair below is separated by two instructions or an s_nop.  s_or_b64 also writes SCC, which the
// compiler may be holding a loop condition in: the blocks that use it say so in their clobber lists.  A carry that leaves a
// block in an SGPR pair is only read by a scalar instruction, or by a vector instruction at least two
// instructions into the next block.
namespace dev {

__device__ __forceinline__ u64 pack(u32 lo, u32 hi) { return ((u64)hi << 32) | lo; }

// w, plus 2^64 when the carry `cin` is set, lies in [0, 2p): subtract p when it is >= p.
// r = w + (2^32 - 1) mod 2^64 is that difference, and it is the answer exactly when one of the two additions wrapped.
__device__ __forceinline__ u64 canon_tail(u32 w0, u32 w1, u64 cin) {
    u32 r0, r1;
    asm("v_add_co_u32 %[r0], vcc, -1, %[w0]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[r1], vcc, 0, %[w1], vcc\n\t"
        "s_or_b64 vcc, vcc, %[cin]\n\t"
        "v_cndmask_b32 %[r0], %[w0], %[r0], vcc\n\t"
        "v_cndmask_b32 %[r1], %[w1], %[r1], vcc"
        : [r0] "=&v"(r0), [r1] "=&v"(r1)
        : [w0] "v"(w0), [w1] "v"(w1), [cin] "s"(cin)
        : "vcc", "scc");
    return pack(r0, r1);
}

__device__ __forceinline__ u64 addc(u64 a, u64 b) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u32 s0, s1, r0, r1;
    u64 st;
    asm("v_add_co_u32 %[s0], vcc, %[a0], %[b0]\n\t"
        "v_add_co_u32 %[r0], %[st], -1, %[s0]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32 %[s1], vcc, %[a1], %[b1], vcc\n\t"
        "v_addc_co_u32 %[r1], %[st], 0, %[s1], %[st]\n\t"
        "s_or_b64 vcc, vcc, %[st]\n\t"
        "v_cndmask_b32 %[r0], %[s0], %[r0], vcc\n\t"
        "v_cndmask_b32 %[r1], %[s1], %[r1], vcc"
        : [s0] "=&v"(s0), [s1] "=&v"(s1), [r0] "=&v"(r0), [r1] "=&v"(r1), [st] "=&s"(st)
        : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1)
        : "vcc", "scc");
    return pack(r0, r1);
}

// a - b, minus 2^32 - 1 more when it borrowed (the mask -borrow is that constant)
__device__ __forceinline__ u64 sub(u64 a, u64 b) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u32 d0, d1, m;
    asm("v_sub_co_u32 %[d0], vcc, %[a0], %[b0]\n\t"
        "s_nop 1\n\t"
        "v_subb_co_u32 %[d1], vcc, %[a1], %[b1], vcc\n\t"
        "s_nop 1\n\t"
        "v_subb_co_u32 %[m], vcc, %[d0], %[d0], vcc\n\t"
        "v_sub_co_u32 %[d0], vcc, %[d0], %[m]\n\t"
        "s_nop 1\n\t"
        "v_subbrev_co_u32 %[d1], vcc, 0, %[d1], vcc"
        : [d0] "=&v"(d0), [d1] "=&v"(d1), [m] "=&v"(m)
        : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1)
        : "vcc");
    return pack(d0, d1);
}

// (u + v, u - v) of canonical u, v in one block: the two carry chains are interleaved so that each carry is read
// three instructions after it was written and no wait has to be inserted
__device__ __forceinline__ void bfly(u64 u, u64 v, u64 &sum, u64 &dif) {
    u32 u0 = (u32)u, u1 = (u32)(u >> 32), v0 = (u32)v, v1 = (u32)(v >> 32);
    u32 s0, s1, r0, r1, d0, d1, m;
    u64 st, sb;
    asm("v_add_co_u32 %[s0], vcc, %[u0], %[v0]\n\t"
        "v_sub_co_u32 %[d0], %[sb], %[u0], %[v0]\n\t"
        "v_add_co_u32 %[r0], %[st], -1, %[s0]\n\t"
        "v_addc_co_u32 %[s1], vcc, %[u1], %[v1], vcc\n\t"
        "v_subb_co_u32 %[d1], %[sb], %[u1], %[v1], %[sb]\n\t"
        "v_addc_co_u32 %[r1], %[st], 0, %[s1], %[st]\n\t"
        "s_or_b64 vcc, vcc, %[st]\n\t"
        "v_subb_co_u32 %[m], %[sb], %[d0], %[d0], %[sb]\n\t"
        "v_sub_co_u32 %[d0], %[sb], %[d0], %[m]\n\t"
        "v_cndmask_b32 %[r0], %[s0], %[r0], vcc\n\t"
        "v_cndmask_b32 %[r1], %[s1], %[r1], vcc\n\t"
        "v_subbrev_co_u32 %[d1], %[sb], 0, %[d1], %[sb]"
        : [s0] "=&v"(s0), [s1] "=&v"(s1), [r0] "=&v"(r0), [r1] "=&v"(r1), [d0] "=&v"(d0), [d1] "=&v"(d1), [m] "=&v"(m),
          [st] "=&s"(st), [sb] "=&s"(sb)
        : [u0] "v"(u0), [u1] "v"(u1), [v0] "v"(v0), [v1] "v"(v1)
        : "vcc", "scc");
    sum = pack(r0, r1);
    dif = pack(d0, d1);
}

__device__ __forceinline__ u64 canon(u64 x) {
    u32 x0 = (u32)x, x1 = (u32)(x >> 32), r0, r1;
    asm("v_add_co_u32 %[r0], vcc, -1, %[x0]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[r1], vcc, 0, %[x1], vcc\n\t"
        "s_nop 1\n\t"
        "v_cndmask_b32 %[r0], %[x0], %[r0], vcc\n\t"
        "v_cndmask_b32 %[r1], %[x1], %[r1], vcc"
        : [r0] "=&v"(r0), [r1] "=&v"(r1)
        : [x0] "v"(x0), [x1] "v"(x1)
        : "vcc");
    return pack(r0, r1);
}

// (hi:lo) given as four words l0 l1 hl hh, minus the borrow-in `bin` -> [0, p):  lo - hh - bin + hl (2^32 - 1).
// hh + bin must be below 2^32.
__device__ __forceinline__ u64 reduce_words(u32 l0, u32 l1, u32 hl, u32 hh, u64 bin) {
    u32 x0, x1, m;
    asm("v_subb_co_u32 %[x0], vcc, %[l0], %[hh], %[bin]\n\t"
        "s_nop 1\n\t"
        "v_subbrev_co_u32 %[x1], vcc, 0, %[l1], vcc\n\t"
        "s_nop 1\n\t"
        "v_subb_co_u32 %[m], vcc, %[x0], %[x0], vcc\n\t"
        "v_sub_co_u32 %[x0], vcc, %[x0], %[m]\n\t"
        "s_nop 1\n\t"
        "v_subbrev_co_u32 %[x1], vcc, 0, %[x1], vcc"
        : [x0] "=&v"(x0), [x1] "=&v"(x1), [m] "=&v"(m)
        : [l0] "v"(l0), [l1] "v"(l1), [hh] "v"(hh), [bin] "s"(bin)
        : "vcc");
    u64 w, st;
    asm("v_mad_u64_u32 %[w], %[st], %[hl], -1, %[x]"
        : [w] "=&v"(w), [st] "=&s"(st)
        : [hl] "v"(hl), [x] "v"(pack(x0, x1)));
    return canon_tail((u32)w, (u32)(w >> 32), st);
}

__device__ __forceinline__ u64 mul(u64 a, u64 b) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u64 p00, mm, p11, st;
    asm("v_mad_u64_u32 %[p00], vcc, %[a0], %[b0], 0\n\t"
        "v_mad_u64_u32 %[mm], vcc, %[a1], %[b0], 0\n\t"
        "v_mad_u64_u32 %[p11], vcc, %[a1], %[b1], 0\n\t"
        "v_mad_u64_u32 %[mm], %[st], %[a0], %[b1], %[mm]"
        : [p00] "=&v"(p00), [mm] "=&v"(mm), [p11] "=&v"(p11), [st] "=&s"(st)
        : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1)
        : "vcc");
    // words of the 128-bit product: p00.lo, p00.hi + mm.lo, p11.lo + mm.hi + carry, p11.hi + carry.  The carry of the
    // cross sum (in st) weighs 2^96 = -1: it goes into the reduction as a borrow.
    u32 w1 = (u32)(p00 >> 32), hl, hh;
    asm("v_add_co_u32 %[w1], vcc, %[w1], %[m0]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[hl], vcc, %[q0], %[m1], vcc\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[hh], vcc, 0, %[q1], vcc"
        : [w1] "+v"(w1), [hl] "=&v"(hl), [hh] "=&v"(hh)
        : [m0] "v"((u32)mm), [m1] "v"((u32)(mm >> 32)), [q0] "v"((u32)p11), [q1] "v"((u32)(p11 >> 32))
        : "vcc");
    return reduce_words((u32)p00, w1, hl, hh, st);
}

// the reduction of reduce_words() without its last step: a 64-bit word congruent to the value, not necessarily
// below p (three instructions instead of six after the multiply-add); good as an operand of a further product
__device__ __forceinline__ u64 reduce_words_lazy(u32 l0, u32 l1, u32 hl, u32 hh, u64 bin) {
    u32 x0, x1, m;
    asm("v_subb_co_u32 %[x0], vcc, %[l0], %[hh], %[bin]\n\t"
        "s_nop 1\n\t"
        "v_subbrev_co_u32 %[x1], vcc, 0, %[l1], vcc\n\t"
        "s_nop 1\n\t"
        "v_subb_co_u32 %[m], vcc, %[x0], %[x0], vcc\n\t"
        "v_sub_co_u32 %[x0], vcc, %[x0], %[m]\n\t"
        "s_nop 1\n\t"
        "v_subbrev_co_u32 %[x1], vcc, 0, %[x1], vcc"
        : [x0] "=&v"(x0), [x1] "=&v"(x1), [m] "=&v"(m)
        : [l0] "v"(l0), [l1] "v"(l1), [hh] "v"(hh), [bin] "s"(bin)
        : "vcc");
    u64 w, st;
    asm("v_mad_u64_u32 %[w], %[st], %[hl], -1, %[x]"
        : [w] "=&v"(w), [st] "=&s"(st)
        : [hl] "v"(hl), [x] "v"(pack(x0, x1)));
    // the sum wrapped past 2^64 (st): add 2^64 mod p = 2^32 - 1; it cannot wrap again (w <= 2^64 - 2^33 then)
    u32 w0 = (u32)w, w1 = (u32)(w >> 32), e;
    asm("s_nop 1\n\t"
        "v_cndmask_b32 %[e], 0, -1, %[st]\n\t"
        "v_add_co_u32 %[w0], vcc, %[w0], %[e]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[w1], vcc, 0, %[w1], vcc"
        : [e] "=&v"(e), [w0] "+v"(w0), [w1] "+v"(w1)
        : [st] "s"(st)
        : "vcc");
    return pack(w0, w1);
}

// the four partial products of a * b (+ c, a 64-bit addend of the lowest one) as the words l0 l1 hl hh of the
// 128-bit result; *st receives the carry of the cross sum, which weighs 2^96 = -1 and goes into the reduction as a
// borrow
template <bool ADD>
__device__ __forceinline__ void mul_words(u64 a, u64 b, u64 c, u32 &l0, u32 &l1, u32 &hl, u32 &hh, u64 &st) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u64 p00, mm, p11, cy = 0;
    if (ADD) {
        asm("v_mad_u64_u32 %[p00], %[cy], %[a0], %[b0], %[c]\n\t"
            "v_mad_u64_u32 %[mm], vcc, %[a1], %[b0], 0\n\t"
            "v_mad_u64_u32 %[p11], vcc, %[a1], %[b1], 0\n\t"
            "v_mad_u64_u32 %[mm], %[st], %[a0], %[b1], %[mm]"
            : [p00] "=&v"(p00), [mm] "=&v"(mm), [p11] "=&v"(p11), [st] "=&s"(st), [cy] "=&s"(cy)
            : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1), [c] "v"(c)
            : "vcc");
    } else {
        asm("v_mad_u64_u32 %[p00], vcc, %[a0], %[b0], 0\n\t"
            "v_mad_u64_u32 %[mm], vcc, %[a1], %[b0], 0\n\t"
            "v_mad_u64_u32 %[p11], vcc, %[a1], %[b1], 0\n\t"
            "v_mad_u64_u32 %[mm], %[st], %[a0], %[b1], %[mm]"
            : [p00] "=&v"(p00), [mm] "=&v"(mm), [p11] "=&v"(p11), [st] "=&s"(st)
            : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1)
            : "vcc");
    }
    u32 q0 = (u32)p11, q1 = (u32)(p11 >> 32);
    if (ADD) {
        // the carry of the lowest product plus c weighs 2^64: into a1 b1 <= (2^32 - 1)^2, which cannot overflow
        asm("v_addc_co_u32 %[q0], vcc, 0, %[q0], %[cy]\n\t"
            "s_nop 1\n\t"
            "v_addc_co_u32 %[q1], vcc, 0, %[q1], vcc"
            : [q0] "+v"(q0), [q1] "+v"(q1)
            : [cy] "s"(cy)
            : "vcc");
    }
    u32 w1 = (u32)(p00 >> 32);
    asm("v_add_co_u32 %[w1], vcc, %[w1], %[m0]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[hl], vcc, %[q0], %[m1], vcc\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[hh], vcc, 0, %[q1], vcc"
        : [w1] "+v"(w1), [hl] "=&v"(hl), [hh] "=&v"(hh)
        : [m0] "v"((u32)mm), [m1] "v"((u32)(mm >> 32)), [q0] "v"(q0), [q1] "v"(q1)
        : "vcc");
    l0 = (u32)p00;
    l1 = w1;
}

// a * b + c -> [0, p): the addend rides on the first partial product (20 instructions against 24 for mul + add)
__device__ __forceinline__ u64 mul_add(u64 a, u64 b, u64 c) {
    u32 l0, l1, hl, hh;
    u64 st;
    mul_words<true>(a, b, c, l0, l1, hl, hh, st);
    return reduce_words(l0, l1, hl, hh, st);
}

// a * b + c as a 64-bit word congruent to it, not necessarily below p
__device__ __forceinline__ u64 mul_add_lazy(u64 a, u64 b, u64 c) {
    u32 l0, l1, hl, hh;
    u64 st;
    mul_words<true>(a, b, c, l0, l1, hl, hh, st);
    return reduce_words_lazy(l0, l1, hl, hh, st);
}

// a * b as a 64-bit word congruent to the product, not necessarily below p
__device__ __forceinline__ u64 mul_lazy(u64 a, u64 b) {
    u32 l0, l1, hl, hh;
    u64 st;
    mul_words<false>(a, b, 0, l0, l1, hl, hh, st);
    return reduce_words_lazy(l0, l1, hl, hh, st);
}

// five words w[0..4] (an integer below 2^160) += a * b, the full 128-bit product, nothing reduced: 13 instructions
// against the 24 of a product reduced to [0, p) followed by a modular addition.  The two carry chains (the words
// of the product, the words of the sum) are interleaved so that each carry is read two slots after it was written.
__device__ __forceinline__ void mul_acc(u32 (&w)[5], u64 a, u64 b) {
    u32 a0 = (u32)a, a1 = (u32)(a >> 32), b0 = (u32)b, b1 = (u32)(b >> 32);
    u64 p00, mm, p11, st;
    asm("v_mad_u64_u32 %[p00], vcc, %[a0], %[b0], 0\n\t"
        "v_mad_u64_u32 %[mm], vcc, %[a1], %[b0], 0\n\t"
        "v_mad_u64_u32 %[p11], vcc, %[a1], %[b1], 0\n\t"
        "v_mad_u64_u32 %[mm], %[st], %[a0], %[b1], %[mm]"
        : [p00] "=&v"(p00), [mm] "=&v"(mm), [p11] "=&v"(p11), [st] "=&s"(st)
        : [a0] "v"(a0), [a1] "v"(a1), [b0] "v"(b0), [b1] "v"(b1)
        : "vcc");
    // product words: p00.lo | p00.hi + mm.lo | p11.lo + mm.hi + carry | p11.hi + carry + st (st = carry of the cross
    // sum; the product is below 2^128, so the top word cannot overflow)
    u32 w1 = (u32)(p00 >> 32), hl, hh;
    u64 cb;
    asm("v_add_co_u32 %[w1], vcc, %[w1], %[m0]\n\t"
        "v_add_co_u32 %[A0], %[cb], %[A0], %[w0]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32 %[hl], vcc, %[q0], %[m1], vcc\n\t"
        "v_addc_co_u32 %[A1], %[cb], %[A1], %[w1], %[cb]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32 %[hh], vcc, 0, %[q1], vcc\n\t"
        "v_addc_co_u32 %[A2], %[cb], %[A2], %[hl], %[cb]\n\t"
        "s_nop 0\n\t"
        "v_addc_co_u32 %[hh], vcc, 0, %[hh], %[st]\n\t"
        "v_addc_co_u32 %[A3], %[cb], %[A3], %[hh], %[cb]\n\t"
        "s_nop 1\n\t"
        "v_addc_co_u32 %[A4], %[cb], 0, %[A4], %[cb]"
        : [w1] "+v"(w1), [hl] "=&v"(hl), [hh] "=&v"(hh), [cb] "=&s"(cb), [A0] "+v"(w[0]), [A1] "+v"(w[1]),
          [A2] "+v"(w[2]), [A3] "+v"(w[3]), [A4] "+v"(w[4])
        : [w0] "v"((u32)p00), [m0] "v"((u32)mm), [m1] "v"((u32)(mm >> 32)), [q0] "v"((u32)p11),
          [q1] "v"((u32)(p11 >> 32)), [st] "s"(st)
        : "vcc");
}

// canonical v times 2^E, 0 <= E < 96, canonical result; s = 32 q + r moves v into limbs m0 m1 m2 at phi^q
// PIN: the three shifts as one asm block.  Plain shifts of a loop-invariant value are hoisted out of a loop even from
// a branch that is not always taken (they are safe to speculate), and then stay live in registers across it; an asm
// block stays where it is written.
// NEG: minus the product, i.e. v times 2^(E + 96); for E >= 32 the last step is a subtraction whose operands swap, so
// the sign is free.
template <int E, bool PIN = false, bool NEG = false>
__device__ __forceinline__ u64 mul_pow2(u64 v) {
    static_assert(E >= 0 && E < 96, "shift out of range");
    if (E == 0) return NEG ? sub(0, v) : v;
    constexpr int q = E >> 5, r = E & 31;
    const u32 v0 = (u32)v, v1 = (u32)(v >> 32);
    u32 m0, m1, m2;
    if constexpr (PIN && r != 0) {
        asm("v_lshlrev_b32 %[m0], %[r], %[v0]\n\t"
            "v_alignbit_b32 %[m1], %[v1], %[v0], %[c]\n\t"
            "v_lshrrev_b32 %[m2], %[c], %[v1]"
            : [m0] "=&v"(m0), [m1] "=&v"(m1), [m2] "=&v"(m2)
            : [v0] "v"(v0), [v1] "v"(v1), [r] "n"(r), [c] "n"(32 - r));
    } else {
        m0 = v0 << r;
        m1 = r ? __builtin_amdgcn_alignbit(v1, v0, (32 - r) & 31) : v1;
        m2 = r ? (v1 >> ((32 - r) & 31)) : 0u;
    }
    if (q == 0) {
        // m0 + m1 phi + m2 phi^2 = (m1:m0) + m2 (2^32 - 1)
        u64 w, st;
        asm("v_mad_u64_u32 %[w], %[st], %[m2], -1, %[x]"
            : [w] "=&v"(w), [st] "=&s"(st)
            : [m2] "v"(m2), [x] "v"(pack(m0, m1)));
        const u64 x = canon_tail((u32)w, (u32)(w >> 32), st);
        return NEG ? sub(0, x) : x;
    } else if (q == 1) {
        // m0 phi + m1 phi^2 + m2 phi^3 = (m0:0) + m1 (2^32 - 1) - m2
        u64 w, st;
        asm("v_mad_u64_u32 %[w], %[st], %[m1], -1, %[x]"
            : [w] "=&v"(w), [st] "=&s"(st)
            : [m1] "v"(m1), [x] "v"(pack(0u, m0)));
        const u64 x = canon_tail((u32)w, (u32)(w >> 32), st);
        if (NEG) return sub((u64)m2, x);                   // m2 = 0 when r = 0
        return r ? sub(x, (u64)m2) : x;
    } else {
        // m0 phi^2 + m1 phi^3 + m2 phi^4 = m0 (2^32 - 1) - (m2:m1); both operands are below p
        u32 e0, e1;
        asm("v_sub_co_u32 %[e0], vcc, 0, %[m0]\n\t"
            "s_nop 1\n\t"
            "v_subbrev_co_u32 %[e1], vcc, 0, %[m0], vcc"
            : [e0] "=&v"(e0), [e1] "=&v"(e1)
            : [m0] "v"(m0)
            : "vcc");
        return NEG ? sub(pack(m1, m2), pack(e0, e1)) : sub(pack(e0, e1), pack(m1, m2));
    }
}

}  // namespace dev
#endif

VI_HD u64 add(u64 a, u64 b) {
    u64 s = a + b;
    if (s < a) s += EPS;             // wrapped past 2^64: add 2^64 mod p
    if (s >= P) s -= P;
    return s;
}

VI_HD u64 sub(u64 a, u64 b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::sub(a, b);
#endif
    u64 d = a - b;
    if (a < b) d -= EPS;             // borrowed 2^64: take 2^64 mod p back out
    return d;
}

VI_HD u64 neg(u64 a) { return a == 0 ? 0 : P - a; }

// Sum of two CANONICAL values (cheaper than add(): the wrap past 2^64 and the
// overshoot past p take the same correction, + (2^32 - 1) mod 2^64, so one select
// serves both).  Not for arbitrary words: with both operands >= p it can be wrong.
VI_HD u64 addc(u64 a, u64 b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::addc(a, b);
#endif
    u64 s = a + b;
    u64 r = s + EPS;
    return ((s < a) | (r < s)) ? r : s;
}

// (u + v, u - v) for canonical u, v
VI_HD void bfly(u64 u, u64 v, u64 &sum, u64 &dif) {
#if defined(__HIP_DEVICE_COMPILE__)
    dev::bfly(u, v, sum, dif);
#else
    sum = addc(u, v);
    dif = sub(u, v);
#endif
}

// x mod p for an arbitrary 64-bit word
VI_HD u64 canon(u64 x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::canon(x);
#endif
    u64 r = x + EPS;
    return (r < x) ? r : x;
}

// (hi:lo) -> [0, p).  hi = hh*2^32 + hl  =>  value = lo - hh + hl*(2^32 - 1).
VI_HD u64 reduce128(u64 lo, u64 hi) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::reduce_words((u32)lo, (u32)(lo >> 32), (u32)hi, (u32)(hi >> 32), 0);
#endif
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
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::mul(a, b);
#endif
    u64 lo, hi;
    mul_wide(a, b, lo, hi);
    return reduce128(lo, hi);
}

// a * b + c in [0, p) for any words a, b, c
VI_HD u64 mul_add(u64 a, u64 b, u64 c) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::mul_add(a, b, c);
#endif
    return add(mul(a, b), canon(c));
}

// a * b + c as a word congruent to it, not necessarily below p
VI_HD u64 mul_add_lazy(u64 a, u64 b, u64 c) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::mul_add_lazy(a, b, c);
#endif
    return mul_add(a, b, c);
}

// product as a non-canonical word (see reduce128_lazy): for chains of multiplications
VI_HD u64 mul_lazy(u64 a, u64 b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::mul_lazy(a, b);
#endif
    u64 lo, hi;
    mul_wide(a, b, lo, hi);
    return reduce128_lazy(lo, hi);
}

// Sums of products kept as plain integers: five 32-bit words, reduced once at the end.
struct Wide {
    u32 w[5];
};
VI_HD void wide_zero(Wide &A) {
    for (int i = 0; i < 5; ++i) A.w[i] = 0;
}
// A += a * b (any 64-bit words); the caller keeps the number of products below 2^32
VI_HD void wide_mul_acc(Wide &A, u64 a, u64 b) {
#if defined(__HIP_DEVICE_COMPILE__)
    dev::mul_acc(A.w, a, b);
#else
    u64 lo, hi;
    mul_wide(a, b, lo, hi);
    const u64 add[4] = {(u32)lo, lo >> 32, (u32)hi, hi >> 32};
    u64 carry = 0;
    for (int i = 0; i < 5; ++i) {
        const u64 t = (u64)A.w[i] + (i < 4 ? add[i] : 0) + carry;
        A.w[i] = (u32)t;
        carry = t >> 32;
    }
#endif
}
// the integer mod p: words 0..3 as a 128-bit value, word 4 weighs 2^128 = -2^32
VI_HD u64 wide_reduce(const Wide &A) {
    const u64 x = reduce128(((u64)A.w[1] << 32) | A.w[0], ((u64)A.w[3] << 32) | A.w[2]);
    return sub(x, (u64)A.w[4] << 32);
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

// the same with the exponent fixed at compile time
template <int E>
VI_HD u64 mul_pow2c(u64 x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return dev::mul_pow2<E>(x);
#else
    return mul_pow2(x, (u32)E);
#endif
}

// x times 2^E for any exponent (2^192 = 1, 2^96 = -1), for use inside a branch of a loop on a value the loop does
// not change (see dev::mul_pow2)
template <int E>
VI_HD u64 mul_pow2c_pinned(u64 x) {
    constexpr int e = ((E % 192) + 192) % 192;
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (e < 96) return dev::mul_pow2<e, true, false>(x);
    else return dev::mul_pow2<e - 96, true, true>(x);
#else
    return e < 96 ? mul_pow2(x, (u32)e) : sub(0, mul_pow2(x, (u32)(e - 96)));
#endif
}

}  // namespace gl

// compile-time loop: f(std::integral_constant<int, I>) for I in [I0, N)
template <int I0, int N, class F>
VI_HD void static_for(F &&f) {
    if constexpr (I0 < N) {
        f(std::integral_constant<int, I0>{});
        static_for<I0 + 1, N>(f);
    }
}

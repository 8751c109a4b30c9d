// Issue-rate probe for the integer VALU instructions the field arithmetic is made of.
//
// Measurement hook, no counterpart in the reference: the transforms and the hashing of this library are bound
// by how fast a SIMD issues 32-bit integer instructions, so the figure they are put against -- wave-instructions
// per second of the whole chip, per instruction class -- is measured here rather than assumed.  A kernel of a
// class runs `iters` times a block of 256 instructions of that class on four independent register chains
// (dependent instructions are four apart, beyond the pipeline depth), on every SIMD of the chip at eight
// wavefronts each; thread 0 of every workgroup also reads the shader clock counter and the constant 100 MHz
// counter before and after, which gives the clock the SIMDs actually ran at during the loop.
#include "common.hpp"

namespace {

#define VI_REP4(...) __VA_ARGS__ __VA_ARGS__ __VA_ARGS__ __VA_ARGS__
#define VI_REP16(...) VI_REP4(VI_REP4(__VA_ARGS__))
#define VI_REP64(...) VI_REP4(VI_REP16(__VA_ARGS__))

// out[0 .. blocks*256): a value that depends on every chain (keeps the loop alive);
// clocks[4b .. 4b+3]: shader-clock ticks and 100 MHz ticks at the start and the end of workgroup b
#define VI_PROBE_KERNEL(name, ...)                                                                        \
    __global__ __launch_bounds__(256) void name(uint64_t *out, uint64_t *clocks, int iters) {             \
        uint32_t a0 = threadIdx.x, a1 = a0 + 1, a2 = a0 + 2, a3 = a0 + 3;                                  \
        uint64_t d0 = a0, d1 = a1, d2 = a2, d3 = a3;                                                       \
        uint64_t c0 = 0, t0 = 0;                                                                           \
        if (threadIdx.x == 0) { c0 = __builtin_readcyclecounter(); t0 = wall_clock64(); }                  \
        for (int i = 0; i < iters; ++i) { VI_REP64(__VA_ARGS__) }                                          \
        if (threadIdx.x == 0) {                                                                            \
            clocks[4 * blockIdx.x + 0] = c0;                                                               \
            clocks[4 * blockIdx.x + 1] = __builtin_readcyclecounter();                                     \
            clocks[4 * blockIdx.x + 2] = t0;                                                               \
            clocks[4 * blockIdx.x + 3] = wall_clock64();                                                   \
        }                                                                                                  \
        out[(size_t)blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + d0 + d1 + d2 + d3;               \
    }

#define VI_A32 "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
#define VI_D64 "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3)

VI_PROBE_KERNEL(k_add_u32, asm volatile("v_add_u32 %0, %0, %1\n v_add_u32 %1, %1, %2\n v_add_u32 %2, %2, %3\n v_add_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_add_co, asm volatile("v_add_co_u32 %0, vcc, %0, %1\n v_add_co_u32 %1, vcc, %1, %2\n v_add_co_u32 %2, vcc, %2, %3\n v_add_co_u32 %3, vcc, %3, %0" : VI_A32 : : "vcc");)
VI_PROBE_KERNEL(k_addc_co, asm volatile("v_addc_co_u32 %0, vcc, %0, %1, vcc\n v_addc_co_u32 %1, vcc, %1, %2, vcc\n v_addc_co_u32 %2, vcc, %2, %3, vcc\n v_addc_co_u32 %3, vcc, %3, %0, vcc" : VI_A32 : : "vcc");)
VI_PROBE_KERNEL(k_alignbit, asm volatile("v_alignbit_b32 %0, %0, %1, 7\n v_alignbit_b32 %1, %1, %2, 9\n v_alignbit_b32 %2, %2, %3, 11\n v_alignbit_b32 %3, %3, %0, 13" : VI_A32);)
VI_PROBE_KERNEL(k_add3, asm volatile("v_add3_u32 %0, %0, %1, %2\n v_add3_u32 %1, %1, %2, %3\n v_add3_u32 %2, %2, %3, %0\n v_add3_u32 %3, %3, %0, %1" : VI_A32);)
VI_PROBE_KERNEL(k_xor, asm volatile("v_xor_b32 %0, %0, %1\n v_xor_b32 %1, %1, %2\n v_xor_b32 %2, %2, %3\n v_xor_b32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_mul_lo, asm volatile("v_mul_lo_u32 %0, %0, %1\n v_mul_lo_u32 %1, %1, %2\n v_mul_lo_u32 %2, %2, %3\n v_mul_lo_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_mul_hi, asm volatile("v_mul_hi_u32 %0, %0, %1\n v_mul_hi_u32 %1, %1, %2\n v_mul_hi_u32 %2, %2, %3\n v_mul_hi_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_mad_u64_u32, asm volatile("v_mad_u64_u32 %0, s[10:11], %4, %5, %0\n v_mad_u64_u32 %1, s[10:11], %5, %6, %1\n v_mad_u64_u32 %2, s[10:11], %6, %7, %2\n v_mad_u64_u32 %3, s[10:11], %7, %4, %3" : VI_D64 : "v"(a0), "v"(a1), "v"(a2), "v"(a3) : "s10", "s11");)
VI_PROBE_KERNEL(k_lshl_add_u64, asm volatile("v_lshl_add_u64 %0, %0, 0, %1\n v_lshl_add_u64 %1, %1, 0, %2\n v_lshl_add_u64 %2, %2, 0, %3\n v_lshl_add_u64 %3, %3, 0, %0" : VI_D64);)
VI_PROBE_KERNEL(k_cmp_u64, asm volatile("v_cmp_lt_u64 vcc, %0, %1\n v_cmp_lt_u64 vcc, %1, %2\n v_cmp_lt_u64 vcc, %2, %3\n v_cmp_lt_u64 vcc, %3, %0" : VI_D64 : : "vcc");)
VI_PROBE_KERNEL(k_mul_u32_u24, asm volatile("v_mul_u32_u24 %0, %0, %1\n v_mul_u32_u24 %1, %1, %2\n v_mul_u32_u24 %2, %2, %3\n v_mul_u32_u24 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_fma_f64, asm volatile("v_fma_f64 %0, %0, %1, %2\n v_fma_f64 %1, %1, %2, %3\n v_fma_f64 %2, %2, %3, %0\n v_fma_f64 %3, %3, %0, %1" : VI_D64);)
// the canonical modular sum as the kernels issue it (six instructions and two scalar ones per element)
VI_PROBE_KERNEL(k_mod_add_seq, {
    uint32_t r0, r1;
    asm volatile("v_add_co_u32 %0, vcc, %0, %2\n v_add_co_u32 %4, s[10:11], -1, %0\n s_nop 0\n"
                 "v_addc_co_u32 %1, vcc, %1, %3, vcc\n v_addc_co_u32 %5, s[10:11], 0, %1, s[10:11]\n"
                 "s_or_b64 vcc, vcc, s[10:11]\n v_cndmask_b32 %0, %0, %4, vcc\n v_cndmask_b32 %1, %1, %5, vcc"
                 : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "=&v"(r0), "=&v"(r1) : : "vcc", "scc", "s10", "s11");
})

// more instruction classes
VI_PROBE_KERNEL(k_sub_u32, asm volatile("v_sub_u32 %0, %0, %1\n v_sub_u32 %1, %1, %2\n v_sub_u32 %2, %2, %3\n v_sub_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_and, asm volatile("v_and_b32 %0, %0, %1\n v_and_b32 %1, %1, %2\n v_and_b32 %2, %2, %3\n v_and_b32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_or, asm volatile("v_or_b32 %0, %0, %1\n v_or_b32 %1, %1, %2\n v_or_b32 %2, %2, %3\n v_or_b32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_lshl, asm volatile("v_lshlrev_b32 %0, 3, %0\n v_lshlrev_b32 %1, 5, %1\n v_lshlrev_b32 %2, 7, %2\n v_lshlrev_b32 %3, 9, %3" : VI_A32);)
VI_PROBE_KERNEL(k_lshr, asm volatile("v_lshrrev_b32 %0, 3, %0\n v_lshrrev_b32 %1, 5, %1\n v_lshrrev_b32 %2, 7, %2\n v_lshrrev_b32 %3, 9, %3" : VI_A32);)
VI_PROBE_KERNEL(k_mov, asm volatile("v_mov_b32 %0, %1\n v_mov_b32 %1, %2\n v_mov_b32 %2, %3\n v_mov_b32 %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_min, asm volatile("v_min_u32 %0, %0, %1\n v_min_u32 %1, %1, %2\n v_min_u32 %2, %2, %3\n v_min_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_cmp_u32, asm volatile("v_cmp_lt_u32 vcc, %0, %1\n v_cmp_lt_u32 vcc, %1, %2\n v_cmp_lt_u32 vcc, %2, %3\n v_cmp_lt_u32 vcc, %3, %0" : VI_A32 : : "vcc");)
VI_PROBE_KERNEL(k_lshl_b64, asm volatile("v_lshlrev_b64 %0, 3, %0\n v_lshlrev_b64 %1, 5, %1\n v_lshlrev_b64 %2, 7, %2\n v_lshlrev_b64 %3, 9, %3" : VI_D64);)
VI_PROBE_KERNEL(k_lshr_b64, asm volatile("v_lshrrev_b64 %0, 3, %0\n v_lshrrev_b64 %1, 5, %1\n v_lshrrev_b64 %2, 7, %2\n v_lshrrev_b64 %3, 9, %3" : VI_D64);)
VI_PROBE_KERNEL(k_subb_co, asm volatile("v_subb_co_u32 %0, vcc, %0, %1, vcc\n v_subb_co_u32 %1, vcc, %1, %2, vcc\n v_subb_co_u32 %2, vcc, %2, %3, vcc\n v_subb_co_u32 %3, vcc, %3, %0, vcc" : VI_A32 : : "vcc");)
VI_PROBE_KERNEL(k_bfe, asm volatile("v_bfe_u32 %0, %0, 3, 20\n v_bfe_u32 %1, %1, 5, 20\n v_bfe_u32 %2, %2, 7, 20\n v_bfe_u32 %3, %3, 9, 20" : VI_A32);)
VI_PROBE_KERNEL(k_lshl_or, asm volatile("v_lshl_or_b32 %0, %0, 3, %1\n v_lshl_or_b32 %1, %1, 5, %2\n v_lshl_or_b32 %2, %2, 7, %3\n v_lshl_or_b32 %3, %3, 9, %0" : VI_A32);)
VI_PROBE_KERNEL(k_perm, asm volatile("v_perm_b32 %0, %0, %1, %2\n v_perm_b32 %1, %1, %2, %3\n v_perm_b32 %2, %2, %3, %0\n v_perm_b32 %3, %3, %0, %1" : VI_A32);)
// how double-rate instructions behave next to others: a dependent chain, alternation with a full-rate class,
// and pairs of each class
VI_PROBE_KERNEL(k_xor_dependent, asm volatile("v_xor_b32 %0, %0, %1\n v_xor_b32 %0, %0, %2\n v_xor_b32 %0, %0, %3\n v_xor_b32 %0, %0, %1" : VI_A32);)
VI_PROBE_KERNEL(k_xor_align_alternating, asm volatile("v_xor_b32 %0, %0, %1\n v_alignbit_b32 %1, %1, %2, 7\n v_xor_b32 %2, %2, %3\n v_alignbit_b32 %3, %3, %0, 13" : VI_A32);)
VI_PROBE_KERNEL(k_xor_align_pairs, asm volatile("v_xor_b32 %0, %0, %1\n v_xor_b32 %1, %1, %2\n v_alignbit_b32 %2, %2, %3, 7\n v_alignbit_b32 %3, %3, %0, 13" : VI_A32);)
VI_PROBE_KERNEL(k_xor_add_alternating, asm volatile("v_xor_b32 %0, %0, %1\n v_add_u32 %1, %1, %2\n v_xor_b32 %2, %2, %3\n v_add_u32 %3, %3, %0" : VI_A32);)
VI_PROBE_KERNEL(k_xor_dep_pairs, asm volatile("v_xor_b32 %0, %0, %1\n v_xor_b32 %1, %0, %2\n v_xor_b32 %2, %1, %3\n v_xor_b32 %3, %2, %0" : VI_A32);)
// one BLAKE3 quarter-round step on four independent columns, as the compiler orders it (column by column) and
// regrouped by instruction (the four adds, then the four xors, ...)
VI_PROBE_KERNEL(k_g_by_column, asm volatile(
    "v_add3_u32 %0, %0, %1, %2\n v_xor_b32 %3, %3, %0\n v_alignbit_b32 %3, %3, %3, 16\n v_add_u32 %2, %2, %3\n v_xor_b32 %1, %1, %2\n v_alignbit_b32 %1, %1, %1, 12\n"
    "v_add3_u32 %4, %4, %5, %6\n v_xor_b32 %7, %7, %4\n v_alignbit_b32 %7, %7, %7, 16\n v_add_u32 %6, %6, %7\n v_xor_b32 %5, %5, %6\n v_alignbit_b32 %5, %5, %5, 12"
    : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(((uint32_t *)&d0)[0]), "+v"(((uint32_t *)&d0)[1]), "+v"(((uint32_t *)&d1)[0]), "+v"(((uint32_t *)&d1)[1]));)
VI_PROBE_KERNEL(k_g_by_instruction, asm volatile(
    "v_add3_u32 %0, %0, %1, %2\n v_add3_u32 %4, %4, %5, %6\n v_xor_b32 %3, %3, %0\n v_xor_b32 %7, %7, %4\n v_alignbit_b32 %3, %3, %3, 16\n v_alignbit_b32 %7, %7, %7, 16\n"
    "v_add_u32 %2, %2, %3\n v_add_u32 %6, %6, %7\n v_xor_b32 %1, %1, %2\n v_xor_b32 %5, %5, %6\n v_alignbit_b32 %1, %1, %1, 12\n v_alignbit_b32 %5, %5, %5, 12"
    : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(((uint32_t *)&d0)[0]), "+v"(((uint32_t *)&d0)[1]), "+v"(((uint32_t *)&d1)[0]), "+v"(((uint32_t *)&d1)[1]));)

// a whole G on four independent columns (48 instructions), sixteen times per loop trip
#define VI_W16 "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7]), "+v"(w[8]), "+v"(w[9]), "+v"(w[10]), "+v"(w[11]), "+v"(w[12]), "+v"(w[13]), "+v"(w[14]), "+v"(w[15])
__global__ __launch_bounds__(256) void k_g4_runs(uint64_t *out, uint64_t *clocks, int iters) {
    uint32_t w[16];
    for (int q = 0; q < 16; ++q) w[q] = threadIdx.x + q;
    uint64_t c0 = 0, t0 = 0;
    if (threadIdx.x == 0) { c0 = __builtin_readcyclecounter(); t0 = wall_clock64(); }
    for (int i = 0; i < iters; ++i) {
        VI_REP16(asm volatile("v_add3_u32 %0, %0, %4, %9\n v_add3_u32 %1, %1, %5, %10\n v_add3_u32 %2, %2, %6, %11\n v_add3_u32 %3, %3, %7, %8\n v_xor_b32 %12, %12, %0\n v_xor_b32 %13, %13, %1\n v_xor_b32 %14, %14, %2\n v_xor_b32 %15, %15, %3\n v_alignbit_b32 %12, %12, %12, 16\n v_alignbit_b32 %13, %13, %13, 16\n v_alignbit_b32 %14, %14, %14, 16\n v_alignbit_b32 %15, %15, %15, 16\n v_add_u32 %8, %8, %12\n v_add_u32 %9, %9, %13\n v_add_u32 %10, %10, %14\n v_add_u32 %11, %11, %15\n v_xor_b32 %4, %4, %8\n v_xor_b32 %5, %5, %9\n v_xor_b32 %6, %6, %10\n v_xor_b32 %7, %7, %11\n v_alignbit_b32 %4, %4, %4, 12\n v_alignbit_b32 %5, %5, %5, 12\n v_alignbit_b32 %6, %6, %6, 12\n v_alignbit_b32 %7, %7, %7, 12\n v_add3_u32 %0, %0, %4, %9\n v_add3_u32 %1, %1, %5, %10\n v_add3_u32 %2, %2, %6, %11\n v_add3_u32 %3, %3, %7, %8\n v_xor_b32 %12, %12, %0\n v_xor_b32 %13, %13, %1\n v_xor_b32 %14, %14, %2\n v_xor_b32 %15, %15, %3\n v_alignbit_b32 %12, %12, %12, 8\n v_alignbit_b32 %13, %13, %13, 8\n v_alignbit_b32 %14, %14, %14, 8\n v_alignbit_b32 %15, %15, %15, 8\n v_add_u32 %8, %8, %12\n v_add_u32 %9, %9, %13\n v_add_u32 %10, %10, %14\n v_add_u32 %11, %11, %15\n v_xor_b32 %4, %4, %8\n v_xor_b32 %5, %5, %9\n v_xor_b32 %6, %6, %10\n v_xor_b32 %7, %7, %11\n v_alignbit_b32 %4, %4, %4, 7\n v_alignbit_b32 %5, %5, %5, 7\n v_alignbit_b32 %6, %6, %6, 7\n v_alignbit_b32 %7, %7, %7, 7" : VI_W16);)
    }
    if (threadIdx.x == 0) {
        clocks[4 * blockIdx.x + 0] = c0;
        clocks[4 * blockIdx.x + 1] = __builtin_readcyclecounter();
        clocks[4 * blockIdx.x + 2] = t0;
        clocks[4 * blockIdx.x + 3] = wall_clock64();
    }
    uint32_t x = 0;
    for (int q = 0; q < 16; ++q) x ^= w[q];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = x;
}
__global__ __launch_bounds__(256) void k_g4_columns(uint64_t *out, uint64_t *clocks, int iters) {
    uint32_t w[16];
    for (int q = 0; q < 16; ++q) w[q] = threadIdx.x + q;
    uint64_t c0 = 0, t0 = 0;
    if (threadIdx.x == 0) { c0 = __builtin_readcyclecounter(); t0 = wall_clock64(); }
    for (int i = 0; i < iters; ++i) {
        VI_REP16(asm volatile("v_add3_u32 %0, %0, %4, %9\n v_xor_b32 %12, %12, %0\n v_alignbit_b32 %12, %12, %12, 16\n v_add_u32 %8, %8, %12\n v_xor_b32 %4, %4, %8\n v_alignbit_b32 %4, %4, %4, 12\n v_add3_u32 %0, %0, %4, %9\n v_xor_b32 %12, %12, %0\n v_alignbit_b32 %12, %12, %12, 8\n v_add_u32 %8, %8, %12\n v_xor_b32 %4, %4, %8\n v_alignbit_b32 %4, %4, %4, 7\n v_add3_u32 %1, %1, %5, %10\n v_xor_b32 %13, %13, %1\n v_alignbit_b32 %13, %13, %13, 16\n v_add_u32 %9, %9, %13\n v_xor_b32 %5, %5, %9\n v_alignbit_b32 %5, %5, %5, 12\n v_add3_u32 %1, %1, %5, %10\n v_xor_b32 %13, %13, %1\n v_alignbit_b32 %13, %13, %13, 8\n v_add_u32 %9, %9, %13\n v_xor_b32 %5, %5, %9\n v_alignbit_b32 %5, %5, %5, 7\n v_add3_u32 %2, %2, %6, %11\n v_xor_b32 %14, %14, %2\n v_alignbit_b32 %14, %14, %14, 16\n v_add_u32 %10, %10, %14\n v_xor_b32 %6, %6, %10\n v_alignbit_b32 %6, %6, %6, 12\n v_add3_u32 %2, %2, %6, %11\n v_xor_b32 %14, %14, %2\n v_alignbit_b32 %14, %14, %14, 8\n v_add_u32 %10, %10, %14\n v_xor_b32 %6, %6, %10\n v_alignbit_b32 %6, %6, %6, 7\n v_add3_u32 %3, %3, %7, %8\n v_xor_b32 %15, %15, %3\n v_alignbit_b32 %15, %15, %15, 16\n v_add_u32 %11, %11, %15\n v_xor_b32 %7, %7, %11\n v_alignbit_b32 %7, %7, %7, 12\n v_add3_u32 %3, %3, %7, %8\n v_xor_b32 %15, %15, %3\n v_alignbit_b32 %15, %15, %15, 8\n v_add_u32 %11, %11, %15\n v_xor_b32 %7, %7, %11\n v_alignbit_b32 %7, %7, %7, 7" : VI_W16);)
    }
    if (threadIdx.x == 0) {
        clocks[4 * blockIdx.x + 0] = c0;
        clocks[4 * blockIdx.x + 1] = __builtin_readcyclecounter();
        clocks[4 * blockIdx.x + 2] = t0;
        clocks[4 * blockIdx.x + 3] = wall_clock64();
    }
    uint32_t x = 0;
    for (int q = 0; q < 16; ++q) x ^= w[q];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = x;
}

typedef void (*probe_fn)(uint64_t *, uint64_t *, int);
struct Probe {
    const char *name;
    probe_fn fn;
    int per_block;          // VALU instructions per unrolled block of the loop body
};
const Probe PROBES[] = {
    {"v_add_u32", k_add_u32, 256},          {"v_add_co_u32", k_add_co, 256},       {"v_addc_co_u32", k_addc_co, 256},
    {"v_alignbit_b32", k_alignbit, 256},   {"v_add3_u32", k_add3, 256},
    {"v_xor_b32", k_xor, 256},              {"v_mul_lo_u32", k_mul_lo, 256},       {"v_mul_hi_u32", k_mul_hi, 256},
    {"v_mad_u64_u32", k_mad_u64_u32, 256},  {"v_lshl_add_u64", k_lshl_add_u64, 256}, {"v_cmp_lt_u64", k_cmp_u64, 256},
    {"v_mul_u32_u24", k_mul_u32_u24, 256},  {"v_fma_f64", k_fma_f64, 256},         {"modular add sequence (6 VALU)", k_mod_add_seq, 384},
    {"v_sub_u32", k_sub_u32, 256},          {"v_and_b32", k_and, 256},             {"v_or_b32", k_or, 256},
    {"v_lshlrev_b32", k_lshl, 256},         {"v_lshrrev_b32", k_lshr, 256},        {"v_mov_b32", k_mov, 256},
    {"v_min_u32", k_min, 256},              {"v_cmp_lt_u32", k_cmp_u32, 256},
    {"v_perm_b32", k_perm, 256},
    {"v_lshlrev_b64", k_lshl_b64, 256},     {"v_lshrrev_b64", k_lshr_b64, 256},
    {"v_subb_co_u32", k_subb_co, 256},      {"v_bfe_u32", k_bfe, 256},             {"v_lshl_or_b32", k_lshl_or, 256},
    {"v_xor_b32, each reads the one before", k_xor_dependent, 256},
    {"v_xor_b32 / v_alignbit_b32 alternating", k_xor_align_alternating, 256},
    {"v_xor_b32 x2 / v_alignbit_b32 x2", k_xor_align_pairs, 256},
    {"v_xor_b32 / v_add_u32 alternating", k_xor_add_alternating, 256},
    {"v_xor_b32 chain through four registers", k_xor_dep_pairs, 256},
    {"BLAKE3 half G, two columns one after the other", k_g_by_column, 768},
    {"BLAKE3 half G, two columns instruction by instruction", k_g_by_instruction, 768},
    {"BLAKE3 G, four columns, runs of four per instruction", k_g4_runs, 768},
    {"BLAKE3 G, four columns, column after column", k_g4_columns, 768},
};
constexpr int N_PROBES = sizeof(PROBES) / sizeof(PROBES[0]);

}  // namespace

extern "C" {

int vi_valu_probe_count(void) { return N_PROBES; }

/* rate of the constant counter the probe reads beside the shader clock, in kHz (0 if unknown) */
int vi_wall_clock_khz(void) {
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
    return khz;
}

const char *vi_valu_probe_name(int kind) { return kind >= 0 && kind < N_PROBES ? PROBES[kind].name : ""; }

int vi_valu_probe(int kind, int iters, int blocks, uint64_t *out, uint64_t *clocks, int64_t *wave_instructions,
                  void *stream) {
    if (kind < 0 || kind >= N_PROBES) return vi::fail(VI_EINVAL, "vi_valu_probe: kind %d (0..%d)", kind, N_PROBES - 1);
    if (iters < 1 || blocks < 1 || !out || !clocks) return vi::fail(VI_EINVAL, "vi_valu_probe: bad argument");
    hipLaunchKernelGGL(PROBES[kind].fn, dim3(blocks), dim3(256), 0, (hipStream_t)stream, out, clocks, iters);
    VI_LAUNCH_CHECK("valu probe");
    if (wave_instructions) *wave_instructions = (int64_t)blocks * 4 * iters * PROBES[kind].per_block;
    return VI_OK;
}

}  // extern "C"

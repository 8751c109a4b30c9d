// Register-blocked form of one NTT pass for digits of 2^5 .. 2^8 points.
//
// The length-L sub-transform (L = 16 * E2, E2 = 2, 4, 8 or 16) is itself split as
// n = n1*E2 + n2, k = k1 + 16*k2:
//   stage 1   A[k1][n2] = sum_{n1<16} x[n1*E2 + n2] w_16^(n1 k1), times w_L^(n2 k1)
//   stage 2   X[k1 + 16 k2] = sum_{n2<E2} A[k1][n2] w_E2^(n2 k2)
// Every thread runs one 16-point stage-1 transform and 16/E2 stage-2 transforms
// entirely in registers; the tile crosses LDS exactly once in between.  Because
// the 64th roots of unity of this field are powers of two (w_64 = 2^39), every
// butterfly twiddle inside a register transform is +-2^s and costs a shift and a
// fold instead of a 64x64 multiplication; full multiplications remain only for
// the w_L^(n2 k1) layer, the inter-pass twiddles and the coset pre-multipliers.
//
// Global accesses: a strided pass reads/writes runs of T consecutive elements (T =
// TILE / L columns), the final pass reads whole contiguous sub-rows and writes runs of
// T consecutive outputs.  LDS holds [k1][n2][column] with one element of padding per
// (k1, n2) row so both access directions are bank-conflict free.
//
// Written as per-thread phases (see ntt_pass.hpp) so the CPU build can run it.
#pragma once
#include "ntt_pass.hpp"

// Outputs of a pass are not read again by the launch that writes them: a non-temporal store keeps them
// from displacing the source lines that the coset workgroups of a tile share in the L2.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(VI_PLAIN_STORES)
#define VI_STREAM_STORE(p, v) __builtin_nontemporal_store((v), (p))
#define VI_STREAM_LOAD(p) __builtin_nontemporal_load(p)
#else
#define VI_STREAM_STORE(p, v) (*(p) = (v))
#define VI_STREAM_LOAD(p) (*(p))
#endif

namespace ntt {

// exponent e such that w = 2^e for the twiddle w_(2^A)^(j * 2^(A-1-s)) of level s
template <int A, bool INV>
VI_HD constexpr int level_exp(int s, int j) {
    int e = (39 * (64 >> A) * (j << (A - 1 - s))) % 192;
    return INV ? (192 - e) % 192 : e;
}

template <int A>
VI_HD constexpr int brev(int i) {
    int r = 0;
    for (int b = 0; b < A; ++b) r |= ((i >> b) & 1) << (A - 1 - b);
    return r;
}

// in-register transform of 2^A points, natural order in and out; inputs must be
// canonical, outputs are canonical.  Every exponent is a compile-time constant, so a
// twiddle is two or three fixed shifts and one fold (gl::mul_pow2c).
// HALF: the upper half of the inputs, x[N/2 ..], is zero (a source row no wider than half the transform): the first
// level's butterflies (x[m], x[m + N/2]) -> (sum, difference) are copies.
template <int A, bool INV, bool HALF = false>
VI_HD void dft_reg(u64 (&x)[1 << A]) {
    constexpr int N = 1 << A;
    u64 y[N];
#pragma unroll
    for (int i = 0; i < N; ++i) y[i] = x[brev<A>(i)];
    static_for<0, A>([&](auto s_) {
        constexpr int s = decltype(s_)::value;
        static_for<0, N / 2>([&](auto b_) {
            constexpr int b = decltype(b_)::value;
            constexpr int half = 1 << s;
            constexpr int j = b & (half - 1), i0 = ((b >> s) << (s + 1)) + j, i1 = i0 + half;
            constexpr int e = level_exp<A, INV>(s, j);
            const u64 u = y[i0];
            if constexpr (HALF && s == 0) {                // y[i1] = x[brev(i0) + N/2] = 0
                y[i1] = u;
            } else if constexpr (e < 96) {
                const u64 v = gl::mul_pow2c<e>(y[i1]);
                gl::bfly(u, v, y[i0], y[i1]);
            } else {                                   // 2^e = -2^(e-96)
                const u64 v = gl::mul_pow2c<e - 96>(y[i1]);
                gl::bfly(u, v, y[i1], y[i0]);
            }
        });
    });
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] = y[i];
}

constexpr int FAST_A1 = 4;
constexpr int FAST_E1 = 16;
VI_HD bool fast_ok(int a) { return a >= 5 && a <= 8; }
VI_HD bool fast512_ok(int a) { return a == 9; }                  // 512 = 16 x 32: single-pass transforms only (fast_stage2_512)
VI_HD int fast_lds_words(int a) { return TILE + (1 << a); }      // (L rows) x (T + 1)

// per-thread description of the one column it serves in a stage
struct ColRef {
    bool valid;
    i64 src_base;      // element offset of (column, point 0) in src
    i64 idx_base;      // index inside the source row of (column, point 0)
    i64 dst_base;      // element offset of (column, output 0) in dst
    i64 tw_base;       // r (strided pass): twiddle index of output k is (k << logR) + r
    int t;             // coset of the column (final pass)
};

VI_HD ColRef col_ref(const PassArgs &A, i64 tile, int c) {
    ColRef R;
    const i64 T = (i64)1 << logT(A);
    const i64 g = tile * T + c;
    R.t = 0;
    if (!A.is_final) {
        const int lc = A.B + A.logR;
        const i64 row = g >> lc, col = g & (((i64)1 << lc) - 1);
        R.valid = row < A.n_rows;
        const i64 prefix = col >> A.logR, r = col & (((i64)1 << A.logR) - 1);
        R.idx_base = (prefix << (A.a + A.logR)) + r;
        R.src_base = row * A.src_row_stride + R.idx_base;
        R.dst_base = row * A.dst_row_stride + R.idx_base;
        R.tw_base = r;
    } else {
        const int lc = A.B + A.log_rho;
        const i64 row = g >> lc, v = g & (((i64)1 << lc) - 1);
        R.valid = row < A.n_rows;
        R.t = (int)(v & (((i64)1 << A.log_rho) - 1));
        R.idx_base = storage_prefix(A, v >> A.log_rho) << A.a;
        R.src_base = (i64)R.t * A.src_coset_stride + row * A.src_row_stride + R.idx_base;
        R.dst_base = row * A.dst_row_stride + v;
        R.tw_base = 0;
    }
    return R;
}

// A pass whose every tile the workgroup can address with one set of bases and 32-bit per-thread offsets ("uniform
// pass"): the columns of a tile lie in one batch row, every row of the launch exists (a row is a whole number of
// tiles), which of a thread's sixteen inputs exist depends only on their position n1, and the offsets that differ
// between threads stay below 2^29 elements.  The bases are then the same for all threads of the workgroup and live
// in scalar registers; a load or store is "scalar base + thread offset" with no 64-bit vector arithmetic and no
// per-element test.  Passes that do not qualify (short transforms whose rows are narrower than a tile, source rows
// of a ragged width) take the per-element path; the host decides per launch (pass_uniform) and the kernel is
// compiled for one or the other.
struct TileU {
    i64 src_u;        // element offset into src of (first column, point 0), without the per-thread part
    i64 dst_u;        // the same into dst (without the coset plane of a strided pass)
    i64 pre_u;        // index inside the source row of (first column, point 0)
    i64 tw_u;         // strided pass: r of the first column
    int sh1;          // log2 of the element stride between a thread's stage-1 inputs n1, n1 + 1
    int sh2;          // log2 of the element stride between a thread's stage-2 outputs k2, k2 + 1
    int shk;          // log2 of the element stride between outputs k1, k1 + 1
    int shc;          // final pass: log2 of the source stride between column groups (c >> log_rho)
    int shcd;         // log2 of the output stride between columns (0 except in a single-pass transform, whose columns are rows)
};

// does the pass qualify?  On success *n1_valid = how many of a thread's sixteen stage-1 inputs exist (the first
// n1_valid; 16 unless the source rows are narrower than the transform).
inline bool pass_uniform(const PassArgs &A, int *n1_valid) {
    const int lt = logT(A), a2 = A.a - 4;
    *n1_valid = 16;
    if (A.logn > 26 || A.n_rows < 1) return false;
    const i64 n = (i64)1 << A.logn;
    if (!A.is_final) {
        const int lc = A.B + A.logR;
        if (lc < lt || A.logR < lt) return false;
        if (A.src_width == n) return true;
        // a narrower source: only on the first pass (B = 0, so input n1 of a thread has the index
        // (n1 << sh1) + its 32-bit thread offset).  The first n1_valid inputs exist for every thread, input n1_valid for
        // the threads whose index inside that plane is below the remainder of the width (src_width mod 2^sh1), the others for none.
        const int sh1 = a2 + A.logR;
        // (at least the first plane whole, so that word 0 of a tile always exists for the loads that stand in for
        // missing inputs)
        if (A.B != 0 || (A.src_width >> sh1) < 1) return false;
        *n1_valid = (int)(A.src_width >> sh1);
        return true;
    }
    if (A.ndig == 0) {
        // a single-pass transform of contiguous rows: a tile is 2^lt whole rows = TILE consecutive words, in and out
        if (A.pre || A.log_rho != 0 || A.B != 0 || A.logR != 0 || A.a != A.logn) return false;
        if (A.src_width != n || A.src_row_stride != n || A.dst_row_stride != n) return false;
        return (A.n_rows & (((i64)1 << lt) - 1)) == 0;
    }
    const int lc = A.B + A.log_rho;
    if (A.pre || A.ndig < 1 || lc < lt || lt < A.log_rho || lt - A.log_rho > A.dig[0]) return false;
    if (A.src_width != n || A.logn + A.log_rho > 28) return false;
    return (((i64)1 << A.log_rho) - 1) * A.src_coset_stride + n < ((i64)1 << 29);
}

// a uniform first pass whose source rows end within the first eight of a thread's sixteen input planes: inputs
// 8 .. 15 are zero for every thread (A.n1_valid as set by pass_uniform)
inline bool upper_half_zero(const PassArgs &A) {
    if (A.is_final || A.pre || A.n1_valid > 8) return false;
    const int sh1 = (A.a - 4) + A.logR;
    return A.n1_valid < 8 || A.src_width == ((i64)8 << sh1);
}

template <int A2>
VI_HD TileU tile_uniform(const PassArgs &A, i64 tile) {
    TileU U;
    U.src_u = U.dst_u = U.pre_u = U.tw_u = 0;
    U.sh1 = U.sh2 = U.shk = U.shc = U.shcd = 0;
    const int lt = logT(A);
    if (!A.is_final) {
        const int lc = A.B + A.logR;
        const i64 row = tile >> (lc - lt);
        const i64 col0 = (tile & (((i64)1 << (lc - lt)) - 1)) << lt;
        const i64 prefix = col0 >> A.logR, r0 = col0 & (((i64)1 << A.logR) - 1);
        const i64 idx_u = (prefix << (A.a + A.logR)) + r0;
        U.src_u = row * A.src_row_stride + idx_u;
        U.dst_u = row * A.dst_row_stride + idx_u;
        U.pre_u = idx_u;
        U.tw_u = r0;
        U.sh1 = A2 + A.logR;
        U.sh2 = 4 + A.logR;
        U.shk = A.logR;
    } else if (A.ndig == 0) {
        // single-pass transform: column c of the tile is row (tile << lt) + c, point l of it word (c << a) + l of the tile
        U.src_u = (tile << lt) * A.src_row_stride;
        U.dst_u = (tile << lt) * A.dst_row_stride;
        U.sh1 = A2;
        U.sh2 = 4;
        U.shk = 0;
        U.shc = A.a;
        U.shcd = A.a;
    } else {
        const int lc = A.B + A.log_rho;
        const i64 row = tile >> (lc - lt);
        const i64 v0 = (tile & (((i64)1 << (lc - lt)) - 1)) << lt;
        U.src_u = row * A.src_row_stride + (storage_prefix(A, v0 >> A.log_rho) << A.a);
        U.dst_u = row * A.dst_row_stride + v0;
        U.sh1 = A2;
        U.sh2 = 4 + lc;
        U.shk = lc;
        U.shc = A.B - A.dig[0] + A.a;
    }
    return U;
}

// A run of elements addressed as "uniform base + uniform element offset + per-thread element offset" (all three
// below 2^29 elements).  On the device this is a raw buffer access: the base sits in a buffer resource in scalar
// registers, the uniform offset in a scalar register and the thread offset in one vector register, so an access
// costs no vector arithmetic at all and keeps no 64-bit address alive (global_load needs one register pair per
// address, which the compiler hoists out of the coset loop).  On the host it is pointer arithmetic.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((__vector_size__(2 * sizeof(u32)))) u32 vi_u32x2;
struct URun { __amdgpu_buffer_rsrc_t r; };
__device__ __forceinline__ URun urun(const u64 *base) {
    // raw buffer (stride 0), 4 GiB window, 32-bit data format
    return URun{__builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)0xFFFFFFFFu, 0x00020000)};
}
__device__ __forceinline__ u64 uload(const URun &b, u32 uni, u32 off) {
    const vi_u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(b.r, off * 8u, uni * 8u, 0);
    return ((u64)v[1] << 32) | v[0];
}
// read once by this launch and by no later one
__device__ __forceinline__ u64 uload_stream(const URun &b, u32 uni, u32 off) {
    const vi_u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(b.r, off * 8u, uni * 8u, 2);
    return ((u64)v[1] << 32) | v[0];
}
__device__ __forceinline__ void ustore(const URun &b, u32 uni, u32 off, u64 x) {
    const vi_u32x2 v = {(u32)x, (u32)(x >> 32)};
    __builtin_amdgcn_raw_buffer_store_b64(v, b.r, off * 8u, uni * 8u, 0);
}
// not read again by this launch: non-temporal
__device__ __forceinline__ void ustore_stream(const URun &b, u32 uni, u32 off, u64 x) {
    const vi_u32x2 v = {(u32)x, (u32)(x >> 32)};
#if defined(VI_PLAIN_STORES)
    __builtin_amdgcn_raw_buffer_store_b64(v, b.r, off * 8u, uni * 8u, 0);
#else
    __builtin_amdgcn_raw_buffer_store_b64(v, b.r, off * 8u, uni * 8u, 2);
#endif
}
#else
struct URun { u64 *p; };
inline URun urun(const u64 *base) { return URun{const_cast<u64 *>(base)}; }
inline u64 uload(const URun &b, u32 uni, u32 off) { return b.p[(size_t)uni + off]; }
inline u64 uload_stream(const URun &b, u32 uni, u32 off) { return b.p[(size_t)uni + off]; }
inline void ustore(const URun &b, u32 uni, u32 off, u64 x) { b.p[(size_t)uni + off] = x; }
inline void ustore_stream(const URun &b, u32 uni, u32 off, u64 x) { b.p[(size_t)uni + off] = x; }
#endif

// the per-thread part of the stage-1 source offset in a tile described by a TileU
template <int A2>
VI_HD u32 lane_src_off(const PassArgs &A, const TileU &U, int c, int n2) {
    if (!A.is_final) return (u32)c + ((u32)n2 << A.logR);
    const u32 t = (u32)c & ((1u << A.log_rho) - 1), cu = (u32)c >> A.log_rho;
    return t * (u32)A.src_coset_stride + (cu << U.shc) + (u32)n2;
}

// stage-1 thread -> (column, n2)
template <int A2>
VI_HD void s1_coords(const PassArgs &A, int tid, int &c, int &n2) {
    // low bits / high bits of the thread id, then one select each: written as two branches that assign c and n2
    // crosswise the compiler routed the values through scratch memory (a store and a load in front of the
    // first address computation of every workgroup)
    const int sh = A.is_final ? A2 : logT(A);
    const int lo = tid & ((1 << sh) - 1), hi = tid >> sh;
    c = A.is_final ? hi : lo;
    n2 = A.is_final ? lo : hi;
}

// phase 1: this thread's 16 stage-1 inputs x[n1*E2 + n2] as loaded, and in `ok` which of them exist.
// All sixteen loads are issued before the first value is looked at: an element that does not exist (a row past
// the batch, a point past the source width) reads word 0 of the source instead and is zeroed in fast_fix.  With
// the load inside the test, and the reduction mod p right behind it, every second load waited for the one
// before -- eight memory round trips per tile instead of one.
// HALF (uniform passes whose source rows end within the first eight planes, upper_half_zero()): inputs 8 .. 15 are
// not loaded.
template <int A2, bool UNI, bool HALF = false, bool STREAM = false>
VI_HD void fast_load(const PassArgs &A, i64 tile, int tid, u64 (&reg)[16], u32 &ok) {
    int c, n2;
    s1_coords<A2>(A, tid, c, n2);
    if constexpr (UNI) {
        constexpr int NL = HALF ? 8 : 16;
        const TileU U = tile_uniform<A2>(A, tile);
        const u32 off = lane_src_off<A2>(A, U, c, n2);
        // an input past the source width reads input 0 instead (and is zeroed in fast_fix): the choice is the same
        // for every thread, so it is made on the scalar base
        const URun src = urun(A.src + U.src_u);
#pragma unroll
        for (int n1 = 0; n1 < NL; ++n1)
            reg[n1] = STREAM ? uload_stream(src, (u32)(n1 < A.n1_valid ? n1 : 0) << U.sh1, off)
                             : uload(src, (u32)(n1 < A.n1_valid ? n1 : 0) << U.sh1, off);
#pragma unroll
        for (int n1 = NL; n1 < 16; ++n1) reg[n1] = 0;
        ok = A.n1_valid >= 16 ? 0xFFFFu : ((1u << A.n1_valid) - 1u);
        if (A.n1_valid < NL) {
            // the plane the width ends in: this thread's input there exists if its offset is below the remainder
            const u32 rem = (u32)(A.src_width - ((i64)A.n1_valid << U.sh1));
            const bool mine = (u32)U.pre_u + off < rem;           // pre_u: index of the tile's first column inside the row
            const u64 v = uload(src, 0u, mine ? off + ((u32)A.n1_valid << U.sh1) : 0u);     // the others read word 0 of the tile
#pragma unroll
            for (int n1 = 0; n1 < NL; ++n1) reg[n1] = (n1 == A.n1_valid) ? v : reg[n1];
            ok |= mine ? (1u << A.n1_valid) : 0u;
        }
        return;
    }
    const ColRef R = col_ref(A, tile, c);
    const int sh = A.is_final ? 0 : A.logR;
    ok = 0;
#pragma unroll
    for (int n1 = 0; n1 < 16; ++n1) {
        const i64 l = (i64)((n1 << A2) + n2) << sh;
        const bool there = R.valid && R.idx_base + l < A.src_width;
        ok |= there ? (1u << n1) : 0u;
        reg[n1] = A.src[there ? R.src_base + l : 0];
    }
}

// zero for the elements that do not exist, caller data reduced mod p
template <bool HALF = false>
VI_HD void fast_fix(const PassArgs &A, u32 ok, u64 (&reg)[16]) {
    constexpr int NL = HALF ? 8 : 16;                      // HALF: inputs 8 .. 15 are zeros already
    // both as blocks behind one test each, so that the passes that need neither (all elements there, source
    // written by an earlier pass) skip them: as per-element selects they ran in every pass
    if (ok != (HALF ? 0xFFu : 0xFFFFu)) {
#pragma unroll
        for (int n1 = 0; n1 < NL; ++n1) reg[n1] = ((ok >> n1) & 1) ? reg[n1] : 0;
    }
    if (A.canon_src) {
#pragma unroll
        for (int n1 = 0; n1 < NL; ++n1) reg[n1] = gl::canon(reg[n1]);
    }
}

// Where w_L^(n2 k1) sits in a workgroup's LDS copy of the inner twiddle table.  In a final pass consecutive lanes
// hold consecutive n2, and the table's own order [n2][k1] would put sixteen lanes on two LDS banks, so the kernels
// keep the copy of a final pass as [k1][n2] (TWT); in a strided pass sixteen lanes share one n2 (a broadcast) and
// the order stays.
template <int A2, bool TWT>
VI_HD constexpr int twi_slot(int n2, int k1) { return TWT ? (k1 << A2) + n2 : n2 * 16 + k1; }

// Where (k1, n2, column c) sits in LDS between the two stages: [k1][n2][c] with one word of padding per (k1, n2) row.
// SGL (a single-pass transform over whole tiles, pass_uniform): stage 2 runs k1 along the lanes there, so that a
// wavefront's stores are 128-byte runs of output rows (with the columns along the lanes, as in the other passes,
// consecutive lanes would store whole rows apart: the columns of such a tile ARE its rows); the k1 pitch is then
// padded to 4 mod 8 words, which puts the sixteen k1 of a wavefront on different banks.
// The 512-point kernel has no LDS to spare (with any padding of the k1 pitch a fourth workgroup no longer fits a CU):
// there the n2 rows of a k1 block are rotated by 2 k1 instead, which spreads the sixteen k1 over the even banks.
template <int A2>
struct SglLds {
    static constexpr int E2 = 1 << A2, T = TILE >> (4 + A2), ST = T + 1, RAW = E2 * ST;
    static constexpr int S1 = A2 == 5 ? RAW : RAW + ((4 - RAW % 8) + 8) % 8;
    static constexpr int WORDS = 16 * S1;
};
template <int A2, bool SGL>
VI_HD int lds_slot(int st, int k1, int n2, int c) {
    if constexpr (SGL && A2 == 5) return k1 * SglLds<A2>::S1 + ((n2 + 2 * k1) & 31) * SglLds<A2>::ST + c;
    if constexpr (SGL) return k1 * SglLds<A2>::S1 + n2 * SglLds<A2>::ST + c;
    return ((k1 << A2) + n2) * st + c;
}

// phase 2: optional coset pre-multiplier, 16-point transform, w_L^(n2 k1), into LDS
// twi: w_L^(n2 k1) at [n2 * 16 + k1]
// the coset pre-multipliers of this thread's sixteen inputs (a column that does not exist takes those of
// point 0 of coset 0; its data are zero); requested before the tile so that they are there when it arrives
template <int A2, bool UNI>
VI_HD void fast_pre_load(const PassArgs &A, i64 tile, int tid, int t_loop, u64 (&pw)[16]) {
    int c, n2;
    s1_coords<A2>(A, tid, c, n2);
    if constexpr (UNI) {                                   // a strided pass: a final pass with pre-multipliers is never uniform
        const TileU U = tile_uniform<A2>(A, tile);
        const u32 off = lane_src_off<A2>(A, U, c, n2);
        const URun pre = urun(A.pre + ((i64)t_loop << A.logn) + U.pre_u);
#pragma unroll
        for (int n1 = 0; n1 < 16; ++n1) pw[n1] = uload(pre, (u32)n1 << U.sh1, off);
        return;
    }
    const ColRef R = col_ref(A, tile, c);
    const int sh = A.is_final ? 0 : A.logR;
    const int t = A.is_final ? R.t : t_loop;
    const u64 *pre = A.pre + (R.valid ? ((i64)t << A.logn) + R.idx_base : 0);
#pragma unroll
    for (int n1 = 0; n1 < 16; ++n1) pw[n1] = pre[R.valid ? (i64)((n1 << A2) + n2) << sh : 0];
}

template <int A2, bool INV, bool HALF = false, bool TWT = false, bool SGL = false>
VI_HD void fast_stage1(const PassArgs &A, i64 tile, int tid, int t_loop, u32 ok, const u64 (&reg)[16],
                       const u64 (&pw)[16], const u64 *twi, u64 *lds) {
    int c, n2;
    s1_coords<A2>(A, tid, c, n2);
    u64 x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = reg[i];
    fast_fix<HALF>(A, ok, x);
    if (A.pre) {
#pragma unroll
        for (int g = 0; g < 16; g += 4) {
#pragma unroll
            for (int n1 = g; n1 < g + 4; ++n1) x[n1] = gl::mul(x[n1], pw[n1]);
            VI_SCHED_FENCE();
        }
    }
    VI_SCHED_FENCE();
    dft_reg<4, INV, HALF>(x);
    VI_SCHED_FENCE();
    const int st = (1 << logT(A)) + 1;
#pragma unroll
    for (int g = 0; g < 16; g += 4) {
#pragma unroll
        for (int k1 = g; k1 < g + 4; ++k1) {
            u64 v = x[k1];
            if (k1 > 0) v = gl::mul(v, twi[twi_slot<A2, TWT>(n2, k1)]);
            lds[lds_slot<A2, SGL>(st, k1, n2, c)] = v;
        }
        VI_SCHED_FENCE();
    }
}

// phase 3: 16/E2 stage-2 transforms, inter-pass twiddle (or final scale), scatter
template <int A2, bool INV, bool UNI, bool SGL = false>
VI_HD void fast_stage2(const PassArgs &A, i64 tile, int tid, int t_loop, const u64 *lds) {
    constexpr int E2 = 1 << A2;
    const int lt = logT(A);
    const int st = (1 << lt) + 1;
    const int c = tid & ((1 << lt) - 1);
    if constexpr (SGL) {
        // whole tiles of a single-pass transform: thread (k1 = low four bits, sixteen columns per trip), outputs
        // k1 + 16 k2 of row c at word (c << a) + k1 + 16 k2 of the tile
        static_assert(UNI, "whole tiles are addressed through scalar bases");
        const TileU U = tile_uniform<A2>(A, tile);
        const URun dst = urun(A.dst + U.dst_u);
        const int k1 = tid & 15;
#pragma unroll
        for (int i = 0; i < 16 / E2; ++i) {
            const int cc = (tid >> 4) + 16 * i;
            const u32 off = ((u32)cc << U.shcd) + (u32)k1;
            u64 x[E2];
#pragma unroll
            for (int n2 = 0; n2 < E2; ++n2) x[n2] = lds[lds_slot<A2, true>(st, k1, n2, cc)];
            VI_SCHED_FENCE();
            dft_reg<A2, INV>(x);
            VI_SCHED_FENCE();
#pragma unroll
            for (int k2 = 0; k2 < E2; ++k2) {
                u64 v = x[k2];
                if (A.scale != 1) v = gl::mul(v, A.scale);
                ustore_stream(dst, (u32)k2 << 4, off, v);
                if ((k2 & 3) == 3) VI_SCHED_FENCE();
            }
        }
        return;
    }
    if constexpr (UNI) {
        const TileU U = tile_uniform<A2>(A, tile);
        const URun dst = urun(A.dst + U.dst_u + (A.is_final ? 0 : (i64)t_loop * A.dst_coset_stride));
        const URun twr = urun(A.is_final ? A.dst : A.tw + U.tw_u);
#pragma unroll
        for (int i = 0; i < 16 / E2; ++i) {
            const int k1 = (tid + i * NTHREADS) >> lt;
            const u32 off = ((u32)c << U.shcd) + ((u32)k1 << U.shk);
            u64 x[E2], tw[E2];
            if (!A.is_final) {
#pragma unroll
                for (int k2 = 0; k2 < E2; ++k2) tw[k2] = uload(twr, (u32)k2 << U.sh2, off);
            }
#pragma unroll
            for (int n2 = 0; n2 < E2; ++n2) x[n2] = lds[((k1 << A2) + n2) * st + c];
            VI_SCHED_FENCE();
            dft_reg<A2, INV>(x);
            VI_SCHED_FENCE();
#pragma unroll
            for (int k2 = 0; k2 < E2; ++k2) {
                u64 v = x[k2];
                if (!A.is_final) v = gl::mul(v, tw[k2]);
                else if (A.scale != 1) v = gl::mul(v, A.scale);
                ustore_stream(dst, (u32)k2 << U.sh2, off, v);
                if ((k2 & 3) == 3) VI_SCHED_FENCE();
            }
        }
        return;
    }
    const ColRef R = col_ref(A, tile, c);
    const int lc = A.B + A.log_rho;
#pragma unroll
    for (int i = 0; i < 16 / E2; ++i) {
        const int k1 = (tid + i * NTHREADS) >> lt;
        u64 x[E2];
        // the inter-pass twiddles are requested before the LDS reads and the transform, which then cover their latency
        u64 tw[E2];
        if (!A.is_final && R.valid) {
#pragma unroll
            for (int k2 = 0; k2 < E2; ++k2) tw[k2] = A.tw[((i64)(k1 + 16 * k2) << A.logR) + R.tw_base];
        }
#pragma unroll
        for (int n2 = 0; n2 < E2; ++n2) x[n2] = lds[((k1 << A2) + n2) * st + c];
        VI_SCHED_FENCE();
        dft_reg<A2, INV>(x);
        VI_SCHED_FENCE();
        if (!R.valid) continue;
#pragma unroll
        for (int k2 = 0; k2 < E2; ++k2) {
            const i64 k = k1 + 16 * k2;
            u64 v = x[k2];
            if (!A.is_final) {
                v = gl::mul(v, tw[k2]);
                VI_STREAM_STORE(&A.dst[(i64)t_loop * A.dst_coset_stride + R.dst_base + (k << A.logR)], v);
            } else {
                if (A.scale != 1) v = gl::mul(v, A.scale);
                VI_STREAM_STORE(&A.dst[R.dst_base + (k << lc)], v);
            }
            if ((k2 & 3) == 3) VI_SCHED_FENCE();
        }
    }
}


// Stage 2 of a 512-point single pass (16 x 32): the 32-point transforms over n2.  Two threads share one
// transform, decimated in frequency: both read its 32 values, thread h = 0 forms the sixteen sums
// x[j] + x[j + 16] and gets the even outputs from a 16-point transform, thread h = 1 forms the differences times
// w_32^j (shifts) and gets the odd outputs -- no exchange between the two.  h is the top bit of the thread id, so a
// wavefront is all sums or all differences.  Per-element addressing (a single pass is never a uniform pass).
template <bool INV, bool UNI = false>
VI_HD void fast_stage2_512(const PassArgs &A, i64 tile, int tid, const u64 *lds) {
    constexpr int A2 = 5;
    const int lt = logT(A);                                // 3: eight columns per tile
    const int st = (1 << lt) + 1;
    // UNI (whole tiles of contiguous rows): k1 along the lanes, see lds_slot
    const int c = UNI ? (tid >> 4) & ((1 << lt) - 1) : tid & ((1 << lt) - 1);
    const int k1 = UNI ? tid & 15 : (tid >> lt) & 15, h = tid >> (lt + 4);
    ColRef R{};
    if (!UNI) R = col_ref(A, tile, c);
    const int lc = A.B + A.log_rho;
    u64 x[32], y[16];
#pragma unroll
    for (int n2 = 0; n2 < 32; ++n2) x[n2] = lds[lds_slot<A2, UNI>(st, k1, n2, c)];
    if (h == 0) {
#pragma unroll
        for (int j = 0; j < 16; ++j) y[j] = gl::addc(x[j], x[j + 16]);
    } else {
        static_for<0, 16>([&](auto j_) {
            constexpr int j = decltype(j_)::value;
            constexpr int e = level_exp<5, INV>(4, j);         // w_32^j = 2^e
            const u64 d = gl::sub(x[j], x[j + 16]);
            if constexpr (e == 0) y[j] = d;
            else if constexpr (e < 96) y[j] = gl::mul_pow2c<e>(d);
            else y[j] = gl::neg(gl::mul_pow2c<e - 96>(d));
        });
    }
    VI_SCHED_FENCE();
    dft_reg<4, INV>(y);
    VI_SCHED_FENCE();
    if constexpr (UNI) {                                   // contiguous rows (pass_uniform): output k of column c is word (c << 9) + k of the tile
        const TileU U = tile_uniform<A2>(A, tile);
        const URun dst = urun(A.dst + U.dst_u);
        const u32 off = ((u32)c << U.shcd) + (u32)k1 + 16u * (u32)h;
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            u64 v = y[m];
            if (A.scale != 1) v = gl::mul(v, A.scale);
            ustore_stream(dst, 32u * (u32)m, off, v);
        }
        return;
    }
    if (!R.valid) return;
#pragma unroll
    for (int m = 0; m < 16; ++m) {
        const i64 k = k1 + 16 * (2 * m + h);
        u64 v = y[m];
        if (A.scale != 1) v = gl::mul(v, A.scale);
        VI_STREAM_STORE(&A.dst[R.dst_base + (k << lc)], v);
    }
}

// The last inverse pass and the first forward pass of a coset extension share their tiles when K = L * L: the last
// inverse pass leaves, in the thread that ran the stage-2 transforms (column c, outputs k1 = q + E2 i, i < 16 / E2),
// the coefficients of points k = k1 + 16 k2 of that column, and the first forward pass wants thread (c, n2) to hold
// points n1 E2 + n2 -- the same thread with n2 = q and n1 = i + (16 / E2) k2.  So a workgroup can go on to the rho
// coset transforms without the coefficients leaving its registers (they are still written out when the caller
// wants them: A.dst non-null).  Uniform passes only.
template <int A2>
VI_HD void fused_stage2_inv(const PassArgs &A, i64 tile, int tid, const u64 *lds, u64 (&coef)[16]) {
    constexpr int E2 = 1 << A2;
    const int lt = logT(A);
    const int st = (1 << lt) + 1;
    const int c = tid & ((1 << lt) - 1);
    const TileU U = tile_uniform<A2>(A, tile);
#pragma unroll
    for (int i = 0; i < 16 / E2; ++i) {
        const int k1 = (tid + i * NTHREADS) >> lt;
        u64 x[E2];
#pragma unroll
        for (int n2 = 0; n2 < E2; ++n2) x[n2] = lds[((k1 << A2) + n2) * st + c];
        VI_SCHED_FENCE();
        dft_reg<A2, true>(x);
        VI_SCHED_FENCE();
#pragma unroll
        for (int k2 = 0; k2 < E2; ++k2) {
            u64 v = x[k2];
            if (A.scale != 1) v = gl::mul(v, A.scale);
            coef[i + (16 / E2) * k2] = v;
        }
    }
    if (A.dst) {
        const URun dst = urun(A.dst + U.dst_u);
#pragma unroll
        for (int i = 0; i < 16 / E2; ++i) {
            const int k1 = (tid + i * NTHREADS) >> lt;
            const u32 off = (u32)c + ((u32)k1 << U.shk);
#pragma unroll
            for (int k2 = 0; k2 < E2; ++k2) ustore(dst, (u32)k2 << U.sh2, off, coef[i + (16 / E2) * k2]);
        }
    }
}


// x[n1] = c[n1] * 2^(39 M n1): the part w_N^(t n1 K/16) of the coset factors, M = t * merge_unit (2^96 = -1)
template <int M>
VI_HD void coset_shift(const u64 (&c)[16], u64 (&x)[16]) {
    x[0] = c[0];
    static_for<1, 16>([&](auto n_) {
        constexpr int n1 = decltype(n_)::value;
        constexpr int e = (39 * M * n1) % 192;
        x[n1] = gl::mul_pow2c_pinned<e>(c[n1]);
        if constexpr ((n1 & 3) == 3) VI_SCHED_FENCE();
    });
}

// MRG: the part of the coset factors that does not depend on the coset, shift^i, applied to the coefficients once
template <int A2>
VI_HD void fused_twist(const PassArgs &A, i64 tile, int tid, u64 (&coef)[16]) {
    int c, n2;
    s1_coords<A2>(A, tid, c, n2);
    const TileU U = tile_uniform<A2>(A, tile);
    const u32 off = lane_src_off<A2>(A, U, c, n2);
    const URun pre = urun(A.pre + U.pre_u);                // pre[0][i] = shift^i
#pragma unroll
    for (int g = 0; g < 16; g += 4) {
        u64 pw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pw[j] = uload(pre, (u32)(g + j) << U.sh1, off);
#pragma unroll
        for (int j = 0; j < 4; ++j) coef[g + j] = gl::mul(coef[g + j], pw[j]);
        VI_SCHED_FENCE();
    }
}

// Stage 1 and stage 2 of the first forward pass inside the fused launch.  The sixteen coefficients stay live in
// registers over all cosets there, so the multipliers and twiddles are fetched four at a time, right before use,
// instead of all sixteen ahead of the tile: other wavefronts cover the latency, and the kernel fits 128 registers.
// MRG: the coefficients already carry shift^i (fused_twist), the coset's own factors are a shift per input here,
// the inner twiddle table of coset t (twi) and the inter-pass table of coset t in stage 2.
template <int A2, bool MRG>
VI_HD void fused_stage1_fwd(const PassArgs &A, i64 tile, int tid, int t, const u64 (&coef)[16], const u64 *twi, u64 *lds) {
    int c, n2;
    s1_coords<A2>(A, tid, c, n2);
    u64 x[16];
    if constexpr (MRG) {
        switch (t * A.merge_unit) {                        // the same for every thread of the launch
            case 1: coset_shift<1>(coef, x); break;
            case 2: coset_shift<2>(coef, x); break;
            case 3: coset_shift<3>(coef, x); break;
            default:
#pragma unroll
                for (int i = 0; i < 16; ++i) x[i] = coef[i];
                break;
        }
    } else {
        const TileU U = tile_uniform<A2>(A, tile);
        const u32 off = lane_src_off<A2>(A, U, c, n2);
        const URun pre = urun(A.pre + ((i64)t << A.logn) + U.pre_u);
#pragma unroll
        for (int g = 0; g < 16; g += 4) {
            u64 pw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) pw[j] = uload(pre, (u32)(g + j) << U.sh1, off);
#pragma unroll
            for (int j = 0; j < 4; ++j) x[g + j] = gl::mul(coef[g + j], pw[j]);
            VI_SCHED_FENCE();
        }
    }
    VI_SCHED_FENCE();
    dft_reg<4, false>(x);
    VI_SCHED_FENCE();
    const int st = (1 << logT(A)) + 1;
    const bool all_k1 = MRG && t > 0;                      // coset t > 0: the k1 = 0 column carries w_N^(t n2 R)
#pragma unroll
    for (int g = 0; g < 16; g += 4) {
#pragma unroll
        for (int k1 = g; k1 < g + 4; ++k1) {
            u64 v = x[k1];
            if (k1 > 0 || all_k1) v = gl::mul(v, twi[n2 * 16 + k1]);
            lds[((k1 << A2) + n2) * st + c] = v;
        }
        VI_SCHED_FENCE();
    }
}

template <int A2, bool MRG>
VI_HD void fused_stage2_fwd(const PassArgs &A, i64 tile, int tid, int t, const u64 *lds) {
    constexpr int E2 = 1 << A2;
    constexpr int G = E2 < 4 ? E2 : 4;
    const int lt = logT(A);
    const int st = (1 << lt) + 1;
    const int c = tid & ((1 << lt) - 1);
    const TileU U = tile_uniform<A2>(A, tile);
    const URun dst = urun(A.dst + U.dst_u + (i64)t * A.dst_coset_stride);
    const URun twr = urun(MRG ? A.twm + ((i64)t << A.logn) + U.tw_u : A.tw + U.tw_u);
#pragma unroll
    for (int i = 0; i < 16 / E2; ++i) {
        const int k1 = (tid + i * NTHREADS) >> lt;
        const u32 off = (u32)c + ((u32)k1 << U.shk);
        u64 x[E2];
#pragma unroll
        for (int n2 = 0; n2 < E2; ++n2) x[n2] = lds[((k1 << A2) + n2) * st + c];
        VI_SCHED_FENCE();
        dft_reg<A2, false>(x);
        VI_SCHED_FENCE();
#pragma unroll
        for (int g = 0; g < E2; g += G) {
            u64 tw[G];
#pragma unroll
            for (int j = 0; j < G; ++j) tw[j] = uload(twr, (u32)(g + j) << U.sh2, off);
#pragma unroll
            for (int j = 0; j < G; ++j) ustore_stream(dst, (u32)(g + j) << U.sh2, off, gl::mul(x[g + j], tw[j]));
            VI_SCHED_FENCE();
        }
    }
}

// Rows of 2^(A0 + 8) points in one launch, A0 = 2, 3 or 4.  A tile is 16 >> A0 whole rows.  Thread r < 256 first
// runs the 2^A0-point transforms over the elements r, r + 256, r + 512, ... of each of the tile's rows (the strided
// first digit: P0 with a = A0, logR = 8) and multiplies by the inter-pass twiddles; the results go to LDS as the
// sixteen 256-point columns [row, k][r] the last digit (P1, a = 8) works on, each padded to ROW_ST words so that the
// four columns a wavefront gathers from start on alternating halves of the banks.  The last digit is the
// register-blocked final pass (fast_stage1 / fast_stage2) with the gather from LDS in the place of its load.
constexpr int ROW_ST = 256 + 16;
template <int A0, bool INV>
VI_HD void row_stage0(const PassArgs &A, i64 tile, int tid, u64 *lds) {
    static_assert(NTHREADS == 256 && A0 >= 2 && A0 <= 4, "one thread per residue mod 256");
    constexpr int E0 = 1 << A0, NSUB = 16 / E0;
    u64 x[16], tw[E0];
    u32 ok = 0;
#pragma unroll
    for (int j = 0; j < NSUB; ++j) {
        const i64 row = tile * NSUB + j;
#pragma unroll
        for (int n1 = 0; n1 < E0; ++n1) {
            const i64 idx = ((i64)n1 << 8) + tid;
            const bool there = row < A.n_rows && idx < A.src_width;
            ok |= there ? (1u << (j * E0 + n1)) : 0u;
            x[j * E0 + n1] = VI_STREAM_LOAD(&A.src[there ? row * A.src_row_stride + idx : 0]);     // read once
        }
    }
    // w_n^(k r), the same for every row; row 0 of the table is 1 forward and 1/n inverse
#pragma unroll
    for (int k = 0; k < E0; ++k) tw[k] = (k > 0 || INV) ? A.tw[(k << 8) + tid] : 1;
    fast_fix(A, ok, x);
    VI_SCHED_FENCE();
#pragma unroll
    for (int j = 0; j < NSUB; ++j) {
        u64 y[E0];
#pragma unroll
        for (int n1 = 0; n1 < E0; ++n1) y[n1] = x[j * E0 + n1];
        dft_reg<A0, INV>(y);
#pragma unroll
        for (int k = 0; k < E0; ++k) {
            u64 v = y[k];
            if (k > 0 || INV) v = gl::mul(v, tw[k]);
            lds[(j * E0 + k) * ROW_ST + tid] = v;
        }
        VI_SCHED_FENCE();
    }
}

// the stage-1 inputs of the last digit, x[n1 * 16 + n2] of column c, out of the columns row_stage0 left in LDS
VI_HD void row_gather(const u64 *lds, int tid, u64 (&reg)[16]) {
    const int c = tid >> 4, n2 = tid & 15;
#pragma unroll
    for (int n1 = 0; n1 < 16; ++n1) reg[n1] = lds[c * ROW_ST + (n1 << 4) + n2];
}

// can passes Ai (last inverse) and Af (first forward, expanding into cosets) run as one fused launch?
inline bool passes_fusable(const PassArgs &Ai_in, const PassArgs &Af_in) {
    PassArgs Ai = Ai_in, Af = Af_in;
    int nv = 16;
    if (!Ai.is_final || Af.is_final || !Af.loop_cosets || !Ai.inverse || Af.inverse) return false;
    if (Ai.a != Af.a || Ai.logn != Af.logn || Ai.logn != 2 * Ai.a || !fast_ok(Ai.a)) return false;
    if (Ai.log_rho != 0 || Ai.pre || !Af.pre || Af.canon_src || Ai.n_rows != Af.n_rows) return false;
    if (Af.src_width != ((i64)1 << Af.logn)) return false;
    if (!pass_uniform(Ai, &nv) || nv != 16) return false;
    if (!pass_uniform(Af, &nv) || nv != 16) return false;
    return pass_tiles(Ai) == pass_tiles(Af);
}

}  // namespace ntt

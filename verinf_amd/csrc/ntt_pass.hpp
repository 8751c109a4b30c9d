// One pass of the multi-pass Goldilocks NTT, written as per-thread phases so that
// the same code runs as a HIP kernel (phases separated by workgroup barriers) and
// as a plain host loop in the CPU build used by the test-suite.
//
// A transform of length n = 2^logn is split into digits n = L_1 * L_2 * ... * L_p.
// With the input index written j = ((j_1 L_2 + j_2) L_3 + j_3)..., pass q runs the
// length-L_q sub-transform over digit j_q (element stride R_q = L_{q+1}...L_p),
// multiplies output k_q of the sub-problem of size M_q = L_q R_q by w_{M_q}^{k_q r}
// (r = the digits below) and leaves the data in place: layout [k_1]..[k_q][j_{q+1}]..
// The last pass (R = 1) has no twiddle and writes X[k_1 + L_1 k_2 + L_1 L_2 k_3 ...],
// i.e. the digit-reversed scatter that restores natural order.
//
// A workgroup owns a tile of TILE elements = T columns x L points, staged in LDS
// as [point][column] with one element of padding per point-row so that both the
// column-major and the point-major access patterns are free of bank conflicts.
// Global accesses are runs of T consecutive elements (strided passes) or whole
// contiguous tiles.
//
// Coset extension (the Reed-Solomon LDE) adds a coset index t < rho:
//   * a non-final pass can loop over t, re-using one gathered source tile and
//     multiplying it by pre[t][i] before each sub-transform (loop_cosets);
//   * the final pass treats t as the lowest output digit: column id v = u*rho + t,
//     so that the interleaved codeword out[rho*k + t] is written in contiguous runs.
#pragma once
#include "gl_field.hpp"

namespace ntt {

constexpr int TILE_LOG = 12;
constexpr int TILE = 1 << TILE_LOG;       // elements per workgroup tile (32 KiB of LDS + padding)
constexpr int EPT = 16;                   // elements per thread
constexpr int NTHREADS = TILE / EPT;
constexpr int MAX_A = 8;                  // largest digit of a multi-pass split
constexpr int TWL_LOG = 12;               // master table of w_4096^j, j < 2048 (TILE_LOG <= 12)
constexpr int LDS_WORDS = TILE + (TILE >> 1);   // worst-case padded size (T = 1 needs none, T >= 2 needs L <= TILE/2 pads)

struct PassArgs {
    const u64 *src;
    u64 *dst;
    i64 src_row_stride, dst_row_stride;       // elements between batch rows
    i64 src_coset_stride, dst_coset_stride;   // elements between coset planes
    i64 n_rows;                               // batch rows in this launch
    i64 src_width;                            // valid elements of a source row; the rest reads as zero
    int logn;                                 // row length of the transform
    int a;                                    // log2 L of this pass
    int logR;                                 // log2 R (0 on the final pass)
    int B;                                    // logn - a - logR
    int is_final;
    int ndig;                                 // final pass: number of earlier digits
    int dig[3];                               // final pass: their widths a_1 .. a_{p-1}
    int log_rho;                              // log2 number of cosets
    int loop_cosets;                          // non-final pass: produce all rho cosets from one source tile
    const u64 *tw;                            // non-final: w_M^(k r) at [(k << logR) + r]
    const u64 *pre;                           // optional pre-multipliers at [(t << logn) + i]
    const u64 *twl;                           // w_4096^j (or its inverse), j < 2048
    const u64 *twi;                           // register-blocked kernel: w_L^(n2 k1) at [n2 * 16 + k1]
    u64 scale;                                // final pass: scalar multiplier (1 = none)
    int inverse;                              // direction of the transform
    int canon_src;                            // src is caller data: reduce every word mod p on load
    int uniform;                              // register-blocked kernel: every tile is addressed by scalar bases (ntt_fast.hpp)
    int n1_valid;                             // uniform pass: how many of a thread's sixteen stage-1 inputs exist
    int fuse_next;                            // last inverse pass of a coset extension: runs fused with the pass after it (dst may be null)
    // first forward pass inside the fused launch, coset factors split up (null / 0: pre[t] is applied whole):
    const u64 *twm;                           // [t][(k << logR) + r] = tw[(k << logR) + r] * w_N^(t r)
    const u64 *twim;                          // [t][n2 * 16 + k1] = twi[n2 * 16 + k1] * w_N^(t n2 R)
    int merge_unit;                           // w_N^(t n1 K/16) = 2^(39 * merge_unit * t * n1); merge_unit * t <= 3
};

VI_HD int logT(const PassArgs &A) { return TILE_LOG - A.a; }
VI_HD int lds_stride(const PassArgs &A) { return (1 << logT(A)) + ((A.a < TILE_LOG) ? 1 : 0); }

VI_HD u32 bitrev(u32 x, int bits) {
    u32 r = 0;
    for (int i = 0; i < bits; ++i) r |= ((x >> i) & 1u) << (bits - 1 - i);
    return r;
}

// number of tiles of a launch
inline i64 pass_tiles(const PassArgs &A) {
    i64 cols_per_row = A.is_final ? ((i64)1 << (A.B + A.log_rho)) : ((i64)1 << (A.B + A.logR));
    i64 total = cols_per_row * A.n_rows;
    i64 T = (i64)1 << logT(A);
    return (total + T - 1) / T;
}

// final pass: column u in output order (k_1 lowest) -> prefix index in storage order (k_1 highest)
VI_HD i64 storage_prefix(const PassArgs &A, i64 u) {
    i64 pre = 0;
    // at most three earlier digits; spelled out so that the by-value argument
    // struct is never indexed dynamically (that would force it into scratch memory)
    if (A.ndig > 0) { pre = u & (((i64)1 << A.dig[0]) - 1); u >>= A.dig[0]; }
    if (A.ndig > 1) { pre = (pre << A.dig[1]) | (u & (((i64)1 << A.dig[1]) - 1)); u >>= A.dig[1]; }
    if (A.ndig > 2) { pre = (pre << A.dig[2]) | (u & (((i64)1 << A.dig[2]) - 1)); }
    return pre;
}

struct Elem {
    int l, c;          // point and column inside the tile
    bool valid;        // column exists
    i64 addr;          // element offset into src (gather) or dst (scatter)
    i64 idx;           // index inside the source row (for zero-fill / pre-multiplier)
    int t;             // coset of the column (final pass)
    i64 k_r;           // (k << logR) + r : twiddle index (non-final scatter)
};

// tile element e in GATHER order
VI_HD Elem gather_elem(const PassArgs &A, i64 tile, int e) {
    Elem E;
    const int lt = logT(A);
    const i64 T = (i64)1 << lt;
    E.t = 0;
    E.k_r = 0;
    if (!A.is_final) {
        if (A.logR >= lt) { E.c = e & (int)(T - 1); E.l = e >> lt; }
        else {
            int rlow = e & ((1 << A.logR) - 1);
            E.l = (e >> A.logR) & ((1 << A.a) - 1);
            E.c = ((e >> (A.logR + A.a)) << A.logR) | rlow;
        }
        i64 g = tile * T + E.c;
        int lc = A.B + A.logR;
        i64 row = g >> lc, col = g & (((i64)1 << lc) - 1);
        E.valid = row < A.n_rows;
        i64 prefix = col >> A.logR, r = col & (((i64)1 << A.logR) - 1);
        E.idx = (prefix << (A.a + A.logR)) + ((i64)E.l << A.logR) + r;
        E.addr = row * A.src_row_stride + E.idx;
    } else {
        E.l = e & ((1 << A.a) - 1);
        E.c = e >> A.a;
        i64 g = tile * T + E.c;
        int lc = A.B + A.log_rho;
        i64 row = g >> lc, v = g & (((i64)1 << lc) - 1);
        E.valid = row < A.n_rows;
        E.t = (int)(v & (((i64)1 << A.log_rho) - 1));
        i64 u = v >> A.log_rho;
        E.idx = (storage_prefix(A, u) << A.a) + E.l;
        E.addr = (i64)E.t * A.src_coset_stride + row * A.src_row_stride + E.idx;
    }
    return E;
}

// tile element e in SCATTER order (LDS now holds sub-transform output k = E.l)
VI_HD Elem scatter_elem(const PassArgs &A, i64 tile, int e, int t_loop) {
    Elem E;
    const int lt = logT(A);
    const i64 T = (i64)1 << lt;
    E.t = t_loop;
    E.idx = 0;
    E.k_r = 0;
    if (!A.is_final) {
        if (A.logR >= lt) { E.c = e & (int)(T - 1); E.l = e >> lt; }
        else {
            int rlow = e & ((1 << A.logR) - 1);
            E.l = (e >> A.logR) & ((1 << A.a) - 1);
            E.c = ((e >> (A.logR + A.a)) << A.logR) | rlow;
        }
        i64 g = tile * T + E.c;
        int lc = A.B + A.logR;
        i64 row = g >> lc, col = g & (((i64)1 << lc) - 1);
        E.valid = row < A.n_rows;
        i64 prefix = col >> A.logR, r = col & (((i64)1 << A.logR) - 1);
        E.k_r = ((i64)E.l << A.logR) + r;
        E.addr = (i64)t_loop * A.dst_coset_stride + row * A.dst_row_stride +
                 (prefix << (A.a + A.logR)) + E.k_r;
    } else {
        E.c = e & (int)(T - 1);
        E.l = e >> lt;
        i64 g = tile * T + E.c;
        int lc = A.B + A.log_rho;
        i64 row = g >> lc, v = g & (((i64)1 << lc) - 1);
        E.valid = row < A.n_rows;
        E.addr = row * A.dst_row_stride + v + ((i64)E.l << lc);
    }
    return E;
}

// phase 1: gather this thread's EPT source elements (zero beyond src_width)
VI_HD void ph_load(const PassArgs &A, i64 tile, int tid, u64 (&reg)[EPT]) {
    // every load is issued before the first value is used: an element that does not exist reads word 0
    // of the source and is zeroed afterwards
    bool ok[EPT];
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        Elem E = gather_elem(A, tile, tid + i * NTHREADS);
        ok[i] = E.valid && E.idx < A.src_width;
        reg[i] = A.src[ok[i] ? E.addr : 0];
    }
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
        const u64 v = ok[i] ? reg[i] : 0;
        reg[i] = A.canon_src ? gl::canon(v) : v;
    }
}

// phase 2: (optionally pre-multiplied) values into LDS at the bit-reversed point
VI_HD void ph_stage(const PassArgs &A, i64 tile, int tid, int t_loop, const u64 (&reg)[EPT], u64 *lds) {
    const int st = lds_stride(A);
    for (int i = 0; i < EPT; ++i) {
        Elem E = gather_elem(A, tile, tid + i * NTHREADS);
        u64 v = reg[i];
        if (A.pre && E.valid) {
            int t = A.is_final ? E.t : t_loop;
            v = gl::mul(v, A.pre[((i64)t << A.logn) + E.idx]);
        }
        lds[(i64)bitrev((u32)E.l, A.a) * st + E.c] = v;
    }
}

// phase 3: radix-2 decimation-in-time level s (half-span 2^s) over every column
VI_HD void ph_level(const PassArgs &A, int tid, int s, u64 *lds) {
    const int st = lds_stride(A), lt = logT(A);
    const int half = 1 << s;
    for (int i = 0; i < EPT / 2; ++i) {
        int b = tid + i * NTHREADS;                 // butterfly id in [0, TILE/2)
        int c = b & ((1 << lt) - 1), bf = b >> lt;
        int j = bf & (half - 1), grp = bf >> s;
        int i0 = (grp << (s + 1)) + j, i1 = i0 + half;
        u64 x = lds[(i64)i0 * st + c], y = lds[(i64)i1 * st + c];
        if (s > 0) y = gl::mul(y, A.twl[(i64)j << (TWL_LOG - 1 - s)]);
        lds[(i64)i0 * st + c] = gl::addc(x, y);
        lds[(i64)i1 * st + c] = gl::sub(x, y);
    }
}

// phase 4: twiddle / scale and scatter
VI_HD void ph_store(const PassArgs &A, i64 tile, int tid, int t_loop, const u64 *lds) {
    const int st = lds_stride(A);
    for (int i = 0; i < EPT; ++i) {
        Elem E = scatter_elem(A, tile, tid + i * NTHREADS, t_loop);
        if (!E.valid) continue;
        u64 v = lds[(i64)E.l * st + E.c];
        if (!A.is_final) v = gl::mul(v, A.tw[E.k_r]);
        else if (A.scale != 1) v = gl::mul(v, A.scale);
        A.dst[E.addr] = v;
    }
}

}  // namespace ntt

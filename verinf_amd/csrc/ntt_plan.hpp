// Host-side planning for the multi-pass NTT: digit split, twiddle tables and the
// list of passes (ntt::PassArgs) that realise a batched in-place transform or a
// coset low-degree extension.  Pure host C++ (no HIP calls) so that both the HIP
// launcher and the CPU build used by the tests share it.
#pragma once
#include <vector>

#include "ntt_fast.hpp"

namespace ntt {

// 7^((p-1)/2^logn): the root the reference uses (prover/ref/goldilocks_ref.py:45-49,
// prover/kernels/ntt.cuh:310-344)
inline u64 root_of_unity(int logn) { return gl::pow(7, (gl::P - 1) >> logn); }
inline u64 inverse(u64 a) { return gl::pow(a, gl::P - 2); }

struct Split {
    int p;
    int a[4];
};

// n < 2^10 is a single in-LDS pass; from 2^10 on the digits are as even as possible and at most
// 2^MAX_A, largest first, so that every pass is a register-blocked one (2^10 .. 2^12 would fit a
// single in-LDS pass, but two register-blocked passes are 1.5 x faster: 0.65 vs 1.0 ms for 2^26 points).
inline Split split_digits(int logn) {
    Split s{};
    if (logn < 10) { s.p = 1; s.a[0] = logn; return s; }
    s.p = (logn + MAX_A - 1) / MAX_A;
    int base = logn / s.p, extra = logn % s.p;
    for (int q = 0; q < s.p; ++q) s.a[q] = base + (q < extra ? 1 : 0);
    return s;
}

// Rows of 2^10 .. 2^12 points as ONE launch (k_ntt_row): a first digit of 4, 8 or 16 points at stride 256 and a last
// digit of 256 points, the tile (whole rows) staying in LDS between the two.
inline bool row_single_ok(int logn) { return logn >= 10 && logn <= TILE_LOG; }
inline Split row_split(int logn) {
    Split s{};
    s.p = 2;
    s.a[0] = logn - MAX_A;
    s.a[1] = MAX_A;
    return s;
}

// host copies of the tables of one (logn, direction)
struct HostTables {
    int logn, inverse;
    Split sp;
    std::vector<u64> tw[3];     // one per non-final pass: [(k << logR) + r] = w_M^(k r) (pass 0 also carries 1/n on the inverse)
    std::vector<u64> twi[4];    // per pass with a digit of 2^5..2^9: w_L^(n2 k1) at [n2 * 16 + k1]
    u64 scale;                  // 1/n when inverse and single pass, else 1
};

inline HostTables make_tables(int logn, int inv, const Split *split = nullptr) {
    HostTables H;
    H.logn = logn;
    H.inverse = inv;
    H.sp = split ? *split : split_digits(logn);
    u64 n_inv = inverse(((u64)1 << logn) % gl::P);
    H.scale = (inv && H.sp.p == 1) ? n_inv : 1;
    int used = 0;
    for (int q = 0; q + 1 < H.sp.p; ++q) {
        int a = H.sp.a[q], logR = logn - used - a, logM = a + logR;
        u64 w = root_of_unity(logM);
        if (inv) w = inverse(w);
        std::vector<u64> &t = H.tw[q];
        t.resize((size_t)1 << logM);
        u64 first = (inv && q == 0) ? n_inv : 1;
        u64 wk = 1;                                   // w^k
        for (i64 k = 0; k < ((i64)1 << a); ++k) {
            u64 cur = first;
            u64 *row = t.data() + (k << logR);
            for (i64 r = 0; r < ((i64)1 << logR); ++r) { row[r] = cur; cur = gl::mul(cur, wk); }
            wk = gl::mul(wk, w);
        }
        used += a;
    }
    for (int q = 0; q < H.sp.p; ++q) {
        int a = H.sp.a[q];
        if (!fast_ok(a) && !fast512_ok(a)) continue;
        u64 w = root_of_unity(a);
        if (inv) w = inverse(w);
        std::vector<u64> &t = H.twi[q];
        t.resize((size_t)1 << a);
        u64 wn = 1;                                   // w^n2
        for (int n2 = 0; n2 < (1 << (a - FAST_A1)); ++n2) {
            u64 cur = 1;
            for (int k1 = 0; k1 < FAST_E1; ++k1) { t[n2 * FAST_E1 + k1] = cur; cur = gl::mul(cur, wn); }
            wn = gl::mul(wn, w);
        }
    }
    return H;
}

// w_4096^j (or inverse), j < 2048
inline std::vector<u64> make_twl(int inv) {
    std::vector<u64> t((size_t)1 << (TWL_LOG - 1));
    u64 w = root_of_unity(TWL_LOG);
    if (inv) w = inverse(w);
    u64 c = 1;
    for (auto &x : t) { x = c; c = gl::mul(c, w); }
    return t;
}

// pre[t][i] = (shift * w_N^t)^i, t < rho, i < K: the coefficient twist that moves the
// evaluation domain of coset t onto shift * w_N^t * <w_K>
// (layergkr/gpu.py:128-138 for t = 0; prover/core.py:702-718 for the rho cosets)
inline std::vector<u64> make_coset_pre(int logK, int logN, u64 shift) {
    int log_rho = logN - logK;
    std::vector<u64> t((size_t)1 << (logK + log_rho));
    u64 wN = root_of_unity(logN);
    u64 g = shift % gl::P;
    for (i64 c = 0; c < ((i64)1 << log_rho); ++c) {
        u64 cur = 1;
        u64 *row = t.data() + (c << logK);
        for (i64 i = 0; i < ((i64)1 << logK); ++i) { row[i] = cur; cur = gl::mul(cur, g); }
        g = gl::mul(g, wN);
    }
    return t;
}

// The coset factor (shift * w_N^t)^i of coefficient i = n1 K/16 + n2 R + r (first forward pass of K = L * L, R = L)
// splits into shift^i, w_N^(t r), w_N^(t n2 R) and w_N^(t n1 K/16).  The last is a power of two when 16 rho <= 64
// (w_64 = 2^39), the second rides on the inter-pass twiddle w_K^(k r) and the third on the inner twiddle
// w_L^(n2 k1); shift^i does not depend on the coset and is applied once.  Only the fused launch uses this form.
inline bool coset_mergeable(int logK, int logN) {
    const Split sp = split_digits(logK);
    const int log_rho = logN - logK;
    return sp.p == 2 && sp.a[0] == sp.a[1] && fast_ok(sp.a[0]) && log_rho >= 1 && log_rho <= 2;
}

// appended behind pre: twm[t][(k << logR) + r] (rho * K words), then twim[t][n2 * 16 + k1] (rho * L words)
inline void append_coset_merged(int logK, int logN, std::vector<u64> &t) {
    const int log_rho = logN - logK, a = logK / 2, logR = a;
    const i64 K = (i64)1 << logK, L = (i64)1 << a, R = (i64)1 << logR, rho = (i64)1 << log_rho;
    const HostTables H = make_tables(logK, 0);
    const u64 wN = root_of_unity(logN);
    const size_t base = t.size();
    t.resize(base + (size_t)(rho * K + rho * L));
    u64 *twm = t.data() + base, *twim = twm + rho * K;
    for (i64 c = 0; c < rho; ++c) {
        const u64 wc = gl::pow(wN, (u64)c);                // w_N^t
        std::vector<u64> pr((size_t)R);                    // w_N^(t r)
        u64 cur = 1;
        for (i64 r = 0; r < R; ++r) { pr[(size_t)r] = cur; cur = gl::mul(cur, wc); }
        for (i64 k = 0; k < L; ++k)
            for (i64 r = 0; r < R; ++r) twm[c * K + (k << logR) + r] = gl::mul(H.tw[0][(size_t)((k << logR) + r)], pr[(size_t)r]);
        const u64 wr = gl::pow(wc, (u64)R);                // w_N^(t R)
        u64 pn = 1;                                        // w_N^(t n2 R)
        for (i64 n2 = 0; n2 < L / FAST_E1; ++n2) {
            for (int k1 = 0; k1 < FAST_E1; ++k1) twim[c * L + n2 * FAST_E1 + k1] = gl::mul(H.twi[0][(size_t)(n2 * FAST_E1 + k1)], pn);
            pn = gl::mul(pn, wr);
        }
    }
}

// device (or host) addresses of the tables of one (logn, direction)
struct Tables {
    Split sp;
    int logn;
    const u64 *tw[3];
    const u64 *twi[4];
    const u64 *twl;
    u64 scale;
    int inverse;
};

inline PassArgs base_pass(const Tables &T, int q, i64 n_rows) {
    PassArgs A{};
    int used = 0;
    for (int i = 0; i < q; ++i) used += T.sp.a[i];
    A.logn = T.logn;
    A.a = T.sp.a[q];
    A.is_final = (q == T.sp.p - 1);
    A.logR = T.logn - used - A.a;
    A.B = used;
    A.n_rows = n_rows;
    A.src_width = (i64)1 << T.logn;
    A.tw = A.is_final ? nullptr : T.tw[q];
    A.twl = T.twl;
    A.twi = T.twi[q];
    A.inverse = T.inverse;
    A.scale = A.is_final ? T.scale : 1;
    A.ndig = 0;
    if (A.is_final) {
        A.ndig = T.sp.p - 1;
        for (int i = 0; i < A.ndig; ++i) A.dig[i] = T.sp.a[i];
    }
    return A;
}

// In-place batched transform of m rows (row pitch = n) held at `buf`.
// Multi-pass sizes go buf -> ws -> ... -> buf, so ws must hold m*n elements.
inline void build_ntt_passes(const Tables &T, u64 *buf, u64 *ws, i64 m, std::vector<PassArgs> &out) {
    const i64 n = (i64)1 << T.logn;
    for (int q = 0; q < T.sp.p; ++q) {
        PassArgs A = base_pass(T, q, m);
        A.src = (q == 0) ? buf : ws;
        A.canon_src = (q == 0);
        A.dst = A.is_final ? buf : ws;
        A.src_row_stride = A.dst_row_stride = n;
        out.push_back(A);
    }
}

// The same transform for rows of 2^10 .. 2^12 points as the pass pair of one k_ntt_row launch (T: tables of
// row_split(logn)); no workspace.
inline void build_row_passes(const Tables &T, u64 *buf, i64 m, PassArgs &P0, PassArgs &P1) {
    const i64 n = (i64)1 << T.logn;
    P0 = base_pass(T, 0, m);
    P1 = base_pass(T, 1, m);
    P0.src = buf;
    P0.canon_src = 1;
    P0.dst = nullptr;                                      // the intermediate stays in LDS
    P1.src = nullptr;
    P1.dst = buf;
    P0.src_row_stride = P0.dst_row_stride = P1.src_row_stride = P1.dst_row_stride = n;
}

// Coset LDE of m rows:  in (m rows of `w` values, pitch in_stride)  ->  out (m, N).
//   inverse passes:  in -> [S] -> C           (values at w_K^c -> coefficients)
//   forward passes:  C -> [S_t, t < rho] -> out, coefficients twisted per coset by pre[t][i],
//                    cosets interleaved out[rho*k + t]
// Workspace: C = m*K elements, followed by S = rho*m*K elements when K needs more
// than one pass.
inline i64 lde_ws_elems(int logK, int logN, i64 m) {
    i64 K = (i64)1 << logK, rho = (i64)1 << (logN - logK);
    return split_digits(logK).p == 1 ? m * K : m * K * (1 + rho);
}

// in -> [inverse passes] -> coefficients -> [forward passes over rho cosets] -> out.
// The coefficients live in the workspace unless the caller wants them (coeffs != nullptr: the
// last inverse pass writes them there, row pitch coeffs_stride).  in_is_coeffs skips the
// inverse passes: `in` already holds coefficients (width w, the rest zero).  merged: the tables of
// append_coset_merged() for this (K, N, shift), used by the fused launch when there is one.
inline void build_lde_passes(const Tables &Ti, const Tables &Tf, const u64 *pre, int logN,
                             const u64 *in, i64 w, i64 in_stride, u64 *out, i64 out_stride,
                             u64 *ws, i64 m, std::vector<PassArgs> &passes,
                             u64 *coeffs = nullptr, i64 coeffs_stride = 0, bool in_is_coeffs = false,
                             bool allow_fuse = true, const u64 *merged = nullptr) {
    const int logK = Ti.logn, log_rho = logN - logK, p = Ti.sp.p;
    const i64 K = (i64)1 << logK;
    u64 *C = coeffs ? coeffs : ws, *S = ws + m * K;
    const i64 c_stride = coeffs ? coeffs_stride : K;
    // inverse: in -> S (plane 0) -> C
    for (int q = 0; q < p && !in_is_coeffs; ++q) {
        PassArgs A = base_pass(Ti, q, m);
        A.src = (q == 0) ? in : S;
        A.canon_src = (q == 0);
        A.src_row_stride = (q == 0) ? in_stride : K;
        A.src_width = (q == 0) ? w : K;
        A.dst = A.is_final ? C : S;
        A.dst_row_stride = A.is_final ? c_stride : K;
        passes.push_back(A);
    }
    if (!out) return;
    // forward over rho cosets
    for (int q = 0; q < p; ++q) {
        bool first = (q == 0), last = (q == p - 1);
        PassArgs A = base_pass(Tf, q, (first || last) ? m : (m << log_rho));
        A.log_rho = (first || last) ? log_rho : 0;     // middle passes see rho*m plain rows
        A.loop_cosets = first && !last;
        A.pre = first ? pre : nullptr;
        A.src = first ? (in_is_coeffs ? in : C) : S;
        A.src_row_stride = first ? (in_is_coeffs ? in_stride : c_stride) : K;
        if (first && in_is_coeffs) { A.src_width = w; A.canon_src = 1; }
        A.src_coset_stride = first ? 0 : m * K;
        A.dst = last ? out : S;
        A.dst_row_stride = last ? out_stride : K;
        A.dst_coset_stride = m * K;
        if (last && !first) A.log_rho = log_rho;
        passes.push_back(A);
    }
    // K = L * L: the last inverse pass and the first forward pass run as one launch and the coefficients stay in
    // registers.  The inverse intermediate then lives in the workspace's coefficient region (the forward planes
    // are written while other workgroups still read it), and the coefficients go to memory only for the caller.
    if (allow_fuse && !in_is_coeffs && p == 2) {
        PassArgs &I0 = passes[passes.size() - 4], &I1 = passes[passes.size() - 3], &F0 = passes[passes.size() - 2];
        PassArgs T0 = I0, T1 = I1;
        T0.dst = ws;
        T0.dst_row_stride = K;
        T1.src = ws;
        T1.src_row_stride = K;
        T1.dst = coeffs;                                   // null when the caller does not want them
        T1.dst_row_stride = coeffs ? coeffs_stride : K;
        if (passes_fusable(T1, F0)) {
            T1.fuse_next = 1;
            I0 = T0;
            I1 = T1;
            if (merged && coset_mergeable(logK, logN)) {   // tables of append_coset_merged()
                F0.twm = merged;
                F0.twim = merged + (K << log_rho);
                F0.merge_unit = 4 >> log_rho;
            }
        }
    }
}

}  // namespace ntt

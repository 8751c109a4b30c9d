// Multilinear sumcheck round kernels (prover side).
//
// The reference composes a round out of elementwise torch launches
// (layergkr/gpu.py:341-410): per evaluation point and factor a sub, a mul and an
// add launch, a product chain, a log-depth gl_sum, and a host sync per sample.
// Here one launch does the whole round: every thread takes an index i of the
// (folded) half-table, forms f(x) = f[i] + x (f[h+i] - f[i]) for x = 0..deg by
// repeated addition, multiplies the factors of every term and accumulates the
// deg+1 partial sums; wavefront shuffles, then LDS, then a second single-block
// launch over the per-block partials finish the reduction, so the only host
// round trip per round is the read-back of the deg+1 samples that the verifier
// coin needs.
//
// The fold by the previous challenge is fused into the same pass: thread i reads
// the four entries {i, i+h', h+i, h+i+h'} (h = old half, h' = h/2) of each table,
// writes the two folded values and immediately evaluates the next round on them.
// Per fused round a table is read once and its folded half written once.
//
// Variable order is most-significant first, pairs are (i, half + i)
// (layergkr/sumcheck.py:51-54).
#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "gl_field.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int MAX_BLOCKS = 2048;
constexpr int MAX_DEG = 7;                  // samples per round <= 8
constexpr int NSAMP = MAX_DEG + 1;
constexpr int REG_TABLES = 8;               // tables a thread can keep in registers

// A list of small numbers (< 256) inside a kernel argument, four to a 32-bit word.  An index that is the same for a
// whole wavefront is then a scalar load of the word and a scalar shift.  As `unsigned char[N]` the compiler fetched an
// entry with a byte load per lane from the argument segment: a round trip to memory in front of the table address, and
// so of the table loads, that depend on it -- once per term of a thread's walk over the sum.
template <int N>
struct Bytes {
    u32 w[(N + 3) / 4];
    __host__ __device__ __forceinline__ int operator[](int j) const { return (int)((w[j >> 2] >> ((j & 3) * 8)) & 0xFFu); }
    __host__ void set(int j, int v) {
        const int sh = (j & 3) * 8;
        w[j >> 2] = (w[j >> 2] & ~(0xFFu << sh)) | (((u32)v & 0xFFu) << sh);
    }
};

struct Desc {
    const u64 *src[VI_SC_MAX_TABLES];
    u64 *dst[VI_SC_MAX_TABLES];
    u64 coeff[VI_SC_MAX_TERMS];
    Bytes<VI_SC_MAX_TERMS + 1> term_off;
    Bytes<VI_SC_MAX_FACTORS> fidx;
    // Several terms are stored factored:
    //   S(x) = common(x) * ( c0 + sum_k lin_coeff[k] f_lin[k](x) + sum_k coeff[k] prod_j f_kj(x) )
    // where `common` is a table every term contains (eq(z, .) in a batched gate check, layergkr/relations.py:117-121;
    // -1 = none, the bracket alone), a term left without factors adds its coefficient to c0, a term left with one
    // factor is linear in x (its coefficient is applied once per pair to the value and the step of that factor,
    // not once per evaluation point), and coeff / term_off / fidx keep only the terms with two or more factors left.
    u64 lin_coeff[VI_SC_MAX_TERMS];
    Bytes<VI_SC_MAX_TERMS> lin_idx;
    u64 c0;
    int n_lin, common;
    int n_tables, n_terms, deg;
    int coeff_at_end;                       // single term: apply its coefficient in the final reduction
    u64 out_scale;                          // factor the finished samples are multiplied by (1 = none): the single
                                            // term's coefficient, or the first product term's coefficient of a
                                            // factored sum, whose other coefficients are divided by it
    int product;                            // one term whose factors are exactly the n_tables tables, once each
    int gate;                               // four tables [common, f0, f1, lin]: common * (f0 * f1 + lin_coeff[0] * lin)
    int skip1;                              // S(1) is not summed: it is claim - S(0) (the round's known total)
    u64 claim;                              // S(0) + S(1) when skip1
    int canon_src;                          // the fold reads caller data: words are reduced mod p on load (sub() and the
                                            // ladders want canonical operands); 0 for tables this library has folded
};

__device__ __forceinline__ u64 fold1(u64 lo, u64 hi, u64 r) { return gl::add(lo, gl::mul(r, gl::sub(hi, lo))); }

__device__ __forceinline__ u64 wave_sum(u64 v) {
    for (int off = 32; off > 0; off >>= 1) v = gl::addc(v, __shfl_xor(v, off, 64));
    return v;
}

// MODE 0: evaluate pairs (src[i], src[half+i]), i < half
// MODE 1: fold by r into dst (i < half), no evaluation
// MODE 2: fold by r and evaluate the next round: i < half/2
// U = indices per thread per loop trip: the evaluation-only round issues just two
// loads per table and index, so two indices are kept in flight to cover HBM latency.
// `direct`: a single-workgroup launch writes the finished samples itself (small rounds
// need no second launch).
// `flag`: when non-zero (and direct), out[NSAMP] = flag is stored after the samples have reached system scope, so a
// host that owns `out` as pinned memory can wait on that word instead of on the stream.
// PROD: the sum is a single product of all NT tables (a matmul contraction, eq * a * b, the
// three-factor benchmark instance): the term interpreter below -- scalar loads of the term
// description and a register picked by index per factor -- gives way to a fully unrolled product.
// NS: evaluation points the general path keeps per pair (4 when the degree is at most 3, else NSAMP)
// SHAPE 2: the hadamard gate batch eq * (a * b + c' * c) (layergkr/relations.py:104-124: eq * a * b - eq * c with the
// coefficients normalised on the host), tables ordered [eq, a, b, c] by the host: unrolled like the single product.
template <int NT, int MODE, int U, int SHAPE, int NS>
__global__ __launch_bounds__(BLOCK) void k_round(const Desc D, i64 half, u64 r, u64 *partial, u64 *out,
                                                 u64 scale, int direct, u64 flag) {
    constexpr bool PROD = SHAPE == 1, GATE = SHAPE == 2, FIXED = SHAPE != 0;
    __shared__ u64 red[BLOCK / 64][NSAMP];
    const i64 count = (MODE == 2) ? (half >> 1) : half;
    const i64 stride = (i64)gridDim.x * BLOCK;
    u64 acc[NSAMP];
#pragma unroll
    for (int x = 0; x < NSAMP; ++x) acc[x] = 0;

    // U = 2 (evaluation-only rounds): a thread takes the adjacent indices 2j, 2j + 1 and loads each table's two
    // lower and two upper words as one 16-byte access each (the host selects it only for even counts and 16-byte
    // aligned tables)
    const i64 trips = (U == 2) ? (count >> 1) : count;
    for (i64 i0 = (i64)blockIdx.x * BLOCK + threadIdx.x; i0 < trips; i0 += stride) {
      u64 lo_u[U][NT], hi_u[U][NT];
      if constexpr (U == 2) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (FIXED || t < D.n_tables) {
                const ulonglong2 lo2 = *reinterpret_cast<const ulonglong2 *>(D.src[t] + 2 * i0);
                const ulonglong2 hi2 = *reinterpret_cast<const ulonglong2 *>(D.src[t] + half + 2 * i0);
                lo_u[0][t] = gl::canon(lo2.x);
                lo_u[U - 1][t] = gl::canon(lo2.y);
                hi_u[0][t] = gl::canon(hi2.x);
                hi_u[U - 1][t] = gl::canon(hi2.y);
            }
        }
      }
#pragma unroll
      for (int u = 0; u < (U == 2 ? 0 : U); ++u) {
        const i64 i = i0;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (FIXED || t < D.n_tables) {
                const u64 *f = D.src[t];
                if (MODE == 0) {
                    // caller data: any 64-bit word is taken as its residue (the ladders below add canonical values)
                    lo_u[u][t] = gl::canon(f[i]);
                    hi_u[u][t] = gl::canon(f[half + i]);
                } else if (MODE == 1) {
                    u64 a0 = f[i], b0 = f[half + i];
                    if (D.canon_src) { a0 = gl::canon(a0); b0 = gl::canon(b0); }
                    D.dst[t][i] = fold1(a0, b0, r);
                } else {
                    const i64 h2 = half >> 1;
                    u64 a0 = f[i], a1 = f[i + h2], b0 = f[half + i], b1 = f[half + i + h2];
                    if (D.canon_src) { a0 = gl::canon(a0); a1 = gl::canon(a1); b0 = gl::canon(b0); b1 = gl::canon(b1); }
                    lo_u[u][t] = fold1(a0, b0, r);
                    hi_u[u][t] = fold1(a1, b1, r);
                    D.dst[t][i] = lo_u[u][t];
                    D.dst[t][i + h2] = hi_u[u][t];
                }
            }
        }
      }
      if (MODE == 1) continue;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        u64 (&lo)[NT] = lo_u[u];
        u64 (&hi)[NT] = hi_u[u];
        // f(x) for x = 0, 1, 2, ... by repeated addition of (hi - lo)
        u64 cur[NT], dif[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            if (FIXED || t < D.n_tables) { cur[t] = lo[t]; dif[t] = gl::sub(hi[t], lo[t]); }
        if constexpr (GATE) {
            // S(x) = eq(x) * (a(x) b(x) + c'(x)), c' = lin_coeff * c carried as value and step
            u64 lc = gl::mul(D.lin_coeff[0], cur[3]);
            const u64 ld = gl::mul(D.lin_coeff[0], dif[3]);
#pragma unroll
            for (int x = 0; x <= 3; ++x) {
                if (!(x == 1 && D.skip1)) {
                    const u64 inner = gl::addc(gl::mul(cur[1], cur[2]), lc);
                    acc[x] = gl::addc(acc[x], gl::mul(inner, cur[0]));
                }
                if (x < 3) {
                    // f(1) is the loaded upper value itself: the first step of the ladder costs nothing
#pragma unroll
                    for (int t = 0; t < 3; ++t) cur[t] = (x == 0) ? hi[t] : gl::addc(cur[t], dif[t]);
                    lc = gl::addc(lc, ld);
                }
            }
            continue;
        }
        if (PROD) {
#pragma unroll
            for (int x = 0; x <= NT; ++x) {
                if (!(x == 1 && D.skip1)) {
                    u64 prod = cur[0];
#pragma unroll
                    for (int t = 1; t < NT; ++t) prod = (t + 1 < NT) ? gl::mul_lazy(prod, cur[t]) : gl::mul(prod, cur[t]);
                    acc[x] = gl::addc(acc[x], NT == 1 ? gl::canon(prod) : prod);
                }
                if (x < NT) {
                    // f(1) is the loaded upper value itself: the first step of the ladder costs nothing
#pragma unroll
                    for (int t = 0; t < NT; ++t) cur[t] = (x == 0) ? hi[t] : gl::addc(cur[t], dif[t]);
                }
            }
            continue;
        }
        // General sums: the term description is walked once per pair, and each factor it names (a register
        // picked by a wave-uniform index) is applied to all evaluation points before the next one is
        // fetched, so the cost of interpreting is paid per factor and not per factor and point.
        u64 sx[NS];
        {
            // the terms that are linear in x, as value and step
            u64 lc = D.c0, ld = 0;
            for (int k = 0; k < D.n_lin; ++k) {
                const int t = D.lin_idx[k];
                const u64 c = D.lin_coeff[k];
                lc = gl::addc(lc, gl::mul(c, cur[t]));
                ld = gl::addc(ld, gl::mul(c, dif[t]));
            }
#pragma unroll
            for (int x = 0; x < NS; ++x) {
                sx[x] = lc;
                if (D.n_lin && x < D.deg) lc = gl::addc(lc, ld);
            }
        }
        for (int k = 0; k < D.n_terms; ++k) {
            // factors are canonical; the running products stay non-canonical words and are
            // reduced fully once, when the term is added
            u64 prod[NS];
            int j = D.term_off[k];
            const int j1 = D.term_off[k + 1];
            const u64 c = D.coeff[k];
            if (D.coeff_at_end || c == 1) {
                const int t = D.fidx[j++];
                u64 v = cur[t];
                const u64 d = dif[t];
#pragma unroll
                for (int x = 0; x < NS; ++x) {
                    prod[x] = v;
                    if (x < D.deg) v = gl::addc(v, d);
                }
            } else {
#pragma unroll
                for (int x = 0; x < NS; ++x) prod[x] = c;
            }
            for (; j < j1; ++j) {
                const int t = D.fidx[j];
                u64 v = cur[t];
                const u64 d = dif[t];
#pragma unroll
                for (int x = 0; x < NS; ++x) {
                    if (x <= D.deg && !(D.skip1 && x == 1)) prod[x] = gl::mul_lazy(prod[x], v);
                    if (x < D.deg) v = gl::addc(v, d);
                }
            }
#pragma unroll
            for (int x = 0; x < NS; ++x)
                if (x <= D.deg) sx[x] = gl::addc(sx[x], gl::canon(prod[x]));
        }
        if (D.common >= 0) {
            u64 v = cur[D.common];
            const u64 d = dif[D.common];
#pragma unroll
            for (int x = 0; x < NS; ++x) {
                if (x <= D.deg && !(D.skip1 && x == 1)) sx[x] = gl::mul(sx[x], v);
                if (x < D.deg) v = gl::addc(v, d);
            }
        }
#pragma unroll
        for (int x = 0; x < NS; ++x)
            if (x <= D.deg) acc[x] = gl::addc(acc[x], sx[x]);
      }
    }
    if (MODE == 1) return;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int x = 0; x < NSAMP; ++x) {
        u64 v = wave_sum(acc[x]);
        if (lane == 0) red[w][x] = v;
    }
    __syncthreads();
    if (!direct) {
        if (threadIdx.x < NSAMP) {
            u64 v = red[0][threadIdx.x];
            for (int i = 1; i < BLOCK / 64; ++i) v = gl::add(v, red[i][threadIdx.x]);
            partial[(i64)blockIdx.x * NSAMP + threadIdx.x] = v;
        }
        return;
    }
    // single workgroup: thread 0 finishes every sample, so that its one fence orders all of them before the flag
    if (threadIdx.x == 0) {
        u64 s0 = 0;
        for (int x = 0; x <= D.deg; ++x) {
            u64 v;
            if (D.skip1 && x == 1) {                     // S(1) = claim - S(0)
                v = gl::sub(D.claim, s0);
            } else {
                v = red[0][x];
                for (int i = 1; i < BLOCK / 64; ++i) v = gl::add(v, red[i][x]);
                if (scale != 1) v = gl::mul(v, scale);
            }
            if (x == 0) s0 = v;
            out[x] = v;
        }
        if (flag) {
            __threadfence_system();
            __hip_atomic_store(out + NSAMP, flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

// tables kept in memory: for problems with more than REG_TABLES distinct tables.
// The fold (if any) has already been done by k_round<*, 1>.
// A problem too large for one descriptor is evaluated as several launches over groups of its terms: each multiplies
// its block sums by its own `scale` and, from the second group on (`accumulate`), adds them to what the slots hold.
// Small rounds are bound by the latency of one thread's chain of loads (two per factor slot), so the grid's y dimension
// deals the terms out: workgroup row ty takes the terms k = ty (mod gridDim.y) of the bracket -- the constant c0 goes
// to row 0 -- and multiplies its share by the common factor; the shares add up in k_final like any other partials.
// a linear combination of tables: sum_k coeff[k] src[k]
constexpr int LIN_MAX = 128;
struct LinFoldDesc {
    const u64 *src[LIN_MAX];
    u64 coeff[LIN_MAX];
    int n;
};

// What k_eval_mem<*, true> does besides evaluating: it writes every table folded by the round's challenge, so
// that a round is one pass over the tables (read both halves, write the folded half) instead of an evaluation pass
// and a fold pass.  A table may be fetched several times on the walk over the terms; its fold is written where it is
// fetched LAST (wb_*), so that folding in place never shows a later fetch the folded value.  `virt`: one table of
// the descriptor that does not exist yet -- its two values of a pair are the linear combination V of other tables,
// formed on the spot (the single table that stands for all the terms linear under the common factor, see
// reduce_linear_terms), and its fold is written like any other.
struct FoldOut {
    u64 r;
    int virt;
    int wb_common;
    Bytes<VI_SC_MAX_TERMS> wb_lin;
    Bytes<VI_SC_MAX_FACTORS> wb_fac;
};

// NS: evaluation points kept per pair (4 when the degree is at most 3, else NSAMP).
// Sums of products are kept as plain five-word integers and reduced once (gl::wide_mul_acc): the linear part as
// L = sum_k c_k lo_k and H = sum_k c_k hi_k over the raw table words (its value is c0 + L at x = 0, c0 + H at x = 1 and
// moves by H - L per step: two multiply-accumulates per term and pair, no subtraction, no reduction of the words),
// a product term's last factor into the bracket of its point, the bracket times the common factor into the
// thread's sample.  D.skip1: S(1) is not summed (the proof's finishing kernel takes it from the claim).
// FOLD: see FoldOut (one row of workgroups only: a table's last fetch must belong to the thread that fetched it first).
// where the tables of a descriptor are: in memory at the descriptor's own addresses, or packed in LDS
struct TabGlobal {
    const Desc &D;
    __device__ __forceinline__ const u64 *src(int t) const { return D.src[t]; }
    __device__ __forceinline__ u64 *dst(int t) const { return D.dst[t]; }
    // a table word is fetched once per round (now and then a few times by the terms of one thread): streaming hint,
    // 1.72-1.75 -> 1.67-1.69 ms on the 97-table batch (the same hint in the register kernels' loads: no difference)
    static __device__ __forceinline__ u64 ld(const u64 *p) { return __builtin_nontemporal_load(p); }
};
struct TabLds {
    u64 *base;
    int pitch;                               // words between tables
    __device__ __forceinline__ const u64 *src(int t) const { return base + t * pitch; }
    __device__ __forceinline__ u64 *dst(int t) const { return base + t * pitch; }
    static __device__ __forceinline__ u64 ld(const u64 *p) { return *p; }
};

// Pair i of a round of `half` pairs: the samples of the factored sum into acc and, with FOLD, the tables folded by r
// (row ty of ny rows of workgroups takes its share of the terms).
// a thread's sample sums: five-word integers reduced at the end (k_tail_mem, whose threads see few pairs), or residues
// added up pair by pair (k_eval_mem: twelve registers fewer, for one more wavefront per SIMD)
__device__ __forceinline__ void acc_mul_add(gl::Wide &A, u64 a, u64 b) { gl::wide_mul_acc(A, a, b); }
__device__ __forceinline__ void acc_mul_add(u64 &A, u64 a, u64 b) { A = gl::mul_add(a, b, A); }

// SKIP: 1 = S(1) is not summed (the caller derives it from the round's known total), 0 = it is, -1 = as skip1 says
template <int NS, bool FOLD, int SKIP, class TAB, class ACC>
__device__ __forceinline__ void eval_mem_pair(const Desc &D, const FoldOut &W, const LinFoldDesc *V, const TAB &T, u64 r, int skip1_rt,
                                              i64 i, i64 half, int ty, int ny, ACC (&acc)[NS]) {
    const bool skip1 = SKIP < 0 ? skip1_rt != 0 : SKIP != 0;
    // the factored form described at Desc, every factor fetched from its table.  Loads go out in batches ahead
    // of the arithmetic that uses them (the common factor first, used last; four linear terms; two factor slots
    // of a product): one thread's loads are otherwise a chain of round trips to memory.  A slot past the end of
    // its list repeats a valid load (a cache hit) with coefficient 0 or is skipped by a wavefront-uniform test.
    u64 v_lo = 0, v_hi = 0;              // the virtual table's pair
    if (FOLD && W.virt >= 0) {
        gl::Wide L, H;
        gl::wide_zero(L);
        gl::wide_zero(H);
        for (int k0 = 0; k0 < V->n; k0 += 4) {
            u64 a[4], b[4], c[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const bool on = k0 + u < V->n;
                const u64 *f = V->src[on ? k0 + u : k0];
                a[u] = TAB::ld(&f[i]);
                b[u] = TAB::ld(&f[half + i]);
                c[u] = on ? V->coeff[k0 + u] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                gl::wide_mul_acc(L, c[u], a[u]);
                gl::wide_mul_acc(H, c[u], b[u]);
            }
        }
        v_lo = gl::wide_reduce(L);
        v_hi = gl::wide_reduce(H);
        T.dst(W.virt)[i] = gl::mul_add(r, gl::sub(v_hi, v_lo), v_lo);
    }
    u64 com_lo = 0, com_hi = 0;
    if (D.common >= 0) {
        if (FOLD && D.common == W.virt) {
            com_lo = v_lo;
            com_hi = v_hi;
        } else {
            const u64 *f = T.src(D.common);
            com_lo = TAB::ld(&f[i]);
            com_hi = TAB::ld(&f[half + i]);
        }
    }
    u64 lin[NS];
    {
        gl::Wide L, H;
        gl::wide_zero(L);
        gl::wide_zero(H);
        for (int k0 = ty; k0 < D.n_lin; k0 += 4 * ny) {
            u64 a[4], b[4], c[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = k0 + u * ny;
                const bool on = k < D.n_lin;
                const int t = D.lin_idx[on ? k : k0];
                if (FOLD && t == W.virt) {
                    a[u] = v_lo;
                    b[u] = v_hi;
                } else {
                    const u64 *f = T.src(t);
                    a[u] = TAB::ld(&f[i]);
                    b[u] = TAB::ld(&f[half + i]);
                }
                c[u] = on ? D.lin_coeff[k] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                gl::wide_mul_acc(L, c[u], a[u]);
                gl::wide_mul_acc(H, c[u], b[u]);
                if (FOLD) {
                    const int k = k0 + u * ny;
                    if (k < D.n_lin && W.wb_lin[k]) {
                        const u64 lo = gl::canon(a[u]), hi = gl::canon(b[u]);
                        T.dst(D.lin_idx[k])[i] = gl::mul_add(r, gl::sub(hi, lo), lo);
                    }
                }
            }
        }
        const u64 c0 = ty == 0 ? D.c0 : 0;
        const u64 l0 = gl::wide_reduce(L), l1 = gl::wide_reduce(H);
        const u64 ld = gl::sub(l1, l0);
        u64 lc = gl::addc(l0, c0);
#pragma unroll
        for (int x = 0; x < NS; ++x) {
            lin[x] = lc;
            if (D.n_lin && x + 1 < NS) lc = gl::addc(lc, ld);
        }
    }
    gl::Wide br[NS];                     // the product terms of the bracket, per point
#pragma unroll
    for (int x = 0; x < NS; ++x) gl::wide_zero(br[x]);
    for (int k = ty; k < D.n_terms; k += ny) {
        u64 prod[NS];
#pragma unroll
        for (int x = 0; x < NS; ++x) prod[x] = D.coeff[k];
        const int j1 = D.term_off[k + 1];
        for (int j = D.term_off[k]; j < j1; j += 2) {
            const bool two = j + 1 < j1;
            const int t0 = D.fidx[j], t1 = D.fidx[two ? j + 1 : j];
            u64 a0, b0, a1, b1;
            if (FOLD && t0 == W.virt) { a0 = v_lo; b0 = v_hi; }
            else { const u64 *f0 = T.src(t0); a0 = TAB::ld(&f0[i]); b0 = TAB::ld(&f0[half + i]); }
            if (FOLD && t1 == W.virt) { a1 = v_lo; b1 = v_hi; }
            else { const u64 *f1 = T.src(t1); a1 = TAB::ld(&f1[i]); b1 = TAB::ld(&f1[half + i]); }
            // the value of a factor at x = 0, 1, 2, ...: lo, hi, then steps of hi - lo
            u64 cur = gl::canon(a0), nxt = gl::canon(b0);
            u64 dif = gl::sub(nxt, cur);
            if (FOLD && W.wb_fac[j]) T.dst(t0)[i] = gl::mul_add(r, dif, cur);
            const bool last0 = !two && j + 1 == j1;
#pragma unroll
            for (int x = 0; x < NS; ++x) {
                if (x <= D.deg && !(skip1 && x == 1)) {
                    if (last0) gl::wide_mul_acc(br[x], prod[x], cur);
                    else prod[x] = gl::mul_lazy(prod[x], cur);
                }
                if (x + 1 < NS) cur = (x == 0) ? nxt : gl::addc(cur, dif);
            }
            if (two) {
                cur = gl::canon(a1);
                nxt = gl::canon(b1);
                dif = gl::sub(nxt, cur);
                if (FOLD && W.wb_fac[j + 1]) T.dst(t1)[i] = gl::mul_add(r, dif, cur);
                const bool last1 = j + 2 == j1;
#pragma unroll
                for (int x = 0; x < NS; ++x) {
                    if (x <= D.deg && !(skip1 && x == 1)) {
                        if (last1) gl::wide_mul_acc(br[x], prod[x], cur);
                        else prod[x] = gl::mul_lazy(prod[x], cur);
                    }
                    if (x + 1 < NS) cur = (x == 0) ? nxt : gl::addc(cur, dif);
                }
            }
        }
    }
    {
        u64 cur = 1, nxt = 1, dif = 0;
        if (D.common >= 0) {
            cur = gl::canon(com_lo);
            nxt = gl::canon(com_hi);
            dif = gl::sub(nxt, cur);
            if (FOLD && W.wb_common) T.dst(D.common)[i] = gl::mul_add(r, dif, cur);
        }
#pragma unroll
        for (int x = 0; x < NS; ++x) {
            if (x <= D.deg && !(skip1 && x == 1)) acc_mul_add(acc[x], gl::addc(lin[x], gl::wide_reduce(br[x])), cur);
            if (x + 1 < NS) cur = (x == 0) ? nxt : gl::addc(cur, dif);
        }
    }
}

// SKIP1: D.skip1, fixed at compile time (the sample at 1 and everything that leads to it are not in the kernel then)
template <int NS, bool FOLD, bool SKIP1>
__global__ __launch_bounds__(BLOCK) void k_eval_mem(const Desc D, const FoldOut W, const LinFoldDesc V, i64 half, u64 *partial,
                                                    int accumulate, u64 scale) {
    __shared__ u64 red[BLOCK / 64][NSAMP];
    const int ty = blockIdx.y, ny = gridDim.y;
    const i64 stride = (i64)gridDim.x * BLOCK;
    u64 acc[NS];
#pragma unroll
    for (int x = 0; x < NS; ++x) acc[x] = 0;
    const TabGlobal T{D};
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < half; i += stride)
        eval_mem_pair<NS, FOLD, SKIP1 ? 1 : 0>(D, W, &V, T, W.r, 0, i, half, ty, ny, acc);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        u64 v = wave_sum(acc[x]);
        if (lane == 0) red[w][x] = v;
    }
    __syncthreads();
    if (threadIdx.x < NSAMP) {
        u64 v = 0;
        if (threadIdx.x < NS) {
            v = red[0][threadIdx.x];
            for (int i = 1; i < BLOCK / 64; ++i) v = gl::add(v, red[i][threadIdx.x]);
            if (scale != 1) v = gl::mul(v, scale);
        }
        u64 *slot = partial + ((i64)blockIdx.y * gridDim.x + blockIdx.x) * NSAMP + threadIdx.x;
        *slot = accumulate ? gl::add(v, *slot) : v;
    }
}

// fold of many tables in one launch: blockIdx.y = table, the x dimension strides over the lower half
constexpr int FOLD_MANY = 64;
struct FoldDesc {
    const u64 *src[FOLD_MANY];
    u64 *dst[FOLD_MANY];
};
// canon_src: the tables are caller data, reduced mod p on load (the kernel is bound by memory either way)
__global__ __launch_bounds__(BLOCK) void k_fold_many(const FoldDesc F, i64 half, u64 r, int canon_src) {
    const u64 *src = F.src[blockIdx.y];
    u64 *dst = F.dst[blockIdx.y];
    const i64 stride = (i64)gridDim.x * BLOCK;
    i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x;
    for (; i + stride < half; i += 2 * stride) {         // two independent indices in flight
        u64 lo0 = src[i], hi0 = src[half + i];
        u64 lo1 = src[i + stride], hi1 = src[half + i + stride];
        if (canon_src) { lo0 = gl::canon(lo0); hi0 = gl::canon(hi0); lo1 = gl::canon(lo1); hi1 = gl::canon(hi1); }
        dst[i] = fold1(lo0, hi0, r);
        dst[i + stride] = fold1(lo1, hi1, r);
    }
    if (i < half) {
        u64 lo0 = src[i], hi0 = src[half + i];
        if (canon_src) { lo0 = gl::canon(lo0); hi0 = gl::canon(hi0); }
        dst[i] = fold1(lo0, hi0, r);
    }
}

// cross-block tree: one workgroup adds the per-block partials of every sample
// skip1: sample 1 was not summed; it is claim - sample 0
// flag: as in k_round
__global__ __launch_bounds__(BLOCK) void k_final(const u64 *partial, int nb, int deg, u64 scale, int skip1, u64 claim,
                                                 u64 *out, u64 flag) {
    __shared__ u64 red[BLOCK / 64];
    u64 s0 = 0;
    for (int x = 0; x <= deg; ++x) {
        if (skip1 && x == 1) {
            if (threadIdx.x == 0) out[1] = gl::sub(claim, s0);
            continue;
        }
        u64 acc = 0;
        for (int b = threadIdx.x; b < nb; b += BLOCK) acc = gl::addc(acc, partial[(i64)b * NSAMP + x]);
        acc = wave_sum(acc);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            u64 v = red[0];
            for (int i = 1; i < BLOCK / 64; ++i) v = gl::add(v, red[i]);
            v = scale == 1 ? v : gl::mul(v, scale);
            out[x] = v;
            if (x == 0) s0 = v;
        }
        __syncthreads();
    }
    if (flag && threadIdx.x == 0) {                      // every sample above was stored by this thread
        __threadfence_system();
        __hip_atomic_store(out + NSAMP, flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// Rewrites the terms of D (already validated and copied) into the factored form described at Desc.
void factor_terms(Desc &D, const int *term_off, const int *factor_idx, int n_terms) {
    // a table that occurs in every term
    for (int j = term_off[0]; j < term_off[1] && D.common < 0; ++j) {
        bool everywhere = true;
        for (int k = 1; k < n_terms && everywhere; ++k) {
            bool found = false;
            for (int i = term_off[k]; i < term_off[k + 1]; ++i) found = found || factor_idx[i] == factor_idx[j];
            everywhere = found;
        }
        if (everywhere) D.common = factor_idx[j];
    }
    int n_prod = 0, n_fac = 0;
    for (int k = 0; k < n_terms; ++k) {
        const u64 c = D.coeff[k];           // reads entry k before entry n_prod <= k is overwritten
        int rest[MAX_DEG], nr = 0;
        bool dropped = false;
        for (int i = term_off[k]; i < term_off[k + 1]; ++i) {
            if (!dropped && factor_idx[i] == D.common) { dropped = true; continue; }
            rest[nr++] = factor_idx[i];
        }
        if (nr == 0) {
            D.c0 = gl::add(D.c0, c);
        } else if (nr == 1) {
            D.lin_idx.set(D.n_lin, rest[0]);
            D.lin_coeff[D.n_lin++] = c;
        } else {
            D.coeff[n_prod] = c;
            D.term_off.set(n_prod, n_fac);
            for (int i = 0; i < nr; ++i) D.fidx.set(n_fac++, rest[i]);
            ++n_prod;
        }
    }
    D.term_off.set(n_prod, n_fac);
    D.n_terms = n_prod;
    // the first product term's coefficient leaves the sum: one multiplication per evaluation point less
    if (n_prod >= 1 && D.coeff[0] > 1) {
        const u64 s = D.coeff[0], s_inv = gl::inv(s);
        D.out_scale = s;
        D.coeff[0] = 1;
        for (int k = 1; k < n_prod; ++k) D.coeff[k] = gl::mul(D.coeff[k], s_inv);
        for (int k = 0; k < D.n_lin; ++k) D.lin_coeff[k] = gl::mul(D.lin_coeff[k], s_inv);
        D.c0 = gl::mul(D.c0, s_inv);
    }
}

int fill_desc(Desc &D, const uint64_t *const *src, uint64_t *const *dst, int n_tables, const int *term_off,
              const int *factor_idx, const uint64_t *coeffs, int n_terms, bool need_terms, const char *who,
              bool mem_path = false) {
    if (n_tables < 1 || n_tables > VI_SC_MAX_TABLES) return vi::fail(VI_EINVAL, "%s: n_tables = %d (1..%d)", who, n_tables, VI_SC_MAX_TABLES);
    D.n_tables = n_tables;
    for (int t = 0; t < n_tables; ++t) {
        if (!src[t] || (dst && !dst[t])) return vi::fail(VI_EINVAL, "%s: null table %d", who, t);
        D.src[t] = src[t];
        D.dst[t] = dst ? dst[t] : nullptr;
    }
    D.n_terms = 0;
    D.n_lin = 0;
    D.common = -1;
    D.c0 = 0;
    D.deg = 0;
    D.coeff_at_end = 0;
    D.out_scale = 1;
    D.product = 0;
    D.gate = 0;
    D.skip1 = 0;
    D.claim = 0;
    D.canon_src = 1;
    if (!need_terms) return VI_OK;
    if (n_terms < 1 || n_terms > VI_SC_MAX_TERMS) return vi::fail(VI_EINVAL, "%s: n_terms = %d (1..%d)", who, n_terms, VI_SC_MAX_TERMS);
    if (!term_off || !factor_idx || !coeffs) return vi::fail(VI_EINVAL, "%s: null term descriptor", who);
    if (term_off[0] != 0 || term_off[n_terms] > VI_SC_MAX_FACTORS) return vi::fail(VI_EINVAL, "%s: %d factors exceed %d", who, term_off[n_terms], VI_SC_MAX_FACTORS);
    D.n_terms = n_terms;
    for (int k = 0; k < n_terms; ++k) {
        int nf = term_off[k + 1] - term_off[k];
        if (nf < 1 || nf > MAX_DEG) return vi::fail(VI_EINVAL, "%s: term %d has %d factors (1..%d)", who, k, nf, MAX_DEG);
        if (nf > D.deg) D.deg = nf;
        D.coeff[k] = coeffs[k] % gl::P;
        D.term_off.set(k, term_off[k]);
    }
    D.term_off.set(n_terms, term_off[n_terms]);
    for (int j = 0; j < term_off[n_terms]; ++j) {
        if (factor_idx[j] < 0 || factor_idx[j] >= n_tables) return vi::fail(VI_EINVAL, "%s: factor index %d out of range", who, factor_idx[j]);
        D.fidx.set(j, factor_idx[j]);
    }
    D.coeff_at_end = (n_terms == 1);
    if (n_terms == 1 && n_tables <= REG_TABLES && !mem_path) D.out_scale = D.coeff[0];     // k_eval_mem applies it per term instead
    if (n_terms == 1 && term_off[1] == n_tables && n_tables <= 4) {
        unsigned seen = 0;
        for (int j = 0; j < n_tables; ++j) seen |= 1u << factor_idx[j];
        D.product = (seen == (1u << n_tables) - 1);
    }
    if (n_terms >= 2) factor_terms(D, term_off, factor_idx, n_terms);
    if (mem_path) return VI_OK;             // k_eval_mem walks the terms by index: no fixed shapes, no table order
    // the hadamard gate batch: four distinct tables, common * (f0 * f1 + c * lin).  The tables are put in that order
    // (sources and destinations together), so the kernel needs no indices.
    if (n_terms >= 2 && n_tables == 4 && D.common >= 0 && D.n_terms == 1 && D.term_off[1] == 2 && D.n_lin == 1 &&
        D.c0 == 0 && D.coeff[0] == 1) {
        const int order[4] = {D.common, D.fidx[0], D.fidx[1], D.lin_idx[0]};
        unsigned seen = 0;
        for (int t = 0; t < 4; ++t) seen |= 1u << order[t];
        if (seen == 0xFu) {
            const u64 *s4[4];
            u64 *d4[4];
            for (int t = 0; t < 4; ++t) { s4[t] = D.src[order[t]]; d4[t] = D.dst[order[t]]; }
            for (int t = 0; t < 4; ++t) { D.src[t] = s4[t]; D.dst[t] = d4[t]; }
            D.gate = 1;
        }
    }
    return VI_OK;
}

inline int blocks_for(i64 count) {
    i64 b = (count + BLOCK - 1) / BLOCK;
    return (int)(b < 1 ? 1 : (b > MAX_BLOCKS ? MAX_BLOCKS : b));
}

// rounds this small run as ONE workgroup that also finishes the reduction
constexpr i64 DIRECT_MAX = 256;     // one loop trip per thread

// The round kernels are grid-stride loops: a grid larger than what is resident at once
// would run its surplus workgroups as a second, mostly empty wave (measured: 8 waves
// per SIMD requested, 7 resident -> almost 2x the time).  So the grid is capped at the
// kernel's own occupancy times the CU count.
// max_per_cu: the fused fold + evaluate round streams four runs per table and is faster with at most five
// workgroups per CU than with the seven or eight its registers would allow (rounds 1-3 of the 3 x 2^26 proof:
// 5,140 / 4,870 / 4,520 GB/s against 4,850 / 4,560 / 4,200); the evaluation-only round wants all it can get.
template <typename K>
int resident_blocks(K kernel, int max_per_cu) {
    int per_cu = 0, dev = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, BLOCK, 0) != hipSuccess || per_cu < 1) per_cu = 4;
    if (per_cu > max_per_cu) per_cu = max_per_cu;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
        cus = 256;
    int nb = per_cu * cus;
    return nb > MAX_BLOCKS ? MAX_BLOCKS : nb;
}

template <int NT, int MODE, int U, int SHAPE, int NS>
int launch_kp(const Desc &D, i64 half, u64 r, u64 *partial, int nb, u64 *out, u64 scale, int direct, u64 flag, hipStream_t s) {
    // per instantiation and device, looked up on first use there (devices of one process may differ)
    static std::mutex mu;
    static int caps[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int cap;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!caps[dev]) caps[dev] = resident_blocks(k_round<NT, MODE, U, SHAPE, NS>, MODE == 2 ? 5 : 64);
        cap = caps[dev];
    }
    if (nb > cap) nb = cap;
    hipLaunchKernelGGL((k_round<NT, MODE, U, SHAPE, NS>), dim3(nb), dim3(BLOCK), 0, s, D, half, r, partial, out, scale, direct, flag);
    return nb;
}

template <int NT, int MODE, int U>
int launch_k(const Desc &D, i64 half, u64 r, u64 *partial, int nb, u64 *out, u64 scale, int direct, u64 flag, hipStream_t s) {
    if (MODE != 1 && NT <= 4 && D.product && D.n_tables == NT)
        return launch_kp<NT, MODE, U, (MODE != 1 && NT <= 4) ? 1 : 0, NSAMP>(D, half, r, partial, nb, out, scale, direct, flag, s);
    if (MODE != 1 && NT == 4 && D.gate && D.n_tables == 4)
        return launch_kp<NT, MODE, U, (MODE != 1 && NT == 4) ? 2 : 0, NSAMP>(D, half, r, partial, nb, out, scale, direct, flag, s);
    if (MODE != 1 && D.deg <= 3) return launch_kp<NT, MODE, U, 0, (MODE != 1 ? 4 : NSAMP)>(D, half, r, partial, nb, out, scale, direct, flag, s);
    return launch_kp<NT, MODE, U, 0, NSAMP>(D, half, r, partial, nb, out, scale, direct, flag, s);
}

template <int MODE, int U>
int launch_round_u(const Desc &D, i64 half, u64 r, u64 *partial, int nb, u64 *out, u64 scale, int direct,
                   u64 flag, hipStream_t s) {
    int nt = D.n_tables;
    if (nt <= 1) return launch_k<1, MODE, U>(D, half, r, partial, nb, out, scale, direct, flag, s);
    if (nt <= 2) return launch_k<2, MODE, U>(D, half, r, partial, nb, out, scale, direct, flag, s);
    if (nt <= 3) return launch_k<3, MODE, U>(D, half, r, partial, nb, out, scale, direct, flag, s);
    if (nt <= 4) return launch_k<4, MODE, U>(D, half, r, partial, nb, out, scale, direct, flag, s);
    return launch_k<REG_TABLES, MODE, U>(D, half, r, partial, nb, out, scale, direct, flag, s);
}

// returns the number of workgroups actually launched (= partials written)
template <int MODE>
int launch_round(const Desc &D, i64 half, u64 r, u64 *partial, int nb, u64 *out, u64 scale, int direct,
                 u64 flag, hipStream_t s) {
    // two indices in flight for the load-light evaluation round on few tables
    if (MODE == 0 && D.n_tables <= 4 && nb > 1 && (half & 1) == 0) {
        bool aligned = true;
        for (int t = 0; t < D.n_tables; ++t) aligned = aligned && ((uintptr_t)D.src[t] & 15) == 0;
        if (aligned) return launch_round_u<MODE, 2>(D, half, r, partial, nb, out, scale, direct, flag, s);
    }
    return launch_round_u<MODE, 1>(D, half, r, partial, nb, out, scale, direct, flag, s);
}

// Where each table of D is fetched last on k_eval_mem's walk (linear terms, then the factor slots of the product terms,
// the common factor's values being used at the very end): W.wb_*.  Tables of D that no term fetches are returned in
// `unused` (they are folded by a launch of their own).
void fill_fold_flags(const Desc &D, FoldOut &W, std::vector<int> &unused) {
    for (int k = 0; k < VI_SC_MAX_TERMS; ++k) W.wb_lin.set(k, 0);
    for (int j = 0; j < VI_SC_MAX_FACTORS; ++j) W.wb_fac.set(j, 0);
    W.wb_common = 0;
    std::vector<int> last_lin(D.n_tables, -1), last_fac(D.n_tables, -1);
    for (int k = 0; k < D.n_lin; ++k) last_lin[D.lin_idx[k]] = k;
    const int nf = D.n_terms > 0 ? D.term_off[D.n_terms] : 0;
    for (int j = 0; j < nf; ++j) last_fac[D.fidx[j]] = j;
    unused.clear();
    for (int t = 0; t < D.n_tables; ++t) {
        if (t == W.virt) continue;                       // written where it is formed
        if (t == D.common) W.wb_common = 1;
        else if (last_fac[t] >= 0) W.wb_fac.set(last_fac[t], 1);
        else if (last_lin[t] >= 0) W.wb_lin.set(last_lin[t], 1);
        else unused.push_back(t);
    }
}

// k_eval_mem over `half` pairs: returns the number of partial slots written (x workgroups times term rows).
// W != NULL: the launch also writes every table folded by W->r (D.dst), see FoldOut.
// one instantiation of k_eval_mem over a grid-stride loop: no more workgroups than are resident at once (see
// resident_blocks), looked up per instantiation and device
template <int NS, bool FOLD, bool SKIP1>
int launch_eval_mem_as(const Desc &D, const FoldOut &w, const LinFoldDesc &v, i64 half, u64 *partial, int accumulate, u64 scale,
                       hipStream_t s) {
    static std::mutex mu;
    static int caps[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int cap;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!caps[dev]) caps[dev] = resident_blocks(k_eval_mem<NS, FOLD, SKIP1>, 64);
        cap = caps[dev];
    }
    int nbx = blocks_for(half);
    if (nbx > cap) nbx = cap;
    int ny = 1;
    if (!FOLD)
        while (ny < 16 && nbx * ny * 2 <= 1024) ny *= 2;     // deal the terms out while the grid is below ~4 workgroups per CU
    const dim3 grid(nbx, ny), block(BLOCK);
    hipLaunchKernelGGL((k_eval_mem<NS, FOLD, SKIP1>), grid, block, 0, s, D, w, v, half, partial, accumulate, scale);
    return nbx * ny;
}

int launch_eval_mem(const Desc &D, i64 half, u64 *partial, int accumulate, u64 scale, hipStream_t s,
                    const FoldOut *W = nullptr, const LinFoldDesc *V = nullptr) {
    static const FoldOut no_fold = {};
    static const LinFoldDesc no_virt = {};
    const FoldOut &w = W ? *W : no_fold;
    const LinFoldDesc &v = V ? *V : no_virt;
    switch ((W ? 4 : 0) + (D.deg <= 3 ? 2 : 0) + (D.skip1 ? 1 : 0)) {
        case 7: return launch_eval_mem_as<4, true, true>(D, w, v, half, partial, accumulate, scale, s);
        case 6: return launch_eval_mem_as<4, true, false>(D, w, v, half, partial, accumulate, scale, s);
        case 5: return launch_eval_mem_as<NSAMP, true, true>(D, w, v, half, partial, accumulate, scale, s);
        case 4: return launch_eval_mem_as<NSAMP, true, false>(D, w, v, half, partial, accumulate, scale, s);
        case 3: return launch_eval_mem_as<4, false, true>(D, w, v, half, partial, accumulate, scale, s);
        case 2: return launch_eval_mem_as<4, false, false>(D, w, v, half, partial, accumulate, scale, s);
        case 1: return launch_eval_mem_as<NSAMP, false, true>(D, w, v, half, partial, accumulate, scale, s);
        default: return launch_eval_mem_as<NSAMP, false, false>(D, w, v, half, partial, accumulate, scale, s);
    }
}

// fold `n` tables by r: up to REG_TABLES through the register kernel, more through k_fold_many (FOLD_MANY per launch)
int fold_tables(const uint64_t *const *src, uint64_t *const *dst, int n, i64 half, u64 r, hipStream_t s, int canon_src = 1) {
    for (int t = 0; t < n; ++t)
        if (!src[t] || !dst[t]) return vi::fail(VI_EINVAL, "vi_sumcheck_fold_eval: null table %d", t);
    int nbx = blocks_for((half + 1) / 2);
    for (int t0 = 0; t0 < n; t0 += FOLD_MANY) {
        const int cnt = (n - t0 < FOLD_MANY) ? (n - t0) : FOLD_MANY;
        FoldDesc F;
        for (int t = 0; t < FOLD_MANY; ++t) {
            F.src[t] = t < cnt ? src[t0 + t] : nullptr;
            F.dst[t] = t < cnt ? dst[t0 + t] : nullptr;
        }
        // a few thousand workgroups fill the chip; beyond that a workgroup takes more indices
        int bx = nbx;
        while (bx > 1 && (i64)bx * cnt > 8192) bx = (bx + 1) / 2;
        hipLaunchKernelGGL(k_fold_many, dim3(bx, cnt), dim3(BLOCK), 0, s, F, half, r, canon_src);
        VI_LAUNCH_CHECK("sumcheck fold (many tables)");
    }
    return VI_OK;
}

// ---- problems beyond one descriptor -------------------------------------------------------------------------
// A descriptor travels to the kernel by value, which bounds it (VI_SC_MAX_TABLES / _TERMS / _FACTORS).  A larger
// sum -- the batched gate check of a whole layer (layergkr/relations.py:104-124) has a few tables per gate and
// eq(z, .) in every term -- is cut into groups of consecutive terms that each fit one descriptor; the groups are
// evaluated one launch each over tables in memory and add into the same per-workgroup slots.

struct TermGroup {
    std::vector<int> tables;                // indices into the caller's table list, in order of first use
    std::vector<int> term_off, fidx;        // the group's terms over positions in `tables`
    std::vector<u64> coeffs;
};

inline bool fits_one_desc(int n_tables, const int *term_off, int n_terms) {
    return n_tables <= VI_SC_MAX_TABLES && n_terms <= VI_SC_MAX_TERMS && term_off && term_off[0] == 0 &&
           term_off[n_terms] <= VI_SC_MAX_FACTORS;
}

// argument checks for a term list of any length; *deg = the largest factor count
int check_terms(const char *who, const uint64_t *const *tables, int n_tables, const int *term_off, const int *factor_idx,
                const uint64_t *coeffs, int n_terms, int *deg) {
    if (n_tables < 1 || !tables) return vi::fail(VI_EINVAL, "%s: n_tables = %d", who, n_tables);
    for (int t = 0; t < n_tables; ++t)
        if (!tables[t]) return vi::fail(VI_EINVAL, "%s: null table %d", who, t);
    if (n_terms < 1) return vi::fail(VI_EINVAL, "%s: n_terms = %d", who, n_terms);
    if (!term_off || !factor_idx || !coeffs) return vi::fail(VI_EINVAL, "%s: null term descriptor", who);
    if (term_off[0] != 0) return vi::fail(VI_EINVAL, "%s: term_off[0] = %d", who, term_off[0]);
    *deg = 0;
    for (int k = 0; k < n_terms; ++k) {
        const int nf = term_off[k + 1] - term_off[k];
        if (nf < 1 || nf > MAX_DEG) return vi::fail(VI_EINVAL, "%s: term %d has %d factors (1..%d)", who, k, nf, MAX_DEG);
        if (nf > *deg) *deg = nf;
    }
    for (int j = 0; j < term_off[n_terms]; ++j)
        if (factor_idx[j] < 0 || factor_idx[j] >= n_tables) return vi::fail(VI_EINVAL, "%s: factor index %d out of range", who, factor_idx[j]);
    return VI_OK;
}

// consecutive terms, as many per group as one descriptor holds (a single term always fits: <= MAX_DEG factors)
void split_terms(int n_tables, const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms,
                 std::vector<TermGroup> &groups) {
    std::vector<int> local(n_tables, -1);
    groups.clear();
    groups.emplace_back();
    groups.back().term_off.push_back(0);
    for (int k = 0; k < n_terms; ++k) {
        const int nf = term_off[k + 1] - term_off[k];
        for (int attempt = 0;; ++attempt) {
            TermGroup &G = groups.back();
            int fresh = 0;
            for (int j = term_off[k]; j < term_off[k + 1]; ++j) {
                bool earlier = false;
                for (int i = term_off[k]; i < j; ++i) earlier = earlier || factor_idx[i] == factor_idx[j];
                if (local[factor_idx[j]] < 0 && !earlier) ++fresh;
            }
            const bool fits = (int)G.coeffs.size() < VI_SC_MAX_TERMS && (int)G.fidx.size() + nf <= VI_SC_MAX_FACTORS &&
                              (int)G.tables.size() + fresh <= VI_SC_MAX_TABLES;
            if (fits || attempt == 1) break;
            for (int t : G.tables) local[t] = -1;          // close the group, open the next
            groups.emplace_back();
            groups.back().term_off.push_back(0);
        }
        TermGroup &G = groups.back();
        for (int j = term_off[k]; j < term_off[k + 1]; ++j) {
            const int t = factor_idx[j];
            if (local[t] < 0) {
                local[t] = (int)G.tables.size();
                G.tables.push_back(t);
            }
            G.fidx.push_back(local[t]);
        }
        G.term_off.push_back((int)G.fidx.size());
        G.coeffs.push_back(coeffs[k]);
    }
}

// samples of sum over all groups at x = 0..deg from `tables` (pairs (i, half + i)); partial: MAX_BLOCKS * NSAMP words.
// nb_out != NULL: the per-workgroup sums are left in `partial` (*nb_out rows) for a later kernel to add up.
int eval_groups(const char *who, const uint64_t *const *tables, const std::vector<TermGroup> &groups, int deg, i64 half,
                u64 *partial, u64 *out_samples, u64 flag, hipStream_t s, int *nb_out = nullptr, int skip1 = 0) {
    int nb = 0;
    for (size_t g = 0; g < groups.size(); ++g) {
        const TermGroup &G = groups[g];
        const uint64_t *src[VI_SC_MAX_TABLES];
        for (size_t t = 0; t < G.tables.size(); ++t) src[t] = tables[G.tables[t]];
        Desc D;
        int rc = fill_desc(D, src, nullptr, (int)G.tables.size(), G.term_off.data(), G.fidx.data(), G.coeffs.data(),
                           (int)G.coeffs.size(), true, who, true);
        if (rc) return rc;
        D.deg = deg;                        // every group yields all the samples of the whole sum
        D.skip1 = skip1;
        nb = launch_eval_mem(D, half, partial, g > 0 ? 1 : 0, D.out_scale, s);    // the same grid for every group
        VI_LAUNCH_CHECK("sumcheck eval (term group)");
    }
    if (nb_out) {
        *nb_out = nb;
        return VI_OK;
    }
    hipLaunchKernelGGL(k_final, dim3(1), dim3(BLOCK), 0, s, (const u64 *)partial, nb, deg, (u64)1, 0, (u64)0, out_samples, flag);
    VI_LAUNCH_CHECK("sumcheck final");
    return VI_OK;
}

}  // namespace

extern "C" {

size_t vi_sumcheck_workspace_bytes(void) { return (size_t)MAX_BLOCKS * NSAMP * sizeof(u64); }

namespace {

int sumcheck_eval_on(const char *who, const uint64_t *const *tables, int n_tables, int64_t half, const int *term_off,
                     const int *factor_idx, const uint64_t *coeffs, int n_terms, uint64_t *out_samples, u64 *partial,
                     u64 flag, void *stream, const std::vector<TermGroup> *groups = nullptr, bool may_split = true) {
    if (half < 1) return vi::fail(VI_EINVAL, "%s: half = %lld", who, (long long)half);
    if (!out_samples) return vi::fail(VI_EINVAL, "%s: null out_samples", who);
    hipStream_t s = (hipStream_t)stream;
    if (may_split && n_terms >= 1 && term_off && !fits_one_desc(n_tables, term_off, n_terms)) {
        int deg = 0;
        int rc = check_terms(who, tables, n_tables, term_off, factor_idx, coeffs, n_terms, &deg);
        if (rc) return rc;
        std::vector<TermGroup> mine;
        if (!groups) {
            split_terms(n_tables, term_off, factor_idx, coeffs, n_terms, mine);
            groups = &mine;
        }
        return eval_groups(who, tables, *groups, deg, half, partial, out_samples, flag, s);
    }
    Desc D;
    int rc = fill_desc(D, tables, nullptr, n_tables, term_off, factor_idx, coeffs, n_terms, true, who);
    if (rc) return rc;
    int nb = blocks_for(half);
    const u64 scale = D.out_scale;
    if (n_tables <= REG_TABLES && half <= DIRECT_MAX) {
        launch_round<0>(D, half, 0, partial, 1, out_samples, scale, 1, flag, s);
        VI_LAUNCH_CHECK("sumcheck eval");
        return VI_OK;
    }
    if (n_tables <= REG_TABLES) nb = launch_round<0>(D, half, 0, partial, nb, nullptr, 1, 0, 0, s);
    else nb = launch_eval_mem(D, half, partial, 0, 1, s);
    VI_LAUNCH_CHECK("sumcheck eval");
    hipLaunchKernelGGL(k_final, dim3(1), dim3(BLOCK), 0, s, (const u64 *)partial, nb, D.deg, scale, 0, (u64)0, out_samples, flag);
    VI_LAUNCH_CHECK("sumcheck final");
    return VI_OK;
}

}  // namespace

int vi_sumcheck_eval(const uint64_t *const *tables, int n_tables, int64_t half, const int *term_off,
                     const int *factor_idx, const uint64_t *coeffs, int n_terms,
                     uint64_t *out_samples, void *ws, size_t ws_bytes, void *stream) {
    if (!ws || ws_bytes < vi_sumcheck_workspace_bytes()) return vi::fail(VI_ENOMEM, "vi_sumcheck_eval: workspace below %zu bytes", vi_sumcheck_workspace_bytes());
    return sumcheck_eval_on("vi_sumcheck_eval", tables, n_tables, half, term_off, factor_idx, coeffs, n_terms, out_samples,
                            (u64 *)ws, 0, stream);
}

// The per-workgroup partial sums of vi_sumcheck_eval_static: MAX_BLOCKS x NSAMP words (128 KiB) per GPU for the
// life of the process.  In host code this name is only a handle for hipGetSymbolAddress; kernels get the address.
static __device__ __align__(256) u64 scratch[MAX_BLOCKS * NSAMP];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
u64 *g_scratch_ptr[MAX_DEVICES] = {nullptr};

// device address of `scratch` on the current device, looked up once per device
int scratch_on_current_device(u64 **out) {
    int dev = 0;
    VI_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return vi::fail(VI_EINVAL, "vi_sumcheck_eval_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        VI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = (u64 *)p;
    }
    *out = g_scratch_ptr[dev];
    return VI_OK;
}
}  // namespace

int vi_sumcheck_eval_static(const uint64_t *const *tables, int n_tables, int64_t half, const int *term_off,
                            const int *factor_idx, const uint64_t *coeffs, int n_terms, uint64_t *out_samples,
                            void *stream) {
    if (half > VI_SC_STATIC_MAX_HALF)
        return vi::fail(VI_EINVAL, "vi_sumcheck_eval_static: half = %lld exceeds the limit of %lld pairs; use vi_sumcheck_eval",
                        (long long)half, (long long)VI_SC_STATIC_MAX_HALF);
    u64 *partial = nullptr;
    int rc = scratch_on_current_device(&partial);
    if (rc) return rc;
    // every workgroup of the launch overwrites its own NSAMP words and the final kernel reads exactly those, so
    // nothing of an earlier call has to be cleared
    return sumcheck_eval_on("vi_sumcheck_eval_static", tables, n_tables, half, term_off, factor_idx, coeffs, n_terms,
                            out_samples, partial, 0, stream, nullptr, false);
}

namespace {
int fold_eval_on(const uint64_t *const *src, uint64_t *const *dst, int n_tables, int64_t half, uint64_t r,
                 const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, const uint64_t *claim,
                 uint64_t *out_samples, void *ws, size_t ws_bytes, u64 flag, void *stream,
                 const std::vector<TermGroup> *groups = nullptr, int canon_src = 1);
}

int vi_sumcheck_fold_eval(const uint64_t *const *src, uint64_t *const *dst, int n_tables,
                          int64_t half, uint64_t r, const int *term_off, const int *factor_idx,
                          const uint64_t *coeffs, int n_terms, const uint64_t *claim,
                          uint64_t *out_samples, void *ws, size_t ws_bytes, void *stream) {
    return fold_eval_on(src, dst, n_tables, half, r, term_off, factor_idx, coeffs, n_terms, claim, out_samples, ws, ws_bytes,
                        0, stream);
}

namespace {
// flag: non-zero = the kernel that finishes the samples also stores out_samples[NSAMP] = flag after them
int fold_eval_on(const uint64_t *const *src, uint64_t *const *dst, int n_tables, int64_t half, uint64_t r,
                 const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, const uint64_t *claim,
                 uint64_t *out_samples, void *ws, size_t ws_bytes, u64 flag, void *stream,
                 const std::vector<TermGroup> *groups, int canon_src) {
    const bool eval = out_samples != nullptr;
    Desc D;
    if (!dst) return vi::fail(VI_EINVAL, "vi_sumcheck_fold_eval: null dst");
    if (!eval && src && n_tables > REG_TABLES) {
        // folding alone has no limit on the number of tables
        if (half < 1) return vi::fail(VI_EINVAL, "vi_sumcheck_fold_eval: half = %lld", (long long)half);
        return fold_tables(src, dst, n_tables, half, r % gl::P, (hipStream_t)stream, canon_src);
    }
    if (eval && src && n_terms >= 1 && term_off && !fits_one_desc(n_tables, term_off, n_terms)) {
        // more than one descriptor holds: fold every table, then evaluate the folded tables group by group
        const char *who = "vi_sumcheck_fold_eval";
        int deg = 0;
        int rc = check_terms(who, src, n_tables, term_off, factor_idx, coeffs, n_terms, &deg);
        if (rc) return rc;
        if (half < 2) return vi::fail(VI_EINVAL, "%s: no next round after half = %lld; pass out_samples = NULL", who, (long long)half);
        if (!ws || ws_bytes < vi_sumcheck_workspace_bytes()) return vi::fail(VI_ENOMEM, "%s: workspace below %zu bytes", who, vi_sumcheck_workspace_bytes());
        rc = fold_eval_on(src, dst, n_tables, half, r, nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr, 0, 0, stream,
                          nullptr, canon_src);
        if (rc) return rc;
        std::vector<TermGroup> mine;
        if (!groups) {
            split_terms(n_tables, term_off, factor_idx, coeffs, n_terms, mine);
            groups = &mine;
        }
        return eval_groups(who, (const uint64_t *const *)dst, *groups, deg, half >> 1, (u64 *)ws, out_samples, flag,
                           (hipStream_t)stream);
    }
    int rc = fill_desc(D, src, dst, n_tables, term_off, factor_idx, coeffs, n_terms, eval, "vi_sumcheck_fold_eval");
    if (rc) return rc;
    D.canon_src = canon_src;
    if (half < 1) return vi::fail(VI_EINVAL, "vi_sumcheck_fold_eval: half = %lld", (long long)half);
    if (eval && half < 2) return vi::fail(VI_EINVAL, "vi_sumcheck_fold_eval: no next round after half = 1; pass out_samples = NULL");
    if (eval && (!ws || ws_bytes < vi_sumcheck_workspace_bytes())) return vi::fail(VI_ENOMEM, "vi_sumcheck_fold_eval: workspace below %zu bytes", vi_sumcheck_workspace_bytes());
    r %= gl::P;
    // the tables-in-memory path sums every sample itself
    if (eval && claim && n_tables <= REG_TABLES) {
        D.skip1 = 1;
        D.claim = *claim % gl::P;
    }
    hipStream_t s = (hipStream_t)stream;
    if (!eval) {                                                  // at most REG_TABLES tables: one launch
        launch_round<1>(D, half, r, nullptr, blocks_for(half), nullptr, 1, 0, 0, s);
        VI_LAUNCH_CHECK("sumcheck fold");
        return VI_OK;
    }
    int nb;
    const u64 scale = D.out_scale;
    if (n_tables <= REG_TABLES) {
        if ((half >> 1) <= DIRECT_MAX) {
            launch_round<2>(D, half, r, (u64 *)ws, 1, out_samples, scale, 1, flag, s);
            VI_LAUNCH_CHECK("sumcheck fold+eval");
            return VI_OK;
        }
        nb = launch_round<2>(D, half, r, (u64 *)ws, blocks_for(half >> 1), nullptr, 1, 0, 0, s);
        VI_LAUNCH_CHECK("sumcheck fold+eval");
    } else {
        rc = fold_tables(src, dst, n_tables, half, r, s, canon_src);
        if (rc) return rc;
        Desc E = D;
        for (int t = 0; t < n_tables; ++t) E.src[t] = D.dst[t];
        nb = launch_eval_mem(E, half >> 1, (u64 *)ws, 0, 1, s);
        VI_LAUNCH_CHECK("sumcheck eval");
    }
    hipLaunchKernelGGL(k_final, dim3(1), dim3(BLOCK), 0, s, (const u64 *)ws, nb, D.deg, scale, D.skip1, D.claim, out_samples, flag);
    VI_LAUNCH_CHECK("sumcheck final");
    return VI_OK;
}

// Lagrange weights of the points 0..n-1: winv[i] = 1 / prod_{k != i} (i - k)
void lagrange_weights(int n, u64 *winv) {
    for (int i = 0; i < n; ++i) {
        u64 den = 1;
        for (int k = 0; k < n; ++k)
            if (k != i) den = gl::mul(den, gl::sub((u64)i, (u64)k));
        winv[i] = gl::pow(den, gl::P - 2);
    }
}

// value at x of the polynomial through (0, y[0]), ..., (n-1, y[n-1])
u64 interpolate_at(const u64 *y, const u64 *winv, int n, u64 x) {
    u64 total = 0;
    for (int i = 0; i < n; ++i) {
        u64 num = gl::mul(y[i], winv[i]);
        for (int k = 0; k < n; ++k)
            if (k != i) num = gl::mul(num, gl::sub(x, (u64)k));
        total = gl::add(total, num);
    }
    return total;
}

// Waits until the kernel that finishes a round's samples has stored `seq` behind them.  The word is polled (a stream
// synchronisation costs several microseconds more per round); every 2^16 polls the stream is queried, so a failed
// launch or a stream that drained without the store ends the wait with an error instead of spinning.
int wait_for_samples(const volatile u64 *flag, u64 seq, hipStream_t s) {
    for (unsigned spins = 1;; ++spins) {
        if (*flag == seq) break;
        __builtin_ia32_pause();
        if ((spins & 0xFFFF) == 0) {
            hipError_t e = hipStreamQuery(s);
            if (e == hipErrorNotReady) {
                (void)hipGetLastError();                 // "not ready" is no error for the launch checks that follow
                continue;
            }
            if (e != hipSuccess) return vi::fail(VI_EHIP, "vi_sumcheck_prove: %s while waiting for a round", hipGetErrorString(e));
            // drained: host memory that is not coherent while a kernel runs shows the store now
            if (*flag == seq) break;
            return vi::fail(VI_EHIP, "vi_sumcheck_prove: the stream drained without the round's samples");
        }
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    return VI_OK;
}
}  // namespace

int vi_sumcheck_prove(const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                      const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms,
                      vi_coin_fn coin, void *user, uint64_t *host_samples, size_t host_words, uint64_t *out_samples,
                      uint64_t *out_challenges, void *ws, size_t ws_bytes, void *stream) {
    if (size < 2 || (size & (size - 1))) return vi::fail(VI_EINVAL, "vi_sumcheck_prove: size must be a power of two >= 2, got %lld", (long long)size);
    if (!coin || !host_samples || !out_samples || !out_challenges || !work) return vi::fail(VI_EINVAL, "vi_sumcheck_prove: null pointer");
    if (host_words < VI_SC_HOST_WORDS) return vi::fail(VI_EINVAL, "vi_sumcheck_prove: host_samples holds %zu words, %d are needed", host_words, VI_SC_HOST_WORDS);
    if (!ws || ws_bytes < vi_sumcheck_workspace_bytes()) return vi::fail(VI_ENOMEM, "vi_sumcheck_prove: workspace below %zu bytes", vi_sumcheck_workspace_bytes());
    int deg = 0;
    int rc = check_terms("vi_sumcheck_prove", tables, n_tables, term_off, factor_idx, coeffs, n_terms, &deg);
    if (rc) return rc;
    for (int t = 0; t < n_tables; ++t)
        if (!work[t]) return vi::fail(VI_EINVAL, "vi_sumcheck_prove: null work buffer %d", t);
    // a sum beyond one descriptor is cut into groups of terms once for all rounds
    std::vector<TermGroup> groups;
    const bool split = !fits_one_desc(n_tables, term_off, n_terms);
    if (split) split_terms(n_tables, term_off, factor_idx, coeffs, n_terms, groups);
    const int ns = deg + 1;
    u64 winv[NSAMP];
    lagrange_weights(ns, winv);
    hipStream_t s = (hipStream_t)stream;
    int64_t half = size / 2;
    // host_samples[NSAMP] is the arrival word: round k's kernel stores (call number << 32) + k + 1 there behind its
    // samples, so that nothing an earlier call may have left in flight on this buffer can pass for a round of this one
    static std::atomic<u64> calls{0};
    const u64 tag = (calls.fetch_add(1) + 1) << 32;
    volatile u64 *arrived = host_samples + NSAMP;
    *arrived = 0;
    std::atomic_thread_fence(std::memory_order_seq_cst);
    rc = sumcheck_eval_on("vi_sumcheck_prove", tables, n_tables, half, term_off, factor_idx, coeffs, n_terms, host_samples,
                          (u64 *)ws, tag + 1, stream, split ? &groups : nullptr);
    if (rc) return rc;                       // nothing has been queued
    // From here on kernels may be in flight that write host_samples, work[] and ws: every error exit waits for
    // them to retire first, so that the caller may release those buffers as soon as the call has returned.
    const uint64_t *const *src = tables;
    int round = 0;
    for (;;) {
        rc = wait_for_samples(arrived, tag + (u64)round + 1, s);
        if (rc) break;
        u64 y[NSAMP];
        for (int x = 0; x < ns; ++x) y[x] = out_samples[(size_t)round * ns + x] = ((const volatile u64 *)host_samples)[x];
        uint64_t r = 0;
        if (coin(round, y, ns, &r, user)) {
            rc = vi::fail(VI_EINVAL, "vi_sumcheck_prove: coin callback asked to stop in round %d", round);
            break;
        }
        r %= gl::P;
        out_challenges[round] = r;
        ++round;
        if (half < 2) break;
        const uint64_t claim = interpolate_at(y, winv, ns, r);
        // only the first fold reads the caller's words; the work buffers hold canonical values
        rc = fold_eval_on(src, work, n_tables, half, r, term_off, factor_idx, coeffs, n_terms, &claim, host_samples, ws,
                          ws_bytes, tag + (u64)round + 1, stream, split ? &groups : nullptr, src == tables ? 1 : 0);
        if (rc) break;
        src = work;
        half /= 2;
    }
    // the last kernel retires before the caller releases its buffers
    const hipError_t e = hipStreamSynchronize(s);
    if (rc) return rc;
    if (e != hipSuccess) return vi::fail(VI_EHIP, "vi_sumcheck_prove: %s", hipGetErrorString(e));
    return VI_OK;
}

}  // extern "C"

#include "sumcheck_fast.hpp"

namespace {

// ---- the last rounds of a sum whose tables are read from memory, in one workgroup -----------------------------
// Once all tables of a round fit a workgroup's LDS together, one launch runs every remaining round: the tables are
// copied in (reduced mod p on the way); a round evaluates its pairs with the walk of k_eval_mem over the LDS copies
// (eval_mem_pair), the terms dealt over as many rows of threads as the workgroup has for the round's pairs -- a
// thread's walk over all terms is what a small round costs --, leaves ONE row of partial sums for k_finish, and then
// folds every table in place.  Small rounds are otherwise a fold launch and an evaluation launch each, both bound by
// launch latency.  The folded tables are not written back.
constexpr int TAIL_MEM_WORDS = 5632;            // 44 KiB of table words
constexpr int TAIL_MEM_ROUNDS = 9;              // nine or more tables share the words: a table has at most 2^9

// C: the proof's rounds; those before C.n_prior have left their partial sums in the workspace, the launch runs the
// rest and finishes the proof like k_finish (round 0 of a proof sums S(1), later ones do not).
// rows: power of two, rows of threads that have a share of the terms.
template <int NS>
__global__ __launch_bounds__(TAIL_THREADS) void k_tail_mem(const Desc D, const ChainDesc C, int rows, int size, const u64 *part, u64 *out) {
    __shared__ u64 tab[TAIL_MEM_WORDS];
    __shared__ u64 wsum[TAIL_MEM_ROUNDS][TAIL_THREADS / 64][NS];     // per round and wavefront
    __shared__ FinishShared sh;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    for (int t = 0; t < D.n_tables; ++t) {
        const u64 *src = D.src[t];
        for (int i = tid; i < size; i += TAIL_THREADS) tab[t * size + i] = gl::canon(src[i]);
    }
    finish_begin(C, part, sh);                             // the earlier rounds' sums and the Lagrange bases: sh.raw[k < n_prior], sh.lag
    __syncthreads();
    const TabLds T{tab, size};
    const FoldOut none = {};
    int half = size >> 1, log_half = 0;
    while ((1 << log_half) < half) ++log_half;
    for (int k = C.n_prior; k < C.n_rounds; ++k, half >>= 1, --log_half) {
        gl::Wide acc[NS];
#pragma unroll
        for (int x = 0; x < NS; ++x) gl::wide_zero(acc[x]);
        const int skip1 = k > 0 ? 1 : 0;
        if (half >= TAIL_THREADS) {
            for (int i = tid; i < half; i += TAIL_THREADS)
                eval_mem_pair<NS, false, -1>(D, none, nullptr, T, 0, skip1, (i64)i, (i64)half, 0, 1, acc);
        } else {
            // row ty of ny takes its share of the terms of pair i; no more rows than there are shares (every row pays
            // for the common factor and the reductions of its sums, and the workgroup has one CU to run on)
            int ny = TAIL_THREADS >> log_half;
            if (ny > rows) ny = rows;
            const int ty = tid >> log_half, i = tid & (half - 1);
            if (ty < ny) eval_mem_pair<NS, false, -1>(D, none, nullptr, T, 0, skip1, (i64)i, (i64)half, ty, ny, acc);
        }
        // the wavefront's sums of this round, the samples side by side so that their shuffles are in flight together;
        // the wavefronts are added up for all rounds at once behind the loop
        {
            u64 v[NS];
#pragma unroll
            for (int x = 0; x < NS; ++x) v[x] = gl::wide_reduce(acc[x]);
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                u64 o[NS];
#pragma unroll
                for (int x = 0; x < NS; ++x) o[x] = __shfl_xor(v[x], off, 64);
#pragma unroll
                for (int x = 0; x < NS; ++x) v[x] = gl::addc(v[x], o[x]);
            }
            if (lane == 0) {
#pragma unroll
                for (int x = 0; x < NS; ++x) wsum[k - C.n_prior][w][x] = v[x];
            }
        }
        __syncthreads();                                   // every read of this round's tables is done
        // fold in place: entry i of a table from entries i and half + i, each by one thread
        const u64 r = C.r[k];
        for (int e = tid; e < (D.n_tables << log_half); e += TAIL_THREADS) {
            const int t = e >> log_half, i = e & (half - 1);
            u64 *p = tab + t * size;
            const u64 lo = p[i];
            p[i] = gl::mul_add(r, gl::sub(p[half + i], lo), lo);
        }
        __syncthreads();
    }
    // the rounds of this launch: thread (round, sample) adds up the wavefronts
    {
        const int n_mine = C.n_rounds - C.n_prior;
        if (tid < n_mine * NS) {
            const int kk = tid / NS, x = tid - kk * NS;
            u64 v = wsum[kk][0][x];
            for (int j = 1; j < TAIL_THREADS / 64; ++j) v = gl::add(v, wsum[kk][j][x]);
            sh.raw[C.n_prior + kk][x] = v;
        }
    }
    __syncthreads();
    finish_samples(C, sh, out);
}

}  // namespace

extern "C" {

size_t vi_sumcheck_prove_coins_workspace_bytes(int64_t size) {
    if (size < 2 || (size & (size - 1))) return 0;
    return (size_t)(vi::ilog2(size) + 1) * MAX_BLOCKS * NSAMP * sizeof(u64);     // a region per round + one of single rows
}

namespace {

// ---- the terms that are linear once a common factor is taken out, as ONE table --------------------------------
// In a batched gate check (layergkr/relations.py:104-124) most terms are eq(z, .) times a single table (the c of a
// hadamard gate, the three tables of a rescale or affine gate, the b of a booleanity gate).  Folding is linear, so
// after round 0 all of them together are the one table lambda = sum_k c_k T_k, folded like any other: the tables
// that occur in no product are never read again, and every later round walks the product tables and lambda only.
// lambda is built already folded by the first challenge (half the size: it fits the work buffer of a table that
// has dropped out), from the raw words of its tables through five-word sums.

__global__ __launch_bounds__(BLOCK) void k_lin_fold(const LinFoldDesc F, i64 half, u64 r, u64 *dst, int accumulate) {
    const i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < half; i += stride) {
        gl::Wide L, H;
        gl::wide_zero(L);
        gl::wide_zero(H);
        for (int k0 = 0; k0 < F.n; k0 += 4) {            // four tables' loads in flight
            u64 a[4], b[4], c[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const bool on = k0 + u < F.n;
                const u64 *f = F.src[on ? k0 + u : k0];
                a[u] = f[i];
                b[u] = f[half + i];
                c[u] = on ? F.coeff[k0 + u] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                gl::wide_mul_acc(L, c[u], a[u]);
                gl::wide_mul_acc(H, c[u], b[u]);
            }
        }
        const u64 lo = gl::wide_reduce(L), hi = gl::wide_reduce(H);
        u64 v = gl::mul_add(r, gl::sub(hi, lo), lo);
        if (accumulate) v = gl::addc(v, dst[i]);
        dst[i] = v;
    }
}

// the rewritten problem: the tables that stay (indices into the caller's list) and lambda as the last table
struct LinearReduction {
    std::vector<int> keep;                   // tables folded one by one, ascending
    std::vector<int> lin_tab;                // tables of lambda
    std::vector<u64> lin_c;                  // and their coefficients
    int lambda_buf;                          // the table whose work buffer receives lambda
    std::vector<int> term_off, fidx;         // terms over positions in keep + [lambda]
    std::vector<u64> coeffs;
};

// false: nothing to gain (fewer than two linear tables, no table has dropped out, or the degree would change)
bool reduce_linear_terms(int n_tables, const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, int deg,
                         LinearReduction &R) {
    if (n_terms < 2) return false;
    // a table every term holds
    int common = -1;
    for (int j = term_off[0]; j < term_off[1] && common < 0; ++j) {
        bool everywhere = true;
        for (int k = 1; k < n_terms && everywhere; ++k) {
            bool found = false;
            for (int q = term_off[k]; q < term_off[k + 1]; ++q) found = found || factor_idx[q] == factor_idx[j];
            everywhere = found;
        }
        if (everywhere) common = factor_idx[j];
    }
    std::vector<u64> lin_coeff(n_tables, 0);
    std::vector<char> is_lin(n_tables, 0), in_kept(n_tables, 0);
    std::vector<int> kept_terms;
    for (int k = 0; k < n_terms; ++k) {
        int rest = -1, n_rest = 0;
        bool dropped = common < 0;
        for (int q = term_off[k]; q < term_off[k + 1]; ++q) {
            if (!dropped && factor_idx[q] == common) { dropped = true; continue; }
            rest = factor_idx[q];
            ++n_rest;
        }
        if (n_rest == 1) {
            lin_coeff[rest] = gl::add(lin_coeff[rest], coeffs[k] % gl::P);
            is_lin[rest] = 1;
        } else {
            kept_terms.push_back(k);
            for (int q = term_off[k]; q < term_off[k + 1]; ++q) in_kept[factor_idx[q]] = 1;
        }
    }
    if (common >= 0) in_kept[common] = 1;
    R.lin_tab.clear();
    R.lin_c.clear();
    R.lambda_buf = -1;
    for (int t = 0; t < n_tables; ++t) {
        if (!is_lin[t]) continue;
        R.lin_tab.push_back(t);
        R.lin_c.push_back(lin_coeff[t]);
        if (!in_kept[t] && R.lambda_buf < 0) R.lambda_buf = t;
    }
    if (R.lin_tab.size() < 2 || R.lambda_buf < 0) return false;
    const int lam_deg = common >= 0 ? 2 : 1;
    int new_deg = lam_deg;
    for (int k : kept_terms) new_deg = std::max(new_deg, term_off[k + 1] - term_off[k]);
    if (new_deg != deg) return false;
    std::vector<int> pos(n_tables, -1);
    R.keep.clear();
    for (int t = 0; t < n_tables; ++t)
        if (in_kept[t]) { pos[t] = (int)R.keep.size(); R.keep.push_back(t); }
    const int lambda_pos = (int)R.keep.size();
    R.term_off.assign(1, 0);
    R.fidx.clear();
    R.coeffs.clear();
    for (int k : kept_terms) {
        for (int q = term_off[k]; q < term_off[k + 1]; ++q) R.fidx.push_back(pos[factor_idx[q]]);
        R.term_off.push_back((int)R.fidx.size());
        R.coeffs.push_back(coeffs[k]);
    }
    if (common >= 0) R.fidx.push_back(pos[common]);
    R.fidx.push_back(lambda_pos);
    R.term_off.push_back((int)R.fidx.size());
    R.coeffs.push_back(1);
    return true;
}

int prove_coins_impl(const char *who, const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                     const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, int deg,
                     const uint64_t *challenges, uint64_t *samples, u64 *part, hipStream_t s, bool may_reduce);

// rounds of at least this many pairs evaluate and fold in one launch (k_eval_mem<*, true>, one row of workgroups);
// smaller ones are bound by the latency of a thread's walk and deal the terms over rows of workgroups instead
constexpr i64 FUSE_MIN_PAIRS = (i64)1 << 18;

// round 0 on the problem as given, then every later round on the rewritten one
int prove_coins_reduced(const char *who, const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                        const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, int deg,
                        const uint64_t *challenges, uint64_t *samples, u64 *part, hipStream_t s, const LinearReduction &R) {
    const i64 half = size / 2;
    const u64 r0 = challenges[0] % gl::P;
    u64 *lambda = work[R.lambda_buf];
    const int n_red = (int)R.keep.size() + 1;
    int rc = VI_OK;
    bool done = false;
    if (half >= FUSE_MIN_PAIRS && R.lin_tab.size() <= (size_t)LIN_MAX &&
        fits_one_desc(n_red, R.term_off.data(), (int)R.coeffs.size())) {
        // ONE pass over the caller's tables: round 0 of the rewritten sum -- lambda's two values of a pair are formed
        // from its tables on the spot -- and every table that stays, lambda included, written folded by r_0
        const uint64_t *src[VI_SC_MAX_TABLES];
        uint64_t *dst[VI_SC_MAX_TABLES];
        for (int q = 0; q + 1 < n_red; ++q) { src[q] = tables[R.keep[q]]; dst[q] = work[R.keep[q]]; }
        src[n_red - 1] = lambda;                           // never read: the table does not exist yet
        dst[n_red - 1] = lambda;
        Desc D;
        rc = fill_desc(D, src, dst, n_red, R.term_off.data(), R.fidx.data(), R.coeffs.data(), (int)R.coeffs.size(), true, who, true);
        if (rc) return rc;
        FoldOut W;
        W.r = r0;
        W.virt = n_red - 1;
        std::vector<int> unused;
        fill_fold_flags(D, W, unused);
        if (unused.empty()) {
            LinFoldDesc V;
            V.n = (int)R.lin_tab.size();
            for (int k = 0; k < LIN_MAX; ++k) {
                V.src[k] = k < V.n ? tables[R.lin_tab[k]] : nullptr;
                V.coeff[k] = k < V.n ? R.lin_c[k] : 0;
            }
            const int nb = launch_eval_mem(D, half, part, 0, 1, s, &W, &V);
            VI_LAUNCH_CHECK("sumcheck eval + fold (round 0)");
            hipLaunchKernelGGL(k_final, dim3(1), dim3(BLOCK), 0, s, (const u64 *)part, nb, deg, D.out_scale, 0, (u64)0, samples, (u64)0);
            VI_LAUNCH_CHECK("sumcheck final");
            done = true;
        }
    }
    if (!done) {
        rc = sumcheck_eval_on(who, tables, n_tables, half, term_off, factor_idx, coeffs, n_terms, samples, part, 0, (void *)s);
        if (rc) return rc;
        std::vector<const uint64_t *> src;
        std::vector<uint64_t *> dst;
        for (int t : R.keep) { src.push_back(tables[t]); dst.push_back(work[t]); }
        rc = fold_tables(src.data(), dst.data(), (int)src.size(), half, r0, s, 1);
        if (rc) return rc;
        for (size_t k0 = 0; k0 < R.lin_tab.size(); k0 += LIN_MAX) {
            LinFoldDesc F;
            F.n = (int)std::min<size_t>(LIN_MAX, R.lin_tab.size() - k0);
            for (int k = 0; k < LIN_MAX; ++k) {
                F.src[k] = k < F.n ? tables[R.lin_tab[k0 + k]] : nullptr;
                F.coeff[k] = k < F.n ? R.lin_c[k0 + k] : 0;
            }
            hipLaunchKernelGGL(k_lin_fold, dim3(blocks_for(half)), dim3(BLOCK), 0, s, F, half, r0, lambda, k0 > 0 ? 1 : 0);
            VI_LAUNCH_CHECK("sumcheck linear combination");
        }
    }
    // the rewritten problem lives in the work buffers and is folded in place from here on
    std::vector<const uint64_t *> rt;
    std::vector<uint64_t *> rw;
    for (int t : R.keep) { rt.push_back(work[t]); rw.push_back(work[t]); }
    rt.push_back(lambda);
    rw.push_back(lambda);
    return prove_coins_impl(who, rt.data(), rw.data(), (int)rt.size(), half, R.term_off.data(), R.fidx.data(), R.coeffs.data(),
                            (int)R.coeffs.size(), deg, challenges + 1, samples + NSAMP, part, s, false);
}

// all rounds of the sum over tables of `size` words; samples: log2(size) rows of NSAMP words
int prove_coins_impl(const char *who, const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                     const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms, int deg,
                     const uint64_t *challenges, uint64_t *samples, u64 *part, hipStream_t s, bool may_reduce) {
    const int v = vi::ilog2(size);
    int rc = VI_OK;
    ChainDesc C;
    for (int k = 0; k < MAX_ROUNDS; ++k) {
        C.r[k] = k < v ? challenges[k] % gl::P : 0;
        C.off[k] = 0;
        C.nb[k] = 0;
    }
    for (int x = 0; x < NSAMP; ++x) C.winv[x] = 0;
    lagrange_weights(deg + 1, C.winv);
    C.scale = 1;
    C.skip_mask = 0;
    C.inf_node = 0;
    C.dfact = 1;
    for (int x = 0; x < NSAMP; ++x) C.cinf[x] = 0;
    C.n_rounds = v;
    C.n_prior = v;
    C.deg = deg;

    // many terms that are a single table under the common factor: from round 1 on they are one table (needs a round
    // to fold into, so at least two rounds)
    if (may_reduce && v >= 2) {
        LinearReduction R;
        if (reduce_linear_terms(n_tables, term_off, factor_idx, coeffs, n_terms, deg, R))
            return prove_coins_reduced(who, tables, work, n_tables, size, term_off, factor_idx, coeffs, n_terms, deg, challenges,
                                       samples, part, s, R);
    }
    const bool split = !fits_one_desc(n_tables, term_off, n_terms);
    if (!split) {
        Desc D;
        rc = fill_desc(D, tables, work, n_tables, term_off, factor_idx, coeffs, n_terms, true, who);
        if (rc) return rc;
        // the shapes with a kernel of their own: several rounds per launch
        if ((D.product && n_tables <= 4) || D.gate) {
            FastDesc F;
            for (int t = 0; t < 4; ++t) {
                F.src[t] = t < n_tables ? D.src[t] : nullptr;
                F.dst[t] = t < n_tables ? D.dst[t] : nullptr;
            }
            F.lin_coeff = D.gate ? D.lin_coeff[0] : 1;
            C.scale = D.out_scale;
            if (D.gate) return prove_fast_shape<4, 2>(F, size, C, part, samples, s);
            switch (n_tables) {
                case 1: return prove_fast_shape<1, 1>(F, size, C, part, samples, s);
                case 2: return prove_fast_shape<2, 1>(F, size, C, part, samples, s);
                case 3: return prove_fast_shape<3, 1>(F, size, C, part, samples, s);
                default: return prove_fast_shape<4, 1>(F, size, C, part, samples, s);
            }
        }
        // a whole proof whose tables fit one workgroup's LDS together: one launch (k_tail_mem), whatever the table count
        if ((i64)n_tables * size <= TAIL_MEM_WORDS && v <= TAIL_MEM_ROUNDS) {
            Desc M;
            rc = fill_desc(M, tables, work, n_tables, term_off, factor_idx, coeffs, n_terms, true, who, true);
            if (rc) return rc;
            const int shares = std::max(std::max(M.n_terms, (M.n_lin + 3) / 4), 1);
            int rows = 1;
            while (rows < shares) rows <<= 1;
            C.scale = M.out_scale;
            C.n_prior = 0;
            for (int j = 1; j < v; ++j) C.skip_mask |= 1ull << j;
            if (M.deg <= 3) hipLaunchKernelGGL(k_tail_mem<4>, dim3(1), dim3(TAIL_THREADS), 0, s, M, C, rows, (int)size, (const u64 *)part, samples);
            else hipLaunchKernelGGL(k_tail_mem<NSAMP>, dim3(1), dim3(TAIL_THREADS), 0, s, M, C, rows, (int)size, (const u64 *)part, samples);
            VI_LAUNCH_CHECK("sumcheck in one workgroup");
            return VI_OK;
        }
        // any other sum of at most one descriptor: one launch per round, queued back to back
        i64 half = size / 2;
        unsigned off = 0;
        const bool regs = n_tables <= REG_TABLES;
        C.scale = D.out_scale;
        if (regs) {
            // the same sum as k_tail_mem reads it (a single term's coefficient per term there, at the end here: the
            // two must scale the samples alike for the tail to take over part of the way)
            Desc M;
            rc = fill_desc(M, tables, work, n_tables, term_off, factor_idx, coeffs, n_terms, true, who, true);
            if (rc) return rc;
            const bool tail_ok = M.out_scale == D.out_scale;
            for (int k = 0; k < v; ++k, half >>= 1) {
                int nb;
                if (k > 0 && tail_ok && (i64)n_tables * 2 * half <= TAIL_MEM_WORDS && v - k <= TAIL_MEM_ROUNDS) {
                    // every table of this round fits one workgroup's LDS: fold into place, then all remaining rounds
                    // in one launch
                    rc = fold_tables(k == 1 ? D.src : (const uint64_t *const *)D.dst, D.dst, n_tables, 2 * half, C.r[k - 1], s, k == 1);
                    if (rc) return rc;
                    for (int t = 0; t < n_tables; ++t) M.src[t] = D.dst[t];
                    const int shares = std::max(std::max(M.n_terms, (M.n_lin + 3) / 4), 1);
                    int rows = 1;
                    while (rows < shares) rows <<= 1;
                    for (int j = k; j < v; ++j) C.skip_mask |= 1ull << j;
                    C.n_prior = k;
                    if (M.deg <= 3) hipLaunchKernelGGL(k_tail_mem<4>, dim3(1), dim3(TAIL_THREADS), 0, s, M, C, rows, (int)(2 * half), (const u64 *)part, samples);
                    else hipLaunchKernelGGL(k_tail_mem<NSAMP>, dim3(1), dim3(TAIL_THREADS), 0, s, M, C, rows, (int)(2 * half), (const u64 *)part, samples);
                    VI_LAUNCH_CHECK("sumcheck tail (tables folded into place)");
                    return VI_OK;
                }
                if (k == 0) {
                    nb = launch_round<0>(D, half, 0, part + off, blocks_for(half), nullptr, 1, 0, 0, s);
                    VI_LAUNCH_CHECK("sumcheck eval");
                } else {
                    // half = pairs of this round; the fold by r_(k-1) halves tables of 4 * half words
                    Desc E = D;
                    E.canon_src = k == 1;
                    if (k > 1) for (int t = 0; t < n_tables; ++t) E.src[t] = D.dst[t];
                    E.skip1 = 1;             // S(1) of a later round is the claim minus S(0): not summed
                    C.skip_mask |= 1ull << k;
                    nb = launch_round<2>(E, 2 * half, C.r[k - 1], part + off, blocks_for(half), nullptr, 1, 0, 0, s);
                    VI_LAUNCH_CHECK("sumcheck fold+eval");
                }
                C.off[k] = off;
                C.nb[k] = (unsigned short)nb;
                off += (unsigned)nb * NSAMP;
            }
        } else {
            // tables in memory: a round of many pairs evaluates and writes the folded tables in one launch; a
            // round of few folds first (one launch) and deals its terms over rows of workgroups
            bool folded = true;              // the tables of round k are in place (false: still to be folded by r_(k-1))
            for (int k = 0; k < v; ++k, half >>= 1) {
                Desc E = D;
                if (k > 0) for (int t = 0; t < n_tables; ++t) E.src[t] = D.dst[t];
                if (!folded) {
                    // tables of round k - 1 (2 * half pairs) -> tables of round k
                    rc = fold_tables(k == 1 ? D.src : (const uint64_t *const *)D.dst, D.dst, n_tables, 2 * half, C.r[k - 1], s, k == 1);
                    if (rc) return rc;
                    folded = true;
                }
                if ((i64)n_tables * 2 * half <= TAIL_MEM_WORDS && v - k <= TAIL_MEM_ROUNDS) {
                    // every table of this round fits one workgroup's LDS: all remaining rounds in one launch
                    const int shares = std::max(std::max(E.n_terms, (E.n_lin + 3) / 4), 1);
                    int rows = 1;
                    while (rows < shares) rows <<= 1;
                    for (int j = std::max(k, 1); j < v; ++j) C.skip_mask |= 1ull << j;
                    C.n_prior = k;
                    if (E.deg <= 3) hipLaunchKernelGGL(k_tail_mem<4>, dim3(1), dim3(TAIL_THREADS), 0, s, E, C, rows, (int)(2 * half), (const u64 *)part, samples);
                    else hipLaunchKernelGGL(k_tail_mem<NSAMP>, dim3(1), dim3(TAIL_THREADS), 0, s, E, C, rows, (int)(2 * half), (const u64 *)part, samples);
                    VI_LAUNCH_CHECK("sumcheck tail (tables from memory)");
                    return VI_OK;                          // the tail has written every round's samples
                }
                if (k > 0) {
                    E.skip1 = 1;
                    C.skip_mask |= 1ull << k;
                }
                int nb;
                if (k + 1 < v && half >= FUSE_MIN_PAIRS) {
                    FoldOut W;
                    W.r = C.r[k];
                    W.virt = -1;
                    std::vector<int> unused;
                    fill_fold_flags(E, W, unused);
                    if (!unused.empty()) {
                        std::vector<const uint64_t *> us;
                        std::vector<uint64_t *> ud;
                        for (int t : unused) { us.push_back(E.src[t]); ud.push_back(E.dst[t]); }
                        rc = fold_tables(us.data(), ud.data(), (int)us.size(), half, C.r[k], s, k == 0);
                        if (rc) return rc;
                    }
                    nb = launch_eval_mem(E, half, part + off, 0, 1, s, &W, nullptr);
                    VI_LAUNCH_CHECK("sumcheck eval + fold");
                } else {
                    nb = launch_eval_mem(E, half, part + off, 0, 1, s);
                    VI_LAUNCH_CHECK("sumcheck eval");
                    folded = false;
                }
                C.off[k] = off;
                C.nb[k] = (unsigned short)nb;
                off += (unsigned)nb * NSAMP;
            }
        }
    } else {
        // beyond one descriptor: fold every table, then evaluate group by group, per round
        std::vector<TermGroup> groups;
        split_terms(n_tables, term_off, factor_idx, coeffs, n_terms, groups);
        i64 half = size / 2;
        unsigned off = 0;
        for (int k = 0; k < v; ++k, half >>= 1) {
            int nb = 0;
            if (k > 0) {
                rc = fold_tables(k == 1 ? tables : (const uint64_t *const *)work, work, n_tables, 2 * half, C.r[k - 1], s, k == 1);
                if (rc) return rc;
            }
            rc = eval_groups(who, k == 0 ? tables : (const uint64_t *const *)work, groups, deg, half, part + off, nullptr, 0, s, &nb,
                             k > 0 ? 1 : 0);
            if (rc) return rc;
            if (k > 0) C.skip_mask |= 1ull << k;
            C.off[k] = off;
            C.nb[k] = (unsigned short)nb;
            off += (unsigned)nb * NSAMP;
        }
    }
    hipLaunchKernelGGL(k_finish, dim3(1), dim3(TAIL_THREADS), 0, s, C, (const u64 *)part, samples);
    VI_LAUNCH_CHECK("sumcheck finish");
    return VI_OK;
}

}  // namespace

int vi_sumcheck_prove_coins(const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                            const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms,
                            const uint64_t *challenges, uint64_t *samples, void *ws, size_t ws_bytes, void *stream) {
    const char *who = "vi_sumcheck_prove_coins";
    if (size < 2 || (size & (size - 1))) return vi::fail(VI_EINVAL, "%s: size must be a power of two >= 2, got %lld", who, (long long)size);
    const int v = vi::ilog2(size);
    if (v > MAX_ROUNDS) return vi::fail(VI_EINVAL, "%s: %d rounds exceed %d", who, v, MAX_ROUNDS);
    if (!challenges || !samples || !work) return vi::fail(VI_EINVAL, "%s: null pointer", who);
    if (!ws || ws_bytes < vi_sumcheck_prove_coins_workspace_bytes(size))
        return vi::fail(VI_ENOMEM, "%s: workspace below %zu bytes", who, vi_sumcheck_prove_coins_workspace_bytes(size));
    int deg = 0;
    int rc = check_terms(who, tables, n_tables, term_off, factor_idx, coeffs, n_terms, &deg);
    if (rc) return rc;
    for (int t = 0; t < n_tables; ++t)
        if (!work[t]) return vi::fail(VI_EINVAL, "%s: null work buffer %d", who, t);
    return prove_coins_impl(who, tables, work, n_tables, size, term_off, factor_idx, coeffs, n_terms, deg, challenges, samples,
                            (u64 *)ws, (hipStream_t)stream, true);
}

}  // extern "C"

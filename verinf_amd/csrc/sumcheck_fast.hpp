// Sumcheck proofs whose challenges are all known before the first launch.
//
// The reference's prover asks its verifier coin for a challenge by round number only
// (layergkr/gpu.py:403, layergkr/sumcheck.py:217: `r = coin(rnd)`) and every caller draws the coins before
// the proof starts (layergkr/full_layer.py:222-224, layergkr/relations.py:122-123), so nothing the host
// contributes to a round depends on that round's samples.  With the challenges in hand the rounds need no
// host round trip, and more than that: several rounds fit in ONE pass over the tables.  The fold pairs index
// i with i + n/2 (most significant variable first), so the 2^R entries i + c n/2^R, c < 2^R, of a table are
// closed under R rounds of folding.  A thread of k_pass3 loads those eight entries of every table (eight
// coalesced streams), evaluates round k on the four pairs (c, c + 4), folds them by r_k, evaluates round
// k + 1 on the two pairs of folded values, folds by r_(k+1), evaluates round k + 2 on the last pair and
// writes ONE folded value per table: a table is read once and an eighth of it written per three rounds,
// instead of read once and half of it written per round.  When the tables have become small enough for one
// workgroup's LDS, k_tail runs every remaining round in a single launch, adds up the per-workgroup partial
// sums the passes left behind, and finishes all samples of the proof: S_k(1) = claim_k - S_k(0), where
// claim_(k+1) = S_k(r_k) follows from the samples by Lagrange interpolation -- a chain over the rounds that a
// launch per round used to carry through the host.
//
// Shapes with their own unrolled evaluation (the ones the layer proof consists of): a single product of up to
// four distinct tables (a matmul contraction, eq * a * b, the three-factor benchmark instance) and the hadamard
// gate batch eq * (a * b + c' * c).  Other sums keep one launch per round (k_round / k_eval_mem) but are queued
// back to back in the same way and finished by k_finish.
#pragma once

namespace {

constexpr int MAX_ROUNDS = 40;              // tables of up to 2^40 words
constexpr int TAIL_THREADS = 1024;
constexpr int TAIL_WORDS = 6144;            // table words a tail workgroup keeps in LDS (48 KiB)

// What the kernel that finishes a proof needs to know about its rounds.
struct ChainDesc {
    u64 r[MAX_ROUNDS];                      // challenges, canonical
    u64 winv[NSAMP];                        // Lagrange weights of the points 0..deg
    u64 scale;                              // factor of every summed sample (1 = none)
    u64 skip_mask;                          // bit k: round k did not sum S(1); it is claim_k - S_k(0)
    // inf_node: slot deg of a round holds the leading coefficient L of S_k (the "value at infinity": the sum of
    // the products of the differences hi - lo) instead of S_k(deg), which costs the kernels one step less of every
    // table's ladder; S(deg) = sum_{j<deg} cinf[j] S(j) + deg! L  (the polynomial through the values at 0..deg-1,
    // extrapolated to deg, plus L x (x-1) ... (x-deg+1) there)
    u64 cinf[NSAMP];
    u64 dfact;
    int inf_node;
    unsigned off[MAX_ROUNDS];               // word offset of round k's per-workgroup partial sums in the workspace
    unsigned short nb[MAX_ROUNDS];          // rows of NSAMP words round k left there
    int n_rounds, n_prior, deg;             // rounds of the proof; rounds whose partial sums are in the workspace
};

struct FinishShared {
    u64 raw[MAX_ROUNDS][NSAMP];             // summed samples per round, before scale and chain
    u64 lag[MAX_ROUNDS][NSAMP];             // Lagrange basis of the points 0..deg at r_k
    u64 a[MAX_ROUNDS], b[MAX_ROUNDS];       // claim_(k+1) = a_k claim_k + b_k
    u64 claim[MAX_ROUNDS + 1];
};

// Lagrange basis at the challenges (one thread per round) and the sums of the partials the earlier launches left
// (one wavefront per round).  The caller synchronises the workgroup before finish_samples().
__device__ __forceinline__ void finish_begin(const ChainDesc &C, const u64 *part, FinishShared &sh) {
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, nw = blockDim.x >> 6;
    if (tid < C.n_rounds) {
        const u64 r = C.r[tid];
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            if (x <= C.deg) {
                u64 num = C.winv[x];
#pragma unroll
                for (int j = 0; j < NSAMP; ++j)
                    if (j <= C.deg && j != x) num = gl::mul(num, gl::sub(r, (u64)j));
                sh.lag[tid][x] = num;
            }
        }
    }
    for (int k = w; k < C.n_prior; k += nw) {
        const u64 *p = part + C.off[k];
        const int nb = C.nb[k];
        u64 v[NSAMP];
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) v[x] = 0;
        // four rows per lane in flight (a lane's loads are otherwise a chain of round trips to memory)
        for (int b0 = lane; b0 < nb; b0 += 256) {
            u64 t[4][NSAMP];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int b = b0 + 64 * u;
#pragma unroll
                for (int x = 0; x < NSAMP; ++x) t[u][x] = (x <= C.deg && b < nb) ? p[(i64)b * NSAMP + x] : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int x = 0; x < NSAMP; ++x)
                    if (x <= C.deg) v[x] = gl::addc(v[x], t[u][x]);
        }
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            if (x <= C.deg) {
                const u64 sum = wave_sum(v[x]);
                if (lane == 0) sh.raw[k][x] = sum;
            }
        }
    }
}

// sh.raw holds every round's sums (the workgroup has synchronised): scale, chain the claims, store the samples.
// out: n_rounds rows of NSAMP words, S_k(x) at out[k * NSAMP + x].
__device__ __forceinline__ void finish_samples(const ChainDesc &C, FinishShared &sh, u64 *out) {
    const int k = threadIdx.x;
    const bool mine = k < C.n_rounds;
    const bool skip = mine && ((C.skip_mask >> k) & 1);
    const bool inf = C.inf_node != 0;
    u64 y[NSAMP];
    u64 top_a = 0, top_b = 0;                // S_k(deg) = top_a claim_k + top_b when it is not summed itself
    if (mine) {
        // every sample is a + b claim_k for known a, b: S(1) = claim - S(0) where it was skipped, S(deg) from
        // the leading coefficient; so claim_(k+1) = sum_x L_x(r_k) S_k(x) = a_k claim_k + b_k
        u64 a = 0, b = 0;
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            y[x] = 0;
            if (x <= C.deg && !(skip && x == 1)) {
                y[x] = sh.raw[k][x];
                if (C.scale != 1) y[x] = gl::mul(y[x], C.scale);
            }
        }
        // S(1) = claim - S(0) when skipped: its part that does not depend on the claim
        const u64 one_b = skip ? gl::neg(y[0]) : y[1];
        if (inf) {
            u64 lead = 0;
#pragma unroll
            for (int x = 0; x < NSAMP; ++x) {
                if (x == C.deg) lead = y[x];
                if (x < C.deg && x != 1) top_b = gl::addc(top_b, gl::mul(C.cinf[x], y[x]));
            }
            top_b = gl::addc(top_b, gl::mul(C.cinf[1], one_b));
            top_b = gl::addc(top_b, gl::mul(C.dfact, lead));
            top_a = skip ? C.cinf[1] : 0;
        }
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            if (x <= C.deg) {
                const u64 l = sh.lag[k][x];
                if (x == 1) {
                    b = gl::addc(b, gl::mul(l, one_b));
                    if (skip) a = gl::addc(a, l);
                } else if (inf && x == C.deg) {
                    b = gl::addc(b, gl::mul(l, top_b));
                    a = gl::addc(a, gl::mul(l, top_a));
                } else {
                    b = gl::addc(b, gl::mul(l, y[x]));
                }
            }
        }
        sh.a[k] = a;
        sh.b[k] = b;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        u64 claim = 0;                       // a round that summed every sample does not read it
        for (int j = 0; j < C.n_rounds; ++j) {
            sh.claim[j] = claim;
            claim = gl::addc(gl::mul(sh.a[j], claim), sh.b[j]);
        }
    }
    __syncthreads();
    if (mine) {
        const u64 claim = sh.claim[k];
        if (skip) y[1] = gl::sub(claim, y[0]);
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            if (x <= C.deg) {
                u64 v = y[x];
                if (inf && x == C.deg) v = gl::addc(gl::mul(top_a, claim), top_b);
                out[(i64)k * NSAMP + x] = v;
            }
        }
    }
}

// finishes a proof whose rounds all left partial sums in the workspace
__global__ __launch_bounds__(TAIL_THREADS) void k_finish(const ChainDesc C, const u64 *part, u64 *out) {
    __shared__ FinishShared sh;
    finish_begin(C, part, sh);
    __syncthreads();
    finish_samples(C, sh, out);
}

// ---- the fixed shapes ------------------------------------------------------------------------------------------
// SHAPE 1: the product of the NT tables (degree NT, NT + 1 samples).
// SHAPE 2: four tables [eq, a, b, c]: eq (a b + c) (degree 3); the coefficient of c is multiplied into the table
//          when the caller's words are first loaded, so that every later round sees a plain sum.
struct FastDesc {
    const u64 *src[4];
    u64 *dst[4];
    u64 lin_coeff;
};

template <int NT, int SHAPE>
struct FastShape {
    static constexpr int NS = SHAPE == 2 ? 4 : NT + 1;
    // degree >= 2: the last slot takes the leading coefficient instead of S(deg) (ChainDesc::inf_node)
    static constexpr bool INF = NS >= 3;
};

// accumulators of the samples of one round: plain integers of five words (a product is added without being
// reduced, gl::wide_mul_acc) in the passes, canonical field elements in the tail, where a thread adds few pairs
template <bool WIDE>
struct SampleAcc;
template <>
struct SampleAcc<true> {
    gl::Wide v;
    __device__ __forceinline__ void zero() { gl::wide_zero(v); }
    __device__ __forceinline__ void add_product(u64 a, u64 b) { gl::wide_mul_acc(v, a, b); }
    __device__ __forceinline__ u64 value() const { return gl::wide_reduce(v); }
};
template <>
struct SampleAcc<false> {
    u64 v;
    __device__ __forceinline__ void zero() { v = 0; }
    __device__ __forceinline__ void add_product(u64 a, u64 b) { v = gl::addc(v, gl::mul(a, b)); }
    __device__ __forceinline__ u64 value() const { return v; }
};

// One pair (lo, hi) of every table: adds S(x) of the pair to acc[x] for x = 0..deg-1 (x = 1 left out when SKIP1)
// and the pair's leading coefficient to acc[deg] (or S(deg) when the degree is 1), and returns the differences
// hi - lo, which the fold needs again.  All values canonical.
template <int NT, int SHAPE, bool SKIP1, bool WIDE>
__device__ __forceinline__ void eval_pair(const u64 (&lo)[NT], const u64 (&hi)[NT], u64 (&dif)[NT],
                                          SampleAcc<WIDE> (&acc)[FastShape<NT, SHAPE>::NS]) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    constexpr bool INF = FastShape<NT, SHAPE>::INF;
    u64 cur[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        cur[t] = lo[t];
        dif[t] = gl::sub(hi[t], lo[t]);
    }
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        const bool at_inf = INF && x == NS - 1;
        if (!(SKIP1 && x == 1)) {
            if constexpr (SHAPE == 2) {
                // eq (a b + c): the c term has degree 2 and does not reach the leading coefficient
                if (at_inf) acc[x].add_product(gl::mul_lazy(dif[1], dif[2]), dif[0]);
                else acc[x].add_product(gl::mul_add_lazy(cur[1], cur[2], cur[3]), cur[0]);
            } else if constexpr (NT == 1) {
                acc[x].add_product(cur[0], 1);
            } else {
                u64 v = at_inf ? dif[0] : cur[0];
#pragma unroll
                for (int t = 1; t + 1 < NT; ++t) v = gl::mul_lazy(v, at_inf ? dif[t] : cur[t]);
                acc[x].add_product(v, at_inf ? dif[NT - 1] : cur[NT - 1]);
            }
        }
        if (x + 1 < NS - (INF ? 1 : 0)) {
            // f(1) is the upper value itself: the first step of the ladder costs nothing
#pragma unroll
            for (int t = 0; t < NT; ++t) cur[t] = (x == 0) ? hi[t] : gl::addc(cur[t], dif[t]);
        }
    }
}

template <int NT, int SHAPE, bool FIRST>
__device__ __forceinline__ u64 fast_load(const FastDesc &D, int t, i64 idx) {
    u64 v = D.src[t][idx];
    if (FIRST) {
        v = gl::canon(v);                    // caller data: any 64-bit word is taken as its residue
        if (SHAPE == 2 && t == 3) v = gl::mul(v, D.lin_coeff);
    }
    return v;
}

// sum over the rows of NSAMP words at `rows` -> out[0..ns), by one workgroup of BLOCK threads
template <int NS>
__device__ __forceinline__ void block_sum_rows(const u64 *rows, int n_rows, u64 *out, u64 (*red)[NSAMP]) {
    u64 v[NS];
#pragma unroll
    for (int x = 0; x < NS; ++x) v[x] = 0;
    for (int b0 = threadIdx.x; b0 < n_rows; b0 += 2 * BLOCK) {         // two rows per thread in flight
        u64 t[2][NS];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int x = 0; x < NS; ++x) t[u][x] = (b0 + u * BLOCK < n_rows) ? rows[(i64)(b0 + u * BLOCK) * NSAMP + x] : 0;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int x = 0; x < NS; ++x) v[x] = gl::addc(v[x], t[u][x]);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        const u64 sum = wave_sum(v[x]);
        if (lane == 0) red[w][x] = sum;
    }
    __syncthreads();
    if (threadIdx.x < NS) {
        u64 sum = red[0][threadIdx.x];
        for (int i = 1; i < BLOCK / 64; ++i) sum = gl::addc(sum, red[i][threadIdx.x]);
        out[threadIdx.x] = sum;
    }
    __syncthreads();
}

// Three rounds in one pass.  cols = n / 8 for tables of n words; thread i < cols owns entries i + c cols.
// FIRST: the tables are the caller's (words reduced on load, round 0 sums every sample).
// part: three regions of gridDim.x rows of NSAMP words, one per round.
// prev_part / prev_rows / prev_sums: the previous pass's three regions of prev_rows rows each; workgroup j < 3 adds
// region j up into row j of prev_sums before it starts on its own columns, so that the kernel that finishes the
// proof finds one row per round instead of a thousand (prev_rows = 0: nothing to add up).
template <int NT, int SHAPE, bool FIRST>
__global__ __launch_bounds__(BLOCK) void k_pass3(const FastDesc D, i64 cols, u64 r0, u64 r1, u64 r2, u64 *part,
                                                 const u64 *prev_part, int prev_rows, u64 *prev_sums) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    __shared__ u64 red[BLOCK / 64][3][NS];
    __shared__ u64 red_prev[BLOCK / 64][NSAMP];
    if (prev_rows > 0 && blockIdx.x < 3)
        block_sum_rows<NS>(prev_part + (i64)blockIdx.x * prev_rows * NSAMP, prev_rows, prev_sums + blockIdx.x * NSAMP, red_prev);
    SampleAcc<true> acc0[NS], acc1[NS], acc2[NS];
#pragma unroll
    for (int x = 0; x < NS; ++x) { acc0[x].zero(); acc1[x].zero(); acc2[x].zero(); }
    const i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < cols; i += stride) {
        u64 v[NT][8];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int c = 0; c < 8; ++c) v[t][c] = D.src[t][i + c * cols];
        if (FIRST) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    v[t][c] = gl::canon(v[t][c]);
                    if (SHAPE == 2 && t == 3) {
                        v[t][c] = gl::mul(v[t][c], D.lin_coeff);
                        VI_SCHED_FENCE();
                    }
                }
        }
        // the scheduler is kept from interleaving the pairs: each one's temporaries die before the next starts
        u64 lo[NT], hi[NT], dif[NT];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            VI_SCHED_FENCE();
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = v[t][c]; hi[t] = v[t][c + 4]; }
            eval_pair<NT, SHAPE, !FIRST, true>(lo, hi, dif, acc0);
#pragma unroll
            for (int t = 0; t < NT; ++t) v[t][c] = gl::mul_add(r0, dif[t], lo[t]);
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            VI_SCHED_FENCE();
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = v[t][c]; hi[t] = v[t][c + 2]; }
            eval_pair<NT, SHAPE, true, true>(lo, hi, dif, acc1);
#pragma unroll
            for (int t = 0; t < NT; ++t) v[t][c] = gl::mul_add(r1, dif[t], lo[t]);
        }
        VI_SCHED_FENCE();
#pragma unroll
        for (int t = 0; t < NT; ++t) { lo[t] = v[t][0]; hi[t] = v[t][1]; }
        eval_pair<NT, SHAPE, true, true>(lo, hi, dif, acc2);
#pragma unroll
        for (int t = 0; t < NT; ++t) D.dst[t][i] = gl::mul_add(r2, dif[t], lo[t]);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        const u64 s0 = wave_sum(acc0[x].value()), s1 = wave_sum(acc1[x].value()), s2 = wave_sum(acc2[x].value());
        if (lane == 0) { red[w][0][x] = s0; red[w][1][x] = s1; red[w][2][x] = s2; }
    }
    __syncthreads();
    if (threadIdx.x < 3 * NS) {
        const int j = threadIdx.x / NS, x = threadIdx.x % NS;
        u64 s = red[0][j][x];
        for (int i = 1; i < BLOCK / 64; ++i) s = gl::addc(s, red[i][j][x]);
        part[((i64)j * gridDim.x + blockIdx.x) * NSAMP + x] = s;
    }
}

// pairs per table a tail workgroup holds after its first fold
template <int NT>
struct TailCap {
    static constexpr int HALF = NT == 1 ? 4096 : (NT <= 3 ? 2048 : 1024);
    static_assert(NT * HALF <= TAIL_WORDS, "tail tables exceed their LDS share");
};

// sums of one round over the workgroup: every wavefront that had pairs leaves its sums in red_par, the caller
// synchronises, and threads x < NS add them up into raw_k
template <int NS>
__device__ __forceinline__ void tail_wave_sums(const SampleAcc<false> (&acc)[NS], u64 (*red_par)[NSAMP], int active_waves) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (w < active_waves) {
#pragma unroll
        for (int x = 0; x < NS; ++x) {
            const u64 s = wave_sum(acc[x].v);
            if (lane == 0) red_par[w][x] = s;
        }
    }
}
template <int NS>
__device__ __forceinline__ void tail_round_total(u64 (*red_par)[NSAMP], int active_waves, u64 *raw_k) {
    if (threadIdx.x < NS) {
        u64 s = red_par[0][threadIdx.x];
        for (int i = 1; i < active_waves; ++i) s = gl::addc(s, red_par[i][threadIdx.x]);
        raw_k[threadIdx.x] = s;
    }
}

// Every remaining round in one workgroup: tables of `size` <= 2 TailCap<NT>::HALF words; rounds C.n_prior .. C.n_rounds - 1.
// FIRST: the proof starts here (the tables are the caller's).  The folded tables live in LDS and are not written back.
// A round costs its longest thread, so what a round does besides its one pair per thread is kept off that path:
//  - rounds of more than TAIL_DEFER pairs add their sums up across the workgroup as they go (every wavefront is busy);
//  - smaller rounds leave each thread's sums in LDS -- the round of h pairs in lane_sums[.][h .. 2h) -- and nine
//    wavefronts add the nine of them up at the end, all at once;
//  - once a table fits the lanes of one wavefront (64 entries) the first wavefront goes on alone, a table entry per
//    lane and partners fetched by lane shuffles: no LDS traffic for the tables, no workgroup barrier per round.
constexpr int TAIL_DEFER = 256;

template <int NT, int SHAPE, bool FIRST>
__global__ __launch_bounds__(TAIL_THREADS) void k_tail(const FastDesc D, i64 size, const ChainDesc C, const u64 *part, u64 *out) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    constexpr int HALF = TailCap<NT>::HALF;
    __shared__ u64 tab[NT][HALF];
    __shared__ u64 red[2][TAIL_THREADS / 64][NSAMP];
    __shared__ u64 lane_sums[NS][2 * TAIL_DEFER];
    __shared__ FinishShared sh;
    finish_begin(C, part, sh);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    int k = C.n_prior, par = 0;
    int h = (int)(size >> 1);
    const int h_first = h;
    SampleAcc<false> acc[NS];
    u64 lo[NT], hi[NT], dif[NT];
    {
        // first round of this launch: pairs from memory, folded values into LDS
#pragma unroll
        for (int x = 0; x < NS; ++x) acc[x].zero();
        const u64 r = C.r[k];
        for (int i = tid; i < h; i += TAIL_THREADS) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                lo[t] = fast_load<NT, SHAPE, FIRST>(D, t, i);
                hi[t] = fast_load<NT, SHAPE, FIRST>(D, t, (i64)h + i);
            }
            eval_pair<NT, SHAPE, !FIRST, false>(lo, hi, dif, acc);
            if (h > 1) {
#pragma unroll
                for (int t = 0; t < NT; ++t) tab[t][i] = gl::mul_add(r, dif[t], lo[t]);
            }
        }
        if (h > TAIL_DEFER) {
            const int aw = h >= TAIL_THREADS ? TAIL_THREADS / 64 : (h + 63) >> 6;
            tail_wave_sums<NS>(acc, red[par], aw);
            __syncthreads();
            tail_round_total<NS>(red[par], aw, sh.raw[k]);
            par ^= 1;
        } else {
            if (tid < h) {
#pragma unroll
                for (int x = 0; x < NS; ++x) lane_sums[x][h + tid] = acc[x].v;
            }
            __syncthreads();
        }
    }
    // rounds on tables of more than 64 entries: pairs from LDS, a workgroup barrier per round
    for (h >>= 1; h >= 64; h >>= 1) {
        ++k;
#pragma unroll
        for (int x = 0; x < NS; ++x) acc[x].zero();
        const u64 r = C.r[k];
        for (int i = tid; i < h; i += TAIL_THREADS) {
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = tab[t][i]; hi[t] = tab[t][h + i]; }
            eval_pair<NT, SHAPE, true, false>(lo, hi, dif, acc);
#pragma unroll
            for (int t = 0; t < NT; ++t) tab[t][i] = gl::mul_add(r, dif[t], lo[t]);
        }
        if (h > TAIL_DEFER) {
            const int aw = h >= TAIL_THREADS ? TAIL_THREADS / 64 : (h + 63) >> 6;
            tail_wave_sums<NS>(acc, red[par], aw);
            __syncthreads();
            tail_round_total<NS>(red[par], aw, sh.raw[k]);
            par ^= 1;
        } else {
            if (tid < h) {
#pragma unroll
                for (int x = 0; x < NS; ++x) lane_sums[x][h + tid] = acc[x].v;
            }
            __syncthreads();
        }
    }
    // tables of at most 64 entries: the first wavefront alone, lane i holding entry i of every table
    if (w == 0 && h >= 1) {
        u64 val[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) val[t] = (lane < 2 * h) ? tab[t][lane] : 0;
        for (; h >= 1; h >>= 1) {
            ++k;
#pragma unroll
            for (int x = 0; x < NS; ++x) acc[x].zero();
            const u64 r = C.r[k];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                lo[t] = val[t];
                hi[t] = __shfl_down(val[t], (unsigned)h, 64);      // lanes past the pairs compute on what they get and drop it
            }
            eval_pair<NT, SHAPE, true, false>(lo, hi, dif, acc);
#pragma unroll
            for (int t = 0; t < NT; ++t) val[t] = gl::mul_add(r, dif[t], lo[t]);
            if (lane < h) {
#pragma unroll
                for (int x = 0; x < NS; ++x) lane_sums[x][h + lane] = acc[x].v;
            }
        }
    }
    __syncthreads();
    // the deferred rounds: wavefront j adds up the round of TAIL_DEFER >> j pairs, the (log2 of that + 1)-th from last
    {
        const int hd = TAIL_DEFER >> w;
        if (w < 9 && hd <= h_first) {
            int lg = 0;
            while ((1 << lg) < hd) ++lg;
            const int kd = C.n_rounds - 1 - lg;
            const bool skip1 = (C.skip_mask >> kd) & 1;
#pragma unroll
            for (int x = 0; x < NS; ++x) {
                if (!(skip1 && x == 1)) {
                    u64 v = 0;
                    for (int i = lane; i < hd; i += 64) v = gl::addc(v, lane_sums[x][hd + i]);
                    v = wave_sum(v);
                    if (lane == 0) sh.raw[kd][x] = v;
                }
            }
        }
    }
    __syncthreads();
    finish_samples(C, sh, out);
}

template <int NT, int SHAPE, bool FIRST>
int launch_pass3(const FastDesc &F, i64 cols, const u64 *r, u64 *part, const u64 *prev_part, int prev_rows,
                 u64 *prev_sums, hipStream_t s) {
    static std::mutex mu;
    static int caps[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int cap;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!caps[dev]) caps[dev] = resident_blocks(k_pass3<NT, SHAPE, FIRST>, 64);
        cap = caps[dev];
    }
    int nb = blocks_for(cols);
    if (nb > cap) nb = cap;
    if (nb < 3 && prev_rows > 0) nb = 3;     // the first three workgroups add up the previous pass's sums
    hipLaunchKernelGGL((k_pass3<NT, SHAPE, FIRST>), dim3(nb), dim3(BLOCK), 0, s, F, cols, r[0], r[1], r[2], part,
                       prev_part, prev_rows, prev_sums);
    return nb;
}

// constants of ChainDesc::inf_node for degree d: S(d) = sum_{j<d} cinf[j] S(j) + d! L
void fill_inf_node(ChainDesc &C, int d) {
    C.inf_node = 1;
    C.dfact = 1;
    for (int m = 1; m <= d; ++m) C.dfact = gl::mul(C.dfact, (u64)m);
    for (int j = 0; j < NSAMP; ++j) C.cinf[j] = 0;
    for (int j = 0; j < d; ++j) {
        // Lagrange basis of the nodes 0..d-1 at x = d
        u64 num = 1, den = 1;
        for (int m = 0; m < d; ++m) {
            if (m == j) continue;
            num = gl::mul(num, (u64)(d - m));
            den = gl::mul(den, gl::sub((u64)j, (u64)m));
        }
        C.cinf[j] = gl::mul(num, gl::inv(den));
    }
}

// The whole proof of a fixed shape: passes of three rounds while the tables exceed a tail workgroup, then the tail.
// part: workspace of at least (n_rounds + 1) * MAX_BLOCKS * NSAMP words; C arrives with r, winv, scale, deg, n_rounds set.
template <int NT, int SHAPE>
int prove_fast_shape(FastDesc F, i64 size, ChainDesc &C, u64 *part, u64 *out, hipStream_t s) {
    constexpr i64 TAIL_MAX = 2 * (i64)TailCap<NT>::HALF;
    int k = 0;
    unsigned off = 0;
    bool first = true;
    C.skip_mask = 0;
    for (int j = 1; j < C.n_rounds; ++j) C.skip_mask |= 1ull << j;
    if (FastShape<NT, SHAPE>::INF) fill_inf_node(C, C.deg);
    // one row per round for the sums that a pass adds up for the pass before it: the last MAX_ROUNDS rows of the workspace
    const unsigned sums_off = (unsigned)C.n_rounds * MAX_BLOCKS * NSAMP;
    const u64 *prev_part = nullptr;
    int prev_rows = 0, prev_k = 0;
    while (size > TAIL_MAX) {
        const i64 cols = size >> 3;
        u64 *prev_sums = part + sums_off + (unsigned)prev_k * NSAMP;
        const int nb = first ? launch_pass3<NT, SHAPE, true>(F, cols, C.r + k, part + off, prev_part, prev_rows, prev_sums, s)
                             : launch_pass3<NT, SHAPE, false>(F, cols, C.r + k, part + off, prev_part, prev_rows, prev_sums, s);
        VI_LAUNCH_CHECK("sumcheck pass (three rounds)");
        if (prev_rows > 0) {
            for (int j = 0; j < 3; ++j) {    // this launch has left the previous pass's rounds as one row each
                C.off[prev_k + j] = sums_off + (unsigned)(prev_k + j) * NSAMP;
                C.nb[prev_k + j] = 1;
            }
        }
        for (int j = 0; j < 3; ++j) {
            C.off[k + j] = off + (unsigned)j * (unsigned)nb * NSAMP;
            C.nb[k + j] = (unsigned short)nb;
        }
        prev_part = part + off;
        prev_rows = nb;
        prev_k = k;
        off += 3u * (unsigned)nb * NSAMP;
        k += 3;
        size >>= 3;
        if (first) {
            for (int t = 0; t < NT; ++t) F.src[t] = F.dst[t];    // later passes fold the work buffers in place
            first = false;
        }
    }
    C.n_prior = k;
    if (first) hipLaunchKernelGGL((k_tail<NT, SHAPE, true>), dim3(1), dim3(TAIL_THREADS), 0, s, F, size, C, (const u64 *)part, out);
    else hipLaunchKernelGGL((k_tail<NT, SHAPE, false>), dim3(1), dim3(TAIL_THREADS), 0, s, F, size, C, (const u64 *)part, out);
    VI_LAUNCH_CHECK("sumcheck tail");
    return VI_OK;
}

}  // namespace

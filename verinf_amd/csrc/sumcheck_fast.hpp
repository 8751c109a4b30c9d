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
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            if (x <= C.deg) {
                u64 v = 0;
                for (int b = lane; b < nb; b += 64) v = gl::addc(v, p[(i64)b * NSAMP + x]);
                v = wave_sum(v);
                if (lane == 0) sh.raw[k][x] = v;
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
    u64 y[NSAMP];
    if (mine) {
        // claim_(k+1) = sum_x L_x(r_k) S_k(x); with S_k(1) = claim_k - S_k(0) that is a_k claim_k + b_k
        u64 b = 0;
#pragma unroll
        for (int x = 0; x < NSAMP; ++x) {
            y[x] = 0;
            if (x <= C.deg && !(skip && x == 1)) {
                y[x] = sh.raw[k][x];
                if (C.scale != 1) y[x] = gl::mul(y[x], C.scale);
                b = gl::addc(b, gl::mul(sh.lag[k][x], y[x]));
            }
        }
        u64 a = 0;
        if (skip) {
            a = sh.lag[k][1];
            b = gl::sub(b, gl::mul(a, y[0]));
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
        if (skip) y[1] = gl::sub(sh.claim[k], y[0]);
#pragma unroll
        for (int x = 0; x < NSAMP; ++x)
            if (x <= C.deg) out[(i64)k * NSAMP + x] = y[x];
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
};

// One pair (lo, hi) of every table: adds S(x) of the pair to acc[x] for x = 0..deg (x = 1 left out when SKIP1) and
// returns the differences hi - lo, which the fold needs again.  All values canonical.
template <int NT, int SHAPE, bool SKIP1>
__device__ __forceinline__ void eval_pair(const u64 (&lo)[NT], const u64 (&hi)[NT], u64 (&dif)[NT],
                                          u64 (&acc)[FastShape<NT, SHAPE>::NS]) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    u64 cur[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        cur[t] = lo[t];
        dif[t] = gl::sub(hi[t], lo[t]);
    }
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        if (!(SKIP1 && x == 1)) {
            u64 v;
            if constexpr (SHAPE == 2) {
                v = gl::mul(gl::addc(gl::mul(cur[1], cur[2]), cur[3]), cur[0]);
            } else {
                v = cur[0];
#pragma unroll
                for (int t = 1; t < NT; ++t) v = gl::mul(v, cur[t]);
            }
            acc[x] = gl::addc(acc[x], v);
        }
        if (x + 1 < NS) {
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

// Three rounds in one pass.  cols = n / 8 for tables of n words; thread i < cols owns entries i + c cols.
// FIRST: the tables are the caller's (words reduced on load, round 0 sums every sample).
// part: three regions of gridDim.x rows of NSAMP words, one per round.
template <int NT, int SHAPE, bool FIRST>
__global__ __launch_bounds__(BLOCK) void k_pass3(const FastDesc D, i64 cols, u64 r0, u64 r1, u64 r2, u64 *part) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    __shared__ u64 red[BLOCK / 64][3][NS];
    u64 acc0[NS], acc1[NS], acc2[NS];
#pragma unroll
    for (int x = 0; x < NS; ++x) acc0[x] = acc1[x] = acc2[x] = 0;
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
                    if (SHAPE == 2 && t == 3) v[t][c] = gl::mul(v[t][c], D.lin_coeff);
                }
        }
        u64 lo[NT], hi[NT], dif[NT];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = v[t][c]; hi[t] = v[t][c + 4]; }
            eval_pair<NT, SHAPE, !FIRST>(lo, hi, dif, acc0);
#pragma unroll
            for (int t = 0; t < NT; ++t) v[t][c] = gl::addc(lo[t], gl::mul(r0, dif[t]));
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = v[t][c]; hi[t] = v[t][c + 2]; }
            eval_pair<NT, SHAPE, true>(lo, hi, dif, acc1);
#pragma unroll
            for (int t = 0; t < NT; ++t) v[t][c] = gl::addc(lo[t], gl::mul(r1, dif[t]));
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) { lo[t] = v[t][0]; hi[t] = v[t][1]; }
        eval_pair<NT, SHAPE, true>(lo, hi, dif, acc2);
#pragma unroll
        for (int t = 0; t < NT; ++t) D.dst[t][i] = gl::addc(lo[t], gl::mul(r2, dif[t]));
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int x = 0; x < NS; ++x) {
        const u64 s0 = wave_sum(acc0[x]), s1 = wave_sum(acc1[x]), s2 = wave_sum(acc2[x]);
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
__device__ __forceinline__ void tail_wave_sums(const u64 (&acc)[NS], u64 (*red_par)[NSAMP], int active_waves) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (w < active_waves) {
#pragma unroll
        for (int x = 0; x < NS; ++x) {
            const u64 s = wave_sum(acc[x]);
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
template <int NT, int SHAPE, bool FIRST>
__global__ __launch_bounds__(TAIL_THREADS) void k_tail(const FastDesc D, i64 size, const ChainDesc C, const u64 *part, u64 *out) {
    constexpr int NS = FastShape<NT, SHAPE>::NS;
    constexpr int HALF = TailCap<NT>::HALF;
    __shared__ u64 tab[NT][HALF];
    __shared__ u64 red[2][TAIL_THREADS / 64][NSAMP];
    __shared__ FinishShared sh;
    finish_begin(C, part, sh);

    const int tid = threadIdx.x;
    int k = C.n_prior, par = 0;
    int h = (int)(size >> 1);
    u64 acc[NS];
    u64 lo[NT], hi[NT], dif[NT];
    {
        // first round of this launch: pairs from memory, folded values into LDS
#pragma unroll
        for (int x = 0; x < NS; ++x) acc[x] = 0;
        const u64 r = C.r[k];
        for (int i = tid; i < h; i += TAIL_THREADS) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                lo[t] = fast_load<NT, SHAPE, FIRST>(D, t, i);
                hi[t] = fast_load<NT, SHAPE, FIRST>(D, t, (i64)h + i);
            }
            eval_pair<NT, SHAPE, !FIRST>(lo, hi, dif, acc);
            if (h > 1) {
#pragma unroll
                for (int t = 0; t < NT; ++t) tab[t][i] = gl::addc(lo[t], gl::mul(r, dif[t]));
            }
        }
        const int aw = h >= TAIL_THREADS ? TAIL_THREADS / 64 : (h + 63) >> 6;
        tail_wave_sums<NS>(acc, red[par], aw);
        __syncthreads();
        tail_round_total<NS>(red[par], aw, sh.raw[k]);
        par ^= 1;
    }
    for (h >>= 1; h >= 1; h >>= 1) {
        ++k;
#pragma unroll
        for (int x = 0; x < NS; ++x) acc[x] = 0;
        const u64 r = C.r[k];
        for (int i = tid; i < h; i += TAIL_THREADS) {
#pragma unroll
            for (int t = 0; t < NT; ++t) { lo[t] = tab[t][i]; hi[t] = tab[t][h + i]; }
            eval_pair<NT, SHAPE, true>(lo, hi, dif, acc);
            if (h > 1) {
#pragma unroll
                for (int t = 0; t < NT; ++t) tab[t][i] = gl::addc(lo[t], gl::mul(r, dif[t]));
            }
        }
        const int aw = h >= TAIL_THREADS ? TAIL_THREADS / 64 : (h + 63) >> 6;
        tail_wave_sums<NS>(acc, red[par], aw);
        __syncthreads();
        tail_round_total<NS>(red[par], aw, sh.raw[k]);
        par ^= 1;
    }
    __syncthreads();
    finish_samples(C, sh, out);
}

template <int NT, int SHAPE, bool FIRST>
int launch_pass3(const FastDesc &F, i64 cols, const u64 *r, u64 *part, hipStream_t s) {
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
    hipLaunchKernelGGL((k_pass3<NT, SHAPE, FIRST>), dim3(nb), dim3(BLOCK), 0, s, F, cols, r[0], r[1], r[2], part);
    return nb;
}

// The whole proof of a fixed shape: passes of three rounds while the tables exceed a tail workgroup, then the tail.
// part: workspace of at least n_rounds * MAX_BLOCKS * NSAMP words; C arrives with r, winv, scale, deg, n_rounds set.
template <int NT, int SHAPE>
int prove_fast_shape(FastDesc F, uint64_t *const *work, i64 size, ChainDesc &C, u64 *part, u64 *out, hipStream_t s) {
    constexpr i64 TAIL_MAX = 2 * (i64)TailCap<NT>::HALF;
    int k = 0;
    unsigned off = 0;
    bool first = true;
    C.skip_mask = 0;
    for (int j = 1; j < C.n_rounds; ++j) C.skip_mask |= 1ull << j;
    while (size > TAIL_MAX) {
        const i64 cols = size >> 3;
        const int nb = first ? launch_pass3<NT, SHAPE, true>(F, cols, C.r + k, part + off, s)
                             : launch_pass3<NT, SHAPE, false>(F, cols, C.r + k, part + off, s);
        VI_LAUNCH_CHECK("sumcheck pass (three rounds)");
        for (int j = 0; j < 3; ++j) {
            C.off[k + j] = off + (unsigned)j * (unsigned)nb * NSAMP;
            C.nb[k + j] = (unsigned short)nb;
        }
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

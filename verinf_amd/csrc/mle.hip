// Multilinear helpers that feed and close the sumchecks, on the device:
//   eq_vector(z)[i] = prod_j (bit_j(i) ? z_j : 1 - z_j) (layergkr/logup.py:61-69; its doubling
//                     loop puts z_0 on the LEAST significant index bit);
//   mle_eval(f, r)  = sum_i f[i] * prod_j (bit_j(i) ? r_j : 1 - r_j) with r_0 on the MOST
//                     significant bit (layergkr/sumcheck.py:40-48 computes it by folding f once
//                     per variable).
// Inside this file a point is stored most significant variable first; vi_eq_vector reverses
// its argument unless asked for the mle_eval order.
// The reference builds eq by n doublings of a Python list and evaluates by n folds; here a
// thread derives sixteen entries from one running product -- the n - 4 factors of the bits
// it shares, then a 4-level split e -> (e - e z, e z) -- so eq costs about 3 multiplications
// per entry and one coalesced store, and mle_eval is ONE streaming pass over f that never
// writes eq or any folded table.
#include "common.hpp"
#include "gl_field.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int MAX_VARS = 32;
constexpr int PARTIAL_BLOCKS = 1024;

struct Point {
    u64 z[MAX_VARS];          // canonical
};

// e[j], j < 2^JB: eq entries of the indices (j << (n - JB)) | g.
// Constant indices into pt.z only, so that the by-value argument stays in the kernarg segment.
template <int JB>
__device__ __forceinline__ void eq_entries(const Point &pt, int n, i64 g, u64 (&e)[1 << JB]) {
    u64 prefix = 1;
#pragma unroll
    for (int zi = JB; zi < MAX_VARS; ++zi) {
        if (zi < n) {
            const u64 z = pt.z[zi];
            const bool bit = (g >> (n - 1 - zi)) & 1;
            prefix = gl::mul(prefix, bit ? z : gl::sub(1, z));
        }
    }
    e[0] = prefix;
#pragma unroll
    for (int zi = JB - 1; zi >= 0; --zi) {
        // variable zi is bit (JB - 1 - zi) of j; entries with lower bits of j are already split
        const int step = 1 << (JB - 1 - zi);
        const u64 z = pt.z[zi];
#pragma unroll
        for (int x = 0; x < step; ++x) {
            const u64 hi = gl::mul(e[x], z);
            e[x + step] = hi;
            e[x] = gl::sub(e[x], hi);
        }
    }
}

template <int JB>
__global__ __launch_bounds__(BLOCK) void k_eq_vector(const Point pt, int n, u64 *__restrict__ out) {
    const i64 threads = (i64)1 << (n - JB);
    const i64 g = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (g >= threads) return;
    u64 e[1 << JB];
    eq_entries<JB>(pt, n, g, e);
#pragma unroll
    for (int j = 0; j < (1 << JB); ++j) out[((i64)j << (n - JB)) | g] = e[j];
}

__device__ __forceinline__ u64 block_sum(u64 v, u64 *lds4) {
    for (int off = 32; off > 0; off >>= 1) v = gl::add(v, __shfl_xor(v, off, 64));
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
    __syncthreads();
    u64 r = 0;
    if (threadIdx.x == 0) {
        r = lds4[0];
        for (int i = 1; i < BLOCK / 64; ++i) r = gl::add(r, lds4[i]);
    }
    __syncthreads();
    return r;
}

// partial[row * gridDim.x + block] = sum over this block's share of f_row[i] * eq[i], for the up to TB
// tables row = blockIdx.y * TB + 0 .. TB-1: the eq entries of an index are computed once and used for all
// of them.
constexpr int TB = 4;

template <int JB>
__global__ __launch_bounds__(BLOCK) void k_mle_partial(const Point pt, int n, const u64 *__restrict__ tables, i64 row_stride,
                                                       int n_tables, u64 *__restrict__ partial) {
    __shared__ u64 lds4[BLOCK / 64];
    const i64 threads = (i64)1 << (n - JB);
    const int row0 = blockIdx.y * TB;
    const int rows = n_tables - row0 < TB ? n_tables - row0 : TB;
    u64 acc[TB];
#pragma unroll
    for (int r = 0; r < TB; ++r) acc[r] = 0;
    for (i64 g = (i64)blockIdx.x * BLOCK + threadIdx.x; g < threads; g += (i64)gridDim.x * BLOCK) {
        u64 e[1 << JB];
        eq_entries<JB>(pt, n, g, e);
#pragma unroll
        for (int r = 0; r < TB; ++r) {
            if (r < rows) {
                const u64 *f = tables + (i64)(row0 + r) * row_stride;
                u64 v[1 << JB];
#pragma unroll
                for (int j = 0; j < (1 << JB); ++j) v[j] = f[((i64)j << (n - JB)) | g];
#pragma unroll
                for (int j = 0; j < (1 << JB); ++j) acc[r] = gl::add(acc[r], gl::mul(e[j], v[j]));
            }
        }
    }
#pragma unroll
    for (int r = 0; r < TB; ++r) {
        const u64 s = block_sum(acc[r], lds4);
        if (threadIdx.x == 0 && r < rows) partial[(i64)(row0 + r) * gridDim.x + blockIdx.x] = s;
    }
}

__global__ __launch_bounds__(BLOCK) void k_mle_final(const u64 *__restrict__ partial, int nb, u64 *__restrict__ out) {
    __shared__ u64 lds4[BLOCK / 64];
    u64 acc = 0;
    for (int i = threadIdx.x; i < nb; i += BLOCK) acc = gl::add(acc, partial[(i64)blockIdx.x * nb + i]);
    const u64 r = block_sum(acc, lds4);
    if (threadIdx.x == 0) out[blockIdx.x] = r;
}

int load_point(const char *who, const uint64_t *z, int n, bool msb_first, Point &pt) {
    if (n < 0 || n > MAX_VARS) return vi::fail(VI_EINVAL, "%s: %d variables (0 .. %d supported)", who, n, MAX_VARS);
    if (n > 0 && !z) return vi::fail(VI_EINVAL, "%s: null point", who);
    for (int i = 0; i < MAX_VARS; ++i) pt.z[i] = i < n ? gl::canon(z[msb_first ? i : n - 1 - i]) : 0;
    return VI_OK;
}

}  // namespace

extern "C" {

int vi_eq_vector(const uint64_t *z, int n_vars, int msb_first, uint64_t *out, void *stream) {
    Point pt;
    int rc = load_point("vi_eq_vector", z, n_vars, msb_first != 0, pt);
    if (rc) return rc;
    if (!out) return vi::fail(VI_EINVAL, "vi_eq_vector: null out");
    const int jb = n_vars < 4 ? n_vars : 4;
    const i64 threads = (i64)1 << (n_vars - jb);
    const dim3 grid((unsigned)((threads + BLOCK - 1) / BLOCK)), block(BLOCK);
    hipStream_t s = (hipStream_t)stream;
    switch (jb) {
        case 0: hipLaunchKernelGGL(k_eq_vector<0>, grid, block, 0, s, pt, n_vars, out); break;
        case 1: hipLaunchKernelGGL(k_eq_vector<1>, grid, block, 0, s, pt, n_vars, out); break;
        case 2: hipLaunchKernelGGL(k_eq_vector<2>, grid, block, 0, s, pt, n_vars, out); break;
        case 3: hipLaunchKernelGGL(k_eq_vector<3>, grid, block, 0, s, pt, n_vars, out); break;
        default: hipLaunchKernelGGL(k_eq_vector<4>, grid, block, 0, s, pt, n_vars, out); break;
    }
    VI_LAUNCH_CHECK("k_eq_vector");
    return VI_OK;
}

size_t vi_mle_eval_workspace_bytes(int64_t n_tables) {
    return n_tables <= 0 ? 0 : (size_t)n_tables * PARTIAL_BLOCKS * sizeof(u64);
}

int vi_mle_eval(const uint64_t *tables, int64_t n_tables, int64_t row_stride, const uint64_t *z, int n_vars,
                uint64_t *out, void *ws, size_t ws_bytes, void *stream) {
    Point pt;
    int rc = load_point("vi_mle_eval", z, n_vars, true, pt);
    if (rc) return rc;
    if (n_tables < 0 || n_tables > 65535) return vi::fail(VI_EINVAL, "vi_mle_eval: n_tables = %lld (0 .. 65535)", (long long)n_tables);
    if (n_tables == 0) return VI_OK;
    if (!tables || !out) return vi::fail(VI_EINVAL, "vi_mle_eval: null pointer");
    if (n_tables > 1 && row_stride < ((int64_t)1 << n_vars)) return vi::fail(VI_EINVAL, "vi_mle_eval: row_stride below the table length");
    if (!ws || ws_bytes < vi_mle_eval_workspace_bytes(n_tables)) return vi::fail(VI_ENOMEM, "vi_mle_eval: workspace too small");
    const int jb = n_vars < 4 ? n_vars : 4;
    const i64 threads = (i64)1 << (n_vars - jb);
    i64 nb = (threads + BLOCK - 1) / BLOCK;
    if (nb > PARTIAL_BLOCKS) nb = PARTIAL_BLOCKS;
    const dim3 grid((unsigned)nb, (unsigned)((n_tables + TB - 1) / TB)), block(BLOCK);
    hipStream_t s = (hipStream_t)stream;
    u64 *partial = (u64 *)ws;
    switch (jb) {
        case 0: hipLaunchKernelGGL(k_mle_partial<0>, grid, block, 0, s, pt, n_vars, tables, (i64)row_stride, (int)n_tables, partial); break;
        case 1: hipLaunchKernelGGL(k_mle_partial<1>, grid, block, 0, s, pt, n_vars, tables, (i64)row_stride, (int)n_tables, partial); break;
        case 2: hipLaunchKernelGGL(k_mle_partial<2>, grid, block, 0, s, pt, n_vars, tables, (i64)row_stride, (int)n_tables, partial); break;
        case 3: hipLaunchKernelGGL(k_mle_partial<3>, grid, block, 0, s, pt, n_vars, tables, (i64)row_stride, (int)n_tables, partial); break;
        default: hipLaunchKernelGGL(k_mle_partial<4>, grid, block, 0, s, pt, n_vars, tables, (i64)row_stride, (int)n_tables, partial); break;
    }
    VI_LAUNCH_CHECK("k_mle_partial");
    hipLaunchKernelGGL(k_mle_final, dim3((unsigned)n_tables), block, 0, s, (const u64 *)partial, (int)nb, out);
    VI_LAUNCH_CHECK("k_mle_final");
    return VI_OK;
}

}  // extern "C"

// Dense field products over Goldilocks: C = A B, w = M v, and Horner evaluation.
//
// The reference kernels reduce after every term (s = add(s, mul(a, b)),
// prover/kernels/gl_matmul.cuh:29-59).  Here a dot product is accumulated as an exact
// integer -- 128-bit running sum plus a count of its wrap-arounds -- and reduced once
// at the end: per term four v_mad_u64_u32 and a carry chain instead of a full modular
// multiply-add.  Results are the same canonical residues.
//
// k_matmul is built for the shape the prover uses it in: few rows of A (1 for the
// projection seam `chi^T W`, layergkr/projection.py:150-167, and for combine_t,
// layergkr/gpu.py:301-308) against a tall B that is streamed once per row of A.  Lanes
// run along the columns of B (coalesced), the inner dimension is split across
// workgroups so that even a single output row fills the GPU, and a second small
// kernel adds the partial sums.
#include "common.hpp"
#include "gl_field.hpp"

namespace {

constexpr int BLOCK = 256;

// exact running sum of 64x64-bit products: value = lo + hi*2^64 + wraps*2^128
struct WideAcc {
    u64 lo = 0, hi = 0;
    u32 wraps = 0;
    __device__ __forceinline__ void fma(u64 a, u64 b) {
        u64 pl, ph;
        gl::mul_wide(a, b, pl, ph);
        u64 nl = lo + pl;
        u64 c = nl < pl ? 1 : 0;
        u64 nh = hi + ph;
        u32 w = nh < ph ? 1u : 0u;
        u64 nh2 = nh + c;
        w += nh2 < nh ? 1u : 0u;
        lo = nl;
        hi = nh2;
        wraps += w;
    }
    // 2^128 = 2^96 * 2^32 = -2^32 (mod p)
    __device__ __forceinline__ u64 reduce() const {
        u64 r = gl::reduce128(lo, hi);
        return gl::sub(r, gl::mul((u64)wraps, (u64)1 << 32));
    }
};

// partial[s][i][j] = sum over the s-th slice of the inner dimension of A[i][l] * B[l][j]
// A thread owns column j for MB consecutive rows of A, so B is streamed once per MB rows, and requests UN
// elements of its column before it uses the first (one row of A against a 4096 x 65536 B: 5.5 TB/s with eight
// loads in flight, 4.9 TB/s with the loop left to the compiler).  B is read once and with the streaming hint: the
// projections of a layer's weight codewords 4.19-4.31 -> 3.87 ms, 6.3 TB/s, what a kernel that only reads reaches.
template <int MB, int UN>
__global__ __launch_bounds__(BLOCK) void k_matmul(const u64 *__restrict__ A, const u64 *__restrict__ B, u64 *__restrict__ out,
                                                  i64 m, i64 k, i64 n, i64 k_per_split) {
    const i64 j = (i64)blockIdx.x * BLOCK + threadIdx.x;
    const i64 i0 = (i64)blockIdx.y * MB, s = blockIdx.z;
    if (j >= n) return;
    const i64 l0 = s * k_per_split, l1 = (l0 + k_per_split < k) ? l0 + k_per_split : k;
    const int rows = (m - i0 < MB) ? (int)(m - i0) : MB;
    WideAcc acc[MB];
    i64 l = l0;
    for (; l + UN <= l1; l += UN) {
        u64 b[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) b[u] = __builtin_nontemporal_load(&B[(l + u) * n + j]);
#pragma unroll
        for (int r = 0; r < MB; ++r) {
            if (r < rows) {
                const u64 *a = A + (i0 + r) * k + l;
#pragma unroll
                for (int u = 0; u < UN; ++u) acc[r].fma(a[u], b[u]);
            }
        }
    }
    for (; l < l1; ++l) {
        const u64 b = B[l * n + j];
#pragma unroll
        for (int r = 0; r < MB; ++r)
            if (r < rows) acc[r].fma(A[(i0 + r) * k + l], b);
    }
#pragma unroll
    for (int r = 0; r < MB; ++r)
        if (r < rows) out[(s * m + i0 + r) * n + j] = acc[r].reduce();
}

// an empty inner dimension gives the zero matrix (a kernel, not a memset: the call may be under stream capture)
__global__ __launch_bounds__(BLOCK) void k_zero(u64 *__restrict__ out, i64 n) {
    const i64 e = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (e < n) out[e] = 0;
}

__global__ __launch_bounds__(BLOCK) void k_add_partials(const u64 *__restrict__ partial, u64 *__restrict__ out, i64 mn, int splits) {
    const i64 e = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (e >= mn) return;
    u64 acc = partial[e];
    for (int s = 1; s < splits; ++s) acc = gl::add(acc, partial[(i64)s * mn + e]);
    out[e] = acc;
}

// TPR threads per row of M (a wavefront, or the whole workgroup when there are too few rows for a wavefront
// each to fill the GPU): they stride over the columns with four row elements requested before the first is
// used, exact accumulation, shuffle tree, and for a workgroup a last sum over its wavefronts in LDS.
// 1024 x 262144: 2.01 ms with a wavefront per row and one load in flight, 0.72 ms with four, TPR = 256 below.
// The matrix is read once, with the streaming hint (4096 x 65536: 4.7 -> 4.8 TB/s, 65536 x 4096: 5.0 -> 5.2 TB/s).
template <int TPR>
__global__ __launch_bounds__(BLOCK) void k_matvec(const u64 *__restrict__ M, const u64 *__restrict__ v, u64 *__restrict__ w, i64 m, i64 n) {
    __shared__ u64 part[BLOCK / 64];
    const int lane = threadIdx.x & 63, t = threadIdx.x & (TPR - 1);
    const i64 row = ((i64)blockIdx.x * BLOCK + threadIdx.x) / TPR;
    u64 x = 0;
    if (row < m) {
        const u64 *r = M + row * n;
        WideAcc acc;
        i64 j = t;
        for (; j + 3 * TPR < n; j += 4 * TPR) {
            u64 a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) { a[u] = __builtin_nontemporal_load(&r[j + u * TPR]); b[u] = v[j + u * TPR]; }
#pragma unroll
            for (int u = 0; u < 4; ++u) acc.fma(a[u], b[u]);
        }
        for (; j < n; j += TPR) acc.fma(r[j], v[j]);
        x = acc.reduce();
    }
    for (int off = 32; off > 0; off >>= 1) x = gl::add(x, __shfl_xor(x, off, 64));
    if (TPR == 64) {
        if (lane == 0 && row < m) w[row] = x;
    } else {
        if (lane == 0) part[threadIdx.x >> 6] = x;
        __syncthreads();
        if (threadIdx.x == 0 && row < m) {
            u64 sum = part[0];
            for (int i = 1; i < BLOCK / 64; ++i) sum = gl::add(sum, part[i]);
            w[row] = sum;
        }
    }
}

// out[r][p] = sum_i coeffs[r][i] x_p^i by Horner's rule (prover/kernels/gl_extras.cuh:93-108)
__global__ __launch_bounds__(BLOCK) void k_poly_eval(const u64 *__restrict__ coeffs, i64 m, i64 d, const u64 *__restrict__ points, i64 kp,
                                                     u64 *__restrict__ out) {
    const i64 p = (i64)blockIdx.x * BLOCK + threadIdx.x;
    const i64 r = blockIdx.y;
    if (p >= kp) return;
    const u64 x = points[p];
    const u64 *row = coeffs + r * d;
    u64 acc = 0;
    for (i64 i = d - 1; i >= 0; --i) acc = gl::add(gl::mul(acc, x), row[i]);
    out[r * kp + p] = acc;
}

// rows of A a thread takes together
inline int pick_mb(i64 m) { return m >= 4 ? 4 : (m >= 2 ? 2 : 1); }

int pick_splits(i64 m, i64 k, i64 n) {
    i64 col_blocks = (n + BLOCK - 1) / BLOCK;
    i64 row_blocks = (m + pick_mb(m) - 1) / pick_mb(m);
    i64 want = 4096 / (col_blocks * row_blocks > 0 ? col_blocks * row_blocks : 1);      // aim at a few thousand workgroups
    i64 cap = k / 32;                                                  // at least 32 terms per slice
    if (want > cap) want = cap;
    if (want > 64) want = 64;
    return (int)(want < 1 ? 1 : want);
}

}  // namespace

extern "C" {

size_t vi_gl_matmul_workspace_bytes(int64_t m, int64_t k, int64_t n) {
    if (m <= 0 || k <= 0 || n <= 0) return 0;
    int s = pick_splits(m, k, n);
    return s > 1 ? (size_t)s * (size_t)m * (size_t)n * sizeof(u64) : 0;
}

int vi_gl_matmul(const uint64_t *A, const uint64_t *B, uint64_t *C, int64_t m, int64_t k, int64_t n, void *ws,
                 size_t ws_bytes, void *stream) {
    if (m < 0 || k < 0 || n < 0) return vi::fail(VI_EINVAL, "vi_gl_matmul: negative dimension");
    if (m == 0 || n == 0) return VI_OK;
    if (!C || (k > 0 && (!A || !B))) return vi::fail(VI_EINVAL, "vi_gl_matmul: null pointer");
    if (m > 65535) return vi::fail(VI_EINVAL, "vi_gl_matmul: at most 65535 rows of A per call, got %lld", (long long)m);
    hipStream_t s = (hipStream_t)stream;
    if (k == 0) {
        const i64 mn = m * n;
        hipLaunchKernelGGL(k_zero, dim3((unsigned)((mn + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, s, C, mn);
        VI_LAUNCH_CHECK("k_zero");
        return VI_OK;
    }
    const int splits = pick_splits(m, k, n);
    if (splits > 1 && (!ws || ws_bytes < vi_gl_matmul_workspace_bytes(m, k, n)))
        return vi::fail(VI_ENOMEM, "vi_gl_matmul: workspace below %zu bytes", vi_gl_matmul_workspace_bytes(m, k, n));
    const i64 per = (k + splits - 1) / splits;
    const int mb = pick_mb(m);
    dim3 grid((unsigned)((n + BLOCK - 1) / BLOCK), (unsigned)((m + mb - 1) / mb), (unsigned)splits);
    u64 *dst = splits > 1 ? (u64 *)ws : C;
    if (mb == 1) hipLaunchKernelGGL((k_matmul<1, 8>), grid, dim3(BLOCK), 0, s, A, B, dst, (i64)m, (i64)k, (i64)n, per);
    if (mb == 2) hipLaunchKernelGGL((k_matmul<2, 4>), grid, dim3(BLOCK), 0, s, A, B, dst, (i64)m, (i64)k, (i64)n, per);
    if (mb == 4) hipLaunchKernelGGL((k_matmul<4, 4>), grid, dim3(BLOCK), 0, s, A, B, dst, (i64)m, (i64)k, (i64)n, per);
    VI_LAUNCH_CHECK("k_matmul");
    if (splits > 1) {
        const i64 mn = m * n;
        hipLaunchKernelGGL(k_add_partials, dim3((unsigned)((mn + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, s, (const u64 *)ws, C, mn, splits);
        VI_LAUNCH_CHECK("k_add_partials");
    }
    return VI_OK;
}

int vi_gl_matvec(const uint64_t *M, const uint64_t *v, uint64_t *w, int64_t m, int64_t n, void *stream) {
    if (m < 0 || n < 0) return vi::fail(VI_EINVAL, "vi_gl_matvec: negative dimension");
    if (m == 0) return VI_OK;
    if (!w || (n > 0 && (!M || !v))) return vi::fail(VI_EINVAL, "vi_gl_matvec: null pointer");
    const bool wide = m < 8192 && n >= 4096;          // few long rows: a workgroup per row
    const i64 blocks = wide ? m : (m * 64 + BLOCK - 1) / BLOCK;
    if (blocks > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "vi_gl_matvec: too many rows");
    if (wide) hipLaunchKernelGGL(k_matvec<BLOCK>, dim3((unsigned)blocks), dim3(BLOCK), 0, (hipStream_t)stream, M, v, w, (i64)m, (i64)n);
    else hipLaunchKernelGGL(k_matvec<64>, dim3((unsigned)blocks), dim3(BLOCK), 0, (hipStream_t)stream, M, v, w, (i64)m, (i64)n);
    VI_LAUNCH_CHECK("k_matvec");
    return VI_OK;
}

int vi_poly_eval(const uint64_t *coeffs, int64_t m, int64_t d, const uint64_t *points, int64_t k, uint64_t *out,
                 void *stream) {
    if (m < 0 || d < 0 || k < 0) return vi::fail(VI_EINVAL, "vi_poly_eval: negative dimension");
    if (m == 0 || k == 0) return VI_OK;
    if (!out || !points || (d > 0 && !coeffs)) return vi::fail(VI_EINVAL, "vi_poly_eval: null pointer");
    if (m > 65535) return vi::fail(VI_EINVAL, "vi_poly_eval: at most 65535 polynomials per call, got %lld", (long long)m);
    dim3 grid((unsigned)((k + BLOCK - 1) / BLOCK), (unsigned)m);
    hipLaunchKernelGGL(k_poly_eval, grid, dim3(BLOCK), 0, (hipStream_t)stream, coeffs, (i64)m, (i64)d, points, (i64)k, out);
    VI_LAUNCH_CHECK("k_poly_eval");
    return VI_OK;
}

}  // extern "C"

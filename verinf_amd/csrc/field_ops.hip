// Elementwise Goldilocks kernels and the field sum reduction.
//
// All of these are pure HBM streaming (24 B per element for a binary op) with a
// handful of integer VALU ops per element; they use 64-bit indexing and a
// grid-stride loop sized to keep every CU busy (the reference kernels index with
// int, prover/cuda_primitives.py:208-233).
#include "common.hpp"
#include "gl_field.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int MAX_BLOCKS = 256 * 16;      // 16 workgroups per CU

inline unsigned grid_for(i64 n) {
    i64 b = (n + BLOCK - 1) / BLOCK;
    return (unsigned)(b < 1 ? 1 : (b > MAX_BLOCKS ? MAX_BLOCKS : b));
}

template <int OP>
__device__ __forceinline__ u64 apply(u64 a, u64 b) {
    return OP == 0 ? gl::add(a, b) : OP == 1 ? gl::sub(a, b) : gl::mul(a, b);
}

template <int OP>
__global__ __launch_bounds__(BLOCK) void k_binop(const u64 *a, const u64 *b, u64 *out, i64 n) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride)
        __builtin_nontemporal_store(apply<OP>(__builtin_nontemporal_load(a + i), __builtin_nontemporal_load(b + i)), out + i);
}

// two elements per lane through 16-byte accesses (operands 16-byte aligned, n even)
template <int OP>
__global__ __launch_bounds__(BLOCK) void k_binop_v2(const ulonglong2 *a, const ulonglong2 *b, ulonglong2 *out, i64 n2) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n2; i += stride) {
        // operands read once, result not read back by this launch: streaming hints (2^24 elements 5.1 -> 5.9 TB/s,
        // 2^27 4.40 -> 4.50 TB/s)
        typedef u64 v2 __attribute__((ext_vector_type(2)));
        const v2 xv = __builtin_nontemporal_load(reinterpret_cast<const v2 *>(a + i));
        const v2 yv = __builtin_nontemporal_load(reinterpret_cast<const v2 *>(b + i));
        v2 rv;
        rv.x = apply<OP>(xv.x, yv.x);
        rv.y = apply<OP>(xv.y, yv.y);
        __builtin_nontemporal_store(rv, reinterpret_cast<v2 *>(out + i));
    }
}

template <int OP>
__global__ __launch_bounds__(BLOCK) void k_binop_bcast(const u64 *a, const u64 *b, i64 period, u64 *out, i64 n) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride) out[i] = apply<OP>(a[i], b[i % period]);
}

__global__ __launch_bounds__(BLOCK) void k_unop(int op, const u64 *a, u64 arg, u64 *out, i64 n) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride) {
        u64 v = a[i];
        out[i] = op == 0 ? gl::neg(v) : gl::pow(v, arg);
    }
}

// One device field primitive applied elementwise, for the test-suite: the transforms use these through fully
// unrolled code with compile-time exponents, so this is the only place they can be driven with chosen operands.
template <int E>
__device__ __forceinline__ u64 shift_by(u64 v, int e) {
    if constexpr (E >= 96) return 0;
    else {
        if (e == E) return gl::mul_pow2c<E>(v);
        return shift_by<E + 1>(v, e);
    }
}

// the same through the form used inside the coset loop of the fused LDE launch: any exponent below 192, 2^96 = -1
template <int E>
__device__ __forceinline__ u64 shift_pinned_by(u64 v, int e) {
    if constexpr (E >= 192) return 0;
    else {
        if (e == E) return gl::mul_pow2c_pinned<E>(v);
        return shift_pinned_by<E + 1>(v, e);
    }
}

__global__ __launch_bounds__(BLOCK) void k_probe(int op, const u64 *a, const u64 *b, u64 *out, i64 n) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride) {
        const u64 x = a[i], y = b ? b[i] : 0;
        u64 s, d, r;
        gl::bfly(x, y, s, d);
        if (op == 0) r = gl::addc(x, y);
        else if (op == 1) r = gl::sub(x, y);
        else if (op == 2) r = s;
        else if (op == 3) r = d;
        else if (op == 4) r = gl::canon(x);
        else if (op == 5) r = gl::mul(x, y);
        else if (op == 6) r = gl::reduce128(x, y);
        else if (op == 7) r = gl::canon(gl::mul_lazy(x, y));
        else if (op == 8) r = gl::mul_add(x, y, ((x << 17) | (x >> 47)) ^ y);
        else if (op == 9) r = gl::canon(gl::mul_add_lazy(x, y, ((x << 17) | (x >> 47)) ^ y));
        else if (op == 10 || op == 11) {
            gl::Wide A;
            gl::wide_zero(A);
            if (op == 10) {
                gl::wide_mul_acc(A, x, y);
                gl::wide_mul_acc(A, y, y);
                gl::wide_mul_acc(A, x, x);
                gl::wide_mul_acc(A, ~x, ~y);
                gl::wide_mul_acc(A, ~0ull, ~0ull);
            } else {
                for (int k = 0; k < 40; ++k) gl::wide_mul_acc(A, x, y);      // carries into the fifth word
            }
            r = gl::wide_reduce(A);
        }
        else if (op >= 300) r = shift_pinned_by<0>(x, op - 300);
        else r = shift_by<0>(x, op - 100);
        out[i] = r;
    }
}

// Inverses of a whole array by Montgomery's trick in registers (the batching of
// layergkr/field.py:84-101 at the scale of one thread): a thread takes INV_E elements, one
// from each of INV_E equal slabs of the array so that a wavefront's accesses stay contiguous,
// multiplies them up, inverts the product once (74 multiplications) and peels the single
// inverses off with two multiplications each.  Zeros are taken out of the product and map
// to zero, so every output equals the Fermat power a^(p-2) of the reference kernel
// (prover/cuda_primitives.py:289-303).
constexpr int INV_E = 8;

__global__ __launch_bounds__(BLOCK) void k_inv_batched(const u64 *a, u64 *out, i64 n, i64 groups) {
    const i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 g = (i64)blockIdx.x * BLOCK + threadIdx.x; g < groups; g += stride) {
        u64 x[INV_E], pre[INV_E];
        unsigned zero = 0;
#pragma unroll
        for (int j = 0; j < INV_E; ++j) {
            const i64 i = (i64)j * groups + g;
            u64 v = i < n ? gl::canon(a[i]) : 1;
            if (v == 0) { zero |= 1u << j; v = 1; }
            x[j] = v;
        }
        pre[0] = x[0];
#pragma unroll
        for (int j = 1; j < INV_E; ++j) pre[j] = gl::mul(pre[j - 1], x[j]);
        u64 acc = gl::inv(pre[INV_E - 1]);
#pragma unroll
        for (int j = INV_E - 1; j >= 0; --j) {
            const u64 r = j ? gl::mul(acc, pre[j - 1]) : acc;
            if (j) acc = gl::mul(acc, x[j]);
            const i64 i = (i64)j * groups + g;
            if (i < n) out[i] = (zero >> j) & 1 ? 0 : r;
        }
    }
}

__global__ __launch_bounds__(BLOCK) void k_axpy(u64 *y, u64 alpha, const u64 *x, i64 n) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride) y[i] = gl::add(y[i], gl::mul(alpha, x[i]));
}

__device__ __forceinline__ u64 wave_sum(u64 v) {
    for (int off = 32; off > 0; off >>= 1) v = gl::add(v, __shfl_xor(v, off, 64));
    return v;
}

// block-wide field sum; the result is valid in thread 0
__device__ __forceinline__ u64 block_sum(u64 v, u64 *lds4) {
    v = wave_sum(v);
    int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) lds4[w] = v;
    __syncthreads();
    u64 r = 0;
    if (threadIdx.x == 0) {
        r = lds4[0];
        for (int i = 1; i < BLOCK / 64; ++i) r = gl::add(r, lds4[i]);
    }
    __syncthreads();
    return r;
}

constexpr int SUM_BLOCKS = 1024;

__global__ __launch_bounds__(BLOCK) void k_sum_partial(const u64 *a, i64 n, u64 *partial) {
    __shared__ u64 lds4[BLOCK / 64];
    i64 stride = (i64)gridDim.x * BLOCK;
    u64 acc = 0;
    i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {     // four loads in flight
        u64 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(&a[i + u * stride]);     // read once: streaming
#pragma unroll
        for (int u = 0; u < 4; ++u) acc = gl::add(acc, v[u] >= gl::P ? v[u] - gl::P : v[u]);
    }
    for (; i < n; i += stride) {
        u64 v = a[i];
        acc = gl::add(acc, v >= gl::P ? v - gl::P : v);
    }
    u64 r = block_sum(acc, lds4);
    if (threadIdx.x == 0) partial[blockIdx.x] = r;
}

__global__ __launch_bounds__(BLOCK) void k_sum_final(const u64 *partial, int nb, u64 *out) {
    __shared__ u64 lds4[BLOCK / 64];
    u64 acc = 0;
    for (int i = threadIdx.x; i < nb; i += BLOCK) acc = gl::add(acc, partial[i]);
    u64 r = block_sum(acc, lds4);
    if (threadIdx.x == 0) out[0] = r;
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

extern "C" {

const char *vi_last_error(void) { return vi::err_buf(); }
const char *vi_version(void) { return "0.2"; }

int vi_gl_binop(int op, const uint64_t *a, const uint64_t *b, uint64_t *out, int64_t n, void *stream) {
    if (op < 0 || op > 2) return vi::fail(VI_EINVAL, "vi_gl_binop: op %d", op);
    if (n < 0) return vi::fail(VI_EINVAL, "vi_gl_binop: n = %lld", (long long)n);
    if (n == 0) return VI_OK;
    if (!a || !b || !out) return vi::fail(VI_EINVAL, "vi_gl_binop: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if ((n & 1) == 0 && aligned16(a) && aligned16(b) && aligned16(out)) {
        i64 n2 = n / 2;
        auto A = (const ulonglong2 *)a, B = (const ulonglong2 *)b;
        auto O = (ulonglong2 *)out;
        if (op == 0) hipLaunchKernelGGL(k_binop_v2<0>, dim3(grid_for(n2)), dim3(BLOCK), 0, s, A, B, O, n2);
        if (op == 1) hipLaunchKernelGGL(k_binop_v2<1>, dim3(grid_for(n2)), dim3(BLOCK), 0, s, A, B, O, n2);
        if (op == 2) hipLaunchKernelGGL(k_binop_v2<2>, dim3(grid_for(n2)), dim3(BLOCK), 0, s, A, B, O, n2);
    } else {
        if (op == 0) hipLaunchKernelGGL(k_binop<0>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, out, (i64)n);
        if (op == 1) hipLaunchKernelGGL(k_binop<1>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, out, (i64)n);
        if (op == 2) hipLaunchKernelGGL(k_binop<2>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, out, (i64)n);
    }
    VI_LAUNCH_CHECK("k_binop");
    return VI_OK;
}

int vi_gl_binop_bcast(int op, const uint64_t *a, const uint64_t *b, int64_t period, uint64_t *out,
                      int64_t n, void *stream) {
    if (op < 0 || op > 2) return vi::fail(VI_EINVAL, "vi_gl_binop_bcast: op %d", op);
    if (n < 0 || period <= 0) return vi::fail(VI_EINVAL, "vi_gl_binop_bcast: n = %lld period = %lld", (long long)n, (long long)period);
    if (n == 0) return VI_OK;
    if (!a || !b || !out) return vi::fail(VI_EINVAL, "vi_gl_binop_bcast: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (op == 0) hipLaunchKernelGGL(k_binop_bcast<0>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, (i64)period, out, (i64)n);
    if (op == 1) hipLaunchKernelGGL(k_binop_bcast<1>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, (i64)period, out, (i64)n);
    if (op == 2) hipLaunchKernelGGL(k_binop_bcast<2>, dim3(grid_for(n)), dim3(BLOCK), 0, s, a, b, (i64)period, out, (i64)n);
    VI_LAUNCH_CHECK("k_binop_bcast");
    return VI_OK;
}

int vi_gl_unop(int op, const uint64_t *a, uint64_t arg, uint64_t *out, int64_t n, void *stream) {
    if (op < 0 || op > 2) return vi::fail(VI_EINVAL, "vi_gl_unop: op %d", op);
    if (n < 0) return vi::fail(VI_EINVAL, "vi_gl_unop: n = %lld", (long long)n);
    if (n == 0) return VI_OK;
    if (!a || !out) return vi::fail(VI_EINVAL, "vi_gl_unop: null pointer");
    if (op == 2) {
        const i64 groups = (n + INV_E - 1) / INV_E;
        hipLaunchKernelGGL(k_inv_batched, dim3(grid_for(groups)), dim3(BLOCK), 0, (hipStream_t)stream, a, out, (i64)n, groups);
        VI_LAUNCH_CHECK("k_inv_batched");
        return VI_OK;
    }
    hipLaunchKernelGGL(k_unop, dim3(grid_for(n)), dim3(BLOCK), 0, (hipStream_t)stream, op, a, (u64)arg, out, (i64)n);
    VI_LAUNCH_CHECK("k_unop");
    return VI_OK;
}

int vi_gl_axpy(uint64_t *y, uint64_t alpha, const uint64_t *x, int64_t n, void *stream) {
    if (n < 0) return vi::fail(VI_EINVAL, "vi_gl_axpy: n = %lld", (long long)n);
    if (n == 0) return VI_OK;
    if (!y || !x) return vi::fail(VI_EINVAL, "vi_gl_axpy: null pointer");
    hipLaunchKernelGGL(k_axpy, dim3(grid_for(n)), dim3(BLOCK), 0, (hipStream_t)stream, y, (u64)alpha, x, (i64)n);
    VI_LAUNCH_CHECK("k_axpy");
    return VI_OK;
}

int vi_gl_probe(int op, const uint64_t *a, const uint64_t *b, uint64_t *out, int64_t n, void *stream) {
    const bool shift = (op >= 100 && op < 196) || (op >= 300 && op < 492);
    if (!shift && (op < 0 || op > 11)) return vi::fail(VI_EINVAL, "vi_gl_probe: op = %d", op);
    if (n < 0) return vi::fail(VI_EINVAL, "vi_gl_probe: n = %lld", (long long)n);
    if (n == 0) return VI_OK;
    const bool needs_b = !shift && op != 4;
    if (!a || !out || (needs_b && !b)) return vi::fail(VI_EINVAL, "vi_gl_probe: null pointer");
    hipLaunchKernelGGL(k_probe, dim3(grid_for(n)), dim3(BLOCK), 0, (hipStream_t)stream, op, a, needs_b ? b : nullptr, out, (i64)n);
    VI_LAUNCH_CHECK("k_probe");
    return VI_OK;
}

size_t vi_gl_sum_workspace_bytes(int64_t n) {
    (void)n;
    return SUM_BLOCKS * sizeof(u64);
}

int vi_gl_sum(const uint64_t *a, int64_t n, uint64_t *out, void *ws, size_t ws_bytes, void *stream) {
    if (n < 0) return vi::fail(VI_EINVAL, "vi_gl_sum: n = %lld", (long long)n);
    if (!out || (n > 0 && !a)) return vi::fail(VI_EINVAL, "vi_gl_sum: null pointer");
    if (!ws || ws_bytes < SUM_BLOCKS * sizeof(u64)) return vi::fail(VI_ENOMEM, "vi_gl_sum: workspace below %zu bytes", SUM_BLOCKS * sizeof(u64));
    i64 b = (n + BLOCK - 1) / BLOCK;
    int nb = (int)(b < 1 ? 1 : (b > SUM_BLOCKS ? SUM_BLOCKS : b));
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(k_sum_partial, dim3(nb), dim3(BLOCK), 0, s, a, (i64)n, (u64 *)ws);
    VI_LAUNCH_CHECK("k_sum_partial");
    hipLaunchKernelGGL(k_sum_final, dim3(1), dim3(BLOCK), 0, s, (const u64 *)ws, nb, out);
    VI_LAUNCH_CHECK("k_sum_final");
    return VI_OK;
}

}  // extern "C"

// Fused K-quant super-block -> Goldilocks field decode.
//
// The value map is the one the reference declares to be the committed model
// (prover/kquant_cuda.py:42-111): fp16 d/dmin widened to fp32, the fp32 expression
// (d*sc)*q - dmin*mn (Q4_K, Q5_K) or (d*sc)*q (Q6_K) with every operation rounded
// separately (no FMA contraction -- this file is built with -ffp-contract=off and
// uses the explicit round-to-nearest intrinsics), then round-half-even of
// double(v)*S, negatives stored as p - |x|.
//
// k_kq<QT>: one wavefront per 256-weight super-block.  Lane l decodes weights
// {2l, 2l+1} and {128+2l, 129+2l} (decode_block<QT>): for Q4_K it needs two 16-bit quant
// loads, the 4-byte d/dmin header and the 12 scale bytes (three dwords, identical for all
// lanes of the wave), and issues two 16-byte stores, so each store instruction writes 1 KiB
// of consecutive output.  The reference uses one thread per weight with byte loads.
//
// k_kq_t<QT>: the same decode, written as the transposed matrix through an LDS tile.
//
// k_generic: one thread per weight, byte loads, any alignment (buffers whose base is not
// aligned for the wavefront kernels).
#include "common.hpp"
#include "gl_field.hpp"

namespace {

constexpr int BLOCK = 256;

__device__ __forceinline__ float half_bits_to_float(u32 bits) {
    _Float16 h = __builtin_bit_cast(_Float16, (unsigned short)bits);
    return (float)h;
}

__device__ __forceinline__ u64 to_field(float v, double S) {
    long long x = __double2ll_rn(__dmul_rn((double)v, S));
    return x >= 0 ? (u64)x : gl::P - (u64)(-x);
}

// 6-bit (scale, min) of sub-block s from the 12 packed bytes held as three dwords
__device__ __forceinline__ void scale_min(u32 w0, u32 w1, u32 w2, int s, u32 &sc, u32 &mn) {
    // bytes 0..3 = w0, 4..7 = w1, 8..11 = w2
    int j = s & 3, sh = 8 * j;
    u32 b_lo = (w0 >> sh) & 0xFF, b_mid = (w1 >> sh) & 0xFF, b_hi = (w2 >> sh) & 0xFF;
    if (s < 4) {
        sc = b_lo & 0x3F;
        mn = b_mid & 0x3F;
    } else {
        sc = (b_hi & 0x0F) | ((b_lo >> 2) & 0x30);
        mn = (b_hi >> 4) | ((b_mid >> 2) & 0x30);
    }
}

// 16-byte streaming store: the decoded matrix is written once and not read back by this kernel, so it should
// not displace anything in the L2 (measured on 4096 x 11008 Q4_K: 0.083 -> 0.067 ms).
__device__ __forceinline__ void stream_store(ulonglong2 *p, ulonglong2 v) {
    __builtin_nontemporal_store(v.x, &p->x);
    __builtin_nontemporal_store(v.y, &p->y);
}

__device__ __forceinline__ float dequant(float d, float dmin, u32 sc, u32 mn, u32 q) {
    return __fsub_rn(__fmul_rn(__fmul_rn(d, (float)sc), (float)q), __fmul_rn(dmin, (float)mn));
}

// The four weights a lane decodes in every layout: 2l, 2l+1 (lo) and 128+2l, 129+2l (hi) of its super-block.
struct Quad {
    ulonglong2 lo, hi;
};

template <int QT>
__device__ __forceinline__ Quad decode_block(const unsigned char *p, int lane, double S);

template <>
__device__ __forceinline__ Quad decode_block<4>(const unsigned char *p, int lane, double S) {
    const u32 *hdr = (const u32 *)p;
    u32 h = hdr[0], w0 = hdr[1], w1 = hdr[2], w2 = hdr[3];
    float d = half_bits_to_float(h & 0xFFFF), dmin = half_bits_to_float(h >> 16);
    int s = lane >> 4;                                  // sub-block of weights 2l, 2l+1
    int nib = 4 * (s & 1);
    const unsigned short *qs = (const unsigned short *)(p + 16 + (lane >> 5) * 32 + ((2 * lane) & 31));
    u32 qa = qs[0], qb = qs[32];                        // +64 bytes: same position, sub-block s+4
    u32 sc, mn;
    Quad r;
    scale_min(w0, w1, w2, s, sc, mn);
    r.lo.x = to_field(dequant(d, dmin, sc, mn, (qa >> nib) & 0xF), S);
    r.lo.y = to_field(dequant(d, dmin, sc, mn, (qa >> (8 + nib)) & 0xF), S);
    scale_min(w0, w1, w2, s + 4, sc, mn);
    r.hi.x = to_field(dequant(d, dmin, sc, mn, (qb >> nib) & 0xF), S);
    r.hi.y = to_field(dequant(d, dmin, sc, mn, (qb >> (8 + nib)) & 0xF), S);
    return r;
}

// Q5_K (176 B: d, dmin, 12 scale bytes, 32 bytes of fifth bits, 128 quant bytes): as Q4_K, plus
// one 16-bit load of the fifth-bit bytes of weights (2l, 2l+1) mod 32; bit s belongs to sub-block s.
template <>
__device__ __forceinline__ Quad decode_block<5>(const unsigned char *p, int lane, double S) {
    const u32 *hdr = (const u32 *)p;
    u32 h = hdr[0], w0 = hdr[1], w1 = hdr[2], w2 = hdr[3];
    float d = half_bits_to_float(h & 0xFFFF), dmin = half_bits_to_float(h >> 16);
    int s = lane >> 4;
    int nib = 4 * (s & 1);
    const u32 qh = *(const unsigned short *)(p + 16 + ((2 * lane) & 31));
    const unsigned short *qs = (const unsigned short *)(p + 48 + (lane >> 5) * 32 + ((2 * lane) & 31));
    u32 qa = qs[0], qb = qs[32];
    u32 sc, mn;
    Quad r;
    scale_min(w0, w1, w2, s, sc, mn);
    r.lo.x = to_field(dequant(d, dmin, sc, mn, ((qa >> nib) & 0xF) | (((qh >> s) & 1) << 4)), S);
    r.lo.y = to_field(dequant(d, dmin, sc, mn, ((qa >> (8 + nib)) & 0xF) | (((qh >> (8 + s)) & 1) << 4)), S);
    scale_min(w0, w1, w2, s + 4, sc, mn);
    r.hi.x = to_field(dequant(d, dmin, sc, mn, ((qb >> nib) & 0xF) | (((qh >> (s + 4)) & 1) << 4)), S);
    r.hi.y = to_field(dequant(d, dmin, sc, mn, ((qb >> (8 + nib)) & 0xF) | (((qh >> (12 + s)) & 1) << 4)), S);
    return r;
}

// Q6_K (210 B: 128 low-nibble bytes, 64 bytes of two-bit highs, 16 int8 scales, d).  210 is not a
// multiple of four, so a block is only 2-byte aligned: 16-bit loads throughout.
template <>
__device__ __forceinline__ Quad decode_block<6>(const unsigned char *p, int lane, double S) {
    const float d = half_bits_to_float(*(const unsigned short *)(p + 208));
    const int nib = 4 * (lane >> 5), two = 2 * ((lane >> 4) & 3);
    Quad r;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const u32 ql = *(const unsigned short *)(p + half * 64 + ((2 * lane) & 63));
        const u32 qh = *(const unsigned short *)(p + 128 + half * 32 + ((2 * lane) & 31));
        const int sc = (int)(signed char)p[192 + half * 8 + (lane >> 3)];
        const float ds = __fmul_rn(d, (float)sc);
        const int q0 = (int)(((ql >> nib) & 0xF) | (((qh >> two) & 3) << 4)) - 32;
        const int q1 = (int)(((ql >> (8 + nib)) & 0xF) | (((qh >> (8 + two)) & 3) << 4)) - 32;
        ulonglong2 v;
        v.x = to_field(__fmul_rn(ds, (float)q0), S);
        v.y = to_field(__fmul_rn(ds, (float)q1), S);
        if (half == 0) r.lo = v; else r.hi = v;
    }
    return r;
}

template <int QT>
__device__ __forceinline__ constexpr int block_bytes() { return QT == 4 ? 144 : (QT == 5 ? 176 : 210); }

// one wavefront per super-block, output in the order of the input
template <int QT>
__global__ __launch_bounds__(BLOCK) void k_kq(const unsigned char *__restrict__ raw, u64 *__restrict__ out, i64 n_blocks, double S) {
    const int lane = threadIdx.x & 63;
    const i64 wave = ((i64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const i64 n_waves = ((i64)gridDim.x * BLOCK) >> 6;
    for (i64 b = wave; b < n_blocks; b += n_waves) {
        const Quad r = decode_block<QT>(raw + b * block_bytes<QT>(), lane, S);
        ulonglong2 *o = (ulonglong2 *)(out + b * 256);
        stream_store(&o[lane], r.lo);
        stream_store(&o[64 + lane], r.hi);
    }
}

// Decode and transpose: raw holds a (d_out, d_in) matrix, row r = d_in/256 consecutive super-blocks; out is
// the (d_in, d_out) matrix out[c * d_out + r], the (k_in, n_out) order the reference's loader produces
// with a separate `.T.contiguous()` pass over the decoded matrix (prover/loader.py:427-436).
// A workgroup owns T_ROWS rows of one super-block column: each wavefront decodes T_ROWS/4 super-blocks into
// an LDS tile [row][column] (16-byte writes, row pitch 258 words), then every thread collects two
// consecutive rows of one column and stores them, so that a wavefront store covers eight runs of
// T_ROWS * 8 = 128 consecutive bytes.
constexpr int T_ROWS = 16;       // 8-row tiles were twice as slow, 32-row tiles no faster (4096 x 11008 Q4_K)
constexpr int T_PITCH = 258;

template <int QT>
__global__ __launch_bounds__(BLOCK) void k_kq_t(const unsigned char *__restrict__ raw, u64 *__restrict__ out,
                                                i64 d_out, i64 blocks_per_row, i64 row_tiles, double S) {
    __shared__ __attribute__((aligned(16))) u64 tile[T_ROWS * T_PITCH];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const i64 bcol = blockIdx.x / row_tiles, r0 = (blockIdx.x % row_tiles) * T_ROWS;
#pragma unroll
    for (int i = 0; i < T_ROWS / 4; ++i) {
        const int lr = w * (T_ROWS / 4) + i;
        if (r0 + lr < d_out) {
            const Quad q = decode_block<QT>(raw + ((r0 + lr) * blocks_per_row + bcol) * block_bytes<QT>(), lane, S);
            *(ulonglong2 *)&tile[lr * T_PITCH + 2 * lane] = q.lo;
            *(ulonglong2 *)&tile[lr * T_PITCH + 128 + 2 * lane] = q.hi;
        }
    }
    __syncthreads();
    constexpr int RP = T_ROWS / 2;                        // row pairs of the tile
    const int rp = threadIdx.x & (RP - 1);                // rows 2rp, 2rp+1 of the tile
    u64 *dst = out + (bcol * 256) * d_out + r0 + 2 * rp;
#pragma unroll
    for (int i = 0; i < 256 / (BLOCK / RP); ++i) {
        const int c = (threadIdx.x / RP) + i * (BLOCK / RP);
        const u64 v0 = tile[(2 * rp) * T_PITCH + c], v1 = tile[(2 * rp + 1) * T_PITCH + c];
        u64 *o = dst + (i64)c * d_out;
        // streaming stores (ordinary ones were a third slower).  With an even row count a pair of rows is
        // there or not as a whole and sits at a 16-byte boundary: one 16-byte store, so that the eight lanes of a
        // run write whole 32-byte sectors (two 8-byte stores per lane wrote 1.66 x the bytes)
        if ((d_out & 1) == 0 && ((uintptr_t)out & 15) == 0) {
            if (r0 + 2 * rp < d_out) {
                ulonglong2 v;
                v.x = v0;
                v.y = v1;
                stream_store((ulonglong2 *)o, v);
            }
        } else {
            if (r0 + 2 * rp < d_out) __builtin_nontemporal_store(v0, o);
            if (r0 + 2 * rp + 1 < d_out) __builtin_nontemporal_store(v1, o + 1);
        }
    }
}

// d_out > 0: transposed store as in k_kq_t (d_in = n / d_out)
template <int QT>
__global__ __launch_bounds__(BLOCK) void k_generic(const unsigned char *__restrict__ raw, u64 *__restrict__ out, i64 n, double S,
                                                   i64 d_out) {
    i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 idx = (i64)blockIdx.x * BLOCK + threadIdx.x; idx < n; idx += stride) {
        i64 b = idx >> 8;
        int e = (int)(idx & 255);
        float v;
        if (QT == 6) {
            const unsigned char *p = raw + b * 210;
            float d = half_bits_to_float((u32)p[208] | ((u32)p[209] << 8));
            int lo = (p[(e >> 7) * 64 + (e & 63)] >> (4 * ((e >> 6) & 1))) & 0xF;
            int hi = (p[128 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3;
            int q = (int)(signed char)(lo | (hi << 4)) - 32;
            int sc = (int)(signed char)p[192 + (e >> 4)];
            v = __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
        } else {
            const unsigned char *p = raw + b * (QT == 4 ? 144 : 176);
            float d = half_bits_to_float((u32)p[0] | ((u32)p[1] << 8));
            float dmin = half_bits_to_float((u32)p[2] | ((u32)p[3] << 8));
            int s = e >> 5;
            u32 sc, mn;
            if (s < 4) {
                sc = p[4 + s] & 0x3F;
                mn = p[8 + s] & 0x3F;
            } else {
                int j = s - 4;
                sc = (p[12 + j] & 0x0F) | ((p[4 + j] >> 2) & 0x30);
                mn = (p[12 + j] >> 4) | ((p[8 + j] >> 2) & 0x30);
            }
            const unsigned char *qs = p + (QT == 4 ? 16 : 48);
            u32 q = (qs[(e >> 6) * 32 + (e & 31)] >> (4 * ((e >> 5) & 1))) & 0xF;
            if (QT == 5) q |= (u32)((p[16 + (e & 31)] >> (e >> 5)) & 1) << 4;
            v = dequant(d, dmin, sc, mn, q);
        }
        if (d_out > 0) {
            const i64 d_in = n / d_out;
            out[(idx % d_in) * d_out + idx / d_in] = to_field(v, S);
        } else {
            out[idx] = to_field(v, S);
        }
    }
}

inline unsigned grid_cap(i64 blocks_needed, i64 cap) {
    return (unsigned)(blocks_needed < 1 ? 1 : (blocks_needed > cap ? cap : blocks_needed));
}

}  // namespace

extern "C" int vi_kquant_to_field(int qtype, const uint8_t *raw, int64_t n_blocks, double S, uint64_t *out, void *stream) {
    if (qtype != 4 && qtype != 5 && qtype != 6) return vi::fail(VI_EINVAL, "vi_kquant_to_field: unsupported qtype %d", qtype);
    if (n_blocks < 0) return vi::fail(VI_EINVAL, "vi_kquant_to_field: n_blocks = %lld", (long long)n_blocks);
    if (n_blocks == 0) return VI_OK;
    if (!raw || !out) return vi::fail(VI_EINVAL, "vi_kquant_to_field: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const i64 n = n_blocks * 256;
    const bool out16 = ((uintptr_t)out & 15) == 0;
    // one wavefront per super-block and a workgroup per four of them: 0.062 ms on 4096 x 11008 Q4_K against 0.067 ms
    // for a grid capped at 32 workgroups per CU that strides over the blocks (the loop in the kernel covers the
    // sizes beyond the grid limit)
    const unsigned gw = grid_cap((n_blocks + 3) / 4, 0x7FFFFFFF);
    if (qtype == 4 && ((uintptr_t)raw & 3) == 0 && out16) {
        hipLaunchKernelGGL(k_kq<4>, dim3(gw), dim3(BLOCK), 0, s, raw, out, (i64)n_blocks, S);
    } else if (qtype == 5 && ((uintptr_t)raw & 3) == 0 && out16) {
        hipLaunchKernelGGL(k_kq<5>, dim3(gw), dim3(BLOCK), 0, s, raw, out, (i64)n_blocks, S);
    } else if (qtype == 6 && ((uintptr_t)raw & 1) == 0 && out16) {
        hipLaunchKernelGGL(k_kq<6>, dim3(gw), dim3(BLOCK), 0, s, raw, out, (i64)n_blocks, S);
    } else {
        unsigned g = grid_cap((n + BLOCK - 1) / BLOCK, 256 * 32);
        if (qtype == 4) hipLaunchKernelGGL(k_generic<4>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)0);
        if (qtype == 5) hipLaunchKernelGGL(k_generic<5>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)0);
        if (qtype == 6) hipLaunchKernelGGL(k_generic<6>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)0);
    }
    VI_LAUNCH_CHECK("kquant");
    return VI_OK;
}

extern "C" int vi_kquant_to_field_transposed(int qtype, const uint8_t *raw, int64_t d_out, int64_t d_in, double S,
                                             uint64_t *out, void *stream) {
    if (qtype != 4 && qtype != 5 && qtype != 6) return vi::fail(VI_EINVAL, "vi_kquant_to_field_transposed: unsupported qtype %d", qtype);
    if (d_out < 0 || d_in < 0 || (d_in & 255)) return vi::fail(VI_EINVAL, "vi_kquant_to_field_transposed: d_out = %lld, d_in = %lld (a multiple of 256)", (long long)d_out, (long long)d_in);
    if (d_out == 0 || d_in == 0) return VI_OK;
    if (!raw || !out) return vi::fail(VI_EINVAL, "vi_kquant_to_field_transposed: null pointer");
    const i64 bpr = d_in >> 8, row_tiles = (d_out + T_ROWS - 1) / T_ROWS;
    if (d_out > ((i64)1 << 40) / d_in) return vi::fail(VI_EINVAL, "vi_kquant_to_field_transposed: %lld x %lld is too large", (long long)d_out, (long long)d_in);
    hipStream_t s = (hipStream_t)stream;
    const i64 tiles = bpr * row_tiles;
    const bool aligned = ((uintptr_t)raw & (qtype == 6 ? 1 : 3)) == 0 && tiles <= 0x7FFFFFFF;
    if (aligned) {
        if (qtype == 4) hipLaunchKernelGGL(k_kq_t<4>, dim3((unsigned)tiles), dim3(BLOCK), 0, s, raw, out, (i64)d_out, bpr, row_tiles, S);
        if (qtype == 5) hipLaunchKernelGGL(k_kq_t<5>, dim3((unsigned)tiles), dim3(BLOCK), 0, s, raw, out, (i64)d_out, bpr, row_tiles, S);
        if (qtype == 6) hipLaunchKernelGGL(k_kq_t<6>, dim3((unsigned)tiles), dim3(BLOCK), 0, s, raw, out, (i64)d_out, bpr, row_tiles, S);
    } else {
        const i64 n = d_out * d_in;
        unsigned g = grid_cap((n + BLOCK - 1) / BLOCK, 256 * 32);
        if (qtype == 4) hipLaunchKernelGGL(k_generic<4>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)d_out);
        if (qtype == 5) hipLaunchKernelGGL(k_generic<5>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)d_out);
        if (qtype == 6) hipLaunchKernelGGL(k_generic<6>, dim3(g), dim3(BLOCK), 0, s, raw, out, n, S, (i64)d_out);
    }
    VI_LAUNCH_CHECK("kquant transposed");
    return VI_OK;
}

// BLAKE3 column hashing and Merkle levels for committed codeword matrices.
//
// digest_j = BLAKE3(column j of a row-major (m, n) uint64 matrix as little-endian bytes)
// (prover/cuda_primitives.py:796-808, prover/protocol.py:100-105); a Merkle parent is
// BLAKE3(left || right), an odd last node is paired with itself (layergkr/rs.py:135-146).
//
// The reference walks a whole column with one thread and keeps BLAKE3's merge stack
// per column (prover/kernels/blake3_columns.cuh:47-170).  Here the work is split the
// other way: k_chunk_cvs gives every (1 KiB chunk, column) pair its own thread -- lanes
// run along the columns, so the eight 8-byte loads of a 64-byte block are each one
// coalesced 512-byte wavefront access -- and stores the chunk's chaining value;
// k_merge_levels then quarters the number of chaining values per launch.  Pairing adjacent
// nodes and carrying an odd last node up unchanged reproduces BLAKE3's left-full tree,
// and the last merge carries the ROOT flag.  The chunk stage is therefore a streaming
// pass over the matrix with as many independent threads as the GPU wants, and it can be
// fed in row slabs (vi_hash_columns_update) while the codewords are produced.
#include "common.hpp"
#include "gl_field.hpp"

namespace {

typedef uint32_t u32;
typedef uint64_t u64;
typedef int64_t i64;

constexpr int BLOCK = 256;
constexpr u32 CHUNK_START = 1, CHUNK_END = 2, PARENT = 4, ROOT = 8;
constexpr int ROWS_PER_CHUNK = 128;          // 1024 bytes of 8-byte words
constexpr int ROWS_PER_BLOCK = 8;            // 64 bytes

__device__ __constant__ const u32 IV[8] = {0x6A09E667u, 0xBB67AE85u, 0x3C6EF372u, 0xA54FF53Au,
                                           0x510E527Fu, 0x9B05688Cu, 0x1F83D9ABu, 0x5BE0CD19u};

// message word index used at position i of round r (the round permutation applied r times)
__host__ __device__ constexpr int sched(int r, int i) {
    constexpr int perm[16] = {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8};
    int idx = i;
    for (int k = 0; k < r; ++k) idx = perm[idx];
    return idx;
}

__device__ __forceinline__ u32 rotr(u32 x, int n) { return __builtin_amdgcn_alignbit(x, x, n); }

#define B3_G(a, b, c, d, mx, my)            \
    a = a + b + (mx); d = rotr(d ^ a, 16);  \
    c = c + d;        b = rotr(b ^ c, 12);  \
    a = a + b + (my); d = rotr(d ^ a, 8);   \
    c = c + d;        b = rotr(b ^ c, 7);

template <int R>
__device__ __forceinline__ void b3_round(u32 (&s)[16], const u32 (&m)[16]) {
    B3_G(s[0], s[4], s[8], s[12], m[sched(R, 0)], m[sched(R, 1)])
    B3_G(s[1], s[5], s[9], s[13], m[sched(R, 2)], m[sched(R, 3)])
    B3_G(s[2], s[6], s[10], s[14], m[sched(R, 4)], m[sched(R, 5)])
    B3_G(s[3], s[7], s[11], s[15], m[sched(R, 6)], m[sched(R, 7)])
    B3_G(s[0], s[5], s[10], s[15], m[sched(R, 8)], m[sched(R, 9)])
    B3_G(s[1], s[6], s[11], s[12], m[sched(R, 10)], m[sched(R, 11)])
    B3_G(s[2], s[7], s[8], s[13], m[sched(R, 12)], m[sched(R, 13)])
    B3_G(s[3], s[4], s[9], s[14], m[sched(R, 14)], m[sched(R, 15)])
}

// cv <- first eight words of compress(cv, m, counter, block_len, flags)
__device__ __forceinline__ void compress(u32 (&cv)[8], const u32 (&m)[16], u64 counter, u32 block_len, u32 flags) {
    u32 s[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = cv[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) s[8 + i] = IV[i];
    s[12] = (u32)counter;
    s[13] = (u32)(counter >> 32);
    s[14] = block_len;
    s[15] = flags;
    b3_round<0>(s, m); b3_round<1>(s, m); b3_round<2>(s, m); b3_round<3>(s, m);
    b3_round<4>(s, m); b3_round<5>(s, m); b3_round<6>(s, m);
#pragma unroll
    for (int i = 0; i < 8; ++i) cv[i] = s[i] ^ s[i + 8];
}

// Chaining value of chunk (chunk0 + blockIdx.y) of every column.
//   rows          first row of the slab (row pitch `stride` words), slab_rows rows in it
//   single_root   the whole message is this one chunk: its last block carries ROOT
// cvs[(chunk0 + c) * n + col] receives 8 words.
__global__ __launch_bounds__(BLOCK) void k_chunk_cvs(const u64 *__restrict__ rows, i64 slab_rows, i64 n, i64 stride, i64 chunk0,
                                                     int single_root, u32 *__restrict__ cvs) {
    const i64 col = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (col >= n) return;
    const i64 c = blockIdx.y;
    const i64 r0 = c * ROWS_PER_CHUNK;
    const i64 nrows = (slab_rows - r0 < ROWS_PER_CHUNK) ? (slab_rows - r0) : ROWS_PER_CHUNK;   // >= 0
    const int n_blocks = nrows == 0 ? 1 : (int)((nrows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    const u64 *p = rows + r0 * stride + col;
    u32 cv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) cv[i] = IV[i];
    for (int b = 0; b < n_blocks; ++b) {
        u32 m[16];
        const i64 left = nrows - (i64)b * ROWS_PER_BLOCK;
        const int here = left >= ROWS_PER_BLOCK ? ROWS_PER_BLOCK : (int)left;
#pragma unroll
        for (int i = 0; i < ROWS_PER_BLOCK; ++i) {
            u64 v = i < here ? p[((i64)b * ROWS_PER_BLOCK + i) * stride] : 0;
            m[2 * i] = (u32)v;
            m[2 * i + 1] = (u32)(v >> 32);
        }
        u32 flags = 0;
        if (b == 0) flags |= CHUNK_START;
        if (b == n_blocks - 1) flags |= CHUNK_END | (single_root ? ROOT : 0u);
        compress(cv, m, (u64)(chunk0 + c), (u32)(here * 8), flags);
    }
    u32 *o = cvs + ((chunk0 + c) * n + col) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = cv[i];
}

// BLAKE3's internal tree over `count` nodes per column, LV levels per launch: node pairs (2i, 2i+1) become a parent,
// an odd last node moves up unchanged.  in/out: [node][col][8 words].  The thread of (column, i) forms node i of
// level LV above the input level from the up to 2^LV input nodes under it (2^LV - 1 compressions, the lower ones
// first), so the levels in between are never written.  cnt[j] = nodes of level j (cnt[0] = count of the input
// level); the merge of the last two nodes of a level is the root.
template <int LV>
__device__ __forceinline__ void merge_node(const u32 *__restrict__ in, i64 n, i64 col, i64 idx, const i64 (&cnt)[4], u32 (&o)[8]) {
    if constexpr (LV == 0) {
        const u32 *p = in + (idx * n + col) * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k) o[k] = p[k];
    } else {
        if (2 * idx + 1 >= cnt[LV - 1]) {
            merge_node<LV - 1>(in, n, col, 2 * idx, cnt, o);
            return;
        }
        u32 l[8], r[8], m[16];
        merge_node<LV - 1>(in, n, col, 2 * idx, cnt, l);
        merge_node<LV - 1>(in, n, col, 2 * idx + 1, cnt, r);
#pragma unroll
        for (int k = 0; k < 8; ++k) { m[k] = l[k]; m[8 + k] = r[k]; o[k] = IV[k]; }
        compress(o, m, 0, 64, PARENT | (cnt[LV - 1] == 2 ? ROOT : 0u));
    }
}

template <int LV>
__global__ __launch_bounds__(BLOCK) void k_merge_levels(const u32 *__restrict__ in, i64 count, i64 n, i64 idx0, u32 *__restrict__ out) {
    const i64 col = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (col >= n) return;
    i64 cnt[4];
    cnt[0] = count;
#pragma unroll
    for (int j = 1; j < 4; ++j) cnt[j] = (cnt[j - 1] + 1) / 2;
    const i64 i = idx0 + blockIdx.y;
    u32 o[8];
    merge_node<LV>(in, n, col, i, cnt, o);
    u32 *dst = out + (i * n + col) * 8;
#pragma unroll
    for (int k = 0; k < 8; ++k) dst[k] = o[k];
}

// Merkle level over 32-byte nodes: parent i = BLAKE3(node[2i] || node[2i+1]), the odd last
// node is paired with itself.  A 64-byte message is one block: CHUNK_START|CHUNK_END|ROOT.
__global__ __launch_bounds__(BLOCK) void k_merkle_level(const u32 *__restrict__ nodes, i64 count, u32 *__restrict__ out) {
    const i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x;
    const i64 parents = (count + 1) / 2;
    if (i >= parents) return;
    const u32 *l = nodes + (2 * i) * 8;
    const u32 *r = nodes + ((2 * i + 1 < count) ? (2 * i + 1) : (2 * i)) * 8;
    u32 m[16], cv[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) { m[k] = l[k]; m[8 + k] = r[k]; cv[k] = IV[k]; }
    compress(cv, m, 0, 64, CHUNK_START | CHUNK_END | ROOT);
#pragma unroll
    for (int k = 0; k < 8; ++k) out[i * 8 + k] = cv[k];
}

// Up to SUB_LEVELS Merkle levels in one launch.  A workgroup owns 2^SUB_LEVELS consecutive nodes of the input
// level, builds the parents of every level above them that lies inside its block (children of a block-aligned
// node are in the block too), keeps the newest level in LDS for the next one and writes every level to `out`:
// level j (1-based) of this launch starts at out + 8 * (c_1 + ... + c_{j-1}) words, c_j = ceil(c_{j-1} / 2),
// c_0 = count.  The odd last node of a level is paired with itself, as in k_merkle_level.
constexpr int SUB_LEVELS = 9;

__global__ __launch_bounds__(BLOCK) void k_merkle_subtree(const u32 *__restrict__ nodes, i64 count, int levels, u32 *__restrict__ out) {
    __shared__ u32 buf[2][BLOCK * 8];
    const i64 base = (i64)blockIdx.x << SUB_LEVELS;            // first input node of the block
    i64 c_prev = count, off = 0;                               // nodes of the level below, word offset of this level in out
    for (int j = 1; j <= levels; ++j) {
        const i64 c = (c_prev + 1) >> 1;
        const i64 first = base >> j;                           // first node of level j in the block
        const int in_block = 1 << (SUB_LEVELS - j);
        const i64 i = first + threadIdx.x;
        if ((int)threadIdx.x < in_block && i < c) {
            u32 m[16], cv[8];
            const bool has_right = 2 * i + 1 < c_prev;
            if (j == 1) {
                const u32 *l = nodes + (2 * i) * 8;
                const u32 *r = nodes + (has_right ? 2 * i + 1 : 2 * i) * 8;
#pragma unroll
                for (int k = 0; k < 8; ++k) { m[k] = l[k]; m[8 + k] = r[k]; }
            } else {
                const u32 *l = buf[j & 1] + (2 * threadIdx.x) * 8;
                const u32 *r = buf[j & 1] + (has_right ? 2 * threadIdx.x + 1 : 2 * threadIdx.x) * 8;
#pragma unroll
                for (int k = 0; k < 8; ++k) { m[k] = l[k]; m[8 + k] = r[k]; }
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) cv[k] = IV[k];
            compress(cv, m, 0, 64, CHUNK_START | CHUNK_END | ROOT);
            u32 *o = out + off + i * 8;
            u32 *keep = buf[(j + 1) & 1] + threadIdx.x * 8;
#pragma unroll
            for (int k = 0; k < 8; ++k) { o[k] = cv[k]; keep[k] = cv[k]; }
        }
        __syncthreads();
        off += c * 8;
        c_prev = c;
    }
}

// Zero-knowledge pad generator (prover/cuda_primitives.py:870-930, k_row_prg / k_row_prg_indexed):
//   out[r][k] = (first 8 bytes of BLAKE3(seed[32] || row_le8 || k_le8), little-endian) mod p.
// The 48-byte message is a single block, so a value costs one compression, of which only the
// first two output words are used.  One thread per value, consecutive threads along k, so
// that stores are coalesced; the reference gives a whole row to one thread.
// row = row_indices[r] when row_indices is given, else the 32-bit sum row_offset + r (the
// reference's contiguous variant computes the row number in uint32).
__global__ __launch_bounds__(BLOCK) void k_row_prg(const u32 *__restrict__ seed, const u64 *__restrict__ row_indices, u32 row_offset,
                                                   i64 n_rows, i64 slack, u64 *__restrict__ out, i64 out_stride) {
    const i64 g = (i64)blockIdx.x * BLOCK + threadIdx.x;
    if (g >= n_rows * slack) return;
    const i64 r = g / slack, k = g - r * slack;
    const u64 row = row_indices ? row_indices[r] : (u64)(u32)(row_offset + (u32)r);
    u32 m[16], cv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { m[i] = seed[i]; cv[i] = IV[i]; }
    m[8] = (u32)row; m[9] = (u32)(row >> 32);
    m[10] = (u32)k;  m[11] = (u32)((u64)k >> 32);
    m[12] = m[13] = m[14] = m[15] = 0;
    compress(cv, m, 0, 48, CHUNK_START | CHUNK_END | ROOT);
    const u64 raw = ((u64)cv[1] << 32) | cv[0];
    out[r * out_stride + k] = raw >= 0xFFFFFFFF00000001ull ? raw - 0xFFFFFFFF00000001ull : raw;
}

// The test-combiner challenge of the protocol (prover/protocol.py:127-135, device twin
// prover/kernels/gl_spmv.cuh:46-70):
//   challenge(seed, cid, label) = le128(BLAKE3(seed[32] || label || cid_le8)[0:16]) mod p.
// label has at most 8 bytes, so the message is one block; `tail` holds label || cid packed into
// the 16 bytes that follow the seed.
struct ChallengeKey {
    u32 seed[8];
    int label_len;
    u64 label;                 // label bytes as a little-endian integer
};

__device__ __forceinline__ ChallengeKey load_key(const u32 *__restrict__ seed, const unsigned char *__restrict__ label, int label_len) {
    ChallengeKey k;
#pragma unroll
    for (int i = 0; i < 8; ++i) k.seed[i] = seed[i];
    k.label_len = label_len;
    k.label = 0;
    for (int i = 0; i < label_len; ++i) k.label |= (u64)label[i] << (8 * i);
    return k;
}

__device__ __forceinline__ u64 challenge(const ChallengeKey &k, u64 cid) {
    u32 m[16], cv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { m[i] = k.seed[i]; cv[i] = IV[i]; }
    const int sh = 8 * k.label_len;                      // 0 .. 64 bits of label before the cid
    const u64 lo = sh == 64 ? k.label : (k.label | (cid << sh));
    const u64 hi = sh == 0 ? 0 : (sh == 64 ? cid : (cid >> (64 - sh)));
    m[8] = (u32)lo;  m[9] = (u32)(lo >> 32);
    m[10] = (u32)hi; m[11] = (u32)(hi >> 32);
    m[12] = m[13] = m[14] = m[15] = 0;
    compress(cv, m, 0, (u32)(40 + k.label_len), CHUNK_START | CHUNK_END | ROOT);
    return gl::reduce128(((u64)cv[1] << 32) | cv[0], ((u64)cv[3] << 32) | cv[2]);
}

// out[i] = challenge(seed, cids ? cids[i] : i, label)      (challenge_vec / challenge_at)
__global__ __launch_bounds__(BLOCK) void k_challenge(const u32 *__restrict__ seed, const unsigned char *__restrict__ label, int label_len,
                                                     const u64 *__restrict__ cids, i64 n, u64 *__restrict__ out) {
    const ChallengeKey key = load_key(seed, label, label_len);
    const i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += stride) out[i] = challenge(key, cids ? cids[i] : (u64)i);
}

// CSR matrix times vector over the field (prover/kernels/gl_spmv.cuh:25-41, 72-92):
//   y[i] = sum_{p in row i} values[p] * x[col_idx[p]],   x[c] = challenge(seed, c, label) when x is null.
// WAVE = false: one thread per row (rows of a few entries).  WAVE = true: one wavefront per row, lanes
// stride over the row so that values and column indices are read coalesced, then a shuffle reduction.
template <bool WAVE>
__global__ __launch_bounds__(BLOCK) void k_spmv(const u64 *__restrict__ values, const u64 *__restrict__ col_idx,
                                                const u64 *__restrict__ row_ptr, const u64 *__restrict__ x, const u32 *__restrict__ seed,
                                                const unsigned char *__restrict__ label, int label_len, i64 n_rows,
                                                u64 *__restrict__ y) {
    ChallengeKey key;
    if (!x) key = load_key(seed, label, label_len);
    const i64 gid = (i64)blockIdx.x * BLOCK + threadIdx.x;
    const i64 n_workers = ((i64)gridDim.x * BLOCK) >> (WAVE ? 6 : 0);
    const int lane = WAVE ? (threadIdx.x & 63) : 0;
    for (i64 row = WAVE ? (gid >> 6) : gid; row < n_rows; row += n_workers) {
        const u64 start = row_ptr[row], end = row_ptr[row + 1];
        u64 acc = 0;
        for (u64 p = start + lane; p < end; p += WAVE ? 64 : 1) {
            const u64 c = col_idx[p];
            acc = gl::add(acc, gl::mul(values[p], x ? x[c] : challenge(key, c)));
        }
        if (WAVE) {
            for (int off = 32; off > 0; off >>= 1) acc = gl::add(acc, __shfl_xor(acc, off, 64));
            if (lane == 0) y[row] = acc;
        } else {
            y[row] = acc;
        }
    }
}

// LogUp multiplicities (prover/kernels/gl_extras.cuh:118-150): mult[j] += 1 for the first j with
// table[j] == x[i]; values that are not in the table count nowhere.  t_len_range > 0 says the
// table is literally 0 .. t_len_range-1, so x[i] is its own index.
__global__ __launch_bounds__(BLOCK) void k_lookup_mult(const u64 *__restrict__ x, i64 n_x, const u64 *__restrict__ table, i64 n_table,
                                                       i64 t_len_range, unsigned long long *__restrict__ mult) {
    const i64 stride = (i64)gridDim.x * BLOCK;
    for (i64 i = (i64)blockIdx.x * BLOCK + threadIdx.x; i < n_x; i += stride) {
        const u64 xi = x[i];
        if (t_len_range > 0) {
            if (xi < (u64)t_len_range) atomicAdd(&mult[xi], 1ULL);
            continue;
        }
        for (i64 j = 0; j < n_table; ++j) {
            if (table[j] == xi) {
                atomicAdd(&mult[j], 1ULL);
                break;
            }
        }
    }
}

inline i64 chunks_of(i64 m) { return m <= 0 ? 1 : (m + ROWS_PER_CHUNK - 1) / ROWS_PER_CHUNK; }

}  // namespace

extern "C" {

size_t vi_hash_columns_workspace_bytes(int64_t m, int64_t n) {
    if (m < 0 || n <= 0) return 0;
    // chunk chaining values + one ping-pong level
    i64 c = chunks_of(m);
    return (size_t)(c + (c + 1) / 2) * (size_t)n * 32;
}

int vi_hash_columns_update(const uint64_t *rows, int64_t slab_rows, int64_t n, int64_t row_stride, int64_t chunk0,
                           int64_t n_chunks_total, void *ws, size_t ws_bytes, void *stream) {
    if (n <= 0 || slab_rows < 0 || row_stride < n || chunk0 < 0 || n_chunks_total < 1)
        return vi::fail(VI_EINVAL, "vi_hash_columns_update: bad shape rows=%lld n=%lld stride=%lld", (long long)slab_rows, (long long)n, (long long)row_stride);
    const i64 slab_chunks = chunks_of(slab_rows);
    if (chunk0 + slab_chunks > n_chunks_total) return vi::fail(VI_EINVAL, "vi_hash_columns_update: slab exceeds the declared %lld chunks", (long long)n_chunks_total);
    if (chunk0 + slab_chunks < n_chunks_total && slab_rows % ROWS_PER_CHUNK)
        return vi::fail(VI_EINVAL, "vi_hash_columns_update: only the last slab may hold a partial 128-row chunk");
    if (slab_rows == 0 && n_chunks_total > 1) return vi::fail(VI_EINVAL, "vi_hash_columns_update: empty slab of a multi-chunk message");
    if (slab_rows > 0 && !rows) return vi::fail(VI_EINVAL, "vi_hash_columns_update: null rows");
    if (!ws || ws_bytes < (size_t)(n_chunks_total + (n_chunks_total + 1) / 2) * (size_t)n * 32)
        return vi::fail(VI_ENOMEM, "vi_hash_columns_update: workspace too small");
    if (slab_chunks > 65535) return vi::fail(VI_EINVAL, "vi_hash_columns_update: at most 65535 chunks (8,388,480 rows) per call");
    dim3 grid((unsigned)((n + BLOCK - 1) / BLOCK), (unsigned)slab_chunks);
    hipLaunchKernelGGL(k_chunk_cvs, grid, dim3(BLOCK), 0, (hipStream_t)stream, rows, (i64)slab_rows, (i64)n, (i64)row_stride,
                       (i64)chunk0, n_chunks_total == 1 ? 1 : 0, (u32 *)ws);
    VI_LAUNCH_CHECK("k_chunk_cvs");
    return VI_OK;
}

int vi_hash_columns_finalize(int64_t n, int64_t n_chunks_total, void *ws, size_t ws_bytes, uint8_t *digests, void *stream) {
    if (n <= 0 || n_chunks_total < 1 || !digests) return vi::fail(VI_EINVAL, "vi_hash_columns_finalize: bad arguments");
    if (!ws || ws_bytes < (size_t)(n_chunks_total + (n_chunks_total + 1) / 2) * (size_t)n * 32)
        return vi::fail(VI_ENOMEM, "vi_hash_columns_finalize: workspace too small");
    hipStream_t s = (hipStream_t)stream;
    u32 *a = (u32 *)ws;                               // n_chunks_total nodes
    u32 *b = a + (size_t)n_chunks_total * n * 8;      // ceil(n_chunks_total / 2) nodes
    i64 count = n_chunks_total;
    if (count == 1) {
        VI_HIP(hipMemcpyAsync(digests, a, (size_t)n * 32, hipMemcpyDeviceToDevice, s));
        return VI_OK;
    }
    // MERGE_LEVELS levels of the tree per launch; the launch that reaches the root writes the digests themselves
    // (through a copy when the caller's buffer is not word-aligned)
    constexpr int MERGE_LEVELS = 2;
    const bool direct = ((uintptr_t)digests & 3) == 0;
    while (count > 1) {
        int lv = 0;
        i64 top = count;
        while (top > 1 && lv < MERGE_LEVELS) { top = (top + 1) / 2; ++lv; }
        u32 *dst = (top == 1 && direct) ? (u32 *)digests : b;
        for (i64 lo = 0; lo < top; lo += 65535) {                 // grid.y limit
            const i64 cnt = top - lo < 65535 ? top - lo : 65535;
            dim3 grid((unsigned)((n + BLOCK - 1) / BLOCK), (unsigned)cnt);
            if (lv == 1) hipLaunchKernelGGL(k_merge_levels<1>, grid, dim3(BLOCK), 0, s, (const u32 *)a, count, (i64)n, lo, dst);
            else hipLaunchKernelGGL(k_merge_levels<2>, grid, dim3(BLOCK), 0, s, (const u32 *)a, count, (i64)n, lo, dst);
            VI_LAUNCH_CHECK("k_merge_levels");
        }
        u32 *t = a; a = b; b = t;
        count = top;
    }
    if (!direct) VI_HIP(hipMemcpyAsync(digests, a, (size_t)n * 32, hipMemcpyDeviceToDevice, s));
    return VI_OK;
}

int vi_hash_columns(const uint64_t *mat, int64_t m, int64_t n, int64_t row_stride, uint8_t *digests, void *ws,
                    size_t ws_bytes, void *stream) {
    if (m < 0) return vi::fail(VI_EINVAL, "vi_hash_columns: m = %lld", (long long)m);
    const i64 total = chunks_of(m);
    for (i64 c0 = 0; c0 < total; c0 += 65535) {
        const i64 cc = total - c0 < 65535 ? total - c0 : 65535;
        const i64 r0 = c0 * ROWS_PER_CHUNK;
        const i64 rows = (c0 + cc == total) ? m - r0 : cc * ROWS_PER_CHUNK;
        int rc = vi_hash_columns_update(mat ? mat + r0 * row_stride : nullptr, rows, n, row_stride, c0, total, ws, ws_bytes, stream);
        if (rc) return rc;
    }
    return vi_hash_columns_finalize(n, total, ws, ws_bytes, digests, stream);
}

int vi_merkle_level(const uint8_t *nodes, int64_t count, uint8_t *out, void *stream) {
    if (count < 1 || !nodes || !out) return vi::fail(VI_EINVAL, "vi_merkle_level: bad arguments");
    if (((uintptr_t)nodes | (uintptr_t)out) & 3) return vi::fail(VI_EINVAL, "vi_merkle_level: nodes must be 4-byte aligned");
    const i64 parents = (count + 1) / 2;
    hipLaunchKernelGGL(k_merkle_level, dim3((unsigned)((parents + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, (hipStream_t)stream,
                       (const u32 *)nodes, (i64)count, (u32 *)out);
    VI_LAUNCH_CHECK("k_merkle_level");
    return VI_OK;
}

int64_t vi_merkle_tree_nodes(int64_t count) {
    int64_t total = 0;
    for (int64_t c = count; c > 1;) { c = (c + 1) / 2; total += c; }
    return count < 1 ? 0 : total;
}

int vi_merkle_tree(const uint8_t *leaves, int64_t count, uint8_t *levels_out, void *stream) {
    if (count < 1 || !leaves) return vi::fail(VI_EINVAL, "vi_merkle_tree: bad arguments");
    if (count == 1) return VI_OK;
    if (!levels_out) return vi::fail(VI_EINVAL, "vi_merkle_tree: null output");
    if (((uintptr_t)leaves | (uintptr_t)levels_out) & 3) return vi::fail(VI_EINVAL, "vi_merkle_tree: nodes must be 4-byte aligned");
    const u32 *cur = (const u32 *)leaves;
    u32 *out = (u32 *)levels_out;
    i64 c = count;
    while (c > 1) {
        int levels = 0;
        i64 written = 0, cl = c;
        while (cl > 1 && levels < SUB_LEVELS) { cl = (cl + 1) / 2; written += cl; ++levels; }
        const i64 blocks = (c + ((i64)1 << SUB_LEVELS) - 1) >> SUB_LEVELS;
        if (blocks > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "vi_merkle_tree: too many leaves");
        hipLaunchKernelGGL(k_merkle_subtree, dim3((unsigned)blocks), dim3(BLOCK), 0, (hipStream_t)stream, cur, c, levels, out);
        VI_LAUNCH_CHECK("k_merkle_subtree");
        cur = out + (written - cl) * 8;                       // the last level written is the next input
        out += written * 8;
        c = cl;
    }
    return VI_OK;
}

int vi_row_prg(const uint8_t *seed, const uint64_t *row_indices, int64_t row_offset, int64_t n_rows, int64_t slack,
               uint64_t *out, int64_t out_stride, void *stream) {
    if (n_rows < 0 || slack < 0 || out_stride < slack) return vi::fail(VI_EINVAL, "vi_row_prg: bad shape n_rows=%lld slack=%lld out_stride=%lld", (long long)n_rows, (long long)slack, (long long)out_stride);
    if (n_rows == 0 || slack == 0) return VI_OK;
    if (!seed || !out) return vi::fail(VI_EINVAL, "vi_row_prg: null pointer");
    if ((uintptr_t)seed & 3) return vi::fail(VI_EINVAL, "vi_row_prg: seed must be 4-byte aligned");
    const i64 total = n_rows * slack;
    const i64 blocks = (total + BLOCK - 1) / BLOCK;
    if (blocks > 0x7FFFFFFF) return vi::fail(VI_EINVAL, "vi_row_prg: %lld values exceed one launch", (long long)total);
    hipLaunchKernelGGL(k_row_prg, dim3((unsigned)blocks), dim3(BLOCK), 0, (hipStream_t)stream, (const u32 *)seed, row_indices,
                       (u32)row_offset, (i64)n_rows, (i64)slack, out, (i64)out_stride);
    VI_LAUNCH_CHECK("k_row_prg");
    return VI_OK;
}

namespace {
int check_key(const char *who, const uint8_t *seed, const uint8_t *label, int label_len) {
    if (!seed || ((uintptr_t)seed & 3)) return vi::fail(VI_EINVAL, "%s: seed must be a 4-byte aligned device pointer", who);
    if (label_len < 0 || label_len > 8 || (label_len > 0 && !label)) return vi::fail(VI_EINVAL, "%s: label of %d bytes (0 .. 8)", who, label_len);
    return VI_OK;
}
inline unsigned capped_grid(i64 work_items) {
    i64 b = (work_items + BLOCK - 1) / BLOCK;
    return (unsigned)(b < 1 ? 1 : (b > 256 * 32 ? 256 * 32 : b));
}
}  // namespace

int vi_challenge(const uint8_t *seed, const uint8_t *label, int label_len, const uint64_t *cids, int64_t n, uint64_t *out,
                 void *stream) {
    int rc = check_key("vi_challenge", seed, label, label_len);
    if (rc) return rc;
    if (n < 0) return vi::fail(VI_EINVAL, "vi_challenge: n = %lld", (long long)n);
    if (n == 0) return VI_OK;
    if (!out) return vi::fail(VI_EINVAL, "vi_challenge: null out");
    hipLaunchKernelGGL(k_challenge, dim3(capped_grid(n)), dim3(BLOCK), 0, (hipStream_t)stream, (const u32 *)seed, label, label_len,
                       cids, (i64)n, out);
    VI_LAUNCH_CHECK("k_challenge");
    return VI_OK;
}

int vi_gl_spmv(const uint64_t *values, const uint64_t *col_idx, const uint64_t *row_ptr, int64_t n_rows, int64_t nnz,
               const uint64_t *x, const uint8_t *seed, const uint8_t *label, int label_len, uint64_t *y, void *stream) {
    if (n_rows < 0 || nnz < 0) return vi::fail(VI_EINVAL, "vi_gl_spmv: n_rows = %lld, nnz = %lld", (long long)n_rows, (long long)nnz);
    if (!x) {
        int rc = check_key("vi_gl_spmv", seed, label, label_len);
        if (rc) return rc;
    }
    if (n_rows == 0) return VI_OK;
    if (!row_ptr || !y || (nnz > 0 && (!values || !col_idx))) return vi::fail(VI_EINVAL, "vi_gl_spmv: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (nnz / n_rows >= 32) {
        hipLaunchKernelGGL(k_spmv<true>, dim3(capped_grid(n_rows * 64)), dim3(BLOCK), 0, s, values, col_idx, row_ptr, x, (const u32 *)seed,
                           label, label_len, (i64)n_rows, y);
    } else {
        hipLaunchKernelGGL(k_spmv<false>, dim3(capped_grid(n_rows)), dim3(BLOCK), 0, s, values, col_idx, row_ptr, x, (const u32 *)seed,
                           label, label_len, (i64)n_rows, y);
    }
    VI_LAUNCH_CHECK("k_spmv");
    return VI_OK;
}

int vi_lookup_multiplicities(const uint64_t *x, int64_t n_x, const uint64_t *table, int64_t n_table, int table_is_range,
                             uint64_t *mult, void *stream) {
    if (n_x < 0 || n_table < 0) return vi::fail(VI_EINVAL, "vi_lookup_multiplicities: n_x = %lld, n_table = %lld", (long long)n_x, (long long)n_table);
    if (n_x == 0 || n_table == 0) return VI_OK;
    if (!x || !mult || (!table_is_range && !table)) return vi::fail(VI_EINVAL, "vi_lookup_multiplicities: null pointer");
    hipLaunchKernelGGL(k_lookup_mult, dim3(capped_grid(n_x)), dim3(BLOCK), 0, (hipStream_t)stream, x, (i64)n_x, table, (i64)n_table,
                       (i64)(table_is_range ? n_table : 0), (unsigned long long *)mult);
    VI_LAUNCH_CHECK("k_lookup_mult");
    return VI_OK;
}

}  // extern "C"

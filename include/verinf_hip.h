/*
 * libverinf_hip -- C ABI of the MI355X (gfx950) Goldilocks prover kernels.
 *
 * Every entry point takes plain device pointers, sizes and a hipStream_t (passed
 * as void*; NULL = the null stream), launches asynchronously on that stream and
 * returns 0, or a negative VI_E* code after recording a message readable through
 * vi_last_error().  Nothing throws across the boundary.  Unless stated otherwise
 * an entry point allocates no device memory: scratch is passed in as a workspace
 * whose size the matching *_workspace_bytes() query returns.  Twiddle tables are
 * the exception: they are built once per (length, direction, device) on first use
 * and cached for the life of the process, like the reference's NTT contexts.  That
 * first use of a length (and of a coset shift) allocates and copies synchronously;
 * only later calls with it are asynchronous.  Coset multiplier tables (N words per
 * (K, N, shift, device)) are kept for the sixteen most recently used combinations.
 *
 * All field elements are uint64 words, canonical in [0, p), p = 2^64 - 2^32 + 1.
 * "reference" below = JamesPetrie/VerInf; each entry point names the interface it
 * replaces.
 */
#ifndef VERINF_HIP_H
#define VERINF_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VI_OK 0
#define VI_EINVAL (-1)   /* bad argument (shape, size, null pointer)   */
#define VI_EHIP (-2)     /* a HIP runtime call failed                  */
#define VI_ENOMEM (-3)   /* workspace too small                        */

/* Message of the last failing call on this thread ("" if none). */
const char *vi_last_error(void);
/* Library version, "major.minor". */
const char *vi_version(void);

/* ---- elementwise field ops --------------------------------------------------
 * Replaces gl_mul / gl_add / gl_sub (prover/cuda_primitives.py:208-271, 1086-1088):
 * out[i] = a[i] op b[i].  op: 0 add, 1 sub, 2 mul.  out may alias a or b. */
int vi_gl_binop(int op, const uint64_t *a, const uint64_t *b, uint64_t *out, int64_t n, void *stream);

/* Same with a broadcast right operand: out[i] = a[i] op b[i % period].  Serves the
 * coset twist gl_mul(coeffs, gamma^l expanded) of prover/core.py:736-739 and
 * layergkr/gpu.py:198 without materialising the expanded operand. */
int vi_gl_binop_bcast(int op, const uint64_t *a, const uint64_t *b, int64_t period, uint64_t *out,
                      int64_t n, void *stream);

/* Replaces gl_neg (cuda_primitives.py:272-280; gl_extras.cuh:22-28) and
 * gl_pow / gl_inv / gl_inv_batched (cuda_primitives.py:281-303, 1089-1101):
 * op 0: out = -a;  op 1: out = a^arg;  op 2: out = a^(p-2) (arg ignored). */
int vi_gl_unop(int op, const uint64_t *a, uint64_t arg, uint64_t *out, int64_t n, void *stream);

/* Test hook (no counterpart in the reference): one device field primitive of the transform and sumcheck kernels
 * applied elementwise, so that the test-suite can drive it with chosen operands.
 * op 0: modular add of canonical a, b;  1: a - b;  2 / 3: sum / difference of the butterfly (a, b);
 * 4: a mod p of any word;  5: a * b of any words;  6: (hi = b, lo = a) mod p;
 * 7: the lazily reduced product, made canonical;  8 / 9: a * b + c with c = rotl(a, 17) ^ b, canonical / lazily
 * reduced then made canonical;  10: the five-word sum a b + b b + a a + ~a ~b + (2^64 - 1)^2 reduced;
 * 11: forty times a b summed in five words, reduced;
 * 100 + e, 0 <= e < 96: canonical a times 2^e (the compile-time shift twiddle);
 * 300 + e, 0 <= e < 192: the same for any exponent (2^96 = -1), in the form the coset loop of the fused LDE launch uses. */
int vi_gl_probe(int op, const uint64_t *a, const uint64_t *b, uint64_t *out, int64_t n, void *stream);

/* Replaces gl_axpy (cuda_primitives.py:282-288, 1104-1106; gl_extras.cuh:33-41):
 * y[i] += alpha * x[i], in place. */
int vi_gl_axpy(uint64_t *y, uint64_t alpha, const uint64_t *x, int64_t n, void *stream);

/* Replaces layergkr/gpu.py:326-338 gl_sum: out[0] = sum of a[0..n) in the field.
 * ws: vi_gl_sum_workspace_bytes(n) bytes of device scratch. */
size_t vi_gl_sum_workspace_bytes(int64_t n);
int vi_gl_sum(const uint64_t *a, int64_t n, uint64_t *out, void *ws, size_t ws_bytes, void *stream);

/* ---- dense products and Horner evaluation ------------------------------------------
 * Replace gl_matmul / gl_matvec (prover/cuda_primitives.py:485-510,
 * prover/kernels/gl_matmul.cuh:29-59) and poly_eval (cuda_primitives.py:462-479,
 * prover/kernels/gl_extras.cuh:93-108).  All matrices row-major and dense.
 *   vi_gl_matmul   C (m x n) = A (m x k) B (k x n); at most 65535 rows of A; the shape it is
 *                  tuned for is a few rows of A against a tall B (projection seam, combine).
 *   vi_gl_matvec   w (m) = M (m x n) v (n)
 *   vi_poly_eval   out[r][p] = sum_i coeffs[r][i] points[p]^i, coeffs (m x d), out (m x k) */
size_t vi_gl_matmul_workspace_bytes(int64_t m, int64_t k, int64_t n);
int vi_gl_matmul(const uint64_t *A, const uint64_t *B, uint64_t *C, int64_t m, int64_t k, int64_t n,
                 void *ws, size_t ws_bytes, void *stream);
int vi_gl_matvec(const uint64_t *M, const uint64_t *v, uint64_t *w, int64_t m, int64_t n, void *stream);
int vi_poly_eval(const uint64_t *coeffs, int64_t m, int64_t d, const uint64_t *points, int64_t k,
                 uint64_t *out, void *stream);

/* ---- NTT ---------------------------------------------------------------------
 * Replaces ntt_forward / ntt_inverse / ntt_forward_batched / ntt_inverse_batched
 * (prover/cuda_primitives.py:347-409, 1111-1114; prover/kernels/ntt.cuh:667-770):
 * in-place natural-order transform of each of the m contiguous rows of length n
 * (a power of two >= 2): X[k] = sum_j x[j] w^(jk), w = 7^((p-1)/n); the inverse
 * uses w^-1 and multiplies by n^-1.  Rows of more than 4096 elements are transformed in
 * several passes and need vi_ntt_workspace_bytes(m, n) bytes of scratch (0 for shorter rows:
 * up to 512 elements are one pass, 1024 .. 4096 one launch of two digits that meet in LDS).
 * Environment: VI_NTT_ROW=0 (read once per process) runs rows of 1024 .. 4096 elements as two
 * passes through the workspace instead; vi_ntt_workspace_bytes then reports what that needs. */
size_t vi_ntt_workspace_bytes(int64_t m, int64_t n);
int vi_ntt_batched(uint64_t *rows, int64_t m, int64_t n, int inverse, void *ws, size_t ws_bytes,
                   void *stream);

/* ---- coset low-degree extension ------------------------------------------------
 * Replaces the host recipe layergkr/gpu.py:141-203 (encode_batch_ntt) and
 * prover/core.py:721-743 (_coset_encode_codewords after ntt_inverse_batched,
 * core.py:798):  row r of `in` holds `width` <= K values of a polynomial at
 * w_K^c (slots [width, K) read as zero);  row r of `out` receives its N values at
 * shift * w_N^j.  K, N powers of two, 2 <= K <= N.  `in` rows are in_stride
 * elements apart, `out` rows out_stride >= N.  in and out must not overlap.
 * width = 0 is the zero polynomial: zero rows are written and `in` is not read.
 * The workspace may be smaller than vi_coset_lde_workspace_bytes(m, K, N): rows
 * are then processed in chunks; vi_coset_lde_min_workspace_bytes(K, N) is the
 * least that is accepted (one row).
 * Environment: VI_LDE_MERGED=0 (read once per process) makes the fused middle launch apply the coset factors
 * (shift * w_N^t)^i as one multiplication per coefficient and coset instead of split into shift^i, a power of two
 * and per-coset twiddle tables; same results, for measurements only. */
size_t vi_coset_lde_workspace_bytes(int64_t m, int64_t K, int64_t N);
size_t vi_coset_lde_min_workspace_bytes(int64_t K, int64_t N);
/* Number of kernel launches one vi_coset_lde call with these arguments issues
 * (for profilers and benchmarks); 0 on bad arguments. */
int64_t vi_coset_lde_launches(int64_t m, int64_t K, int64_t N, size_t ws_bytes);
int vi_coset_lde(const uint64_t *in, int64_t m, int64_t width, int64_t in_stride, int64_t K,
                 int64_t N, uint64_t shift, uint64_t *out, int64_t out_stride, void *ws,
                 size_t ws_bytes, void *stream);

/* The two halves of the coset LDE for callers that keep the row polynomials, as the production prover
 * does (prover/core.py:795-802: row_polys = iNTT_K(padded); codewords = _coset_encode_codewords(row_polys)).
 *
 * vi_coset_lde_coeffs: values -> coefficients (m rows of K words at `coeffs`, row pitch coeffs_stride >= K)
 * and, when out is not NULL, on to the codewords exactly as vi_coset_lde.  The coefficients replace
 * ntt_inverse_batched(padded.clone()) (prover/core.py:797-798); coeffs may equal `in` (same stride) for an
 * in-place transform.  out == NULL is need_codewords=False (prover/core.py:799-800).
 *
 * vi_coset_extend: coefficients (m rows of `width` <= K words, the rest read as zero) -> codewords; replaces
 * _coset_encode_codewords / _coset_encode_via_coset_ntt (prover/core.py:702-743).
 * Workspace and chunking as for vi_coset_lde. */
int vi_coset_lde_coeffs(const uint64_t *in, int64_t m, int64_t width, int64_t in_stride, int64_t K, int64_t N,
                        uint64_t shift, uint64_t *coeffs, int64_t coeffs_stride, uint64_t *out, int64_t out_stride,
                        void *ws, size_t ws_bytes, void *stream);
int vi_coset_extend(const uint64_t *coeffs, int64_t m, int64_t width, int64_t coeffs_stride, int64_t K, int64_t N,
                    uint64_t shift, uint64_t *out, int64_t out_stride, void *ws, size_t ws_bytes, void *stream);

/* ---- K-quant super-blocks -> field ---------------------------------------------
 * Replaces q4k_to_field / q5k_to_field / q6k_to_field behind kquant_to_field
 * (prover/kquant_cuda.py:60-139, 170-177): raw holds n_blocks super-blocks of
 * 144 / 176 / 210 bytes (qtype 4 / 5 / 6); out receives n_blocks*256 field
 * elements, round-half-even(double(fp32 dequant) * S), negatives as p - |x|. */
int vi_kquant_to_field(int qtype, const uint8_t *raw, int64_t n_blocks, double S, uint64_t *out,
                       void *stream);
/* The same decode of a (d_out, d_in) matrix stored row by row (d_in a multiple of 256), written
 * transposed: out[c * d_out + r] = weight (r, c).  Replaces the decode followed by the
 * `.view(d_out, d_in).T.contiguous()` pass with which the loader brings an expert matrix into
 * (k_in, n_out) order (prover/loader.py:427-436). */
int vi_kquant_to_field_transposed(int qtype, const uint8_t *raw, int64_t d_out, int64_t d_in, double S,
                                  uint64_t *out, void *stream);

/* ---- multilinear sumcheck --------------------------------------------------------
 * Replace the per-round torch composition of layergkr/gpu.py:341-410 (fold_t,
 * gl_sum, prove_terms_gpu) with fused kernels.
 *
 * A problem is n_tables tables of `len` = 2*half values and n_terms terms; term k
 * has coefficient coeffs[k] and factors tables[factor_idx[term_off[k] ..
 * term_off[k+1])].  deg = the largest factor count.  For x = 0..deg
 *   S(x) = sum_k coeffs[k] * sum_{i<half} prod_j (f_j[i] + x (f_j[half+i] - f_j[i])).
 *
 * The descriptor arrays (tables, term_off, factor_idx, coeffs) are HOST memory;
 * they are passed to the kernel by value, VI_SC_MAX_TABLES / _TERMS / _FACTORS at a
 * time: a larger sum (like the reference's, any number of tables and terms; at most 7
 * factors per term) is evaluated in groups of consecutive terms, one launch each --
 * only vi_sumcheck_eval_static keeps to a single descriptor.  out_samples: deg+1 words
 * the GPU can write -- device memory or pinned host memory (hipHostMalloc), the latter
 * saves the copy back.  ws: device scratch of vi_sumcheck_workspace_bytes() bytes. */
#define VI_SC_MAX_TABLES 64
#define VI_SC_MAX_TERMS 64
#define VI_SC_MAX_FACTORS 128
size_t vi_sumcheck_workspace_bytes(void);

/* samples of the current round (sumcheck.py:194-205 / gpu.py:384-394) */
int vi_sumcheck_eval(const uint64_t *const *tables, int n_tables, int64_t half, const int *term_off,
                     const int *factor_idx, const uint64_t *coeffs, int n_terms,
                     uint64_t *out_samples, void *ws, size_t ws_bytes, void *stream);

/* vi_sumcheck_eval without a workspace argument and without any allocation: for callers that cannot call
 * hipMalloc (code under HIP graph capture, tight serving loops, harnesses that forbid it).  It has no
 * counterpart in the reference.  The per-workgroup partial sums live in a file-scope device array of the
 * library, vi_sumcheck_workspace_bytes() = 128 KiB per GPU, held until the process ends; its device address is
 * looked up once per device on the first call there.  half above VI_SC_STATIC_MAX_HALF is rejected (VI_EINVAL).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race;
 * calls queued on one stream do not.  Same results as vi_sumcheck_eval. */
#define VI_SC_STATIC_MAX_HALF ((int64_t)1 << 32)
int vi_sumcheck_eval_static(const uint64_t *const *tables, int n_tables, int64_t half, const int *term_off,
                            const int *factor_idx, const uint64_t *coeffs, int n_terms, uint64_t *out_samples,
                            void *stream);

/* fold every table by r (sumcheck.py:51-54 / gpu.py:341-347): dst[t][i] = src[t][i] +
 * r (src[t][half+i] - src[t][i]), i < half; and, when half >= 2, also return the
 * NEXT round's samples computed from the folded tables in the same pass.
 * dst[t] may equal src[t] (fold in place).  out_samples may be NULL (fold only).
 * claim (host pointer, may be NULL): the value the next round's polynomial must sum to,
 * S(0) + S(1) = S_previous(r), which the caller knows by interpolating the previous
 * samples at r.  When given, S(1) is returned as claim - S(0) instead of being summed
 * (same value, a quarter less work at degree 3). */
int vi_sumcheck_fold_eval(const uint64_t *const *src, uint64_t *const *dst, int n_tables,
                          int64_t half, uint64_t r, const int *term_off, const int *factor_idx,
                          const uint64_t *coeffs, int n_terms, const uint64_t *claim,
                          uint64_t *out_samples, void *ws, size_t ws_bytes, void *stream);

/* The whole prover loop of layergkr/gpu.py:381-409 / layergkr/sumcheck.py:191-223 on the
 * host side of the library: evaluate, wait, hand the round's deg+1 samples to `coin`, fold
 * by the challenge it returns while evaluating the next round, ... for log2(size) rounds.
 * `coin(round, samples, n_samples, &r, user)` runs on the calling thread between launches
 * and returns 0, or non-zero to abort (the call then returns VI_EINVAL).
 *   tables        n_tables device tables of `size` = 2^v words (left untouched)
 *   work          n_tables device buffers of size/2 words (the folded tables live here)
 *   host_samples  host_words >= VI_SC_HOST_WORDS (16) words of PINNED host memory (hipHostMalloc): words 0..7 receive
 *                 each round's samples and word 8 a tag of the call and round that has arrived; the host thread waits
 *                 on that word (and queries the stream from time to time) rather than synchronising the stream
 *                 every round.  One buffer per proof in flight.  A smaller host_words is rejected (VI_EINVAL).
 *   out_samples   host, v * (deg+1) words: S_round(x) for x = 0..deg (no mask applied)
 *   out_challenges host, v words: the challenges, reduced mod p
 * The final fold (after the last round) is not performed, as nothing reads it.  The call returns, also with an
 * error, only after every kernel it has queued has retired.  Use it when the coin needs a round's samples; the
 * reference's own coin takes the round number alone, which vi_sumcheck_prove_coins serves without host waits. */
#define VI_SC_HOST_WORDS 16
typedef int (*vi_coin_fn)(int round, const uint64_t *samples, int n_samples, uint64_t *challenge, void *user);
int vi_sumcheck_prove(const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                      const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms,
                      vi_coin_fn coin, void *user, uint64_t *host_samples, size_t host_words, uint64_t *out_samples,
                      uint64_t *out_challenges, void *ws, size_t ws_bytes, void *stream);

/* The same proof with every challenge known up front, which is what the reference's interface provides: its prover
 * calls `coin(rnd)` with the round number only (layergkr/gpu.py:403, layergkr/sumcheck.py:217) and its callers draw
 * the coins before the proof starts (layergkr/full_layer.py:222-224, layergkr/relations.py:122-123,
 * layergkr/layer.py:123-125).  All rounds are queued on the stream without a host round trip, and the call returns
 * without waiting.  A single product of up to four distinct tables and the hadamard gate batch eq * (a * b + c' * c)
 * run three rounds per pass over the tables and every round of the last few thousand entries in one workgroup; other
 * sums keep one launch per round.
 *   challenges    host, v = log2(size) words (reduced mod p by the callee)
 *   samples       v rows of 8 words the GPU can write (device memory or pinned host memory): S_round(x) at
 *                 samples[8 * round + x], x = 0..deg, complete once the stream has reached the end of the call's work
 *   work          n_tables device buffers of size/2 words; tables are left untouched
 *   ws            vi_sumcheck_prove_coins_workspace_bytes(size) bytes of device scratch
 * At most 40 rounds. */
size_t vi_sumcheck_prove_coins_workspace_bytes(int64_t size);
int vi_sumcheck_prove_coins(const uint64_t *const *tables, uint64_t *const *work, int n_tables, int64_t size,
                            const int *term_off, const int *factor_idx, const uint64_t *coeffs, int n_terms,
                            const uint64_t *challenges, uint64_t *samples, void *ws, size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------
 * BLAKE3 column digests and Merkle levels of a committed codeword matrix.
 *
 * vi_hash_columns replaces hash_columns_streamed (prover/cuda_primitives.py:1252-1254,
 * kernel prover/kernels/blake3_columns.cuh:47-170): digests[j] = BLAKE3 of column j of the
 * row-major (m, n) matrix (row pitch row_stride words) taken as m little-endian 8-byte words,
 * the leaf prover/protocol.py:100-104 defines.  m = 0 hashes the empty message.
 * Workspace: vi_hash_columns_workspace_bytes(m, n) = 48 * n * ceil(m / 128) bytes.
 *
 * vi_hash_columns_update / _finalize replace the streaming accumulator
 * (prover/cuda_primitives.py:1297-1386: hash_columns_stream_init/_update/_finalize): the matrix
 * arrives in row slabs; every slab but the last holds a multiple of 128 rows (one BLAKE3 chunk)
 * and states its first chunk's index chunk0; n_chunks_total = ceil(m / 128) is fixed up front.
 * Slabs may arrive in any order and on any stream as long as finalize is ordered after them.
 * The workspace is the accumulator state and must persist from the first update to finalize.
 *
 * vi_merkle_level replaces merkle_one_level + the odd-node duplication around it
 * (prover/cuda_primitives.py:1388-1402, layergkr/rs.py:135-144): out[i] = BLAKE3(nodes[2i] ||
 * nodes[2i+1]) over 32-byte nodes, the odd last node paired with itself; out holds
 * ceil(count / 2) nodes.  nodes and out must not overlap.
 *
 * vi_merkle_tree builds every level above `count` leaves with up to nine levels per launch (the loop of
 * merkle_build_blake3, prover/cuda_primitives.py:1388-1402): levels_out receives level 1 (ceil(count/2)
 * nodes), then level 2, ... up to the root, vi_merkle_tree_nodes(count) nodes of 32 bytes in all. */
size_t vi_hash_columns_workspace_bytes(int64_t m, int64_t n);
int vi_hash_columns(const uint64_t *mat, int64_t m, int64_t n, int64_t row_stride, uint8_t *digests, void *ws,
                    size_t ws_bytes, void *stream);
int vi_hash_columns_update(const uint64_t *rows, int64_t slab_rows, int64_t n, int64_t row_stride, int64_t chunk0,
                           int64_t n_chunks_total, void *ws, size_t ws_bytes, void *stream);
int vi_hash_columns_finalize(int64_t n, int64_t n_chunks_total, void *ws, size_t ws_bytes, uint8_t *digests,
                             void *stream);
int vi_merkle_level(const uint8_t *nodes, int64_t count, uint8_t *out, void *stream);
int64_t vi_merkle_tree_nodes(int64_t count);
int vi_merkle_tree(const uint8_t *leaves, int64_t count, uint8_t *levels_out, void *stream);

/* Zero-knowledge pad generator; replaces row_prg / row_prg_indexed (prover/cuda_primitives.py:1262-1294,
 * kernels :877-930): out[r * out_stride + k] = (BLAKE3(seed[32] || row_le8 || k_le8)[0:8] as a little-endian
 * word) mod p for r < n_rows, k < slack, with row = row_indices[r] if row_indices is not NULL, else the
 * 32-bit sum (uint32)(row_offset + r) as in the reference's contiguous variant.  seed is a device pointer.
 * out_stride >= slack lets the pad be written straight into columns [ELL, K) of the padded message
 * matrix (prover/core.py:783-794) without an intermediate tensor. */
int vi_row_prg(const uint8_t *seed, const uint64_t *row_indices, int64_t row_offset, int64_t n_rows, int64_t slack,
               uint64_t *out, int64_t out_stride, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Multilinear helpers around the sumchecks.  A point z is a HOST array of n_vars <= 32 words (reduced
 * mod p by the callee).
 *
 * vi_eq_vector replaces eq_vector (layergkr/logup.py:61-69) for device consumers:
 *   out[i] = prod_j (bit(i, pos_j) ? z_j : 1 - z_j), 2^n_vars words,
 * with pos_j = j when msb_first == 0 -- z_0 on the least significant index bit, which is what the
 * reference's doubling loop produces -- and pos_j = n_vars - 1 - j when msb_first != 0, the variable
 * order of mle_eval and of the sumcheck folds.
 * vi_mle_eval replaces mle_eval (layergkr/sumcheck.py:40-48) for device tables: out[t] = the
 * multilinear extension of row t of `tables` (n_tables rows of 2^n_vars words, pitch row_stride)
 * at z (z_0 on the most significant bit), one pass per table; out is a device array of n_tables words.
 * Workspace: vi_mle_eval_workspace_bytes(n_tables) = 8 KiB per table. */
int vi_eq_vector(const uint64_t *z, int n_vars, int msb_first, uint64_t *out, void *stream);
size_t vi_mle_eval_workspace_bytes(int64_t n_tables);
int vi_mle_eval(const uint64_t *tables, int64_t n_tables, int64_t row_stride, const uint64_t *z, int n_vars,
                uint64_t *out, void *ws, size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------
 * The remaining field primitives of the production prover that sit next to the path.
 *
 * vi_challenge replaces challenge_vec / challenge_at (prover/cuda_primitives.py:551-592, 1233-1248):
 *   out[i] = challenge(seed, cid_i, label) = le128(BLAKE3(seed[32] || label || cid_le8)[0:16]) mod p
 * (prover/protocol.py:127-135) with cid_i = cids[i], or i when cids is NULL.  seed (32 bytes, 4-byte aligned) and
 * label (label_len <= 8 bytes) are device pointers.
 *
 * vi_gl_spmv replaces gl_spmv / gl_spmv_challenged (prover/cuda_primitives.py:512-548, prover/kernels/gl_spmv.cuh):
 *   y[i] = sum over p in [row_ptr[i], row_ptr[i+1]) of values[p] * x[col_idx[p]]   (CSR, all words uint64),
 * and with x == NULL the combiner entry is challenge(seed, col_idx[p], label) computed in place.
 *
 * vi_lookup_multiplicities replaces lookup_multiplicities[_into] and its range form
 * (prover/cuda_primitives.py:1008-1052, prover/kernels/gl_extras.cuh:118-150): mult[j] += 1 for every i whose
 * x[i] equals table[j] (the first such j); values not in the table count nowhere.  table_is_range != 0 promises
 * table[j] == j, which makes the search an index.  mult accumulates: zero it for a fresh histogram. */
int vi_challenge(const uint8_t *seed, const uint8_t *label, int label_len, const uint64_t *cids, int64_t n, uint64_t *out,
                 void *stream);
int vi_gl_spmv(const uint64_t *values, const uint64_t *col_idx, const uint64_t *row_ptr, int64_t n_rows, int64_t nnz,
               const uint64_t *x, const uint8_t *seed, const uint8_t *label, int label_len, uint64_t *y, void *stream);
int vi_lookup_multiplicities(const uint64_t *x, int64_t n_x, const uint64_t *table, int64_t n_table, int table_is_range,
                             uint64_t *mult, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Measurement hook (no counterpart in the reference): the issue rate of the integer VALU instructions the field
 * arithmetic and the hashing consist of, which is the bound their kernels are put against.
 * vi_valu_probe launches `blocks` workgroups of 256 threads that each run `iters` times a block of one instruction
 * class (kind < vi_valu_probe_count(), named by vi_valu_probe_name) on independent registers; the caller times the
 * launch.  *wave_instructions receives the VALU instructions issued, counted per wavefront.  out: blocks * 256
 * words, clocks: blocks * 4 words of device memory; clocks[4b .. 4b+3] = the shader-clock counter at the start and
 * the end of workgroup b, then the constant-rate counter (vi_wall_clock_khz() ticks per millisecond) at the same
 * two moments: their ratio is the clock the SIMDs ran at. */
int vi_valu_probe_count(void);
const char *vi_valu_probe_name(int kind);
int vi_wall_clock_khz(void);
int vi_valu_probe(int kind, int iters, int blocks, uint64_t *out, uint64_t *clocks, int64_t *wave_instructions,
                  void *stream);

#ifdef __cplusplus
}
#endif
#endif /* VERINF_HIP_H */

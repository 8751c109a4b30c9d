"""Drop-in for the reference's `prover/cuda_primitives.py` on MI355X.

Same public names, argument conventions and error behaviour
(prover/cuda_primitives.py:1-41, 198-1446): every function works on contiguous
`torch.uint64` (hashes: `torch.uint8`) tensors that live on the GPU ("cuda" is
ROCm's device name in PyTorch), binary ops want equal shapes and return a new
tensor, the NTTs are in place and return None, violations raise RuntimeError.
Underneath, each call is one ctypes hop into libverinf_hip.so on torch's current
stream; nothing is JIT-compiled and there is no CPU fallback.

Covered: field ops, NTTs, Reed-Solomon / coset encoding, polynomial helpers,
gl_matmul / gl_matvec / gl_spmv[_challenged], challenge_vec / challenge_at,
hash_columns_streamed / MerkleColumnAccumulator / merkle_build_blake3, row_prg[_indexed],
lookup_multiplicities[_into].  Not provided: the `interp_band*` family.

Additions over the reference surface:
  coset_lde(messages, k_deg, n_lig, shift)   the fused iNTT -> twist -> zero-extend -> NTT
  coset_lde_with_coeffs(...)                 the same, also returning the row polynomials
  coset_extend(coeffs, k_deg, n_lig, shift)  coefficients -> coset evaluations
  gl_mul_bcast(a, b_row)                     a * (b_row broadcast over rows) without materialising it
  row_prg(..., out=)                         the pad written straight into a column slice
"""
import torch

from .. import _lib

P = (1 << 64) - (1 << 32) + 1
GLOBAL_G = 7

_OPS = {"add": 0, "sub": 1, "mul": 2}


def _check_u64(t, name):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be CUDA")
    if t.dtype != torch.uint64:
        raise RuntimeError(f"{name} dtype must be uint64")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _binop(op, a, b, who):
    _check_u64(a, "a")
    _check_u64(b, "b")
    if a.shape != b.shape:
        raise RuntimeError(f"{who}: shape mismatch")
    out = torch.empty_like(a)
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().vi_gl_binop(_OPS[op], a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                          a.numel(), _lib.stream_ptr()))
    return out


# ---- elementwise field (cuda_primitives.py:1086-1106) ---------------------------
def gl_mul(a, b):
    return _binop("mul", a, b, "gl_mul")


def gl_add(a, b):
    return _binop("add", a, b, "gl_add")


def gl_sub(a, b):
    return _binop("sub", a, b, "gl_sub")


def gl_mul_bcast(a, b_row):
    """a[..., i] * b_row[i]: the coset twist without `expand().contiguous()`."""
    _check_u64(a, "a")
    _check_u64(b_row, "b_row")
    if b_row.dim() != 1 or a.shape[-1] != b_row.numel():
        raise RuntimeError("gl_mul_bcast: last dimension mismatch")
    out = torch.empty_like(a)
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().vi_gl_binop_bcast(2, a.data_ptr(), b_row.data_ptr(), b_row.numel(),
                                                out.data_ptr(), a.numel(), _lib.stream_ptr()))
    return out


def _unop(op, a, arg):
    _check_u64(a, "a")
    out = torch.empty_like(a)
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().vi_gl_unop(op, a.data_ptr(), int(arg) & ((1 << 64) - 1), out.data_ptr(),
                                         a.numel(), _lib.stream_ptr()))
    return out


def gl_neg(a):
    return _unop(0, a, 0)


def gl_pow(base, exp):
    exp = int(exp)
    if exp < 0 or exp >= (1 << 64):
        raise RuntimeError("gl_pow: exponent must fit an unsigned 64-bit integer")
    return _unop(1, base, exp)


def gl_inv(a):
    """Elementwise Fermat inverse a^(P-2)."""
    return _unop(2, a, 0)


def gl_inv_batched(a):
    """Inverse of every element of a 1-D tensor, 0 -> 0, the values of the reference's
    per-lane Fermat power (cuda_primitives.py:289-303); computed eight elements to one
    inversion with Montgomery's trick in registers."""
    _check_u64(a, "a")
    if a.dim() != 1:
        raise RuntimeError("gl_inv_batched: 1-D input only")
    return _unop(2, a, 0)


def gl_axpy(y, alpha, x):
    """In-place y += alpha * x mod P."""
    _check_u64(y, "y")
    _check_u64(x, "x")
    if y.shape != x.shape:
        raise RuntimeError("gl_axpy: shape mismatch")
    with torch.cuda.device(y.device):
        _lib.check(_lib.lib().vi_gl_axpy(y.data_ptr(), int(alpha) % P, x.data_ptr(), y.numel(),
                                         _lib.stream_ptr()))


# ---- NTT (cuda_primitives.py:347-409, 1111-1114) --------------------------------
def _is_pow2(n):
    return n > 0 and (n & (n - 1)) == 0


_NTT_WS_CAP = 1 << 30


def _ntt(rows, m, n, inverse):
    L = _lib.lib()
    with torch.cuda.device(rows.device):
        # the library transforms the rows in chunks that fit the workspace it is given: one row is the minimum,
        # 1 GiB is enough to fill the GPU, and a large batch does not double its footprint for the process's life
        need = min(L.vi_ntt_workspace_bytes(m, n), max(_NTT_WS_CAP, n * 8))
        ws = _lib.workspace(need, rows.device, "ntt") if need else None
        _lib.check(L.vi_ntt_batched(rows.data_ptr(), m, n, int(inverse),
                                    ws.data_ptr() if ws is not None else None,
                                    ws.numel() if ws is not None else 0, _lib.stream_ptr()))


def _ntt_1d(a, inverse):
    _check_u64(a, "a")
    if a.dim() != 1:
        raise RuntimeError("NTT input must be 1-D")
    n = a.numel()
    if not (_is_pow2(n) and n >= 2):
        raise RuntimeError("NTT length must be power of 2 >= 2")
    _ntt(a, 1, n, inverse)


def _ntt_2d(rows, inverse):
    _check_u64(rows, "rows")
    if rows.dim() != 2:
        raise RuntimeError("batched NTT expects (m, n)")
    m, n = int(rows.shape[0]), int(rows.shape[1])
    if not (_is_pow2(n) and n >= 2):
        raise RuntimeError("row length must be power of 2 >= 2")
    if m:
        _ntt(rows, m, n, inverse)


def ntt_forward(a):
    _ntt_1d(a, False)


def ntt_inverse(a):
    _ntt_1d(a, True)


def ntt_forward_batched(rows):
    _ntt_2d(rows, False)


def ntt_inverse_batched(rows):
    _ntt_2d(rows, True)


# ---- Reed-Solomon ------------------------------------------------------------------
def _lde_args(messages, k_deg, n_lig, what="messages"):
    if not isinstance(messages, torch.Tensor) or not messages.is_cuda:
        raise RuntimeError(f"{what} must be CUDA")
    if messages.dtype != torch.uint64:
        raise RuntimeError(f"{what} dtype must be uint64")
    if messages.dim() != 2:
        raise RuntimeError(f"expected (m, width) {what}")
    k_deg, n_lig = int(k_deg), int(n_lig)
    m, w = int(messages.shape[0]), int(messages.shape[1])
    if not (_is_pow2(k_deg) and k_deg >= 2):
        raise RuntimeError("k_deg must be power of 2 >= 2")
    if not (_is_pow2(n_lig) and n_lig >= k_deg):
        raise RuntimeError("n_lig must be a power of 2 >= k_deg")
    if w > k_deg:
        raise RuntimeError(f"{what}' second dim must be <= k_deg")
    if m and w and messages.stride(1) != 1:
        raise RuntimeError(f"{what} must have unit column stride")
    in_stride = int(messages.stride(0)) if (m > 1 and w) else max(w, 1)
    if in_stride < w:
        raise RuntimeError(f"{what} rows overlap")
    return k_deg, n_lig, m, w, in_stride


def _lde_out(out, m, n_lig, device):
    if out is None:
        return torch.empty((m, n_lig), dtype=torch.uint64, device=device)
    _check_u64(out, "out")
    if tuple(out.shape) != (m, n_lig):
        raise RuntimeError("out must be (m, n_lig)")
    return out


def coset_lde(messages, k_deg, n_lig, shift=GLOBAL_G, out=None):
    """(m, w <= K) values at the K-th roots of unity -> (m, N) codewords on the coset
    shift * <w_N>, in one fused pipeline: inverse NTT_K, coefficient twist, zero
    extension and forward transform (the recipe of layergkr/gpu.py:141-203 and
    prover/core.py:721-743, 798).  Rows may be a strided view with unit column
    stride, so `buf[:, :ELL]` needs no copy."""
    k_deg, n_lig, m, w, in_stride = _lde_args(messages, k_deg, n_lig)
    out = _lde_out(out, m, n_lig, messages.device)
    if m == 0:
        return out
    if w == 0:                      # an empty message is the zero polynomial
        return out.view(torch.int64).zero_().view(torch.uint64)
    L = _lib.lib()
    with torch.cuda.device(messages.device):
        ws = _lib.workspace(L.vi_coset_lde_workspace_bytes(m, k_deg, n_lig), messages.device, "lde")
        _lib.check(L.vi_coset_lde(messages.data_ptr(), m, w, in_stride, k_deg, n_lig, int(shift) % P,
                                  out.data_ptr(), n_lig, ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    return out


def coset_lde_with_coeffs(messages, k_deg, n_lig, shift=GLOBAL_G, need_codewords=True, out=None, in_place=False):
    """As coset_lde, but also returns the row polynomials the pipeline passes through:
    (coeffs (m, K), codewords (m, N) or None).  One call stands for
    `row_polys = padded.clone(); ntt_inverse_batched(row_polys); _coset_encode_codewords(row_polys)`
    (prover/core.py:795-802); need_codewords=False stops after the coefficients.
    in_place: `messages` is a contiguous (m, K) tensor the caller gives up; the coefficients overwrite it and it is
    returned as `coeffs` (the reference's clone has no counterpart then)."""
    k_deg, n_lig, m, w, in_stride = _lde_args(messages, k_deg, n_lig)
    if in_place:
        if w != k_deg or in_stride != k_deg:
            raise RuntimeError("coset_lde_with_coeffs(in_place=True) needs a contiguous (m, K_DEG) tensor")
        coeffs = messages
    else:
        coeffs = torch.empty((m, k_deg), dtype=torch.uint64, device=messages.device)
    out = _lde_out(out, m, n_lig, messages.device) if need_codewords else None
    if m == 0:
        return coeffs, out
    if w == 0:
        coeffs.view(torch.int64).zero_()
        if out is not None:
            out.view(torch.int64).zero_()
        return coeffs, out
    L = _lib.lib()
    with torch.cuda.device(messages.device):
        ws = _lib.workspace(L.vi_coset_lde_workspace_bytes(m, k_deg, n_lig), messages.device, "lde")
        _lib.check(L.vi_coset_lde_coeffs(messages.data_ptr(), m, w, in_stride, k_deg, n_lig, int(shift) % P,
                                         coeffs.data_ptr(), k_deg, out.data_ptr() if out is not None else None, n_lig,
                                         ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    return coeffs, out


def coset_extend(coeffs, k_deg, n_lig, shift=GLOBAL_G, out=None):
    """(m, w <= K) polynomial coefficients -> (m, N) evaluations on shift * <w_N>: the
    twist, zero extension and forward transform of prover/core.py:721-743 (and its
    cosets formulation :702-718) without the `(m, N)` staging buffer."""
    k_deg, n_lig, m, w, in_stride = _lde_args(coeffs, k_deg, n_lig, "coeffs")
    out = _lde_out(out, m, n_lig, coeffs.device)
    if m == 0:
        return out
    if w == 0:
        return out.view(torch.int64).zero_().view(torch.uint64)
    L = _lib.lib()
    with torch.cuda.device(coeffs.device):
        ws = _lib.workspace(L.vi_coset_lde_workspace_bytes(m, k_deg, n_lig), coeffs.device, "lde")
        _lib.check(L.vi_coset_extend(coeffs.data_ptr(), m, w, in_stride, k_deg, n_lig, int(shift) % P,
                                     out.data_ptr(), n_lig, ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    return out


def rs_encode_rows(messages, n_lig, k_deg):
    """(m, K_DEG) uint64 -> (m, N_LIG): iNTT_K, zero-extend, NTT_N with NO coset shift
    (cuda_primitives.py:417-456) -- the legacy encoder, i.e. the LDE with shift 1."""
    _check_u64(messages, "messages")
    if messages.dim() != 2:
        raise RuntimeError("rs_encode_rows expects (m, K_DEG)")
    if int(messages.shape[1]) != int(k_deg):
        raise RuntimeError("messages's second dim must equal k_deg")
    return coset_lde(messages, k_deg, n_lig, shift=1)


# ---- linear algebra mod P (cuda_primitives.py:485-510, 1188-1189) --------------------
def gl_matmul(A, B):
    """(m, k) @ (k, n) over the field."""
    _check_u64(A, "A")
    _check_u64(B, "B")
    if A.dim() != 2 or B.dim() != 2:
        raise RuntimeError("gl_matmul: 2-D inputs")
    m, k, kb, n = int(A.shape[0]), int(A.shape[1]), int(B.shape[0]), int(B.shape[1])
    if k != kb:
        raise RuntimeError("gl_matmul: inner dim mismatch")
    C = torch.empty((m, n), dtype=torch.uint64, device=A.device)
    L = _lib.lib()
    with torch.cuda.device(A.device):
        for lo in range(0, m, 65535):
            hi = min(lo + 65535, m)
            need = L.vi_gl_matmul_workspace_bytes(hi - lo, k, n)
            ws = _lib.workspace(need, A.device, "matmul") if need else None
            _lib.check(L.vi_gl_matmul(A[lo:hi].data_ptr() if m else None, B.data_ptr(), C[lo:hi].data_ptr() if m else None,
                                      hi - lo, k, n, ws.data_ptr() if ws is not None else None,
                                      ws.numel() if ws is not None else 0, _lib.stream_ptr()))
    return C


def gl_matvec(M, v):
    """(m, n) @ (n,) over the field."""
    _check_u64(M, "M")
    _check_u64(v, "v")
    if M.dim() != 2 or v.dim() != 1:
        raise RuntimeError("gl_matvec: (m,n) @ (n,)")
    m, n = int(M.shape[0]), int(M.shape[1])
    if int(v.shape[0]) != n:
        raise RuntimeError("gl_matvec: dim mismatch")
    out = torch.empty((m,), dtype=torch.uint64, device=M.device)
    with torch.cuda.device(M.device):
        _lib.check(_lib.lib().vi_gl_matvec(M.data_ptr(), v.data_ptr(), out.data_ptr(), m, n, _lib.stream_ptr()))
    return out


# ---- polynomials in coefficient form (cuda_primitives.py:1138-1183) -----------------
def poly_eval(coeffs, points):
    """Horner evaluation; coeffs (d,) -> (k,) or (m, d) -> (m, k)."""
    _check_u64(coeffs, "coeffs")
    _check_u64(points, "points")
    if points.dim() != 1:
        raise RuntimeError("points must be 1-D")
    if coeffs.dim() not in (1, 2):
        raise RuntimeError("coeffs must be 1-D or 2-D")
    one_d = coeffs.dim() == 1
    m = 1 if one_d else int(coeffs.shape[0])
    d = int(coeffs.shape[-1])
    k = int(points.shape[0])
    out = torch.empty((m, k), dtype=torch.uint64, device=coeffs.device)
    L = _lib.lib()
    with torch.cuda.device(coeffs.device):
        for lo in range(0, m, 65535):
            hi = min(lo + 65535, m)
            src = coeffs if one_d else coeffs[lo:hi]
            _lib.check(L.vi_poly_eval(src.data_ptr(), hi - lo, d, points.data_ptr(), k, out[lo:hi].data_ptr(),
                                      _lib.stream_ptr()))
    return out.reshape(k) if one_d else out


def _next_pow2(n):
    p = 2
    while p < n:
        p *= 2
    return p


def _padded(src, shape):
    out = torch.zeros(shape, dtype=torch.uint64, device=src.device)
    if src.dim() == 1:
        out.view(torch.int64)[: src.numel()] = src.view(torch.int64)
    else:
        out.view(torch.int64)[:, : src.shape[1]] = src.view(torch.int64)
    return out


def poly_mul(a, b):
    """Product of two coefficient vectors via NTT."""
    assert a.dim() == 1 and b.dim() == 1
    if a.numel() == 0 or b.numel() == 0:
        return torch.empty(0, dtype=torch.uint64, device=a.device)
    out_len = a.numel() + b.numel() - 1
    n = _next_pow2(out_len)
    fa, fb = _padded(a, (n,)), _padded(b, (n,))
    ntt_forward(fa)
    ntt_forward(fb)
    prod = gl_mul(fa, fb)
    ntt_inverse(prod)
    return prod[:out_len].contiguous()


def poly_add(a, b):
    """Sum of two coefficient vectors of possibly different lengths."""
    assert a.dim() == 1 and b.dim() == 1
    n = max(a.numel(), b.numel())
    if n == 0:
        return torch.empty(0, dtype=torch.uint64, device=a.device)
    return gl_add(_padded(a, (n,)), _padded(b, (n,)))


def poly_mul_batched(A, B):
    """Row-wise poly_mul of two (m, d) tensors -> (m, 2d - 1)."""
    assert A.dim() == 2 and B.dim() == 2 and A.shape == B.shape
    m, d = int(A.shape[0]), int(A.shape[1])
    out_len = 2 * d - 1
    n = _next_pow2(out_len)
    fa, fb = _padded(A, (m, n)), _padded(B, (m, n))
    ntt_forward_batched(fa)
    ntt_forward_batched(fb)
    prod = gl_mul(fa, fb)
    ntt_inverse_batched(prod)
    return prod.view(torch.int64)[:, :out_len].contiguous().view(torch.uint64)


# ---- BLAKE3 column hash + Merkle (prover/cuda_primitives.py:1250-1402) ----

_BLAKE3_CHUNK_ROWS = 128          # a BLAKE3 chunk is 1024 bytes = 128 uint64 rows of one column


def _n_chunks(n_rows):
    return max(1, (int(n_rows) + _BLAKE3_CHUNK_ROWS - 1) // _BLAKE3_CHUNK_ROWS)


def hash_columns_streamed(matrix):
    """(m, n) uint64 -> (n, 32) uint8 BLAKE3 column digests
    (prover/cuda_primitives.py:1252-1254).  No row cap; rows may be strided, the
    columns of a row must be adjacent."""
    if not isinstance(matrix, torch.Tensor) or not matrix.is_cuda:
        raise RuntimeError("matrix must be CUDA")
    if matrix.dtype != torch.uint64:
        raise RuntimeError("matrix dtype must be uint64")
    if matrix.dim() != 2:
        raise RuntimeError("matrix must be 2D")
    m, n = int(matrix.shape[0]), int(matrix.shape[1])
    if n == 0:
        return torch.empty((0, 32), dtype=torch.uint8, device=matrix.device)
    if n > 1 and m > 0 and matrix.stride(1) != 1:
        raise RuntimeError("matrix must be contiguous")
    stride = int(matrix.stride(0)) if m > 1 else n
    if stride < n:
        raise RuntimeError("matrix must be contiguous")
    L = _lib.lib()
    out = torch.empty((n, 32), dtype=torch.uint8, device=matrix.device)
    nbytes = L.vi_hash_columns_workspace_bytes(m, n)
    ws = _lib.workspace(nbytes, matrix.device, "hash")
    _lib.check(L.vi_hash_columns(matrix.data_ptr(), m, n, stride, out.data_ptr(), ws.data_ptr(), ws.numel(),
                                 _lib.stream_ptr()))
    return out


class MerkleColumnAccumulator:
    """Column digests of a tall matrix that arrives in row slabs
    (prover/cuda_primitives.py:1297-1386): same digests as hash_columns_streamed on
    the concatenation, without ever holding the whole matrix.

    `n_total_rows` is fixed up front.  update() takes any number of rows; rows
    short of a 128-row BLAKE3 chunk are kept until a later call completes them.
    All complete chunks of a slab go to the device in one launch, and the state
    between calls is the table of chunk chaining values (32 bytes per chunk and
    column).  Like the reference it wants more than one chunk in total."""

    def __init__(self, n_cols: int, n_total_rows: int):
        assert n_total_rows > _BLAKE3_CHUNK_ROWS, (
            "MerkleColumnAccumulator requires multi-BLAKE3-chunk input; "
            "for <=128 rows use hash_columns_streamed directly")
        self.n_cols = int(n_cols)
        self.n_total_rows = int(n_total_rows)
        self.n_chunks_total = _n_chunks(n_total_rows)
        L = _lib.lib()
        nbytes = L.vi_hash_columns_workspace_bytes(self.n_total_rows, self.n_cols)
        self._states = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        self._chunks_seen = 0
        self._rows_seen = 0
        self._partial = None

    def _emit(self, rows):
        L = _lib.lib()
        rows = rows if rows.stride(1) == 1 else rows.contiguous()
        k = int(rows.size(0))
        _lib.check(L.vi_hash_columns_update(rows.data_ptr(), k, self.n_cols, int(rows.stride(0)) if k > 1 else self.n_cols,
                                            self._chunks_seen, self.n_chunks_total, self._states.data_ptr(),
                                            self._states.numel(), _lib.stream_ptr()))
        self._chunks_seen += _n_chunks(k)
        self._rows_seen += k

    def update(self, rows):
        """rows: (k, n_cols) uint64, any k >= 0."""
        assert rows.dtype == torch.uint64 and rows.is_cuda
        assert rows.dim() == 2 and rows.size(1) == self.n_cols
        if self._partial is not None:
            rows = torch.cat([self._partial, rows])
            self._partial = None
        k = int(rows.size(0))
        if k == 0:
            return
        assert self._rows_seen + k <= self.n_total_rows, "more rows than n_total_rows"
        if self._rows_seen + k == self.n_total_rows:
            self._emit(rows)                       # the last slab may end in a partial chunk
            return
        full = (k // _BLAKE3_CHUNK_ROWS) * _BLAKE3_CHUNK_ROWS
        if full:
            self._emit(rows[:full])
        if full < k:
            self._partial = rows[full:].clone()

    def finalize(self):
        """Returns (n_cols, 32) uint8 column digests."""
        assert self._chunks_seen == self.n_chunks_total, (
            f"expected {self.n_chunks_total} chunks, saw {self._chunks_seen}"
            f" (rows_seen={self._rows_seen}/{self.n_total_rows})")
        L = _lib.lib()
        out = torch.empty((self.n_cols, 32), dtype=torch.uint8, device=self._states.device)
        _lib.check(L.vi_hash_columns_finalize(self.n_cols, self.n_chunks_total, self._states.data_ptr(),
                                              self._states.numel(), out.data_ptr(), _lib.stream_ptr()))
        return out


# ---- ZK pad generator (prover/cuda_primitives.py:1262-1294) ----

def _check_seed(master_seed):
    assert isinstance(master_seed, torch.Tensor)
    if master_seed.dtype != torch.uint8:
        raise RuntimeError("master_seed must be uint8")
    if master_seed.numel() != 32:
        raise RuntimeError("master_seed must be 32 bytes")
    if not master_seed.is_cuda:
        raise RuntimeError("master_seed must be on CUDA")
    if not master_seed.is_contiguous():
        raise RuntimeError("master_seed must be contiguous")


def _row_prg(master_seed, row_indices, row_offset, n_rows, slack, out):
    if n_rows and slack:
        _lib.check(_lib.lib().vi_row_prg(master_seed.data_ptr(), row_indices.data_ptr() if row_indices is not None else None,
                                         int(row_offset), n_rows, slack, out.data_ptr(),
                                         int(out.stride(0)) if n_rows > 1 else max(slack, int(out.stride(0))),
                                         _lib.stream_ptr()))
    return out


def row_prg(master_seed, row_offset, n_rows, slack_per_row, out=None):
    """(n_rows, slack_per_row) uint64 with
    out[r, k] = BLAKE3(master_seed || (row_offset + r)_le8 || k_le8)[0:8] mod P
    (prover/cuda_primitives.py:1262-1286).  `out` may be a column slice of a wider
    matrix (unit column stride), e.g. `padded[:, ELL:]`, which is then filled in place."""
    _check_seed(master_seed)
    n_rows, slack = int(n_rows), int(slack_per_row)
    if n_rows < 0 or slack < 0:
        raise RuntimeError("n_rows and slack_per_row must be >= 0")
    if out is None:
        out = torch.empty((n_rows, slack), dtype=torch.uint64, device=master_seed.device)
    else:
        if out.dtype != torch.uint64 or not out.is_cuda or tuple(out.shape) != (n_rows, slack):
            raise RuntimeError("out must be a (n_rows, slack_per_row) CUDA uint64 tensor")
        if n_rows and slack and (out.stride(1) != 1 or (n_rows > 1 and out.stride(0) < slack)):
            raise RuntimeError("out must have unit column stride and non-overlapping rows")
    return _row_prg(master_seed, None, row_offset, n_rows, slack, out)


def row_prg_indexed(master_seed, row_indices, slack_per_row):
    """row_prg for a list of absolute row indices (cuda uint64 tensor), one launch
    (prover/cuda_primitives.py:1289-1294)."""
    _check_seed(master_seed)
    if (not isinstance(row_indices, torch.Tensor) or row_indices.dtype != torch.uint64 or not row_indices.is_cuda
            or not row_indices.is_contiguous()):
        raise RuntimeError("row_indices must be a contiguous CUDA uint64 tensor")
    n_rows, slack = int(row_indices.numel()), int(slack_per_row)
    out = torch.empty((n_rows, slack), dtype=torch.uint64, device=master_seed.device)
    return _row_prg(master_seed, row_indices, 0, n_rows, slack, out)


def merkle_one_level(nodes):
    """(k, 32) uint8 (or (k, 8) uint32) nodes -> (ceil(k / 2), 32) uint8 parents;
    an odd last node is paired with itself (layergkr/rs.py:135-144)."""
    if not nodes.is_cuda or not nodes.is_contiguous():
        raise RuntimeError("nodes must be CUDA and contiguous")
    k = int(nodes.size(0))
    if k < 1 or nodes.numel() * nodes.element_size() != 32 * k:
        raise RuntimeError("nodes must be (k, 32) uint8")
    out = torch.empty(((k + 1) // 2, 32), dtype=torch.uint8, device=nodes.device)
    _lib.check(_lib.lib().vi_merkle_level(nodes.data_ptr(), k, out.data_ptr(), _lib.stream_ptr()))
    return out


def merkle_build_blake3(leaves):
    """(N, 32) uint8 leaves -> (root: (32,) uint8, levels: list of (k_i, 32) uint8);
    levels[0] = leaves, levels[-1] = (1, 32) holding the root
    (prover/cuda_primitives.py:1388-1402).  All levels above the leaves are built by one library
    call (up to nine levels per launch) into one buffer; the list holds views of it."""
    assert leaves.dim() == 2 and leaves.size(1) == 32
    assert leaves.dtype == torch.uint8 and leaves.is_cuda
    cur = leaves.contiguous()
    levels = [leaves]
    k = int(cur.size(0))
    if k > 1:
        L = _lib.lib()
        buf = torch.empty((int(L.vi_merkle_tree_nodes(k)), 32), dtype=torch.uint8, device=cur.device)
        with torch.cuda.device(cur.device):
            _lib.check(L.vi_merkle_tree(cur.data_ptr(), k, buf.data_ptr(), _lib.stream_ptr()))
        off = 0
        while k > 1:
            k = (k + 1) // 2
            levels.append(buf[off:off + k])
            off += k
    root = levels[-1].view(-1)[:32].clone()
    return root, levels


# ---- combiner challenges, CSR matvec, LogUp multiplicities (prover/cuda_primitives.py:512-592, 1008-1052) ----

def _check_key(seed, label):
    if not (isinstance(seed, torch.Tensor) and seed.is_cuda and seed.dtype == torch.uint8 and seed.numel() == 32
            and seed.is_contiguous()):
        raise RuntimeError("seed must be a 32-byte CUDA uint8 tensor")
    if not (isinstance(label, torch.Tensor) and label.is_cuda and label.dtype == torch.uint8 and label.numel() <= 8
            and label.is_contiguous()):
        raise RuntimeError("label must be a CUDA uint8 tensor of <= 8 bytes")


def challenge_at(seed, label, cids):
    """challenge(seed, cid, label) for an arbitrary cid tensor (uint64, any shape):
    int.from_bytes(BLAKE3(seed || label || cid_le8)[:16], "little") % P
    (prover/cuda_primitives.py:1233-1237, prover/protocol.py:127-135)."""
    _check_key(seed, label)
    if not (isinstance(cids, torch.Tensor) and cids.is_cuda and cids.dtype == torch.uint64):
        raise RuntimeError("cids must be a CUDA uint64 tensor")
    cc = cids.contiguous()
    n = int(cc.numel())
    if n >= (1 << 31):
        raise RuntimeError("challenge_at: too many cids")
    out = torch.empty_like(cc)
    if n:
        _lib.check(_lib.lib().vi_challenge(seed.data_ptr(), label.data_ptr(), int(label.numel()), cc.data_ptr(), n,
                                           out.data_ptr(), _lib.stream_ptr()))
    return out


def challenge_vec(seed, label, n):
    """r[i] = challenge(seed, i, label) for i in [0, n) on the device
    (prover/cuda_primitives.py:1240-1248)."""
    n = int(n)
    if n == 0:
        return torch.empty(0, dtype=torch.uint64, device="cuda")
    _check_key(seed, label)
    if n < 0 or n >= (1 << 31):
        raise RuntimeError("challenge_vec n must be in [0, 2^31)")
    out = torch.empty(n, dtype=torch.uint64, device=seed.device)
    _lib.check(_lib.lib().vi_challenge(seed.data_ptr(), label.data_ptr(), int(label.numel()), None, n, out.data_ptr(),
                                       _lib.stream_ptr()))
    return out


def _spmv(values, col_idx, row_ptr, n_rows, x, seed, label):
    for t, name in ((values, "values"), (col_idx, "col_idx"), (row_ptr, "row_ptr")):
        _check_u64(t, name)
        if t.dim() != 1:
            raise RuntimeError(f"{name} must be 1-D")
    n_rows = int(n_rows)
    if int(row_ptr.size(0)) != n_rows + 1:
        raise RuntimeError("row_ptr length must be n_rows + 1")
    if int(values.numel()) != int(col_idx.numel()):
        raise RuntimeError("values and col_idx must have one entry per non-zero")
    y = torch.empty(n_rows, dtype=torch.uint64, device=values.device)
    if n_rows:
        _lib.check(_lib.lib().vi_gl_spmv(values.data_ptr(), col_idx.data_ptr(), row_ptr.data_ptr(), n_rows, int(values.numel()),
                                         x.data_ptr() if x is not None else None,
                                         seed.data_ptr() if seed is not None else None,
                                         label.data_ptr() if label is not None else None,
                                         int(label.numel()) if label is not None else 0, y.data_ptr(), _lib.stream_ptr()))
    return y


def gl_spmv(values, col_idx, row_ptr, x, n_rows):
    """CSR mod-P matvec; row_ptr length must be n_rows + 1 (prover/cuda_primitives.py:1192-1194)."""
    _check_u64(x, "x")
    if x.dim() != 1:
        raise RuntimeError("x must be 1-D")
    return _spmv(values, col_idx, row_ptr, n_rows, x, None, None)


def gl_spmv_challenged(values, col_idx, row_ptr, seed, label, n_rows):
    """CSR mod-P matvec whose combiner x[cid] = challenge(seed, cid, label) is computed in place
    (prover/cuda_primitives.py:1197-1202)."""
    _check_key(seed, label)
    return _spmv(values, col_idx, row_ptr, n_rows, None, seed, label)


_range_table_cache: dict = {}


def _is_range_table(table):
    """One probe per table tensor: is table[i] == i for all i?  Cached by storage address and
    length, as the reference does (tables are immutable once built, cuda_primitives.py:1411-1423)."""
    key = (table.data_ptr(), table.numel())
    if key not in _range_table_cache:
        ref = torch.arange(table.numel(), dtype=torch.int64, device=table.device).view(torch.uint64)
        _range_table_cache[key] = bool(torch.equal(table, ref))
    return _range_table_cache[key]


def lookup_multiplicities_into(x, table, mult, label=""):
    """In-place mult[j] += #{i : x[i] == table[j]}; values outside the table count nowhere
    (prover/cuda_primitives.py:1431-1446).  A table that is literally 0 .. T-1 is indexed directly."""
    _check_u64(x, "x")
    _check_u64(table, "table")
    _check_u64(mult, "mult")
    if x.dim() != 1 or table.dim() != 1 or mult.dim() != 1:
        raise RuntimeError("x, table and mult must be 1-D")
    if mult.numel() != table.numel():
        raise RuntimeError("mult length must match table")
    if x.numel() == 0 or table.numel() == 0:
        return
    _lib.check(_lib.lib().vi_lookup_multiplicities(x.data_ptr(), int(x.numel()), table.data_ptr(), int(table.numel()),
                                                   1 if _is_range_table(table) else 0, mult.data_ptr(), _lib.stream_ptr()))


def lookup_multiplicities(x, table):
    """Per-table-entry multiplicity histogram (prover/cuda_primitives.py:1426-1428)."""
    _check_u64(x, "x")
    _check_u64(table, "table")
    mult = torch.zeros(int(table.numel()), dtype=torch.int64, device=table.device).view(torch.uint64)
    if x.dim() != 1 or table.dim() != 1:
        raise RuntimeError("x and table must be 1-D")
    lookup_multiplicities_into(x, table, mult)
    return mult

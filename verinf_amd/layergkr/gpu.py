"""Drop-in for the hot-path functions of the reference's `layergkr/gpu.py` on MI355X.

Kept, with the reference's names and argument meaning:
  available()                                   gpu.py:75-76
  encode_batch_ntt(cfg, messages)               gpu.py:141-203   (Python rows or a device tensor)
  selftest_ntt / selftest_ntt_spot              gpu.py:206-253   (bit-exactness gates)
  gl_sum(t), fold_t(f, r_t)                     gpu.py:326-347
  prove_terms_gpu(terms, coin, field_p, mask, mu0)   gpu.py:350-410
  MAX_GRID_ROWS, _chunk_rows, _coset_powers     gpu.py:33-61, 128-138

  hash_and_tree(cfg, mat), levels_to_host       gpu.py:274-297
  linear_combination, combine_t, column         gpu.py:113-122, 301-315

What changes underneath: encode is ONE fused library call (no (rows, N) zero
buffer, no expanded gamma powers, no per-chunk copies), and a sumcheck round is
one fused launch instead of ~(deg+1)*(4*factors + log n) elementwise launches; the
only host wait per round is for the deg+1 samples that the verifier coin needs.

Added for device consumers: eq_vector_t, mle_eval_t (the reference's eq_vector /
mle_eval work on Python lists).  The dense Lagrange-matrix encoders
(`encode_batch[_t]`) of the reference module are not provided: the NTT encoder is
the one encoder here.
"""
import contextlib
import ctypes
import threading
from typing import Optional, Sequence

import torch

from .. import _lib
from ..prover import cuda_primitives as cp
from ..prover.protocol import GLOBAL_G, Config, P

# The reference caps a chunk at 65535 rows because its kernels use one grid row per
# message (gpu.py:33-35).  These kernels have no such cap; the constant survives so
# that callers and tests which lower it to force chunking still work.
MAX_GRID_ROWS = 65535

_COSET: dict = {}


def available() -> bool:
    return torch.cuda.is_available()


def _require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("verinf_amd: no GPU visible (there is no CPU fallback)")


def _chunk_rows(cfg: Config, rows: int) -> int:
    """Rows per library call.  Chunking is exact (rows are independent); the fused
    encoder needs only its fixed-size workspace, so the free-memory term of the
    reference (gpu.py:47-61) disappears and only the row cap remains."""
    return max(1, min(rows, MAX_GRID_ROWS))


def _coset_powers(cfg: Config):
    """gamma^i for i < K_DEG on the device (gpu.py:128-138)."""
    _require_gpu()
    key = (cfg.K_DEG, torch.cuda.current_device())
    if key not in _COSET:
        import numpy as np
        pw = np.empty(cfg.K_DEG, dtype=np.uint64)
        cur = 1
        for i in range(cfg.K_DEG):
            pw[i] = cur
            cur = cur * GLOBAL_G % P
        _COSET[key] = torch.from_numpy(pw).cuda()
    return _COSET[key]


def _to_device_rows(messages, width: int):
    """Python rows -> (rows, width) uint64 device tensor (short rows zero-padded)."""
    import numpy as np
    arr = np.zeros((len(messages), width), dtype=np.uint64)
    for i, m in enumerate(messages):
        if len(m):
            arr[i, : len(m)] = np.array([int(v) % P for v in m], dtype=np.uint64)
    return torch.from_numpy(arr).cuda()


def encode_batch_ntt(cfg: Config, messages):
    """Messages (values at the K-th roots of unity, at most K_DEG per row) ->
    (rows, N_LIG) codewords on the coset GLOBAL_G * <w_N>, as a device tensor."""
    _require_gpu()
    on_device = hasattr(messages, "shape")
    if on_device:
        msgs = messages
        if msgs.dtype != torch.uint64 or not msgs.is_cuda or msgs.dim() != 2:
            raise RuntimeError("encode_batch_ntt: messages must be a 2-D CUDA uint64 tensor")
    else:
        width = max([len(m) for m in messages], default=0)
        if width > cfg.K_DEG:
            raise ValueError(f"message {width} > K_DEG {cfg.K_DEG}")
        msgs = _to_device_rows(messages, max(width, 1))
    rows = int(msgs.shape[0])
    out = torch.empty((rows, cfg.N_LIG), dtype=torch.uint64, device=msgs.device)
    step = _chunk_rows(cfg, rows) if rows else 1
    for lo in range(0, rows, step):
        hi = min(lo + step, rows)
        cp.coset_lde(msgs[lo:hi], cfg.K_DEG, cfg.N_LIG, GLOBAL_G, out=out[lo:hi])
    return out


def selftest_ntt(cfg: Config, n_rows: int = 4, seed: int = 2) -> Optional[str]:
    """Whole-codeword bit-exactness against the Lagrange definition
    (prover.protocol.eval_zeta_form).  None on agreement, else the first mismatch."""
    if not available():
        return "no CUDA"
    import random
    from ..prover.protocol import eval_zeta_form
    r = random.Random(seed)
    msgs = [[r.randrange(P) for _ in range(cfg.ELL)] for _ in range(n_rows)]
    got = encode_batch_ntt(cfg, msgs).cpu().tolist()
    for i, m in enumerate(msgs):
        for j in range(cfg.N_LIG):
            ref = eval_zeta_form(cfg, m, cfg.eta(j))
            if ref != int(got[i][j]):
                return f"row {i} column {j}: dense {ref} != ntt {int(got[i][j])}"
    return None


def selftest_ntt_spot(cfg: Config, n_cols: int = 24, seed: int = 5) -> Optional[str]:
    """Sampled-column bit-exactness where whole codewords are too costly to
    evaluate from the definition (gpu.py:226-253)."""
    if not available():
        return "no CUDA"
    import random
    from ..prover.protocol import eval_zeta_form
    r = random.Random(seed)
    msg = [r.randrange(P) for _ in range(cfg.ELL)]
    got = encode_batch_ntt(cfg, [msg])[0].cpu().tolist()
    for _ in range(n_cols):
        j = r.randrange(cfg.N_LIG)
        ref = eval_zeta_form(cfg, msg, cfg.eta(j))
        if ref != int(got[j]):
            return f"column {j}: dense {ref} != ntt {int(got[j])}"
    return None


def _u64_row(values):
    import numpy as np
    return torch.from_numpy(np.array([[int(v) % P for v in values]], dtype=np.uint64)).cuda()


def linear_combination(cfg: Config, codewords, coeffs: Sequence[int]):
    """sum_i coeffs[i] * codewords[i] as a (1 x rows) @ (rows x N) product; Python rows in,
    Python list out (gpu.py:113-122)."""
    _require_gpu()
    import numpy as np
    if len(codewords) != len(coeffs):
        raise ValueError("coeffs/codewords length mismatch")
    B = torch.from_numpy(np.array([[int(v) % P for v in c] for c in codewords], dtype=np.uint64)).cuda()
    return [int(v) for v in cp.gl_matmul(_u64_row(coeffs), B)[0].cpu().tolist()]


def combine_t(cfg: Config, mat, coeffs: Sequence[int]):
    """sum_i coeffs[i] * mat[i] for a device matrix, staying on the device: (1, N) tensor
    (gpu.py:301-308)."""
    _require_gpu()
    return cp.gl_matmul(_u64_row(coeffs), mat)


def hash_and_tree(cfg: Config, mat):
    """Column digests and the Merkle tree of a device codeword matrix, both computed on the
    device (gpu.py:274-288): returns (root bytes, list of (k_i, 32) uint8 level tensors)."""
    _require_gpu()
    dig = cp.hash_columns_streamed(mat)
    root_t, levels_t = cp.merkle_build_blake3(dig)
    return bytes(root_t.cpu().tolist()), levels_t


def levels_to_host(levels_t):
    """The (small) tree as lists of 32-byte nodes, so that opening paths cost nothing
    (gpu.py:291-297)."""
    out = []
    for lvl in levels_t:
        raw = lvl.cpu().numpy().tobytes()
        out.append([raw[32 * r:32 * r + 32] for r in range(lvl.shape[0])])
    return out


def column(mat, col: int):
    """One codeword column back to the host."""
    return [int(v) for v in mat.view(torch.int64)[:, col].contiguous().view(torch.uint64).cpu().tolist()]


# ---- multilinear helpers ---------------------------------------------------------------
def _point(z):
    arr = (ctypes.c_uint64 * max(len(z), 1))(*[int(v) % P for v in z])
    return arr


def eq_vector_t(z: Sequence[int], msb_first: bool = False):
    """eq(z, .) over the hypercube as a device tensor of 2^len(z) field elements, built on
    the device.  Default order is that of the reference's eq_vector (layergkr/logup.py:61-69,
    z[0] on the least significant index bit), so the tensor can stand in for its list as a
    sumcheck factor; msb_first=True gives the variable order of mle_eval / fold_t."""
    _require_gpu()
    n = len(z)
    if n > 32:
        raise RuntimeError("eq_vector_t: at most 32 variables")
    out = torch.empty(1 << n, dtype=torch.uint64, device="cuda")
    _lib.check(_lib.lib().vi_eq_vector(_point(z), n, 1 if msb_first else 0, out.data_ptr(), _lib.stream_ptr()))
    return out


def mle_eval_t(tables, point: Sequence[int]):
    """Multilinear extension of a device table (or of every row of a (k, 2^n) matrix) at
    `point`, point[0] on the most significant index bit as in layergkr/sumcheck.py:40-48.
    One streaming pass per table; returns an int (1-D input) or a list of ints."""
    _require_gpu()
    cp._check_u64(tables, "tables")
    n = len(point)
    one = tables.dim() == 1
    mat = tables.view(1, -1) if one else tables
    if mat.dim() != 2 or int(mat.shape[1]) != (1 << n):
        raise RuntimeError(f"mle_eval_t: tables of length {tuple(tables.shape)} do not match {n} variables")
    k = int(mat.shape[0])
    out = torch.empty(max(k, 1), dtype=torch.uint64, device=tables.device)
    L = _lib.lib()
    ws = _lib.workspace(L.vi_mle_eval_workspace_bytes(k), tables.device, "mle")
    _lib.check(L.vi_mle_eval(mat.data_ptr(), k, 1 << n, _point(point), n, out.data_ptr(), ws.data_ptr(), ws.numel(),
                             _lib.stream_ptr()))
    vals = [int(v) for v in out[:k].cpu().tolist()]
    return vals[0] if one else vals


# ---- sumcheck ------------------------------------------------------------------------
def gl_sum(t):
    """Field sum of a uint64 device tensor -> 1-element device tensor."""
    _require_gpu()
    v = t.reshape(-1)
    if v.dtype != torch.uint64 or not v.is_cuda:
        raise RuntimeError("gl_sum: expected a CUDA uint64 tensor")
    v = v.contiguous()
    out = torch.empty(1, dtype=torch.uint64, device=v.device)
    L = _lib.lib()
    with torch.cuda.device(v.device):
        ws = _lib.workspace(L.vi_gl_sum_workspace_bytes(v.numel()), v.device, "sum")
        _lib.check(L.vi_gl_sum(v.data_ptr(), v.numel(), out.data_ptr(), ws.data_ptr(), ws.numel(),
                               _lib.stream_ptr()))
    return out


class _Problem:
    """Host-side descriptor of a sum-of-products problem in the C ABI's shape."""

    def __init__(self, tables, terms):
        self.n_tables = len(tables)
        off, idx = [0], []
        for _, fs in terms:
            idx.extend(fs)
            off.append(len(idx))
        self.n_terms = len(terms)
        self.deg = max(len(fs) for _, fs in terms)
        self.term_off = (ctypes.c_int * len(off))(*off)
        self.factor_idx = (ctypes.c_int * max(len(idx), 1))(*idx)
        self.coeffs = (ctypes.c_uint64 * len(terms))(*[c % P for c, _ in terms])

    @staticmethod
    def ptrs(tensors):
        return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _fold_tables(src, dst, half: int, r: int):
    L = _lib.lib()
    with torch.cuda.device(src[0].device):
        _lib.check(L.vi_sumcheck_fold_eval(_Problem.ptrs(src), _Problem.ptrs(dst), len(src), half, r % P,
                                           None, None, None, 0, None, None, None, 0, _lib.stream_ptr()))


def fold_t(f, r_t):
    """(f[:h] + r*(f[h:] - f[:h])) mod P as a new device tensor; r_t is a 1-element
    device tensor or an int."""
    _require_gpu()
    if f.dtype != torch.uint64 or not f.is_cuda:
        raise RuntimeError("fold_t: expected a CUDA uint64 tensor")
    f = f.reshape(-1).contiguous()
    h = f.numel() // 2
    r = int(r_t.item()) if hasattr(r_t, "item") else int(r_t)
    out = torch.empty(h, dtype=torch.uint64, device=f.device)
    if h:
        _fold_tables([f], [out], h, r)
    return out


def _as_table(v, field_p):
    if hasattr(v, "shape"):
        if v.dtype != torch.uint64 or not v.is_cuda:
            raise RuntimeError("prove_terms_gpu: tensor factors must be CUDA uint64")
        return v if v.dim() == 1 and v.is_contiguous() else v.reshape(-1).contiguous()
    import numpy as np
    return torch.from_numpy(np.array([int(x) % field_p for x in v], dtype=np.uint64)).cuda()


def _sumcheck_problem(terms, field_p, who):
    """Distinct factor objects as device tables + the terms over their indices."""
    if field_p != P:
        raise ValueError(f"{who}: only the Goldilocks field is supported")
    if not terms:
        raise ValueError("no terms")
    uniq, tables, tterms = {}, [], []
    for c, fs in terms:
        ids = []
        for f in fs:
            k = id(f)
            if k not in uniq:
                uniq[k] = len(tables)
                tables.append(_as_table(f, field_p))
            ids.append(uniq[k])
        tterms.append((int(c) % field_p, ids))
    size = int(tables[0].numel())
    if any(int(t.numel()) != size for t in tables):
        raise ValueError(f"{who}: factors of different lengths")
    if size < 1 or size & (size - 1):
        raise ValueError(f"{who}: table length must be a power of two")
    return tables, tterms, size


def _single_point(tables, tterms, mu0, field_p):
    """No variables: the claim is the term sum at the one point there is."""
    total = 0
    vals = [int(t.cpu()[0].item()) for t in tables]
    for c, ids in tterms:
        prod = c
        for i in ids:
            prod = prod * vals[i] % field_p
        total += prod
    mu = mu0 % field_p
    return (total + mu) % field_p, [], [], mu


def prove_terms_gpu(terms, coin, field_p: int, mask=None, mu0: int = 0):
    """Sumcheck prover for sum_x sum_k c_k prod_j f_kj(x) with the tables on the device.

    terms  [(coefficient, [factor, ...]), ...]; a factor is a Python sequence or a
           CUDA uint64 tensor (tensors are used where they are, never copied to the
           host); a factor object that appears several times is held once.
    coin   host callback round -> challenge (reduced mod p here).
    mask   optional callback (deg, mu) -> ascending coefficients of the scalar mask
           polynomial added to the samples (gpu.py:397-406).
    Returns (claim, round_polys, challenges, mu) exactly as gpu.py:350-410.
    The caller's tensors are never modified.

    `coin` is asked by round number only and `mask` by (deg, mu) (gpu.py:398, 403): neither
    sees a round's samples, so both are called for every round BEFORE the first launch -- in
    the reference's order mask(deg, mu_k), coin(k), mu_(k+1) = h_k(r_k), so that callbacks
    sharing state (one random.Random, a tape) draw exactly what they draw there -- and the
    whole proof is queued on the stream without a host round trip
    (vi_sumcheck_prove_coins).  prove_terms_gpu_interactive is the variant for a coin that
    does need the samples."""
    _require_gpu()
    tables, tterms, size = _sumcheck_problem(terms, field_p, "prove_terms_gpu")
    n_rounds = size.bit_length() - 1
    if n_rounds == 0:
        return _single_point(tables, tterms, mu0, field_p)
    prob = _Problem(tables, tterms)
    deg = prob.deg
    mu = mu0 % field_p
    challenges, masks = [], []
    for rnd in range(n_rounds):
        h = mask(deg, mu) if mask is not None else None
        r = coin(rnd) % field_p
        challenges.append(r)
        masks.append(h)
        if h is not None:
            mu = _poly_eval(h, r, field_p)
    L = _lib.lib()
    dev = tables[0].device
    with _on_device(dev):
        stream = torch.cuda.current_stream()
        sp = stream.cuda_stream
        ws = _lib.workspace(L.vi_sumcheck_prove_coins_workspace_bytes(size), dev, "sumcheck_coins", sp)
        # the folded tables live in one cached scratch buffer, a half-length slice per table (the caller's
        # tensors are never written)
        half_bytes = (size // 2) * 8
        work = _lib.workspace(max(prob.n_tables * half_bytes, 256), dev, "sumcheck_work", sp)
        work_p = (ctypes.c_void_p * prob.n_tables)(*[work.data_ptr() + t * half_bytes for t in range(prob.n_tables)])
        samples_host, samples_np = _pinned_samples(8 * n_rounds, sp)
        chal = (ctypes.c_uint64 * n_rounds)(*challenges)
        _lib.check(L.vi_sumcheck_prove_coins(_Problem.ptrs(tables), work_p, prob.n_tables, size,
                                             prob.term_off, prob.factor_idx, prob.coeffs, prob.n_terms, chal,
                                             samples_host.data_ptr(), ws.data_ptr(), ws.numel(), sp))
        stream.synchronize()
        rows = samples_np[:8 * n_rounds].reshape(n_rounds, 8)[:, :deg + 1].tolist()
    if mask is None:
        round_polys = [list(enumerate(ys)) for ys in rows]
    else:
        round_polys = [[(x, (y + _poly_eval(h, x, field_p)) % field_p) for x, y in enumerate(ys)]
                       for ys, h in zip(rows, masks)]
    # S(0) + S(1) of the first round is the sum over the cube
    claim = (rows[0][0] + rows[0][1] + mu0) % field_p
    return claim, round_polys, challenges, mu


def prove_terms_gpu_interactive(terms, coin, field_p: int, mask=None, mu0: int = 0):
    """prove_terms_gpu for a verifier coin that needs the samples: coin(round, samples) with
    samples = [(x, S(x))] of that round (mask applied) -> challenge.  One launch and one host
    wait per round (vi_sumcheck_prove); same return value."""
    _require_gpu()
    tables, tterms, size = _sumcheck_problem(terms, field_p, "prove_terms_gpu_interactive")
    n_rounds = size.bit_length() - 1
    if n_rounds == 0:
        return _single_point(tables, tterms, mu0, field_p)
    prob = _Problem(tables, tterms)
    deg = prob.deg
    L = _lib.lib()
    dev = tables[0].device
    mu = mu0 % field_p

    with torch.cuda.device(dev):
        ws = _lib.workspace(L.vi_sumcheck_workspace_bytes(), dev, "sumcheck")
        # The round loop runs inside the library: per round one fused launch, a wait on a word of pinned host
        # memory that the kernel stores behind its samples, and this callback -- the only Python left in the
        # loop -- which applies the optional scalar mask and asks the verifier coin for the challenge.
        samples_host, _ = _pinned_samples(16, torch.cuda.current_stream().cuda_stream)
        work = _work_tables(tables, size, dev)
        round_polys, challenges = [], []
        state = {"mu": mu, "error": None}

        def on_round(rnd, samples_p, n, r_out, _user):
            try:
                samples = [(x, samples_p[x]) for x in range(n)]
                if mask is not None:
                    h = mask(deg, state["mu"])
                    samples = [(x, (y + _poly_eval(h, x, field_p)) % field_p) for x, y in samples]
                round_polys.append(samples)
                r = coin(rnd, samples) % field_p
                challenges.append(r)
                if mask is not None:
                    state["mu"] = _poly_eval(h, r, field_p)
                r_out[0] = r
                return 0
            except BaseException as exc:            # never unwind through the C frames
                state["error"] = exc
                return 1

        cb = _lib.COIN_FN(on_round)
        out_samples = (ctypes.c_uint64 * (n_rounds * (deg + 1)))()
        out_chals = (ctypes.c_uint64 * n_rounds)()
        rc = L.vi_sumcheck_prove(_Problem.ptrs(tables), _Problem.ptrs(work), prob.n_tables, size, prob.term_off,
                                 prob.factor_idx, prob.coeffs, prob.n_terms, cb, None, samples_host.data_ptr(),
                                 samples_host.numel(), out_samples, out_chals, ws.data_ptr(), ws.numel(),
                                 torch.cuda.current_stream().cuda_stream)
        if state["error"] is not None:
            raise state["error"]
        _lib.check(rc)
        # S(0) + S(1) of the first round is the sum over the cube
        claim = (int(out_samples[0]) + int(out_samples[1]) + mu0) % field_p
        mu = state["mu"]
    return claim, round_polys, challenges, mu


def _work_tables(tables, size, dev):
    """Half-length buffers the folded tables live in (the caller's tensors are never written)."""
    if size < 4:
        return tables                        # one round: nothing is folded
    return [torch.empty(size // 2, dtype=torch.uint64, device=dev) for _ in tables]


_PINNED = threading.local()
_NO_GUARD = contextlib.nullcontext()


def _on_device(dev):
    """Context that makes `dev` current; nothing to do (and nothing paid) when it already is."""
    return _NO_GUARD if dev.index is None or dev.index == torch.cuda.current_device() else torch.cuda.device(dev)


def _pinned_samples(words: int, stream_ptr: int):
    """Pinned host words the sumcheck kernels write their samples into (and, for the interactive loop, the tag of
    the round that has arrived), with a numpy view of the same memory.  One buffer per host thread and stream: a
    proof is read back before the next one on that stream starts, and two threads (or two streams) never see each
    other's samples."""
    bufs = getattr(_PINNED, "bufs", None)
    if bufs is None:
        bufs = _PINNED.bufs = {}
    key = (torch.cuda.current_device(), stream_ptr)
    buf = bufs.get(key)
    if buf is None or buf[0].numel() < words:
        t = torch.zeros(max(words, 512), dtype=torch.uint64).pin_memory()
        buf = bufs[key] = (t, t.numpy())
    return buf


def _poly_eval(coeffs: Sequence[int], x: int, p: int) -> int:
    acc = 0
    for c in reversed(coeffs):
        acc = (acc * x + c) % p
    return acc


# ---- dense Lagrange encoder (layergkr/gpu.py:80-122, 256-271) ------------------------------------------
_LAGRANGE_GPU = {}


def lagrange_gpu(cfg: Config):
    """The ELL x N_LIG matrix L[c][j] = L_c(eta_j) = zeta_c (eta_j^K - 1) / (K (eta_j - zeta_c)) as a device tensor,
    cached per geometry.  The two domains go up as vectors; the ELL * N_LIG differences are inverted on the device
    with one batched inversion, so no entry is computed on the host."""
    _require_gpu()
    if cfg.ELL * cfg.N_LIG > (1 << 27):
        raise RuntimeError(f"lagrange_gpu: the dense {cfg.ELL} x {cfg.N_LIG} matrix would take "
                           f"{cfg.ELL * cfg.N_LIG * 8 / 2**30:.0f} GiB; use encode_batch_ntt at this geometry")
    key = (cfg.ELL, cfg.K_DEG, cfg.N_LIG, torch.cuda.current_device())
    if key not in _LAGRANGE_GPU:
        k_inv = pow(cfg.K_DEG, P - 2, P)
        eta, zeta, num = [], [], []
        e, w_n = GLOBAL_G % P, cfg.W_N
        for _ in range(cfg.N_LIG):
            eta.append(e)
            num.append((pow(e, cfg.K_DEG, P) - 1) * k_inv % P)        # (eta^K - 1) / K
            e = e * w_n % P
        z, w_k = 1, cfg.W_K
        for _ in range(cfg.ELL):
            zeta.append(z)
            z = z * w_k % P
        eta_t, num_t, zeta_t = _u64_row(eta), _u64_row(num), _u64_row(zeta)
        zeta_cols = zeta_t.view(torch.int64).view(-1, 1).expand(cfg.ELL, cfg.N_LIG).contiguous().view(torch.uint64)
        eta_rows = eta_t.view(torch.int64).view(1, -1).expand(cfg.ELL, cfg.N_LIG).contiguous().view(torch.uint64)
        inv = cp.gl_inv_batched(cp.gl_sub(eta_rows, zeta_cols).view(-1)).view(cfg.ELL, cfg.N_LIG)
        _LAGRANGE_GPU[key] = cp.gl_mul(cp.gl_mul_bcast(inv, num_t.view(-1)), zeta_cols)
    return _LAGRANGE_GPU[key]


def encode_batch_t(cfg: Config, messages):
    """(rows x ELL) @ (ELL x N_LIG) over the field, result left on the device (gpu.py:256-271): the dense form of
    the encoder, O(ELL * N_LIG) per row -- for small geometries and as a cross-check of encode_batch_ntt."""
    _require_gpu()
    return cp.gl_matmul(_to_device_rows(messages, cfg.ELL), lagrange_gpu(cfg))


def encode_batch(cfg: Config, messages):
    """The same as Python lists (gpu.py:92-111)."""
    return [[int(v) for v in row] for row in encode_batch_t(cfg, messages).cpu().tolist()]


def selftest(cfg: Config, n_rows: int = 4, seed: int = 1) -> Optional[str]:
    """Gate of the dense encoder and of the linear combination against the definition on the host
    (prover.protocol.eval_zeta_form, Python integers), as gpu.py:413-434.  None on agreement."""
    if not available():
        return "no CUDA"
    import random
    from ..prover.protocol import eval_zeta_form
    r = random.Random(seed)
    msgs = [[r.randrange(P) for _ in range(cfg.ELL)] for _ in range(n_rows)]
    got = encode_batch(cfg, msgs)
    want = [[eval_zeta_form(cfg, m, cfg.eta(j)) for j in range(cfg.N_LIG)] for m in msgs]
    for i in range(n_rows):
        if want[i] != got[i]:
            j = next(k for k in range(cfg.N_LIG) if want[i][k] != got[i][k])
            return f"row {i} column {j}: definition {want[i][j]} != dense {got[i][j]}"
    co = [r.randrange(P) for _ in range(n_rows)]
    from . import rs
    if rs.linear_combination(cfg, want, co) != [int(v) for v in linear_combination(cfg, want, co)]:
        return "linear_combination disagrees"
    return None

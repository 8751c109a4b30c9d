"""ctypes front end of the C oracle (oracle/vi_oracle.c) plus a pure-Python-int
restatement of the same definitions.

TEST INFRASTRUCTURE ONLY.  Two independent statements of every algorithm live here
so that each can pin the other:

  * `C.*`  -- the compiled scalar C restatement (fast enough for 2^16..2^26 sizes)
  * `py_*` -- arbitrary-precision Python, written straight from the mathematical
              definition (a*b % p, the DFT sum, the Lagrange closed form, the
              sumcheck sum), usable only at toy sizes.

Reference lines each function follows are cited in vi_oracle.c; the `py_*`
functions cite theirs below.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_double, c_int, c_size_t, c_uint64, c_uint8, c_void_p

import numpy as np

P = (1 << 64) - (1 << 32) + 1          # prover/protocol.py:27
G = 7                                   # prover/protocol.py:28

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvi_oracle.so")


def build(force: bool = False) -> str:
    """Compile the C oracle in place (gcc, a second or two)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libvi_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        u64p, u8p, ip = POINTER(c_uint64), POINTER(c_uint8), POINTER(c_int)
        for name in ("vo_add", "vo_sub", "vo_mul", "vo_pow"):
            getattr(L, name).restype = c_uint64
            getattr(L, name).argtypes = [c_uint64, c_uint64]
        L.vo_inv.restype = c_uint64
        L.vo_inv.argtypes = [c_uint64]
        L.vo_root_of_unity.restype = c_uint64
        L.vo_root_of_unity.argtypes = [c_uint64]
        L.vo_binop_vec.argtypes = [c_int, u64p, u64p, u64p, c_size_t]
        L.vo_ntt.argtypes = [u64p, c_size_t, c_int]
        L.vo_ntt_rows.argtypes = [u64p, c_size_t, c_size_t, c_int]
        L.vo_dft_naive.argtypes = [u64p, u64p, c_size_t, c_int]
        L.vo_coset_lde_rows.argtypes = [u64p, c_size_t, c_size_t, c_size_t, c_size_t,
                                        c_size_t, c_uint64, u64p]
        L.vo_lagrange.restype = c_uint64
        L.vo_lagrange.argtypes = [c_uint64, c_uint64, c_uint64]
        L.vo_lde_dense_row.argtypes = [u64p, c_size_t, c_size_t, c_size_t, c_uint64, u64p]
        L.vo_fold.argtypes = [u64p, c_size_t, c_uint64, u64p]
        L.vo_sumcheck_prove.restype = c_int
        L.vo_sumcheck_prove.argtypes = [POINTER(c_void_p), c_int, c_size_t, ip, ip, u64p,
                                        c_int, u64p, u64p, u64p, u64p]
        L.vo_kquant_to_field.restype = c_int
        L.vo_kquant_to_field.argtypes = [c_int, u8p, c_size_t, c_double, u64p]
        L.vo_num_threads.restype = c_int
        L.vo_blake3.argtypes = [u8p, c_size_t, u8p]
        L.vo_hash_columns.argtypes = [u64p, c_size_t, c_size_t, u8p]
        L.vo_merkle_level.restype = c_size_t
        L.vo_merkle_level.argtypes = [u8p, c_size_t, u8p]
        L.vo_row_prg.argtypes = [u8p, u64p, c_uint64, c_size_t, c_size_t, u64p]
        L.vo_eq_vector.argtypes = [u64p, c_int, u64p]
        L.vo_challenge_vec.argtypes = [u8p, u8p, c_int, u64p, c_size_t, u64p]
        L.vo_spmv.argtypes = [u64p, u64p, u64p, c_size_t, u64p, u8p, u8p, c_int, u64p]
        L.vo_lookup_multiplicities.argtypes = [u64p, c_size_t, u64p, c_size_t, u64p]
        _lib = L
    return _lib


def _p64(a: np.ndarray):
    assert a.dtype == np.uint64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(POINTER(c_uint64))


def num_threads() -> int:
    return int(lib().vo_num_threads())


# ---------------------------------------------------------------- C oracle ----
def binop(op: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint64)
    b = np.ascontiguousarray(b, dtype=np.uint64)
    out = np.empty_like(a)
    lib().vo_binop_vec({"add": 0, "sub": 1, "mul": 2}[op], _p64(a), _p64(b), _p64(out), a.size)
    return out


def ntt(a: np.ndarray, inverse: bool = False) -> np.ndarray:
    out = np.array(a, dtype=np.uint64, copy=True)
    lib().vo_ntt(_p64(out), out.size, int(inverse))
    return out


def ntt_rows(rows: np.ndarray, inverse: bool = False) -> np.ndarray:
    out = np.array(rows, dtype=np.uint64, copy=True, order="C")
    m, n = out.shape
    lib().vo_ntt_rows(_p64(out), m, n, int(inverse))
    return out


def dft_naive(a: np.ndarray, inverse: bool = False) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint64)
    out = np.empty_like(a)
    lib().vo_dft_naive(_p64(a), _p64(out), a.size, int(inverse))
    return out


def coset_lde_rows(msgs: np.ndarray, K: int, N: int, shift: int = G) -> np.ndarray:
    msgs = np.ascontiguousarray(msgs, dtype=np.uint64)
    m, w = msgs.shape
    out = np.empty((m, N), dtype=np.uint64)
    lib().vo_coset_lde_rows(_p64(msgs), m, w, w, K, N, shift, _p64(out))
    return out


def lde_dense_row(msg: np.ndarray, K: int, N: int, shift: int = G) -> np.ndarray:
    msg = np.ascontiguousarray(msg, dtype=np.uint64)
    out = np.empty(N, dtype=np.uint64)
    lib().vo_lde_dense_row(_p64(msg), msg.size, K, N, shift, _p64(out))
    return out


def fold(f: np.ndarray, r: int) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.uint64)
    out = np.empty(f.size // 2, dtype=np.uint64)
    lib().vo_fold(_p64(f), f.size, r % P, _p64(out))
    return out


def sumcheck_prove(tables, terms, coins):
    """tables: list of uint64 arrays of equal power-of-two length.
    terms: list of (coeff, [table indices]).  coins: list of ints (one per round).
    Returns (claim, samples[v][deg+1], finals[n_tables])."""
    tabs = [np.ascontiguousarray(t, dtype=np.uint64) for t in tables]
    size = tabs[0].size
    v = size.bit_length() - 1
    ptrs = (c_void_p * len(tabs))(*[t.ctypes.data for t in tabs])
    off, idx = [0], []
    for _, fs in terms:
        idx.extend(fs)
        off.append(len(idx))
    deg = max(len(fs) for _, fs in terms)
    off_a = (c_int * len(off))(*off)
    idx_a = (c_int * max(len(idx), 1))(*idx)
    co = np.array([c % P for c, _ in terms], dtype=np.uint64)
    cn = np.array([c % P for c in coins[:v]] + [0] * max(0, 1 - v), dtype=np.uint64)
    claim = c_uint64(0)
    samples = np.zeros(max(v, 1) * (deg + 1), dtype=np.uint64)
    finals = np.zeros(len(tabs), dtype=np.uint64)
    lib().vo_sumcheck_prove(ptrs, len(tabs), size, off_a, idx_a, _p64(co), len(terms),
                            _p64(cn), ctypes.byref(claim), _p64(samples), _p64(finals))
    return (int(claim.value),
            [[int(x) for x in samples[r * (deg + 1):(r + 1) * (deg + 1)]] for r in range(v)],
            [int(x) for x in finals])


QTYPE_ID = {"Q4_K": 4, "Q5_K": 5, "Q6_K": 6}
BLOCK_BYTES = {"Q4_K": 144, "Q5_K": 176, "Q6_K": 210}


def kquant_to_field(raw: np.ndarray, qtype: str, S: float) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    nb = raw.size // BLOCK_BYTES[qtype]
    assert nb * BLOCK_BYTES[qtype] == raw.size
    out = np.empty(nb * 256, dtype=np.uint64)
    rc = lib().vo_kquant_to_field(QTYPE_ID[qtype], raw.ctypes.data_as(POINTER(c_uint8)), nb,
                                  float(S), _p64(out))
    assert rc == 0
    return out


def _p8(a: np.ndarray):
    return a.ctypes.data_as(POINTER(c_uint8))


def blake3(data: bytes) -> bytes:
    """32-byte BLAKE3 digest (default hash mode)."""
    buf = np.frombuffer(bytes(data) + b"\x00", dtype=np.uint8).copy()
    out = np.empty(32, dtype=np.uint8)
    lib().vo_blake3(_p8(buf), len(data), _p8(out))
    return out.tobytes()


def hash_columns(mat: np.ndarray) -> np.ndarray:
    """(m, n) uint64 -> (n, 32) uint8: BLAKE3 of each column's little-endian words."""
    mat = np.ascontiguousarray(mat, dtype=np.uint64)
    m, n = mat.shape
    out = np.empty((n, 32), dtype=np.uint8)
    if n:
        lib().vo_hash_columns(_p64(mat if m else np.zeros(1, dtype=np.uint64)), m, n, _p8(out))
    return out


def merkle_level(nodes: np.ndarray) -> np.ndarray:
    """(k, 32) uint8 -> (ceil(k/2), 32): parent = BLAKE3(left || right), odd last node doubled."""
    nodes = np.ascontiguousarray(nodes, dtype=np.uint8).reshape(-1, 32)
    k = nodes.shape[0]
    out = np.empty(((k + 1) // 2, 32), dtype=np.uint8)
    got = lib().vo_merkle_level(_p8(nodes), k, _p8(out))
    assert got == out.shape[0]
    return out


def row_prg(seed: bytes, row_offset: int, n_rows: int, slack: int, row_indices=None) -> np.ndarray:
    """(n_rows, slack) pad words: le64(BLAKE3(seed || row_le8 || k_le8)[:8]) mod p."""
    assert len(seed) == 32
    sd = np.frombuffer(bytes(seed), dtype=np.uint8).copy()
    idx = None
    if row_indices is not None:
        idx = np.ascontiguousarray(row_indices, dtype=np.uint64)
        n_rows = idx.size
    out = np.empty((n_rows, slack), dtype=np.uint64)
    if n_rows and slack:
        lib().vo_row_prg(_p8(sd), _p64(idx) if idx is not None else None, int(row_offset) & ((1 << 64) - 1), n_rows, slack, _p64(out))
    return out


def eq_vector(z) -> np.ndarray:
    """layergkr/logup.py:61-69: 2^n words, z[0] on the least significant index bit."""
    zz = np.array([int(v) % P for v in z], dtype=np.uint64)
    out = np.empty(1 << len(zz), dtype=np.uint64)
    lib().vo_eq_vector(_p64(zz) if len(zz) else None, len(zz), _p64(out))
    return out


def mle_eval(values: np.ndarray, point) -> int:
    """layergkr/sumcheck.py:40-48 by repeated vo_fold, point[0] on the most significant bit."""
    cur = np.ascontiguousarray(values, dtype=np.uint64) % np.uint64(P)
    for r in point:
        cur = fold(cur, int(r) % P)
    return int(cur[0])


def _bytes8(b: bytes):
    return np.frombuffer(bytes(b) + b"\x00", dtype=np.uint8).copy()


def challenge_vec(seed: bytes, label: bytes, n: int = 0, cids=None) -> np.ndarray:
    """challenge(seed, cid, label) for cid = 0..n-1 or for the given cids (prover/protocol.py:127-135)."""
    assert len(seed) == 32 and len(label) <= 8
    idx = None if cids is None else np.ascontiguousarray(cids, dtype=np.uint64)
    n = n if idx is None else idx.size
    out = np.empty(n, dtype=np.uint64)
    if n:
        lib().vo_challenge_vec(_p8(_bytes8(seed)), _p8(_bytes8(label)), len(label), _p64(idx) if idx is not None else None, n, _p64(out))
    return out


def spmv(values, col_idx, row_ptr, x=None, seed: bytes = b"", label: bytes = b"") -> np.ndarray:
    """CSR matrix times x over the field; x = None uses the challenged combiner of (seed, label)."""
    values, col_idx, row_ptr = (np.ascontiguousarray(a, dtype=np.uint64) for a in (values, col_idx, row_ptr))
    n_rows = row_ptr.size - 1
    y = np.zeros(max(n_rows, 0), dtype=np.uint64)
    if n_rows > 0:
        xv = None if x is None else np.ascontiguousarray(x, dtype=np.uint64)
        pad = np.zeros(1, dtype=np.uint64)
        lib().vo_spmv(_p64(values if values.size else pad), _p64(col_idx if col_idx.size else pad), _p64(row_ptr), n_rows,
                      _p64(xv) if xv is not None else None, _p8(_bytes8(seed.ljust(32, b"\0"))), _p8(_bytes8(label)), len(label), _p64(y))
    return y


def lookup_multiplicities(x, table) -> np.ndarray:
    x, table = np.ascontiguousarray(x, dtype=np.uint64), np.ascontiguousarray(table, dtype=np.uint64)
    mult = np.zeros(table.size, dtype=np.uint64)
    if x.size and table.size:
        lib().vo_lookup_multiplicities(_p64(x), x.size, _p64(table), table.size, _p64(mult))
    return mult


def merkle_levels(leaves: np.ndarray):
    """All levels from the leaves up to the (1, 32) root."""
    levels = [np.ascontiguousarray(leaves, dtype=np.uint8).reshape(-1, 32)]
    while levels[-1].shape[0] > 1:
        levels.append(merkle_level(levels[-1]))
    return levels


# ------------------------------------------------- pure-Python definitions ----
def py_root(n: int) -> int:
    """prover/ref/goldilocks_ref.py:45-49"""
    assert (P - 1) % n == 0
    return pow(G, (P - 1) // n, P)


def py_dft(a, inverse: bool = False):
    """X[k] = sum_j a[j] w^(jk)  (inverse: w^-1 and a 1/n factor)."""
    n = len(a)
    w = py_root(n)
    if inverse:
        w = pow(w, -1, P)
    out = []
    for k in range(n):
        wk = pow(w, k, P)
        acc, cur = 0, 1
        for x in a:
            acc += int(x) * cur
            cur = cur * wk % P
        out.append(acc % P)
    if inverse:
        ni = pow(n, -1, P)
        out = [x * ni % P for x in out]
    return out


def py_lagrange(K: int, c: int, eta: int) -> int:
    """prover/protocol.py:75-84"""
    zc = pow(py_root(K), c, P)
    return zc * (pow(eta, K, P) - 1) % P * pow(K * (eta - zc) % P, -1, P) % P


def py_lde_dense(msg, K: int, N: int, shift: int = G):
    """prover/protocol.py:86-93 with eta_j = shift * w_N^j (protocol.py:56-58)."""
    wn = py_root(N)
    out = []
    for j in range(N):
        eta = shift * pow(wn, j, P) % P
        acc = 0
        for c, v in enumerate(msg):
            if v:
                acc += int(v) * py_lagrange(K, c, eta)
        out.append(acc % P)
    return out


def py_sumcheck(tables, terms, coins):
    """Brute-force statement of layergkr/sumcheck.py:153-226 on Python ints.
    Same argument/return shapes as `sumcheck_prove`."""
    cur = [[int(x) % P for x in t] for t in tables]
    size = len(cur[0])
    deg = max(len(fs) for _, fs in terms)
    claim = 0
    for i in range(size):
        for c, fs in terms:
            prod = c % P
            for j in fs:
                prod = prod * cur[j][i] % P
            claim += prod
    claim %= P
    samples, rnd = [], 0
    while len(cur[0]) > 1:
        half = len(cur[0]) // 2
        row = []
        for x in range(deg + 1):
            acc = 0
            for c, fs in terms:
                for i in range(half):
                    prod = c % P
                    for j in fs:
                        f = cur[j]
                        prod = prod * ((f[i] + x * (f[half + i] - f[i])) % P) % P
                    acc += prod
            row.append(acc % P)
        samples.append(row)
        r = coins[rnd] % P
        cur = [[(f[i] + r * (f[half + i] - f[i])) % P for i in range(half)] for f in cur]
        rnd += 1
    return claim, samples, [f[0] for f in cur]


def py_mle_eval(values, point):
    """layergkr/sumcheck.py:40-48"""
    cur = [int(v) % P for v in values]
    for r in point:
        half = len(cur) // 2
        cur = [(cur[i] + r * (cur[half + i] - cur[i])) % P for i in range(half)]
    return cur[0] % P


def np_kquant_to_field(raw: np.ndarray, qtype: str, S: float) -> np.ndarray:
    """Vectorised numpy-float32 restatement of prover/kquant_cuda.py:42-111,
    independent of the C one (array ops instead of a per-weight loop)."""
    bb = BLOCK_BYTES[qtype]
    blk = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, bb)
    nb = blk.shape[0]
    e = np.arange(256)
    if qtype == "Q6_K":
        ql, qh = blk[:, 0:128], blk[:, 128:192]
        sc = blk[:, 192:208].view(np.int8)
        d = blk[:, 208:210].copy().view(np.float16).astype(np.float32)          # (nb,1)
        lo = (ql[:, (e >> 7) * 64 + (e & 63)] >> (4 * ((e >> 6) & 1))) & 0xF
        hi = (qh[:, (e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3
        q = (lo | (hi << 4)).astype(np.int8).astype(np.int32) - 32
        v = (d * sc[:, e >> 4].astype(np.float32)) * q.astype(np.float32)
    else:
        d = blk[:, 0:2].copy().view(np.float16).astype(np.float32)
        dmin = blk[:, 2:4].copy().view(np.float16).astype(np.float32)
        s12 = blk[:, 4:16].astype(np.uint32)
        sc = np.empty((nb, 8), dtype=np.uint32)
        mn = np.empty((nb, 8), dtype=np.uint32)
        sc[:, :4] = s12[:, 0:4] & 0x3F
        mn[:, :4] = s12[:, 4:8] & 0x3F
        sc[:, 4:] = (s12[:, 8:12] & 0x0F) | ((s12[:, 0:4] >> 2) & 0x30)
        mn[:, 4:] = (s12[:, 8:12] >> 4) | ((s12[:, 4:8] >> 2) & 0x30)
        qs = blk[:, 16:144] if qtype == "Q4_K" else blk[:, 48:176]
        q = ((qs[:, (e >> 6) * 32 + (e & 31)] >> (4 * ((e >> 5) & 1))) & 0xF).astype(np.int32)
        if qtype == "Q5_K":
            qhb = blk[:, 16:48]
            q = q | (((qhb[:, e & 31] >> (e >> 5)) & 1).astype(np.int32) << 4)
        scf = sc[:, e >> 5].astype(np.float32)
        mnf = mn[:, e >> 5].astype(np.float32)
        v = (d * scf) * q.astype(np.float32) - (dmin * mnf)
    assert v.dtype == np.float32
    x = np.rint(v.astype(np.float64) * np.float64(S)).astype(np.int64).reshape(-1)
    out = x.astype(np.uint64)
    neg = x < 0
    out[neg] = np.uint64(P) - (-x[neg]).astype(np.uint64)
    return out

"""The pure-maths part of the prover/verifier contract that the hot path needs:
the Goldilocks field, the evaluation domains and the Lagrange closed form
(reference: prover/protocol.py:27-93), plus the column-Merkle helpers a verifier
needs to check an opening (prover/protocol.py:97-112).  Fiat-Shamir and the claim
serialiser of that module are outside this package.

The reference takes BLAKE3 from the `blake3` wheel; the host side here carries its
own small implementation (`blake3_digest`) because an opening hashes a handful of
short messages only.  Bulk hashing is the device's job (cuda_primitives.
hash_columns_streamed / merkle_build_blake3).

Field elements are Python ints in [0, P).
"""
from dataclasses import dataclass
from typing import List, Tuple

P = (1 << 64) - (1 << 32) + 1          # Goldilocks prime
GLOBAL_G = 7                            # generator of the multiplicative group; also the coset shift


def add(a, b):
    return (a + b) % P


def sub(a, b):
    return (a - b) % P


def mul(a, b):
    return (a * b) % P


def inv(a):
    return pow(a % P, P - 2, P)


@dataclass(frozen=True)
class Config:
    """Same four fields as the reference Config (prover/protocol.py:38-58)."""
    ELL: int          # message slots per row
    K_DEG: int        # degree bound  (ELL <= K_DEG)
    N_LIG: int        # codeword length (K_DEG <= N_LIG)
    T_QUERIES: int    # opened columns

    @property
    def W_K(self):
        return pow(GLOBAL_G, (P - 1) // self.K_DEG, P)

    @property
    def W_N(self):
        return pow(GLOBAL_G, (P - 1) // self.N_LIG, P)

    def zeta(self, c: int) -> int:
        """Message point: the c-th K-th root of unity."""
        return pow(self.W_K, c, P)

    def eta(self, j: int) -> int:
        """Codeword point on the coset GLOBAL_G * <w_N>."""
        return GLOBAL_G * pow(self.W_N, j, P) % P


def poly_eval(coeffs: List[int], x: int) -> int:
    acc = 0
    for c in reversed(coeffs):
        acc = (acc * x + c) % P
    return acc


def lagrange(cfg: Config, c: int, eta: int) -> int:
    """L_c(eta) = zeta_c (eta^K - 1) / (K (eta - zeta_c)) on the K-th roots of unity."""
    K = cfg.K_DEG
    zc = cfg.zeta(c)
    return zc * ((pow(eta, K, P) - 1) % P) % P * inv(K * ((eta - zc) % P) % P) % P


def eval_zeta_form(cfg: Config, values: List[int], eta: int) -> int:
    """sum_c values[c] * L_c(eta): the definition every encoder must reproduce."""
    acc = 0
    for c, v in enumerate(values):
        if v:
            acc += v * lagrange(cfg, c, eta)
    return acc % P


# ----------------------------------------------------------------------
# BLAKE3 (host side, short messages) and column-Merkle checks
# ----------------------------------------------------------------------
_B3_IV = (0x6A09E667, 0xBB67AE85, 0x3C6EF372, 0xA54FF53A, 0x510E527F, 0x9B05688C, 0x1F83D9AB, 0x5BE0CD19)
_B3_PERM = (2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8)
_B3_CHUNK_START, _B3_CHUNK_END, _B3_PARENT, _B3_ROOT = 1, 2, 4, 8
_M32 = 0xFFFFFFFF


def _b3_compress(cv, m, counter, block_len, flags):
    s = list(cv) + list(_B3_IV[:4]) + [counter & _M32, (counter >> 32) & _M32, block_len, flags]

    def g(a, b, c, d, x, y):
        s[a] = (s[a] + s[b] + x) & _M32
        v = s[d] ^ s[a]; s[d] = ((v >> 16) | (v << 16)) & _M32
        s[c] = (s[c] + s[d]) & _M32
        v = s[b] ^ s[c]; s[b] = ((v >> 12) | (v << 20)) & _M32
        s[a] = (s[a] + s[b] + y) & _M32
        v = s[d] ^ s[a]; s[d] = ((v >> 8) | (v << 24)) & _M32
        s[c] = (s[c] + s[d]) & _M32
        v = s[b] ^ s[c]; s[b] = ((v >> 7) | (v << 25)) & _M32

    m = list(m)
    for r in range(7):
        g(0, 4, 8, 12, m[0], m[1]); g(1, 5, 9, 13, m[2], m[3])
        g(2, 6, 10, 14, m[4], m[5]); g(3, 7, 11, 15, m[6], m[7])
        g(0, 5, 10, 15, m[8], m[9]); g(1, 6, 11, 12, m[10], m[11])
        g(2, 7, 8, 13, m[12], m[13]); g(3, 4, 9, 14, m[14], m[15])
        m = [m[i] for i in _B3_PERM]
    return [s[i] ^ s[i + 8] for i in range(8)]


def _b3_words(block: bytes):
    block = block + b"\x00" * (64 - len(block))
    return [int.from_bytes(block[4 * i:4 * i + 4], "little") for i in range(16)]


def _b3_chunk_cv(chunk: bytes, counter: int, root: bool):
    cv = list(_B3_IV)
    n_blocks = max(1, (len(chunk) + 63) // 64)
    for b in range(n_blocks):
        blk = chunk[64 * b:64 * b + 64]
        flags = (_B3_CHUNK_START if b == 0 else 0)
        if b == n_blocks - 1:
            flags |= _B3_CHUNK_END | (_B3_ROOT if root else 0)
        cv = _b3_compress(cv, _b3_words(blk), counter, len(blk), flags)
    return cv


def blake3_digest(data: bytes) -> bytes:
    """32-byte BLAKE3 hash (default mode).  Chunks of 1024 bytes; the tree over the
    chunk chaining values pairs neighbours level by level and carries an odd last node
    up unchanged, which is BLAKE3's left-full tree; the final compression carries ROOT."""
    data = bytes(data)
    n_chunks = max(1, (len(data) + 1023) // 1024)
    nodes = [_b3_chunk_cv(data[1024 * c:1024 * c + 1024], c, n_chunks == 1) for c in range(n_chunks)]
    while len(nodes) > 1:
        root = len(nodes) == 2
        nxt = [_b3_compress(_B3_IV, nodes[i] + nodes[i + 1], 0, 64, _B3_PARENT | (_B3_ROOT if root else 0))
               for i in range(0, len(nodes) - 1, 2)]
        if len(nodes) & 1:
            nxt.append(nodes[-1])
        nodes = nxt
    return b"".join(w.to_bytes(4, "little") for w in nodes[0])


def challenge(seed, index: int, label: str = "") -> int:
    """The (label, index)-th field challenge of `seed` on the host (prover/protocol.py:127-135): the low 128 bits of
    BLAKE3(seed32 || label || index_le8), little-endian, mod p.  `seed` is bytes (padded / cut to 32) or an int
    (its 32-byte little-endian form).  cuda_primitives.challenge_vec / challenge_at give the same values on the
    device."""
    key = bytes(seed).ljust(32, b"\x00")[:32] if isinstance(seed, (bytes, bytearray)) else int(seed).to_bytes(32, "little")
    digest = blake3_digest(key + label.encode() + int(index).to_bytes(8, "little"))
    return int.from_bytes(digest[:16], "little") % P


EMPTY_COMMIT_ROOT = b"\x00" * 32        # sentinel for a commit with no rows


def pack_column(col: List[int]) -> bytes:
    return b"".join(int(v).to_bytes(8, "little") for v in col)


def merkle_leaf(col: List[int]) -> bytes:
    """Leaf of the column tree: BLAKE3 of the column's values as little-endian 8-byte words
    (prover/protocol.py:100-104)."""
    return blake3_digest(pack_column(col))


def merkle_verify(leaf: bytes, path: List[Tuple[bytes, int]], root: bytes) -> bool:
    """path: list of (sibling, side); side == 0 means the sibling is the left child
    (prover/protocol.py:106-111)."""
    h = leaf
    for sibling, side in path:
        h = blake3_digest((sibling + h) if side == 0 else (h + sibling))
    return h == root

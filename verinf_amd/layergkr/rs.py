"""Drop-in for the encode side of the reference's `layergkr/rs.py`.

`Commit.from_messages` (rs.py:195-213) encodes through the fused coset LDE after
the one-time bit-exactness gate `_ntt_ok` (rs.py:49-63).  The gate compares the
device codewords with the Lagrange definition `protocol.eval_zeta_form` -- whole
codewords at small geometries, sampled columns at large ones -- and a failing
gate raises instead of switching to another encoder.

The commitment itself (rs.py:135-157, 160-252) is the device path of the reference:
the codeword matrix never leaves the GPU, `gpu.hash_and_tree` hashes its columns and
builds the Merkle tree there, and only the tree (32 bytes per node) and the opened
columns come back to the host.
"""
from typing import List, Sequence, Tuple
import torch

from ..prover.protocol import (  # noqa: F401  (re-exported like the reference)
    Config, P, blake3_digest, challenge, eval_zeta_form, merkle_leaf, merkle_verify)

Codeword = List[int]
Path = List[Tuple[bytes, int]]


def build_tree(leaves: List[bytes]) -> List[List[bytes]]:
    """The Merkle tree over `leaves` on the host, bottom level first and the root alone in the last level
    (rs.py:135-144).  A level of odd length hashes its last node with itself.  The device builds the same tree
    in cuda_primitives.merkle_build_blake3; this one serves the few-leaf trees of tests and openings."""
    tree = [list(leaves)]
    nodes = tree[0]
    while len(nodes) > 1:
        if len(nodes) % 2:
            nodes = nodes + nodes[-1:]
        nodes = [blake3_digest(left + right) for left, right in zip(nodes[0::2], nodes[1::2])]
        tree.append(nodes)
    return tree


def merkle_path(levels: List[List[bytes]], idx: int) -> Path:
    """What a verifier needs to walk from leaf `idx` to the root: per level below the root the sibling's digest and
    on which side it stands, 1 = to the right of the running node (rs.py:147-157; merkle_verify reads it).  The
    last node of an odd level is its own sibling."""
    steps: Path = []
    position = idx
    for nodes in levels[:-1]:
        is_left = position % 2 == 0
        neighbour = position + 1 if is_left else position - 1
        steps.append((nodes[min(neighbour, len(nodes) - 1)], 1 if is_left else 0))
        position >>= 1
    return steps


_GPU_OK: dict = {}
_NTT_OK: dict = {}


def _gpu_ok(cfg: Config) -> bool:
    """Gate of the dense device encoder and the device linear combination (rs.py:38-47): open for a geometry only
    after gpu.selftest has found them bit-identical to the definition on the host; cached per geometry."""
    key = (cfg.ELL, cfg.K_DEG, cfg.N_LIG)
    if key not in _GPU_OK:
        from . import gpu
        _GPU_OK[key] = gpu.available() and gpu.selftest(cfg) is None
    return _GPU_OK[key]


def _ntt_ok(cfg: Config) -> bool:
    key = (cfg.ELL, cfg.K_DEG, cfg.N_LIG)
    if key not in _NTT_OK:
        from . import gpu
        if not gpu.available():
            _NTT_OK[key] = False
        elif cfg.ELL * cfg.N_LIG <= (1 << 16):
            _NTT_OK[key] = gpu.selftest_ntt(cfg, n_rows=2) is None
        else:
            _NTT_OK[key] = gpu.selftest_ntt_spot(cfg) is None
    return _NTT_OK[key]


def linear_combination(cfg: Config, codewords: List[Codeword], coeffs: Sequence[int]) -> Codeword:
    """sum_i coeffs[i] * codewords[i] in Python integers on the host (rs.py:262-281): the second side of the
    cross-check in gpu.selftest and of the reference's own test; gpu.linear_combination / Commit.combine are the
    device forms."""
    if len(codewords) != len(coeffs):
        raise ValueError("coeffs/codewords length mismatch")
    totals = [0] * cfg.N_LIG
    for row, a in zip(codewords, coeffs):
        a %= P
        if a:
            totals = [t + a * int(v) for t, v in zip(totals, row)]
    return [t % P for t in totals]


def sample_columns(seed: bytes, count: int, n_lig: int) -> List[int]:
    """`count` distinct column indices below n_lig drawn from the verifier coin `seed`, in draw order
    (rs.py:282-294): challenge(seed, i, "cols") mod n_lig for i = 0, 1, ..., repeats dropped."""
    if count > n_lig:
        raise ValueError(f"cannot draw {count} distinct columns out of {n_lig}")
    picked: List[int] = []
    taken = set()
    i = 0
    while len(picked) < count:
        col = challenge(seed, i, "cols") % n_lig
        i += 1
        if col not in taken:
            taken.add(col)
            picked.append(col)
    return picked


def lagrange_matrix(cfg: Config) -> List[List[int]]:
    """L[j][c] = L_c(eta_j) as Python integers, N_LIG rows of ELL entries (rs.py:66-77): the device-built dense
    matrix of gpu.lagrange_gpu brought to the host (the definition itself is prover.protocol.lagrange)."""
    from . import gpu
    return [[int(v) for v in row] for row in gpu.lagrange_gpu(cfg).view(torch.int64).t().contiguous().view(torch.uint64).cpu().tolist()]


def encode_row(cfg: Config, message: Sequence[int]) -> Codeword:
    """One message -> its codeword, through the device encoder (the reference's
    CPU version of this function is the dense Lagrange sum, rs.py:110-132)."""
    if len(message) > cfg.ELL:
        raise ValueError(f"message {len(message)} > ELL {cfg.ELL}")
    from . import gpu
    if not _ntt_ok(cfg):
        raise RuntimeError("verinf_amd: the device encoder failed its bit-exactness gate")
    return [int(v) for v in gpu.encode_batch_ntt(cfg, [list(message)])[0].cpu().tolist()]


class Commit:
    """A column-Merkle commitment to Reed-Solomon codewords that stay on the device
    (the `mat=` branch of rs.py:176-187).  Hashing happens on first use of `root`,
    `levels` or `open`, so callers that only encode and combine do not pay for it."""

    def __init__(self, cfg: Config, codewords=None, mat=None):
        """`codewords`: rows as Python lists (the reference's host backend, rs.py:176-193; here they are uploaded
        and committed on the device like any other matrix) or a device tensor; `mat=`: the (rows, N_LIG) device
        tensor of the reference's device backend."""
        if mat is None:
            if codewords is None:
                raise ValueError("Commit needs codewords or mat")
            mat = codewords
        if not isinstance(mat, torch.Tensor):
            from . import gpu
            if not gpu.available():
                raise RuntimeError("verinf_amd.rs.Commit needs a GPU (there is no CPU fallback)")
            rows = [[int(v) % P for v in row] for row in mat]
            if any(len(row) != cfg.N_LIG for row in rows):
                raise ValueError("a codeword has N_LIG entries")
            signed = [[v - (1 << 64) if v >= (1 << 63) else v for v in row] for row in rows]
            mat = torch.tensor(signed, dtype=torch.int64, device="cuda").view(torch.uint64).reshape(len(rows), cfg.N_LIG)
        self.cfg = cfg
        self.mat = mat
        self._root = None
        self._levels_dev = None
        self._levels = None

    def _hash(self):
        if self._root is None:
            from . import gpu
            self._root, self._levels_dev = gpu.hash_and_tree(self.cfg, self.mat)

    @classmethod
    def from_messages(cls, cfg: Config, messages) -> "Commit":
        """`messages`: Python rows or an on-device (rows, <= K_DEG) uint64 tensor."""
        from . import gpu
        if not gpu.available():
            raise RuntimeError("verinf_amd.rs.Commit needs a GPU (there is no CPU fallback)")
        if not _ntt_ok(cfg):
            raise RuntimeError("verinf_amd: the device encoder failed its bit-exactness gate")
        return cls(cfg, gpu.encode_batch_ntt(cfg, messages))

    @property
    def on_gpu(self) -> bool:
        return True

    @property
    def n_rows(self) -> int:
        return int(self.mat.shape[0])

    @property
    def codewords(self) -> List[Codeword]:
        return [[int(v) for v in row] for row in self.mat.cpu().tolist()]

    def col_values(self, col: int) -> List[int]:
        from . import gpu
        return gpu.column(self.mat, col)

    def combine(self, coeffs: Sequence[int]):
        """sum_i coeffs[i] * row_i as a (1, N) device tensor (rs.py:254-259)."""
        from . import gpu
        return gpu.combine_t(self.cfg, self.mat, coeffs)

    @property
    def root(self) -> bytes:
        self._hash()
        return self._root

    @property
    def levels(self) -> List[List[bytes]]:
        if self._levels is None:
            from . import gpu
            self._hash()
            self._levels = gpu.levels_to_host(self._levels_dev)
        return self._levels

    def open(self, col: int) -> Tuple[List[int], Path]:
        return self.col_values(col), merkle_path(self.levels, col)

    def check_open(self, col: int, values: List[int], path: Path) -> bool:
        return merkle_verify(merkle_leaf(values), path, self.root)

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
    Config, P, blake3_digest, eval_zeta_form, merkle_leaf, merkle_verify)

Codeword = List[int]
Path = List[Tuple[bytes, int]]


def _b3(a: bytes, b: bytes) -> bytes:
    return blake3_digest(a + b)


def build_tree(leaves: List[bytes]) -> List[List[bytes]]:
    """Host-side tree over a few leaves (rs.py:135-144): levels[0] = leaves, last level =
    [root]; an odd node is paired with itself.  The device builds the same tree in
    cuda_primitives.merkle_build_blake3."""
    levels = [list(leaves)]
    while len(levels[-1]) > 1:
        cur = levels[-1]
        levels.append([_b3(cur[i], cur[i + 1] if i + 1 < len(cur) else cur[i]) for i in range(0, len(cur), 2)])
    return levels


def merkle_path(levels: List[List[bytes]], idx: int) -> Path:
    """Opening path of leaf `idx` as (sibling, side) pairs, side 1 = sibling on the right
    (rs.py:147-157); a missing sibling is the node itself."""
    path: Path = []
    for level in levels[:-1]:
        sib = idx ^ 1
        if sib >= len(level):
            sib = idx
        path.append((level[sib], 1 if (idx & 1) == 0 else 0))
        idx //= 2
    return path

_NTT_OK: dict = {}


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

    def __init__(self, cfg: Config, mat):
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

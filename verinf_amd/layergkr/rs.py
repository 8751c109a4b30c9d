"""Drop-in for the encode side of the reference's `layergkr/rs.py`.

`Commit.from_messages` (rs.py:195-213) encodes through the fused coset LDE after
the one-time bit-exactness gate `_ntt_ok` (rs.py:49-63).  The gate compares the
device codewords with the Lagrange definition `protocol.eval_zeta_form` -- whole
codewords at small geometries, sampled columns at large ones -- and a failing
gate raises instead of switching to another encoder.

Column hashing and the Merkle tree (rs.py:135-157, BLAKE3) are outside this
package, so a Commit here carries the codeword matrix and the linear operations on
it, not a root.
"""
from typing import List, Sequence

from ..prover.protocol import Config, P, eval_zeta_form  # noqa: F401  (re-exported like the reference)

Codeword = List[int]

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
    """Reed-Solomon codewords of a set of rows, resident on the device."""

    def __init__(self, cfg: Config, mat):
        self.cfg = cfg
        self.mat = mat

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
        raise NotImplementedError("column hashing / Merkle tree are outside verinf_amd")

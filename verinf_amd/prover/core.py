"""Drop-in for the encode side of the reference's `prover/core.py`: the production
commit recipe `encode_messages` (prover/core.py:746-802) and the coefficient-form
encoder `_coset_encode_codewords` (:702-743), served by the fused device pipeline.

The reference builds `padded = [message | row_prg pad]`, clones it, runs the inverse
NTT for the row polynomials, multiplies by materialised powers of the coset shift,
copies into a zeroed (m, N) buffer and runs the forward NTT.  Here the pad is
generated straight into the padded matrix and ONE library call turns that matrix, in place, into
the row polynomials and writes the codewords; no clone, no (m, N) staging buffer, no expanded powers.
Everything else of that module (the interactive protocol, blinding rows, openings)
is outside this package.
"""
import warnings
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .cuda_primitives import (  # noqa: F401  (re-exported like the reference)
    MerkleColumnAccumulator, coset_extend, coset_lde_with_coeffs, hash_columns_streamed, merkle_build_blake3, row_prg,
    row_prg_indexed)
from .protocol import GLOBAL_G, P


@dataclass(frozen=True)
class LigeroConfig:
    """Same fields, checks and derived values as prover/core.py:196-240."""
    ELL: int
    K_DEG: int
    N_LIG: int
    T_QUERIES: int

    def __post_init__(self):
        assert self.ELL <= self.K_DEG <= self.N_LIG
        assert self.K_DEG & (self.K_DEG - 1) == 0
        assert self.N_LIG & (self.N_LIG - 1) == 0
        assert (P - 1) % self.K_DEG == 0
        assert (P - 1) % self.N_LIG == 0
        assert 2 * self.K_DEG <= self.N_LIG, (
            f"2 * K_DEG = {2 * self.K_DEG} must be <= N_LIG = {self.N_LIG} "
            f"(needed for 2K-sized blinding rows for q_lin / p_0)")

    @property
    def W_K(self) -> int:
        return pow(GLOBAL_G, (P - 1) // self.K_DEG, P)

    @property
    def W_N(self) -> int:
        return pow(GLOBAL_G, (P - 1) // self.N_LIG, P)

    @property
    def coset_shift(self) -> int:
        return GLOBAL_G


def _coset_encode_codewords(coeffs: torch.Tensor, cfg: LigeroConfig) -> torch.Tensor:
    """(m, width <= K_DEG ... 2 K_DEG) coefficient rows -> (m, N_LIG) evaluations at
    eta_j = shift * w_N^j (prover/core.py:721-743).  Rows wider than K_DEG (the 2K
    blinding polynomials, :663-666) are transformed with the next power of two as degree
    bound, which gives the same values."""
    m = int(coeffs.size(0))
    if m == 0:
        return torch.empty((0, cfg.N_LIG), dtype=torch.uint64, device="cuda")
    k = cfg.K_DEG
    while k < int(coeffs.size(1)):
        k *= 2
    return coset_extend(coeffs, k, cfg.N_LIG, cfg.coset_shift)


_coset_encode_via_coset_ntt = _coset_encode_codewords      # the cosets formulation is what the device runs


def encode_messages(messages: torch.Tensor, cfg: LigeroConfig, *, master_seed: torch.Tensor, row_offset: int = 0,
                    need_codewords: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """messages: (m, ELL).  Returns (row_polys (m, K_DEG), codewords (m, N_LIG) or None)
    with the K_DEG - ELL slack slots of row i filled by row_prg(master_seed, row_offset + i)
    (prover/core.py:746-802)."""
    m = int(messages.size(0))
    if m == 0:
        return (torch.empty((0, cfg.K_DEG), dtype=torch.uint64, device="cuda"),
                torch.empty((0, cfg.N_LIG), dtype=torch.uint64, device="cuda"))
    if int(messages.size(1)) != cfg.ELL:
        raise RuntimeError("messages must be (m, ELL)")
    slack = cfg.K_DEG - cfg.ELL
    if slack > 0:
        if slack <= cfg.T_QUERIES:
            warnings.warn(
                f"ZK pad too small for column-query confidentiality: "
                f"slack=K_DEG-ELL={slack}, T_QUERIES={cfg.T_QUERIES}. "
                f"Proof is sound but not zero-knowledge under this config.",
                UserWarning, stacklevel=2)
        padded = torch.empty((m, cfg.K_DEG), dtype=torch.uint64, device=messages.device)
        padded.view(torch.int64)[:, :cfg.ELL] = messages.view(torch.int64)
        row_prg(master_seed, row_offset, m, slack, out=padded[:, cfg.ELL:])
        # `padded` is ours: the row polynomials take its place
        return coset_lde_with_coeffs(padded, cfg.K_DEG, cfg.N_LIG, cfg.coset_shift, need_codewords=need_codewords,
                                     in_place=True)
    return coset_lde_with_coeffs(messages, cfg.K_DEG, cfg.N_LIG, cfg.coset_shift, need_codewords=need_codewords)

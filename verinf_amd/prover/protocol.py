"""The pure-maths part of the prover/verifier contract that the hot path needs:
the Goldilocks field, the evaluation domains and the Lagrange closed form
(reference: prover/protocol.py:27-93).  Hashing, Fiat-Shamir and the claim
serialiser of that module are outside this package.

Field elements are Python ints in [0, P).
"""
from dataclasses import dataclass
from typing import List

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

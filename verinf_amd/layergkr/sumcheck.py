"""Drop-in for the reference's `layergkr/sumcheck.py`: multilinear sumcheck prover
and verifier plus the affine mask tape.

The prover (`prove_terms`, `prove`) always runs on the GPU through
`gpu.prove_terms_gpu`: the reference switches to its device path above
`GPU_MIN_SUMCHECK_WORK` and otherwise loops in CPython (sumcheck.py:153-226); both
produce the same proof, so here there is one path and no CPU fallback.  The
verifier, the Lagrange interpolation and the mask algebra are host-side scalar
work on Python ints, as in the reference (sumcheck.py:40-111, 235-298).
"""
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence, Tuple

from ..prover.protocol import P as FIELD_P, inv

INV2 = inv(2)


# ---- multilinear helpers -----------------------------------------------------------
def _fold(values: List[int], r: int) -> List[int]:
    """Fix the most significant variable to r."""
    h = len(values) // 2
    return [(lo + r * (hi - lo)) % FIELD_P for lo, hi in zip(values[:h], values[h:])]


def mle_eval(values: Sequence[int], point: Sequence[int]) -> int:
    """Multilinear extension of 2^n cube values at `point`, most significant variable first."""
    cur = [int(v) for v in values]
    for r in point:
        cur = _fold(cur, r)
    return cur[0] % FIELD_P


def _lagrange_interpolate(points: Sequence[Tuple[int, int]], x: int) -> int:
    """Value at x of the polynomial through `points`."""
    total = 0
    for i, (xi, yi) in enumerate(points):
        num = den = 1
        for k, (xk, _) in enumerate(points):
            if k != i:
                num = num * (x - xk) % FIELD_P
                den = den * (xi - xk) % FIELD_P
        total += yi * num % FIELD_P * inv(den)
    return total % FIELD_P


# ---- mask tape -----------------------------------------------------------------------
# Interface of layergkr/sumcheck.py:74-111.  A masked round adds a scalar polynomial h of the round's degree d
# to the samples.  h is fixed by d tape words and the running value mu: the tape supplies the coefficients of
# x^1 .. x^d, and the constant term follows from h(0) + h(1) = 2 h_0 + (h_1 + ... + h_d) = mu.
class MaskTape:
    """Field elements drawn (and committed to) before the first challenge, consumed front to back."""

    def __init__(self, values, pos: int = 0):
        self.values = list(values)
        self.pos = pos

    def remaining(self) -> int:
        return len(self.values) - self.pos

    def take(self, n: int) -> List[int]:
        if n > self.remaining():
            raise RuntimeError("mask tape exhausted")
        start, self.pos = self.pos, self.pos + n
        return self.values[start:self.pos]


def mask_poly_coeffs(mu: int, u: Sequence[int]) -> List[int]:
    """[h_0, h_1, ..., h_d], lowest degree first, for tape words u = (h_1 .. h_d) and running value mu."""
    upper = [int(w) % FIELD_P for w in u]
    h0 = (mu - sum(upper)) * INV2 % FIELD_P
    return [h0, *upper]


def poly_eval_coeffs(coeffs: Sequence[int], x: int) -> int:
    """Value at x of the polynomial with the given coefficients, lowest degree first."""
    value, power = 0, 1
    for c in coeffs:
        value = (value + c * power) % FIELD_P
        power = power * x % FIELD_P
    return value


def solve_tape_for_target(mu: int, target_h: Sequence[int]) -> Optional[List[int]]:
    """The tape words that make mask_poly_coeffs(mu, .) equal target_h, or None when target_h does not
    satisfy h(0) + h(1) = mu (then no tape produces it).  The map tape -> h is injective: the words are
    h's non-constant coefficients."""
    h = [int(c) % FIELD_P for c in target_h]
    if not h:
        return None
    words = h[1:]
    return words if mask_poly_coeffs(mu, words) == h else None


# ---- proofs ----------------------------------------------------------------------------
@dataclass
class SumcheckProof:
    claim: int
    round_polys: List[List[Tuple[int, int]]] = field(default_factory=list)   # (x, y) samples, x = 0..deg
    challenges: List[int] = field(default_factory=list)
    final_point: List[int] = field(default_factory=list)
    masked: bool = False
    final_mask: int = 0
    n_terms: int = 1


Term = Tuple[int, Sequence[Sequence[int]]]

GPU_MIN_SUMCHECK_WORK = 1 << 16     # kept for callers that read it; every size takes the GPU path here
_SC_GPU: dict = {}


def _sumcheck_gpu_ok() -> bool:
    """One-time gate: the device prover must produce a proof that the host verifier
    accepts and whose claim matches a direct host sum, on the reference's own gate
    instance (sumcheck.py:141-149: Random(1), two 64-long factors, six coins)."""
    if "ok" not in _SC_GPU:
        from . import gpu
        if not gpu.available():
            _SC_GPU["ok"] = False
        else:
            import random
            rr = random.Random(1)
            f = [[rr.randrange(FIELD_P) for _ in range(64)] for _ in range(2)]
            terms = [(1, [f[0], f[1]]), (FIELD_P - 1, [f[0]])]
            coins = [rr.randrange(FIELD_P) for _ in range(6)]
            claim, polys, chals, _ = gpu.prove_terms_gpu(terms, lambda i: coins[i], FIELD_P)
            direct = sum(a * b - a for a, b in zip(f[0], f[1])) % FIELD_P
            pf = SumcheckProof(claim=claim, round_polys=polys, challenges=chals, final_point=list(chals))
            ok, _why = verify_terms(pf, terms, lambda i: coins[i])
            _SC_GPU["ok"] = bool(ok and claim == direct and chals == coins)
    return _SC_GPU["ok"]


def prove_terms(terms: Sequence[Term], coin: Callable[[int], int],
                tape: Optional[MaskTape] = None, mu0: int = 0) -> SumcheckProof:
    """Sumcheck for sum_x sum_k coeff_k prod_j terms[k].factors[j](x); the round degree
    is the widest term.  Factors may be Python sequences or CUDA uint64 tensors."""
    if not terms:
        raise ValueError("no terms")
    from . import gpu
    if not gpu.available():
        raise RuntimeError("verinf_amd.sumcheck.prove_terms needs a GPU (there is no CPU fallback)")
    if not _sumcheck_gpu_ok():
        raise RuntimeError("verinf_amd: the device sumcheck failed its bit-exactness gate")
    mk = (lambda d, mu: mask_poly_coeffs(mu, tape.take(d))) if tape is not None else None
    claim, polys, chals, mu = gpu.prove_terms_gpu(terms, coin, FIELD_P, mk, mu0)
    return SumcheckProof(claim=claim, round_polys=polys, challenges=chals, final_point=list(chals),
                         masked=tape is not None, final_mask=mu, n_terms=len(terms))


def prove(factors: Sequence[Sequence[int]], coin: Callable[[int], int],
          tape: Optional[MaskTape] = None, mu0: int = 0) -> SumcheckProof:
    """Single product of `factors`."""
    return prove_terms([(1, list(factors))], coin, tape, mu0)


def _terminal_value(f, point, cache):
    """f~(point) for a factor given as a Python list (host fold, layergkr/sumcheck.py:40-48) or as a
    device table (one device pass); a table object shared by several terms is evaluated once."""
    key = id(f)
    if key not in cache:
        if hasattr(f, "shape"):
            from . import gpu
            cache[key] = gpu.mle_eval_t(f.reshape(-1), point)
        else:
            cache[key] = mle_eval(f, point)
    return cache[key]


def verify_terms(proof: SumcheckProof, terms: Sequence[Term],
                 coin: Callable[[int], int]) -> Tuple[bool, str]:
    """Round chain plus terminal evaluation; a masked proof's terminal subtracts the carried mask."""
    running = proof.claim % FIELD_P
    deg = max(len(fs) for _, fs in terms)
    for rnd, samples in enumerate(proof.round_polys):
        if len(samples) != deg + 1:
            return False, f"round {rnd}: expected {deg + 1} samples"
        if (_lagrange_interpolate(samples, 0) + _lagrange_interpolate(samples, 1)) % FIELD_P != running:
            return False, f"round {rnd}: g(0)+g(1) != claim"
        r = coin(rnd) % FIELD_P
        if r != proof.challenges[rnd]:
            return False, f"round {rnd}: challenge mismatch"
        running = _lagrange_interpolate(samples, r)
    terminal, seen = 0, {}
    for c, fs in terms:
        prod = c % FIELD_P
        for f in fs:
            prod = prod * _terminal_value(f, proof.final_point, seen) % FIELD_P
        terminal += prod
    terminal %= FIELD_P
    if proof.masked:
        terminal = (terminal + proof.final_mask) % FIELD_P
    if running != terminal:
        return False, "terminal evaluation mismatch"
    return True, "ok"


def verify(proof: SumcheckProof, factors: Sequence[Sequence[int]],
           coin: Callable[[int], int]) -> Tuple[bool, str]:
    """Single-product form of verify_terms."""
    return verify_terms(proof, [(1, list(factors))], coin)


def masked_product_ok(x: int, y: int, a: int, b: int, c: int) -> bool:
    """z = xy carried as X = x+a, Y = y+b, Z = z+c satisfies Z - c = XY - Xb - Ya + ab."""
    X, Y, Z = (x + a) % FIELD_P, (y + b) % FIELD_P, (x * y + c) % FIELD_P
    return (Z - c) % FIELD_P == (X * Y - X * b - Y * a + a * b) % FIELD_P

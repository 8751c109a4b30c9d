"""`layergkr/sumcheck.py` driven the way the reference's own gates drive it (layergkr/tests/test_sumcheck.py:45-155):
host lists in, the device prover underneath, the host verifier on what comes back.  Positive: bare and masked proofs
of degree 2 and 3 verify, a masked proof carries claim + mu0.  Hiding: the tape -> mask-polynomial map is inverted on
targets inside and outside the affine space.  Negative: a wrong claim, an edited round polynomial, a changed challenge
and a tampered terminal are each rejected with the verifier's own reason, and a tape that runs out raises."""
import random

import pytest

from verinf_amd.prover.protocol import P

pytestmark = pytest.mark.gpu

N_VARS = 4


@pytest.fixture(scope="module")
def sc():
    from verinf_amd.layergkr import gpu, sumcheck
    if not gpu.available():
        pytest.skip("needs a GPU")
    assert sumcheck._sumcheck_gpu_ok()
    return sumcheck


def _factors(k=2, seed=17):
    r = random.Random(seed)
    return [[r.randrange(P) for _ in range(1 << N_VARS)] for _ in range(k)]


def _coin(seed=99):
    r = random.Random(seed)
    vals = [r.randrange(P) for _ in range(N_VARS)]
    return lambda i: vals[i]


def _tape(sc, n, seed=5):
    r = random.Random(seed)
    return sc.MaskTape([r.randrange(P) for _ in range(n)])


@pytest.mark.parametrize("k,seed", [(2, 17), (3, 23), (1, 4), (4, 31)])
def test_bare_proofs_verify_and_claim_the_sum(sc, k, seed):
    f = _factors(k, seed)
    proof = sc.prove(f, _coin())
    ok, why = sc.verify(proof, f, _coin())
    assert ok, why
    total = 0
    for i in range(1 << N_VARS):
        term = 1
        for t in f:
            term = term * t[i] % P
        total += term
    assert proof.claim == total % P
    assert len(proof.round_polys) == N_VARS and all(len(rp) == k + 1 for rp in proof.round_polys)


def test_masked_proof_verifies_and_shifts_the_claim(sc):
    f = _factors(2)
    mu0 = 123456789
    bare = sc.prove(f, _coin())
    masked = sc.prove(f, _coin(), tape=_tape(sc, 2 * N_VARS), mu0=mu0)
    ok, why = sc.verify(masked, f, _coin())
    assert ok, why
    assert masked.claim == (bare.claim + mu0) % P
    assert masked.round_polys[0] != bare.round_polys[0]
    assert masked.challenges == bare.challenges


def test_mask_polynomial_splits_the_carried_mask(sc):
    r = random.Random(4)
    for d in (1, 2, 3, 4):
        mu = r.randrange(P)
        u = [r.randrange(P) for _ in range(d)]
        h = sc.mask_poly_coeffs(mu, u)
        assert len(h) == d + 1
        assert (sc.poly_eval_coeffs(h, 0) + sc.poly_eval_coeffs(h, 1)) % P == mu


def test_tape_to_polynomial_map_is_one_to_one_onto_the_affine_space(sc):
    r = random.Random(8)
    d = 3
    mu = r.randrange(P)
    for _ in range(20):
        top = [r.randrange(P) for _ in range(d)]
        target = sc.mask_poly_coeffs(mu, top)
        assert sc.solve_tape_for_target(mu, target) == top
    outside = list(sc.mask_poly_coeffs(mu, [1, 2, 3]))
    outside[0] = (outside[0] + 1) % P
    assert sc.solve_tape_for_target(mu, outside) is None


def test_masked_product_identity(sc):
    r = random.Random(12)
    for _ in range(50):
        x, y, a, b, c = (r.randrange(P) for _ in range(5))
        assert sc.masked_product_ok(x, y, a, b, c)


def test_wrong_claim_edited_polynomial_and_changed_challenge_are_rejected(sc):
    f = _factors(2)
    proof = sc.prove(f, _coin())
    proof.claim = (proof.claim + 1) % P
    ok, why = sc.verify(proof, f, _coin())
    assert not ok and "claim" in why, why

    proof = sc.prove(f, _coin())
    x, y = proof.round_polys[1][0]
    proof.round_polys[1][0] = (x, (y + 1) % P)
    ok, why = sc.verify(proof, f, _coin())
    assert not ok, why

    proof = sc.prove(f, _coin())
    proof.challenges[2] = (proof.challenges[2] + 1) % P
    ok, why = sc.verify(proof, f, _coin())
    assert not ok and "challenge" in why, why


def test_tampered_terminal_is_rejected_masked_and_bare(sc):
    f = _factors(2)
    for tape, mu0 in ((None, 0), (_tape(sc, 2 * N_VARS), 4242)):
        proof = sc.prove(f, _coin(), tape=tape, mu0=mu0)
        bad = [list(f[0]), list(f[1])]
        bad[0][3] = (bad[0][3] + 1) % P
        ok, why = sc.verify(proof, bad, _coin())
        assert not ok and "terminal" in why, (tape is not None, why)


def test_a_tape_that_runs_out_raises(sc):
    f = _factors(2)
    with pytest.raises(RuntimeError):
        sc.prove(f, _coin(), tape=_tape(sc, 2), mu0=1)       # two words per round, four rounds

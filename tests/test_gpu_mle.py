"""GPU parity: eq_vector and mle_eval on the device through the C ABI against the CPU oracle
(bit-exact), plus their use as sumcheck factors."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402


@pytest.fixture(scope="module")
def gpu():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.layergkr import gpu
    return gpu


@pytest.mark.parametrize("n", [0, 1, 2, 3, 4, 5, 8, 9, 12, 13, 17, 20])
def test_eq_vector_matches_oracle(gpu, n):
    rng = random.Random(n)
    z = [rng.randrange(P) for _ in range(n)]
    got = to_np(gpu.eq_vector_t(z))
    assert np.array_equal(got, O.eq_vector(z))
    # the other variable order is the same table for the reversed point
    assert np.array_equal(to_np(gpu.eq_vector_t(z[::-1], msb_first=True)), got)


def test_eq_vector_reduces_its_point_and_handles_boolean_points(gpu):
    z = [P + 3, (1 << 64) - 1, 5]
    assert np.array_equal(to_np(gpu.eq_vector_t(z)), O.eq_vector([v % P for v in z]))
    bits = [1, 0, 0, 1, 1, 0, 1]
    eq = to_np(gpu.eq_vector_t(bits))
    idx = sum(b << j for j, b in enumerate(bits))
    assert int(eq[idx]) == 1 and int(eq.astype(object).sum()) == 1


def test_eq_vector_sums_to_one_at_full_size(gpu):
    rng = random.Random(3)
    z = [rng.randrange(P) for _ in range(24)]
    eq = gpu.eq_vector_t(z)
    assert int(gpu.gl_sum(eq).cpu().item()) == 1
    want = O.eq_vector(z)
    assert np.array_equal(to_np(eq), want)


@pytest.mark.parametrize("n,k", [(0, 1), (1, 1), (3, 2), (4, 1), (7, 5), (12, 3), (16, 2), (21, 1)])
def test_mle_eval_matches_oracle(gpu, n, k):
    rng = random.Random(10 * n + k)
    pt = [rng.randrange(P) for _ in range(n)]
    tabs = rand_field((k, 1 << n), 50 + n)
    tabs[0, 0] = np.uint64(0xFFFFFFFFFFFFFFFF)          # a non-canonical word counts as its residue
    got = gpu.mle_eval_t(to_dev(tabs), pt)
    assert got == [O.mle_eval(tabs[i], pt) for i in range(k)]
    assert gpu.mle_eval_t(to_dev(tabs[0]), pt) == got[0]
    if n:
        i = rng.randrange(1 << n)
        assert gpu.mle_eval_t(to_dev(tabs[k - 1]), [(i >> (n - 1 - j)) & 1 for j in range(n)]) == int(tabs[k - 1, i]) % P


def test_mle_eval_is_what_the_folds_leave(gpu):
    n = 10
    rng = random.Random(5)
    pt = [rng.randrange(P) for _ in range(n)]
    f = to_dev(rand_field((1 << n,), 8))
    cur = f
    for r in pt:
        cur = gpu.fold_t(cur, r)
    assert int(to_np(cur)[0]) == gpu.mle_eval_t(f, pt)


def test_eq_factor_sumcheck_closes_with_mle_evals(gpu):
    """The gate pattern of layergkr/relations.py:104-124: sum_x eq(z, x) a(x) b(x), proven on the
    device with a device-built eq table; the terminal check uses device mle_evals."""
    from verinf_amd.layergkr import sumcheck as sc
    n = 11
    rng = random.Random(9)
    z = [rng.randrange(P) for _ in range(n)]
    a, b = rand_field((1 << n,), 1), rand_field((1 << n,), 2)
    eq = gpu.eq_vector_t(z)
    coins = [rng.randrange(P) for _ in range(n)]
    claim, round_polys, challenges, _ = gpu.prove_terms_gpu([(1, [eq, to_dev(a), to_dev(b)])], lambda i: coins[i], P)
    want_claim = sum(int(e) * int(x) * int(y) for e, x, y in zip(O.eq_vector(z), a, b)) % P
    assert claim == want_claim
    ev = gpu.mle_eval_t(torch.stack([eq.view(torch.int64), to_dev(a).view(torch.int64), to_dev(b).view(torch.int64)]).view(torch.uint64),
                        challenges)
    last = round_polys[-1]
    assert sc._lagrange_interpolate(last, challenges[-1]) == ev[0] * ev[1] * ev[2] % P
    # eq's own extension has the closed form prod_j (z_j r_j + (1 - z_j)(1 - r_j)), z_j on bit j
    closed = 1
    for j in range(n):
        r = challenges[n - 1 - j]
        closed = closed * ((z[j] * r + (1 - z[j]) * (1 - r)) % P) % P
    assert ev[0] == closed

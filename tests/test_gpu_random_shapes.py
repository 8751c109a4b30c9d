"""GPU parity on seeded random shapes: the same bit-exact comparisons as the targeted tests, over
combinations of sizes, widths, pitches and row counts that nobody picked by hand."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def test_lde_random_geometries(cp):
    rng = random.Random(2024)
    for case in range(40):
        logK = rng.randint(1, 15)
        logN = rng.randint(logK, min(logK + 5, 17))
        K, N = 1 << logK, 1 << logN
        m = rng.choice([1, 2, 3, 5, 17, 64, 130]) if logN <= 14 else rng.choice([1, 2, 3, 5])
        w = rng.choice([K, rng.randint(1, K), max(1, K // 2)])
        pitch = w + rng.choice([0, 0, 1, 7, 64])
        shift = rng.choice([7, 1, rng.randrange(2, P)])
        big = rand_field((m, pitch), 1000 + case)
        view = to_dev(big).view(torch.int64)[:, :w].view(torch.uint64)
        want = O.coset_lde_rows(np.ascontiguousarray(big[:, :w]), K, N, shift)
        got = cp.coset_lde(view, K, N, shift)
        assert np.array_equal(to_np(got), want), (case, logK, logN, m, w, pitch, shift)
        co, code = cp.coset_lde_with_coeffs(view, K, N, shift)
        assert torch.equal(code, got), (case, "with_coeffs")
        assert torch.equal(cp.coset_extend(co, K, N, shift), got), (case, "extend")


def test_lde_random_widths_around_the_plane_boundaries(cp):
    """Transform lengths whose middle launch is fused (K = L * L) and their neighbours, rates 1 to 1/8, source widths at
    and around multiples of K/16 (a thread's input planes: the first pass skips the zero half of its inputs, whole or
    partly filled planes), and a workspace of one to three rows, which forces row chunks."""
    from verinf_amd import _lib
    L = _lib.lib()
    rng = random.Random(5)
    for case in range(40):
        logK = rng.choice([12, 12, 13, 14, 14, 16, 11, 10])
        logN = logK + rng.choice([0, 1, 2, 2, 3])
        K, N = 1 << logK, 1 << logN
        unit = K // 16
        w = rng.choice([K, K // 2, K // 4, unit, unit + 1, 8 * unit - 1, 8 * unit + 1, 3 * unit + rng.randint(0, unit - 1),
                        rng.randint(1, K), 7 * unit, 9 * unit, K - 1])
        m = rng.choice([1, 2, 3, 5]) if logN >= 17 else rng.choice([1, 2, 7, 33])
        pitch = w + rng.choice([0, 0, 1, 5, 64])
        shift = rng.choice([7, 7, 1, rng.randrange(2, P)])
        big = rand_field((m, pitch), 5000 + case)
        view = to_dev(big).view(torch.int64)[:, :w].view(torch.uint64)
        want = O.coset_lde_rows(np.ascontiguousarray(big[:, :w]), K, N, shift)
        got = cp.coset_lde(view, K, N, shift)
        assert np.array_equal(to_np(got), want), (case, logK, logN, m, w, pitch, shift)
        out2 = torch.empty((m, N), dtype=torch.uint64, device="cuda")
        ws_bytes = L.vi_coset_lde_min_workspace_bytes(K, N) * rng.choice([1, 2, 3])
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        _lib.check(L.vi_coset_lde(view.data_ptr(), m, w, pitch, K, N, shift, out2.data_ptr(), N, ws.data_ptr(), ws_bytes,
                                  _lib.stream_ptr()))
        assert torch.equal(out2, got), (case, "chunked")


def test_ntt_random_sizes_round_trip_and_oracle(cp):
    rng = random.Random(7)
    for case in range(25):
        logn = rng.randint(1, 18)
        m = rng.choice([1, 2, 3, 9, 33]) if logn <= 15 else rng.choice([1, 2])
        a = rand_field((m, 1 << logn), 2000 + case)
        rows = to_dev(a)
        cp.ntt_forward_batched(rows)
        assert np.array_equal(to_np(rows), O.ntt_rows(a)), (case, logn, m)
        cp.ntt_inverse_batched(rows)
        assert np.array_equal(to_np(rows), a), (case, logn, m, "inverse")


def test_hash_tree_shapes_up_to_a_hundred_chunks(cp):
    """Chunk counts whose BLAKE3 tree has an odd node on some level, a single node, exact powers of two, and the 86
    chunks of an 11008-row matrix: the merge launches take two levels of the tree at a time."""
    rng = random.Random(3)
    for chunks in (1, 2, 3, 4, 5, 6, 7, 8, 9, 15, 16, 17, 31, 33, 43, 64, 85, 86, 87, 100):
        m = (chunks - 1) * 128 + rng.choice([1, 7, 64, 127, 128])
        n = rng.choice([1, 3, 64, 65, 300])
        a = rand_field((m, n), 9000 + chunks)
        assert np.array_equal(to_np(cp.hash_columns_streamed(to_dev(a))), O.hash_columns(a)), (chunks, m, n)


def test_hash_random_shapes_and_slabs(cp):
    rng = random.Random(11)
    for case in range(30):
        m = rng.choice([1, 2, 127, 128, 129, 255, 256, 257, rng.randint(1, 3000)])
        n = rng.choice([1, 2, 63, 64, 65, 255, 256, 257, rng.randint(1, 1500)])
        pitch = n + rng.choice([0, 0, 3, 64])
        big = rand_field((m, pitch), 3000 + case)
        dev = to_dev(big).view(torch.int64)[:, :n].view(torch.uint64)
        want = O.hash_columns(np.ascontiguousarray(big[:, :n]))
        assert np.array_equal(to_np(cp.hash_columns_streamed(dev)), want), (case, m, n, pitch)
        if m > 128:
            acc = cp.MerkleColumnAccumulator(n, m)
            r = 0
            while r < m:
                k = min(m - r, rng.choice([1, 50, 128, 129, 300, 1024]))
                acc.update(dev[r:r + k])
                r += k
            assert np.array_equal(to_np(acc.finalize()), want), (case, m, n, "accumulator")
        root, levels = cp.merkle_build_blake3(to_dev(want))
        assert to_np(root).tobytes() == O.merkle_levels(want)[-1][0].tobytes(), (case, "root")


def test_sumcheck_random_term_structures():
    from verinf_amd.layergkr import gpu
    rng = random.Random(5)
    for case in range(25):
        v = rng.randint(1, 14)
        n_tables = rng.randint(1, 12)
        n_terms = rng.randint(1, 5)
        terms_idx = [(rng.randrange(P), [rng.randrange(n_tables) for _ in range(rng.randint(1, 4))]) for _ in range(n_terms)]
        tabs = [rand_field((1 << v,), 4000 + 20 * case + j) for j in range(n_tables)]
        dev = [to_dev(t) for t in tabs]
        coins = [rng.randrange(P) for _ in range(v)]
        claim, polys, chal, _ = gpu.prove_terms_gpu([(c, [dev[i] for i in idx]) for c, idx in terms_idx], lambda i: coins[i], P)
        want_claim, want_samples, _ = O.sumcheck_prove(tabs, terms_idx, coins)
        deg = max(len(idx) for _, idx in terms_idx)
        assert claim == want_claim, (case, v, terms_idx)
        assert [[y for _, y in s] for s in polys] == [list(s[: deg + 1]) for s in want_samples], (case, v, terms_idx)
        assert chal == coins

"""GPU parity: gl_matmul / gl_matvec / poly_eval / linear combinations through the C ABI
against Python big-int arithmetic (bit-exact)."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def _matmul_ref(A, B):
    Ao, Bo = A.astype(object), B.astype(object)
    return (Ao.dot(Bo) % P).astype(np.uint64)


@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (1, 7, 300), (3, 64, 64), (5, 200, 513), (1, 4096, 8192),
                                   (2, 1000, 70000), (16, 16, 1000), (40, 33, 257),
                                   (4, 129, 300), (7, 50, 600), (6, 4100, 256), (3, 9, 5)])
def test_matmul_matches_bigint(cp, m, k, n):
    A, B = rand_field((m, k), 1 + m), rand_field((k, n), 2 + n)
    got = cp.gl_matmul(to_dev(A), to_dev(B))
    assert tuple(got.shape) == (m, n)
    assert np.array_equal(to_np(got), _matmul_ref(A, B))


def test_matmul_extreme_values_many_wraps(cp):
    """All entries p-1: every product is (p-1)^2 and the exact accumulator wraps 2^128 often."""
    k, n = 1 << 16, 300
    A = np.full((1, k), P - 1, dtype=np.uint64)
    B = np.full((k, n), P - 1, dtype=np.uint64)
    got = to_np(cp.gl_matmul(to_dev(A), to_dev(B)))
    assert (got == np.uint64(k % P)).all()                 # (p-1)^2 = 1, summed k times
    B[::2] = 1
    got = to_np(cp.gl_matmul(to_dev(A), to_dev(B)))
    assert (got == np.uint64((k // 2 + (k // 2) * (P - 1)) % P)).all()


@pytest.mark.parametrize("m,n", [(1, 1), (37, 1001), (3, 4096), (5, 5000), (9000, 70), (300, 255), (2, 20011)])
def test_matvec_matches_bigint(cp, m, n):
    """Short and long rows (a wavefront or a whole workgroup per row), lengths around the unrolled stride."""
    M, v = rand_field((m, n), 3 + m), rand_field(n, 4 + n)
    got = to_np(cp.gl_matvec(to_dev(M), to_dev(v)))
    assert np.array_equal(got, _matmul_ref(M, v.reshape(-1, 1)).reshape(-1))


def test_matvec_and_poly_eval(cp):
    M, v = rand_field((37, 1001), 3), rand_field(1001, 4)
    got = to_np(cp.gl_matvec(to_dev(M), to_dev(v)))
    assert np.array_equal(got, _matmul_ref(M, v.reshape(-1, 1)).reshape(-1))
    r = random.Random(5)
    coeffs = [r.randrange(P) for _ in range(33)]
    pts = [0, 1, P - 1] + [r.randrange(P) for _ in range(300)]
    want = [sum(c * pow(x, i, P) for i, c in enumerate(coeffs)) % P for x in pts]
    got = cp.poly_eval(to_dev(np.array(coeffs, dtype=np.uint64)), to_dev(np.array(pts, dtype=np.uint64)))
    assert to_np(got).tolist() == want
    C2 = rand_field((4, 9), 6)
    got2 = to_np(cp.poly_eval(to_dev(C2), to_dev(np.array(pts[:50], dtype=np.uint64))))
    for i in range(4):
        assert got2[i].tolist() == [sum(int(c) * pow(x, j, P) for j, c in enumerate(C2[i])) % P for x in pts[:50]]
    with pytest.raises(RuntimeError):
        cp.gl_matmul(to_dev(M), to_dev(M))
    with pytest.raises(RuntimeError):
        cp.gl_matvec(to_dev(M), to_dev(v[:5].copy()))


def test_linear_combination_is_the_codeword_of_the_combined_messages():
    """RS codes are linear: combining codewords = encoding the combined messages
    (the identity the projection seam rests on, layergkr/rs.py:262-279)."""
    from verinf_amd.layergkr import gpu, rs
    cfg = rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8)
    r = random.Random(5)
    msgs = [[r.randrange(P) for _ in range(cfg.ELL)] for _ in range(6)]
    co = [r.randrange(P) for _ in range(6)]
    commit = rs.Commit.from_messages(cfg, msgs)
    combined = commit.combine(co)
    assert tuple(combined.shape) == (1, cfg.N_LIG)
    mixed = [sum(c * m[j] for c, m in zip(co, msgs)) % P for j in range(cfg.ELL)]
    want = to_np(gpu.encode_batch_ntt(cfg, [mixed]))[0]
    assert np.array_equal(to_np(combined)[0], want)
    assert gpu.linear_combination(cfg, commit.codewords, co) == [int(v) for v in want]

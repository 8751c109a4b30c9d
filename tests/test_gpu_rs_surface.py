"""The commit / encode surface of `layergkr/rs.py` and `layergkr/gpu.py`, driven the way the reference's own tests
drive it (layergkr/tests/test_gpu.py:33-121, layergkr/tests/test_rs.py:23-62), with the package's modules in the place
of the reference's: what the device returns is compared with the definition in Python integers
(`protocol.eval_zeta_form`, `protocol.lagrange`) and with the host-side tree over the same codewords."""
import random

import pytest
import torch

from verinf_amd.prover.protocol import P, blake3_digest, eval_zeta_form, lagrange, merkle_leaf

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    from verinf_amd.layergkr import gpu, rs
    if not gpu.available():
        pytest.skip("needs a GPU")
    return gpu, rs


def _configs(rs):
    return [rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4), rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8),
            rs.Config(ELL=256, K_DEG=512, N_LIG=1024, T_QUERIES=8)]


def test_selftest_is_green_at_every_geometry(mods):
    gpu, rs = mods
    for cfg in _configs(rs):
        assert gpu.selftest(cfg, n_rows=6) is None, (cfg.ELL, cfg.N_LIG)


def test_rows_that_are_mostly_padding(mods):
    """Real rows are mostly zeros; the dense encoder and the transform encoder must treat them like any other."""
    gpu, rs = mods
    cfg = _configs(rs)[1]
    r = random.Random(3)
    msgs = [[r.randrange(P) if j < 3 else 0 for j in range(cfg.ELL)] for _ in range(5)]
    dense = gpu.encode_batch(cfg, msgs)
    for i, m in enumerate(msgs):
        row = rs.encode_row(cfg, m)
        assert dense[i] == row, i
        for j in (0, 1, cfg.N_LIG // 3, cfg.N_LIG - 1):
            assert row[j] == eval_zeta_form(cfg, m, cfg.eta(j)), (i, j)


def test_commit_root_is_the_same_from_lists_and_from_the_device_matrix(mods):
    """The reference builds a Commit either from Python rows or from the device matrix and pins that both give one
    root; here both end on the device, and the root is also rebuilt on the host from the definition of the tree."""
    gpu, rs = mods
    cfg = _configs(rs)[2]
    r = random.Random(9)
    msgs = [[r.randrange(P) for _ in range(cfg.ELL)] for _ in range(8)]
    from_lists = rs.Commit(cfg, gpu.encode_batch(cfg, msgs))
    from_rows = rs.Commit(cfg, [rs.encode_row(cfg, m) for m in msgs])
    from_mat = rs.Commit(cfg, mat=gpu.encode_batch_ntt(cfg, msgs))
    assert from_lists.root == from_rows.root == from_mat.root
    code = from_mat.codewords
    leaves = [merkle_leaf([row[j] for row in code]) for j in range(cfg.N_LIG)]
    assert rs.build_tree(leaves)[-1][0] == from_mat.root
    assert from_lists.levels == rs.build_tree(leaves)
    col = 777
    values, path = from_lists.open(col)
    assert values == [row[col] for row in code] and from_mat.check_open(col, values, path)
    with pytest.raises(ValueError):
        rs.Commit(cfg, [[1, 2, 3]])
    with pytest.raises(ValueError):
        rs.Commit(cfg)


def test_linear_combination_host_and_device(mods):
    gpu, rs = mods
    cfg = _configs(rs)[1]
    r = random.Random(5)
    cw = [rs.encode_row(cfg, [r.randrange(P) for _ in range(cfg.ELL)]) for _ in range(6)]
    co = [r.randrange(P) for _ in range(6)]
    want = [sum(a * row[j] for a, row in zip(co, cw)) % P for j in range(cfg.N_LIG)]
    assert rs.linear_combination(cfg, cw, co) == want
    assert [int(v) for v in gpu.linear_combination(cfg, cw, co)] == want
    with pytest.raises(ValueError):
        rs.linear_combination(cfg, cw, co[:-1])


def test_lagrange_matrix_cells(mods):
    gpu, rs = mods
    small, larger = _configs(rs)[:2]
    M = rs.lagrange_matrix(small)
    for j in range(small.N_LIG):
        for c in range(small.ELL):
            assert M[j][c] == lagrange(small, c, small.eta(j)), (j, c)
    M = rs.lagrange_matrix(larger)
    r = random.Random(5)
    for _ in range(200):
        j, c = r.randrange(larger.N_LIG), r.randrange(larger.ELL)
        assert M[j][c] == lagrange(larger, c, larger.eta(j)), (j, c)


def test_encode_row_short_sparse_and_too_long(mods):
    gpu, rs = mods
    cfg = _configs(rs)[0]
    r = random.Random(11)
    short = [r.randrange(P) for _ in range(cfg.ELL // 2)]
    assert rs.encode_row(cfg, short) == rs.encode_row(cfg, short + [0] * (cfg.ELL - len(short)))
    sparse = [r.randrange(P) if i % 3 == 0 else 0 for i in range(cfg.ELL)]
    cw = rs.encode_row(cfg, sparse)
    for j in (0, 2, cfg.N_LIG - 1):
        assert cw[j] == eval_zeta_form(cfg, sparse, cfg.eta(j))
    with pytest.raises(ValueError):
        rs.encode_row(cfg, [1] * (cfg.ELL + 1))


def test_sampled_columns_are_distinct_and_reproducible(mods):
    gpu, rs = mods
    cols = rs.sample_columns(b"root-bytes", 8, 256)
    assert len(cols) == len(set(cols)) == 8 and all(0 <= c < 256 for c in cols)
    assert cols == rs.sample_columns(b"root-bytes", 8, 256) != rs.sample_columns(b"other", 8, 256)
    assert sorted(rs.sample_columns(b"x", 16, 16)) == list(range(16))
    with pytest.raises(ValueError):
        rs.sample_columns(b"x", 17, 16)
    assert blake3_digest(b"") == bytes.fromhex("af1349b9f5f9a1a6a0404dea36dcc9499bcb25c9adc112b7cc9a93cae41f3262")

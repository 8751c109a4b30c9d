"""GPU parity: the combiner challenge PRF, CSR matvec (plain and challenged) and LogUp
multiplicities through the C ABI against the CPU oracle (bit-exact)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402

SEED = bytes((91 * i + 7) % 256 for i in range(32))


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def _u8(b):
    return torch.tensor(list(b), dtype=torch.uint8, device="cuda")


@pytest.mark.parametrize("label", [b"", b"lin", b"irs", b"quad", b"1234567", b"12345678"])
def test_challenge_vec_and_at(cp, label):
    n = 5000
    got = to_np(cp.challenge_vec(_u8(SEED), _u8(label), n))
    want = O.challenge_vec(SEED, label, n)
    assert np.array_equal(got, want) and int(got.max()) < P
    cids = np.array([0, 1, 4999, 1 << 31, 1 << 40, (1 << 64) - 1], dtype=np.uint64)
    at = to_np(cp.challenge_at(_u8(SEED), _u8(label), to_dev(cids)))
    assert np.array_equal(at, O.challenge_vec(SEED, label, cids=cids))
    assert np.array_equal(at[:3], want[[0, 1, 4999]])
    shaped = cp.challenge_at(_u8(SEED), _u8(label), to_dev(cids.reshape(2, 3)))
    assert tuple(shaped.shape) == (2, 3)
    assert cp.challenge_vec(_u8(SEED), _u8(label), 0).numel() == 0


def _csr(n_rows, n_cols, max_nnz, seed, min_nnz=0):
    rng = np.random.default_rng(seed)
    counts = rng.integers(min_nnz, max_nnz + 1, n_rows)
    row_ptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint64)
    nnz = int(row_ptr[-1])
    return rand_field((nnz,), seed + 1), rng.integers(0, n_cols, nnz).astype(np.uint64), row_ptr


@pytest.mark.parametrize("n_rows,n_cols,max_nnz,min_nnz", [(1, 1, 1, 1), (100, 1000, 8, 0), (5000, 300, 3, 0), (64, 5000, 700, 300),
                                                           (3, 100000, 50000, 40000), (1000, 10, 0, 0)])
def test_spmv_matches_oracle(cp, n_rows, n_cols, max_nnz, min_nnz):
    val, col, row_ptr = _csr(n_rows, n_cols, max_nnz, 7 + n_rows, min_nnz)
    x = rand_field((n_cols,), 3)
    got = cp.gl_spmv(to_dev(val), to_dev(col), to_dev(row_ptr), to_dev(x), n_rows)
    assert np.array_equal(to_np(got), O.spmv(val, col, row_ptr, x))
    got_c = cp.gl_spmv_challenged(to_dev(val), to_dev(col), to_dev(row_ptr), _u8(SEED), _u8(b"lin"), n_rows)
    want_c = O.spmv(val, col, row_ptr, None, SEED, b"lin")
    assert np.array_equal(to_np(got_c), want_c)
    # the challenged form is the plain form on the materialised combiner
    r = cp.challenge_vec(_u8(SEED), _u8(b"lin"), n_cols)
    assert torch.equal(cp.gl_spmv(to_dev(val), to_dev(col), to_dev(row_ptr), r, n_rows), got_c)


def test_spmv_rejects_bad_row_ptr(cp):
    val, col, row_ptr = _csr(10, 20, 4, 1)
    with pytest.raises(RuntimeError):
        cp.gl_spmv(to_dev(val), to_dev(col), to_dev(row_ptr), to_dev(rand_field((20,), 2)), 11)


def test_lookup_multiplicities(cp):
    rng = np.random.default_rng(5)
    # a range table is indexed directly; out-of-range values count nowhere
    T = 1 << 12
    table = np.arange(T, dtype=np.uint64)
    x = rng.integers(0, T + 500, 200000).astype(np.uint64)
    got = to_np(cp.lookup_multiplicities(to_dev(x), to_dev(table)))
    want = np.bincount(x[x < T].astype(np.int64), minlength=T).astype(np.uint64)
    assert np.array_equal(got, want)
    # an arbitrary table, with a duplicate entry (the first occurrence collects) and field-sized values
    tab = rand_field((300,), 6)
    tab[17] = tab[3]
    xs = np.concatenate([tab[rng.integers(0, 300, 5000)], rand_field((100,), 8)])
    got = to_np(cp.lookup_multiplicities(to_dev(xs), to_dev(tab)))
    assert np.array_equal(got, O.lookup_multiplicities(xs, tab))
    assert int(got[17]) == 0 and int(got.sum()) <= 5100
    # accumulation across calls
    mult = torch.zeros(300, dtype=torch.int64, device="cuda").view(torch.uint64)
    dev_tab = to_dev(tab)
    cp.lookup_multiplicities_into(to_dev(xs[:2000]), dev_tab, mult)
    cp.lookup_multiplicities_into(to_dev(xs[2000:]), dev_tab, mult)
    assert np.array_equal(to_np(mult), got)

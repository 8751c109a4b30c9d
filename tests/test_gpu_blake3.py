"""GPU parity: BLAKE3 column digests, the streaming accumulator and the Merkle tree through
the C ABI against the CPU oracle and the published known answers (byte-exact)."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import rand_field, to_dev, to_np  # noqa: E402


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def _words(n_bytes):
    """The published test pattern (byte i = i mod 251) as little-endian uint64 rows."""
    data = bytes(i % 251 for i in range(n_bytes))
    return np.frombuffer(data, dtype="<u8").astype(np.uint64)


def test_known_answers_as_columns(cp):
    """Every known answer whose length is a multiple of 8 bytes, each laid out as one column
    of a matrix whose other columns hold unrelated data."""
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "blake3_kat.json")
    cases = [c for c in json.load(open(here))["cases"] if c["len"] % 8 == 0]
    assert len(cases) >= 7
    for c in cases:
        m = c["len"] // 8
        mat = rand_field((m, 5), 100 + m)
        if m:
            mat[:, 3] = _words(c["len"])
        dig = to_np(cp.hash_columns_streamed(to_dev(mat) if m else torch.empty((0, 5), dtype=torch.uint64, device="cuda")))
        assert dig.shape == (5, 32)
        assert dig[3].tobytes().hex() == c["hash"], c["len"]


@pytest.mark.parametrize("m,n", [(1, 1), (3, 7), (8, 64), (9, 65), (127, 300), (128, 256), (129, 257), (255, 3),
                                 (256, 1000), (257, 33), (384, 100), (385, 100), (1000, 513), (1024, 2048),
                                 (1025, 40), (4096, 700), (5000, 129)])
def test_hash_columns_matches_oracle(cp, m, n):
    mat = rand_field((m, n), 7 * m + n)
    # non-canonical words hash as they are: bytes, not field elements
    mat[0, 0] = np.uint64(0xFFFFFFFFFFFFFFFF)
    got = to_np(cp.hash_columns_streamed(to_dev(mat)))
    assert np.array_equal(got, O.hash_columns(mat))


def test_hash_columns_row_strided_view(cp):
    mat = rand_field((300, 96), 5)
    dev = to_dev(mat)
    view = dev.view(torch.int64)[:, 16:80].view(torch.uint64)       # row pitch 96, 64 columns
    assert not view.is_contiguous()
    got = to_np(cp.hash_columns_streamed(view))
    assert np.array_equal(got, O.hash_columns(mat[:, 16:80]))


def test_hash_columns_rejects_bad_input(cp):
    with pytest.raises(RuntimeError):
        cp.hash_columns_streamed(torch.zeros((4, 4), dtype=torch.int64, device="cuda"))
    with pytest.raises(RuntimeError):
        cp.hash_columns_streamed(torch.zeros((4, 4), dtype=torch.uint64))
    with pytest.raises(RuntimeError):
        cp.hash_columns_streamed(torch.zeros(16, dtype=torch.uint64, device="cuda"))


@pytest.mark.parametrize("m,n,slabs", [(129, 10, [129]), (300, 50, [3, 100, 197]), (1024, 64, [256, 256, 256, 256]),
                                       (1027, 33, [3, 1024]), (2000, 20, [1, 127, 128, 500, 0, 1244]),
                                       (640, 17, [64] * 10), (257, 5, [128, 128, 1])])
def test_accumulator_matches_one_shot(cp, m, n, slabs):
    assert sum(slabs) == m
    mat = rand_field((m, n), m + 3 * n)
    dev = to_dev(mat)
    acc = cp.MerkleColumnAccumulator(n, m)
    r = 0
    for k in slabs:
        acc.update(dev[r:r + k])
        r += k
    got = to_np(acc.finalize())
    assert np.array_equal(got, O.hash_columns(mat))
    assert np.array_equal(got, to_np(cp.hash_columns_streamed(dev)))


def test_accumulator_requires_all_rows(cp):
    acc = cp.MerkleColumnAccumulator(4, 300)
    acc.update(to_dev(rand_field((128, 4), 1)))
    with pytest.raises(AssertionError):
        acc.finalize()
    with pytest.raises(AssertionError):
        cp.MerkleColumnAccumulator(4, 128)


# counts around the 512-leaf blocks of the fused tree kernel and around its nine levels per launch
@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 31, 32, 33, 511, 512, 513, 1000, 1023, 1025, 4097, 65536, 65537,
                               262143, 262144, 262147, 524289])
def test_merkle_build_matches_oracle(cp, k):
    rng = np.random.default_rng(k)
    leaves = rng.integers(0, 256, (k, 32), dtype=np.uint8)
    root, levels = cp.merkle_build_blake3(to_dev(leaves))
    want = O.merkle_levels(leaves)
    assert len(levels) == len(want)
    for g, w in zip(levels, want):
        assert np.array_equal(to_np(g), w)
    assert to_np(root).tobytes() == want[-1][0].tobytes()
    # the level-by-level entry point gives the same nodes
    cur = to_dev(leaves)
    for w in want[1:]:
        cur = cp.merkle_one_level(cur)
        assert np.array_equal(to_np(cur), w)


def test_commit_root_and_openings(cp):
    """End to end through the rs.Commit mirror: encode on the device, hash, open a few columns,
    check the paths with the host verifier, and compare the root with the oracle's."""
    from verinf_amd.layergkr import rs
    from verinf_amd.prover.protocol import Config
    cfg = Config(ELL=48, K_DEG=64, N_LIG=256, T_QUERIES=4)
    msgs = rand_field((37, 48), 9)
    com = rs.Commit.from_messages(cfg, to_dev(msgs))
    code = to_np(com.mat)
    want_levels = O.merkle_levels(O.hash_columns(code))
    assert com.root == want_levels[-1][0].tobytes()
    for col in (0, 1, 100, 255):
        values, path = com.open(col)
        assert values == [int(v) for v in code[:, col]]
        assert com.check_open(col, values, path)
        values[3] ^= 1
        assert not com.check_open(col, values, path)


def test_full_size_properties(cp):
    """At the commit's full width (2^18 columns) the oracle is only run on sampled columns:
    digest j depends on column j alone, and permuting columns permutes digests."""
    m, n = 1024, 1 << 18
    mat = torch.randint(0, 2 ** 62, (m, n), dtype=torch.int64, device="cuda").view(torch.uint64)
    dig = cp.hash_columns_streamed(mat)
    cols = [0, 1, 63, 64, 255, 256, 4095, 77777, n - 2, n - 1]
    sub = to_np(mat.view(torch.int64)[:, cols].contiguous().view(torch.uint64))
    assert np.array_equal(to_np(dig)[cols], O.hash_columns(sub))
    rolled = torch.roll(mat.view(torch.int64), 5, dims=1).view(torch.uint64)
    assert torch.equal(cp.hash_columns_streamed(rolled), torch.roll(dig, 5, dims=0))
    root, levels = cp.merkle_build_blake3(dig)
    assert len(levels) == 19 and levels[-1].shape == (1, 32)
    # a path read off the device tree verifies on the host
    from verinf_amd.prover.protocol import merkle_verify
    idx = 123457
    path = []
    i = idx
    for lvl in levels[:-1]:
        sib = i ^ 1 if (i ^ 1) < lvl.shape[0] else i
        path.append((bytes(lvl[sib].cpu().tolist()), 1 if (i & 1) == 0 else 0))
        i //= 2
    assert merkle_verify(bytes(dig[idx].cpu().tolist()), path, bytes(root.cpu().tolist()))

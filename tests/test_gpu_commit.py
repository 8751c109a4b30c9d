"""GPU parity: the production commit recipe -- ZK pad generator, values -> (row polynomials,
codewords), coefficients -> codewords, encode_messages -- through the C ABI against the CPU
oracle (bit-exact)."""
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


SEED = bytes((37 * i + 11) % 256 for i in range(32))


def _seed_dev():
    return torch.tensor(list(SEED), dtype=torch.uint8, device="cuda")


@pytest.mark.parametrize("row_offset,n_rows,slack", [(0, 1, 1), (0, 3, 5), (7, 64, 33), (1000, 257, 100), (123456, 5, 1000),
                                                     ((1 << 32) - 2, 4, 3), (0, 0, 4), (0, 4, 0)])
def test_row_prg_matches_oracle(cp, row_offset, n_rows, slack):
    got = cp.row_prg(_seed_dev(), row_offset, n_rows, slack)
    assert tuple(got.shape) == (n_rows, slack) and got.dtype == torch.uint64
    want = O.row_prg(SEED, row_offset, n_rows, slack)
    assert np.array_equal(to_np(got), want)
    if n_rows and slack:
        assert int(want.max()) < P


def test_row_prg_indexed_and_in_place_slice(cp):
    idx = np.array([0, 1, 7, 8, 1 << 20, (1 << 33) + 5, 7], dtype=np.uint64)
    got = cp.row_prg_indexed(_seed_dev(), to_dev(idx), 19)
    assert np.array_equal(to_np(got), O.row_prg(SEED, 0, 0, 19, row_indices=idx))
    # row r of the contiguous form is the indexed form at row_offset + r
    assert np.array_equal(to_np(cp.row_prg(_seed_dev(), 7, 2, 19)), to_np(got)[2:4])
    padded = torch.zeros((9, 64), dtype=torch.int64, device="cuda").view(torch.uint64)
    cp.row_prg(_seed_dev(), 40, 9, 24, out=padded[:, 40:])
    host = to_np(padded)
    assert not host[:, :40].any()
    assert np.array_equal(host[:, 40:], O.row_prg(SEED, 40, 9, 24))


def test_row_prg_rejects_bad_seed(cp):
    with pytest.raises(RuntimeError):
        cp.row_prg(torch.zeros(31, dtype=torch.uint8, device="cuda"), 0, 1, 1)
    with pytest.raises(RuntimeError):
        cp.row_prg(torch.zeros(32, dtype=torch.uint8), 0, 1, 1)
    with pytest.raises(RuntimeError):
        cp.row_prg(torch.zeros(32, dtype=torch.int8, device="cuda"), 0, 1, 1)


@pytest.mark.parametrize("K,N,m,w", [(16, 32, 5, 16), (64, 256, 9, 40), (1024, 2048, 3, 1024), (4096, 16384, 4, 3000),
                                     (8192, 32768, 3, 8192), (1 << 14, 1 << 16, 5, 8192), (1 << 16, 1 << 18, 2, 1 << 16)])
def test_coefficients_and_codewords_in_one_call(cp, K, N, m, w):
    msgs = rand_field((m, w), K + m)
    padded = np.zeros((m, K), dtype=np.uint64)
    padded[:, :w] = msgs
    want_c = O.ntt_rows(padded, inverse=True)
    want = O.coset_lde_rows(msgs, K, N, 7)
    co, code = cp.coset_lde_with_coeffs(to_dev(msgs), K, N, 7)
    assert np.array_equal(to_np(co), want_c)
    assert np.array_equal(to_np(code), want)
    co2, none = cp.coset_lde_with_coeffs(to_dev(msgs), K, N, 7, need_codewords=False)
    assert none is None and np.array_equal(to_np(co2), want_c)
    # in place: the padded matrix becomes the coefficients (what encode_messages does with its own buffer)
    own = to_dev(padded)
    co3, code3 = cp.coset_lde_with_coeffs(own, K, N, 7, in_place=True)
    assert co3.data_ptr() == own.data_ptr() and np.array_equal(to_np(own), want_c) and np.array_equal(to_np(code3), want)
    if w < K:
        with pytest.raises(RuntimeError):
            cp.coset_lde_with_coeffs(to_dev(msgs), K, N, 7, in_place=True)     # not (m, K)
    # the reference's two-step form gives the same coefficients
    ref = to_dev(padded)
    cp.ntt_inverse_batched(ref)
    assert torch.equal(ref, co)
    assert np.array_equal(to_np(cp.coset_extend(co, K, N, 7)), want)
    # low-degree input: trailing zero coefficients need not be passed
    if w < K:
        low = to_dev(np.ascontiguousarray(want_c[:, : K // 2]))
        full = np.zeros((m, K), dtype=np.uint64)
        full[:, : K // 2] = want_c[:, : K // 2]
        assert torch.equal(cp.coset_extend(low, K, N, 7), cp.coset_extend(to_dev(full), K, N, 7))


def test_coset_extend_is_polynomial_evaluation(cp):
    """Pinned by the definition: out[j] = sum_i c_i (shift * w_N^j)^i, by Horner on the host."""
    K, N, shift = 32, 128, 7
    co = rand_field((3, K), 77)
    got = to_np(cp.coset_extend(to_dev(co), K, N, shift))
    w_n = pow(7, (P - 1) // N, P)
    for r in range(3):
        for j in (0, 1, 5, 64, 127):
            x = shift * pow(w_n, j, P) % P
            acc = 0
            for c in reversed([int(v) for v in co[r]]):
                acc = (acc * x + c) % P
            assert int(got[r, j]) == acc


def test_many_rows_cross_chunk_boundaries(cp):
    """More rows than one workspace chunk holds, with a row pitch above K for the messages."""
    K, N, m = 1 << 12, 1 << 14, 5000
    big = rand_field((m, K + 8), 5)
    dev = to_dev(big)
    view = dev.view(torch.int64)[:, :K].view(torch.uint64)
    co, code = cp.coset_lde_with_coeffs(view, K, N, 7)
    rows = [0, 1, 1279, 1280, 2500, 4999]
    sub = np.ascontiguousarray(big[rows, :K])
    assert np.array_equal(to_np(co)[rows], O.ntt_rows(sub, inverse=True))
    assert np.array_equal(to_np(code)[rows], O.coset_lde_rows(sub, K, N, 7))
    assert torch.equal(code, cp.coset_lde(view, K, N, 7))


@pytest.mark.parametrize("ELL,K,N,m,row_offset", [(12, 16, 32, 5, 0), (48, 64, 256, 33, 100), (3000, 4096, 8192, 6, 7),
                                                  (8192, 1 << 14, 1 << 16, 3, 58000), (64, 64, 128, 4, 0)])
def test_encode_messages_matches_recipe(cp, ELL, K, N, m, row_offset):
    from verinf_amd.prover import core
    cfg = core.LigeroConfig(ELL=ELL, K_DEG=K, N_LIG=N, T_QUERIES=1)
    msgs = rand_field((m, ELL), ELL + m)
    polys, code = core.encode_messages(to_dev(msgs), cfg, master_seed=_seed_dev(), row_offset=row_offset)
    padded = np.zeros((m, K), dtype=np.uint64)
    padded[:, :ELL] = msgs
    if K > ELL:
        padded[:, ELL:] = O.row_prg(SEED, row_offset, m, K - ELL)
    assert np.array_equal(to_np(polys), O.ntt_rows(padded, inverse=True))
    assert np.array_equal(to_np(code), O.coset_lde_rows(padded, K, N, 7))
    polys2, none = core.encode_messages(to_dev(msgs), cfg, master_seed=_seed_dev(), row_offset=row_offset,
                                        need_codewords=False)
    assert none is None and torch.equal(polys2, polys)
    assert torch.equal(core._coset_encode_codewords(polys, cfg), code)
    # the row polynomial interpolates the message: Horner at zeta_c = w_K^c returns slot c
    w_k = cfg.W_K
    co = [int(v) for v in to_np(polys)[0]]
    for c in (0, 1, ELL - 1):
        x, acc = pow(w_k, c, P), 0
        for v in reversed(co):
            acc = (acc * x + v) % P
        assert acc == int(msgs[0, c])


def test_encode_messages_empty_and_small_pad_warning(cp):
    from verinf_amd.prover import core
    cfg = core.LigeroConfig(ELL=60, K_DEG=64, N_LIG=128, T_QUERIES=8)
    polys, code = core.encode_messages(torch.empty((0, 60), dtype=torch.uint64, device="cuda"), cfg, master_seed=_seed_dev())
    assert tuple(polys.shape) == (0, 64) and tuple(code.shape) == (0, 128)
    with pytest.warns(UserWarning):
        core.encode_messages(to_dev(rand_field((2, 60), 1)), cfg, master_seed=_seed_dev())


def test_commit_phase_integration_production_geometry(cp):
    """The commit pipeline at ELL = 8192, K = 2^14, N = 2^16 with m = 64 rows, as the
    reference's integration smoke does (prover/tests/test_cuda_primitives.py:432-453):
    encode, hash the columns, build the tree -- here also checked end to end: codeword rows
    and column digests against the oracle, the streamed accumulator against the one-shot
    hash, and an opening path with the host verifier."""
    import random
    from verinf_amd.prover import core
    from verinf_amd.prover.protocol import merkle_leaf, merkle_verify
    ELL, K, N, m = 8192, 1 << 14, 1 << 16, 64
    msgs = np.zeros((m, K), dtype=np.uint64)
    msgs[:, :ELL] = rand_field((m, ELL), 80)
    dev = to_dev(msgs)
    code = cp.rs_encode_rows(dev, n_lig=N, k_deg=K)
    dig = cp.hash_columns_streamed(code)
    root, levels = cp.merkle_build_blake3(dig)
    assert tuple(code.shape) == (m, N) and tuple(dig.shape) == (N, 32) and tuple(root.shape) == (32,)
    host_code = to_np(code)
    assert np.array_equal(host_code[[0, 31, 63]], O.coset_lde_rows(msgs[[0, 31, 63]], K, N, 1))
    cols = [0, 1, 4097, N - 1]
    assert np.array_equal(to_np(dig)[cols], O.hash_columns(np.ascontiguousarray(host_code[:, cols])))
    want_levels = O.merkle_levels(to_np(dig))
    assert to_np(root).tobytes() == want_levels[-1][0].tobytes()
    # the same matrix through the ZK recipe in three slabs with the streaming accumulator
    cfg = core.LigeroConfig(ELL=ELL, K_DEG=K, N_LIG=N, T_QUERIES=189)
    seed = _seed_dev()
    big = rand_field((300, ELL), 81)
    acc = cp.MerkleColumnAccumulator(N, 300)
    chunks = []
    for lo, hi in ((0, 100), (100, 228), (228, 300)):
        polys, cw = core.encode_messages(to_dev(big[lo:hi]), cfg, master_seed=seed, row_offset=lo)
        assert tuple(polys.shape) == (hi - lo, K)
        acc.update(cw)
        chunks.append(cw)
    dig2 = acc.finalize()
    whole = torch.cat([c.view(torch.int64) for c in chunks]).view(torch.uint64)
    assert torch.equal(dig2, cp.hash_columns_streamed(whole))
    # chunked encoding with row offsets equals one call over all rows
    _, cw_all = core.encode_messages(to_dev(big), cfg, master_seed=seed, row_offset=0)
    assert torch.equal(cw_all, whole)
    root2, levels2 = cp.merkle_build_blake3(dig2)
    from verinf_amd.layergkr import gpu as lg, rs
    host_levels = lg.levels_to_host(levels2)
    col = random.Random(5).randrange(N)
    values = lg.column(whole, col)
    path = rs.merkle_path(host_levels, col)
    assert merkle_verify(merkle_leaf(values), path, bytes(root2.cpu().tolist()))

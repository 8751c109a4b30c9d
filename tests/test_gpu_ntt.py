"""GPU parity: batched NTT and coset LDE through the C ABI vs the oracle (bit-exact)."""
import json
import os
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, rand_field_dev, to_dev, to_np, unhex  # noqa: E402


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def test_ntt_golden_1024(cp, golden_dir):
    g = json.load(open(os.path.join(golden_dir, "ntt_1024.json")))
    x = to_dev(unhex(g["input"]))
    cp.ntt_forward(x)
    assert np.array_equal(to_np(x), unhex(g["forward"]))
    cp.ntt_inverse(x)
    assert np.array_equal(to_np(x), unhex(g["input"]))


@pytest.mark.parametrize("n", [2, 4, 16, 64, 1024])
def test_ntt_small_sizes_match_definition(cp, n):
    """Sizes of the reference's own small-size test (test_cuda_primitives.py:123-131), seed 10."""
    rng = random.Random(10)
    x_cpu = [rng.randrange(P) for _ in range(n)]
    x = to_dev(np.array(x_cpu, dtype=np.uint64))
    cp.ntt_forward(x)
    want = O.py_dft(x_cpu) if n <= 64 else O.dft_naive(np.array(x_cpu, dtype=np.uint64)).tolist()
    assert to_np(x).tolist() == want


@pytest.mark.parametrize("logn,m", [(1, 5), (3, 1000), (5, 77), (8, 33), (9, 9), (10, 6), (11, 5), (12, 16), (13, 3),
                                    (14, 8), (15, 8), (16, 8), (17, 2), (18, 3), (20, 2),
                                    (10, 1), (10, 1023), (11, 1), (11, 514), (12, 1), (12, 257),
                                    (5, 128), (5, 1280), (6, 64), (7, 32), (8, 16), (8, 4096), (9, 8), (9, 1032)])
def test_batched_ntt_matches_oracle(cp, logn, m):
    a = rand_field((m, 1 << logn), 100 + logn)
    rows = to_dev(a)
    cp.ntt_forward_batched(rows)
    assert np.array_equal(to_np(rows), O.ntt_rows(a))
    cp.ntt_inverse_batched(rows)
    assert np.array_equal(to_np(rows), a)


_SWITCHED_OFF = """
import numpy as np
from oracle import oracle as O
from tests.gpu_util import rand_field, to_dev, to_np
from verinf_amd.prover import cuda_primitives as cp
for logn, m in ((10, 6), (11, 3), (12, 5)):
    a = rand_field((m, 1 << logn), 500 + logn)
    rows = to_dev(a)
    cp.ntt_forward_batched(rows)
    assert np.array_equal(to_np(rows), O.ntt_rows(a)), logn
    cp.ntt_inverse_batched(rows)
    assert np.array_equal(to_np(rows), a), logn
for logK, m in ((12, 5), (16, 2)):
    a = rand_field((m, 1 << logK), 600 + logK)
    got = to_np(cp.coset_lde(to_dev(a), 1 << logK, 4 << logK))
    assert np.array_equal(got, O.coset_lde_rows(a, 1 << logK, 4 << logK)), logK
print("switched-off paths agree")
"""


def test_the_schedules_the_environment_switches_select():
    """VI_NTT_ROW=0 (rows of 2^10 .. 2^12 points as two passes through a workspace) and VI_LDE_MERGED=0 (the coset
    factors applied whole in the fused launch) are read once per process, so they are set for a child process,
    which compares both schedules with the oracle; this process runs the default ones."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, VI_NTT_ROW="0", VI_LDE_MERGED="0")
    res = subprocess.run([sys.executable, "-c", _SWITCHED_OFF], cwd=root, env=env, capture_output=True, text=True,
                         timeout=280)
    assert res.returncode == 0 and "switched-off paths agree" in res.stdout, res.stdout + res.stderr


def test_config1_plumbing(cp):
    """The small plumbing workload: 16 x 2^12 (seed 0), forward, inverse, then LDE to 2^14 with shift 7."""
    a = rand_field((16, 1 << 12), 0)
    rows = to_dev(a)
    cp.ntt_forward_batched(rows)
    fwd = to_np(rows)
    assert np.array_equal(fwd, O.ntt_rows(a))
    assert np.array_equal(fwd[3], O.dft_naive(a[3]))
    cp.ntt_inverse_batched(rows)
    assert np.array_equal(to_np(rows), a)
    cw = cp.coset_lde(rows, 1 << 12, 1 << 14, 7)
    assert np.array_equal(to_np(cw), O.coset_lde_rows(a, 1 << 12, 1 << 14, 7))


def test_batched_equals_single_and_roundtrip_at_production_sizes(cp):
    """test_cuda_primitives.py:150-188 shape: batched == per-row, inverse restores."""
    for n in (16384, 32768, 65536):
        a = rand_field((8, n), n)
        rows = to_dev(a)
        cp.ntt_forward_batched(rows)
        for i in (0, 7):
            single = to_dev(a[i].copy())
            cp.ntt_forward(single)
            assert torch.equal(single, rows[i])
        cp.ntt_inverse_batched(rows)
        assert np.array_equal(to_np(rows), a)


def test_ntt_invariants_large(cp):
    """Size-independent properties at 2^22 (three passes): delta -> ones, constant ->
    n*delta, linearity, round trip."""
    n = 1 << 22
    d = torch.zeros(n, dtype=torch.int64, device="cuda")
    d[0] = 1
    d = d.view(torch.uint64)
    cp.ntt_forward(d)
    assert bool((d.view(torch.int64) == 1).all())
    c = torch.full((n,), 5, dtype=torch.int64, device="cuda").view(torch.uint64)
    cp.ntt_forward(c)
    ci = c.view(torch.int64)
    assert int(ci[0].item()) == 5 * n and not bool(ci[1:].any())
    a, b = rand_field(n, 1), rand_field(n, 2)
    da, db = to_dev(a), to_dev(b)
    s = cp.gl_add(da, db)
    cp.ntt_forward(da)
    cp.ntt_forward(db)
    cp.ntt_forward(s)
    assert torch.equal(s, cp.gl_add(da, db))
    cp.ntt_inverse(da)
    assert np.array_equal(to_np(da), a)


def test_poly_mul_is_a_convolution(cp):
    r = random.Random(30)
    for la, lb in [(1, 1), (3, 5), (16, 16), (256, 256)]:
        a = [r.randrange(P) for _ in range(la)]
        b = [r.randrange(P) for _ in range(lb)]
        want = [0] * (la + lb - 1)
        for i, x in enumerate(a):
            for j, y in enumerate(b):
                want[i + j] = (want[i + j] + x * y) % P
        got = cp.poly_mul(to_dev(np.array(a, dtype=np.uint64)), to_dev(np.array(b, dtype=np.uint64)))
        assert to_np(got).tolist() == want
    A, B = rand_field((5, 16), 31), rand_field((5, 16), 32)
    got = to_np(cp.poly_mul_batched(to_dev(A), to_dev(B)))
    for i in range(5):
        single = cp.poly_mul(to_dev(A[i].copy()), to_dev(B[i].copy()))
        assert np.array_equal(got[i], to_np(single))
    s = cp.poly_add(to_dev(A[0, :5].copy()), to_dev(B[0, :9].copy()))
    assert to_np(s).tolist() == [(int(A[0, i]) if i < 5 else 0) + int(B[0, i]) - (P if (int(A[0, i]) if i < 5 else 0) + int(B[0, i]) >= P else 0) for i in range(9)]


# ---------------------------------------------------------------- coset LDE ----
def test_lde_golden(cp, golden_dir):
    for g in json.load(open(os.path.join(golden_dir, "coset_lde.json"))):
        msgs = np.stack([unhex(m) for m in g["messages"]])
        want = np.stack([unhex(c) for c in g["codewords"]])
        got = cp.coset_lde(to_dev(msgs), g["K"], g["N"], g["shift"])
        assert np.array_equal(to_np(got), want), (g["K"], g["N"])


@pytest.mark.parametrize("logK,logN,m,w", [(1, 1, 3, 2), (1, 3, 3, 1), (3, 5, 700, 8), (5, 6, 4, 16), (7, 8, 9, 64),
                                           (9, 10, 3, 256), (10, 10, 3, 1000), (10, 12, 7, 1024), (11, 13, 3, 2000), (4, 7, 5, 11), (12, 14, 16, 4096),
                                           (13, 15, 5, 5000), (14, 16, 9, 8192), (16, 18, 5, 65536),
                                           (16, 17, 3, 40000), (17, 19, 2, 1 << 17), (18, 20, 2, 200000), (20, 22, 1, 1 << 20),
                                           (8, 14, 3, 256), (12, 18, 2, 4000),
                                           # rows at most half as wide as the transform (the first pass skips the zero
                                           # half), with and without a partly filled plane; rate 1/2 in the fused launch
                                           (14, 16, 3, 2816), (14, 16, 2, 4096), (16, 18, 2, 4097), (16, 18, 1, 32768),
                                           (12, 13, 3, 2048), (14, 15, 2, 16384), (13, 15, 2, 2048)])
def test_lde_matches_oracle(cp, logK, logN, m, w):
    msgs = rand_field((m, w), 200 + logK)
    got = cp.coset_lde(to_dev(msgs), 1 << logK, 1 << logN, 7)
    assert np.array_equal(to_np(got), O.coset_lde_rows(msgs, 1 << logK, 1 << logN, 7))


def test_lde_strided_rows_other_shift_and_legacy_encoder(cp):
    big = rand_field((6, 100), 9)
    view = to_dev(big)[:, :40]
    got = cp.coset_lde(view, 64, 256, 11)
    assert np.array_equal(to_np(got), O.coset_lde_rows(np.ascontiguousarray(big[:, :40]), 64, 256, 11))
    # rs_encode_rows = iNTT_K, zero-extend, NTT_N without a coset (test_cuda_primitives.py:195-214)
    msgs = rand_field((16, 8), 20)
    out = cp.rs_encode_rows(to_dev(msgs), n_lig=32, k_deg=8)
    want = np.zeros((16, 32), dtype=np.uint64)
    want[:, :8] = O.ntt_rows(msgs, inverse=True)
    assert np.array_equal(to_np(out), O.ntt_rows(want))
    empty = cp.coset_lde(torch.empty((0, 8), dtype=torch.uint64, device="cuda"), 8, 32)
    assert tuple(empty.shape) == (0, 32)


def test_lde_small_workspace_chunks_are_bit_identical(cp):
    """Forcing the library to process the rows in several chunks changes nothing."""
    from verinf_amd import _lib
    L = _lib.lib()
    K, N, m = 1 << 14, 1 << 16, 37
    msgs = rand_field((m, K), 77)
    d = to_dev(msgs)
    full = cp.coset_lde(d, K, N, 7)
    out = torch.empty((m, N), dtype=torch.uint64, device="cuda")
    one = L.vi_coset_lde_min_workspace_bytes(K, N)
    ws = torch.empty(one * 5 + 8, dtype=torch.uint8, device="cuda")       # 5 rows per chunk
    _lib.check(L.vi_coset_lde(d.data_ptr(), m, K, K, K, N, 7, out.data_ptr(), N, ws.data_ptr(), ws.numel(),
                              _lib.stream_ptr()))
    assert torch.equal(full, out)
    assert np.array_equal(to_np(out), O.coset_lde_rows(msgs, K, N, 7))
    rc = L.vi_coset_lde(d.data_ptr(), m, K, K, K, N, 7, out.data_ptr(), N, ws.data_ptr(), one - 8, _lib.stream_ptr())
    assert rc == -3 and b"workspace" in L.vi_last_error()


def test_lde_of_the_empty_message_through_the_c_abi():
    """width = 0 (no source word exists, the pointer may be null): codewords and coefficients are zero,
    written with the caller's row pitches; the slack beyond a row is left alone."""
    from verinf_amd import _lib
    L = _lib.lib()
    K, N, m = 1 << 10, 1 << 12, 3
    out = torch.full((m, N + 5), 7, dtype=torch.int64, device="cuda").view(torch.uint64)
    coeffs = torch.full((m, K + 2), 9, dtype=torch.int64, device="cuda").view(torch.uint64)
    ws = torch.empty(L.vi_coset_lde_min_workspace_bytes(K, N) * m, dtype=torch.uint8, device="cuda")
    _lib.check(L.vi_coset_lde_coeffs(None, m, 0, 0, K, N, 7, coeffs.data_ptr(), K + 2, out.data_ptr(), N + 5,
                                     ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    o, c = to_np(out), to_np(coeffs)
    assert (o[:, :N] == 0).all() and (o[:, N:] == 7).all()
    assert (c[:, :K] == 0).all() and (c[:, K:] == 9).all()
    out2 = torch.full((m, N), 5, dtype=torch.int64, device="cuda").view(torch.uint64)
    _lib.check(L.vi_coset_lde(None, m, 0, 0, K, N, 7, out2.data_ptr(), N, ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    assert int(out2.view(torch.int64).abs().sum().item()) == 0


def test_lde_gates_and_layergkr_entry_points():
    from verinf_amd.layergkr import gpu, rs
    for cfg in (rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4),
                rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8),
                rs.Config(ELL=256, K_DEG=512, N_LIG=1024, T_QUERIES=8)):
        assert gpu.selftest_ntt(cfg, n_rows=2) is None
        assert rs._ntt_ok(cfg)
    big = rs.Config(ELL=8192, K_DEG=16384, N_LIG=65536, T_QUERIES=80)
    assert gpu.selftest_ntt_spot(big, n_cols=6) is None
    # chunked == unchunked, and a row count past the reference's grid cap completes
    cfg = rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8)
    msgs = rand_field_dev((300, cfg.ELL), 3)                # uniform in [0, p)
    ref = gpu.encode_batch_ntt(cfg, msgs).clone()
    saved = gpu.MAX_GRID_ROWS
    try:
        gpu.MAX_GRID_ROWS = 37
        assert torch.equal(ref, gpu.encode_batch_ntt(cfg, msgs))
    finally:
        gpu.MAX_GRID_ROWS = saved
    assert np.array_equal(to_np(ref), O.coset_lde_rows(to_np(msgs), 128, 256, 7))
    wide = rs.Config(ELL=256, K_DEG=512, N_LIG=1024, T_QUERIES=8)
    out = gpu.encode_batch_ntt(wide, torch.zeros((65535 + 65, wide.ELL), dtype=torch.uint64, device="cuda"))
    assert tuple(out.shape) == (65535 + 65, 1024) and not bool(out.view(torch.int64).any())
    # Python rows in, ragged lengths
    r = random.Random(2)
    rows = [[r.randrange(P) for _ in range(k)] for k in (64, 3, 0, 17)]
    got = to_np(gpu.encode_batch_ntt(cfg, rows))
    pad = np.zeros((4, 64), dtype=np.uint64)
    for i, row in enumerate(rows):
        pad[i, :len(row)] = row
    assert np.array_equal(got, O.coset_lde_rows(pad, 128, 256, 7))
    c = rs.Commit.from_messages(cfg, rows)
    assert c.n_rows == 4 and c.col_values(5) == [int(v) for v in got[:, 5]]


def test_dense_backend_gate_of_rs_at_the_reference_geometries():
    """rs._gpu_ok opens only after gpu.selftest agrees with the definition (layergkr/tests/test_gpu.py:21-23,
    66-82), and the host and device linear combinations agree."""
    from verinf_amd.layergkr import gpu, rs
    configs = [rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4), rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8),
               rs.Config(ELL=256, K_DEG=512, N_LIG=1024, T_QUERIES=8)]
    cfg = configs[1]
    rs._GPU_OK.clear()
    assert rs._gpu_ok(cfg) is True
    assert (cfg.ELL, cfg.K_DEG, cfg.N_LIG) in rs._GPU_OK
    assert rs._gpu_ok(configs[0]) is True
    r = random.Random(5)
    cw = [rs.encode_row(cfg, [r.randrange(P) for _ in range(cfg.ELL)]) for _ in range(6)]
    co = [r.randrange(P) for _ in range(6)]
    assert rs.linear_combination(cfg, cw, co) == gpu.linear_combination(cfg, cw, co)
    cols = rs.sample_columns(b"seed", cfg.T_QUERIES, cfg.N_LIG)
    c = rs.Commit.from_messages(cfg, [[r.randrange(P) for _ in range(cfg.ELL)] for _ in range(3)])
    for col in cols:
        vals, path = c.open(col)
        assert c.check_open(col, vals, path)


def test_dense_lagrange_encoder_and_its_gate():
    """The reference's dense encoder surface (layergkr/gpu.py:80-122, 256-271, 413-434; rs.py:66-77): the matrix
    against the closed form in Python integers, the matmul encoder against the NTT encoder, the gate green."""
    from verinf_amd.layergkr import gpu, rs
    from verinf_amd.prover.protocol import lagrange
    r = random.Random(8)
    for cfg in (rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4), rs.Config(ELL=64, K_DEG=128, N_LIG=256, T_QUERIES=8)):
        assert gpu.selftest(cfg, n_rows=2) is None
        L = rs.lagrange_matrix(cfg)
        assert len(L) == cfg.N_LIG and len(L[0]) == cfg.ELL
        for _ in range(40):
            j, c = r.randrange(cfg.N_LIG), r.randrange(cfg.ELL)
            assert L[j][c] == lagrange(cfg, c, cfg.eta(j))
        rows = [[r.randrange(P) for _ in range(k)] for k in (cfg.ELL, 5, 0)]
        dense = gpu.encode_batch_t(cfg, rows)
        assert torch.equal(dense, gpu.encode_batch_ntt(cfg, rows))
        assert gpu.encode_batch(cfg, rows) == [[int(v) for v in row] for row in to_np(dense)]


def test_lde_full_baseline_shape_properties(cp):
    """The headline LDE shape (1024 x 2^16 -> 2^18): all 1024 rows bit-exact against the oracle, and the codeword
    property (inverse transform has no coefficient >= K) on all rows."""
    K, N, m = 1 << 16, 1 << 18, 1024
    msgs = rand_field_dev((m, K), 2)                     # uniform in [0, p), words above 2^63 included
    assert int((msgs.view(torch.int64) < 0).sum()) > m * K // 4
    out = cp.coset_lde(msgs, K, N, 7)
    host = to_np(msgs)
    for lo in range(0, m, 256):                          # 512 MiB of codewords per slice on the host
        want = O.coset_lde_rows(host[lo:lo + 256], K, N, 7)
        assert np.array_equal(to_np(out[lo:lo + 256]), want), lo
        del want
    for lo in range(0, m, 256):
        blk = out[lo:lo + 256].clone()
        cp.ntt_inverse_batched(blk)
        assert not bool(blk.view(torch.int64)[:, K:].any())
    del out


def test_two_host_threads_on_their_own_streams(cp):
    """The library keeps per-device table caches behind a mutex and no other shared state: two
    host threads, each with its own stream and workspace, transform different data at the same
    time (first use of two table sizes included) and both results are bit-exact."""
    import threading
    from verinf_amd import _lib
    L = _lib.lib()
    jobs = [(1 << 11, 1 << 13, 300, 31), (1 << 15, 1 << 17, 40, 32)]       # sizes no other test has warmed up
    results, errors = {}, []

    def work(i, K, N, m, seed):
        try:
            st = torch.cuda.Stream()
            msgs = rand_field((m, K), seed)
            with torch.cuda.stream(st):
                dev = to_dev(msgs)
                out = torch.empty((m, N), dtype=torch.uint64, device="cuda")
                ws = torch.empty(L.vi_coset_lde_workspace_bytes(m, K, N), dtype=torch.uint8, device="cuda")
                for _ in range(3):
                    _lib.check(L.vi_coset_lde(dev.data_ptr(), m, K, K, K, N, 7, out.data_ptr(), N, ws.data_ptr(),
                                              ws.numel(), st.cuda_stream))
                st.synchronize()
                results[i] = (msgs, to_np(out), K, N)
        except Exception as exc:            # surfaced in the main thread
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,) + j) for i, j in enumerate(jobs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for msgs, got, K, N in results.values():
        rows = [0, msgs.shape[0] - 1]
        assert np.array_equal(got[rows], O.coset_lde_rows(np.ascontiguousarray(msgs[rows]), K, N, 7))

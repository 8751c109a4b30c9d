"""Runs the HIP kernels' pass logic (index maps, twiddle tables, pass sequencing,
field arithmetic) as a CPU build and checks it bit-for-bit against the oracle.
No GPU needed: this is how the kernels' addressing is validated before launch."""
import ctypes
import os
import random
import subprocess
from ctypes import POINTER, c_int, c_long, c_uint, c_uint64

import numpy as np
import pytest

from oracle import oracle as O

P = O.P
HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "cpu_build", "emul_ntt.cpp")
SO = os.path.join(HERE, "cpu_build", "libemul_ntt.so")


@pytest.fixture(scope="module")
def emu():
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-o", SO, SRC])
    L = ctypes.CDLL(SO)
    u64p = POINTER(c_uint64)
    for f in (L.emu_mul, L.emu_add, L.emu_sub):
        f.restype = c_uint64
        f.argtypes = [c_uint64, c_uint64]
    L.emu_mul_pow2.restype = c_uint64
    L.emu_inv.restype = c_uint64
    L.emu_inv.argtypes = [c_uint64]
    L.emu_mul_pow2.argtypes = [c_uint64, c_uint]
    L.emu_set_fast.argtypes = [c_int]
    L.emu_set_uniform.argtypes = [c_int]
    L.emu_set_fusion.argtypes = [c_int]
    L.emu_set_merged.argtypes = [c_int]
    L.emu_merged_runs.restype = c_long
    L.emu_set_half.argtypes = [c_int]
    L.emu_half_runs.restype = c_long
    L.emu_single_uniform_runs.restype = c_long
    L.emu_set_row.argtypes = [c_int]
    L.emu_row_runs.restype = c_long
    L.emu_ntt_batched.argtypes = [u64p, c_long, c_int, c_int]
    L.emu_coset_lde.argtypes = [u64p, c_long, c_long, c_long, c_int, c_int, c_uint64, u64p]
    L.emu_coset_lde_ex.argtypes = [u64p, c_long, c_long, c_long, c_int, c_int, c_uint64, u64p, c_long, u64p, c_int]
    return L


# (register-blocked passes, scalar-base addressing, fused middle launch of the LDE, coset factors split into shifts
# and per-coset twiddle tables inside that launch): every way a pass can run
MODES = ((1, 1, 1, 1), (1, 1, 1, 0), (1, 1, 0, 0), (1, 0, 0, 0), (0, 0, 0, 0))


def _set_mode(emu, fast, uni, fuse, merged):
    emu.emu_set_fast(fast)
    emu.emu_set_uniform(uni)
    emu.emu_set_fusion(fuse)
    emu.emu_set_merged(merged)


def _p(a):
    return a.ctypes.data_as(POINTER(c_uint64))


def _rand(shape, seed):
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 1 << 63, size=shape, dtype=np.uint64) * 2 + rng.integers(0, 2, size=shape, dtype=np.uint64)
    return a % np.uint64(P)


def test_device_field_functions(emu):
    r = random.Random(1)
    edge = [0, 1, P - 1, P - 2, (1 << 32) - 1, 1 << 32, (1 << 32) + 1, 1 << 63, 0xFFFFFFFF00000000,
            P, P + 5, (1 << 64) - 1]                       # includes non-canonical words
    vals = edge + [r.randrange(1 << 64) for _ in range(300)]
    L = O.lib()
    for a in vals:
        for b in vals[:40]:
            assert emu.emu_mul(a, b) == L.vo_mul(a, b)
            assert emu.emu_add(a, b) == L.vo_add(a, b)
            assert emu.emu_sub(a, b) == L.vo_sub(a, b)
    for a in edge[:9] + [r.randrange(P) for _ in range(100)]:
        for s in range(96):
            assert emu.emu_mul_pow2(a, s) == a * (1 << s) % P, (a, s)


def test_device_inverse_chain(emu):
    """The fixed addition chain for x^(p-2): x * inv(x) = 1, inv(0) = 0, non-canonical words
    invert as their residues."""
    rng = random.Random(4)
    for x in [1, 2, P - 1, P - 2, 1 << 32, (1 << 32) - 1, 7] + [rng.randrange(1, P) for _ in range(200)]:
        assert emu.emu_inv(x) == pow(x, P - 2, P), x
    assert emu.emu_inv(0) == 0
    assert emu.emu_inv(P) == 0
    assert emu.emu_inv(P + 5) == pow(5, P - 2, P)


@pytest.mark.parametrize("logn,m", [(1, 3), (2, 5), (4, 300), (5, 9), (6, 7), (7, 70), (8, 33), (9, 6), (10, 5), (11, 4), (12, 3),
                                    (13, 2), (14, 3), (15, 2), (16, 2), (17, 1), (18, 1), (19, 1)])
def test_ntt_passes_match_oracle(emu, logn, m):
    a = _rand((m, 1 << logn), 100 + logn)
    want = O.ntt_rows(a)
    # register-blocked passes with scalar-base and with per-element addressing, then the generic radix-2 passes
    for mode in MODES:
        _set_mode(emu, *mode)
        got = a.copy()
        emu.emu_ntt_batched(_p(got), m, logn, 0)
        assert np.array_equal(got, want), mode
        emu.emu_ntt_batched(_p(got), m, logn, 1)
        assert np.array_equal(got, a), mode
    _set_mode(emu, 1, 1, 1, 1)


@pytest.mark.parametrize("logn,m", [(10, 1), (10, 4), (10, 7), (11, 1), (11, 3), (11, 8), (12, 1), (12, 2), (12, 5)])
def test_short_rows_in_one_launch(emu, logn, m):
    """Rows of 2^10 .. 2^12 points run as one launch (first digit, exchange through LDS, last digit) and as the two
    passes longer rows take: both against the oracle, with row counts that fill the last tile and that do not, and
    with words at and above p in the input (reduced on load)."""
    a = _rand((m, 1 << logn), 900 + 13 * logn + m)
    raw = a.copy()
    raw[0, :5] = np.array([P, P + 1, (1 << 64) - 1, P - 1, 0], dtype=np.uint64)
    a[0, :5] = raw[0, :5] % np.uint64(P)
    want = O.ntt_rows(a)
    _set_mode(emu, 1, 1, 1, 1)
    for row in (1, 0):
        emu.emu_set_row(row)
        before = emu.emu_row_runs()
        got = raw.copy()
        assert emu.emu_ntt_batched(_p(got), m, logn, 0) == (1 if row else 2)
        assert np.array_equal(got, want), row
        emu.emu_ntt_batched(_p(got), m, logn, 1)
        assert np.array_equal(got, a), row
        assert emu.emu_row_runs() - before == (2 if row else 0)
    emu.emu_set_row(1)
    # lengths on either side keep their own schedule
    for other in (9, 13):
        before = emu.emu_row_runs()
        b = _rand((2, 1 << other), 7)
        emu.emu_ntt_batched(_p(b), 2, other, 0)
        assert emu.emu_row_runs() == before


@pytest.mark.parametrize("logn,m,whole", [(5, 128, True), (5, 256, True), (5, 129, False), (6, 64, True), (7, 32, True), (7, 96, True),
                                          (8, 16, True), (8, 48, True), (8, 17, False), (9, 8, True), (9, 24, True), (9, 9, False)])
def test_single_pass_rows_in_whole_tiles(emu, logn, m, whole):
    """A transform of at most 512 points is one pass over tiles of 4096 / n rows.  When the batch is a whole number of
    tiles (and the rows are contiguous) the tiles are addressed through scalar bases; a batch that is not keeps the
    per-element path.  Both against the oracle, forward and inverse, with words at and above p in the input."""
    a = _rand((m, 1 << logn), 1300 + 17 * logn + m)
    raw = a.copy()
    raw[m - 1, -3:] = np.array([P, P + 7, (1 << 64) - 1], dtype=np.uint64)
    a[m - 1, -3:] = raw[m - 1, -3:] % np.uint64(P)
    want = O.ntt_rows(a)
    for uni in (1, 0):
        _set_mode(emu, 1, uni, 1, 1)
        before = emu.emu_single_uniform_runs()
        got = raw.copy()
        emu.emu_ntt_batched(_p(got), m, logn, 0)
        assert np.array_equal(got, want), uni
        emu.emu_ntt_batched(_p(got), m, logn, 1)
        assert np.array_equal(got, a), uni
        assert emu.emu_single_uniform_runs() - before == (2 if (uni and whole) else 0)
    _set_mode(emu, 1, 1, 1, 1)


def test_ntt_25_bit_split_is_well_formed(emu):
    """Digit split for sizes beyond three passes (no transform is run)."""
    # 2^25 needs four digits; only checked structurally through a tiny proxy: 2^17 = 6+6+5
    a = _rand((1, 1 << 17), 7)
    got = a.copy()
    emu.emu_ntt_batched(_p(got), 1, 17, 0)
    assert np.array_equal(got, O.ntt_rows(a))


@pytest.mark.parametrize("logK,logN,m,w", [(5, 6, 4, 16), (7, 8, 9, 64), (9, 10, 3, 256), (3, 5, 700, 8),
                                           (12, 14, 2, 4096), (13, 15, 2, 5000), (14, 16, 1, 8192),
                                           (16, 18, 1, 65536), (10, 10, 3, 1000), (4, 7, 5, 11),
                                           (10, 12, 5, 1024), (11, 13, 3, 2000), (11, 12, 2, 2048),
                                           (14, 16, 2, 2816), (12, 14, 3, 257), (16, 18, 1, 4097), (12, 14, 2, 63),
                                           (10, 11, 3, 1024), (12, 13, 2, 3000), (12, 15, 1, 4096), (14, 15, 1, 16384)])
def test_lde_passes_match_oracle(emu, logK, logN, m, w):
    msgs = _rand((m, w), 200 + logK)
    want = O.coset_lde_rows(msgs, 1 << logK, 1 << logN, 7)
    for mode in MODES:
        _set_mode(emu, *mode)
        before = emu.emu_merged_runs()
        got = np.zeros((m, 1 << logN), dtype=np.uint64)
        emu.emu_coset_lde(_p(msgs), m, w, w, logK, logN, 7, _p(got))
        assert np.array_equal(got, want), mode
        # K = L * L with L >= 64 (a tile then lies inside one row) and rate 1/2 or 1/4: the fused launch runs, and in
        # its split form when allowed
        splits = logK % 2 == 0 and logK >= 12 and 1 <= logN - logK <= 2
        assert (emu.emu_merged_runs() > before) == (splits and mode == (1, 1, 1, 1)), mode
    _set_mode(emu, 1, 1, 1, 1)


def test_lde_strided_input_and_other_shift(emu):
    big = _rand((6, 100), 9)
    want = O.coset_lde_rows(np.ascontiguousarray(big[:, :40]), 64, 256, 11)
    got = np.zeros((6, 256), dtype=np.uint64)
    emu.emu_coset_lde(_p(big), 6, 40, 100, 6, 8, 11, _p(got))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("logK,w,pruned", [(14, 8192, True), (14, 4096, True), (14, 2816, True), (14, 8193, False),
                                           (14, 7000, True), (14, 1024, True), (14, 1000, False), (16, 32768, True),
                                           (16, 32769, False), (16, 100, False), (12, 2048, True), (12, 5, False),
                                           (16, 4097, True), (13, 2048, True), (13, 4097, False)])
def test_lde_of_rows_at_most_half_as_wide_as_the_transform(emu, logK, w, pruned):
    """Source rows that end within the first eight of a thread's sixteen input planes: the first pass does not load
    the zero half and skips the first butterfly level.  Same codewords with and without, and both equal the oracle's;
    the counter says whether the pruned form ran (the width must cover at least one whole plane of K/16 words and end
    within the first eight)."""
    m = 2
    msgs = _rand((m, w), 900 + w)
    want = O.coset_lde_rows(msgs, 1 << logK, 1 << (logK + 2), 7)
    for half in (1, 0):
        emu.emu_set_half(half)
        before = emu.emu_half_runs()
        got = np.zeros((m, 1 << (logK + 2)), dtype=np.uint64)
        emu.emu_coset_lde(_p(msgs), m, w, w, logK, logK + 2, 7, _p(got))
        assert np.array_equal(got, want), half
        assert (emu.emu_half_runs() > before) == bool(half and pruned), (half, emu.emu_half_runs() - before)
    emu.emu_set_half(1)


@pytest.mark.parametrize("logK,logN,m,w", [(5, 6, 4, 16), (9, 10, 3, 256), (12, 14, 2, 4096), (13, 15, 2, 5000),
                                           (14, 16, 1, 8192), (4, 7, 5, 11)])
def test_lde_with_coefficient_output_and_from_coefficients(emu, logK, logN, m, w):
    """The two halves of the pipeline: values -> (coefficients, codewords), coefficients only,
    in place, and coefficients -> codewords."""
    K, N = 1 << logK, 1 << logN
    msgs = _rand((m, w), 300 + logK)
    want = O.coset_lde_rows(msgs, K, N, 7)
    padded = np.zeros((m, K), dtype=np.uint64)
    padded[:, :w] = msgs
    want_c = O.ntt_rows(padded, inverse=True)
    for mode in MODES:
        _set_mode(emu, *mode)
        pitch = K + 3
        co = np.zeros((m, pitch), dtype=np.uint64)
        got = np.zeros((m, N), dtype=np.uint64)
        emu.emu_coset_lde_ex(_p(msgs), m, w, w, logK, logN, 7, _p(co), pitch, _p(got), 0)
        assert np.array_equal(co[:, :K], want_c) and not co[:, K:].any()
        assert np.array_equal(got, want)
        co2 = np.zeros((m, K), dtype=np.uint64)
        emu.emu_coset_lde_ex(_p(msgs), m, w, w, logK, logN, 7, _p(co2), K, None, 0)      # coefficients only
        assert np.array_equal(co2, want_c)
        inpl = padded.copy()
        emu.emu_coset_lde_ex(_p(inpl), m, K, K, logK, logN, 7, _p(inpl), K, None, 0)       # in place
        assert np.array_equal(inpl, want_c)
        got2 = np.zeros((m, N), dtype=np.uint64)
        emu.emu_coset_lde_ex(_p(want_c), m, K, K, logK, logN, 7, None, 0, _p(got2), 1)      # from coefficients
        assert np.array_equal(got2, want)
        # low-degree coefficients: only the first K/2 are given, the rest read as zero
        half = np.ascontiguousarray(want_c[:, : K // 2])
        full = np.zeros((m, K), dtype=np.uint64)
        full[:, : K // 2] = half
        got3 = np.zeros((m, N), dtype=np.uint64)
        emu.emu_coset_lde_ex(_p(half), m, K // 2, K // 2, logK, logN, 7, None, 0, _p(got3), 1)
        got4 = np.zeros((m, N), dtype=np.uint64)
        emu.emu_coset_lde_ex(_p(full), m, K, K, logK, logN, 7, None, 0, _p(got4), 1)
        assert np.array_equal(got3, got4)
    _set_mode(emu, 1, 1, 1, 1)

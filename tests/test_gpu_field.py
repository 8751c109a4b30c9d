"""GPU parity: elementwise field ops through the C ABI vs the oracle (bit-exact)."""
import json
import os
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np, unhex  # noqa: E402


@pytest.fixture(scope="module")
def cp():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import cuda_primitives
    return cuda_primitives


def test_golden_field_vectors(cp, golden_dir):
    vec = json.load(open(os.path.join(golden_dir, "field_vectors.json")))
    a, b = to_dev(unhex([v["a"] for v in vec])), to_dev(unhex([v["b"] for v in vec]))
    assert np.array_equal(to_np(cp.gl_add(a, b)), unhex([v["add"] for v in vec]))
    assert np.array_equal(to_np(cp.gl_sub(a, b)), unhex([v["sub"] for v in vec]))
    assert np.array_equal(to_np(cp.gl_mul(a, b)), unhex([v["mul"] for v in vec]))


@pytest.mark.parametrize("n", [1, 2, 257, 4096, 1000003])
def test_binops_match_oracle(cp, n):
    a, b = rand_field(n, 1), rand_field(n, 2)
    da, db = to_dev(a), to_dev(b)
    for name, fn in (("add", cp.gl_add), ("sub", cp.gl_sub), ("mul", cp.gl_mul)):
        assert np.array_equal(to_np(fn(da, db)), O.binop(name, a, b)), name


def test_binops_on_noncanonical_words_match_reference_formulas(cp):
    """Words >= p: the device functions return the same word as the reference's
    (the oracle restates those formulas), so even these agree bit for bit."""
    r = random.Random(3)
    vals = [P, P + 1, (1 << 64) - 1, (1 << 64) - 2, P - 1, 0, 1] + [r.randrange(1 << 64) for _ in range(500)]
    a = np.array([r.choice(vals) for _ in range(4099)], dtype=np.uint64)
    b = np.array([r.choice(vals) for _ in range(4099)], dtype=np.uint64)
    da, db = to_dev(a), to_dev(b)
    for name, fn in (("add", cp.gl_add), ("sub", cp.gl_sub), ("mul", cp.gl_mul)):
        assert np.array_equal(to_np(fn(da, db)), O.binop(name, a, b)), name


def test_unaligned_views_and_2d_shapes(cp):
    a, b = rand_field(2001, 4), rand_field(2001, 5)
    da, db = to_dev(a)[1:], to_dev(b)[1:]                 # 8-byte aligned only
    assert np.array_equal(to_np(cp.gl_mul(da.contiguous(), db.contiguous())), O.binop("mul", a[1:], b[1:]))
    a2, b2 = rand_field((7, 33), 6), rand_field((7, 33), 7)
    out = cp.gl_add(to_dev(a2), to_dev(b2))
    assert out.shape == (7, 33)
    assert np.array_equal(to_np(out), O.binop("add", a2.reshape(-1), b2.reshape(-1)).reshape(7, 33))


def test_neg_pow_inv_axpy(cp):
    r = random.Random(1)
    a_cpu = [0, 1, P - 1] + [r.randrange(P) for _ in range(254)]
    a = to_dev(np.array(a_cpu, dtype=np.uint64))
    assert to_np(cp.gl_neg(a)).tolist() == [(P - x) % P for x in a_cpu]
    assert to_np(cp.gl_pow(a, 12345)).tolist() == [pow(x, 12345, P) for x in a_cpu]
    assert to_np(cp.gl_pow(a, 0)).tolist() == [1] * len(a_cpu)
    nz = [x for x in a_cpu if x]
    d = to_dev(np.array(nz, dtype=np.uint64))
    want = [pow(x, -1, P) for x in nz]
    assert to_np(cp.gl_inv(d)).tolist() == want
    assert to_np(cp.gl_inv_batched(d)).tolist() == want
    assert torch.equal(cp.gl_mul(d, cp.gl_inv_batched(d)), torch.ones_like(d))
    y_cpu, x_cpu = [r.randrange(P) for _ in range(4096)], [r.randrange(P) for _ in range(4096)]
    alpha = r.randrange(P)
    y, x = to_dev(np.array(y_cpu, dtype=np.uint64)), to_dev(np.array(x_cpu, dtype=np.uint64))
    cp.gl_axpy(y, alpha, x)
    assert to_np(y).tolist() == [(yy + alpha * xx) % P for yy, xx in zip(y_cpu, x_cpu)]


def test_mul_bcast_is_the_expanded_product(cp):
    a, row = rand_field((13, 64), 8), rand_field(64, 9)
    got = cp.gl_mul_bcast(to_dev(a), to_dev(row))
    want = O.binop("mul", a.reshape(-1), np.tile(row, 13)).reshape(13, 64)
    assert np.array_equal(to_np(got), want)


def test_argument_errors_raise_runtime_error(cp):
    a = to_dev(rand_field(8, 1))
    with pytest.raises(RuntimeError):
        cp.gl_mul(a, to_dev(rand_field(9, 1)))
    with pytest.raises(RuntimeError):
        cp.gl_mul(a.cpu(), a.cpu())
    with pytest.raises(RuntimeError):
        cp.gl_add(a, a.view(torch.int64))
    with pytest.raises(RuntimeError):
        cp.gl_add(to_dev(rand_field((4, 4), 1)).view(torch.int64).t().view(torch.uint64), to_dev(rand_field((4, 4), 2)))
    with pytest.raises(RuntimeError):
        cp.gl_inv_batched(to_dev(rand_field((2, 2), 1)))
    with pytest.raises(RuntimeError):
        cp.ntt_forward(to_dev(rand_field(12, 1)))
    with pytest.raises(RuntimeError):
        cp.ntt_forward_batched(to_dev(rand_field(16, 1)))


def test_gl_sum_and_fold_t():
    from verinf_amd.layergkr import gpu
    for n in (1, 2, 3, 255, 4096, 1 << 20, (1 << 20) + 7):
        a = rand_field(n, 10 + n % 7)
        want = int(np.sum(a.astype(object)) % P) if n <= 4096 else sum(int(x) for x in a) % P
        assert int(gpu.gl_sum(to_dev(a)).cpu()[0].item()) == want
    f = rand_field(1 << 12, 11)
    r = 0x123456789ABCDEF1 % P
    got = gpu.fold_t(to_dev(f), torch.tensor([r], dtype=torch.uint64).cuda())
    assert np.array_equal(to_np(got), O.fold(f, r))
    assert np.array_equal(to_np(gpu.fold_t(to_dev(f), r)), O.fold(f, r))


@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 63, 64, 65, 1000, 4099, 1 << 16, (1 << 20) + 3])
def test_inverse_of_arrays_with_zeros_and_ragged_lengths(cp, n):
    """The batched inverse shares one inversion among eight elements: every length class
    (fewer than eight, not a multiple of eight), zeros anywhere (0 -> 0 as the Fermat power
    gives) and non-canonical words."""
    a = rand_field((n,), 40 + n)
    rng = np.random.default_rng(n)
    a[rng.integers(0, n, max(1, n // 50))] = 0
    if n > 4:
        a[3] = np.uint64(P)                          # = 0 mod p
        a[4] = np.uint64(P + 6)                      # = 6 mod p
    got = to_np(cp.gl_inv_batched(to_dev(a)))
    idx = list(range(min(n, 40))) + [int(i) for i in rng.integers(0, n, 60)] + [n - 1]
    for i in idx:
        x = int(a[i]) % P
        assert int(got[i]) == (pow(x, P - 2, P) if x else 0), i
    red = to_dev(a % np.uint64(P))
    prod = to_np(cp.gl_mul(red, to_dev(got)))
    assert np.array_equal(prod, (to_np(red) != 0).astype(np.uint64))


def test_device_field_primitives_one_by_one():
    """The hand-scheduled sequences the transform and sumcheck kernels are built from (modular add, sub, the
    interleaved butterfly, canonicalisation, the product, the 128-bit reduction and all 95 compile-time shift
    twiddles), each on operands chosen around every carry they test: 0, 1, p - 1, p - 2, 2^32 +- 1, 2^63, words whose
    halves are all ones, and random words, in all pairs; against Python integers."""
    from verinf_amd import _lib
    L = _lib.lib()
    r = random.Random(77)
    edge = [0, 1, 2, P - 1, P - 2, P - 3, (1 << 32) - 1, 1 << 32, (1 << 32) + 1, (1 << 63), (1 << 63) - 1,
            0xFFFFFFFF00000000, 0xFFFFFFFEFFFFFFFF, 0x00000001FFFFFFFF, 0x0000000100000000, 0xFFFFFFFE00000001,
            0xFFFFFFFE00000002, 0x8000000080000000, 0x7FFFFFFF7FFFFFFF]
    edge += [(1 << s) % P for s in range(64)] + [((1 << s) - 1) % P for s in range(1, 64)]
    canon = [x % P for x in edge] + [r.randrange(P) for _ in range(200)]
    anyw = canon + [P, P + 1, (1 << 64) - 1, (1 << 64) - 2, P + (1 << 31)] + [r.randrange(1 << 64) for _ in range(100)]

    def run(op, xs, ys):
        a = to_dev(np.array(xs, dtype=np.uint64))
        b = to_dev(np.array(ys, dtype=np.uint64))
        out = torch.empty_like(a)
        _lib.check(L.vi_gl_probe(op, a.data_ptr(), b.data_ptr(), out.data_ptr(), a.numel(), _lib.stream_ptr()))
        return [int(v) for v in to_np(out)]

    xs = [x for x in canon for _ in canon]
    ys = [y for _ in canon for y in canon]
    assert run(0, xs, ys) == [(x + y) % P for x, y in zip(xs, ys)]
    assert run(1, xs, ys) == [(x - y) % P for x, y in zip(xs, ys)]
    assert run(2, xs, ys) == [(x + y) % P for x, y in zip(xs, ys)]
    assert run(3, xs, ys) == [(x - y) % P for x, y in zip(xs, ys)]
    xa = [x for x in anyw for _ in anyw]
    ya = [y for _ in anyw for y in anyw]
    assert run(5, xa, ya) == [x * y % P for x, y in zip(xa, ya)]
    assert run(6, xa, ya) == [((y << 64) + x) % P for x, y in zip(xa, ya)]
    assert run(4, anyw, anyw) == [x % P for x in anyw]
    # the sumcheck passes' own forms: lazily reduced product, fused multiply-add, sums of unreduced products
    M = (1 << 64) - 1
    cs = [(((x << 17) | (x >> 47)) & M) ^ y for x, y in zip(xa, ya)]
    assert run(7, xa, ya) == [x * y % P for x, y in zip(xa, ya)]
    assert run(8, xa, ya) == [(x * y + c) % P for x, y, c in zip(xa, ya, cs)]
    assert run(9, xa, ya) == [(x * y + c) % P for x, y, c in zip(xa, ya, cs)]
    assert run(10, xa, ya) == [(x * y + y * y + x * x + (M - x) * (M - y) + M * M) % P for x, y in zip(xa, ya)]
    assert run(11, xa, ya) == [40 * x * y % P for x, y in zip(xa, ya)]
    for e in range(96):
        assert run(100 + e, canon, canon) == [(x << e) % P for x in canon], e
    for e in range(192):                                   # 2^96 = -1: the upper half are the negated shifts
        assert run(300 + e, canon, canon) == [(x << e) % P for x in canon], e
    with pytest.raises(RuntimeError):
        _lib.check(L.vi_gl_probe(99, 0, 0, 0, 1, None))

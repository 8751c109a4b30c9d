"""GPU parity: sumcheck round kernels through the C ABI vs the oracle (bit-exact
samples per round, challenges, claim) and the host verifier."""
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
def mods():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.layergkr import gpu, sumcheck
    return gpu, sumcheck


def _coins(n, seed):
    r = random.Random(seed)
    vals = [r.randrange(P) for _ in range(n)]
    return vals, (lambda i: vals[i])


def _check(gpu, tables_np, terms_idx, seed, as_tensor):
    """Run the device prover on (tables, terms) and compare with the C oracle."""
    v = tables_np[0].size.bit_length() - 1
    coins, coin = _coins(max(v, 1), seed)
    objs = [to_dev(t) if as_tensor else [int(x) for x in t] for t in tables_np]
    terms = [(c, [objs[i] for i in fs]) for c, fs in terms_idx]
    claim, polys, chals, mu = gpu.prove_terms_gpu(terms, coin, P)
    want_claim, want_samples, _ = O.sumcheck_prove(tables_np, terms_idx, coins)
    assert claim == want_claim
    assert chals == coins[:v]
    assert [[y for _, y in s] for s in polys] == want_samples
    assert all([x for x, _ in s] == list(range(len(s))) for s in polys)
    assert mu == 0
    if as_tensor:
        for t, o in zip(tables_np, objs):
            assert np.array_equal(to_np(o), t), "caller's tensor was modified"
    if v <= 13:
        # the loop that hands every round's samples to the coin (one launch and one host wait per round)
        seen = []

        def coin_with_samples(i, samples):
            seen.append(samples)
            return coins[i]

        assert gpu.prove_terms_gpu_interactive(terms, coin_with_samples, P) == (claim, polys, chals, mu)
        assert seen == polys


def test_sumcheck_golden(mods, golden_dir):
    gpu, _ = mods
    for g in json.load(open(os.path.join(golden_dir, "sumcheck.json"))):
        tables = [[int(x, 16) for x in t] for t in g["tables"]]
        terms = [(int(c, 16), [tables[i] for i in fs]) for c, fs in g["terms"]]
        coins = [int(c, 16) for c in g["coins"]]
        claim, polys, chals, _ = gpu.prove_terms_gpu(terms, lambda i: coins[i], P)
        assert claim == int(g["claim"], 16), g["name"]
        assert [[y for _, y in s] for s in polys] == [[int(x, 16) for x in s] for s in g["samples"]], g["name"]
        assert chals == coins[:len(polys)]


@pytest.mark.parametrize("v", [1, 2, 3, 6, 9, 10, 13, 17])
@pytest.mark.parametrize("nf", [1, 2, 3, 4])
def test_single_product_matches_oracle(mods, v, nf):
    gpu, _ = mods
    tabs = [rand_field(1 << v, 10 * v + j) for j in range(nf)]
    _check(gpu, tabs, [(1, list(range(nf)))], 99, as_tensor=(v % 2 == 1))


def test_sum_of_products_shared_tables_and_coefficients(mods):
    gpu, _ = mods
    r = random.Random(6)
    tabs = [rand_field(1 << 11, 40 + j) for j in range(5)]
    terms = [(r.randrange(P), [0, 1, 2]), (P - 1, [3]), (5, [1, 1]), (7, [0, 3]), (r.randrange(P), [0, 4, 4])]
    _check(gpu, tabs, terms, 7, as_tensor=True)
    _check(gpu, tabs, terms, 8, as_tensor=False)
    # the reference's relation shapes: hadamard a*b - c, booleanity b*b - b, each times eq
    eq, a, b, c = (rand_field(1 << 9, 50 + j) for j in range(4))
    _check(gpu, [eq, a, b, c], [(11, [0, 1, 2]), (P - 11, [0, 3]), (13, [0, 2, 2]), (P - 13, [0, 2])], 9, True)


@pytest.mark.parametrize("name,nt,terms", [
    # every term holds table 0: it is taken out as the common factor
    ("common+products", 5, [(3, [0, 1, 2]), (P - 5, [0, 3, 4]), (7, [1, 0, 4])]),
    # ... and what is left of a term may be one factor (linear part) or nothing (constant part)
    ("common+linear+constant", 4, [(3, [0, 1, 2]), (P - 5, [0, 3]), (9, [0]), (P - 1, [2, 0]), (4, [0])]),
    # the common table twice in one term: only one occurrence leaves the term
    ("common squared", 3, [(6, [0, 0]), (P - 6, [0]), (2, [0, 0, 1]), (5, [2, 0])]),
    # no table in every term: linear and product terms without a common factor
    ("no common", 6, [(3, [0, 1]), (P - 5, [2]), (7, [3]), (11, [4, 5, 0]), (13, [1])]),
    # affine / rescale relations only: every term linear after eq is taken out (layergkr/relations.py:68-82)
    ("all linear", 7, [(3, [0, 1]), (P - 5, [0, 2]), (7, [0, 3]), (P - 1, [0, 4]), (2, [0, 5]), (P - 9, [0, 6])]),
    # only linear terms and no common table: the round polynomial has degree 1
    ("degree one", 3, [(3, [0]), (P - 5, [1]), (7, [2])]),
    # two candidates for the common table
    ("two common", 3, [(3, [0, 1, 2]), (5, [1, 0])]),
    # the first product term's coefficient is divided out of the sum: zero, one and p - 1 as that coefficient
    ("first coefficient zero", 5, [(0, [0, 1, 2]), (5, [0, 3, 4]), (7, [0, 2])]),
    ("first coefficient one", 5, [(1, [0, 1, 2]), (5, [0, 3, 4]), (7, [0, 2]), (9, [0])]),
    ("first coefficient minus one", 5, [(P - 1, [0, 1, 2]), (5, [0, 3, 4]), (7, [0, 2]), (9, [0])]),
    # the hadamard gate batch eq * a * b - eq * c (layergkr/relations.py:104-124) has its own unrolled kernel path:
    # four distinct tables, one product of two and one linear term under a common factor, in any table order
    ("hadamard gate", 4, [(3, [0, 1, 2]), (P - 5, [0, 3])]),
    ("hadamard gate, unit coefficients", 4, [(1, [0, 1, 2]), (P - 1, [0, 3])]),
    ("hadamard gate, other table order", 4, [(P - 5, [2, 1]), (7, [3, 1, 0])]),
    ("hadamard gate, linear term first and zero", 4, [(0, [3, 2]), (9, [1, 3, 0])]),
    # more tables than a thread keeps in registers: the same forms with the factors read from memory
    ("many tables", 11, [(3, [0, 1, 2]), (P - 5, [0, 3]), (7, [0, 4, 5]), (11, [0, 6]), (13, [0, 7, 8]), (17, [0, 9]),
                         (19, [0, 10, 10]), (23, [0])]),
    ("many tables, no common", 10, [(3, [0, 1, 2]), (P - 5, [3]), (7, [4, 5]), (11, [6]), (13, [7, 8, 9, 0])]),
])
@pytest.mark.parametrize("v", [1, 5, 12])
def test_factored_term_forms_match_oracle(mods, name, nt, terms, v):
    """Sums of several terms are evaluated as common * (constant + linear part + products);
    every such form against the oracle, which evaluates the terms as they are written."""
    gpu, _ = mods
    tabs = [rand_field(1 << v, 300 + 7 * v + j) for j in range(nt)]
    _check(gpu, tabs, terms, 21 + v, as_tensor=True)


def test_more_tables_than_fit_in_registers(mods):
    gpu, _ = mods
    r = random.Random(12)
    tabs = [rand_field(1 << 8, 60 + j) for j in range(11)]
    terms = [(r.randrange(P), [j, (j + 1) % 11]) for j in range(11)] + [(3, [0, 5, 10])]
    _check(gpu, tabs, terms, 13, as_tensor=True)


@pytest.mark.parametrize("nt,v", [(9, 1), (9, 4), (12, 9), (22, 8), (23, 8), (44, 7), (45, 7), (64, 6), (10, 11),
                                  (3, 1), (3, 9), (5, 9), (5, 10), (6, 5), (8, 9), (8, 10), (7, 3),
                                  (5, 13), (8, 12), (3, 16), (2, 11)])
def test_last_rounds_from_lds_around_the_capacity(mods, nt, v):
    """Sums at sizes around what one workgroup's LDS holds of their tables (5632 words in all, nine rounds): the
    whole proof inside the single-workgroup launch (round 0 included, which sums every sample), a proof whose first
    rounds run as separate launches, table counts just below and just above the capacity at a size, a common factor
    with linear terms, and a term of degree five (eight samples kept per pair).  With at most eight tables the sizes
    above the capacity run one launch per round with the tables in registers until the tables fit, fold them into
    place and hand over to the single-workgroup launch; all must agree with the oracle."""
    gpu, _ = mods
    r = random.Random(1000 * nt + v)
    tabs = [rand_field(1 << v, 3000 + 37 * nt + j) for j in range(nt)]
    terms = [(r.randrange(P), [0, j, (j % (nt - 1)) + 1]) for j in range(1, nt, 2)]          # common factor 0, products
    terms += [(r.randrange(P), [0, j]) for j in range(2, nt, 2)]                               # linear under it
    _check(gpu, tabs, terms, 7 * nt + v, as_tensor=True)
    if 6 <= nt <= 12:
        terms5 = [(r.randrange(P), [j, (j + 1) % nt]) for j in range(nt)] + [(5, [1, 2, 3, 4, 5])]
        _check(gpu, tabs, terms5, 11 * nt + v, as_tensor=True)


@pytest.mark.parametrize("v", [4, 11, 14])
def test_single_term_sums_with_a_coefficient(mods, v):
    """One term with a coefficient other than 1 (applied once at the end by the register kernels, per term by the
    single-workgroup launch, so these proofs keep one launch per round above the LDS capacity and are one launch
    below it): a factor twice in the term, five distinct factors, and the coefficient 1, which does hand over."""
    gpu, _ = mods
    r = random.Random(77 + v)
    tabs = [rand_field(1 << v, 8100 + j) for j in range(5)]
    _check(gpu, tabs[:2], [(r.randrange(2, P), [0, 0, 1])], 3 * v, as_tensor=True)
    _check(gpu, tabs, [(r.randrange(2, P), [0, 1, 2, 3, 4])], 5 * v, as_tensor=True)
    _check(gpu, tabs, [(1, [0, 1, 2, 3, 4])], 7 * v, as_tensor=True)


def _layer_gate_batch(n_had, n_resc, n_bool, n_aff, v, seed):
    """The shape of relations.prove_batch (layergkr/relations.py:104-124) over many gates: eq(z, .) in every term,
    lambda-weighted hadamard (eq*a*b - eq*c), rescale (three linear terms), booleanity (eq*b*b - eq*b: a factor
    twice in one term) and affine gates.  -> (tables, terms over table indices)"""
    r = random.Random(seed)
    tabs = [rand_field(1 << v, seed * 1000)]                     # stands in for eq(z, .)
    terms = []

    def new_table():
        tabs.append(rand_field(1 << v, seed * 1000 + len(tabs)))
        return len(tabs) - 1

    for _ in range(n_had):
        lam, a, b, c = r.randrange(P), new_table(), new_table(), new_table()
        terms += [(lam, [0, a, b]), ((lam * (P - 1)) % P, [0, c])]
    for _ in range(n_resc):
        lam, raw, q, rem = r.randrange(P), new_table(), new_table(), new_table()
        terms += [(lam, [0, raw]), ((lam * (P - 4096)) % P, [0, q]), ((lam * (P - 1)) % P, [0, rem])]
    for _ in range(n_bool):
        lam, b = r.randrange(P), new_table()
        terms += [(lam, [0, b, b]), ((lam * (P - 1)) % P, [0, b])]
    for _ in range(n_aff):
        lam, x0, x1, y = r.randrange(P), new_table(), new_table(), new_table()
        terms += [(lam, [0, x0]), (lam, [0, x1]), ((lam * (P - 1)) % P, [0, y])]
    return tabs, terms


@pytest.mark.parametrize("v", [1, 4, 9, 13, 20])
def test_gate_batch_of_a_whole_layer_beyond_one_descriptor(mods, v):
    """97 tables and 90 terms: more than a kernel's descriptor holds (64 tables, 64 terms, 128 factors), so the
    library evaluates the sum in groups of terms; the reference's prove_terms_gpu has no such limit.  At 2^20 the
    first rounds evaluate in one row of workgroups, the later ones deal the terms over several rows."""
    gpu, _ = mods
    tabs, terms = _layer_gate_batch(n_had=12, n_resc=10, n_bool=6, n_aff=8, v=v, seed=21)
    assert len(tabs) > 64 and len(terms) > 64
    _check(gpu, tabs, terms, 22, as_tensor=True)


def test_term_groups_cut_at_the_factor_and_table_limits(mods):
    gpu, _ = mods
    # twenty terms of seven factors: 140 factors over 20 tables -- only the factor count exceeds a descriptor
    tabs = [rand_field(1 << 6, 400 + j) for j in range(20)]
    terms = [(j + 2, [(j + i) % 20 for i in range(7)]) for j in range(20)]
    _check(gpu, tabs, terms, 23, as_tensor=True)
    # seventy single-table terms over seventy tables: the table and term counts exceed it, the factor count does not
    tabs = [rand_field(1 << 10, 440 + j) for j in range(70)]
    terms = [(3 * j + 1, [j]) for j in range(70)]
    _check(gpu, tabs, terms, 24, as_tensor=True)
    # a term whose tables straddle two groups, and mixed degrees in each
    tabs = [rand_field(1 << 8, 520 + j) for j in range(72)]
    terms = [(j + 1, [j, j + 1]) for j in range(71)] + [(7, [0, 35, 71]), (P - 1, [71])]
    _check(gpu, tabs, terms, 25, as_tensor=True)
    # exactly one descriptor's worth of tables and terms, and one more
    for n in (64, 65):
        tabs = [rand_field(1 << 7, 600 + j) for j in range(n)]
        terms = [(j + 5, [j, (j + 1) % n]) for j in range(n)]
        _check(gpu, tabs, terms, 26 + n, as_tensor=True)


def test_large_sum_through_the_c_abi_round_by_round(mods):
    """vi_sumcheck_eval and vi_sumcheck_fold_eval on 97 tables / 90 terms against the oracle's rounds 0 and 1;
    the entry point that allocates nothing keeps to one descriptor and says so."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    tabs, terms = _layer_gate_batch(n_had=12, n_resc=10, n_bool=6, n_aff=8, v=11, seed=31)
    n = len(tabs)
    dev = [to_dev(t) for t in tabs]
    dst = [torch.empty(1 << 10, dtype=torch.uint64, device="cuda") for _ in tabs]
    src_p = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dev])
    dst_p = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dst])
    off, idx = [0], []
    for _, fs in terms:
        idx += fs
        off.append(len(idx))
    term_off, factor_idx = (ctypes.c_int * len(off))(*off), (ctypes.c_int * len(idx))(*idx)
    coeffs = (ctypes.c_uint64 * len(terms))(*[c for c, _ in terms])
    out = torch.zeros(8, dtype=torch.uint64, device="cuda")
    ws = torch.empty(L.vi_sumcheck_workspace_bytes(), dtype=torch.uint8, device="cuda")
    r = 0x123456789ABCDEF0 % P
    _, samples, _ = O.sumcheck_prove(tabs, terms, [r] + [1] * 10)
    _lib.check(L.vi_sumcheck_eval(src_p, n, 1 << 10, term_off, factor_idx, coeffs, len(terms), out.data_ptr(),
                                  ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    assert [int(x) for x in out.cpu().tolist()[:4]] == samples[0]
    claim = (ctypes.c_uint64 * 1)(0)
    _lib.check(L.vi_sumcheck_fold_eval(src_p, dst_p, n, 1 << 10, r, term_off, factor_idx, coeffs, len(terms), claim,
                                       out.data_ptr(), ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    assert [int(x) for x in out.cpu().tolist()[:4]] == samples[1]
    for t, d in zip(tabs, dst):
        assert np.array_equal(to_np(d), O.fold(t, r))
    rc = L.vi_sumcheck_eval_static(src_p, n, 1 << 10, term_off, factor_idx, coeffs, len(terms), out.data_ptr(),
                                   _lib.stream_ptr())
    assert rc != 0 and "n_tables" in L.vi_last_error().decode()


def test_tables_in_memory_at_full_grid_size(mods):
    """11 and 40 tables at 2^20 (one descriptor): the first rounds fill the capped grid of the evaluation kernel and
    of the many-table fold, the later ones deal the terms over rows of workgroups."""
    gpu, _ = mods
    r = random.Random(15)
    tabs = [rand_field(1 << 20, 700 + j) for j in range(11)]
    terms = [(r.randrange(P), [j, (j + 1) % 11]) for j in range(11)] + [(3, [0, 5, 10])]
    _check(gpu, tabs, terms, 16, as_tensor=True)
    tabs = [rand_field(1 << 20, 720 + j) for j in range(40)]
    terms = [(r.randrange(P), [0, j, j + 1]) for j in range(1, 39, 2)] + [(r.randrange(P), [0, j]) for j in range(1, 40)]
    _check(gpu, tabs, terms, 17, as_tensor=True)


def test_fold_eval_in_place_with_unused_tables_c_abi(mods):
    """vi_sumcheck_fold_eval, dst == src, at 2^20: 70 tables of which five occur in no term (they are folded all
    the same), the sum beyond one descriptor; and the same tables through one descriptor's worth of terms."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    n, v = 70, 20
    tabs = [rand_field(1 << v, 800 + j) for j in range(n)]
    used = [j for j in range(n) if j % 14 != 3]
    r = 0x0FEDCBA987654321 % P
    folded = [O.fold(t, r) for t in tabs]
    for terms in ([(j + 2, [used[j], used[(j + 1) % len(used)]]) for j in range(len(used))],       # 65 terms: two groups
                  [(j + 2, [used[j], used[j + 1], used[j + 2]]) for j in range(0, 30, 3)]):           # one descriptor
        dev = [to_dev(t) for t in tabs]
        ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dev])
        off, idx = [0], []
        for _, fs in terms:
            idx += fs
            off.append(len(idx))
        term_off, factor_idx = (ctypes.c_int * len(off))(*off), (ctypes.c_int * len(idx))(*idx)
        coeffs = (ctypes.c_uint64 * len(terms))(*[c for c, _ in terms])
        out = torch.zeros(8, dtype=torch.uint64, device="cuda")
        ws = torch.empty(L.vi_sumcheck_workspace_bytes(), dtype=torch.uint8, device="cuda")
        _lib.check(L.vi_sumcheck_fold_eval(ptrs, ptrs, n, 1 << (v - 1), r, term_off, factor_idx, coeffs, len(terms), None,
                                           out.data_ptr(), ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
        deg = max(len(fs) for _, fs in terms)
        _, samples, _ = O.sumcheck_prove(folded, terms, [1] * (v - 1))
        assert [int(x) for x in out.cpu().tolist()[:deg + 1]] == samples[0]
        for t, f in zip(dev, folded):
            assert np.array_equal(to_np(t)[: 1 << (v - 1)], f)


@pytest.mark.parametrize("seed", range(24))
def test_random_term_structures_match_oracle(mods, seed):
    """Seeded random sums: 1..100 tables, 1..100 terms of 1..4 factors (repeats allowed), a table shared by all
    terms or not, tables nobody uses, 2^1..2^11 entries -- the register path, one descriptor in memory, and groups."""
    gpu, _ = mods
    r = random.Random(9000 + seed)
    n_tables = r.choice([1, 2, 3, 4, 5, 8, 9, 17, 33, 64, 65, 100])
    n_terms = r.choice([1, 2, 3, 7, 31, 64, 65, 100])
    v = r.randrange(1, 12)
    shared = r.random() < 0.5
    tabs = [rand_field(1 << v, 9100 + 101 * seed + j) for j in range(n_tables)]
    terms = []
    for _ in range(n_terms):
        fs = [r.randrange(n_tables) for _ in range(r.randrange(1, 5))]
        if shared:
            fs[r.randrange(len(fs))] = 0
        terms.append((r.choice([1, 2, P - 1, r.randrange(P)]), fs))
    _check(gpu, tabs, terms, 9200 + seed, as_tensor=True)


def test_degree_above_three_and_limits(mods):
    gpu, _ = mods
    tabs = [rand_field(1 << 7, 70 + j) for j in range(6)]
    _check(gpu, tabs, [(1, [0, 1, 2, 3, 4, 5]), (2, [0])], 14, as_tensor=True)
    with pytest.raises(RuntimeError):
        obj = [to_dev(t) for t in tabs]
        gpu.prove_terms_gpu([(1, [obj[0]] * 8)], lambda i: 1, P)          # degree 8 is above the kernel limit


@pytest.mark.parametrize("v,nt,terms", [(3, 2, [(1, [0, 1])]), (11, 3, [(1, [0, 1, 2])]),
                                        (12, 4, [(3, [0, 1, 2]), (P - 5, [0, 3])]),
                                        (9, 10, [(3, [0, 1, 2]), (P - 5, [3]), (7, [4, 5]), (11, [6]), (13, [7, 8, 9, 0])])])
def test_tables_with_words_at_or_above_p_are_taken_as_residues(mods, v, nt, terms):
    """A caller's tensor may hold any 64-bit word (the reference's add / sub / mul chain stays congruent on them):
    p, p + 1 and 2^64 - 1 in the tables give the proof of their residues."""
    gpu, _ = mods
    tabs = [rand_field(1 << v, 500 + v + j) for j in range(nt)]
    raw = [t.copy() for t in tabs]
    for j, t in enumerate(raw):
        for pos, word in ((0, P), (1, P + 1), (t.size - 1, (1 << 64) - 1), (t.size // 2, P + 12345), (t.size // 2 + 1, P)):
            t[(pos + j) % t.size] = np.uint64(word)
        # a word at or above p in the lower half opposite a tiny one in the upper half: hi - lo borrows twice unless
        # lo is reduced first
        h = t.size // 2
        if h >= 4:
            for pos, lo, hi in ((2, (1 << 64) - 1, 0), (3, P + 1, 0)):
                t[(pos + j) % h] = np.uint64(lo)
                t[h + (pos + j) % h] = np.uint64(hi)
    residues = [np.array([int(x) % P for x in t], dtype=np.uint64) for t in raw]
    coins, coin = _coins(v, 77)
    objs = [to_dev(t) for t in raw]
    obj_terms = [(c, [objs[i] for i in fs]) for c, fs in terms]
    claim, polys, chals, _ = gpu.prove_terms_gpu(obj_terms, coin, P)
    want_claim, want_samples, _ = O.sumcheck_prove(residues, terms, coins)
    assert claim == want_claim
    assert [[y for _, y in s] for s in polys] == want_samples
    assert gpu.prove_terms_gpu_interactive(obj_terms, lambda i, _s: coins[i], P)[:2] == (claim, polys)


def test_fold_of_words_at_or_above_p_c_abi(mods):
    """vi_sumcheck_fold_eval on caller words: (lo, hi) = (2^64 - 1, 0) and (p + 1, 0) fold like their residues, for
    few tables (register kernel) and for many (the many-table fold)."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    r = 0x0123456789ABCDEF % P
    for n in (2, 12):
        tabs = [rand_field(1 << 8, 950 + j) for j in range(n)]
        raw = [t.copy() for t in tabs]
        for j, t in enumerate(raw):
            t[j], t[128 + j] = np.uint64((1 << 64) - 1), np.uint64(0)
            t[20 + j], t[148 + j] = np.uint64(P + 1), np.uint64(0)
            t[40 + j], t[168 + j] = np.uint64(5), np.uint64((1 << 64) - 2)
        residues = [np.array([int(x) % P for x in t], dtype=np.uint64) for t in raw]
        dev = [to_dev(t) for t in raw]
        dst = [torch.empty(128, dtype=torch.uint64, device="cuda") for _ in raw]
        src_p = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dev])
        dst_p = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dst])
        _lib.check(L.vi_sumcheck_fold_eval(src_p, dst_p, n, 128, r, None, None, None, 0, None, None, None, 0,
                                           _lib.stream_ptr()))
        for d, t in zip(dst, residues):
            assert np.array_equal(to_np(d), O.fold(t, r))


def test_tables_that_are_views_at_an_odd_word_offset(mods):
    """The evaluation round loads two adjacent words per access when every table is 16-byte aligned; a table that
    starts at an odd word (a slice of a larger tensor) must take the other path and give the same proof."""
    gpu, _ = mods
    v = 13
    tabs = [rand_field(1 << v, 700 + j) for j in range(3)]
    coins, coin = _coins(v, 31)
    want_claim, want_samples, _ = O.sumcheck_prove(tabs, [(1, [0, 1, 2])], coins)
    for shifted in ((1, 0, 0), (0, 1, 1), (1, 1, 1), (0, 0, 0)):
        objs = []
        for t, sh in zip(tabs, shifted):
            buf = to_dev(np.concatenate([np.zeros(sh, dtype=np.uint64), t]))
            objs.append(buf[sh:])
            assert objs[-1].data_ptr() % 16 == (8 if sh else 0)
        claim, polys, _, _ = gpu.prove_terms_gpu([(1, objs)], coin, P)
        assert claim == want_claim and [[y for _, y in s] for s in polys] == want_samples, shifted


def test_large_instance_matches_oracle(mods):
    """2^22 x 3 factors, degree 3, 22 rounds: every round's samples against the C oracle."""
    gpu, _ = mods
    tabs = [rand_field(1 << 22, 80 + j) for j in range(3)]
    _check(gpu, tabs, [(1, [0, 1, 2])], 15, as_tensor=True)


def test_prove_verify_masked_and_tamper(mods):
    """The reference's sumcheck gates (layergkr/tests/test_sumcheck.py) on the device prover."""
    gpu, sc = mods
    assert sc._sumcheck_gpu_ok()
    N_VARS = 4

    def factors(k, seed):
        r = random.Random(seed)
        return [[r.randrange(P) for _ in range(1 << N_VARS)] for _ in range(k)]

    def coin():
        r = random.Random(99)
        vals = [r.randrange(P) for _ in range(N_VARS)]
        return lambda i: vals[i]

    def tape(n, seed=5):
        r = random.Random(seed)
        return sc.MaskTape([r.randrange(P) for _ in range(n)])

    for k, seed in ((2, 17), (3, 23)):
        f = factors(k, seed)
        proof = sc.prove(f, coin())
        ok, why = sc.verify(proof, f, coin())
        assert ok, why
    f = factors(2, 17)
    bare = sc.prove(f, coin())
    masked = sc.prove(f, coin(), tape=tape(2 * N_VARS), mu0=123456789)
    ok, why = sc.verify(masked, f, coin())
    assert ok, why
    assert masked.claim == (bare.claim + 123456789) % P
    assert masked.round_polys[0] != bare.round_polys[0]
    # tamper cases
    p1 = sc.prove(f, coin())
    p1.claim = (p1.claim + 1) % P
    ok, why = sc.verify(p1, f, coin())
    assert not ok and "claim" in why
    p2 = sc.prove(f, coin())
    x, y = p2.round_polys[1][0]
    p2.round_polys[1][0] = (x, (y + 1) % P)
    assert not sc.verify(p2, f, coin())[0]
    p3 = sc.prove(f, coin())
    p3.challenges[2] = (p3.challenges[2] + 1) % P
    ok, why = sc.verify(p3, f, coin())
    assert not ok and "challenge" in why
    for tp, mu0 in ((None, 0), (tape(2 * N_VARS), 4242)):
        pf = sc.prove(f, coin(), tape=tp, mu0=mu0)
        bad = [list(f[0]), list(f[1])]
        bad[0][3] = (bad[0][3] + 1) % P
        ok, why = sc.verify(pf, bad, coin())
        assert not ok and "terminal" in why
    with pytest.raises(RuntimeError):
        sc.prove(f, coin(), tape=tape(2), mu0=1)
    # masked device proof == oracle samples + host mask polynomial
    tp = tape(2 * N_VARS)
    vals = list(tp.values)
    pf = sc.prove(f, coin(), tape=tp, mu0=77)
    coins = [coin()(i) for i in range(N_VARS)]
    _, samples, _ = O.sumcheck_prove([np.array(t, dtype=np.uint64) for t in f], [(1, [0, 1])], coins)
    mu = 77
    for rnd in range(N_VARS):
        h = sc.mask_poly_coeffs(mu, vals[2 * rnd:2 * rnd + 2])
        assert [y for _, y in pf.round_polys[rnd]] == [(samples[rnd][x] + sc.poly_eval_coeffs(h, x)) % P for x in range(3)]
        mu = sc.poly_eval_coeffs(h, coins[rnd])
    assert pf.final_mask == mu


def test_fold_eval_in_place_c_abi(mods):
    """vi_sumcheck_fold_eval with dst == src (fold in place) against the oracle."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    tabs = [rand_field(1 << 12, 90 + j) for j in range(3)]
    dev = [to_dev(t) for t in tabs]
    r = 0xDEADBEEFCAFEF00D % P
    ptrs = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in dev])
    off = (ctypes.c_int * 2)(0, 3)
    idx = (ctypes.c_int * 3)(0, 1, 2)
    co = (ctypes.c_uint64 * 1)(1)
    out = torch.zeros(4, dtype=torch.uint64, device="cuda")
    ws = torch.empty(L.vi_sumcheck_workspace_bytes(), dtype=torch.uint8, device="cuda")
    _lib.check(L.vi_sumcheck_fold_eval(ptrs, ptrs, 3, 1 << 11, r, off, idx, co, 1, None, out.data_ptr(),
                                       ws.data_ptr(), ws.numel(), _lib.stream_ptr()))
    folded = [O.fold(t, r) for t in tabs]
    for t, f in zip(dev, folded):
        assert np.array_equal(to_np(t)[: 1 << 11], f)
    _, samples, _ = O.sumcheck_prove(folded, [(1, [0, 1, 2])], [0] * 11)
    assert [int(x) for x in out.cpu().tolist()] == samples[0]


def test_verifier_accepts_and_rejects_device_table_proofs(mods):
    """prove_terms / verify_terms on device tensors at a size where host lists are out of the
    question (2^20): the verifier's terminal check evaluates the tables on the device.  A shared
    factor, two terms, then a tampered sample and a tampered table."""
    gpu, sc = mods
    v = 20
    eq = gpu.eq_vector_t([random.Random(3).randrange(P) for _ in range(v)])
    a, b, c = (to_dev(rand_field((1 << v,), 60 + i)) for i in range(3))
    terms = [(5, [eq, a, b]), (P - 2, [eq, c])]
    coins = [random.Random(4).randrange(P) for _ in range(v)]
    proof = sc.prove_terms(terms, lambda i: coins[i])
    ok, why = sc.verify_terms(proof, terms, lambda i: coins[i])
    assert ok, why
    # the claim is the sum the terms define
    want = (5 * int(gpu.gl_sum(cp_mul(cp_mul(eq, a), b)).cpu().item()) - 2 * int(gpu.gl_sum(cp_mul(eq, c)).cpu().item())) % P
    assert proof.claim == want
    bad = sc.SumcheckProof(**{**proof.__dict__})
    bad.round_polys = [list(s) for s in proof.round_polys]
    x, y = bad.round_polys[7][2]
    bad.round_polys[7][2] = (x, (y + 1) % P)
    assert not sc.verify_terms(bad, terms, lambda i: coins[i])[0]
    c2 = c.clone()
    c2.view(torch.int64)[12345] += 1
    ok, why = sc.verify_terms(proof, [(5, [eq, a, b]), (P - 2, [eq, c2])], lambda i: coins[i])
    assert not ok and "terminal" in why


def test_baseline_shape_three_tables_of_2p26(mods):
    """The benchmark instance at full size (three tables of 2^26 uniform field elements, degree 3, 26 rounds):
    the claim and every round's samples against the C oracle on the same tables, then the properties -- the claim
    is the sum of the elementwise product, every round satisfies S(0) + S(1) = previous claim, and the last claim
    equals the product of the three multilinear extensions at the challenge point (all checked by the verifier,
    the terminal values on the device); a tampered table is rejected."""
    gpu, sc = mods
    from tests.gpu_util import rand_field_dev
    v = 26
    tabs = [rand_field_dev((1 << v,), 260 + j) for j in range(3)]
    rnd = random.Random(5)
    coins = [rnd.randrange(P) for _ in range(v)]
    terms = [(1, tabs)]
    proof = sc.prove_terms(terms, lambda i: coins[i])
    assert len(proof.round_polys) == v and all(len(s) == 4 for s in proof.round_polys)
    want_claim, want_samples, _ = O.sumcheck_prove([t.cpu().numpy() for t in tabs], [(1, [0, 1, 2])], coins)
    assert proof.claim == want_claim
    assert [[y for _, y in s] for s in proof.round_polys] == want_samples
    assert proof.claim == int(gpu.gl_sum(cp_mul(cp_mul(tabs[0], tabs[1]), tabs[2])).cpu().item())
    ok, why = sc.verify_terms(proof, terms, lambda i: coins[i])
    assert ok, why
    tabs[1].view(torch.int64)[(1 << v) - 3] += 1
    ok, why = sc.verify_terms(proof, terms, lambda i: coins[i])
    assert not ok and "terminal" in why


def test_prove_coins_c_abi_with_samples_in_device_memory(mods):
    """vi_sumcheck_prove_coins called directly: samples land in DEVICE memory (rows of 8 words), the call returns
    without waiting, the tables are odd-offset views; a shape with its own multi-round kernels, the gate shape,
    a sum that is rewritten after round 0 (two tables under a common factor become one) and a general one."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    cases = [(15, 3, [(9, [0, 1, 2])]),
             (13, 4, [(3, [0, 1, 2]), (P - 5, [0, 3])]),
             (12, 5, [(3, [0, 1, 2]), (P - 5, [0, 3]), (7, [0, 4])]),
             (10, 6, [(3, [0, 1]), (P - 5, [2, 3, 4]), (7, [5, 0, 1])])]
    for v, nt, terms in cases:
        size = 1 << v
        tabs = [rand_field(size, 1500 + 10 * v + j) for j in range(nt)]
        dev = []
        for t in tabs:
            buf = to_dev(np.concatenate([np.zeros(1, dtype=np.uint64), t]))
            dev.append(buf[1:])
        work = [torch.empty(size // 2, dtype=torch.uint64, device="cuda") for _ in tabs]
        coins, _ = _coins(v, 50 + v)
        off, idx = [0], []
        for _, fs in terms:
            idx += fs
            off.append(len(idx))
        samples = torch.zeros(8 * v, dtype=torch.uint64, device="cuda")
        ws = torch.empty(L.vi_sumcheck_prove_coins_workspace_bytes(size), dtype=torch.uint8, device="cuda")
        _lib.check(L.vi_sumcheck_prove_coins((ctypes.c_void_p * nt)(*[t.data_ptr() for t in dev]),
                                             (ctypes.c_void_p * nt)(*[t.data_ptr() for t in work]), nt, size,
                                             (ctypes.c_int * len(off))(*off), (ctypes.c_int * len(idx))(*idx),
                                             (ctypes.c_uint64 * len(terms))(*[c for c, _ in terms]), len(terms),
                                             (ctypes.c_uint64 * v)(*coins), samples.data_ptr(), ws.data_ptr(), ws.numel(),
                                             _lib.stream_ptr()))
        deg = max(len(fs) for _, fs in terms)
        got = to_np(samples).reshape(v, 8)[:, :deg + 1].tolist()
        want_claim, want_samples, _ = O.sumcheck_prove(tabs, terms, coins)
        assert got == want_samples, (v, nt)
        assert (got[0][0] + got[0][1]) % P == want_claim
        for t, d in zip(tabs, dev):
            assert np.array_equal(to_np(d), t), "caller's table was modified"


def test_coins_and_masks_drawn_up_front_match_the_interactive_loop(mods):
    """prove_terms_gpu calls mask and coin for all rounds before the first launch, in the reference's order
    (mask, coin, mask, coin, ...): with a coin and a mask tape that share one random.Random -- so that any other
    call order would draw other values -- it returns what the round-by-round loop returns, for a shape with its
    own multi-round kernels and for a general sum."""
    gpu, sc = mods
    for v, nt, terms_idx in ((14, 3, [(7, [0, 1, 2])]), (13, 4, [(3, [0, 1, 2]), (P - 5, [0, 3])]),
                            (9, 6, [(3, [0, 1]), (P - 5, [2]), (7, [3]), (11, [4, 5, 0])]), (1, 2, [(1, [0, 1])])):
        tabs = [to_dev(rand_field(1 << v, 1200 + j)) for j in range(nt)]
        terms = [(c, [tabs[i] for i in fs]) for c, fs in terms_idx]
        deg = max(len(fs) for _, fs in terms_idx)

        def run(prover, wrap):
            shared = random.Random(77)
            calls = []

            def coin(i):
                calls.append(("coin", i))
                return shared.randrange(1 << 64)

            def mask(d, mu):
                calls.append(("mask", mu))
                assert d == deg
                return sc.mask_poly_coeffs(mu, [shared.randrange(P) for _ in range(d)])

            return prover(terms, wrap(coin), P, mask=mask, mu0=31337), calls

        up_front, calls_a = run(gpu.prove_terms_gpu, lambda c: c)
        looped, calls_b = run(gpu.prove_terms_gpu_interactive, lambda c: (lambda i, _samples: c(i)))
        assert up_front == looped
        assert calls_a == calls_b and [k for k, _ in calls_a] == ["mask", "coin"] * v
        # and the masked proof verifies: S(0) + S(1) of every round is the previous round's value at its challenge
        claim, polys, chals, mu = up_front
        cur = claim
        for s, r in zip(polys, chals):
            ys = [y for _, y in s]
            assert (ys[0] + ys[1]) % P == cur
            cur = _lagrange_at(ys, r)
        assert cur == (_terminal(tabs, terms_idx, chals) + mu) % P


def _terminal(tabs, terms_idx, chals):
    """sum_k c_k prod_j f_j(r): the tables folded on the host in Python integers"""
    vals = []
    for t in tabs:
        f = [int(x) for x in to_np(t)]
        for r in chals:
            h = len(f) // 2
            f = [(f[i] + r * (f[h + i] - f[i])) % P for i in range(h)]
        vals.append(f[0])
    total = 0
    for c, fs in terms_idx:
        prod = c
        for i in fs:
            prod = prod * vals[i] % P
        total += prod
    return total % P


def _lagrange_at(ys, r):
    n, total = len(ys), 0
    for i, y in enumerate(ys):
        num, den = y, 1
        for k in range(n):
            if k != i:
                num = num * (r - k) % P
                den = den * (i - k) % P
        total += num * pow(den, P - 2, P)
    return total % P


def cp_mul(x, y):
    from verinf_amd.prover import cuda_primitives as cp
    return cp.gl_mul(x, y)

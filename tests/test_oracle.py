"""Pins the CPU oracle (oracle/) -- no GPU needed.

Each oracle function is checked against something it did not come from: the
first-principles fixtures in tests/golden (Python big-int definitions), closed
forms, invariants of the transform, and brute force at toy sizes.
"""
import json
import os
import random

import numpy as np
import pytest

from oracle import oracle as O

P = O.P


def _unhex(v):
    return np.array([int(x, 16) for x in v], dtype=np.uint64)


# ------------------------------------------------------------------ field ----
def test_field_golden_vectors(golden_dir):
    vec = json.load(open(os.path.join(golden_dir, "field_vectors.json")))
    a = _unhex([v["a"] for v in vec])
    b = _unhex([v["b"] for v in vec])
    for op in ("add", "sub", "mul"):
        assert np.array_equal(O.binop(op, a, b), _unhex([v[op] for v in vec])), op


def test_field_against_python_ints():
    r = random.Random(1)
    edge = [0, 1, 2, P - 1, P - 2, (1 << 32) - 1, 1 << 32, (1 << 32) + 1, 1 << 63,
            0xFFFFFFFF00000000, (1 << 63) - 1]
    vals = edge + [r.randrange(P) for _ in range(2000)]
    a = np.array([r.choice(vals) for _ in range(20000)], dtype=np.uint64)
    b = np.array([r.choice(vals) for _ in range(20000)], dtype=np.uint64)
    ai, bi = [int(x) for x in a], [int(x) for x in b]
    assert O.binop("add", a, b).tolist() == [(x + y) % P for x, y in zip(ai, bi)]
    assert O.binop("sub", a, b).tolist() == [(x - y) % P for x, y in zip(ai, bi)]
    assert O.binop("mul", a, b).tolist() == [(x * y) % P for x, y in zip(ai, bi)]


def test_field_identities():
    L = O.lib()
    assert L.vo_mul(1 << 32, 1 << 32) == (1 << 32) - 1          # 2^64 = 2^32 - 1
    assert L.vo_pow(2, 96) == P - 1                               # 2^96 = -1
    assert L.vo_pow(2, 192) == 1
    assert L.vo_mul(P - 1, P - 1) == 1
    assert L.vo_add(P - 1, 1) == 0 and L.vo_sub(0, 1) == P - 1
    assert L.vo_root_of_unity(64) == 1 << 39                      # 64th roots are powers of two
    r = random.Random(2)
    for _ in range(50):
        a = r.randrange(1, P)
        assert L.vo_mul(a, L.vo_inv(a)) == 1
        assert L.vo_pow(a, 12345) == pow(a, 12345, P)


# -------------------------------------------------------------------- NTT ----
def test_ntt_golden_1024(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "ntt_1024.json")))
    a, want = _unhex(g["input"]), _unhex(g["forward"])
    got = O.ntt(a)
    assert np.array_equal(got, want)
    assert np.array_equal(O.ntt(got, inverse=True), a)
    assert np.array_equal(O.dft_naive(a), want)


@pytest.mark.parametrize("n", [2, 4, 8, 16, 64, 256])
def test_ntt_matches_definition(n):
    r = random.Random(10 + n)
    a = [r.randrange(P) for _ in range(n)]
    arr = np.array(a, dtype=np.uint64)
    want = O.py_dft(a)
    assert O.ntt(arr).tolist() == want
    assert O.dft_naive(arr).tolist() == want
    assert O.ntt(np.array(want, dtype=np.uint64), inverse=True).tolist() == a
    assert O.dft_naive(np.array(want, dtype=np.uint64), inverse=True).tolist() == a


def test_ntt_invariants():
    n = 4096
    r = random.Random(11)
    a = np.array([r.randrange(P) for _ in range(n)], dtype=np.uint64)
    delta = np.zeros(n, dtype=np.uint64)
    delta[0] = 1
    assert np.array_equal(O.ntt(delta), np.ones(n, dtype=np.uint64))
    const = np.full(n, 5, dtype=np.uint64)
    out = O.ntt(const)
    assert out[0] == 5 * n and not out[1:].any()
    # shift theorem: NTT(roll(a,1))[k] = w^k NTT(a)[k]
    w = O.py_root(n)
    fa = O.ntt(a)
    fs = O.ntt(np.roll(a, 1))
    wk = np.array([pow(w, k, P) for k in range(n)], dtype=np.uint64)
    assert np.array_equal(fs, O.binop("mul", fa, wk))
    # rows == single
    rows = np.stack([a, np.roll(a, 3)])
    got = O.ntt_rows(rows)
    assert np.array_equal(got[0], fa) and np.array_equal(got[1], O.ntt(np.roll(a, 3)))
    assert np.array_equal(O.ntt_rows(got, inverse=True), rows)


# -------------------------------------------------------------- coset LDE ----
def test_lde_golden(golden_dir):
    for g in json.load(open(os.path.join(golden_dir, "coset_lde.json"))):
        msgs = np.stack([_unhex(m) for m in g["messages"]])
        want = np.stack([_unhex(c) for c in g["codewords"]])
        got = O.coset_lde_rows(msgs, g["K"], g["N"], g["shift"])
        assert np.array_equal(got, want), (g["K"], g["N"])
        assert np.array_equal(O.lde_dense_row(msgs[0], g["K"], g["N"], g["shift"]), want[0])


def test_lde_dense_matches_python_closed_form():
    r = random.Random(3)
    K, N = 16, 64
    msg = [r.randrange(P) for _ in range(11)]
    assert O.lde_dense_row(np.array(msg, dtype=np.uint64), K, N).tolist() == O.py_lde_dense(msg, K, N)
    assert O.lib().vo_lagrange(K, 3, 12345) == O.py_lagrange(K, 3, 12345)


def test_lde_is_a_low_degree_codeword():
    """Untwist + iNTT_N of a codeword has zero coefficients at indices >= K, and
    evaluating those coefficients at w_K^c returns the message."""
    r = random.Random(4)
    K, N, w = 256, 1024, 200
    msg = np.array([[r.randrange(P) for _ in range(w)]], dtype=np.uint64)
    cw = O.coset_lde_rows(msg, K, N)[0]
    coef = [int(x) for x in O.ntt(cw, inverse=True)]
    ginv = pow(7, -1, P)
    coef = [c * pow(ginv, i, P) % P for i, c in enumerate(coef)]
    assert not any(coef[K:])
    wk = O.py_root(K)
    for c in (0, 1, 57, w - 1, w, K - 1):
        x = pow(wk, c, P)
        acc = 0
        for co in reversed(coef[:K]):
            acc = (acc * x + co) % P
        assert acc == (int(msg[0, c]) if c < w else 0)


def test_lde_sampled_columns_large_geometry():
    """The spot check of layergkr/gpu.py:226-253 at K=2^12, N=2^14 (config 1 shape)."""
    r = random.Random(5)
    K, N = 1 << 12, 1 << 14
    msg = [r.randrange(P) for _ in range(K)]
    cw = O.coset_lde_rows(np.array([msg], dtype=np.uint64), K, N)[0]
    wn = O.py_root(N)
    zs = [pow(O.py_root(K), c, P) for c in range(K)]
    for _ in range(6):
        j = r.randrange(N)
        eta = 7 * pow(wn, j, P) % P
        num = (pow(eta, K, P) - 1) % P
        acc = 0
        for c, v in enumerate(msg):
            acc += v * (zs[c] * num % P * pow(K * (eta - zs[c]) % P, -1, P) % P)
        assert acc % P == int(cw[j])


# --------------------------------------------------------------- sumcheck ----
def test_sumcheck_golden(golden_dir):
    for g in json.load(open(os.path.join(golden_dir, "sumcheck.json"))):
        tables = [_unhex(t) for t in g["tables"]]
        terms = [(int(c, 16), fs) for c, fs in g["terms"]]
        coins = [int(c, 16) for c in g["coins"]]
        claim, samples, finals = O.sumcheck_prove(tables, terms, coins)
        assert claim == int(g["claim"], 16), g["name"]
        assert samples == [[int(x, 16) for x in s] for s in g["samples"]], g["name"]
        assert finals == [int(x, 16) for x in g["finals"]], g["name"]


def test_sumcheck_matches_bruteforce_and_verifier_identities():
    r = random.Random(6)
    n = 256
    tabs = [np.array([r.randrange(P) for _ in range(n)], dtype=np.uint64) for _ in range(4)]
    terms = [(r.randrange(P), [0, 1, 2]), (P - 1, [3]), (5, [1, 1]), (7, [0, 3])]
    coins = [r.randrange(P) for _ in range(8)]
    got = O.sumcheck_prove(tabs, terms, coins)
    assert got == O.py_sumcheck(tabs, terms, coins)
    claim, samples, finals = got
    # S(0)+S(1) = running claim; next claim = interpolation at r; terminal = product of MLEs
    cur = claim
    for rnd, s in enumerate(samples):
        assert (s[0] + s[1]) % P == cur
        xs = list(range(len(s)))
        rr = coins[rnd]
        acc = 0
        for i, yi in enumerate(s):
            num = den = 1
            for k in xs:
                if k != i:
                    num = num * (rr - k) % P
                    den = den * (i - k) % P
            acc = (acc + yi * num * pow(den, -1, P)) % P
        cur = acc
    mle = [O.py_mle_eval(t, coins) for t in tabs]
    assert finals == mle
    term = 0
    for c, fs in terms:
        prod = c
        for j in fs:
            prod = prod * mle[j] % P
        term += prod
    assert term % P == cur


def test_fold_matches_definition():
    r = random.Random(7)
    f = np.array([r.randrange(P) for _ in range(64)], dtype=np.uint64)
    c = r.randrange(P)
    want = [(int(f[i]) + c * (int(f[32 + i]) - int(f[i]))) % P for i in range(32)]
    assert O.fold(f, c).tolist() == want


# ---------------------------------------------------------------- K-quant ----
def test_kquant_golden(golden_dir):
    for g in json.load(open(os.path.join(golden_dir, "kquant.json"))):
        raw = np.frombuffer(bytes.fromhex(g["raw"]), dtype=np.uint8)
        want = _unhex(g["field"])
        assert np.array_equal(O.kquant_to_field(raw, g["qtype"], g["S"]), want), g["qtype"]
        assert np.array_equal(O.np_kquant_to_field(raw, g["qtype"], g["S"]), want), g["qtype"]


@pytest.mark.parametrize("qtype", ["Q4_K", "Q5_K", "Q6_K"])
def test_kquant_c_and_numpy_restatements_agree(qtype):
    rng = np.random.default_rng(8)
    nb = 2000
    raw = rng.integers(0, 256, size=(nb, O.BLOCK_BYTES[qtype]), dtype=np.uint8)
    d = np.abs(rng.normal(0, 0.01, size=(nb, 2))).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if qtype == "Q6_K":
        raw[:, 208:210] = d[:, :2]
    else:
        raw[:, 0:4] = d
    for S in (1 << 12, 1 << 16, 1000003):
        assert np.array_equal(O.kquant_to_field(raw, qtype, S), O.np_kquant_to_field(raw, qtype, S))


def test_kquant_closed_forms():
    """d = 1, dmin = 0 -> the output is exactly sc*q*S; all 64 x 16 (sc, q) pairs occur."""
    S = 1 << 12
    blocks = []
    for sc in range(64):
        b = bytearray(144)
        b[0:2] = (0x3C00).to_bytes(2, "little")            # d = 1.0, dmin = 0
        for s in range(4):
            b[4 + s] = sc                                    # sub-blocks 0..3: 6-bit scale
            b[8 + s] = 0
            b[12 + s] = (sc & 0x0F)                          # sub-blocks 4..7: low nibble
            b[4 + s] |= (sc >> 4) << 6                       # ... high two bits
        for i in range(128):
            b[16 + i] = (i % 16) | (((i + 5) % 16) << 4)
        blocks.append(bytes(b))
    raw = np.frombuffer(b"".join(blocks), dtype=np.uint8)
    got = O.kquant_to_field(raw, "Q4_K", S).reshape(64, 256)
    for sc in range(64):
        for e in range(256):
            byte = (e >> 6) * 32 + (e & 31)
            q = (byte % 16) if ((e >> 5) & 1) == 0 else ((byte + 5) % 16)
            assert int(got[sc, e]) == sc * q * S
    # sign mapping: d = 0, dmin = 1 -> value -mn*S -> p - mn*S
    b = bytearray(144)
    b[2:4] = (0x3C00).to_bytes(2, "little")
    b[8] = 9                                                 # mn of sub-block 0
    got = O.kquant_to_field(np.frombuffer(bytes(b), dtype=np.uint8), "Q4_K", S)
    assert int(got[0]) == P - 9 * S and int(got[40]) == 0


# ---- BLAKE3 / Merkle -------------------------------------------------------------------
def _kat():
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    with open(os.path.join(here, "blake3_kat.json")) as f:
        return json.load(f)["cases"]


def test_blake3_known_answers_oracle():
    for c in _kat():
        data = bytes(i % 251 for i in range(c["len"]))
        assert O.blake3(data).hex() == c["hash"], c["len"]


def test_blake3_known_answers_host():
    """The host-side hash of the verifier helpers is a second, differently structured
    implementation (level-wise tree instead of the recursive split)."""
    from verinf_amd.prover.protocol import blake3_digest
    for c in _kat():
        data = bytes(i % 251 for i in range(c["len"]))
        assert blake3_digest(data).hex() == c["hash"], c["len"]


def test_blake3_oracle_vs_host_random_lengths():
    from verinf_amd.prover.protocol import blake3_digest
    rng = np.random.default_rng(11)
    for n in [2, 63, 65, 127, 128, 129, 1023, 1026, 3 * 1024 - 1, 6 * 1024, 6 * 1024 + 1, 11 * 1024 + 5, 16 * 1024, 17 * 1024 + 64]:
        data = rng.integers(0, 256, n, dtype=np.uint8).tobytes()
        assert O.blake3(data) == blake3_digest(data), n


def test_hash_columns_is_blake3_of_packed_column():
    from verinf_amd.prover.protocol import merkle_leaf
    rng = np.random.default_rng(12)
    for m, n in [(0, 3), (1, 5), (7, 4), (8, 4), (128, 3), (129, 3), (300, 2), (1024, 2)]:
        mat = rng.integers(0, 1 << 63, (m, n), dtype=np.uint64) * np.uint64(2) + rng.integers(0, 2, (m, n), dtype=np.uint64)
        dig = O.hash_columns(mat)
        for j in range(n):
            col = [int(v) for v in mat[:, j]]
            packed = b"".join(v.to_bytes(8, "little") for v in col)
            assert dig[j].tobytes() == O.blake3(packed)
            assert dig[j].tobytes() == merkle_leaf(col)


def test_merkle_levels_and_paths_verify():
    from verinf_amd.layergkr import rs
    from verinf_amd.prover.protocol import blake3_digest, merkle_verify
    rng = np.random.default_rng(13)
    for k in [1, 2, 3, 5, 8, 13]:
        leaves = rng.integers(0, 256, (k, 32), dtype=np.uint8)
        levels = O.merkle_levels(leaves)
        host = rs.build_tree([leaves[i].tobytes() for i in range(k)])
        assert len(levels) == len(host)
        for lv, hv in zip(levels, host):
            assert [lv[i].tobytes() for i in range(lv.shape[0])] == hv
        # definition, spelled out once: parent 0 of the first level
        if k >= 2:
            assert host[1][0] == blake3_digest(leaves[0].tobytes() + leaves[1].tobytes())
        if k % 2 == 1 and k > 1:
            assert host[1][-1] == blake3_digest(leaves[-1].tobytes() * 2)
        root = host[-1][0]
        for idx in range(k):
            path = rs.merkle_path(host, idx)
            assert merkle_verify(host[0][idx], path, root)
            if path:
                bad = [(bytes(32), path[0][1])] + path[1:]
                assert not merkle_verify(host[0][idx], bad, root)


def test_row_prg_is_the_stated_hash():
    """Definition spelled out with the independent host hash: first 8 digest bytes, little
    endian, mod p, of seed || row_le8 || k_le8; rows count in uint32 in the contiguous form."""
    from verinf_amd.prover.protocol import blake3_digest
    seed = bytes(range(7, 39))
    out = O.row_prg(seed, 5, 3, 4)
    for r in range(3):
        for k in range(4):
            d = blake3_digest(seed + (5 + r).to_bytes(8, "little") + k.to_bytes(8, "little"))
            assert int(out[r, k]) == int.from_bytes(d[:8], "little") % P
    idx = np.array([0, 5, (1 << 40) + 3], dtype=np.uint64)
    ind = O.row_prg(seed, 0, 0, 2, row_indices=idx)
    assert np.array_equal(ind[1], out[0, :2])
    d = blake3_digest(seed + ((1 << 40) + 3).to_bytes(8, "little") + (1).to_bytes(8, "little"))
    assert int(ind[2, 1]) == int.from_bytes(d[:8], "little") % P
    wrap = O.row_prg(seed, (1 << 32) - 1, 2, 1)          # row (2^32 - 1) + 1 wraps to 0
    assert np.array_equal(wrap[1], O.row_prg(seed, 0, 1, 1)[0])


# ---- multilinear helpers ---------------------------------------------------------------
def test_eq_vector_product_formula_and_invariants():
    rng = random.Random(21)
    for n in [0, 1, 2, 3, 5, 9]:
        z = [rng.randrange(P) for _ in range(n)]
        eq = O.eq_vector(z)
        assert eq.shape == (1 << n,)
        # closed form, z[j] on index bit j (what the reference's doubling loop yields)
        for i in rng.sample(range(1 << n), min(1 << n, 12)):
            want = 1
            for j in range(n):
                want = want * (z[j] if (i >> j) & 1 else (1 - z[j])) % P
            assert int(eq[i]) == want
        assert sum(int(v) for v in eq) % P == 1          # a partition of unity
    # at a Boolean point eq is the indicator of that index
    bits = [1, 0, 1, 1]
    eq = O.eq_vector(bits)
    idx = sum(b << j for j, b in enumerate(bits))
    assert [int(v) for v in eq] == [1 if i == idx else 0 for i in range(16)]


def test_mle_eval_matches_definition():
    rng = random.Random(22)
    for n in [1, 3, 6]:
        f = np.array([rng.randrange(P) for _ in range(1 << n)], dtype=np.uint64)
        pt = [rng.randrange(P) for _ in range(n)]
        got = O.mle_eval(f, pt)
        assert got == O.py_mle_eval([int(v) for v in f], pt)
        # = <f, eq> with the point reversed (mle_eval counts variables from the top bit)
        eq = O.eq_vector(pt[::-1])
        assert got == sum(int(a) * int(b) for a, b in zip(f, eq)) % P
        # Boolean points read the table
        i = rng.randrange(1 << n)
        assert O.mle_eval(f, [(i >> (n - 1 - j)) & 1 for j in range(n)]) == int(f[i])


# ---- combiner challenge, CSR matvec, multiplicities --------------------------------------
def test_challenge_is_the_stated_prf():
    from verinf_amd.prover.protocol import blake3_digest
    seed = bytes((5 * i + 1) % 256 for i in range(32))
    for label in (b"", b"lin", b"irs", b"quad", b"12345678"):
        got = O.challenge_vec(seed, label, 5)
        for i in range(5):
            d = blake3_digest(seed + label + i.to_bytes(8, "little"))
            assert int(got[i]) == int.from_bytes(d[:16], "little") % P
        cids = [7, 1 << 40, (1 << 64) - 1]
        at = O.challenge_vec(seed, label, cids=cids)
        for c, v in zip(cids, at):
            d = blake3_digest(seed + label + c.to_bytes(8, "little"))
            assert int(v) == int.from_bytes(d[:16], "little") % P


def test_spmv_and_multiplicities_match_python():
    rng = random.Random(31)
    n_rows, n_cols = 40, 90
    rows = [[(rng.randrange(n_cols), rng.randrange(P)) for _ in range(rng.randrange(0, 9))] for _ in range(n_rows)]
    row_ptr, col, val = [0], [], []
    for r in rows:
        for c, v in r:
            col.append(c); val.append(v)
        row_ptr.append(len(col))
    x = [rng.randrange(P) for _ in range(n_cols)]
    got = O.spmv(np.array(val, dtype=np.uint64), np.array(col, dtype=np.uint64), np.array(row_ptr, dtype=np.uint64),
                 np.array(x, dtype=np.uint64))
    assert [int(v) for v in got] == [sum(v * x[c] for c, v in r) % P for r in rows]
    seed = bytes(range(32))
    r_vec = O.challenge_vec(seed, b"lin", n_cols)
    got_c = O.spmv(np.array(val, dtype=np.uint64), np.array(col, dtype=np.uint64), np.array(row_ptr, dtype=np.uint64),
                   None, seed, b"lin")
    assert [int(v) for v in got_c] == [sum(v * int(r_vec[c]) for c, v in r) % P for r in rows]
    table = [3, 9, 4, 9, 100]                       # a duplicate entry: the first one collects
    xs = [9, 9, 3, 5, 100, 4, 4, 4, 77]
    assert [int(v) for v in O.lookup_multiplicities(xs, table)] == [1, 2, 3, 0, 1]

"""Writes the small golden fixtures under tests/golden/ from FIRST PRINCIPLES:
Python big-int arithmetic straight from the mathematical definitions (a*b % p, the
DFT sum, the Lagrange closed form, the sumcheck sum).  It imports neither the C
oracle nor the upstream code, so the fixtures pin both the oracle and the HIP path.

The seeds and case lists mirror the ones the upstream tests draw on the fly
(it stores no vector files of its own for this path):
  field    prover/ref/goldilocks_ref.py:166-192   11 edge pairs + 50 pairs from Random(42)
  ntt      prover/ref/goldilocks_ref.py:195-210   Random(123), n = 1024 (here via the O(n^2) sum)
  lde      layergkr/gpu.py:206-224                Random(2), 4 rows, geometries of layergkr/tests/test_gpu.py:21-23
  sumcheck layergkr/sumcheck.py:141-149           Random(1), two 64-long factors, 6 coins
           layergkr/tests/test_sumcheck.py:27-36  N_VARS=4, seeds 17/23, coin seed 99

Run:  python tests/golden/make_fixtures.py
"""
import json
import os
import random

P = (1 << 64) - (1 << 32) + 1
G = 7
HERE = os.path.dirname(os.path.abspath(__file__))


def root(n):
    return pow(G, (P - 1) // n, P)


def dft(a):
    n = len(a)
    w = root(n)
    out = []
    for k in range(n):
        wk = pow(w, k, P)
        acc, cur = 0, 1
        for x in a:
            acc += x * cur
            cur = cur * wk % P
        out.append(acc % P)
    return out


def lagrange(K, c, eta):
    zc = pow(root(K), c, P)
    return zc * (pow(eta, K, P) - 1) % P * pow(K * (eta - zc) % P, -1, P) % P


def lde_dense(msg, K, N):
    wn = root(N)
    zs = [pow(root(K), c, P) for c in range(len(msg))]
    out = []
    for j in range(N):
        eta = G * pow(wn, j, P) % P
        num = (pow(eta, K, P) - 1) % P
        acc = 0
        for c, v in enumerate(msg):
            acc += v * (zs[c] * num % P * pow(K * (eta - zs[c]) % P, -1, P) % P)
        out.append(acc % P)
    return out


def sumcheck(tables, terms, coins):
    cur = [list(t) for t in tables]
    deg = max(len(fs) for _, fs in terms)
    claim = 0
    for i in range(len(cur[0])):
        for c, fs in terms:
            prod = c
            for j in fs:
                prod = prod * cur[j][i] % P
            claim += prod
    samples, rnd = [], 0
    while len(cur[0]) > 1:
        half = len(cur[0]) // 2
        row = []
        for x in range(deg + 1):
            acc = 0
            for c, fs in terms:
                for i in range(half):
                    prod = c
                    for j in fs:
                        f = cur[j]
                        prod = prod * ((f[i] + x * (f[half + i] - f[i])) % P) % P
                    acc += prod
            row.append(acc % P)
        samples.append(row)
        r = coins[rnd] % P
        cur = [[(f[i] + r * (f[half + i] - f[i])) % P for i in range(half)] for f in cur]
        rnd += 1
    return claim % P, samples, [f[0] for f in cur]


def hx(v):
    return [format(x, "016x") for x in v]


def main():
    # ---- field -------------------------------------------------------------
    rng = random.Random(42)
    cases = [(0, 0), (1, 0), (0, 1), (1, 1), (P - 1, 1), (P - 1, P - 1), (0, 1), (1, 2),
             (P - 1, P - 1), (1 << 32, 1 << 32), (1 << 63, 1 << 63)]
    cases += [(rng.randrange(P), rng.randrange(P)) for _ in range(50)]
    cases += [(0xFFFFFFFF00000000, 0xFFFFFFFF00000000), (P - 1, 2), ((1 << 32) - 1, (1 << 32) + 1),
              (0xFFFFFFFF, 0xFFFFFFFF00000000)]
    field = [{"a": format(a, "016x"), "b": format(b, "016x"),
              "add": format((a + b) % P, "016x"), "sub": format((a - b) % P, "016x"),
              "mul": format(a * b % P, "016x")} for a, b in cases]
    json.dump(field, open(os.path.join(HERE, "field_vectors.json"), "w"), indent=0)

    # ---- ntt ---------------------------------------------------------------
    rng = random.Random(123)
    a = [rng.randrange(P) for _ in range(1024)]
    json.dump({"n": 1024, "input": hx(a), "forward": hx(dft(a))},
              open(os.path.join(HERE, "ntt_1024.json"), "w"))

    # ---- coset LDE ---------------------------------------------------------
    lde = []
    for ELL, K, N in [(16, 32, 64), (64, 128, 256), (256, 512, 1024)]:
        r = random.Random(2)
        rows = 4 if N <= 256 else 2
        msgs = [[r.randrange(P) for _ in range(ELL)] for _ in range(rows)]
        lde.append({"ELL": ELL, "K": K, "N": N, "shift": G,
                    "messages": [hx(m) for m in msgs],
                    "codewords": [hx(lde_dense(m, K, N)) for m in msgs]})
    json.dump(lde, open(os.path.join(HERE, "coset_lde.json"), "w"))

    # ---- sumcheck ----------------------------------------------------------
    sc = []
    rr = random.Random(1)
    f = [[rr.randrange(P) for _ in range(64)] for _ in range(2)]
    coins = [rr.randrange(P) for _ in range(6)]
    terms = [(1, [0, 1]), (P - 1, [0])]
    claim, samples, finals = sumcheck(f, terms, coins)
    sc.append({"name": "gate_instance", "tables": [hx(t) for t in f],
               "terms": [[format(c, "016x"), fs] for c, fs in terms], "coins": hx(coins),
               "claim": format(claim, "016x"), "samples": [hx(s) for s in samples],
               "finals": hx(finals)})
    for k, seed in ((2, 17), (3, 23)):
        r = random.Random(seed)
        f = [[r.randrange(P) for _ in range(16)] for _ in range(k)]
        rc = random.Random(99)
        coins = [rc.randrange(P) for _ in range(4)]
        terms = [(1, list(range(k)))]
        claim, samples, finals = sumcheck(f, terms, coins)
        sc.append({"name": f"product_deg{k}", "tables": [hx(t) for t in f],
                   "terms": [[format(c, "016x"), fs] for c, fs in terms], "coins": hx(coins),
                   "claim": format(claim, "016x"), "samples": [hx(s) for s in samples],
                   "finals": hx(finals)})
    json.dump(sc, open(os.path.join(HERE, "sumcheck.json"), "w"))
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()

"""No-GPU checks: the C-ABI library loads and exports every declared symbol, argument
validation answers without touching a device, and the host-side logic of the
package (domains, Lagrange form, verifier, mask algebra) is right."""
import ctypes
import os
import random
import re

import numpy as np
import pytest

from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = O.P


@pytest.fixture(scope="module")
def L():
    from verinf_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from verinf_amd.build import build
        build()
    return _lib.lib()


def test_library_exports_every_declared_symbol(L):
    hdr = open(os.path.join(ROOT, "include", "verinf_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = sorted(set(re.findall(r"\b(vi_[a-z0-9_]+)\s*\(", hdr)))
    assert len(names) >= 17
    from verinf_amd import _lib
    assert sorted(_lib.EXPORTS) == names
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n
    assert L.vi_version() == b"0.2"


def test_size_queries_and_argument_validation_without_a_device(L):
    assert L.vi_ntt_workspace_bytes(4, 1 << 9) == 0
    assert L.vi_ntt_workspace_bytes(4, 1 << 12) == (4 * (1 << 12) * 8 if os.environ.get("VI_NTT_ROW", "1")[:1] == "0" else 0)
    assert L.vi_ntt_workspace_bytes(4, 1 << 13) == 4 * (1 << 13) * 8
    assert L.vi_ntt_workspace_bytes(4, 1 << 16) == 4 * (1 << 16) * 8
    assert L.vi_ntt_workspace_bytes(4, 12) == 0
    one = L.vi_coset_lde_min_workspace_bytes(1 << 16, 1 << 18)
    assert one == (1 << 16) * 8 * 5
    assert L.vi_coset_lde_min_workspace_bytes(1 << 10, 1 << 12) == (1 << 10) * 8 * 5
    assert L.vi_coset_lde_min_workspace_bytes(1 << 8, 1 << 10) == (1 << 8) * 8
    assert L.vi_coset_lde_workspace_bytes(1024, 1 << 16, 1 << 18) % one == 0
    assert L.vi_coset_lde_min_workspace_bytes(24, 96) == 0
    assert L.vi_sumcheck_workspace_bytes() > 0
    # bad arguments are refused before any HIP call
    assert L.vi_gl_binop(7, None, None, None, 4, None) == -1 and b"op" in L.vi_last_error()
    assert L.vi_ntt_batched(None, 1, 12, 0, None, 0, None) == -1 and b"power of 2" in L.vi_last_error()
    assert L.vi_coset_lde(None, 1, 8, 8, 8, 4, 7, None, 4, None, 0, None) == -1
    assert L.vi_coset_lde(None, 1, 9, 9, 8, 32, 7, None, 32, None, 0, None) == -1
    assert L.vi_kquant_to_field(8, None, 1, 4096.0, None, None) == -1 and b"qtype" in L.vi_last_error()
    assert L.vi_gl_binop(0, None, None, None, 0, None) == 0
    assert L.vi_ntt_batched(None, 0, 16, 0, None, 0, None) == 0
    # sumcheck term lists of any length are checked on the host: here 100 tables and 100 terms (beyond one kernel
    # descriptor), with one defect each
    n = 100
    fake = (ctypes.c_void_p * n)(*[0x1000 + 8 * i for i in range(n)])             # never dereferenced
    ws, out = ctypes.c_void_p(0x2000), ctypes.c_void_p(0x3000)
    ws_bytes = L.vi_sumcheck_workspace_bytes()

    def sc_eval(offsets, indices, tables=fake, n_tables=n, half=8):
        off = (ctypes.c_int * len(offsets))(*offsets)
        idx = (ctypes.c_int * max(len(indices), 1))(*indices)
        co = (ctypes.c_uint64 * (len(offsets) - 1))(*([1] * (len(offsets) - 1)))
        return L.vi_sumcheck_eval(tables, n_tables, half, off, idx, co, len(offsets) - 1, out, ws, ws_bytes, None)

    good_off, good_idx = list(range(0, 2 * n + 1, 2)), [j % n for j in range(2 * n)]
    assert sc_eval(good_off, good_idx[:-1] + [n]) == -1 and b"factor index" in L.vi_last_error()
    assert sc_eval(good_off[:-1] + [2 * n + 7], good_idx + [0] * 7) == -1 and b"factors" in L.vi_last_error()
    assert sc_eval([1] + good_off[1:], good_idx) == -1 and b"term_off" in L.vi_last_error()
    assert sc_eval(good_off, good_idx, half=0) == -1 and b"half" in L.vi_last_error()
    holed = (ctypes.c_void_p * n)(*[0 if i == 57 else 0x1000 + 8 * i for i in range(n)])
    assert sc_eval(good_off, good_idx, tables=holed) == -1 and b"null table 57" in L.vi_last_error()
    assert L.vi_sumcheck_eval_static(fake, n, 8, (ctypes.c_int * (n + 1))(*good_off), (ctypes.c_int * (2 * n))(*good_idx),
                                     (ctypes.c_uint64 * n)(*([1] * n)), n, out, None) != 0
    # the proof with all challenges up front: sizes, workspace, pointers and terms are checked before any launch
    assert L.vi_sumcheck_prove_coins_workspace_bytes(1 << 26) == 27 * 2048 * 8 * 8
    assert L.vi_sumcheck_prove_coins_workspace_bytes(24) == 0

    def prove(size, ws_bytes=None, work=fake, chal=True, offsets=good_off, indices=good_idx):
        off = (ctypes.c_int * len(offsets))(*offsets)
        idx = (ctypes.c_int * len(indices))(*indices)
        co = (ctypes.c_uint64 * (len(offsets) - 1))(*([1] * (len(offsets) - 1)))
        ch = (ctypes.c_uint64 * 64)(*([5] * 64)) if chal else None
        need = L.vi_sumcheck_prove_coins_workspace_bytes(size) if ws_bytes is None else ws_bytes
        return L.vi_sumcheck_prove_coins(fake, work, n, size, off, idx, co, len(offsets) - 1, ch, out, ws, need, None)

    assert prove(24) == -1 and b"power of two" in L.vi_last_error()
    assert prove(1) == -1
    assert prove(1 << 41) == -1 and b"rounds" in L.vi_last_error()
    assert prove(1 << 10, ws_bytes=1024) == -3 and b"workspace" in L.vi_last_error()
    assert prove(1 << 10, chal=False) == -1 and b"null" in L.vi_last_error()
    assert prove(1 << 10, work=holed) == -1 and b"null work buffer 57" in L.vi_last_error()
    assert prove(1 << 10, indices=good_idx[:-1] + [n]) == -1 and b"factor index" in L.vi_last_error()
    # vi_sumcheck_prove states the size of its pinned buffer
    coin = _lib_coin()
    assert L.vi_sumcheck_prove(fake, fake, n, 1 << 10, (ctypes.c_int * (n + 1))(*good_off), (ctypes.c_int * (2 * n))(*good_idx),
                               (ctypes.c_uint64 * n)(*([1] * n)), n, coin, None, out, 8, (ctypes.c_uint64 * 64)(),
                               (ctypes.c_uint64 * 16)(), ws, ws_bytes, None) == -1
    assert b"host_samples holds 8 words" in L.vi_last_error()


def _lib_coin():
    from verinf_amd import _lib
    return _lib.COIN_FN(lambda rnd, samples, n, r_out, user: 1)


def test_missing_library_fails_loudly(monkeypatch):
    from verinf_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libverinf_hip.so")
    with pytest.raises(_lib.VerinfHipError):
        _lib.lib()


def test_no_gpu_means_an_error_not_a_cpu_path():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from verinf_amd.layergkr import gpu, rs, sumcheck
    cfg = rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4)
    with pytest.raises(RuntimeError):
        gpu.encode_batch_ntt(cfg, [[1, 2, 3]])
    with pytest.raises(RuntimeError):
        rs.Commit.from_messages(cfg, [[1, 2, 3]])
    with pytest.raises(RuntimeError):
        sumcheck.prove([[1, 2], [3, 4]], lambda i: 5)
    with pytest.raises(RuntimeError):
        gpu.prove_terms_gpu([(1, [[1, 2], [3, 4]])], lambda i: 5, P)


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "verinf_amd")
    pat = re.compile(r"^\s*(from|import)\s+oracle\b|#include.*oracle|vi_oracle|libvi_oracle", re.M)
    for dp, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                assert not pat.search(open(os.path.join(dp, f)).read()), (dp, f)


def test_protocol_domains_and_lagrange_form():
    from verinf_amd.prover import protocol as pr
    cfg = pr.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4)
    assert pow(cfg.W_K, 32, P) == 1 and pow(cfg.W_K, 16, P) == P - 1
    assert cfg.eta(0) == 7 and cfg.zeta(1) == cfg.W_K
    r = random.Random(3)
    msg = [r.randrange(P) for _ in range(16)]
    want = O.lde_dense_row(np.array(msg, dtype=np.uint64), 32, 64, 7)
    for j in (0, 1, 17, 63):
        assert pr.eval_zeta_form(cfg, msg, cfg.eta(j)) == int(want[j])
    assert pr.lagrange(cfg, 5, cfg.eta(9)) == O.py_lagrange(32, 5, cfg.eta(9))
    assert pr.poly_eval([1, 2, 3], 5) == 1 + 10 + 75 and pr.inv(7) * 7 % P == 1


def test_host_verifier_accepts_oracle_proofs_and_rejects_tampering():
    from verinf_amd.layergkr import sumcheck as sc
    r = random.Random(4)
    n = 32
    tabs = [[r.randrange(P) for _ in range(n)] for _ in range(3)]
    terms_idx = [(3, [0, 1, 2]), (P - 1, [1]), (9, [2, 2])]
    coins = [r.randrange(P) for _ in range(5)]
    claim, samples, _ = O.py_sumcheck(tabs, terms_idx, coins)
    terms = [(c, [tabs[i] for i in fs]) for c, fs in terms_idx]
    pf = sc.SumcheckProof(claim=claim, round_polys=[list(enumerate(s)) for s in samples],
                          challenges=list(coins), final_point=list(coins))
    ok, why = sc.verify_terms(pf, terms, lambda i: coins[i])
    assert ok, why
    pf.round_polys[2][1] = (1, (pf.round_polys[2][1][1] + 1) % P)
    assert not sc.verify_terms(pf, terms, lambda i: coins[i])[0]
    assert sc.mle_eval(tabs[0], coins) == O.py_mle_eval(tabs[0], coins)
    assert sc._fold([1, 2, 3, 4], 5) == [11, 12]
    for d in (1, 2, 3, 4):
        mu = r.randrange(P)
        u = [r.randrange(P) for _ in range(d)]
        h = sc.mask_poly_coeffs(mu, u)
        assert (sc.poly_eval_coeffs(h, 0) + sc.poly_eval_coeffs(h, 1)) % P == mu
        assert sc.solve_tape_for_target(mu, h) == u
        bad = list(h)
        bad[0] = (bad[0] + 1) % P
        assert sc.solve_tape_for_target(mu, bad) is None
    assert sc.masked_product_ok(3, 4, 5, 6, 7)
    tp = sc.MaskTape([1, 2, 3])
    assert tp.take(2) == [1, 2]
    with pytest.raises(RuntimeError):
        tp.take(2)


def test_commit_host_helpers_of_rs():
    """The host side of layergkr/rs.py: the challenge PRF against the oracle's, distinct column sampling, the
    Python-integer linear combination, and a host tree whose opening paths verify (odd levels included)."""
    from verinf_amd.layergkr import rs
    from verinf_amd.prover import protocol as pr
    seed = bytes(range(32))
    want = O.challenge_vec(seed, b"cols", 40)
    assert [pr.challenge(seed, i, "cols") for i in range(40)] == [int(v) for v in want]
    assert pr.challenge(5, 3, "lin") == int(O.challenge_vec((5).to_bytes(32, "little"), b"lin", 4)[3])
    assert pr.challenge(b"ab", 0, "x") == pr.challenge(b"ab" + bytes(30), 0, "x")
    cols = rs.sample_columns(seed, 12, 16)
    assert len(cols) == len(set(cols)) == 12 and all(0 <= c < 16 for c in cols)
    draws = [pr.challenge(seed, i, "cols") % 16 for i in range(200)]
    assert cols == list(dict.fromkeys(draws))[:12]           # first occurrences, in draw order
    assert rs.sample_columns(seed, 16, 16) == list(dict.fromkeys(draws))[:16]
    with pytest.raises(ValueError):
        rs.sample_columns(seed, 17, 16)
    cfg = rs.Config(ELL=16, K_DEG=32, N_LIG=64, T_QUERIES=4)
    r = random.Random(6)
    cws = [[r.randrange(P) for _ in range(64)] for _ in range(5)]
    co = [r.randrange(P) for _ in range(4)] + [0]
    assert rs.linear_combination(cfg, cws, co) == [sum(a * cw[j] for a, cw in zip(co, cws)) % P for j in range(64)]
    with pytest.raises(ValueError):
        rs.linear_combination(cfg, cws, co[:3])
    for n in (1, 2, 5, 8, 11):
        leaves = [pr.blake3_digest(bytes([i])) for i in range(n)]
        tree = rs.build_tree(leaves)
        assert tree[0] == leaves and len(tree[-1]) == 1
        want_levels = O.merkle_levels(np.frombuffer(b"".join(leaves), dtype=np.uint8).reshape(n, 32))
        assert [len(l) for l in tree] == [len(l) for l in want_levels]
        assert tree[-1][0] == want_levels[-1][0].tobytes()
        for i in range(n):
            path = rs.merkle_path(tree, i)
            assert pr.merkle_verify(leaves[i], path, tree[-1][0])
            if path:
                sib, side = path[0]
                assert not pr.merkle_verify(leaves[i], [(sib, 1 - side)] + path[1:], tree[-1][0]) or sib == leaves[i]


def test_bench_refuses_more_than_one_gpu():
    """This build runs on one GPU; bench.py says so instead of starting ranks."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "ONE GPU" in res.stderr


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/verinf_hip.h is a C header (no C++ or torch types): it compiles as C99 and as C++,
    and a C program that includes it links against the library and can call the entry points
    that need no device (version string, workspace queries, argument validation)."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hdr = os.path.join(root, "include", "verinf_hip.h")
    lib = os.path.join(root, "verinf_amd", "libverinf_hip.so")
    if not os.path.exists(lib):
        from verinf_amd.build import build
        build()
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", hdr])
    subprocess.check_call(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", hdr])
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "verinf_hip.h"
int main(void) {
    if (!vi_version() || !strlen(vi_version())) return 1;
    if (vi_coset_lde_workspace_bytes(1024, 65536, 262144) == 0) return 2;
    if (vi_coset_lde_min_workspace_bytes(65536, 262144) != (size_t)(65536 + 262144) * 8) return 3;
    if (vi_hash_columns_workspace_bytes(1024, 262144) != (size_t)(8 + 4) * 262144 * 32) return 4;
    if (vi_sumcheck_workspace_bytes() == 0 || vi_mle_eval_workspace_bytes(3) != 3 * 8192) return 5;
    /* bad arguments are refused before anything touches a device */
    static uint64_t dummy[4];     /* never dereferenced: K = 12 is refused first */
    if (vi_coset_lde(dummy, 4, 3, 3, 12, 48, 7, dummy, 48, 0, 0, 0) != VI_EINVAL) return 6;
    if (!strstr(vi_last_error(), "powers of two")) return 7;
    if (vi_kquant_to_field(8, 0, 1, 4096.0, 0, 0) != VI_EINVAL) return 8;
    if (vi_row_prg(0, 0, 0, 4, 4, 0, 2, 0) != VI_EINVAL) return 9;
    puts(vi_version());
    return 0;
}
''')
    exe = tmp_path / "abi"
    hip_lib_dir = "/opt/rocm/lib"
    subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(root, "include"), str(src), "-o", str(exe), lib,
                           "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath," + hip_lib_dir, "-L" + hip_lib_dir, "-lamdhip64"])
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, (res.returncode, res.stdout, res.stderr)

"""Headline benchmark: batched Goldilocks coset LDE, 1024 rows x 2^16 -> 2^18, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" = one pass of the hot path over one batch of synthetic input: the coset
low-degree extension of 1024 seeded rows of 2^16 field elements to 2^18 (the second of the
benchmark configurations), input and output resident in HBM.  Prints ONE JSON line with the
metric (output elements per second), the roofline of the dominant kernel and a CPU
baseline (the C oracle on the host cores, bounded sample, same inputs, outputs
compared bit for bit with the GPU's).  The sumcheck, K-quant, column-hash and
Llama-2-7B-layer legs of the same run are reported under "extra".

    python bench.py --copy-probe      plain device copy of known size (calibrates the
                                      FETCH_SIZE / WRITE_SIZE counters, see profiles/)
"""
import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

P = (1 << 64) - (1 << 32) + 1
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published


# HBM bytes of one step of the default LDE leg (its six launches together: per 512-row chunk the strided inverse
# pass, the fused last-inverse / first-forward launch k_lde_mid, and the final forward pass): FETCH_SIZE and
# WRITE_SIZE read by rocprofv3 in two counter runs of this script, each scaled by what the same counter reads for a
# 1 GiB device copy (x 2.000 / x 1.000): 3.23 GB read + 4.83 GB written per step
# (profiles/k_lde_mid_k_ntt_fast__coset_lde_1024x2p16_to_2p18.md).  roofline.traffic is this figure divided by the
# launches of a step, like roofline.achieved.
LDE_TRAFFIC_BYTES_PER_STEP = 8.06e9
# VALU wave-instructions one LDE step issues (rocprofv3 --pmc SQ_INSTS_VALU, same profile: per 512-row chunk 58.7 M in
# the strided inverse launch, 290.1 M in k_lde_mid and 188.1 M in the final forward launch) and the rate at which
# 1024 SIMDs issue the instruction classes these kernels consist of (carry, multiply, three-operand and shift
# instructions: one per 4.16 cycles per SIMD, measured by `bench.py --valu-probe`,
# profiles/valu_issue_rates__probe.md) at the 2.4 GHz peak clock
LDE_VALU_INSTS_PER_STEP = 2 * (58_785_792 + 290_095_104 + 188_481_536)
VALU_ISSUE_CYCLES_PER_INSTR = 4.16
VALU_ISSUE_PEAK_PER_S = 256 * 4 * 2.4e9 / VALU_ISSUE_CYCLES_PER_INSTR


def _events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def rand_field(torch, shape, seed):
    """Seeded field elements on the device, uniform in [0, p): 64 random bits, and the 2^32 - 1 words at or
    above p taken down by p (as tests/gpu_util.py does with `% p`)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    v = torch.randint(-(1 << 63), (1 << 63) - 1, shape, generator=g, dtype=torch.int64, device="cuda")
    # as unsigned words, [p, 2^64) is the signed range [-(2^32 - 1), -1]; x - p = x + 2^32 - 1 mod 2^64
    v = torch.where((v < 0) & (v >= -((1 << 32) - 1)), v + ((1 << 32) - 1), v)
    return v.view(torch.uint64)


def bench_lde(torch, steps, warmup, ws_mb=0):
    from verinf_amd import _lib
    m, K, N = 1024, 1 << 16, 1 << 18
    msgs = rand_field(torch, (m, K), 0)
    out = torch.empty((m, N), dtype=torch.uint64, device="cuda")
    L = _lib.lib()
    # the library's own default workspace (what cuda_primitives.coset_lde passes), or an override
    ws_bytes = (ws_mb << 20) if ws_mb else L.vi_coset_lde_workspace_bytes(m, K, N)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    stream = _lib.stream_ptr()

    def step():
        _lib.check(L.vi_coset_lde(msgs.data_ptr(), m, K, K, K, N, 7, out.data_ptr(), N, ws.data_ptr(),
                                  ws_bytes, stream))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # one event pair around the K timed steps (the reported figure) and an event after every step,
    # on the stream the kernels run on, for the spread between steps
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    marks[0].record()
    for i in range(steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    ms = marks[0].elapsed_time(marks[steps]) / steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    q = lambda f: per_step[min(steps - 1, int(f * steps))]
    launches = int(L.vi_coset_lde_launches(m, K, N, ws_bytes))
    alg_bytes = 8 * (K + N) * m                       # compulsory traffic of one step
    res = {
        "ms_per_step": ms,
        "ms_per_step_median": q(0.5), "ms_per_step_iqr": [q(0.25), q(0.75)],
        "elems_per_s": m * N / (ms * 1e-3),
        "launches_per_step": launches,
        "kernel_avg_us": ms * 1e3 / launches,
        "alg_bytes_per_launch": alg_bytes / launches,
        "achieved_gbs": alg_bytes / (ms * 1e-3) / 1e9,
    }
    return res, msgs, out


def cpu_baseline_lde(torch, msgs, out, rows, reps):
    """C oracle (radix-2 iNTT -> twist -> zero-extend -> NTT per row, OpenMP over rows)
    on the first `rows` rows of the same input, `reps` times; also the bit-exact check of
    the GPU output."""
    import numpy as np
    from oracle import oracle as O
    K, N = msgs.shape[1], out.shape[1]
    sample = msgs[:rows].cpu().numpy()
    O.coset_lde_rows(sample[:2], K, N, 7)             # warm the library / page in
    t0 = time.perf_counter()
    for _ in range(reps):
        want = O.coset_lde_rows(sample, K, N, 7)
    dt = time.perf_counter() - t0
    got = out[:rows].cpu().numpy()
    return {"value": reps * rows * N / dt, "unit": "elem/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"first {rows} of the 1024 rows, 2^16 -> 2^18, {reps} passes, {dt:.2f} s wall",
            "bit_exact_vs_gpu": bool(np.array_equal(got, want))}


def _time_proof(torch, gpu, terms, coin, reps=24):
    """-> (best wall ms incl. the read-back of the samples, best device ms by HIP events) of prove_terms_gpu"""
    wall, dev = [], []
    s, e = _events(torch)
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        s.record()
        out = gpu.prove_terms_gpu(terms, coin, P)
        e.record()
        torch.cuda.synchronize()
        wall.append((time.perf_counter() - t0) * 1e3)
        dev.append(s.elapsed_time(e))
    return min(wall), min(dev), out


def bench_sumcheck(torch, v=26, cpu=True):
    """Config 4: three 2^26 tables, degree 3, 26 rounds, all challenges drawn before the proof starts (the
    reference's coin takes the round number only): the whole proof is queued on the stream, three rounds per pass
    over the tables."""
    from verinf_amd.layergkr import gpu
    tabs = [rand_field(torch, (1 << v,), 10 + j) for j in range(3)]
    r = random.Random(1)
    coins = [r.randrange(P) for _ in range(v)]
    coin = lambda i: coins[i]
    gpu.prove_terms_gpu([(1, tabs)], coin, P)            # warm-up
    wall, dev, (claim, polys, _, _) = _time_proof(torch, gpu, [(1, tabs)], coin)
    n = 1 << v
    # bytes this schedule moves: a pass reads the tables once and writes an eighth of them (three rounds), until a
    # single workgroup holds them; against 96 N for one fused fold + evaluation launch per round, the figure the
    # per-round rates of earlier builds were quoted on
    moved, size = 0, n
    while size > 4096:
        moved += 3 * 8 * (size + size // 8)
        size //= 8
    moved += 3 * 8 * size
    res = {"total_ms": wall, "device_ms": dev,
           "table_bytes_moved": moved, "moved_gbs": moved / (dev * 1e-3) / 1e9,
           "frac_of_hbm_peak": moved / (dev * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "proof_gbs_per_round_schedule": 96 * n / (wall * 1e-3) / 1e9,
           "note": "total_ms: wall clock of prove_terms_gpu incl. the read-back of all samples; device_ms: HIP events "
                   "around the same call; moved_gbs: bytes this schedule reads and writes / device_ms; "
                   "proof_gbs_per_round_schedule: the 96 N bytes of a launch-per-round schedule / total_ms"}
    # the hadamard gate batch 3 eq a b - 5 eq c (layergkr/relations.py:104-124) over 2^24: four tables, degree 3
    gv = 24
    gt = [t[: 1 << gv] for t in tabs] + [rand_field(torch, (1 << gv,), 14)]
    gterms = [(3, [gt[0], gt[1], gt[2]]), (P - 5, [gt[0], gt[3]])]
    gpu.prove_terms_gpu(gterms, coin, P)
    gw, gd, _ = _time_proof(torch, gpu, gterms, coin)
    res["hadamard_gate_4x2^24_ms"] = gw
    res["hadamard_gate_4x2^24_device_ms"] = gd
    # the matmul contractions of the layer proof: two tables, degree 2, width 2^12 and 2^14 (one launch each)
    for mv in (12, 14):
        mt = [t[: 1 << mv] for t in tabs[:2]]
        gpu.prove_terms_gpu([(1, mt)], coin, P)
        mw, md, _ = _time_proof(torch, gpu, [(1, mt)], coin)
        res[f"matmul_2x2^{mv}_ms"] = mw
    del gt, gterms
    if cpu:
        # C oracle (sumcheck.prove_terms loop, OpenMP) on the same instance, every round compared
        from oracle import oracle as O
        host = [t.cpu().numpy() for t in tabs]
        c0 = time.perf_counter()
        want_claim, want_samples, _ = O.sumcheck_prove(host, [(1, [0, 1, 2])], coins)
        dt = time.perf_counter() - c0
        res["cpu_baseline"] = {"value": 96 * n / dt / 1e9, "unit": "GB/s (96 N bytes per proof)", "ms": dt * 1e3,
                               "cores": O.num_threads(), "kind": "port",
                               "sample": f"the same 3 x 2^{v} tables, all {v} rounds, {dt:.2f} s wall",
                               "bit_exact_vs_gpu": bool(claim == want_claim and [[y for _, y in s] for s in polys] == want_samples)}
    return res


def bench_gate_batch(torch, v=22, cpu=True):
    """The gate batch of a whole layer in the shape of relations.prove_batch (layergkr/relations.py:104-124): one
    eq table in every term, lambda-weighted hadamard (eq*a*b - eq*c), rescale (three linear terms), booleanity
    (eq*b*b - eq*b) and affine gates -- 97 tables, 90 terms, degree 3, more than one kernel descriptor holds, so
    the tables are walked in memory and the terms in groups.  Proved at 2^v, checked through the verifier, and at
    2^14 compared with the C oracle round by round."""
    from verinf_amd.layergkr import gpu
    from verinf_amd.layergkr import sumcheck as sc
    r = random.Random(41)

    def problem(vv):
        tabs = [rand_field(torch, (1 << vv,), 4000)]
        terms = []

        def t():
            tabs.append(rand_field(torch, (1 << vv,), 4000 + len(tabs)))
            return len(tabs) - 1

        for kind, count in (("had", 12), ("resc", 10), ("bool", 6), ("aff", 8)):
            for _ in range(count):
                lam = r.randrange(P)
                neg = lam * (P - 1) % P
                if kind == "had":
                    a, b, c = t(), t(), t()
                    terms += [(lam, [0, a, b]), (neg, [0, c])]
                elif kind == "resc":
                    raw, q, rem = t(), t(), t()
                    terms += [(lam, [0, raw]), (lam * (P - 4096) % P, [0, q]), (neg, [0, rem])]
                elif kind == "bool":
                    b = t()
                    terms += [(lam, [0, b, b]), (neg, [0, b])]
                else:
                    x0, x1, y = t(), t(), t()
                    terms += [(lam, [0, x0]), (lam, [0, x1]), (neg, [0, y])]
        return tabs, terms

    coins = [r.randrange(P) for _ in range(v)]
    tabs, terms = problem(v)
    obj_terms = [(c, [tabs[i] for i in fs]) for c, fs in terms]
    best = None
    for _ in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        proof = sc.prove_terms(obj_terms, lambda i: coins[i])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    ok, why = sc.verify_terms(proof, obj_terms, lambda i: coins[i])
    table_bytes = len(tabs) * (8 << v)
    res = {"tables": len(tabs), "terms": len(terms), "log2_size": v, "ms": best * 1e3,
           "table_gb": table_bytes / 1e9, "verifier_accepts": bool(ok), "verifier_says": why}
    del tabs, obj_terms, proof
    if cpu:
        from oracle import oracle as O
        vs = 14
        tabs, terms = problem(vs)
        claim, polys, _, _ = gpu.prove_terms_gpu([(c, [tabs[i] for i in fs]) for c, fs in terms], lambda i: coins[i], P)
        c0 = time.perf_counter()
        want_claim, want_samples, _ = O.sumcheck_prove([x.cpu().numpy() for x in tabs], terms, coins)
        dt = time.perf_counter() - c0
        res["cpu_baseline"] = {"ms": dt * 1e3, "cores": O.num_threads(), "kind": "port",
                               "sample": f"the same batch at 2^{vs}",
                               "bit_exact_vs_gpu": bool(claim == want_claim and [[y for _, y in s] for s in polys] == want_samples)}
    return res


def bench_kquant(torch, steps=20, cpu=True):
    from verinf_amd.prover import kquant_cuda as kq
    nb = 4096 * 11008 // 256
    g = torch.Generator(device="cuda").manual_seed(3)
    raw = torch.randint(0, 256, (nb, 144), generator=g, dtype=torch.uint8, device="cuda")
    hd = (torch.randn((nb, 2), generator=g, device="cuda") * 0.01).abs().to(torch.float16).view(torch.uint8)
    raw[:, 0:4] = hd.reshape(nb, 4)
    # a launch is 60 us: enough of them before the clock starts that the chip is out of its idle power state
    for _ in range(3 * steps):
        kq.kquant_to_field(raw, "Q4_K", 4096)
    torch.cuda.synchronize()
    s, e = _events(torch)
    s.record()
    for _ in range(steps):
        kq.kquant_to_field(raw, "Q4_K", 4096)
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / steps
    res = {"ms": ms, "weights_per_s": nb * 256 / (ms * 1e-3), "gbs_algorithmic": nb * 2192 / (ms * 1e-3) / 1e9,
           "frac_of_hbm_peak": nb * 2192 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    for qt, bb in (("Q5_K", 176), ("Q6_K", 210)):                     # same weight count in the other two layouts
        other = torch.randint(0, 256, (nb, bb), generator=g, dtype=torch.uint8, device="cuda")
        if qt == "Q6_K":
            other[:, 208:210] = hd.reshape(nb, 4)[:, :2]
        else:
            other[:, 0:4] = hd.reshape(nb, 4)
        for _ in range(3 * steps):
            kq.kquant_to_field(other, qt, 4096)
        torch.cuda.synchronize()
        s.record()
        for _ in range(steps):
            kq.kquant_to_field(other, qt, 4096)
        e.record()
        torch.cuda.synchronize()
        t = s.elapsed_time(e) / steps
        res[qt.lower() + "_ms"] = t
        res[qt.lower() + "_gbs_algorithmic"] = nb * (bb + 2048) / (t * 1e-3) / 1e9
    # the loader's call site (prover/loader.py:427-436) wants the (k_in, n_out) transpose: one fused pass
    # against decode followed by torch's .T.contiguous()
    def two_step():
        return kq.kquant_to_field(raw, "Q4_K", 4096).view(4096, 11008).view(torch.int64).T.contiguous()
    for name, fn in (("transposed_fused_ms", lambda: kq.kquant_to_field_transposed(raw, "Q4_K", 4096, 4096)),
                     ("transposed_two_step_ms", two_step)):
        fn()
        torch.cuda.synchronize()
        s.record()
        for _ in range(steps):
            fn()
        e.record()
        torch.cuda.synchronize()
        res[name] = s.elapsed_time(e) / steps
    if cpu:
        # C oracle (scalar byte map, OpenMP over blocks) on the whole matrix, compared bit for bit
        import numpy as np
        from oracle import oracle as O
        host = raw.cpu().numpy()
        O.kquant_to_field(host[:64], "Q4_K", 4096)
        c0 = time.perf_counter()
        want = O.kquant_to_field(host, "Q4_K", 4096)
        dt = time.perf_counter() - c0
        got = kq.kquant_to_field(raw, "Q4_K", 4096).cpu().numpy()
        res["cpu_baseline"] = {"value": nb * 256 / dt, "unit": "weights/s", "cores": O.num_threads(), "kind": "port",
                               "sample": f"all {nb} super-blocks, {dt:.2f} s wall",
                               "bit_exact_vs_gpu": bool(np.array_equal(got, want))}
    return res


def bench_hash(torch, steps=10, cpu=True):
    """Column digests + Merkle tree of the headline codeword matrix (1024 x 2^18 uint64, 2 GiB):
    what turns the LDE output into a commitment root."""
    from verinf_amd.prover import cuda_primitives as cp
    m, n = 1024, 1 << 18
    g = torch.Generator(device="cuda").manual_seed(9)
    mat = torch.randint(-(1 << 63), (1 << 63) - 1, (m, n), generator=g, dtype=torch.int64, device="cuda").view(torch.uint64)
    for _ in range(steps):                              # ~10 ms of the same work before the clock starts
        dig = cp.hash_columns_streamed(mat)
        root, _ = cp.merkle_build_blake3(dig)
    torch.cuda.synchronize()
    # the steps are queued back to back (no host wait in between) with an event after each part
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record()
        dig = cp.hash_columns_streamed(mat)
        ev[i][1].record()
        root, _ = cp.merkle_build_blake3(dig)
        ev[i][2].record()
    torch.cuda.synchronize()
    t_hash = sum(a.elapsed_time(b) for a, b, _ in ev)
    t_tree = sum(b.elapsed_time(c) for _, b, c in ev)
    hash_ms, tree_ms = t_hash / steps, t_tree / steps
    alg = 8 * m * n + 32 * n
    res = {"matrix": "1024 x 2^18 uint64", "hash_columns_ms": hash_ms, "hash_gbs_algorithmic": alg / hash_ms / 1e6,
           "frac_of_hbm_peak": alg / hash_ms / 1e6 / HBM_PEAK_GBS, "merkle_tree_2^18_leaves_ms": tree_ms,
           "root": bytes(root.cpu().tolist()).hex()}
    if cpu:
        import numpy as np
        from oracle import oracle as O
        cols = 1 << 16                      # 512 MiB sample of the same matrix
        sub = mat.view(torch.int64)[:, :cols].contiguous().view(torch.uint64).cpu().numpy()
        O.hash_columns(sub[:, :64].copy())
        c0 = time.perf_counter()
        want = O.hash_columns(sub)
        dt = time.perf_counter() - c0
        res["cpu_baseline"] = {"value": sub.nbytes / dt / 1e9, "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
                               "sample": f"first {cols} columns of the same matrix, {dt:.2f} s wall",
                               "bit_exact_vs_gpu": bool(np.array_equal(dig[:cols].cpu().numpy(), want))}
    return res


def bench_ntt(torch, steps=20):
    """ntt_forward_batched / ntt_inverse_batched (prover/cuda_primitives.py:388-409) over 2^26 points as rows of
    2^8 ... 2^20: in place, round trip checked."""
    from verinf_amd.prover import cuda_primitives as cp
    res = {}
    for logn in (8, 9, 10, 11, 12, 16, 20):
        rows = rand_field(torch, (1 << (26 - logn), 1 << logn), 40 + logn)
        keep = rows.clone()
        for _ in range(steps):
            cp.ntt_forward_batched(rows)
            cp.ntt_inverse_batched(rows)
        torch.cuda.synchronize()
        s, e = _events(torch)
        s.record()
        for _ in range(steps):
            cp.ntt_forward_batched(rows)
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e) / steps
        for _ in range(steps):
            cp.ntt_inverse_batched(rows)
        torch.cuda.synchronize()
        res[f"rows_of_2^{logn}"] = {"forward_ms": ms, "points_per_s": (1 << 26) / (ms * 1e-3),
                                    "gbs_algorithmic": 16 * (1 << 26) / (ms * 1e-3) / 1e9,
                                    "round_trip_is_identity": bool(torch.equal(rows, keep))}
        del rows, keep
        torch.cuda.empty_cache()
    return res


def bench_layer(torch, check=True):
    """Config 5: one Llama-2-7B-shape layer proof core.  Commit = coset LDE of every weight
    and activation row at the production geometry ELL = 8192, K = 2^14, N = 2^16 (a row of
    n_in > 8192 values spans two rows); then the GKR sumchecks: one degree-2 contraction
    per matmul (width next_pow2(n_in), layergkr/full_layer.py:216-224) and one degree-3
    eq*a*b gate batch over S*d_ff -> 2^24 (layergkr/relations.py:104-124).  Every committed
    matrix is hashed by column and gets its Merkle root (layergkr/rs.py:176-187); the digests
    and tree of a matrix run on a second stream while the next matrix is encoded.  Random field
    tables stand in for the projected vectors of the sumchecks.

    check: after the timed regions, verify the full-shape run by samples and by properties (rows, column
    digests and roots against the CPU oracle, the codeword property on every row, every sumcheck through
    the verifier, the projection against big-integer sums); the verdicts come back under "checks"."""
    from verinf_amd.layergkr import gpu
    from verinf_amd.layergkr import sumcheck as sc
    from verinf_amd.prover import cuda_primitives as cp
    d, dff, S = 4096, 11008, 1000
    ELL, K, N = 8192, 1 << 14, 1 << 16
    g = torch.Generator(device="cuda").manual_seed(5)

    def signed_field(shape, lo, hi):
        v = torch.randint(lo, hi, shape, generator=g, dtype=torch.int64, device="cuda")
        return torch.where(v >= 0, v, v - ((1 << 32) - 1)).view(torch.uint64)   # negatives as p - |x|: p + v = 2^64 + v - (2^32 - 1)

    def rows_of(n_rows, n_in, lo, hi):
        """(n_rows, n_in) values as message rows of at most ELL slots."""
        if n_in <= ELL:
            return [signed_field((n_rows, n_in), lo, hi)]
        return [signed_field((n_rows, ELL), lo, hi), signed_field((n_rows, n_in - ELL), lo, hi)]

    weights = {"Wq": (d, d), "Wk": (d, d), "Wv": (d, d), "Wo": (d, d), "Wgate": (dff, d), "Wup": (dff, d), "Wdown": (d, dff)}
    acts = {"X": (S, d), "Q": (S, d), "K": (S, d), "V": (S, d), "attn": (S, d), "gate": (S, dff), "up": (S, dff),
            "act": (S, dff), "out": (S, d)}
    msgs = []
    for name, (n_out, n_in) in weights.items():
        msgs += rows_of(n_out, n_in, -128, 128)
    for name, (n_rows, n_in) in acts.items():
        msgs += rows_of(n_rows, n_in, -(1 << 15), 1 << 15)
    total_rows = sum(int(m.shape[0]) for m in msgs)
    codes = [torch.empty((int(m.shape[0]), N), dtype=torch.uint64, device="cuda") for m in msgs]    # 31 GB of codewords stay resident
    widths = [1 << 12] * 6 + [1 << 14]
    mm_tabs = [[rand_field(torch, (w,), 100 + 2 * i), rand_field(torch, (w,), 101 + 2 * i)] for i, w in enumerate(widths)]
    r = random.Random(7)
    coins = [r.randrange(P) for _ in range(24)]
    z = [r.randrange(P) for _ in range(24)]
    # gate batch eq(z, .) * a * b: the eq table is built on the device, the two witness tables are random
    gate_tabs = [gpu.eq_vector_t(z)] + [rand_field(torch, (1 << 24,), 200 + j) for j in range(2)]
    hash_stream = torch.cuda.Stream()                     # default priority, like the stream the encoder runs on

    def commit(hash_too=True, overlap=True):
        """-> [(digests, root)] per committed matrix"""
        done = []
        main = torch.cuda.current_stream()
        for m, code in zip(msgs, codes):
            cp.coset_lde(m, K, N, 7, out=code)
            if not hash_too:
                continue
            if overlap:
                hash_stream.wait_stream(main)
                with torch.cuda.stream(hash_stream):
                    dig = cp.hash_columns_streamed(code)
                    done.append((dig, cp.merkle_build_blake3(dig)[0]))
            else:
                dig = cp.hash_columns_streamed(code)
                done.append((dig, cp.merkle_build_blake3(dig)[0]))
        main.wait_stream(hash_stream)
        return done

    def sumchecks():
        for tabs in mm_tabs:
            gpu.prove_terms_gpu([(1, tabs)], lambda i: coins[i], P)
        gpu.prove_terms_gpu([(1, gate_tabs)], lambda i: coins[i], P)

    n_w = sum(2 if n_in > ELL else 1 for (_, n_in) in weights.values())      # weight message blocks
    chis = [rand_field(torch, (1, int(m.shape[0])), 300 + i) for i, m in enumerate(msgs[:n_w])]

    def projections():
        """chi^T C per committed weight block: the (1 x rows) @ (rows x N) combination of
        layergkr/gpu.py:301-308 / projection.py:150-167; streams every weight codeword once."""
        return [cp.gl_matmul(chi, code) for chi, code in zip(chis, codes[:n_w])]

    commit(); commit(overlap=False); projections(); sumchecks()         # warm-up (twiddle tables, workspaces)
    torch.cuda.synchronize()
    tl0 = time.perf_counter()
    commit(hash_too=False)
    torch.cuda.synchronize()
    lde_only_s = time.perf_counter() - tl0
    ts0 = time.perf_counter()
    commit(overlap=False)
    torch.cuda.synchronize()
    seq_commit_s = time.perf_counter() - ts0
    t0 = time.perf_counter()
    committed = commit()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    projected = projections()
    torch.cuda.synchronize()
    tp = time.perf_counter()
    proj_ms = (tp - t1) * 1e3
    proj_bytes = sum(int(c.numel()) * 8 for c in codes[:n_w])
    t1b = time.perf_counter()
    sumchecks()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    t3 = time.perf_counter()
    gpu.prove_terms_gpu([(1, gate_tabs)], lambda i: coins[i], P)
    torch.cuda.synchronize()
    t4 = time.perf_counter()
    spare = gpu.eq_vector_t(z)                            # second buffer of that size into the allocator's cache
    del spare
    torch.cuda.synchronize()
    t5 = time.perf_counter()
    gpu.eq_vector_t(z)
    torch.cuda.synchronize()
    t6 = time.perf_counter()
    stacked = torch.stack([t.view(torch.int64) for t in gate_tabs]).view(torch.uint64)
    gpu.mle_eval_t(stacked, coins)
    t7 = time.perf_counter()
    gpu.mle_eval_t(stacked, coins)                       # the terminal evaluations the verifier's last check needs
    t8 = time.perf_counter()
    del stacked
    lde_bytes = 8 * (K + N) * total_rows
    res = {"rows_committed": total_rows, "geometry": "ELL=8192 K=2^14 N=2^16",
           "end_to_end_ms": (t2 - t0) * 1e3,
           "projection_matvec_ms": proj_ms, "projection_matvec_gbs": proj_bytes / proj_ms / 1e6,
           "commit_ms": (t1 - t0) * 1e3, "commit_sequential_ms": seq_commit_s * 1e3,
           "commit_hash_and_tree_ms": (seq_commit_s - lde_only_s) * 1e3,
           "commit_hash_and_tree_exposed_ms": (t1 - t0 - lde_only_s) * 1e3,
           "commit_lde_ms": lde_only_s * 1e3, "commit_lde_gbs_algorithmic": lde_bytes / lde_only_s / 1e9,
           "commit_lde_gelems_per_s": total_rows * N / lde_only_s / 1e9,
           "sumchecks_ms": (t2 - t1b) * 1e3,
           "gate_sumcheck_2^24_deg3_ms": (t4 - t3) * 1e3,
           "gate_sumcheck_gbs_algorithmic": 96 * (1 << 24) / (t4 - t3) / 1e9,
           "eq_vector_2^24_ms": (t6 - t5) * 1e3, "mle_eval_3x2^24_ms": (t8 - t7) * 1e3,
           "matmul_sumchecks": "6 x width 2^12 + 1 x width 2^14, degree 2, one launch each",
           "note": "commit_ms: digests and tree of matrix i on a second stream while matrix i+1 is encoded; "
                   "commit_sequential_ms: one stream"}
    if check:
        res["checks"] = _check_layer(torch, msgs, codes, committed, chis, projected, mm_tabs, gate_tabs, coins, K, N, n_w)
    return res


def _check_layer(torch, msgs, codes, committed, chis, projected, mm_tabs, gate_tabs, coins, K, N, n_w):
    """The full-shape layer run against the CPU oracle by samples, and by properties over everything."""
    import numpy as np
    from oracle import oracle as O
    from verinf_amd.layergkr import sumcheck as sc
    from verinf_amd.prover import cuda_primitives as cp
    out = {}
    # sampled rows of four matrices (a square weight, the narrow second block of Wdown, two activations)
    which = [0, 7, n_w, len(msgs) - 1]
    ok = True
    for i in which:
        m = int(msgs[i].shape[0])
        rows = sorted({0, m // 2, m - 1})
        sample = msgs[i].view(torch.int64)[rows].contiguous().view(torch.uint64).cpu().numpy()
        got = codes[i].view(torch.int64)[rows].contiguous().view(torch.uint64).cpu().numpy()
        ok = ok and bool(np.array_equal(got, O.coset_lde_rows(sample, K, N, 7)))
    out["sampled_rows_match_oracle"] = ok
    # every row of every committed matrix is a codeword: its interpolant on the coset has no coefficient >= K
    ok = True
    for code in codes:
        for lo in range(0, int(code.shape[0]), 4096):
            blk = code[lo:lo + 4096].clone()
            cp.ntt_inverse_batched(blk)
            ok = ok and not bool(blk.view(torch.int64)[:, K:].any())
            del blk
    out["every_row_is_a_codeword"] = ok
    # sampled column digests against the oracle's BLAKE3, and each root against the oracle's tree over the digests
    ok_d = ok_r = True
    for i in which:
        dig, root = committed[i]
        cols = [0, 777, N - 1]
        sub = codes[i].view(torch.int64)[:, cols].contiguous().view(torch.uint64).cpu().numpy()
        want = O.hash_columns(sub)
        ok_d = ok_d and bool(np.array_equal(dig.cpu().numpy()[cols], want))
        levels = O.merkle_levels(dig.cpu().numpy())
        ok_r = ok_r and levels[-1][0].tobytes() == bytes(root.cpu().tolist())
    out["sampled_column_digests_match_oracle"] = ok_d
    out["roots_match_oracle_tree"] = ok_r
    # the projection chi^T C on sampled columns against big-integer sums
    ok = True
    for i in (0, n_w - 1):
        chi = [int(v) for v in chis[i].cpu().numpy().reshape(-1)]
        for col in (0, 12345, N - 1):
            column = [int(v) for v in codes[i].view(torch.int64)[:, col].contiguous().view(torch.uint64).cpu().numpy()]
            ok = ok and sum(a * b for a, b in zip(chi, column)) % P == int(projected[i].view(torch.int64)[0, col].item()) % (1 << 64)
    out["projection_matches_bigint_sums"] = ok
    # every sumcheck of the layer through the verifier (round consistency + terminal evaluations on the device)
    ok = True
    for tabs in mm_tabs + [gate_tabs]:
        terms = [(1, tabs)]
        proof = sc.prove_terms(terms, lambda i: coins[i])
        good, _ = sc.verify_terms(proof, terms, lambda i: coins[i])
        ok = ok and good
    out["sumchecks_verify"] = ok
    # ... and a tampered table is rejected
    terms = [(1, gate_tabs)]
    proof = sc.prove_terms(terms, lambda i: coins[i])
    gate_tabs[2].view(torch.int64)[54321] += 1
    bad, _ = sc.verify_terms(proof, terms, lambda i: coins[i])
    gate_tabs[2].view(torch.int64)[54321] -= 1
    out["tampered_table_rejected"] = not bad
    return out


def copy_probe(torch):
    """1 GiB device-to-device copy, five times: FETCH_SIZE / WRITE_SIZE read for this
    kernel against the known 2^30 bytes give the counters' scale factor."""
    a = torch.zeros(1 << 27, dtype=torch.int64, device="cuda")
    b = torch.empty_like(a)
    for _ in range(5):
        b.copy_(a)
    torch.cuda.synchronize()
    print(json.dumps({"copy_probe_bytes_read": 1 << 30, "copy_probe_bytes_written": 1 << 30, "launches": 5}))


def valu_probe(torch, iters=400, reps=3):
    """Issue rate of each integer VALU instruction class on the whole chip (vi_valu_probe): wave-instructions per
    second from HIP events around the launch, the shader clock during the loop from the two counters the kernel
    reads, and from both the cycles a SIMD spends per instruction."""
    import ctypes
    from verinf_amd import _lib
    L = _lib.lib()
    props = torch.cuda.get_device_properties(0)
    cus = props.multi_processor_count
    blocks = cus * 8                                   # 8 wavefronts on every SIMD
    out = torch.empty(blocks * 256, dtype=torch.int64, device="cuda")
    clocks = torch.zeros(blocks * 4, dtype=torch.int64, device="cuda")
    wall_khz = L.vi_wall_clock_khz()
    rows = []
    for kind in range(L.vi_valu_probe_count()):
        n = ctypes.c_int64(0)
        best_ms, mhz = None, None
        for rep in range(reps + 1):
            s, e = _events(torch)
            s.record()
            _lib.check(L.vi_valu_probe(kind, 20 if rep == 0 else iters, blocks, out.data_ptr(), clocks.data_ptr(),
                                       ctypes.byref(n), _lib.stream_ptr()))
            e.record()
            torch.cuda.synchronize()
            if rep == 0:
                continue
            ms = s.elapsed_time(e)
            if best_ms is None or ms < best_ms:
                best_ms = ms
                c = clocks.view(-1, 4).cpu()
                ticks, ref = (c[:, 1] - c[:, 0]).double(), (c[:, 3] - c[:, 2]).double()
                mhz = float((ticks / ref).median()) * wall_khz / 1e3 if wall_khz else None
        rate = n.value / (best_ms * 1e-3)
        row = {"instruction": L.vi_valu_probe_name(kind).decode(), "ms": best_ms, "wave_instr_per_s": rate,
               "counter_ratio_mhz": mhz}
        if mhz:
            row["simd_cycles_per_instr"] = cus * 4 * mhz * 1e6 / rate
        rows.append(row)
    return {"device": props.name, "compute_units": cus, "simds": cus * 4, "wavefronts_per_simd": 8, "iters": iters,
            "wall_clock_khz": wall_khz, "rows": rows,
            "note": "counter_ratio_mhz = (shader-clock ticks / constant-rate ticks) x the constant counter's rate, median "
                    "over workgroups; if the two counters tick at one rate on this part it reads that rate, not the clock"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-rows", type=int, default=1024, help="rows of the CPU baseline sample")
    ap.add_argument("--cpu-reps", type=int, default=5, help="passes of the CPU baseline over its sample")
    ap.add_argument("--no-extra", action="store_true", help="skip the sumcheck / K-quant legs")
    ap.add_argument("--copy-probe", action="store_true")
    ap.add_argument("--valu-probe", action="store_true", help="issue rate of the integer VALU instruction classes")
    ap.add_argument("--ws-mb", type=int, default=0, help="override the LDE workspace size (MiB); 0 = library default")
    ap.add_argument("--only", choices=["sumcheck", "kquant", "layer", "hash", "gatebatch", "ntt"], default=None,
                    help="run just one of the extra legs and print its JSON (for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (rows of the LDE are independent, "
                 "so N GPUs would each take 1/N of the rows with no exchange)")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.copy_probe:
        copy_probe(torch)
        return
    if args.valu_probe:
        print(json.dumps(valu_probe(torch)))
        return
    if args.only == "sumcheck":
        print(json.dumps(bench_sumcheck(torch)))
        return
    if args.only == "kquant":
        print(json.dumps(bench_kquant(torch)))
        return
    if args.only == "layer":
        print(json.dumps(bench_layer(torch)))
        return
    if args.only == "hash":
        print(json.dumps(bench_hash(torch)))
        return
    if args.only == "gatebatch":
        print(json.dumps(bench_gate_batch(torch)))
        return
    if args.only == "ntt":
        print(json.dumps(bench_ntt(torch)))
        return

    lde, msgs, out = bench_lde(torch, args.steps, args.warmup, args.ws_mb)
    cpu = cpu_baseline_lde(torch, msgs, out, args.cpu_rows, args.cpu_reps)
    del msgs, out
    torch.cuda.empty_cache()
    extra = {}
    if not args.no_extra:
        extra["sumcheck_3x2^26_deg3"] = bench_sumcheck(torch)
        torch.cuda.empty_cache()
        extra["gate_batch_97_tables_2^22_deg3"] = bench_gate_batch(torch)
        torch.cuda.empty_cache()
        extra["kquant_q4k_4096x11008"] = bench_kquant(torch)
        torch.cuda.empty_cache()
        extra["blake3_commit_1024x2^18"] = bench_hash(torch)
        torch.cuda.empty_cache()
        extra["llama2_7b_layer"] = bench_layer(torch)

    line = {
        "metric": "goldilocks_coset_lde_2^16_to_2^18_output_elems_per_s",
        "value": lde["elems_per_s"],
        "unit": "elem/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": lde["ms_per_step"],
        "ms_per_step_median": lde["ms_per_step_median"],
        "ms_per_step_iqr": lde["ms_per_step_iqr"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u64",
        "data": "synthetic (seeded uniform field elements, resident in HBM)",
        "config": {"workload": "coset LDE 1024 rows x 2^16 -> 2^18, shift 7 (BASELINE configs[1])",
                   "rows": 1024, "K": 1 << 16, "N": 1 << 18},
        "roofline": {"bound": "hbm", "achieved": lde["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": lde["achieved_gbs"] / HBM_PEAK_GBS, "traffic": LDE_TRAFFIC_BYTES_PER_STEP / lde["launches_per_step"],
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by a copy probe "
                                       "(x2.000 / x1.000); not re-measured in this run",
                     "kernel": "k_lde_mid + k_ntt_fast (the three launches of a row chunk)", "launches_per_step": lde["launches_per_step"],
                     "avg_launch_us": lde["kernel_avg_us"],
                     "algorithmic_bytes_per_launch": lde["alg_bytes_per_launch"],
                     # the same launches against the integer-VALU issue rate, which is what bounds this kernel
                     "valu_issue": {"wave_instructions_per_step": LDE_VALU_INSTS_PER_STEP,
                                    "achieved_per_s": LDE_VALU_INSTS_PER_STEP / (lde["ms_per_step"] * 1e-3),
                                    "peak_per_s": VALU_ISSUE_PEAK_PER_S,
                                    "frac": LDE_VALU_INSTS_PER_STEP / (lde["ms_per_step"] * 1e-3) / VALU_ISSUE_PEAK_PER_S,
                                    "source": "instructions: rocprofv3 --pmc SQ_INSTS_VALU of this command; peak: 1024 SIMDs x "
                                              "2.4 GHz / 4.16 cycles per instruction (bench.py --valu-probe, "
                                              "profiles/valu_issue_rates__probe.md); neither re-measured in this run"}},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

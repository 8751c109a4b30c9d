"""The Python wrappers on several streams and host threads at once: scratch buffers are kept per (purpose,
device, stream) and the sumcheck's pinned sample words per (thread, stream), so concurrent callers must not
disturb each other.  Each thread's results are compared bit for bit with the oracle."""
import random
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402


def test_wrappers_from_two_threads_on_their_own_streams():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd import _lib
    from verinf_amd.layergkr import gpu
    from verinf_amd.prover import cuda_primitives as cp

    jobs = [(1 << 12, 1 << 14, 37, 51), (1 << 13, 1 << 15, 19, 52)]
    results, errors = {}, []

    def work(i):
        try:
            K, N, m, seed = jobs[i]
            stream = torch.cuda.Stream()                        # default priority
            msgs = rand_field((m, K), seed)
            tabs = [rand_field(1 << 14, seed + 10 + j) for j in range(3)]
            coins = [random.Random(seed).randrange(P) for _ in range(14)]
            with torch.cuda.stream(stream):
                d_msgs = to_dev(msgs)
                d_tabs = [to_dev(t) for t in tabs]
                outs = []
                for _ in range(6):                              # keep both streams busy at the same time
                    code = cp.coset_lde(d_msgs, K, N, 7)
                    rows = d_msgs.clone()
                    cp.ntt_forward_batched(rows)
                    claim, polys, _, _ = gpu.prove_terms_gpu([(1, d_tabs)], lambda r: coins[r], P)
                    outs.append((code, rows, claim, polys))
                stream.synchronize()
            results[i] = (msgs, tabs, coins, [(to_np(c), to_np(r), cl, po) for c, r, cl, po in outs])
        except Exception as exc:                                # surfaced by the main thread
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, (K, N, m, seed) in enumerate(jobs):
        msgs, tabs, coins, outs = results[i]
        want_code = O.coset_lde_rows(msgs, K, N, 7)
        want_rows = O.ntt_rows(msgs)
        want_claim, want_samples, _ = O.sumcheck_prove(tabs, [(1, [0, 1, 2])], coins)
        for code, rows, claim, polys in outs:
            assert np.array_equal(code, want_code)
            assert np.array_equal(rows, want_rows)
            assert claim == want_claim and [[y for _, y in s] for s in polys] == want_samples
    # one scratch buffer per stream that was used, none shared
    keys = [k for k in _lib._ws_cache if k[0] == "lde"]
    assert len({k[2] for k in keys}) >= 2
    _lib.release_workspaces()
    assert not _lib._ws_cache

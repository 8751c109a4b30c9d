"""GPU integration: the pieces of the path composed the way a layer proof uses them, at a small
Llama-like shape -- quantised weights decoded to field elements, committed (ZK pad, coset LDE,
column digests, Merkle root), the matmul reduced to a sumcheck over the input dimension with a
device-built eq table, the sumcheck verified with device evaluations, the commitment tied to the
claim by the linear combination of codewords, and a column opened.  Every link is an identity that
only holds if the kernels agree with each other and with the host arithmetic."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev, to_np  # noqa: E402


def _ints(t):
    return [int(v) for v in to_np(t).reshape(-1)]


def test_quantised_matmul_layer_flow():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.layergkr import gpu, rs, sumcheck as sc
    from verinf_amd.prover import core, cuda_primitives as cp, kquant_cuda as kq
    from verinf_amd.prover.protocol import merkle_leaf, merkle_verify

    n_out, n_in = 64, 512                      # W is (n_out, n_in), two Q4_K super-blocks per row
    rng = np.random.default_rng(17)
    raw = rng.integers(0, 256, size=(n_out * n_in // 256, 144), dtype=np.uint8)
    raw[:, 0:4] = np.abs(rng.normal(0, 0.01, size=(raw.shape[0], 2))).astype(np.float16).view(np.uint8).reshape(-1, 4)
    S = 1 << 12

    # 1. weights: raw super-blocks -> signed integers in the field
    W = kq.kquant_to_field(torch.from_numpy(raw).cuda(), "Q4_K", S).view(n_out, n_in)
    assert np.array_equal(to_np(W).reshape(-1), O.kquant_to_field(raw, "Q4_K", S))

    # 2. commit the weight rows: pad -> row polynomials -> codewords -> digests -> root
    cfg = core.LigeroConfig(ELL=n_in, K_DEG=1024, N_LIG=4096, T_QUERIES=16)
    seed = torch.tensor(list(range(32)), dtype=torch.uint8, device="cuda")
    polys, code = core.encode_messages(W, cfg, master_seed=seed, row_offset=0)
    com = rs.Commit(cfg, code)
    root = com.root
    assert len(root) == 32 and root == O.merkle_levels(O.hash_columns(to_np(code)))[-1][0].tobytes()

    # 3. the layer's arithmetic: y = W x over the field (x = small signed activations)
    x_int = rng.integers(-(1 << 15), 1 << 15, n_in)
    x = to_dev(np.array([int(v) % P for v in x_int], dtype=np.uint64))
    y = cp.gl_matvec(W, x)
    W_host = [[int(v) for v in row] for row in to_np(W)]
    assert _ints(y) == [sum(w * int(xv) for w, xv in zip(row, x_int)) % P for row in W_host]

    # 4. reduce "y = W x" at a random output point r_o to a sumcheck over the input index k:
    #    y~(r_o) = sum_k (sum_i eq(r_o, i) W[i, k]) * x[k]
    r = random.Random(23)
    r_o = [r.randrange(P) for _ in range(6)]                       # 2^6 = n_out
    eq_o = gpu.eq_vector_t(r_o, msb_first=True)
    w_row = cp.gl_matmul(eq_o.view(1, -1), W).view(-1)            # the chi^T W projection, width n_in
    claim_y = gpu.mle_eval_t(y, r_o)
    coins = [r.randrange(P) for _ in range(9)]                     # 2^9 = n_in
    proof = sc.prove([w_row, x], lambda i: coins[i])
    assert proof.claim == claim_y
    ok, why = sc.verify(proof, [w_row, x], lambda i: coins[i])
    assert ok, why

    # 5. tie the projected row to the commitment: the same combination of the committed codewords is the
    #    codeword of the combined padded messages (encoding is linear), so its restriction to the message
    #    slots, re-encoded, reproduces it
    comb_code = com.combine([int(v) for v in to_np(eq_o)])          # (1, N)
    comb_poly = cp.gl_matmul(eq_o.view(1, -1), polys)               # (1, K) row polynomial of the combination
    assert torch.equal(core._coset_encode_codewords(comb_poly, cfg), comb_code)
    # ... and the combined polynomial interpolates w_row on the message slots: Horner at zeta_c
    co = _ints(comb_poly)
    for c in (0, 1, 255, n_in - 1):
        zeta, acc = pow(cfg.W_K, c, P), 0
        for v in reversed(co):
            acc = (acc * zeta + v) % P
        assert acc == _ints(w_row)[c]

    # 6. open a column of the commitment and check it like the verifier would, also against the combination
    col = r.randrange(cfg.N_LIG)
    values, path = com.open(col)
    assert merkle_verify(merkle_leaf(values), path, root)
    eq_host = [int(v) for v in to_np(eq_o)]
    assert sum(e * v for e, v in zip(eq_host, values)) % P == _ints(comb_code)[col]

"""The Llama-2-7B-shape layer at its full size (58,592 message rows at ELL = 8192, K = 2^14 -> N = 2^16, hashed;
seven matmul sumchecks and the 2^24 gate batch; the projections over the weight codewords), run by the same code
the benchmark times and verified by what does not need a full CPU run: sampled rows, column digests and Merkle
roots against the CPU oracle, the codeword property on every one of the rows, every sumcheck through the
verifier with a tampered table rejected, and the projection against big-integer sums on sampled columns."""
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def test_layer_commit_projection_and_sumchecks_at_full_shape():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import bench
    res = bench.bench_layer(torch, check=True)
    assert res["rows_committed"] == 58592
    checks = res["checks"]
    assert set(checks) == {"sampled_rows_match_oracle", "every_row_is_a_codeword", "sampled_column_digests_match_oracle",
                           "roots_match_oracle_tree", "projection_matches_bigint_sums", "sumchecks_verify",
                           "tampered_table_rejected"}
    assert all(checks.values()), checks
    torch.cuda.empty_cache()

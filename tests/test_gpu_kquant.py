"""GPU parity: fused K-quant -> field decode through the C ABI vs the oracle (bit-exact).

Agreement with the third-party gguf-py dequantiser itself is parity-unpinned here
(package and model file unavailable offline); what is pinned is the byte -> integer
map of the reference kernels, via the exact-rational fixture and two independent
CPU restatements."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import to_np  # noqa: E402


@pytest.fixture(scope="module")
def kq():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd.prover import kquant_cuda
    return kquant_cuda


def synth_blocks(qtype, nb, seed):
    """The K-quant benchmark recipe: scale / quant bytes uniform, d and dmin = fp16(|N(0, 0.01)|)."""
    rng = np.random.default_rng(seed)
    bb = O.BLOCK_BYTES[qtype]
    raw = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    d = np.abs(rng.normal(0, 0.01, size=(nb, 2))).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if qtype == "Q6_K":
        raw[:, 208:210] = d[:, :2]
    else:
        raw[:, 0:4] = d
    return raw


def test_kquant_golden(kq, golden_dir):
    for g in json.load(open(os.path.join(golden_dir, "kquant.json"))):
        raw = np.frombuffer(bytes.fromhex(g["raw"]), dtype=np.uint8).copy()
        got = kq.kquant_to_field(torch.from_numpy(raw).cuda(), g["qtype"], g["S"])
        want = np.array([int(x, 16) for x in g["field"]], dtype=np.uint64)
        assert np.array_equal(to_np(got), want), g["qtype"]


@pytest.mark.parametrize("qtype", ["Q4_K", "Q5_K", "Q6_K"])
@pytest.mark.parametrize("nb", [1, 3, 257, 5000])
def test_kquant_matches_oracle(kq, qtype, nb):
    raw = synth_blocks(qtype, nb, 11 + nb)
    d = torch.from_numpy(raw).cuda()
    for S in (1 << 12, 1 << 16, 1000003):
        got = kq.kquant_to_field(d, qtype, S)
        assert got.shape == (nb * 256,)
        assert np.array_equal(to_np(got), O.kquant_to_field(raw, qtype, S)), (qtype, S)


def test_kquant_arbitrary_header_bits_and_unaligned_buffer(kq):
    """Every fp16 bit pattern that is finite may appear as d / dmin (subnormals, negative)."""
    rng = np.random.default_rng(5)
    for qtype in ("Q4_K", "Q5_K", "Q6_K"):
        raw = rng.integers(0, 256, size=(4000, O.BLOCK_BYTES[qtype]), dtype=np.uint8)
        hdr = slice(208, 210) if qtype == "Q6_K" else slice(0, 4)
        h = raw[:, hdr].copy().view(np.uint16)
        h[(h & 0x7C00) == 0x7C00] &= 0x83FF            # clear inf / nan exponents
        raw[:, hdr] = h.view(np.uint8)
        buf = torch.empty(raw.size + 1, dtype=torch.uint8, device="cuda")
        buf[1:] = torch.from_numpy(raw.reshape(-1)).cuda()
        for t in (torch.from_numpy(raw).cuda(), buf[1:]):          # aligned, then odd address
            got = kq.kquant_to_field(t, qtype, 1 << 12)
            assert np.array_equal(to_np(got), O.kquant_to_field(raw, qtype, 1 << 12)), qtype


def test_kquant_errors(kq):
    with pytest.raises(RuntimeError):
        kq.kquant_to_field(torch.zeros(145, dtype=torch.uint8, device="cuda"), "Q4_K", 4096)
    with pytest.raises(AssertionError):
        kq.kquant_to_field(torch.zeros(144, dtype=torch.uint8, device="cuda"), "Q8_0", 4096)
    assert kq.kquant_to_field(torch.zeros(0, dtype=torch.uint8, device="cuda"), "Q4_K", 4096).numel() == 0


def test_kquant_baseline_shape(kq):
    """The K-quant benchmark workload: a 4096 x 11008 Q4_K matrix (176,128 super-blocks), whole output
    against the C oracle."""
    nb = 4096 * 11008 // 256
    raw = synth_blocks("Q4_K", nb, 3)
    got = kq.kquant_to_field(torch.from_numpy(raw).cuda(), "Q4_K", 1 << 12)
    want = O.kquant_to_field(raw, "Q4_K", 1 << 12)
    assert np.array_equal(to_np(got), want)
    # the caller's reshape/transposition of prover/loader.py:433-436 works on the result
    w = got.view(4096, 11008).view(torch.int64).T.contiguous().view(torch.uint64)
    assert tuple(w.shape) == (11008, 4096)


@pytest.mark.parametrize("qtype", ["Q4_K", "Q5_K", "Q6_K"])
@pytest.mark.parametrize("d_out,bpr", [(1, 1), (16, 1), (37, 3), (64, 2), (130, 5), (1000, 4)])
def test_kquant_transposed_matches_oracle(kq, qtype, d_out, bpr):
    """Decode + transpose in one pass against the oracle's decode transposed on the host:
    row counts below, at and across the 16-row tile, one and several super-blocks per row."""
    raw = synth_blocks(qtype, d_out * bpr, 7 + d_out)
    want = O.kquant_to_field(raw, qtype, 1 << 12).reshape(d_out, bpr * 256).T.reshape(-1)
    d = torch.from_numpy(raw).cuda()
    got = kq.kquant_to_field_transposed(d, qtype, 1 << 12, d_out)
    assert got.shape == (d_out * bpr * 256,)
    assert np.array_equal(to_np(got), want)
    # the two-step form of prover/loader.py:427-436 gives the same tensor
    two = kq.kquant_to_field(d, qtype, 1 << 12).view(d_out, bpr * 256).view(torch.int64).T.contiguous().view(torch.uint64)
    assert torch.equal(got.view(torch.int64), two.reshape(-1).view(torch.int64))
    # a buffer at an odd address takes the one-thread-per-weight kernel
    buf = torch.empty(raw.size + 1, dtype=torch.uint8, device="cuda")
    buf[1:] = d.reshape(-1)
    assert np.array_equal(to_np(kq.kquant_to_field_transposed(buf[1:], qtype, 1 << 12, d_out)), want)


def test_kquant_transposed_errors_and_baseline_shape(kq):
    z = torch.zeros(144 * 6, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError):
        kq.kquant_to_field_transposed(z, "Q4_K", 4096, 4)            # 6 blocks are not 4 rows
    with pytest.raises(RuntimeError):
        kq.kquant_to_field_transposed(z, "Q4_K", 4096, 0)
    assert kq.kquant_to_field_transposed(z[:0], "Q4_K", 4096, 3).numel() == 0
    nb = 4096 * 11008 // 256
    raw = synth_blocks("Q4_K", nb, 3)
    got = kq.kquant_to_field_transposed(torch.from_numpy(raw).cuda(), "Q4_K", 1 << 12, 4096)
    want = O.kquant_to_field(raw, "Q4_K", 1 << 12).reshape(4096, 11008).T
    assert np.array_equal(to_np(got).reshape(11008, 4096), want)

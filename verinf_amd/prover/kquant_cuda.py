"""Drop-in for the reference's `prover/kquant_cuda.py` on MI355X: raw GGUF K-quant
super-block bytes (Q4_K / Q5_K / Q6_K) -> committed Goldilocks integers on the GPU.

Same entry point and conventions (prover/kquant_cuda.py:170-177): any-shape
contiguous uint8 tensor on the GPU in, flat uint64 tensor of n_blocks*256 values
out, row-major as stored.  The byte -> integer map is bit-identical to the
reference kernels (kquant_cuda.py:42-111): fp32 `(d*sc)*q - dmin*mn` with separately
rounded operations, then round-half-even of double(v)*S, negatives as p - |x|.
"""
import torch

from .. import _lib

QK_K = 256
BLOCK_BYTES = {"Q4_K": 144, "Q5_K": 176, "Q6_K": 210}
_QTYPE_ID = {"Q4_K": 4, "Q5_K": 5, "Q6_K": 6}


def kquant_to_field(raw_u8_cuda: torch.Tensor, qtype: str, S: int) -> torch.Tensor:
    """raw K-quant bytes -> flat uint64 field tensor of n_blocks*256 integers."""
    assert qtype in _QTYPE_ID, f"kquant_to_field: unsupported type {qtype}"
    raw = raw_u8_cuda.reshape(-1)
    if not (raw.is_cuda and raw.dtype == torch.uint8 and raw.is_contiguous()):
        raise RuntimeError("kquant_to_field: raw must be a contiguous CUDA uint8 tensor")
    bb = BLOCK_BYTES[qtype]
    n_blocks = raw.numel() // bb
    if n_blocks * bb != raw.numel():
        raise RuntimeError(f"kquant_to_field: {raw.numel()} bytes is not a multiple of the {bb}-byte {qtype} block")
    out = torch.empty(n_blocks * QK_K, dtype=torch.uint64, device=raw.device)
    if n_blocks:
        with torch.cuda.device(raw.device):
            _lib.check(_lib.lib().vi_kquant_to_field(_QTYPE_ID[qtype], raw.data_ptr(), n_blocks, float(S),
                                                     out.data_ptr(), _lib.stream_ptr()))
    return out


def kquant_to_field_transposed(raw_u8_cuda: torch.Tensor, qtype: str, S: int, d_out: int) -> torch.Tensor:
    """raw K-quant bytes of a (d_out, d_in) matrix -> flat uint64 tensor of the (d_in, d_out)
    transpose, i.e. `kquant_to_field(raw, qtype, S).view(d_out, d_in).view(int64).T.contiguous()
    .view(uint64).reshape(-1)` -- the (k_in, n_out) order in which the loader commits an expert
    matrix (prover/loader.py:427-436) -- in one pass, without the intermediate decoded matrix."""
    assert qtype in _QTYPE_ID, f"kquant_to_field_transposed: unsupported type {qtype}"
    raw = raw_u8_cuda.reshape(-1)
    if not (raw.is_cuda and raw.dtype == torch.uint8 and raw.is_contiguous()):
        raise RuntimeError("kquant_to_field_transposed: raw must be a contiguous CUDA uint8 tensor")
    bb = BLOCK_BYTES[qtype]
    n_blocks = raw.numel() // bb
    d_out = int(d_out)
    if n_blocks * bb != raw.numel() or d_out < 1 or n_blocks % d_out:
        raise RuntimeError(f"kquant_to_field_transposed: {raw.numel()} bytes are not {d_out} rows of whole {bb}-byte {qtype} blocks")
    d_in = n_blocks // d_out * QK_K
    out = torch.empty(n_blocks * QK_K, dtype=torch.uint64, device=raw.device)
    if n_blocks:
        with torch.cuda.device(raw.device):
            _lib.check(_lib.lib().vi_kquant_to_field_transposed(_QTYPE_ID[qtype], raw.data_ptr(), d_out, d_in, float(S),
                                                                out.data_ptr(), _lib.stream_ptr()))
    return out

"""ctypes binding of libverinf_hip.so (C ABI: include/verinf_hip.h).

The library is built ahead of time by `python -m verinf_amd.build`; loading fails
loudly if it is missing.  torch is imported first on purpose: its bundled HIP
runtime must be the one the library binds to, so that tensor pointers and stream
handles mean the same thing on both sides.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_int, c_int64, c_size_t, c_uint64, c_void_p

import torch  # noqa: F401  (must precede the CDLL below)

_HERE = os.path.dirname(os.path.abspath(__file__))
# VERINF_HIP_LIB points at an alternative build of the same library (e.g. one compiled
# with different tuning flags); the default is the in-tree build.
LIB_PATH = os.environ.get("VERINF_HIP_LIB") or os.path.join(_HERE, "libverinf_hip.so")

EXPORTS = [
    "vi_last_error", "vi_version",
    "vi_gl_binop", "vi_gl_binop_bcast", "vi_gl_unop", "vi_gl_axpy", "vi_gl_probe",
    "vi_gl_sum_workspace_bytes", "vi_gl_sum",
    "vi_gl_matmul_workspace_bytes", "vi_gl_matmul", "vi_gl_matvec", "vi_poly_eval",
    "vi_ntt_workspace_bytes", "vi_ntt_batched",
    "vi_coset_lde_workspace_bytes", "vi_coset_lde_min_workspace_bytes", "vi_coset_lde_launches",
    "vi_coset_lde", "vi_coset_lde_coeffs", "vi_coset_extend",
    "vi_kquant_to_field",
    "vi_kquant_to_field_transposed",
    "vi_sumcheck_workspace_bytes", "vi_sumcheck_eval", "vi_sumcheck_eval_static", "vi_sumcheck_fold_eval",
    "vi_sumcheck_prove", "vi_sumcheck_prove_coins_workspace_bytes", "vi_sumcheck_prove_coins",
    "vi_hash_columns_workspace_bytes", "vi_hash_columns", "vi_hash_columns_update", "vi_hash_columns_finalize",
    "vi_merkle_level", "vi_merkle_tree_nodes", "vi_merkle_tree", "vi_row_prg",
    "vi_eq_vector", "vi_mle_eval_workspace_bytes", "vi_mle_eval",
    "vi_challenge", "vi_gl_spmv", "vi_lookup_multiplicities",
    "vi_valu_probe_count", "vi_valu_probe_name", "vi_wall_clock_khz", "vi_valu_probe",
]

COIN_FN = ctypes.CFUNCTYPE(c_int, c_int, POINTER(c_uint64), c_int, POINTER(c_uint64), c_void_p)

_lib = None


class VerinfHipError(RuntimeError):
    pass


def lib():
    """The loaded library with argument types declared."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise VerinfHipError(
            f"{LIB_PATH} is missing: build it with `python -m verinf_amd.build` "
            "(there is no CPU fallback)")
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, u64, sz = c_void_p, c_int64, c_uint64, c_size_t
    ip = POINTER(c_int)
    L.vi_last_error.restype = c_char_p
    L.vi_version.restype = c_char_p
    L.vi_gl_binop.argtypes = [c_int, vp, vp, vp, i64, vp]
    L.vi_gl_binop_bcast.argtypes = [c_int, vp, vp, i64, vp, i64, vp]
    L.vi_gl_unop.argtypes = [c_int, vp, u64, vp, i64, vp]
    L.vi_gl_axpy.argtypes = [vp, u64, vp, i64, vp]
    L.vi_gl_probe.argtypes = [c_int, vp, vp, vp, i64, vp]
    L.vi_gl_sum_workspace_bytes.restype = sz
    L.vi_gl_sum_workspace_bytes.argtypes = [i64]
    L.vi_gl_sum.argtypes = [vp, i64, vp, vp, sz, vp]
    L.vi_gl_matmul_workspace_bytes.restype = sz
    L.vi_gl_matmul_workspace_bytes.argtypes = [i64, i64, i64]
    L.vi_gl_matmul.argtypes = [vp, vp, vp, i64, i64, i64, vp, sz, vp]
    L.vi_gl_matvec.argtypes = [vp, vp, vp, i64, i64, vp]
    L.vi_poly_eval.argtypes = [vp, i64, i64, vp, i64, vp, vp]
    L.vi_ntt_workspace_bytes.restype = sz
    L.vi_ntt_workspace_bytes.argtypes = [i64, i64]
    L.vi_ntt_batched.argtypes = [vp, i64, i64, c_int, vp, sz, vp]
    L.vi_coset_lde_workspace_bytes.restype = sz
    L.vi_coset_lde_workspace_bytes.argtypes = [i64, i64, i64]
    L.vi_coset_lde_min_workspace_bytes.restype = sz
    L.vi_coset_lde_min_workspace_bytes.argtypes = [i64, i64]
    L.vi_coset_lde_launches.restype = i64
    L.vi_coset_lde_launches.argtypes = [i64, i64, i64, sz]
    L.vi_coset_lde.argtypes = [vp, i64, i64, i64, i64, i64, u64, vp, i64, vp, sz, vp]
    L.vi_coset_lde_coeffs.argtypes = [vp, i64, i64, i64, i64, i64, u64, vp, i64, vp, i64, vp, sz, vp]
    L.vi_coset_extend.argtypes = [vp, i64, i64, i64, i64, i64, u64, vp, i64, vp, sz, vp]
    L.vi_kquant_to_field.argtypes = [c_int, vp, i64, c_double, vp, vp]
    L.vi_kquant_to_field_transposed.argtypes = [c_int, vp, i64, i64, c_double, vp, vp]
    L.vi_sumcheck_workspace_bytes.restype = sz
    L.vi_sumcheck_workspace_bytes.argtypes = []
    L.vi_sumcheck_eval.argtypes = [POINTER(vp), c_int, i64, ip, ip, POINTER(u64), c_int, vp, vp, sz, vp]
    L.vi_sumcheck_eval_static.argtypes = [POINTER(vp), c_int, i64, ip, ip, POINTER(u64), c_int, vp, vp]
    L.vi_sumcheck_fold_eval.argtypes = [POINTER(vp), POINTER(vp), c_int, i64, u64, ip, ip,
                                        POINTER(u64), c_int, POINTER(u64), vp, vp, sz, vp]
    L.vi_sumcheck_prove.argtypes = [POINTER(vp), POINTER(vp), c_int, i64, ip, ip, POINTER(u64), c_int,
                                    COIN_FN, vp, vp, sz, POINTER(u64), POINTER(u64), vp, sz, vp]
    L.vi_sumcheck_prove.restype = c_int
    L.vi_sumcheck_prove_coins_workspace_bytes.restype = sz
    L.vi_sumcheck_prove_coins_workspace_bytes.argtypes = [i64]
    L.vi_sumcheck_prove_coins.argtypes = [POINTER(vp), POINTER(vp), c_int, i64, ip, ip, POINTER(u64), c_int,
                                          POINTER(u64), vp, vp, sz, vp]
    L.vi_sumcheck_prove_coins.restype = c_int
    L.vi_hash_columns_workspace_bytes.restype = sz
    L.vi_hash_columns_workspace_bytes.argtypes = [i64, i64]
    L.vi_hash_columns.argtypes = [vp, i64, i64, i64, vp, vp, sz, vp]
    L.vi_hash_columns_update.argtypes = [vp, i64, i64, i64, i64, i64, vp, sz, vp]
    L.vi_hash_columns_finalize.argtypes = [i64, i64, vp, sz, vp, vp]
    L.vi_merkle_level.argtypes = [vp, i64, vp, vp]
    L.vi_merkle_tree_nodes.restype = i64
    L.vi_merkle_tree_nodes.argtypes = [i64]
    L.vi_merkle_tree.argtypes = [vp, i64, vp, vp]
    L.vi_row_prg.argtypes = [vp, vp, i64, i64, i64, vp, i64, vp]
    L.vi_challenge.argtypes = [vp, vp, c_int, vp, i64, vp, vp]
    L.vi_gl_spmv.argtypes = [vp, vp, vp, i64, i64, vp, vp, vp, c_int, vp, vp]
    L.vi_lookup_multiplicities.argtypes = [vp, i64, vp, i64, c_int, vp, vp]
    L.vi_eq_vector.argtypes = [POINTER(u64), c_int, c_int, vp, vp]
    L.vi_mle_eval_workspace_bytes.restype = sz
    L.vi_mle_eval_workspace_bytes.argtypes = [i64]
    L.vi_mle_eval.argtypes = [vp, i64, i64, POINTER(u64), c_int, vp, vp, sz, vp]
    L.vi_valu_probe_name.restype = c_char_p
    L.vi_valu_probe_name.argtypes = [c_int]
    L.vi_valu_probe.argtypes = [c_int, c_int, c_int, vp, vp, POINTER(i64), vp]
    for name in EXPORTS:
        getattr(L, name)                     # AttributeError here = stale build
    for name in ("vi_gl_binop", "vi_gl_binop_bcast", "vi_gl_unop", "vi_gl_axpy", "vi_gl_probe", "vi_gl_sum",
                 "vi_gl_matmul", "vi_gl_matvec", "vi_poly_eval",
                 "vi_ntt_batched", "vi_coset_lde", "vi_coset_lde_coeffs", "vi_coset_extend", "vi_kquant_to_field", "vi_kquant_to_field_transposed", "vi_sumcheck_eval", "vi_sumcheck_eval_static",
                 "vi_sumcheck_fold_eval", "vi_hash_columns", "vi_hash_columns_update", "vi_hash_columns_finalize",
                 "vi_merkle_level", "vi_merkle_tree_nodes", "vi_merkle_tree", "vi_row_prg", "vi_eq_vector", "vi_mle_eval",
                 "vi_challenge", "vi_gl_spmv", "vi_lookup_multiplicities", "vi_valu_probe"):
        getattr(L, name).restype = c_int
    _lib = L
    return L


def check(rc: int) -> None:
    """Turn a negative C-ABI return code into an exception carrying vi_last_error()."""
    if rc != 0:
        msg = lib().vi_last_error().decode("utf-8", "replace")
        raise VerinfHipError(f"libverinf_hip error {rc}: {msg}")


def stream_ptr() -> int:
    """hipStream_t of torch's current stream (kernels are queued behind torch's own work)."""
    return torch.cuda.current_stream().cuda_stream


_ws_cache = {}


def workspace(nbytes: int, device=None, tag: str = "ws", stream_ptr=None):
    """A cached uint8 device buffer of at least nbytes for the CURRENT stream of `device`.

    One buffer per (purpose, device, stream): the wrappers launch on torch's current stream, so two streams
    (or two host threads on their own streams) never share scratch, and a buffer is only ever used on the
    stream it was allocated on -- when it is outgrown and dropped, the caching allocator may reuse its memory
    in stream order without further bookkeeping.  Buffers grow and are kept; release_workspaces() drops them."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    # stream_ptr: the current stream's handle when the caller has looked it up already
    key = (tag, device.index, torch.cuda.current_stream(device).cuda_stream if stream_ptr is None else stream_ptr)
    buf = _ws_cache.get(key)
    if buf is None or buf.numel() < nbytes:
        with torch.cuda.device(device):
            buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _ws_cache[key] = buf
    return buf


def release_workspaces() -> None:
    """Drop every cached scratch buffer (they come back on demand).  Call it with the device idle: a buffer
    still in use by queued kernels must not be handed back to the allocator from another stream."""
    _ws_cache.clear()

"""vi_sumcheck_eval_static (the entry point that allocates nothing) against vi_sumcheck_eval, through the C ABI.

Two calls in a row, the second on a smaller problem, so that whatever the first call left in the library's
static scratch array would show; each call is also checked against the oracle's round-0 samples."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from oracle import oracle as O  # noqa: E402
from tests.gpu_util import P, rand_field, to_dev  # noqa: E402


def _call(L, fn_static, tabs_dev, half, terms):
    """samples (deg + 1 words) of the round over the first 2*half entries of each table"""
    from verinf_amd import _lib
    n_tables = len(tabs_dev)
    ptrs = (ctypes.c_void_p * n_tables)(*[t.data_ptr() for t in tabs_dev])
    off, idx = [0], []
    for _, fs in terms:
        idx += fs
        off.append(len(idx))
    term_off = (ctypes.c_int * len(off))(*off)
    factor_idx = (ctypes.c_int * len(idx))(*idx)
    coeffs = (ctypes.c_uint64 * len(terms))(*[c for c, _ in terms])
    out = torch.zeros(8, dtype=torch.uint64, device="cuda")
    stream = _lib.stream_ptr()
    if fn_static:
        rc = L.vi_sumcheck_eval_static(ptrs, n_tables, half, term_off, factor_idx, coeffs, len(terms), out.data_ptr(), stream)
    else:
        ws = torch.empty(L.vi_sumcheck_workspace_bytes(), dtype=torch.uint8, device="cuda")
        rc = L.vi_sumcheck_eval(ptrs, n_tables, half, term_off, factor_idx, coeffs, len(terms), out.data_ptr(),
                                ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc)
    deg = max(len(fs) for _, fs in terms)
    return out.cpu().numpy()[:deg + 1].tolist()


def test_static_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from verinf_amd import _lib
    L = _lib.lib()
    terms = [(3, [0, 1, 2]), (P - 5, [0, 3])]
    big = [rand_field(1 << 20, 900 + j) for j in range(4)]
    small = [rand_field(1 << 11, 910 + j) for j in range(4)]
    tiny = [t[:1 << 6].copy() for t in small]                       # the single-workgroup path
    for tabs in (big, small, tiny):
        dev = [to_dev(t) for t in tabs]
        half = tabs[0].size // 2
        got = _call(L, True, dev, half, terms)
        want = _call(L, False, dev, half, terms)
        assert got == want
        _, samples, _ = O.sumcheck_prove(tabs, terms, [1] * (tabs[0].size.bit_length() - 1))
        assert got == samples[0]


def test_static_entry_point_with_tables_in_memory_and_no_device_allocation():
    """Twenty tables (more than a thread keeps in registers: the kernel that walks the tables in memory, with several
    rows of partial-sum slots at the small size) through the static scratch, at 2^20 and then 2^11; and a warm
    call leaves the device's free memory and torch's allocation count where they were."""
    from verinf_amd import _lib
    L = _lib.lib()
    n = 20
    terms = [(j + 2, [0, j, j + 1]) for j in range(1, n - 1, 2)] + [(P - 7, [0, j]) for j in range(1, n)]
    for v in (20, 11):
        tabs = [rand_field(1 << v, 930 + 31 * v + j) for j in range(n)]
        dev = [to_dev(t) for t in tabs]
        half = 1 << (v - 1)
        got = _call(L, True, dev, half, terms)
        assert got == _call(L, False, dev, half, terms)
        _, samples, _ = O.sumcheck_prove(tabs, terms, [1] * v)
        assert got == samples[0]
        # warm now: nothing may be allocated by a further call
        ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dev])
        off, idx = [0], []
        for _, fs in terms:
            idx += fs
            off.append(len(idx))
        term_off = (ctypes.c_int * len(off))(*off)
        factor_idx = (ctypes.c_int * len(idx))(*idx)
        coeffs = (ctypes.c_uint64 * len(terms))(*[c for c, _ in terms])
        out = torch.zeros(8, dtype=torch.uint64, device="cuda")
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        stats0 = torch.cuda.memory_stats()
        for _ in range(3):
            _lib.check(L.vi_sumcheck_eval_static(ptrs, n, half, term_off, factor_idx, coeffs, len(terms), out.data_ptr(),
                                                 _lib.stream_ptr()))
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        stats1 = torch.cuda.memory_stats()
        assert free1 == free0
        assert stats1["allocation.all.allocated"] == stats0["allocation.all.allocated"]
        assert out.cpu().numpy()[:4].tolist() == got


def test_static_entry_point_rejects_sizes_beyond_its_limit():
    from verinf_amd import _lib
    L = _lib.lib()
    t = to_dev(rand_field(16, 1))
    ptrs = (ctypes.c_void_p * 1)(t.data_ptr())
    off = (ctypes.c_int * 2)(0, 1)
    idx = (ctypes.c_int * 1)(0)
    co = (ctypes.c_uint64 * 1)(1)
    out = torch.zeros(8, dtype=torch.uint64, device="cuda")
    rc = L.vi_sumcheck_eval_static(ptrs, 1, (1 << 32) + 1, off, idx, co, 1, out.data_ptr(), _lib.stream_ptr())
    assert rc != 0
    assert b"exceeds the limit" in L.vi_last_error()

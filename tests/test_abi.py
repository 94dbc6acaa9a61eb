"""CPU-only checks of the drop-in boundary: the shared library loads and exports every symbol
the C header declares and every symbol the reference's loader binds eagerly; host-side argument
checks of the Python mirror behave like the reference's (pysiglib/sig.py:265-272, tests/test_errors.py:77-114)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pysiglib_amd", "csrc", "libcusig.so")

# names bound by the reference loader for its GPU plugin (pysiglib/load_siglib.py:165-182,420-641)
LOADER_PAIRS = """transform_path_cuda transform_path_backprop_cuda log_sig_combine_cuda log_sig_from_path_cuda
log_sig_from_path_backprop_cuda log_sig_combine_backprop_cuda sig_combine_cuda sig_join_cuda sig_join_backprop_cuda
sig_combine_backprop_cuda sig_coef_cuda sig_coef_backprop_cuda signature_cuda sig_backprop_cuda sig_to_log_sig_cuda
sig_to_log_sig_backprop_cuda sig_kernel_cuda sig_kernel_poly_cuda sig_kernel_poly_backprop_cuda branched_sig_kernel_cuda
sig_kernel_backprop_cuda branched_sig_kernel_backprop_cuda branched_sig_kernel_poly_cuda
branched_sig_kernel_poly_backprop_cuda branched_sig_cuda branched_sig_coef_cuda branched_sig_coef_backprop_cuda
branched_sig_combine_cuda branched_sig_to_log_sig_cuda branched_sig_to_log_sig_backprop_cuda branched_log_sig_join_cuda
branched_log_sig_join_backprop_cuda branched_log_sig_from_path_cuda branched_log_sig_from_path_backprop_cuda
branched_sig_combine_backprop_cuda branched_sig_backprop_cuda linear_sig_cuda log_sig_join_cuda
log_sig_join_backprop_cuda logsig_to_sig_cuda logsig_to_sig_backprop_cuda""".split()
LOADER_SINGLES = ["prepare_log_sig_cuda", "clear_cache_cuda", "set_cache_dir_cuda", "cusig_amd_lyndon_tables", "prepare_branched_sig_cuda",
                  "prepare_branched_log_sig_cuda", "prepare_branched_sig_coef_cuda", "cusig_shutdown",
                  "cusig_last_error_message"]


@pytest.fixture(scope="module")
def lib():
    assert os.path.exists(LIB), "build the library first (python __graft_entry__.py)"
    return ctypes.CDLL(LIB)


def test_header_symbols_exported(lib):
    text = open(os.path.join(ROOT, "include", "cusig_amd.h")).read()
    names = re.findall(r"CUSIG_AMD_API\s+[\w\s\*]+?\b(\w+)\s*\(", text)
    assert len(names) >= 11
    for n in names:
        assert hasattr(lib, n), n


def test_reference_loader_symbols_exported(lib):
    for base in LOADER_PAIRS:
        for suf in ("_f", "_d"):
            assert hasattr(lib, base + suf), base + suf
    for n in LOADER_SINGLES:
        assert hasattr(lib, n), n


def test_out_of_scope_symbols_report_not_implemented(lib):
    lib.cusig_last_error_message.restype = ctypes.c_char_p
    assert lib.sig_kernel_cuda_d(None, None, None, 0, 0, 0) == 10
    assert b"not implemented" in lib.cusig_last_error_message()
    assert lib.set_cache_dir_cuda(None) == 10


@pytest.mark.parametrize("d,deg", [(2, 7), (3, 5), (5, 4), (1, 3), (8, 3)])
def test_lyndon_tables_match_the_oracle(lib, d, deg):
    """The host code behind prepare_log_sig_cuda against the oracle's Lyndon words and bracket projection."""
    import numpy as np
    from oracle import lyndon
    fn = lib.cusig_amd_lyndon_tables
    u64p, u32p, i32p = ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_int32)
    fn.argtypes = (ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int, u64p, u64p, u64p, u64p, u32p, i32p)
    count, nnz = ctypes.c_uint64(), ctypes.c_uint64()
    words = lyndon.lyndon_words(d, deg)
    for method in (1, 2):
        assert fn(d, deg, method, ctypes.byref(count), ctypes.byref(nnz), None, None, None, None) == 0
        assert count.value == len(words)
        index = np.zeros(count.value, dtype=np.uint64)
        row_ptr = np.zeros(count.value + 1, dtype=np.uint64)
        col = np.zeros(max(nnz.value, 1), dtype=np.uint32)
        val = np.zeros(max(nnz.value, 1), dtype=np.int32)
        assert fn(d, deg, method, None, None, index.ctypes.data_as(u64p), row_ptr.ctypes.data_as(u64p),
                  col.ctypes.data_as(u32p), val.ctypes.data_as(i32p)) == 0
        assert list(index) == [lyndon.word_index(w, d) for w in words]
        if method == 1:
            assert nnz.value == 0
            continue
        inv = np.eye(len(words))
        for i in range(len(words)):
            for k in range(int(row_ptr[i]), int(row_ptr[i + 1])):
                assert col[k] < i
                inv[i, col[k]] = val[k]
        np.testing.assert_allclose(inv @ lyndon.projection_matrix(d, deg), np.eye(len(words)), rtol=0, atol=1e-9)
    assert fn(d, deg, 3, None, None, None, None, None, None) == 2


def test_sig_length(lib, kats):
    lib.cusig_amd_sig_length.restype = ctypes.c_uint64
    lib.cusig_amd_sig_length.argtypes = (ctypes.c_uint64, ctypes.c_uint64)
    for d, n, expected in kats["sig_length"]:
        assert lib.cusig_amd_sig_length(d, n) == expected
    import pysiglib_amd
    assert pysiglib_amd.sig_length(3, 4, scalar_term=True) == 121
    assert pysiglib_amd.sig_length(3, 4, time_aug=True, lead_lag=True, scalar_term=True) == 2801
    assert pysiglib_amd.sig_length(10, 5) == 111110
    with pytest.raises(ValueError):
        pysiglib_amd.sig_length(100, 100)


def test_shutdown_is_idempotent(lib):
    lib.cusig_shutdown.restype = None
    lib.cusig_shutdown()
    lib.cusig_shutdown()


def test_kernel_table(lib):
    fn = lib.cusig_amd_kernel_choice
    fn.argtypes = (ctypes.c_int, ctypes.c_int, ctypes.c_uint64, ctypes.c_uint64) + (ctypes.POINTER(ctypes.c_int),) * 3
    tail, k, spec = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    for bwd in (0, 1):
        for f64 in (0, 1):
            for (d, n) in ((10, 5), (5, 7), (3, 12), (17, 4)):
                assert fn(bwd, f64, d, n, tail, k, spec) == 1 and spec.value == 1 and 1 <= tail.value < n
            # the table reaches d = 128 at degree 3 (backward: up to 47 channels, where the by-row reverse sweep takes over),
            assert fn(bwd, f64, 100, 3, tail, k, spec) == 1 and spec.value == (0 if bwd else 1)
            assert fn(bwd, f64, 40, 4, tail, k, spec) == 1 and spec.value == 1      # 40 at degree 4, 20 at degree 5
            assert fn(bwd, f64, 20, 5, tail, k, spec) == 1 and spec.value == 1
            assert fn(bwd, f64, 150, 3, tail, k, spec) == 1 and spec.value == 0     # run-time-dimension kernel
            assert fn(bwd, f64, 2, 40, tail, k, spec) == 0                           # served by the run-time-degree sweeps, not by the table


def test_hooks_need_to_be_switched_on(lib):
    """The tuning and test hooks are ignored until cusig_amd_enable_test_hooks(1); switching them off restores the defaults
    (seen through the kernel table, a host-side query)."""
    fn = lib.cusig_amd_kernel_choice
    fn.argtypes = (ctypes.c_int, ctypes.c_int, ctypes.c_uint64, ctypes.c_uint64) + (ctypes.POINTER(ctypes.c_int),) * 3
    lib.cusig_amd_force_partition.argtypes = (ctypes.c_int, ctypes.c_int)
    lib.cusig_amd_force_partition.restype = None
    lib.cusig_amd_enable_test_hooks.argtypes = (ctypes.c_int,)
    lib.cusig_amd_enable_test_hooks.restype = None
    tail, k, spec = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()

    def letters_per_lane():
        assert fn(0, 0, 150, 3, tail, k, spec) == 1
        return k.value

    try:
        lib.cusig_amd_enable_test_hooks(0)
        default = letters_per_lane()
        assert default != 4
        lib.cusig_amd_force_partition(1, 4)
        assert letters_per_lane() == default          # ignored
        lib.cusig_amd_enable_test_hooks(1)
        lib.cusig_amd_force_partition(1, 4)
        assert letters_per_lane() == 4
        lib.cusig_amd_enable_test_hooks(0)
        assert letters_per_lane() == default          # defaults restored
    finally:
        lib.cusig_amd_enable_test_hooks(1)            # the session fixture's state


def test_wrapper_argument_errors():
    import pysiglib_amd as P
    x = torch.zeros(3, 4, 2)
    with pytest.raises(TypeError):
        P.sig(x, 2.0)
    with pytest.raises(ValueError):
        P.sig(x, -1)
    with pytest.raises(TypeError):
        P.sig(x, 2, time_aug=1)
    with pytest.raises(TypeError):
        P.sig(x, 2, end_time=1)
    with pytest.raises(ValueError):
        P.sig(x, 2, n_jobs=0)
    with pytest.raises(TypeError):
        P.sig([[0.0, 1.0]], 2)
    with pytest.raises(TypeError):
        P.sig(torch.zeros(3, 4, 2, dtype=torch.float16), 2)
    with pytest.raises(ValueError):
        P.sig(torch.zeros(4), 2)
    with pytest.raises(ValueError):
        P.sig(torch.zeros(4, 0), 2)
    # this package has no CPU path: host arrays are refused, never silently computed elsewhere
    with pytest.raises(RuntimeError):
        P.sig(np.zeros((4, 2)), 2)
    with pytest.raises(RuntimeError):
        P.sig(x, 2)

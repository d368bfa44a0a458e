"""pydtnn_hip_sgemm_static (the entry point that allocates nothing) against pydtnn_hip_sgemm, through the C ABI.

The two share their kernels; what differs is where the partial sums of the split along k live (an
array inside the library's device image instead of a caller workspace), so the bar is bit-for-bit
equality, on two calls in a row with the second problem smaller than the first (the array keeps the
first call's contents).
"""
import ctypes
import gc

import numpy as np
import pytest
import torch

from gpu_util import announce, assert_close, dev, host

pytestmark = pytest.mark.gpu


def _call_pair(native, m, n, k, ta, tb, bias, relu, seed):
    lib = native.lib()
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
    bias_h = rng.standard_normal(n).astype(np.float32) if bias else None
    a_d, b_d = dev(a), dev(b)
    bias_d = dev(bias_h) if bias else None
    lda, ldb = a.shape[1], b.shape[1]
    c_ws = torch.full((m, n), float("nan"), device="cuda")
    c_st = torch.full((m, n), float("nan"), device="cuda")
    need = lib.pydtnn_hip_sgemm_workspace_bytes(m, n, k)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    stream = native.stream_ptr()
    p = native.ptr
    rc = lib.pydtnn_hip_sgemm(ta, tb, m, n, k, p(a_d), lda, p(b_d), ldb, p(c_ws), n, p(bias_d), int(relu),
                              p(ws), need, stream)
    assert rc == 0, rc
    # everything the static call needs exists already: it must not allocate, neither through torch's caching
    # allocator nor behind its back (free device memory as the driver reports it; taken after a first static call
    # on the device, which loads the library's code object and resolves the address of its scratch array)
    if not _call_pair.warmed:
        rc = lib.pydtnn_hip_sgemm_static(ta, tb, m, n, k, p(a_d), lda, p(b_d), ldb, p(c_st), n, p(bias_d), int(relu),
                                         stream)
        assert rc == 0, rc
        _call_pair.warmed = True
    # tensors of earlier tests that only a collection of reference cycles frees must not be freed between the
    # two readings
    gc.collect()
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.pydtnn_hip_sgemm_static(ta, tb, m, n, k, p(a_d), lda, p(b_d), ldb, p(c_st), n, p(bias_d), int(relu),
                                     stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "the static-scratch call changed the device's free memory"
    ref = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    if bias:
        ref = ref + bias_h
    if relu:
        ref = np.maximum(ref, 0)
    return need, host(c_ws), host(c_st), ref


_call_pair.warmed = False


def test_static_scratch_gemm_equals_the_workspace_gemm_on_two_calls_in_a_row():
    from pydtnn_amd import native
    lib = native.lib()
    cap = lib.pydtnn_hip_sgemm_static_scratch_bytes()
    assert cap == 64 << 20
    # first a split problem that fills a good part of the array (an FC layer at batch 64), then smaller
    # ones, split and unsplit, in the three operand forms FC forward / dW / dX use
    cases = [(64, 4096, 6272, 0, 0, True, True), (64, 1000, 4096, 0, 0, True, False),
             (48, 200, 3000, 0, 1, False, False), (300, 40, 2000, 1, 0, False, False),
             (130, 70, 96, 0, 0, True, True)]
    split_seen = 0
    for i, (m, n, k, ta, tb, bias, relu) in enumerate(cases):
        announce("sgemm_static", m, n, k, ta, tb, bias, relu)
        need, c_ws, c_st, ref = _call_pair(native, m, n, k, ta, tb, bias, relu, seed=i)
        assert need <= cap
        split_seen += need > 0
        assert not np.isnan(c_st).any()
        assert np.array_equal(c_ws, c_st), f"case {i}: static-scratch result differs from the workspace result"
        assert_close(c_st, ref, what=f"sgemm_static case {i} vs fp64")
    assert split_seen >= 3


def test_static_scratch_covers_every_split_the_planner_makes():
    """The planner never asks for more than ~1022 accumulator tiles of partial sums, which is below the
    array's 64 MiB; should that change, the entry point returns PYDTNN_HIP_ERR_WORKSPACE instead."""
    from pydtnn_amd import native
    lib = native.lib()
    cap = lib.pydtnn_hip_sgemm_static_scratch_bytes()
    worst = 0
    for m in (1, 64, 100, 128, 1000, 2040, 4096):
        for n in (1, 64, 1000, 2040, 4096, 16320):
            for k in (16, 300, 4096, 25088, 1 << 20):
                worst = max(worst, lib.pydtnn_hip_sgemm_workspace_bytes(m, n, k))
    assert 0 < worst <= cap

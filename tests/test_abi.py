"""CPU-side checks of the C ABI and of the host logic (no GPU, no compute calls)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", "pydtnn_hip.h"), os.path.join(ROOT, "include", "pydtnn_hip_test.h")]


def declared_functions():
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text)
    keep = [n for n in names if n.startswith("pydtnn_hip_") or n.startswith("sconvGemm") or n == "alloc_pack_buffs"]
    return sorted(set(keep))


@pytest.fixture(scope="module")
def native():
    from pydtnn_amd import native as n
    if not os.path.exists(n.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return n


def test_header_declares_what_the_binding_table_binds(native):
    device_fns = [n for n in declared_functions() if n.startswith("pydtnn_hip_")]
    assert sorted(native.SIGNATURES) == device_fns


def test_device_library_exports_every_declared_symbol(native):
    lib = native.load_library()
    for name in declared_functions():
        if name.startswith("pydtnn_hip_"):
            assert hasattr(lib, name), name
    assert lib.pydtnn_hip_version() >= 100
    assert lib.pydtnn_hip_status_string(0) == b"ok"
    assert b"workspace" in lib.pydtnn_hip_status_string(2)


def test_compat_library_exports_the_reference_symbols(native):
    lib = ctypes.CDLL(native.COMPAT_LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name
    for name in native.COMPAT_SYMBOLS:
        assert hasattr(lib, name), name


def test_workspace_queries_are_pure_host_code(native):
    lib = native.load_library()
    cfg2 = (64, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1)
    kn_k = 256 * 2304 * 4
    # forward: optional scratch of the balanced launch, two 128x128 accumulator tiles for each of 1024 workgroups
    balance = 2 * 1024 * 128 * 128 * 4
    # dW: the partial sums of the reduction split (a multiple of the filter tensor), at least the scratch of the
    # balanced launch
    dw = lib.pydtnn_hip_conv_workspace_bytes(native.OP_DW, 0, *cfg2)
    assert dw == balance or (dw > balance and dw % kn_k == 0 and dw // kn_k <= 64 * 4)
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_FWD, 0, *cfg2) == balance
    # stride 1: dX needs the flipped filter and runs as a forward launch; strided: the (K x P) matrix of the
    # explicit route
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_DX, 0, *cfg2) == kn_k + balance
    strided = (8, 3, 32, 32, 16, 3, 3, 1, 1, 2, 2, 1, 1)
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_DX, 0, *strided) == 27 * 8 * 16 * 16 * 4 + balance
    # the explicit route: the (K x P) product and behind it the scratch of the balanced launch; forward only the latter
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_DX_I2C, 1, *cfg2) == 2304 * 64 * 56 * 56 * 4 + balance
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_FWD_I2C, 0, *cfg2) == balance
    # invalid geometry (kernel larger than the padded image) yields 0, not a crash
    assert lib.pydtnn_hip_conv_workspace_bytes(native.OP_DW, 0, 1, 1, 2, 2, 1, 5, 5, 0, 0, 1, 1, 1, 1) == 0
    assert lib.pydtnn_hip_sgemm_workspace_bytes(4096, 4096, 4096) == 0
    assert lib.pydtnn_hip_sgemm_workspace_bytes(64, 4096, 25088) > 0
    # float64 GEMM: split along k for a small C with a long reduction; for a C of many tiles whose last round of
    # the 512 resident workgroups is nearly empty (3136 tiles = 6.125 rounds) the partial tiles of the tail launch:
    # 64 tiles x 8 chunks of k x 128 x 128 doubles; nothing for a C whose rounds come out even
    assert lib.pydtnn_hip_dgemm_workspace_bytes(256, 2304, 200704) > 0
    assert lib.pydtnn_hip_dgemm_workspace_bytes(256, 200704, 2304) == 64 * 8 * 128 * 128 * 8
    assert lib.pydtnn_hip_dgemm_workspace_bytes(1024, 8192, 512) == 0


def test_dgemm_refuses_leading_dimensions_its_offsets_cannot_hold(native):
    """Argument checks only: the call returns before anything is launched."""
    lib = native.lib()
    one = ctypes.c_void_p(1)
    args = lambda lda, ldb: (0, 0, 4, 4, 4, one, lda, one, ldb, one, 4, None, 0, None, 0, None)
    assert lib.pydtnn_hip_dgemm(*args(1 << 22, 4)) == native.PYDTNN_HIP_ERR_UNSUPPORTED
    assert lib.pydtnn_hip_dgemm(*args(4, 1 << 22)) == native.PYDTNN_HIP_ERR_UNSUPPORTED
    assert lib.pydtnn_hip_dgemm(*args(3, 4)) == native.PYDTNN_HIP_ERR_INVALID      # lda < k


def test_missing_library_is_an_import_error(native):
    with pytest.raises(ImportError):
        native.load_library("/nonexistent/libpydtnn_hip.so")


def test_host_tensors_are_rejected_before_any_launch(native):
    from pydtnn_amd import ops
    with pytest.raises(ValueError):
        ops.im2col_nchw(torch.zeros((1, 1, 4, 4)), 3, 3, 0, 0, 1, 1, 1, 1)
    with pytest.raises(ValueError):  # float64 is the explicit route's second dtype: same rule, no launch
        ops.im2col_nchw(torch.zeros((1, 1, 4, 4), dtype=torch.float64), 3, 3, 0, 0, 1, 1, 1, 1)
    with pytest.raises(TypeError):   # pydtnn/cython_modules/im2col_nchw_cython.pyx:49-50
        ops.im2col_nchw(torch.zeros((1, 1, 4, 4), dtype=torch.int32), 3, 3, 0, 0, 1, 1, 1, 1)
    with pytest.raises(TypeError):   # float32 and float64 operands do not mix
        ops.matmul(torch.zeros((2, 2)), torch.zeros((2, 2), dtype=torch.float64))


def test_tensor_format_helpers():
    from pydtnn_amd.utils import (PYDTNN_TENSOR_FORMAT_NCHW, PYDTNN_TENSOR_FORMAT_NHWC, decode_tensor,
                                  encode_tensor)
    assert encode_tensor((5, 6, 7), PYDTNN_TENSOR_FORMAT_NCHW) == (7, 5, 6)
    assert decode_tensor((7, 5, 6), PYDTNN_TENSOR_FORMAT_NCHW) == (5, 6, 7)
    assert encode_tensor((5, 6, 7), PYDTNN_TENSOR_FORMAT_NHWC) == (5, 6, 7)
    assert decode_tensor((10,), PYDTNN_TENSOR_FORMAT_NCHW) == (10,)


def test_gemm_operand_views():
    from pydtnn_amd.ops import _as_gemm_operand
    a = torch.zeros((3, 5))
    assert _as_gemm_operand(a)[1:] == (0, 5)
    assert _as_gemm_operand(a.t())[1:] == (1, 5)
    with pytest.raises(ValueError):
        _as_gemm_operand(torch.zeros((4, 8))[:, ::2])


def test_conv_gemm_shim_rejects_other_dtypes(native):
    from pydtnn_amd.conv_gemm import ConvGemm
    with pytest.raises(ValueError):
        ConvGemm(dtype=np.float64)
    with pytest.raises(AttributeError):
        ConvGemm(dtype="int8")
    assert ConvGemm(dtype=np.float32).dtype == torch.float32

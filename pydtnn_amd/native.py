"""ctypes binding of libpydtnn_hip.so (C ABI declared in include/pydtnn_hip.h).

PyTorch-ROCm is used only as the owner of device memory and of the HIP stream: every call
passes ``tensor.data_ptr()`` and ``torch.cuda.current_stream().cuda_stream`` to the library.
There is no fallback: if the shared library is missing, or no GPU is present, calls raise.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpydtnn_hip.so")
COMPAT_LIB_PATH = os.path.join(LIB_DIR, "libconvGemm.so")

OP_FWD, OP_DW, OP_DX, OP_DX_I2C, OP_DB, OP_FWD_I2C = range(6)
# status codes of include/pydtnn_hip.h
PYDTNN_HIP_OK, PYDTNN_HIP_ERR_INVALID, PYDTNN_HIP_ERR_WORKSPACE, PYDTNN_HIP_ERR_LAUNCH, PYDTNN_HIP_ERR_UNSUPPORTED = range(5)

_c = ctypes
_f32p, _i8p, _i32p, _vp = _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p
_geom13_i = [_c.c_int] * 13
_geom13_u = [_c.c_uint] * 13

# name -> (restype, argtypes); kept in one table so a test can check every declared symbol loads
SIGNATURES = {
    "pydtnn_hip_version": (_c.c_int, []),
    "pydtnn_hip_status_string": (_c.c_char_p, [_c.c_int]),
    "pydtnn_hip_debug_set_tensor_floats_limit": (_c.c_long, [_c.c_long]),  # test-only (include/pydtnn_hip_test.h)
    "pydtnn_hip_debug_last_launch": (None, [_c.POINTER(_c.c_int)]),  # test-only (include/pydtnn_hip_test.h)
    "pydtnn_hip_im2col_nchw": (_c.c_int, [_f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_col2im_nchw": (_c.c_int, [_f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_im2row_nhwc": (_c.c_int, [_f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_row2im_nhwc": (_c.c_int, [_f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_sgemm_workspace_bytes": (_c.c_size_t, [_c.c_long] * 3),
    "pydtnn_hip_sgemm": (_c.c_int, [_c.c_int, _c.c_int, _c.c_long, _c.c_long, _c.c_long, _f32p, _c.c_long, _f32p,
                                    _c.c_long, _f32p, _c.c_long, _f32p, _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sgemm_static_scratch_bytes": (_c.c_size_t, []),
    "pydtnn_hip_sgemm_static": (_c.c_int, [_c.c_int, _c.c_int, _c.c_long, _c.c_long, _c.c_long, _f32p, _c.c_long, _f32p,
                                           _c.c_long, _f32p, _c.c_long, _f32p, _c.c_int, _vp]),
    "pydtnn_hip_conv_workspace_bytes": (_c.c_size_t, [_c.c_int, _c.c_int] + _geom13_i),
    "pydtnn_hip_sconvGemmNCHW": (_c.c_int, [_c.c_char] + _geom13_u + [_f32p] * 8 + [_c.c_bool, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemmNHWC": (_c.c_int, [_c.c_char] + _geom13_u + [_f32p] * 8 + [_c.c_bool, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemmNCHW_back": (_c.c_int, _geom13_u + [_f32p] * 3 + [_vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemmNHWC_back": (_c.c_int, _geom13_u + [_f32p] * 3 + [_vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemm_pair_nhwc": (_c.c_int, _geom13_u + [_f32p] * 7 + [_c.c_bool, _c.c_uint] + [_f32p] * 7 +
                                       [_c.c_bool, _f32p, _c.c_bool, _vp]),
    "pydtnn_hip_conv_plan_create": (_c.c_int, [_c.POINTER(_c.c_void_p), _c.c_int] + _geom13_i + [_f32p] * 6 + [_c.c_bool]),
    "pydtnn_hip_conv_plan_forward": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_size_t,
                                                _c.c_void_p]),
    "pydtnn_hip_conv_plan_destroy": (None, [_c.c_void_p]),
    "pydtnn_hip_sconvGemm_relu_mask": (_c.c_int, [_c.c_int] + _geom13_u + [_f32p] * 4 + [_i8p, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemm_residual": (_c.c_int, [_c.c_int] + _geom13_u + [_f32p] * 8 + [_c.c_bool, _f32p, _c.c_bool, _vp,
                                                 _c.c_size_t, _vp]),
    "pydtnn_hip_sconvGemm_back_gated": (_c.c_int, [_c.c_int] + _geom13_u + [_f32p] * 3 + [_i8p, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_max_pool_2d_bwd_gated": (_c.c_int, [_c.c_int, _f32p, _i32p, _f32p, _i8p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_conv_i2c_forward": (_c.c_int, [_c.c_int] + _geom13_i + [_f32p] * 4 + [_vp, _c.c_size_t, _vp]),
    "pydtnn_hip_conv_i2c_dw": (_c.c_int, [_c.c_int] + _geom13_i + [_f32p] * 3 + [_vp, _c.c_size_t, _vp]),
    "pydtnn_hip_conv_i2c_dx": (_c.c_int, [_c.c_int] + _geom13_i + [_f32p] * 3 + [_vp, _c.c_size_t, _vp]),
    "pydtnn_hip_chan_eltwise": (_c.c_int, [_f32p, _f32p, _f32p, _c.c_long, _c.c_int, _c.c_int] + [_f32p] * 5 +
                                [_c.c_int, _vp]),
    "pydtnn_hip_relu_fwd": (_c.c_int, [_f32p, _f32p, _i8p, _c.c_long, _vp]),
    "pydtnn_hip_relu_bwd": (_c.c_int, [_f32p, _i8p, _f32p, _c.c_long, _vp]),
    "pydtnn_hip_bias_grad": (_c.c_int, [_f32p, _f32p, _c.c_long, _c.c_int, _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_max_pool_2d_fwd_nchw": (_c.c_int, [_f32p, _f32p, _i32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_max_pool_2d_bwd_nchw": (_c.c_int, [_f32p, _i32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_max_pool_2d_fwd_nhwc": (_c.c_int, [_f32p, _f32p, _i32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_max_pool_2d_bwd_nhwc": (_c.c_int, [_f32p, _i32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_average_pool_2d_fwd": (_c.c_int, [_c.c_int, _f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_average_pool_2d_bwd": (_c.c_int, [_c.c_int, _f32p, _f32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_bn_training_workspace_bytes": (_c.c_size_t, [_c.c_int]),
    "pydtnn_hip_bn_training_fwd": (_c.c_int, [_f32p] * 8 + [_c.c_double, _c.c_double, _c.c_long, _c.c_int, _c.c_int,
                                                        _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_bn_training_bwd": (_c.c_int, [_f32p] * 7 + [_c.c_long, _c.c_int, _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_softmax_fwd": (_c.c_int, [_f32p, _f32p, _c.c_int, _c.c_int, _vp]),
    "pydtnn_hip_softmax_bwd": (_c.c_int, [_f32p, _f32p, _f32p, _c.c_int, _c.c_int, _vp]),
    "pydtnn_hip_categorical_cross_entropy": (_c.c_int, [_f32p, _f32p, _f32p, _f32p, _c.c_int, _c.c_int, _c.c_double,
                                                        _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sgd_momentum": (_c.c_int, [_f32p, _f32p, _f32p, _c.c_long, _c.c_float, _c.c_float, _c.c_float,
                                           _c.c_int, _vp]),
    "pydtnn_hip_sgd_momentum_multi": (_c.c_int, [_c.c_int, _vp, _vp, _vp, _vp, _c.c_float, _c.c_float, _c.c_float,
                                                 _c.c_int, _vp]),
    # float64 route
    "pydtnn_hip_dgemm_workspace_bytes": (_c.c_size_t, [_c.c_long] * 3),
    "pydtnn_hip_dgemm": (_c.c_int, [_c.c_int, _c.c_int, _c.c_long, _c.c_long, _c.c_long, _vp, _c.c_long, _vp, _c.c_long,
                                    _vp, _c.c_long, _vp, _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_im2col_nchw_f64": (_c.c_int, [_vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_col2im_nchw_f64": (_c.c_int, [_vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_im2row_nhwc_f64": (_c.c_int, [_vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_row2im_nhwc_f64": (_c.c_int, [_vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_chan_eltwise_f64": (_c.c_int, [_vp, _vp, _vp, _c.c_long, _c.c_long, _c.c_int] + [_vp] * 5 +
                                    [_c.c_int, _vp]),
    "pydtnn_hip_relu_fwd_f64": (_c.c_int, [_vp, _vp, _i8p, _c.c_long, _vp]),
    "pydtnn_hip_relu_bwd_f64": (_c.c_int, [_vp, _i8p, _vp, _c.c_long, _vp]),
    "pydtnn_hip_bias_grad_f64": (_c.c_int, [_vp, _vp, _c.c_long, _c.c_int, _c.c_long, _vp]),
    "pydtnn_hip_transpose_1023_f64": (_c.c_int, [_vp, _vp, _c.c_int, _c.c_int, _c.c_long, _vp]),
    "pydtnn_hip_max_pool_2d_fwd_f64": (_c.c_int, [_c.c_int, _vp, _vp, _i32p] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_max_pool_2d_bwd_f64": (_c.c_int, [_c.c_int, _vp, _i32p, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_average_pool_2d_fwd_f64": (_c.c_int, [_c.c_int, _vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_average_pool_2d_bwd_f64": (_c.c_int, [_c.c_int, _vp, _vp] + [_c.c_int] * 12 + [_vp]),
    "pydtnn_hip_softmax_fwd_f64": (_c.c_int, [_vp, _vp, _c.c_int, _c.c_int, _vp]),
    "pydtnn_hip_softmax_bwd_f64": (_c.c_int, [_vp, _vp, _vp, _c.c_int, _c.c_int, _vp]),
    "pydtnn_hip_categorical_cross_entropy_f64": (_c.c_int, [_vp, _vp, _vp, _vp, _c.c_int, _c.c_int, _c.c_double,
                                                            _c.c_int, _vp, _c.c_size_t, _vp]),
    "pydtnn_hip_sgd_momentum_f64": (_c.c_int, [_vp, _vp, _vp, _c.c_long, _c.c_double, _c.c_double, _c.c_double,
                                               _c.c_int, _vp]),
    "pydtnn_hip_bn_training_fwd_f64": (_c.c_int, [_vp] * 8 + [_c.c_double, _c.c_double, _c.c_long, _c.c_int, _c.c_long,
                                                            _vp]),
    "pydtnn_hip_bn_training_bwd_f64": (_c.c_int, [_vp] * 7 + [_c.c_long, _c.c_int, _c.c_long, _vp]),
}

# Host-pointer flavour exported by libconvGemm.so with the reference's own names
COMPAT_SYMBOLS = ["alloc_pack_buffs", "sconvGemmNCHW", "sconvGemmNHWC", "sconvGemmNCHW_back", "sconvGemmNHWC_back",
                  "pydtnn_convgemm_last_status"]

_LIB = None


class HipError(RuntimeError):
    pass


def load_library(path=LIB_PATH):
    """Load the shared library and attach prototypes.  Raises ImportError when it is not built."""
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `make -C pydtnn_amd/csrc` "
                          f"(or __graft_entry__.build()); there is no CPU fallback.")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def lib():
    global _LIB
    if _LIB is None:
        _LIB = load_library()
    return _LIB


def check(status, what):
    if status != 0:
        raise HipError(f"{what}: {lib().pydtnn_hip_status_string(status).decode()} (status {status})")


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    """Device address of a dense fp32/int tensor, or NULL for None."""
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("expected a tensor on the GPU")
    if not t.is_contiguous():
        raise ValueError("expected a C-contiguous tensor")
    return ctypes.c_void_p(t.data_ptr())


def f32(t, name="tensor"):
    if t is not None and t.dtype != torch.float32:
        # pydtnn/backends/cpu/libs/conv_gemm.py:101-107: only float32 is supported by this ABI
        raise ValueError(f"Type {t.dtype} of {name} not supported by this version of the library!")
    return ptr(t)


# --------------------------------------------------------------------------- workspace
# One grow-only scratch buffer per (device, stream): work is enqueued on the caller's current stream, so
# consecutive calls on a stream use its buffer strictly one after the other, and calls on different streams
# never share one.  A buffer that is outgrown is released to torch's caching allocator, which keeps a block
# away from other streams until the work queued on its own stream has passed.
_WORKSPACE = {}


def workspace(nbytes, dev=None, raw_stream=None):
    """Returns (void* or None, size) for a scratch buffer of at least ``nbytes`` bytes on the current device and
    stream (or the given ones: a device index and a raw stream handle)."""
    if nbytes == 0:
        return None, 0
    if dev is None:
        dev = torch.cuda.current_device()
    key = (dev, torch.cuda.current_stream().cuda_stream if raw_stream is None else raw_stream)
    buf = _WORKSPACE.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            del _WORKSPACE[key]
            del buf
        buf = torch.empty(int(nbytes * 1.25) + 256, dtype=torch.uint8, device=f"cuda:{dev}")
        _WORKSPACE[key] = buf
    return ctypes.c_void_p(buf.data_ptr()), buf.numel()


def workspace_buffer(key):
    """The tensor that currently backs the scratch buffer of ``key`` = (device index, raw stream handle), or None."""
    return _WORKSPACE.get(key)


_LAUNCH_KINDS = ("none", "tiles", "balanced", "stream_nhwc", "stream_nchw", "pair")


def last_launch():
    """The form of this thread's most recent GEMM or streaming-convolution launch, as the library's test-only query
    pydtnn_hip_debug_last_launch reports it (include/pydtnn_hip_test.h): benchmarks and tests that are about one
    kernel form check with it that the library picked that form."""
    out = (_c.c_int * 6)()
    lib().pydtnn_hip_debug_last_launch(out)
    return {"kind": _LAUNCH_KINDS[out[0]], "tile": [out[1], out[2]], "workgroups": out[3], "cut_tiles": out[4],
            "splits": out[5]}


_WORKSPACE_BYTES = {}


def conv_workspace(op, nhwc, geom13, raw_stream=None):
    """Scratch buffer for one convolution call; the size query is remembered per (device, operation, geometry),
    since it depends on nothing else and a layer asks with the same geometry at every step."""
    key = (torch.cuda.current_device(), op, int(nhwc), tuple(geom13))
    nbytes = _WORKSPACE_BYTES.get(key)
    if nbytes is None:
        nbytes = lib().pydtnn_hip_conv_workspace_bytes(op, int(nhwc), *geom13)
        if len(_WORKSPACE_BYTES) < 4096:
            _WORKSPACE_BYTES[key] = nbytes
    return workspace(nbytes, raw_stream=raw_stream)

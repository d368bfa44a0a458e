"""Tensor-format helpers and host<->device conveniences (mirror of pydtnn/utils/__init__.py:30-44)."""
import numpy as np
import torch

PYDTNN_TENSOR_FORMATS = 2
(PYDTNN_TENSOR_FORMAT_NHWC,
 PYDTNN_TENSOR_FORMAT_NCHW) = range(PYDTNN_TENSOR_FORMATS)


def encode_tensor(shape, tensor_format=PYDTNN_TENSOR_FORMAT_NHWC):
    """(h, w, c) -> per-sample shape in the model's format (pydtnn/utils/__init__.py:34-38)."""
    if len(shape) == 3 and tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
        return (shape[2], shape[0], shape[1])
    return shape


def decode_tensor(shape, tensor_format=PYDTNN_TENSOR_FORMAT_NHWC):
    """Per-sample shape in the model's format -> (h, w, c) (pydtnn/utils/__init__.py:40-44)."""
    if len(shape) == 3 and tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
        return (shape[1], shape[2], shape[0])
    return shape


def to_device(a, dtype=torch.float32):
    """NumPy array (or tensor) -> dense tensor on the current GPU."""
    if isinstance(a, torch.Tensor):
        return a.to(device="cuda", dtype=dtype).contiguous()
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dtype)


def to_host(t):
    """Device tensor -> NumPy array (synchronises)."""
    return t.detach().cpu().numpy()

"""MI355X-native implementation of PyDTNN's conv-as-GEMM hot path.

Conv2D / FC ``forward()`` / ``backward()`` behind PyDTNN's layer protocol, the NCHW / NHWC
``tensor_format`` switch and the conv/BN/ReLU inference fusions, running on hand-written gfx950
kernels (``csrc/``) through a thin C ABI (``include/pydtnn_hip.h``).  There is no CPU fallback:
importing the layers works anywhere, running them needs the built library and a GPU.
"""
from .layers import (EVALUATE_MODE, TRAIN_MODE, UNSPECIFIED_MODE, AdditionBlock, AveragePool2D, BatchNormalization,
                     BatchNormalizationRelu, Conv2D, Conv2DBatchNormalization, Conv2DBatchNormalizationRelu,
                     Conv2DRelu, Dropout, FC, Flatten, Input, Layer, MaxPool2D, Relu, Softmax)
from .model import SGD, CategoricalCrossEntropy, Model
from . import models, tracers
from .best_of import BestOf
from .conv_gemm import ConvGemm
from .utils import (PYDTNN_TENSOR_FORMAT_NCHW, PYDTNN_TENSOR_FORMAT_NHWC, decode_tensor, encode_tensor, to_device,
                    to_host)

__all__ = [name for name in dir() if not name.startswith("_")]

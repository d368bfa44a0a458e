"""Shared problem shapes for the parity tests.

``D`` mirrors the parameter record of the reference's tests
(pydtnn/tests/common.py:35-74) and ``alexnet_layers`` its table of ten AlexNet
convolutions (pydtnn/tests/common.py:77-90).  The hand-made arrays are the
literal inputs of pydtnn/tests/conv_gemm.py:81-209 and
pydtnn/tests/conv2d_conv_gemm.py:72-103 (inputs only: the reference stores no
expected outputs).
"""
import numpy as np


class D:
    def __init__(self, b=1, c=1, h=128, w=100, kn=1, kh=16, kw=10, vpadding=1, hpadding=1,
                 vstride=1, hstride=1, vdilation=1, hdilation=1):
        self.b, self.c, self.h, self.w = b, c, h, w
        self.kn, self.kh, self.kw = kn, kh, kw
        self.vpadding, self.hpadding = vpadding, hpadding
        self.vstride, self.hstride = vstride, hstride
        self.vdilation, self.hdilation = vdilation, hdilation

    @property
    def ho(self):
        return (self.h + 2 * self.vpadding - self.vdilation * (self.kh - 1) - 1) // self.vstride + 1

    @property
    def wo(self):
        return (self.w + 2 * self.hpadding - self.hdilation * (self.kw - 1) - 1) // self.hstride + 1

    def geom(self):
        return (self.kh, self.kw, self.vpadding, self.hpadding, self.vstride, self.hstride,
                self.vdilation, self.hdilation)

    def __repr__(self):
        return (f"D(b={self.b},c={self.c},h={self.h},w={self.w},kn={self.kn},kh={self.kh},kw={self.kw},"
                f"pad=({self.vpadding},{self.hpadding}),stride=({self.vstride},{self.hstride}),"
                f"dil=({self.vdilation},{self.hdilation}))")


alexnet_layers = [
    # AlexNet Cifar
    D(64, 3, 32, 32, 64, 3, 3, 1, 1, 2, 2, 1, 1),
    D(64, 64, 8, 8, 192, 3, 3, 1, 1, 1, 1, 1, 1),
    D(64, 192, 4, 4, 384, 3, 3, 1, 1, 1, 1, 1, 1),
    D(64, 384, 4, 4, 256, 3, 3, 1, 1, 1, 1, 1, 1),
    D(64, 256, 4, 4, 256, 3, 3, 1, 1, 1, 1, 1, 1),
    # AlexNet ImageNet
    D(64, 3, 227, 227, 96, 11, 11, 1, 1, 4, 4, 1, 1),
    D(64, 96, 27, 27, 256, 5, 5, 1, 1, 1, 1, 1, 1),
    D(64, 256, 13, 13, 384, 3, 3, 1, 1, 1, 1, 1, 1),
    D(64, 384, 13, 13, 384, 3, 3, 1, 1, 1, 1, 1, 1),
    D(64, 384, 13, 13, 256, 3, 3, 1, 1, 1, 1, 1, 1),
]

f32 = np.float32

x_2x4 = np.array([[[[1, 2, 4, 8], [16, 32, 64, 128]]]], dtype=f32)
x_2x4_c2 = np.array([[[[1, 2, 4, 8], [16, 32, 64, 128]],
                      [[128, 256, 512, 1024], [2048, 4096, 8192, 16384]]]], dtype=f32)
x_4x4 = np.array([[[[1, 2, 4, 8], [16, 32, 64, 128], [1, 2, 4, 8], [16, 32, 64, 128]]]], dtype=f32)
x_4x8 = np.array([[[[1, 2, 4, 8, 9, 10, 11, 12], [16, 32, 64, 128, 129, 130, 131, 132],
                    [1, 2, 4, 8, 9, 10, 11, 12], [16, 32, 64, 128, 129, 130, 131, 132]]]], dtype=f32)
x_8x8 = (np.arange(1, 9, dtype=f32)[None, :] + 10 * np.arange(1, 9, dtype=f32)[:, None])[None, None]

w_1x1 = np.ones((1, 1, 1, 1), dtype=f32)
w_1x2 = np.ones((1, 1, 1, 2), dtype=f32)
w_2x2 = np.ones((1, 1, 2, 2), dtype=f32)
w_3x3 = np.ones((1, 1, 3, 3), dtype=f32)
w_c2_1234_4567 = np.array([[[[1, 2], [3, 4]], [[4, 5], [6, 7]]]], dtype=f32)

# A spread of small geometries: unequal strides, dilation, rectangular kernels, pad > 0,
# kernels larger than the image interior, and channel / filter counts that are not tile multiples.
small_grid = [
    D(1, 1, 5, 5, 1, 3, 3, 0, 0, 1, 1, 1, 1),
    D(2, 3, 7, 6, 4, 3, 3, 1, 1, 1, 1, 1, 1),
    D(3, 2, 9, 10, 5, 3, 2, 2, 1, 2, 3, 1, 1),
    D(2, 4, 11, 9, 3, 3, 3, 2, 2, 1, 1, 2, 2),
    D(1, 5, 8, 8, 7, 1, 1, 0, 0, 1, 1, 1, 1),
    D(2, 3, 8, 8, 6, 1, 1, 0, 0, 2, 2, 1, 1),
    D(2, 2, 6, 6, 2, 5, 5, 2, 2, 1, 1, 1, 1),
    D(4, 7, 13, 12, 33, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 3, 12, 12, 8, 4, 4, 0, 0, 4, 4, 1, 1),
    D(3, 1, 10, 7, 2, 2, 3, 3, 4, 1, 2, 1, 1),
    D(2, 6, 9, 9, 5, 3, 3, 1, 1, 2, 2, 1, 2),
]

# Channel counts from 32 up, where the NHWC gathers take their LDS-staged form: slabs that are not
# multiples of 64, more than one slab, segments that do not divide the row, strides, dilation,
# rectangular filters, padding larger than the filter reach, a filter wider than the image interior.
wide_channel_grid = [
    D(2, 32, 9, 11, 4, 3, 3, 1, 1, 1, 1, 1, 1),
    D(1, 40, 7, 19, 3, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 64, 12, 17, 5, 3, 3, 1, 1, 2, 2, 1, 1),
    D(1, 96, 10, 10, 2, 5, 3, 2, 1, 1, 1, 1, 1),
    D(1, 130, 8, 21, 2, 3, 3, 2, 2, 1, 1, 2, 2),
    D(2, 72, 9, 33, 2, 2, 4, 0, 3, 1, 3, 1, 1),
    D(1, 300, 6, 6, 2, 1, 1, 0, 0, 1, 1, 1, 1),
    D(1, 64, 5, 40, 2, 3, 7, 1, 3, 2, 1, 1, 2),
    D(1, 48, 14, 14, 2, 3, 3, 3, 3, 2, 2, 1, 1),
    # 3x3 at stride 1: no padding, padding 2, mixed padding, planes of whole and of ragged 8x8 patches
    D(3, 64, 17, 8, 2, 3, 3, 0, 0, 1, 1, 1, 1),
    D(2, 8, 16, 16, 2, 3, 3, 2, 2, 1, 1, 1, 1),
    D(1, 16, 8, 24, 2, 3, 3, 1, 0, 1, 1, 1, 1),
    D(2, 24, 3, 5, 2, 3, 3, 1, 1, 1, 1, 1, 1),
]

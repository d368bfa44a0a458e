"""GPU parity tests of the kernels, through the C ABI, against the CPU oracle on the same seeded inputs.

Bar: bit-exact for the index-only kernels (im2col, col2im, im2row, row2im, ReLU mask, maxpool);
max |a-b| / max |b| <= 1e-4 for fp32 arithmetic (GEMMs and fused epilogues).
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import FP32_REL_TOL, announce, assert_close, dev, host, rel_err
from shapes import D, alexnet_layers, small_grid, wide_channel_grid, x_2x4, x_2x4_c2, x_4x4, x_4x8, x_8x8, w_1x1, w_1x2, w_2x2, w_3x3, \
    w_c2_1234_4567

pytestmark = pytest.mark.gpu

mid_grid = [
    D(3, 5, 20, 17, 70, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 16, 30, 30, 130, 3, 3, 1, 1, 1, 1, 1, 1),
    D(4, 3, 35, 35, 96, 11, 11, 0, 0, 4, 4, 1, 1),
    D(2, 33, 14, 14, 257, 1, 1, 0, 0, 1, 1, 1, 1),
    D(5, 8, 19, 23, 20, 5, 3, 2, 1, 2, 1, 1, 1),
    D(2, 12, 16, 16, 24, 3, 3, 2, 2, 1, 1, 2, 2),
    D(9, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(3, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1, 1, 1),
]
all_grid = small_grid + mid_grid

# NHWC shapes that take the streaming kernel (filter matrix resident in LDS, at most 36864 floats, channels in
# chunks of 64, at least 32768 output pixels): the three convolutions of a ResNet bottleneck, a strided
# 1x1 shortcut, a dilated 3x3, 128 filters
stream_grid = [
    D(16, 256, 56, 56, 64, 1, 1, 0, 0, 1, 1, 1, 1),
    D(16, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(16, 64, 56, 56, 256, 1, 1, 0, 0, 1, 1, 1, 1),
    D(48, 128, 56, 56, 256, 1, 1, 0, 0, 2, 2, 1, 1),
    D(16, 64, 48, 48, 64, 3, 3, 2, 2, 1, 1, 2, 2),
    D(11, 128, 64, 64, 128, 1, 1, 0, 0, 1, 1, 1, 1),
    D(40, 64, 31, 33, 128, 2, 2, 1, 0, 1, 1, 1, 1),
    # 512 filters over 128 channels: two workgroups per pixel range, 256 filters each (the second shape leaves the
    # compute units pixel ranges of unequal length)
    D(16, 128, 48, 48, 512, 1, 1, 0, 0, 1, 1, 1, 1),
    D(13, 128, 56, 56, 512, 1, 1, 0, 0, 1, 1, 1, 1),
]


@pytest.fixture(scope="module")
def ops():
    from pydtnn_amd import ops as _ops, native
    native.lib()  # raises if the HIP library was not built: no fallback
    assert torch.cuda.is_available()
    return _ops


@pytest.fixture(scope="module")
def cg():
    from pydtnn_amd.conv_gemm import ConvGemm
    return ConvGemm()


def case(d, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(np.float32)
    w = (rng.standard_normal((d.kn, d.c, d.kh, d.kw)) * np.sqrt(2.0 / (d.c * d.kh * d.kw))).astype(np.float32)
    b = rng.standard_normal(d.kn).astype(np.float32)
    dy = rng.standard_normal((d.b, d.kn, d.ho, d.wo)).astype(np.float32)
    return x, w, b, dy


def nhwc(a):
    return np.ascontiguousarray(a.transpose(0, 2, 3, 1))


def w_nhwc(w):
    return np.ascontiguousarray(w.transpose(1, 2, 3, 0))  # (kn,c,kh,kw) -> (c,kh,kw,kn)


# ------------------------------------------------------------------ explicit gathers: bit-exact

@pytest.mark.parametrize("d", all_grid, ids=repr)
def test_im2col_col2im_nchw_bit_exact(ops, oracle, d):
    announce("im2col/col2im nchw", d)
    x, _, _, _ = case(d)
    cols = ops.im2col_nchw(dev(x), *d.geom())
    ref = oracle.im2col_nchw(x, *d.geom())
    assert np.array_equal(host(cols), ref)
    rng = np.random.default_rng(1)
    cmat = rng.standard_normal(ref.shape).astype(np.float32)
    dx = ops.col2im_nchw(dev(cmat), d.b, d.c, d.h, d.w, *d.geom())
    # same addends in the same order as the reference's scatter loop: identical fp32 sums
    assert np.array_equal(host(dx), oracle.col2im_nchw(cmat, d.b, d.c, d.h, d.w, *d.geom()))


@pytest.mark.parametrize("d", all_grid, ids=repr)
def test_im2row_row2im_nhwc_bit_exact(ops, oracle, d):
    announce("im2row/row2im nhwc", d)
    x, _, _, _ = case(d)
    xr = nhwc(x)
    rows = ops.im2row_nhwc(dev(xr), *d.geom())
    ref = oracle.im2row_nhwc(xr, *d.geom())
    assert np.array_equal(host(rows), ref)
    rng = np.random.default_rng(1)
    rmat = rng.standard_normal(ref.shape).astype(np.float32)
    dx = ops.row2im_nhwc(dev(rmat), d.b, d.h, d.w, d.c, *d.geom())
    assert np.array_equal(host(dx), oracle.row2im_nhwc(rmat, d.b, d.h, d.w, d.c, *d.geom()))


# 3x3 at unit stride with channels in chunks of 32: row2im walks bands of dx rows (strips of at most 64
# columns; 8, 16, 32, 56 or 64 columns per strip by template), im2row hands its pixel runs to the XCDs
walk_grid = [
    D(3, 32, 7, 7, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 64, 14, 14, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 32, 28, 28, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 96, 56, 56, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(1, 32, 64, 64, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(1, 32, 33, 70, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    D(1, 64, 19, 131, 2, 3, 3, 0, 2, 1, 1, 1, 1),
    D(2, 32, 37, 23, 2, 3, 3, 2, 0, 1, 1, 1, 1),
    D(1, 32, 40, 9, 2, 3, 3, 0, 0, 1, 1, 1, 1),
    D(1, 32, 3, 3, 2, 3, 3, 0, 0, 1, 1, 1, 1),
    D(1, 32, 2, 5, 2, 3, 3, 2, 2, 1, 1, 1, 1),
]


@pytest.mark.parametrize("d", walk_grid, ids=repr)
def test_nhwc_gathers_walk_form_bit_exact(ops, oracle, d):
    announce("im2row/row2im nhwc walk", d)
    rng = np.random.default_rng(3)
    xr = rng.standard_normal((d.b, d.h, d.w, d.c)).astype(np.float32)
    assert np.array_equal(host(ops.im2row_nhwc(dev(xr), *d.geom())), oracle.im2row_nhwc(xr, *d.geom()))
    rmat = rng.standard_normal((d.b * d.ho * d.wo, d.c * d.kh * d.kw)).astype(np.float32)
    dx = ops.row2im_nhwc(dev(rmat), d.b, d.h, d.w, d.c, *d.geom())
    assert np.array_equal(host(dx), oracle.row2im_nhwc(rmat, d.b, d.h, d.w, d.c, *d.geom()))


@pytest.mark.parametrize("d", wide_channel_grid, ids=repr)
def test_nhwc_gathers_staged_form_bit_exact(ops, oracle, d):
    announce("im2row/row2im nhwc staged", d)
    x, _, _, _ = case(d)
    xr = nhwc(x)
    assert np.array_equal(host(ops.im2row_nhwc(dev(xr), *d.geom())), oracle.im2row_nhwc(xr, *d.geom()))
    rng = np.random.default_rng(2)
    rmat = rng.standard_normal((d.b * d.ho * d.wo, d.c * d.kh * d.kw)).astype(np.float32)
    dx = ops.row2im_nhwc(dev(rmat), d.b, d.h, d.w, d.c, *d.geom())
    assert np.array_equal(host(dx), oracle.row2im_nhwc(rmat, d.b, d.h, d.w, d.c, *d.geom()))
    # the NCHW pair on the same geometry (its staged im2col has its own segmenting)
    assert np.array_equal(host(ops.im2col_nchw(dev(x), *d.geom())), oracle.im2col_nchw(x, *d.geom()))
    cmat = np.ascontiguousarray(rmat.T)
    dxc = ops.col2im_nchw(dev(cmat), d.b, d.c, d.h, d.w, *d.geom())
    assert np.array_equal(host(dxc), oracle.col2im_nchw(cmat, d.b, d.c, d.h, d.w, *d.geom()))


def test_im2col_unaligned_column_count(ops, oracle):
    d = D(1, 2, 7, 9, 1, 3, 3, 0, 0, 1, 1)  # P = 35: scalar-store path
    announce("im2col unaligned", d)
    x, _, _, _ = case(d)
    assert np.array_equal(host(ops.im2col_nchw(dev(x), *d.geom())), oracle.im2col_nchw(x, *d.geom()))


def test_unsupported_dtype_raises(ops):
    """float32 and float64 have kernels; anything else, and a mix of the two, is refused."""
    with pytest.raises(TypeError):
        ops.im2col_nchw(torch.zeros((1, 1, 4, 4), dtype=torch.float16, device="cuda"), 3, 3, 0, 0, 1, 1, 1, 1)
    with pytest.raises(TypeError):
        ops.matmul(torch.zeros((4, 4), dtype=torch.float32, device="cuda"),
                   torch.zeros((4, 4), dtype=torch.float64, device="cuda"))


# ------------------------------------------------------------------ GEMM

@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (7, 5, 3), (64, 64, 64), (65, 129, 17), (128, 128, 256), (130, 70, 300),
                                   (300, 40, 33), (40, 300, 1000), (64, 1000, 4096), (257, 255, 129)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sgemm_against_fp64(ops, m, n, k, ta, tb):
    announce("sgemm", m, n, k, ta, tb)
    rng = np.random.default_rng(m * 1000 + n + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    ad = dev(a.T).t() if ta else dev(a)
    bd = dev(b.T).t() if tb else dev(b)
    c = ops.matmul(ad, bd)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert_close(host(c), ref, what="sgemm vs fp64")
    assert_close(host(c), a @ b, what="sgemm vs OpenBLAS fp32")


def test_sgemm_bias_relu_epilogue_with_and_without_split(ops):
    for (m, n, k) in [(64, 96, 8192), (200, 300, 64)]:
        announce("sgemm epilogue", m, n, k)
        rng = np.random.default_rng(3)
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        c = ops.matmul(dev(a), dev(b), bias=dev(bias), relu=True)
        ref = np.maximum(a.astype(np.float64) @ b + bias, 0)
        assert_close(host(c), ref, what="sgemm+bias+relu")


def test_sgemm_rejects_bad_layout(ops):
    a = torch.zeros((8, 8), device="cuda")[:, ::2]
    with pytest.raises(ValueError):
        ops.matmul(a, torch.zeros((4, 4), device="cuda"))


# ------------------------------------------------------------------ implicit conv forward

def _fwd_ref(oracle, x, w, b, d):
    y, _ = oracle.conv2d_forward_nchw_i2c(x, w, b, oracle.ConvParams(*d.geom()))
    return y


def _kw(d):
    return dict(vpadding=d.vpadding, hpadding=d.hpadding, vstride=d.vstride, hstride=d.hstride,
                vdilation=d.vdilation, hdilation=d.hdilation)


@pytest.mark.parametrize("d", all_grid, ids=repr)
def test_conv_gemm_forward_both_formats(cg, oracle, d):
    announce("conv_gemm fwd", d)
    x, w, b, _ = case(d)
    ref = _fwd_ref(oracle, x, w, b, d)
    y = cg.conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), **_kw(d))
    assert_close(host(y), ref, what="nchw")
    y2 = cg.conv_gemm_nhwc(dev(w_nhwc(w)), dev(nhwc(x)), biases_vector=dev(b), **_kw(d))
    ref_nhwc, _ = oracle.conv2d_forward_nhwc_i2c(nhwc(x), w_nhwc(w), b, oracle.ConvParams(*d.geom()))
    assert_close(host(y2), ref_nhwc, what="nhwc")


@pytest.mark.parametrize("d", stream_grid, ids=repr)
def test_streaming_kernel_shapes_nhwc(cg, oracle, d):
    """Forward (with bias, BN and ReLU), filter gradient and input gradient of the shapes above, NHWC."""
    announce("stream shapes", d)
    assert (d.b * d.ho * d.wo) % 32 == 0 and d.b * d.ho * d.wo >= 32768
    x, w, b, dy = case(d)
    rng = np.random.default_rng(9)
    bn = [rng.uniform(0.5, 1.5, d.kn).astype(np.float32) for _ in range(4)]
    xr, wr, dyr = nhwc(x), w_nhwc(w), nhwc(dy)
    p = oracle.ConvParams(*d.geom())
    y_ref, rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, b, p)
    xd = dev(xr)
    y = cg.conv_gemm_nhwc(dev(wr), xd, biases_vector=dev(b), **_kw(d))
    from pydtnn_amd.native import last_launch
    assert last_launch()["kind"] == "stream_nhwc", last_launch()
    assert_close(host(y), y_ref, what="y")
    # the same input again: the kernel now walks the pixel blocks from the other end (it starts where the launch
    # that last touched its input ended), and once more the first way round; not a bit may change
    for _ in range(2):
        assert torch.equal(cg.conv_gemm_nhwc(dev(wr), xd, biases_vector=dev(b), **_kw(d)), y)
    y = cg.conv_gemm_nhwc(dev(wr), dev(xr), biases_vector=dev(b), bn_running_mean=dev(bn[0]), bn_inv_std=dev(bn[1]),
                          bn_gamma=dev(bn[2]), bn_beta=dev(bn[3]), relu=True, **_kw(d))
    assert_close(host(y), oracle.fused_epilogue(y_ref, "NHWC", bn=bn, relu_flag=True), what="fused y")
    dw_ref, _, dx_ref = oracle.conv2d_backward_nhwc_i2c(dyr, rows, wr, xr.shape, p)
    dx = torch.full(xr.shape, np.nan, device="cuda")
    cg.deconv_gemm_nhwc(dev(wr), dev(dyr), dx, **_kw(d))
    assert_close(host(dx), dx_ref, what="dx")
    dw = torch.empty_like(dev(wr))
    cg.conv_gemm_nhwc(dev(dyr), dev(xr), biases=dw, trans=True, **_kw(d))
    assert_close(host(dw), dw_ref, what="dw")


# one shape per chunk count the streaming kernel is built for (1, 2 and 4 chunks of 64 channels at 1x1, 9 at 3x3)
stream_chunk_grid = [D(16, 64, 56, 56, 64, 1, 1, 0, 0, 1, 1, 1, 1), D(16, 128, 56, 56, 64, 1, 1, 0, 0, 1, 1, 1, 1),
                     D(16, 256, 56, 56, 64, 1, 1, 0, 0, 1, 1, 1, 1), D(16, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1),
                     # the form that splits 512 filters between two workgroups
                     D(13, 128, 56, 56, 512, 1, 1, 0, 0, 1, 1, 1, 1)]


@pytest.mark.parametrize("masks", ["none", "relu_mask", "residual", "gate"])
@pytest.mark.parametrize("d", stream_chunk_grid, ids=repr)
def test_streaming_kernel_walks_both_ways_with_every_store(ops, cg, oracle, d, masks):
    """A launch of the streaming kernel walks the pixel blocks forwards or backwards, the opposite way of the launch
    that last walked its input on the same stream.  Calling twice (three times) with the same tensors therefore
    runs both directions of each built (chunk count, store) instance: plain, with the ReLU mask, with the residual
    sum and ReLU, and (the input gradient as a forward launch) with the gate.  Every repetition must give the same
    bits, and they must agree with the oracle."""
    announce("stream kernel both directions", masks, d)
    x, w, b, dy = case(d)
    xr, wr, dyr = nhwc(x), w_nhwc(w), nhwc(dy)
    p = oracle.ConvParams(*d.geom())
    y_ref, rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, b, p)
    xd, wd, bd, dyd = dev(xr), dev(wr), dev(b), dev(dyr)
    rng = np.random.default_rng(4)
    if masks == "none":
        out = torch.empty(y_ref.shape, device="cuda")
        run = lambda: (cg.conv_gemm_nhwc(wd, xd, biases=out, biases_vector=bd, **_kw(d)).clone(),)
        want = (y_ref,)
    elif masks == "relu_mask":
        out, mask = torch.empty(y_ref.shape, device="cuda"), torch.empty(y_ref.shape, dtype=torch.int8, device="cuda")
        run = lambda: (cg.conv_gemm_nhwc(wd, xd, biases=out, biases_vector=bd, relu=True, relu_mask=mask,
                                         **_kw(d)).clone(), mask.clone())
        want = (np.maximum(y_ref, 0), (y_ref > 0).astype(np.int8))
    elif masks == "residual":
        res_np = rng.standard_normal(y_ref.shape).astype(np.float32)
        out, res = torch.empty(y_ref.shape, device="cuda"), dev(res_np)
        run = lambda: (cg.conv_gemm_nhwc(wd, xd, biases=out, biases_vector=bd, residual=res, relu_after_residual=True,
                                         **_kw(d)).clone(),)
        want = (np.maximum(y_ref + res_np, 0),)
    else:
        gate_np = (rng.random(xr.shape) < 0.6).astype(np.int8)
        out, gate = torch.empty(xr.shape, device="cuda"), dev(gate_np)
        run = lambda: (cg.deconv_gemm_nhwc(wd, dyd, out, gate=gate, **_kw(d)).clone(),)
        _, _, dx_ref = oracle.conv2d_backward_nhwc_i2c(dyr, rows, wr, xr.shape, p)
        want = (dx_ref * gate_np,)
    first = run()
    for rep in range(2):
        for a, ref in zip(run(), first):
            assert torch.equal(a, ref), f"repetition {rep + 1} differs from the first launch"
    for a, ref in zip(first, want):
        if ref.dtype == np.int8:
            # a value within rounding of zero may fall on either side of the mask
            assert np.mean(host(a) != ref) < 1e-4
        else:
            assert_close(host(a), ref, what=masks)


# unpadded NCHW layers with wide filter rows (AlexNet-style first layers): rows of 5 .. 12 taps, strides 1 .. 4,
# vertical dilation, filter counts on and off the 96-row tile
quad_grid = [
    D(4, 3, 35, 35, 96, 11, 11, 0, 0, 4, 4, 1, 1), D(3, 2, 30, 41, 64, 3, 5, 0, 0, 1, 1, 1, 1),
    D(2, 5, 33, 40, 130, 7, 6, 0, 0, 2, 3, 1, 1), D(2, 1, 40, 37, 20, 5, 7, 0, 0, 1, 2, 2, 1),
    D(5, 4, 29, 29, 192, 2, 8, 0, 0, 3, 1, 1, 1), D(2, 3, 31, 45, 33, 4, 9, 0, 0, 2, 2, 1, 1),
    D(3, 3, 64, 64, 96, 12, 12, 0, 0, 4, 4, 1, 1), D(2, 7, 26, 30, 257, 1, 10, 0, 0, 1, 1, 1, 1),
]


@pytest.mark.parametrize("d", quad_grid, ids=repr)
def test_wide_unpadded_filter_rows_nchw(cg, oracle, d):
    announce("wide filter rows forward", d)
    x, w, b, _ = case(d)
    ref = _fwd_ref(oracle, x, w, b, d)
    y = cg.conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), **_kw(d))
    assert_close(host(y), ref, what="y")
    y = cg.conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), relu=True, **_kw(d))
    assert_close(host(y), np.maximum(ref, 0), what="relu(y)")
    # a non-finite value in a column no window reaches must not leak in
    x2 = x.copy()
    x2[:, :, :, d.w - 1] = np.inf if (d.w - d.kw) % d.hstride != 0 else x2[:, :, :, d.w - 1]
    if np.isinf(x2).any():
        y2 = host(cg.conv_gemm_nchw(dev(w), dev(x2), biases_vector=dev(b), **_kw(d)))
        ref2 = _fwd_ref(oracle, np.where(np.isinf(x2), 0, x2).astype(np.float32), w, b, d)
        assert np.isfinite(y2).all()
        assert_close(y2, ref2, what="y with an unused non-finite column")


# NCHW first layers that take the NCHW streaming kernel (filter matrix resident in LDS, at least 32768 output
# pixels).  Unpadded, 96 filters, 3 x 11 x 11 taps: AlexNet's, then strides 2 x 3 on a non-square image whose planes
# end inside a unit of 32 pixels, then dilation 2 x 1.  Padded, 64 filters, 17 .. 32 taps (VGG's 3 x 3 x 3, with
# ragged planes, mixed padding and stride, dilation, one channel of 5 x 5) and 145 .. 160 taps (ResNet's 3 x 7 x 7).
stream_nchw_grid = [
    D(11, 3, 227, 227, 96, 11, 11, 0, 0, 4, 4, 1, 1),
    D(15, 3, 120, 131, 96, 11, 11, 0, 0, 2, 3, 1, 1),
    D(9, 3, 140, 90, 96, 11, 11, 0, 0, 2, 1, 2, 1),
    D(2, 3, 224, 224, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(20, 3, 50, 47, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(20, 3, 57, 61, 64, 3, 3, 2, 0, 1, 2, 1, 1),
    D(3, 3, 130, 130, 64, 3, 3, 2, 2, 1, 1, 2, 2),
    D(4, 1, 120, 120, 64, 5, 5, 2, 2, 1, 1, 1, 1),
    D(3, 3, 224, 224, 64, 7, 7, 3, 3, 2, 2, 1, 1),
    D(3, 2, 120, 120, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(2, 27, 130, 130, 64, 1, 1, 1, 1, 1, 1, 1, 1),   # 27 taps that are channels: padded 1 x 1
]


@pytest.mark.parametrize("d", stream_nchw_grid, ids=repr)
def test_streaming_kernel_shapes_nchw(cg, oracle, d):
    """Forward alone, with bias, with bias + BN + ReLU, and with the ReLU mask of the folded training step."""
    announce("stream shapes nchw", d)
    assert d.b * d.ho * d.wo >= 32768
    x, w, b, _ = case(d)
    rng = np.random.default_rng(10)
    bn = [rng.uniform(0.5, 1.5, d.kn).astype(np.float32) for _ in range(4)]
    ref = _fwd_ref(oracle, x, w, b, d)
    xd, wd, bd = dev(x), dev(w), dev(b)
    y = cg.conv_gemm_nchw(wd, xd, **_kw(d))
    assert_close(host(y), ref - b.reshape(1, -1, 1, 1), what="y without bias")
    y = cg.conv_gemm_nchw(wd, xd, biases_vector=bd, **_kw(d))
    assert_close(host(y), ref, what="y")
    y_bn = cg.conv_gemm_nchw(wd, xd, biases_vector=bd, bn_running_mean=dev(bn[0]), bn_inv_std=dev(bn[1]),
                             bn_gamma=dev(bn[2]), bn_beta=dev(bn[3]), relu=True, **_kw(d))
    assert_close(host(y_bn), oracle.fused_epilogue(ref, "NCHW", bn=bn, relu_flag=True), what="fused y")
    y_relu = torch.full(y.shape, np.nan, device="cuda")
    mask = torch.full(y.shape, 7, dtype=torch.int8, device="cuda")
    cg.conv_gemm_nchw(wd, xd, biases=y_relu, biases_vector=bd, relu=True, relu_mask=mask, **_kw(d))
    assert torch.equal(y_relu, torch.clamp(y, min=0)) and torch.equal(mask, (y > 0).to(torch.int8))
    # non-finite values where no window reaches (the last column at some of these strides) must not leak in
    if (d.wo - 1) * d.hstride - d.hpadding + d.hdilation * (d.kw - 1) < d.w - 1:
        x2 = x.copy()
        x2[:, :, :, d.w - 1] = np.inf
        y2 = host(cg.conv_gemm_nchw(wd, dev(x2), biases_vector=bd, **_kw(d)))
        assert np.array_equal(y2, host(y))


# NHWC first layers on the same kernel: VGG's 3 x 3 x 3 -> 64 (ragged planes, mixed padding and stride, dilation),
# ResNet's 7 x 7 x 3 -> 64 at stride 2
# and 32 filters over at most 16 taps (MNIST's 3 x 3 on one channel; 2 x 2 x 4 taps; a padded 1 x 1 on 9 channels)
stream_first_nhwc_grid = [
    D(2, 3, 224, 224, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(20, 3, 50, 47, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    D(20, 3, 57, 61, 64, 3, 3, 2, 0, 1, 2, 1, 1),
    D(3, 3, 130, 130, 64, 3, 3, 2, 2, 1, 1, 2, 2),
    D(4, 3, 224, 224, 64, 7, 7, 3, 3, 2, 2, 1, 1),
    D(9, 3, 131, 117, 64, 7, 7, 3, 2, 2, 2, 1, 1),
    D(64, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1, 1, 1),
    D(7, 4, 70, 81, 32, 2, 2, 1, 1, 1, 1, 1, 1),
    D(3, 9, 110, 110, 32, 1, 1, 1, 1, 1, 1, 1, 1),
]


@pytest.mark.parametrize("d", stream_first_nhwc_grid, ids=repr)
def test_streaming_kernel_first_layers_nhwc(cg, oracle, d):
    announce("stream first layers nhwc", d)
    assert d.b * d.ho * d.wo >= 32768
    x, w, b, _ = case(d)
    rng = np.random.default_rng(11)
    bn = [rng.uniform(0.5, 1.5, d.kn).astype(np.float32) for _ in range(4)]
    xr, wr = nhwc(x), w_nhwc(w)
    ref, _ = oracle.conv2d_forward_nhwc_i2c(xr, wr, b, oracle.ConvParams(*d.geom()))
    xd, wd, bd = dev(xr), dev(wr), dev(b)
    y = cg.conv_gemm_nhwc(wd, xd, **_kw(d))
    assert_close(host(y), ref - b.reshape(1, 1, 1, -1), what="y without bias")
    y = cg.conv_gemm_nhwc(wd, xd, biases_vector=bd, **_kw(d))
    assert_close(host(y), ref, what="y")
    y_bn = cg.conv_gemm_nhwc(wd, xd, biases_vector=bd, bn_running_mean=dev(bn[0]), bn_inv_std=dev(bn[1]),
                             bn_gamma=dev(bn[2]), bn_beta=dev(bn[3]), relu=True, **_kw(d))
    assert_close(host(y_bn), oracle.fused_epilogue(ref, "NHWC", bn=bn, relu_flag=True), what="fused y")
    y_relu = torch.full(y.shape, np.nan, device="cuda")
    mask = torch.full(y.shape, 7, dtype=torch.int8, device="cuda")
    cg.conv_gemm_nhwc(wd, xd, biases=y_relu, biases_vector=bd, relu=True, relu_mask=mask, **_kw(d))
    assert torch.equal(y_relu, torch.clamp(y, min=0)) and torch.equal(mask, (y > 0).to(torch.int8))


@pytest.mark.parametrize("x,w,stride", [
    (x_2x4, w_1x1, 1), (x_2x4, w_1x2, 1), (x_2x4, w_2x2, 1), (x_4x4, w_2x2, 2), (x_4x8, w_2x2, (1, 2)),
    (x_8x8, w_3x3, 3), (x_8x8, w_2x2, 1), (x_2x4_c2, w_c2_1234_4567, 1)])
def test_reference_hand_arrays_exact(cg, oracle, x, w, stride):
    """Inputs of pydtnn/tests/conv_gemm.py:81-209 and conv2d_conv_gemm.py:72-103: small integers, exact in fp32."""
    sv, sh = (stride, stride) if isinstance(stride, int) else stride
    d = D(1, x.shape[1], x.shape[2], x.shape[3], w.shape[0], w.shape[2], w.shape[3], 0, 0, sv, sh)
    announce("hand arrays", d)
    y = cg.conv_gemm_nchw(dev(w), dev(x), **_kw(d))
    assert np.array_equal(host(y), _fwd_ref(oracle, x, w, None, d))
    if x is x_2x4 and w is w_2x2:
        assert np.array_equal(host(y).ravel(), [51, 102, 204])


def test_default_D_ones(cg):
    d = D()
    announce("default D ones", d)
    y = host(cg.conv_gemm_nchw(dev(np.ones((1, 1, d.kh, d.kw), np.float32)),
                               dev(np.ones((1, 1, d.h, d.w), np.float32)), **_kw(d)))
    assert y.shape == (1, 1, 115, 93)
    assert np.all(y[0, 0, 1:-1, 1:-1] == 160) and y[0, 0, 0, 0] == 135


@pytest.mark.parametrize("i", range(10), ids=lambda i: f"alexnet{i}")
def test_alexnet_layers_forward_and_deconv(cg, oracle, i):
    """The ten layers of pydtnn/tests/common.py:77-90 (batch cut to 8 so the CPU oracle stays fast)."""
    L = alexnet_layers[i]
    d = D(8, L.c, L.h, L.w, L.kn, L.kh, L.kw, L.vpadding, L.hpadding, L.vstride, L.hstride)
    announce("alexnet", i, d)
    x, w, b, dy = case(d)
    y = cg.conv_gemm_nchw(dev(w), dev(x), **_kw(d))
    assert_close(host(y), _fwd_ref(oracle, x, w, None, d), what="fwd")
    # pydtnn/tests/conv_gemm.py:489-524: deconv_gemm vs W^T dy + col2im
    dx = torch.empty((d.b, d.c, d.h, d.w), device="cuda")
    cg.deconv_gemm_nchw(dev(w), dev(dy), dx, **_kw(d))
    res = w.reshape(d.kn, -1).T @ dy.transpose(1, 0, 2, 3).reshape(d.kn, -1)
    assert_close(host(dx), oracle.col2im_nchw(res, d.b, d.c, d.h, d.w, *d.geom()), what="deconv")


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("use_bias,use_bn,use_relu", [(1, 0, 1), (0, 1, 0), (1, 1, 1), (0, 0, 1)])
def test_fused_epilogue(cg, oracle, fmt, use_bias, use_bn, use_relu):
    d = mid_grid[1]
    announce("fused epilogue", fmt, use_bias, use_bn, use_relu)
    x, w, b, _ = case(d)
    rng = np.random.default_rng(5)
    mean = rng.normal(0, 0.1, d.kn).astype(np.float32)
    var = rng.uniform(0.5, 1.5, d.kn).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, d.kn).astype(np.float32)
    beta = rng.normal(0, 0.1, d.kn).astype(np.float32)
    inv_std = (1.0 / np.sqrt(var + np.float32(1e-5))).astype(np.float32)
    bn = (mean, inv_std, gamma, beta)
    kw = dict(_kw(d), biases_vector=dev(b) if use_bias else None, relu=bool(use_relu))
    if use_bn:
        kw.update(bn_running_mean=dev(mean), bn_inv_std=dev(inv_std), bn_gamma=dev(gamma), bn_beta=dev(beta))
    p = oracle.ConvParams(*d.geom())
    if fmt == "NCHW":
        y = cg.conv_gemm_nchw(dev(w), dev(x), **kw)
        ref, _ = oracle.conv2d_forward_nchw_i2c(x, w, b if use_bias else None, p)
    else:
        y = cg.conv_gemm_nhwc(dev(w_nhwc(w)), dev(nhwc(x)), **kw)
        ref, _ = oracle.conv2d_forward_nhwc_i2c(nhwc(x), w_nhwc(w), b if use_bias else None, p)
    ref = oracle.fused_epilogue(ref, fmt, bn=bn if use_bn else None, relu_flag=bool(use_relu))
    assert_close(host(y), ref, what="fused")
    if use_relu:
        assert host(y).min() >= 0


def test_bn_arguments_must_come_together(cg):
    d = small_grid[1]
    x, w, b, _ = case(d)
    from pydtnn_amd.native import HipError
    with pytest.raises(HipError):
        cg.conv_gemm_nchw(dev(w), dev(x), bn_running_mean=dev(b), **_kw(d))


# ------------------------------------------------------------------ implicit backward

@pytest.mark.parametrize("d", all_grid, ids=repr)
def test_conv_gemm_backward_both_formats(cg, oracle, d):
    announce("conv_gemm bwd", d)
    x, w, _, dy = case(d)
    p = oracle.ConvParams(*d.geom())
    _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
    dw_ref, _, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
    dw = torch.empty(w.shape, device="cuda")
    cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **_kw(d))
    assert_close(host(dw), dw_ref, what="dw nchw")
    dx = torch.empty(x.shape, device="cuda")
    cg.deconv_gemm_nchw(dev(w), dev(dy), dx, **_kw(d))
    assert_close(host(dx), dx_ref, what="dx nchw")
    # NHWC, mapped back with the transposes of pydtnn/tests/check_tensor_format_models.py:124-129
    dw2 = torch.empty(w_nhwc(w).shape, device="cuda")
    cg.conv_gemm_nhwc(dev(nhwc(dy)), dev(nhwc(x)), biases=dw2, trans=True, **_kw(d))
    assert_close(host(dw2).transpose(3, 0, 1, 2), dw_ref, what="dw nhwc")
    dx2 = torch.empty(nhwc(x).shape, device="cuda")
    cg.deconv_gemm_nhwc(dev(w_nhwc(w)), dev(nhwc(dy)), dx2, **_kw(d))
    assert_close(host(dx2).transpose(0, 3, 1, 2), dx_ref, what="dx nhwc")


def test_dw_split_over_several_images_and_chunks(cg, oracle):
    """Small spatial extent (several images per reduction group) and large one (several chunks per image)."""
    for d in [D(40, 6, 7, 7, 10, 3, 3, 1, 1, 1, 1), D(2, 3, 90, 90, 5, 3, 3, 1, 1, 1, 1)]:
        announce("dw split", d)
        x, w, _, dy = case(d)
        p = oracle.ConvParams(*d.geom())
        _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
        dw_ref, _, _ = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p, need_dx=False)
        dw = torch.empty(w.shape, device="cuda")
        cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **_kw(d))
        assert_close(host(dw), dw_ref, what="dw nchw")
        dw2 = torch.empty(w_nhwc(w).shape, device="cuda")
        cg.conv_gemm_nhwc(dev(nhwc(dy)), dev(nhwc(x)), biases=dw2, trans=True, **_kw(d))
        assert_close(host(dw2).transpose(3, 0, 1, 2), dw_ref, what="dw nhwc")


def test_dw_of_narrow_filter_sets_takes_the_192_long_tiles(cg, oracle):
    """At most 64 filters and kh*kw*c = 576 or 1152: three (six) 192-long tiles instead of 256-long ones, in both
    formats; ragged filter counts, strides, padding and a split over several images included."""
    for d in [D(3, 64, 9, 11, 64, 3, 3, 1, 1, 1, 1), D(5, 64, 12, 12, 40, 3, 3, 1, 1, 2, 2),
              D(2, 128, 7, 9, 64, 3, 3, 0, 1, 1, 1), D(20, 64, 6, 6, 33, 3, 3, 1, 1, 1, 1),
              D(2, 16, 20, 20, 64, 6, 6, 2, 2, 1, 1)]:
        announce("dw 192", d)
        x, w, _, dy = case(d)
        p = oracle.ConvParams(*d.geom())
        _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
        dw_ref, _, _ = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p, need_dx=False)
        dw = torch.full(w.shape, float("nan"), device="cuda")
        cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **_kw(d))
        assert_close(host(dw), dw_ref, what="dw nchw, 192-long tiles")
        dw2 = torch.full(w_nhwc(w).shape, float("nan"), device="cuda")
        cg.conv_gemm_nhwc(dev(nhwc(dy)), dev(nhwc(x)), biases=dw2, trans=True, **_kw(d))
        assert_close(host(dw2).transpose(3, 0, 1, 2), dw_ref, what="dw nhwc, 192-long tiles")


def test_dw_of_wide_filter_sets_takes_the_256x128_tiles(cg, oracle):
    """A multiple of 256 filters (NCHW) / kh*kw*c a multiple of 256 and a multiple of 128 filters (NHWC), filter
    matrix at least 1152 long: 256x128 tiles, reduction split for 512 workgroups; a shape that qualifies in one
    format only, a stride, and a split that spans images included."""
    for d in [D(3, 128, 9, 9, 256, 3, 3, 1, 1, 1, 1), D(2, 256, 8, 10, 128, 3, 3, 1, 1, 1, 1),
              D(12, 256, 6, 6, 256, 3, 3, 1, 1, 2, 2), D(2, 72, 12, 12, 512, 4, 4, 1, 1, 1, 1),
              # a multiple of 128 filters and kh*kw*c a multiple of 192: the 128x192 / 192x128 tiles
              D(3, 128, 10, 9, 128, 3, 3, 1, 1, 1, 1), D(2, 128, 7, 7, 384, 3, 3, 1, 1, 1, 1),
              D(9, 192, 6, 6, 128, 3, 3, 0, 0, 1, 1)]:
        announce("dw 256x128", d)
        x, w, _, dy = case(d)
        p = oracle.ConvParams(*d.geom())
        _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
        dw_ref, _, _ = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p, need_dx=False)
        dw = torch.full(w.shape, float("nan"), device="cuda")
        cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **_kw(d))
        assert_close(host(dw), dw_ref, what="dw nchw, 256x128 tiles")
        dw2 = torch.full(w_nhwc(w).shape, float("nan"), device="cuda")
        cg.conv_gemm_nhwc(dev(nhwc(dy)), dev(nhwc(x)), biases=dw2, trans=True, **_kw(d))
        assert_close(host(dw2).transpose(3, 0, 1, 2), dw_ref, what="dw nhwc, 256x128 tiles")


def test_dw_with_many_tiles_takes_the_balanced_launch(cg, oracle):
    """448 x 4608 filter matrix = 126 tiles of 64 x 256 (a filter count that none of the longer tiles divides):
    the reduction units of all tiles are dealt evenly over the chip and pieces of a tile summed by the fixup kernel
    (NCHW); the library reports that form, and the result must not depend on it."""
    from pydtnn_amd import native
    for d in [D(4, 512, 8, 8, 448, 3, 3, 1, 1, 1, 1), D(6, 512, 14, 14, 448, 3, 3, 1, 1, 1, 1)]:
        announce("dw balanced", d)
        x, w, _, dy = case(d)
        p = oracle.ConvParams(*d.geom())
        _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
        dw_ref, _, _ = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p, need_dx=False)
        dw = torch.full(w.shape, float("nan"), device="cuda")
        cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **_kw(d))
        form = native.last_launch()
        assert form["kind"] == "balanced" and form["cut_tiles"] > 0, form
        assert_close(host(dw), dw_ref, what="dw nchw, balanced")


# ------------------------------------------------------------------ elementwise kernels

def test_chan_eltwise_matches_oracle(ops, oracle):
    rng = np.random.default_rng(7)
    for shape, fmt in [((3, 7, 5, 6), "NCHW"), ((3, 8, 4, 4), "NCHW"), ((3, 5, 6, 7), "NHWC"), ((2, 4, 4, 8), "NHWC"),
                       ((70, 64, 12, 12), "NCHW"), ((40, 9, 9, 256), "NHWC"), ((5, 33, 7, 1024), "NHWC")]:
        announce("chan_eltwise", shape, fmt)
        c = shape[1] if fmt == "NCHW" else shape[3]
        x = rng.standard_normal(shape).astype(np.float32)
        bn = [rng.standard_normal(c).astype(np.float32) for _ in range(4)]
        if fmt == "NCHW":
            y = ops.bn_inference_nchw(dev(x), *[dev(v) for v in bn], relu=True)
            ref = np.maximum(oracle.bn_inference_nchw(x, *bn), 0)
        else:
            y = ops.bn_relu_inference(dev(x.reshape(-1, c)), *[dev(v) for v in bn]).reshape(shape)
            ref = oracle.bn_inference(x.reshape(-1, c), *bn, relu=True).reshape(shape)
        # one fused multiply-add instead of two roundings in the last step: a few ulp at most
        assert_close(host(y), ref, tol=1e-6, what="bn+relu")
    x2 = rng.standard_normal((6, 10)).astype(np.float32)
    b6, b10 = rng.standard_normal(6).astype(np.float32), rng.standard_normal(10).astype(np.float32)
    assert np.array_equal(host(ops.add_nchw(dev(x2), dev(b6))), oracle.add_nchw(x2.copy(), b6))
    assert np.array_equal(host(ops.add_nhwc(dev(x2), dev(b10))), oracle.add_nhwc(x2.copy(), b10))
    acc = dev(x2)
    ops.eltw_sum(acc, dev(2 * x2))
    assert np.array_equal(host(acc), oracle.eltw_sum(x2.copy(), 2 * x2))
    # residual + bias + ReLU in one pass, both layouts (plane and row kernels) and a shape that takes neither
    for shape, channels, inner in [((6, 16, 8, 8), 16, 64), ((50, 128), 128, 1), ((7, 10), 10, 1)]:
        x3 = rng.standard_normal(shape).astype(np.float32)
        r3 = rng.standard_normal(shape).astype(np.float32)
        b3 = rng.standard_normal(channels).astype(np.float32)
        got = ops.chan_eltwise(dev(x3), channels=channels, inner=inner, residual=dev(r3), bias=dev(b3), relu=True)
        bshape = (1, channels, 1, 1) if inner > 1 else (1, channels)
        assert np.array_equal(host(got), np.maximum((x3 + r3) + b3.reshape(bshape), 0))


def test_relu_forward_backward(ops, oracle):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((5, 1001)).astype(np.float32)
    x[0, :4] = [0.0, -0.0, 1e-30, -1e-30]
    y, mask = ops.relu(dev(x))
    y_ref, m_ref = oracle.relu(x)
    assert np.array_equal(host(y), y_ref) and np.array_equal(host(mask), m_ref)
    dy = rng.standard_normal(x.shape).astype(np.float32)
    assert np.array_equal(host(ops.relu_backward(dev(dy), mask)), dy * m_ref)


def test_bias_grad(ops):
    rng = np.random.default_rng(9)
    for shape in [(3, 5, 7, 9), (64, 33, 14, 14), (1, 2, 3, 3)]:
        announce("bias_grad", shape)
        dy = rng.standard_normal(shape).astype(np.float32)
        db = ops.bias_grad(dev(dy), shape[1], shape[2] * shape[3])
        assert_close(host(db), dy.astype(np.float64).sum(axis=(0, 2, 3)), tol=1e-5, what="db nchw")
        dyr = nhwc(dy)
        db2 = ops.bias_grad(dev(dyr), shape[1], 1)
        assert_close(host(db2), dy.astype(np.float64).sum(axis=(0, 2, 3)), tol=1e-5, what="db nhwc")


@pytest.mark.parametrize("rows,channels", [(1, 4), (37, 8), (5000, 64), (70001, 64), (3000, 128), (1111, 256),
                                           (9000, 512), (300, 1024), (129, 2048), (64, 1000), (513, 12)])
def test_bias_grad_of_a_row_matrix(ops, rows, channels):
    """Row-major dy (NHWC conv, FC): widths that take the 16-byte kernel (a power of two of quads up to 1024
    channels), ones that do not, row counts that leave ragged slices, and more rows than one slice holds."""
    rng = np.random.default_rng(rows + channels)
    announce("bias_grad rows", rows, channels)
    dy = rng.standard_normal((rows, channels)).astype(np.float32)
    db = ops.bias_grad(dev(dy), channels, 1)
    assert_close(host(db), dy.astype(np.float64).sum(axis=0), tol=1e-5, what="db rows")


def test_maxpool_matches_oracle(ops, oracle):
    rng = np.random.default_rng(10)
    for (shape, k, s, p) in [((2, 3, 8, 10), 2, 2, 0), ((2, 4, 9, 9), 3, 2, 1), ((1, 2, 7, 7), 3, 1, 1),
                             ((2, 3, 9, 11), 2, 2, 0), ((1, 2, 9, 12), 3, 3, 0), ((3, 5, 14, 14), 2, 2, 0),
                             ((2, 3, 8, 12), 2, 2, 0), ((3, 5, 16, 32), 2, 2, 0)]:  # the last two: pairs of windows
        announce("maxpool", shape, k, s, p)
        x = rng.standard_normal(shape).astype(np.float32)
        x[0, 0, :2, :2] = 1.5  # ties: the first tap must win
        y, idx = ops.max_pool_2d_fwd_nchw(dev(x), k, k, p, p, s, s)
        y_ref, idx_ref = oracle.max_pool_2d_fwd_nchw(x, k, k, p, p, s, s)
        assert np.array_equal(host(y), y_ref) and np.array_equal(host(idx), idx_ref)
        dy = rng.standard_normal(y_ref.shape).astype(np.float32)
        dx = ops.max_pool_2d_bwd_nchw(dev(dy), idx, *shape, k, k, p, p, s, s)
        dx_ref = oracle.max_pool_2d_bwd_nchw(dy, idx_ref, *shape, k, k, p, p, s, s)
        assert_close(host(dx), dx_ref, tol=1e-6, what="maxpool bwd")


def test_sgd_momentum(ops, oracle):
    rng = np.random.default_rng(11)
    w, dw, v = [rng.standard_normal(1000).astype(np.float32) for _ in range(3)]
    wd, vd = dev(w), dev(v)
    ops.sgd_momentum(wd, dev(dw), vd, 0.01, 0.9, 1e-4, False)
    w_ref, v_ref = oracle.sgd_update(w.copy(), dw, v.copy(), np.float32(0.01), np.float32(0.9), np.float32(1e-4))
    assert_close(host(wd), w_ref, tol=1e-6, what="sgd w")
    assert_close(host(vd), v_ref, tol=1e-6, what="sgd v")


def test_maxpool_rectangular_windows_keep_the_reference_decode(ops, oracle):
    """kh != kw: the reference decodes the stored index as (idx // kh, idx % kw), which differs from how it
    was encoded (ii*kw + jj); the backward kernels must reproduce that, also when windows tile the plane."""
    rng = np.random.default_rng(13)
    for (shape, kh, kw, sv, sh) in [((2, 3, 8, 12), 2, 3, 2, 3), ((1, 2, 9, 8), 3, 2, 3, 2), ((1, 2, 7, 9), 2, 3, 1, 1)]:
        announce("maxpool rect", shape, kh, kw, sv, sh)
        x = rng.standard_normal(shape).astype(np.float32)
        g = (kh, kw, 0, 0, sv, sh)
        y, idx = ops.max_pool_2d_fwd_nchw(dev(x), *g)
        y_ref, idx_ref = oracle.max_pool_2d_fwd_nchw(x, *g)
        assert np.array_equal(host(y), y_ref) and np.array_equal(host(idx), idx_ref)
        dy = rng.standard_normal(y_ref.shape).astype(np.float32)
        dx = ops.max_pool_2d_bwd_nchw(dev(dy), idx, *shape, *g)
        assert_close(host(dx), oracle.max_pool_2d_bwd_nchw(dy, idx_ref, *shape, *g), tol=1e-6, what="maxpool bwd")


def test_maxpool_nhwc_matches_oracle(ops, oracle):
    rng = np.random.default_rng(12)
    for (shape, kh, kw, p, s, dil) in [((2, 8, 10, 3), 2, 2, 0, 2, 1), ((2, 9, 9, 70), 3, 3, 1, 2, 1),
                                       ((1, 7, 11, 5), 3, 2, 1, 1, 1), ((1, 9, 9, 2), 2, 2, 1, 1, 2),
                                       ((2, 8, 12, 4), 2, 3, 0, 1, 1), ((1, 8, 12, 3), 2, 3, 1, 2, 1),
                                       # windows that tile the image with c % 4 == 0: the window-owner kernel
                                       ((2, 8, 10, 8), 2, 2, 0, 2, 1), ((3, 6, 9, 12), 3, 3, 0, 3, 1),
                                       ((1, 4, 4, 256), 2, 2, 0, 2, 1), ((2, 9, 10, 8), 2, 2, 0, 2, 1)]:
        announce("maxpool nhwc", shape, kh, kw, p, s, dil)
        x = rng.standard_normal(shape).astype(np.float32)
        x[0, :2, :2, 0] = 1.5  # ties: the first tap must win
        g = (kh, kw, p, p, s, s, dil, dil)
        y, idx = ops.max_pool_2d_fwd_nhwc(dev(x), *g)
        y_ref, idx_ref = oracle.max_pool_2d_fwd_nhwc(x, *g)
        assert np.array_equal(host(y), y_ref) and np.array_equal(host(idx), idx_ref)
        dy = rng.standard_normal(y_ref.shape).astype(np.float32)
        dx = ops.max_pool_2d_bwd_nhwc(dev(dy), idx, *shape, *g)
        dx_ref = oracle.max_pool_2d_bwd_nhwc(dy, idx_ref, *shape, *g)
        assert np.array_equal(host(dx), dx_ref)


@pytest.mark.parametrize("fmt,shape", [("NCHW", (8, 6, 5, 7)), ("NCHW", (70, 3, 4, 4)), ("NHWC", (8, 5, 7, 6)),
                                       ("NHWC", (3, 9, 9, 130)), ("2D", (64, 10)), ("2D", (300, 70)), ("2D", (2, 3)),
                                       # row widths of a power of two of quads: the 16-byte reduction, one to many
                                       # row slices, ragged last slice
                                       ("NHWC", (4, 12, 12, 64)), ("NHWC", (2, 40, 41, 8)), ("NHWC", (3, 7, 7, 256)),
                                       ("2D", (513, 128)), ("2D", (40001, 4)), ("NHWC", (1, 3, 3, 1024)),
                                       # planes smaller than a workgroup: (image, pixel) pairs walked together
                                       ("NCHW", (20, 5, 3, 3)), ("NCHW", (300, 4, 7, 7)), ("NCHW", (9, 2, 15, 17))])
def test_bn_training_forward_backward(ops, oracle, fmt, shape):
    announce("bn training", (fmt, shape))
    rng = np.random.default_rng(sum(shape))
    c = shape[1] if fmt == "NCHW" else shape[-1]
    inner = shape[2] * shape[3] if fmt == "NCHW" else 1
    x = (rng.standard_normal(shape) * 2 + 1).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
    rm, rv = rng.standard_normal(c).astype(np.float32), rng.uniform(0.5, 2, c).astype(np.float32)
    y_ref, xn_ref, std_ref, rm_ref, rv_ref = oracle.bn_training_forward(x, gamma, beta, rm, rv, 0.9, 1e-5,
                                                                        tensor_format=fmt)
    rmd, rvd = dev(rm), dev(rv)
    y, xn, std = ops.bn_training_forward(dev(x), dev(gamma), dev(beta), rmd, rvd, 0.9, 1e-5, c, inner)
    assert_close(host(y), y_ref, tol=1e-5, what="bn y")
    assert_close(host(std), std_ref, tol=1e-5, what="bn std")
    assert_close(host(rmd), rm_ref, tol=1e-5, what="bn running mean")
    assert_close(host(rvd), rv_ref, tol=1e-5, what="bn running var")
    xn_in_format = host(xn).transpose(0, 2, 3, 1).reshape(-1, c) if fmt == "NCHW" else host(xn).reshape(-1, c)
    assert_close(xn_in_format, xn_ref, tol=1e-5, what="bn xn")
    # backward from the oracle's own xn / std so that only this kernel's arithmetic is compared
    xn_dev = xn_ref.reshape((shape[0], shape[2], shape[3], c)).transpose(0, 3, 1, 2) if fmt == "NCHW" \
        else xn_ref.reshape(shape)
    dgamma_ref, dbeta_ref, dx_ref = oracle.bn_training_backward(dy, xn_ref, std_ref, gamma, tensor_format=fmt)
    dgamma, dbeta, dx = ops.bn_training_backward(dev(dy), dev(np.ascontiguousarray(xn_dev)), dev(std_ref),
                                                 dev(gamma), c, inner)
    assert_close(host(dgamma), dgamma_ref, tol=1e-5, what="bn dgamma")
    assert_close(host(dbeta), dbeta_ref, tol=1e-5, what="bn dbeta")
    assert_close(host(dx), dx_ref, tol=2e-5, what="bn dx")
    assert ops.bn_training_backward(dev(dy), dev(np.ascontiguousarray(xn_dev)), dev(std_ref), dev(gamma), c, inner,
                                    need_dx=False)[2] is None


@pytest.mark.parametrize("rows,cols", [(64, 1000), (3, 7), (1, 1), (5, 300), (2, 4097)])
def test_softmax_forward_backward(ops, oracle, rows, cols):
    announce("softmax", (rows, cols))
    rng = np.random.default_rng(rows * 131 + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    y = ops.softmax(dev(x))
    y_ref = oracle.softmax_forward(x)
    assert_close(host(y), y_ref, tol=1e-6, what="softmax y")
    np.testing.assert_allclose(host(y).sum(axis=1), 1.0, rtol=1e-5)
    dx = ops.softmax_backward(dev(dy), dev(y_ref))
    assert_close(host(dx), oracle.softmax_backward(dy, y_ref), tol=1e-5, what="softmax dx")


@pytest.mark.parametrize("rows,cols", [(64, 1000), (3, 7), (1, 1), (5, 300)])
def test_categorical_cross_entropy(ops, oracle, rows, cols):
    announce("cce", (rows, cols))
    rng = np.random.default_rng(rows * 17 + cols)
    y_pred = oracle.softmax_forward(rng.standard_normal((rows, cols)).astype(np.float32) * 3)
    y_targ = np.eye(cols, dtype=np.float32)[rng.integers(0, cols, rows)]
    if rows >= 3 and cols >= 7:
        y_pred[0, :] = 0.0                     # exercises the lower clip bound
        y_targ[1, :] = 0.0                     # all equal: argmax is column 0
        y_targ[2, :] = 0.0
        y_targ[2, 3] = y_targ[2, 5] = 0.5      # tie: first maximum wins
    loss, dx = ops.categorical_cross_entropy(dev(y_pred), dev(y_targ), 2 * rows)
    loss_ref, dx_ref = oracle.categorical_cross_entropy(y_pred, y_targ, 2 * rows)
    assert abs(float(loss) - float(loss_ref)) <= 1e-5 * max(1.0, abs(float(loss_ref)))
    np.testing.assert_allclose(host(dx), dx_ref, rtol=2e-6, atol=0)


# ------------------------------------------------------------------ images of more than 2^16 pixels

@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_images_larger_than_65536_pixels(oracle, fmt):
    """300 x 300 output pixels per image: a reduction index of the filter gradient no longer fits the
    multiply-high division by the image size, so the split must keep one image per group."""
    from pydtnn_amd.conv_gemm import ConvGemm
    d = D(3, 6, 300, 300, 8, 3, 3, 1, 1, 1, 1)
    announce("large images", fmt, d)
    x, w, b, dy = case(d)
    cg = ConvGemm()
    p = oracle.ConvParams(*d.geom())
    kw = dict(vpadding=1, hpadding=1)
    if fmt == "NCHW":
        y = cg.conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), **kw)
        dw = torch.empty_like(dev(w))
        cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **kw)
        dx = torch.empty_like(dev(x))
        cg.deconv_gemm_nchw(dev(w), dev(dy), dx, **kw)
        y_ref, cols = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
        dw_ref, _, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, cols, w, x.shape, p)
    else:
        xr, wr, dyr = nhwc(x), w_nhwc(w), nhwc(dy)
        y = cg.conv_gemm_nhwc(dev(wr), dev(xr), biases_vector=dev(b), **kw)
        dw = torch.empty_like(dev(wr))
        cg.conv_gemm_nhwc(dev(dyr), dev(xr), biases=dw, trans=True, **kw)
        dx = torch.empty_like(dev(xr))
        cg.deconv_gemm_nhwc(dev(wr), dev(dyr), dx, **kw)
        y_ref, rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, b, p)
        dw_ref, _, dx_ref = oracle.conv2d_backward_nhwc_i2c(dyr, rows, wr, xr.shape, p)
    assert_close(host(y), y_ref, what="y")
    assert_close(host(dw), dw_ref, what="dw")
    assert_close(host(dx), dx_ref, what="dx")


# ------------------------------------------------------------------ batches run as groups of images

@pytest.mark.parametrize("d", [D(7, 5, 12, 11, 6, 3, 3, 1, 1, 2, 1), D(8, 4, 9, 10, 8, 3, 3, 1, 1, 1, 1)], ids=repr)
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_large_batches_run_as_image_groups(oracle, fmt, d):
    """With the per-launch tensor limit lowered, forward / dW / dX of a batch run as groups of 3 images (3, 3, 1
    or 3, 3, 2); results must equal the oracle's (dW is summed over the groups)."""
    from pydtnn_amd import native
    from pydtnn_amd.conv_gemm import ConvGemm
    announce("image groups", fmt, d)
    x, w, b, dy = case(d)
    per_image = max(d.c * d.h * d.w, d.kn * d.ho * d.wo)
    lib = native.lib()
    before = lib.pydtnn_hip_debug_set_tensor_floats_limit(3 * per_image + 1)
    try:
        cg = ConvGemm()
        p = oracle.ConvParams(*d.geom())
        kw = dict(vpadding=d.vpadding, hpadding=d.hpadding, vstride=d.vstride, hstride=d.hstride)
        if fmt == "NCHW":
            y = cg.conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), **kw)
            dw = torch.empty_like(dev(w))
            cg.conv_gemm_nchw(dev(dy), dev(x), biases=dw, trans=True, **kw)
            dx = torch.empty_like(dev(x))
            cg.deconv_gemm_nchw(dev(w), dev(dy), dx, **kw)
            y_ref, cols = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
            dw_ref, _, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, cols, w, x.shape, p)
        else:
            xr, wr, dyr = nhwc(x), w_nhwc(w), nhwc(dy)
            y = cg.conv_gemm_nhwc(dev(wr), dev(xr), biases_vector=dev(b), **kw)
            dw = torch.empty_like(dev(wr))
            cg.conv_gemm_nhwc(dev(dyr), dev(xr), biases=dw, trans=True, **kw)
            dx = torch.empty_like(dev(xr))
            cg.deconv_gemm_nhwc(dev(wr), dev(dyr), dx, **kw)
            y_ref, rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, b, p)
            dw_ref, _, dx_ref = oracle.conv2d_backward_nhwc_i2c(dyr, rows, wr, xr.shape, p)
        assert_close(host(y), y_ref, what="y")
        assert_close(host(dw), dw_ref, what="dw")
        assert_close(host(dx), dx_ref, what="dx")
    finally:
        lib.pydtnn_hip_debug_set_tensor_floats_limit(before)


# ------------------------------------------------------------------ ReLU done by the neighbouring layers' stores

fold_grid = [D(2, 16, 30, 30, 130, 3, 3, 1, 1, 1, 1, 1, 1), D(5, 8, 19, 23, 20, 5, 3, 2, 1, 2, 1, 1, 1),
             D(2, 33, 14, 14, 257, 1, 1, 0, 0, 1, 1, 1, 1), D(3, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1, 1, 1),
             D(16, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1),   # takes the balanced launch and its fixup
             # tiles whose gated / masked store runs in several batches of rows: 512 tiles of 256x128 with a long
             # reduction, and the 96-row tile of filter counts that are multiples of 96
             D(64, 256, 32, 32, 256, 3, 3, 1, 1, 1, 1, 1, 1), D(8, 16, 35, 35, 96, 3, 3, 1, 1, 1, 1, 1, 1)]


@pytest.mark.parametrize("d", fold_grid, ids=repr)
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_conv_forward_with_relu_mask_equals_conv_then_relu(ops, cg, fmt, d):
    """y and mask of the folded call are, bit for bit, what relu_fwd makes of the plain convolution's output."""
    announce("conv+relu+mask", fmt, d)
    x, w, b, _ = case(d)
    if fmt == "NCHW":
        conv, xs, ws = cg.conv_gemm_nchw, dev(x), dev(w)
    else:
        conv, xs, ws = cg.conv_gemm_nhwc, dev(nhwc(x)), dev(w_nhwc(w))
    plain = conv(ws, xs, biases_vector=dev(b), **_kw(d))
    y_ref, mask_ref = ops.relu(plain)
    mask = torch.full(plain.shape, 7, dtype=torch.int8, device="cuda")
    y = torch.empty_like(plain)
    conv(ws, xs, biases=y, biases_vector=dev(b), relu=True, relu_mask=mask, **_kw(d))
    assert torch.equal(y, y_ref)
    assert torch.equal(mask, mask_ref)
    assert 0 < int(mask.sum()) < mask.numel()


# shapes of the bottleneck's last convolution (1x1, few reduction steps, 256 filters) join the grid here
residual_grid = fold_grid + [D(4, 64, 28, 28, 256, 1, 1, 0, 0, 1, 1, 1, 1), D(2, 256, 14, 14, 64, 1, 1, 0, 0, 1, 1, 1, 1),
                             stream_grid[0], stream_grid[2], stream_grid[3]]


@pytest.mark.parametrize("d", residual_grid, ids=repr)
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("relu_after", [False, True], ids=["sum", "sum_relu"])
def test_conv_forward_with_residual_equals_conv_then_sum_then_relu(ops, cg, fmt, d, relu_after):
    """The addition block's sum (and the Relu after it) done by the convolution's store: bit for bit what
    eltw_sum and relu make of the plain fused call's output."""
    announce("conv+residual", fmt, d, relu_after)
    x, w, b, dy = case(d)
    rng = np.random.default_rng(11)
    bn = [rng.uniform(0.5, 1.5, d.kn).astype(np.float32) for _ in range(4)]
    res_np = rng.standard_normal(dy.shape).astype(np.float32)
    if fmt == "NCHW":
        conv, xs, ws, res = cg.conv_gemm_nchw, dev(x), dev(w), dev(res_np)
    else:
        conv, xs, ws, res = cg.conv_gemm_nhwc, dev(nhwc(x)), dev(w_nhwc(w)), dev(nhwc(res_np))
    epi = dict(biases_vector=dev(b), bn_running_mean=dev(bn[0]), bn_inv_std=dev(bn[1]), bn_gamma=dev(bn[2]),
               bn_beta=dev(bn[3]), **_kw(d))
    ref = conv(ws, xs, **epi)
    ops.eltw_sum(ref, res)
    if relu_after:
        ref, _ = ops.relu(ref, with_mask=False)
    y = torch.full(ref.shape, np.nan, device="cuda")
    conv(ws, xs, biases=y, residual=res, relu_after_residual=relu_after, **epi)
    assert torch.equal(y, ref)
    assert torch.equal(res, dev(res_np if fmt == "NCHW" else nhwc(res_np))), "the residual must stay untouched"


@pytest.mark.parametrize("d", fold_grid, ids=repr)
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_conv_dx_with_gate_equals_dx_then_relu_backward(ops, cg, fmt, d):
    """Both dX routes (as a forward kernel at stride 1, GEMM + col2im / row2im otherwise)."""
    announce("gated dx", fmt, d)
    x, w, _, dy = case(d)
    gate_np = (np.random.default_rng(3).random(x.shape) < 0.6).astype(np.int8)
    if fmt == "NCHW":
        deconv, ws, dys, gate = cg.deconv_gemm_nchw, dev(w), dev(dy), dev(gate_np)
    else:
        deconv, ws, dys, gate = cg.deconv_gemm_nhwc, dev(w_nhwc(w)), dev(nhwc(dy)), dev(nhwc(gate_np))
    plain = deconv(ws, dys, torch.empty(gate.shape, device="cuda"), **_kw(d))
    ref = ops.relu_backward(plain, gate)
    dx = deconv(ws, dys, torch.full(gate.shape, np.nan, device="cuda"), gate=gate, **_kw(d))
    assert torch.equal(dx, ref)


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_folded_relu_with_batches_run_as_image_groups(ops, cg, fmt):
    from pydtnn_amd import native
    d = D(7, 5, 12, 11, 6, 3, 3, 1, 1, 1, 1)
    announce("folded relu, image groups", fmt, d)
    x, w, b, dy = case(d)
    gate_np = (np.random.default_rng(4).random(x.shape) < 0.5).astype(np.int8)
    if fmt == "NCHW":
        conv, deconv, xs, ws, dys, gate = cg.conv_gemm_nchw, cg.deconv_gemm_nchw, dev(x), dev(w), dev(dy), dev(gate_np)
    else:
        conv, deconv = cg.conv_gemm_nhwc, cg.deconv_gemm_nhwc
        xs, ws, dys, gate = dev(nhwc(x)), dev(w_nhwc(w)), dev(nhwc(dy)), dev(nhwc(gate_np))
    y_ref, mask_ref = ops.relu(conv(ws, xs, biases_vector=dev(b), **_kw(d)))
    dx_ref = ops.relu_backward(deconv(ws, dys, torch.empty(gate.shape, device="cuda"), **_kw(d)), gate)
    lib = native.lib()
    before = lib.pydtnn_hip_debug_set_tensor_floats_limit(3 * max(d.c * d.h * d.w, d.kn * d.ho * d.wo) + 1)
    try:
        y, mask = torch.empty_like(y_ref), torch.empty_like(mask_ref)
        conv(ws, xs, biases=y, biases_vector=dev(b), relu=True, relu_mask=mask, **_kw(d))
        dx = deconv(ws, dys, torch.empty(gate.shape, device="cuda"), gate=gate, **_kw(d))
    finally:
        lib.pydtnn_hip_debug_set_tensor_floats_limit(before)
    assert torch.equal(y, y_ref) and torch.equal(mask, mask_ref) and torch.equal(dx, dx_ref)


def test_relu_mask_and_gate_arguments_are_checked(cg):
    d = D(2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1)
    x, w, b, dy = case(d)
    y = torch.empty((2, 4, 8, 8), device="cuda")
    good = torch.empty(y.shape, dtype=torch.int8, device="cuda")
    with pytest.raises(AssertionError):  # a mask without ReLU
        cg.conv_gemm_nchw(dev(w), dev(x), biases=y, relu_mask=good, **_kw(d))
    with pytest.raises(AssertionError):  # wrong shape
        cg.conv_gemm_nchw(dev(w), dev(x), biases=y, relu=True, relu_mask=good[:1], **_kw(d))
    with pytest.raises(AssertionError):  # wrong dtype
        cg.deconv_gemm_nchw(dev(w), dev(dy), torch.empty(x.shape, device="cuda"),
                            gate=torch.ones(x.shape, device="cuda"), **_kw(d))


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_pooling_batches_beyond_the_addressing_limit_run_as_image_groups(ops, fmt):
    """Pooling works plane by plane; with the per-launch limit lowered so that 7 images need 3 launches the
    results equal the single launch bit for bit (max and average pooling, forward, backward and gated)."""
    from pydtnn_amd import native
    n, c, h, w = 7, 5, 12, 10
    announce("pooling in image groups", fmt)
    rng = np.random.default_rng(17)
    nh = fmt == "NHWC"
    x = dev(rng.standard_normal((n, h, w, c) if nh else (n, c, h, w)).astype(np.float32))
    g = (3, 3, 1, 1, 2, 2)
    fwd, bwd = (ops.max_pool_2d_fwd_nhwc, ops.max_pool_2d_bwd_nhwc) if nh else (ops.max_pool_2d_fwd_nchw, ops.max_pool_2d_bwd_nchw)
    dims = (n, h, w, c) if nh else (n, c, h, w)

    def run():
        y, idx = fwd(x, *g)
        dy = torch.arange(y.numel(), device="cuda", dtype=torch.float32).reshape(y.shape) / 16.0
        gate = (x > 0).to(torch.int8)
        out = [y, idx, bwd(dy, idx, *dims, *g), bwd(dy, idx, *dims, *g, gate=gate)]
        ya = ops.average_pool_2d_fwd(x, nh, *g)
        out += [ya, ops.average_pool_2d_bwd(dy, nh, n, c, h, w, *g)]
        return out

    whole = run()
    lib = native.lib()
    before = lib.pydtnn_hip_debug_set_tensor_floats_limit(3 * c * h * w + 1)
    try:
        grouped = run()
    finally:
        lib.pydtnn_hip_debug_set_tensor_floats_limit(before)
    for a, b in zip(whole, grouped):
        assert torch.equal(a, b)


def test_maxpool_backward_with_gate_equals_backward_then_relu_backward(ops):
    rng = np.random.default_rng(12)
    for (shape, kh, kw, s, p) in [((2, 3, 8, 10), 2, 2, 2, 0), ((2, 4, 9, 9), 3, 3, 2, 1), ((2, 3, 9, 11), 2, 2, 2, 0),
                                  ((1, 2, 9, 12), 3, 3, 3, 0), ((3, 5, 14, 14), 2, 2, 2, 0), ((2, 3, 8, 9), 2, 3, 2, 0), ((2, 4, 8, 10), 2, 2, 2, 0),
                                  ((2, 8, 9, 12), 3, 3, 3, 0), ((1, 64, 6, 6), 2, 2, 2, 0), ((2, 3, 8, 12), 2, 2, 2, 0),
                                  ((3, 5, 16, 32), 2, 2, 2, 0)]:
        announce("gated maxpool bwd", shape, kh, kw, s, p)
        x = rng.standard_normal(shape).astype(np.float32)
        gate = dev((rng.random(shape) < 0.6).astype(np.int8))
        y, idx = ops.max_pool_2d_fwd_nchw(dev(x), kh, kw, p, p, s, s)
        dy = torch.randn(y.shape, device="cuda")
        ref = ops.relu_backward(ops.max_pool_2d_bwd_nchw(dy, idx, *shape, kh, kw, p, p, s, s), gate)
        got = ops.max_pool_2d_bwd_nchw(dy, idx, *shape, kh, kw, p, p, s, s, gate=gate)
        assert torch.equal(got, ref)
        xr = dev(nhwc(x))
        gr = gate.permute(0, 2, 3, 1).contiguous()
        n, c, h, w = shape
        y2, idx2 = ops.max_pool_2d_fwd_nhwc(xr, kh, kw, p, p, s, s)
        dy2 = dy.permute(0, 2, 3, 1).contiguous()
        ref2 = ops.relu_backward(ops.max_pool_2d_bwd_nhwc(dy2, idx2, n, h, w, c, kh, kw, p, p, s, s), gr)
        got2 = ops.max_pool_2d_bwd_nhwc(dy2, idx2, n, h, w, c, kh, kw, p, p, s, s, gate=gr)
        assert torch.equal(got2, ref2)


# ------------------------------------------------------------------ host-pointer compatibility ABI

def test_libconvgemm_compat_abi_runs_like_the_reference_shim(oracle):
    """Calls libconvGemm.so exactly the way pydtnn/backends/cpu/libs/conv_gemm.py:191-205, :299-307 does."""
    from pydtnn_amd import native
    lib = ctypes.CDLL(native.COMPAT_LIB_PATH)
    ac, bc = ctypes.POINTER(ctypes.c_float)(), ctypes.POINTER(ctypes.c_float)()
    lib.alloc_pack_buffs.restype = ctypes.c_int
    assert lib.alloc_pack_buffs(ctypes.byref(ac), ctypes.byref(bc)) == 0
    d = mid_grid[0]
    announce("compat abi", d)
    x, w, b, dy = case(d)
    y = np.empty((d.b, d.kn, d.ho, d.wo), np.float32)
    u = ctypes.c_uint
    none = ctypes.c_void_p(None)
    lib.sconvGemmNCHW(ctypes.c_char(b'N'), u(d.b), u(d.c), u(d.h), u(d.w), u(d.kn), u(d.kh), u(d.kw),
                      u(d.vpadding), u(d.hpadding), u(d.vstride), u(d.hstride), u(d.vdilation), u(d.hdilation),
                      ctypes.c_void_p(w.ctypes.data), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(y.ctypes.data),
                      ctypes.c_void_p(b.ctypes.data), none, none, none, none, ctypes.c_bool(True), ac, bc)
    ref = np.maximum(_fwd_ref(oracle, x, w, b, d), 0)
    assert_close(y, ref, what="compat fwd")
    lib.pydtnn_convgemm_last_status.restype = ctypes.c_int
    assert lib.pydtnn_convgemm_last_status() == 0
    # calls the library must refuse return, report through the status function and leave the output alone:
    # a filter that does not fit the image, a zero stride, a missing BN vector, an image beyond the addressing limit
    y[:] = 7.0
    bad_calls = [dict(kh=d.h + 5), dict(vstride=0), dict(bn=(ctypes.c_void_p(b.ctypes.data), none, none, none)),
                 dict(b=1, c=1, h=1 << 15, w=1 << 15, kn=1, kh=1, kw=1)]
    for bad in bad_calls:
        a = dict(b=d.b, c=d.c, h=d.h, w=d.w, kn=d.kn, kh=d.kh, kw=d.kw, vpadding=d.vpadding, hpadding=d.hpadding,
                 vstride=d.vstride, hstride=d.hstride, vdilation=d.vdilation, hdilation=d.hdilation)
        bn_args = bad.pop("bn", (none, none, none, none))
        a.update(bad)
        announce("compat abi, refused call", bad or "bn vectors")
        lib.sconvGemmNCHW(ctypes.c_char(b'N'), *[u(a[k]) for k in ("b", "c", "h", "w", "kn", "kh", "kw", "vpadding",
                                                                    "hpadding", "vstride", "hstride", "vdilation",
                                                                    "hdilation")],
                          ctypes.c_void_p(w.ctypes.data), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(y.ctypes.data),
                          ctypes.c_void_p(b.ctypes.data), *bn_args, ctypes.c_bool(True), ac, bc)
        assert lib.pydtnn_convgemm_last_status() in (native.PYDTNN_HIP_ERR_INVALID, native.PYDTNN_HIP_ERR_UNSUPPORTED)
        assert np.all(y == 7.0), "a refused call must not touch its output"
    dw = np.empty(w.shape, np.float32)
    lib.sconvGemmNCHW(ctypes.c_char(b'Y'), u(d.b), u(d.c), u(d.h), u(d.w), u(d.kn), u(d.kh), u(d.kw),
                      u(d.vpadding), u(d.hpadding), u(d.vstride), u(d.hstride), u(d.vdilation), u(d.hdilation),
                      ctypes.c_void_p(dy.ctypes.data), ctypes.c_void_p(x.ctypes.data),
                      ctypes.c_void_p(dw.ctypes.data), none, none, none, none, none, ctypes.c_bool(False), ac, bc)
    p = oracle.ConvParams(*d.geom())
    _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
    dw_ref, _, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
    assert_close(dw, dw_ref, what="compat dw")
    dx = np.zeros(x.shape, np.float32)
    lib.sconvGemmNCHW_back(u(d.b), u(d.c), u(d.h), u(d.w), u(d.kn), u(d.kh), u(d.kw), u(d.vstride), u(d.hstride),
                           u(d.vpadding), u(d.hpadding), u(d.vdilation), u(d.hdilation),
                           ctypes.c_void_p(w.ctypes.data), ctypes.c_void_p(dy.ctypes.data),
                           ctypes.c_void_p(dx.ctypes.data), ac, bc)
    assert_close(dx, dx_ref, what="compat dx")
    assert lib.pydtnn_convgemm_last_status() == 0       # a good call clears the status of the refused ones
    # a batch that travels as several groups of images, the last one smaller (16 MiB of the larger tensor per group)
    d3 = D(11, 32, 160, 160, 64, 3, 3, 1, 1, 1, 1, 1, 1)
    announce("compat abi, several groups", d3)
    x3, w3, b3, dy3 = case(d3)
    y3 = np.full((d3.b, d3.kn, d3.ho, d3.wo), np.nan, np.float32)
    g3 = [u(v) for v in (d3.b, d3.c, d3.h, d3.w, d3.kn, d3.kh, d3.kw)]
    lib.sconvGemmNCHW(ctypes.c_char(b'N'), *g3, u(1), u(1), u(1), u(1), u(1), u(1), ctypes.c_void_p(w3.ctypes.data),
                      ctypes.c_void_p(x3.ctypes.data), ctypes.c_void_p(y3.ctypes.data), ctypes.c_void_p(b3.ctypes.data),
                      none, none, none, none, ctypes.c_bool(False), ac, bc)
    assert lib.pydtnn_convgemm_last_status() == 0
    assert_close(y3, _fwd_ref(oracle, x3, w3, b3, d3), what="compat fwd in groups")
    dx3 = np.full(x3.shape, np.nan, np.float32)
    lib.sconvGemmNCHW_back(*g3, u(1), u(1), u(1), u(1), u(1), u(1), ctypes.c_void_p(w3.ctypes.data),
                           ctypes.c_void_p(dy3.ctypes.data), ctypes.c_void_p(dx3.ctypes.data), ac, bc)
    dw3 = np.full(w3.shape, np.nan, np.float32)
    lib.sconvGemmNCHW(ctypes.c_char(b'Y'), *g3, u(1), u(1), u(1), u(1), u(1), u(1), ctypes.c_void_p(dy3.ctypes.data),
                      ctypes.c_void_p(x3.ctypes.data), ctypes.c_void_p(dw3.ctypes.data), none, none, none, none, none,
                      ctypes.c_bool(False), ac, bc)
    p3 = oracle.ConvParams(*d3.geom())
    _, cols3 = oracle.conv2d_forward_nchw_i2c(x3, w3, None, p3)
    dw_ref3, _, dx_ref3 = oracle.conv2d_backward_nchw_i2c(dy3, cols3, w3, x3.shape, p3)
    assert_close(dx3, dx_ref3, what="compat dx in groups")
    assert_close(dw3, dw_ref3, what="compat dw, inputs streamed")
    # the NHWC entry points and the batch-normalisation arguments (pydtnn/backends/cpu/libs/conv_gemm.py:234-248,
    # :321-328), on a larger and then a smaller problem so that the library's cached device buffers are reused
    # at a different size
    vp = lambda a: ctypes.c_void_p(a.ctypes.data)
    rng = np.random.default_rng(12)
    for d2 in (mid_grid[6], small_grid[1]):
        announce("compat abi nhwc", d2)
        x2, w2, b2, dy2 = case(d2)
        xr, wr, dyr = nhwc(x2), w_nhwc(w2), nhwc(dy2)
        g = [u(v) for v in (d2.b, d2.h, d2.w, d2.c, d2.kn, d2.kh, d2.kw)]
        pads = [u(d2.vpadding), u(d2.hpadding)]
        strides = [u(d2.vstride), u(d2.hstride)]
        dils = [u(d2.vdilation), u(d2.hdilation)]
        bn = [rng.uniform(0.5, 1.5, d2.kn).astype(np.float32) for _ in range(4)]
        y2 = np.full((d2.b, d2.ho, d2.wo, d2.kn), np.nan, np.float32)
        lib.sconvGemmNHWC(ctypes.c_char(b'N'), *g, *pads, *strides, *dils, vp(wr), vp(xr), vp(y2), vp(b2), vp(bn[0]),
                          vp(bn[1]), vp(bn[2]), vp(bn[3]), ctypes.c_bool(True), ac, bc)
        p2 = oracle.ConvParams(*d2.geom())
        ref2, rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, b2, p2)
        assert_close(y2, oracle.fused_epilogue(ref2, "NHWC", bn=bn, relu_flag=True), what="compat nhwc fused fwd")
        dw2 = np.full(wr.shape, np.nan, np.float32)
        lib.sconvGemmNHWC(ctypes.c_char(b'Y'), *g, *pads, *strides, *dils, vp(dyr), vp(xr), vp(dw2), none, none, none,
                          none, none, ctypes.c_bool(False), ac, bc)
        dw_ref2, _, dx_ref2 = oracle.conv2d_backward_nhwc_i2c(dyr, rows, wr, xr.shape, p2)
        assert_close(dw2, dw_ref2, what="compat nhwc dw")
        dx2 = np.zeros(xr.shape, np.float32)
        lib.sconvGemmNHWC_back(*g, *strides, *pads, *dils, vp(wr), vp(dyr), vp(dx2), ac, bc)   # stride before padding
        assert_close(dx2, dx_ref2, what="compat nhwc dx")
    libc = ctypes.CDLL("libc.so.6")
    libc.free(ac)
    libc.free(bc)


# ------------------------------------------------------------------ two convolutions of a bottleneck in one launch
@pytest.mark.parametrize("kn2,with_bias,residual,relu_after", [(256, True, True, True), (256, False, True, False),
                                                               (128, True, False, False), (64, False, True, True)])
@pytest.mark.parametrize("d", [D(16, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1), D(34, 64, 32, 31, 64, 3, 3, 1, 1, 1, 1, 1, 1)],
                         ids=repr)
def test_fused_pair_of_bottleneck_convolutions_equals_the_two_launches(ops, cg, oracle, d, kn2, with_bias, residual,
                                                                        relu_after):
    """3x3 (64 -> 64) + BN + ReLU followed by 1x1 (64 -> kn2) + BN (+ residual, + ReLU) as one launch: bit for bit
    the result of the two launches it replaces, and within 1e-4 of the oracle's chain of separate passes
    (pydtnn/backends/cpu/layers/conv_2d_batch_normalization_relu_cpu.py:79-94, addition_block_cpu.py:34-46).  The
    second shape has an odd number of pixel blocks per compute unit and images whose rows do not align with them;
    both directions of the walk are taken (the call is repeated on the same tensors)."""
    from pydtnn_amd.native import last_launch
    announce("fused pair", d, kn2, with_bias, residual, relu_after)
    assert (d.b * d.ho * d.wo) % 32 == 0 and d.b * d.ho * d.wo >= 32768
    x, w, b, _ = case(d)
    rng = np.random.default_rng(21)
    w2 = (rng.standard_normal((64, 1, 1, kn2)) * np.sqrt(2.0 / 64)).astype(np.float32)
    b2 = rng.standard_normal(kn2).astype(np.float32)
    bn1 = [rng.uniform(0.5, 1.5, 64).astype(np.float32) for _ in range(4)]
    bn2 = [rng.uniform(0.5, 1.5, kn2).astype(np.float32) for _ in range(4)]
    xr, wr = nhwc(x), w_nhwc(w)
    res_np = rng.standard_normal((d.b, d.ho, d.wo, kn2)).astype(np.float32)
    xd, wd, w2d, res = dev(xr), dev(wr), dev(w2), dev(res_np) if residual else None
    e1 = dict(biases_vector=dev(b) if with_bias else None, bn_running_mean=dev(bn1[0]), bn_inv_std=dev(bn1[1]),
              bn_gamma=dev(bn1[2]), bn_beta=dev(bn1[3]), relu=True)
    e2 = dict(biases_vector=dev(b2) if with_bias else None, bn_running_mean=dev(bn2[0]), bn_inv_std=dev(bn2[1]),
              bn_gamma=dev(bn2[2]), bn_beta=dev(bn2[3]))
    mid = cg.conv_gemm_nhwc(wd, xd, **e1, **_kw(d))
    two = cg.conv_gemm_nhwc(w2d, mid, residual=res, relu_after_residual=relu_after, **e2)
    for rep in range(3):
        one = cg.conv_gemm_pair_nhwc(wd, xd, w2d, residual=res, relu_after_residual=relu_after, **e1, **_kw(d),
                                     **{k + "2": v for k, v in e2.items()})
        assert one is not None, "the library refused a shape it is built for"
        assert last_launch()["kind"] == "pair"
        assert torch.equal(one, two), f"fused launch differs from the two launches (repetition {rep})"
    p = oracle.ConvParams(*d.geom())
    y1, _ = oracle.conv2d_forward_nhwc_i2c(xr, wr, b if with_bias else None, p)
    y1 = oracle.fused_epilogue(y1, "NHWC", bn=bn1, relu_flag=True)
    y2, _ = oracle.conv2d_forward_nhwc_i2c(y1, w2, b2 if with_bias else None, oracle.ConvParams(1, 1))
    y2 = oracle.fused_epilogue(y2, "NHWC", bn=bn2, relu_flag=False)
    if residual:
        y2 = oracle.eltw_sum(np.ascontiguousarray(y2), res_np)
    if relu_after:
        y2, _ = oracle.relu(y2)
    assert_close(host(two), y2, what="fused pair vs oracle")
    # shapes it is not built for are declined, not computed wrongly
    assert cg.conv_gemm_pair_nhwc(wd, xd, dev(np.zeros((64, 1, 1, 320), np.float32)), **e1, **_kw(d),
                                  bn_running_mean2=dev(np.zeros(320, np.float32)), bn_inv_std2=dev(np.ones(320, np.float32)),
                                  bn_gamma2=dev(np.ones(320, np.float32)), bn_beta2=dev(np.zeros(320, np.float32))) is None

"""Pins the CPU oracle (no GPU): closed forms, adjoint identities, brute force, library routines.

Each check is chosen so that a plausible restatement mistake (swapped v/h
parameter, wrong row/col formula, transposed operand, dropped padding term,
wrong accumulation target) fails at least one of them.  Nothing here retypes
the oracle's own formula as the expectation.
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from shapes import (D, alexnet_layers, small_grid, x_2x4, x_2x4_c2, x_4x4, x_4x8, x_8x8,
                    w_1x1, w_1x2, w_2x2, w_3x3, w_c2_1234_4567)


# ------------------------------------------------------------------ helpers (independent of the oracle)

def direct_conv_nchw(x, w, d):
    """Textbook 7-loop cross-correlation in float64."""
    n, c, h, wi = x.shape
    kn = w.shape[0]
    y = np.zeros((n, kn, d.ho, d.wo), dtype=np.float64)
    for nn, k, oy, ox in itertools.product(range(n), range(kn), range(d.ho), range(d.wo)):
        acc = 0.0
        for cc, i, j in itertools.product(range(c), range(d.kh), range(d.kw)):
            iy = oy * d.vstride + i * d.vdilation - d.vpadding
            ix = ox * d.hstride + j * d.hdilation - d.hpadding
            if 0 <= iy < h and 0 <= ix < wi:
                acc += float(x[nn, cc, iy, ix]) * float(w[k, cc, i, j])
        y[nn, k, oy, ox] = acc
    return y


def torch_conv(x, w, d, dtype=torch.float64):
    return F.conv2d(torch.from_numpy(x).to(dtype), torch.from_numpy(w).to(dtype),
                    stride=(d.vstride, d.hstride), padding=(d.vpadding, d.hpadding),
                    dilation=(d.vdilation, d.hdilation)).numpy()


def rng_case(d, seed=0, dtype=np.float32):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(dtype)
    w = rng.standard_normal((d.kn, d.c, d.kh, d.kw)).astype(dtype)
    return x, w


# ------------------------------------------------------------------ im2col / im2row

def test_im2col_1x1_is_a_transpose(oracle):
    x = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    cols = oracle.im2col_nchw(x, 1, 1, 0, 0, 1, 1, 1, 1)
    assert np.array_equal(cols, x.transpose(1, 0, 2, 3).reshape(3, -1))
    rows = oracle.im2row_nhwc(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), 1, 1, 0, 0, 1, 1, 1, 1)
    assert np.array_equal(rows, x.transpose(0, 2, 3, 1).reshape(-1, 3))


def test_im2col_stride_equals_kernel_is_a_block_reshape(oracle):
    n, c, kh, kw, gh, gw = 2, 3, 2, 3, 4, 5
    x = np.arange(n * c * gh * kh * gw * kw, dtype=np.float64).reshape(n, c, gh * kh, gw * kw)
    cols = oracle.im2col_nchw(x, kh, kw, 0, 0, kh, kw, 1, 1)
    # x[n, c, gy*kh+i, gx*kw+j] -> cols[(c,i,j), (n,gy,gx)]
    expect = x.reshape(n, c, gh, kh, gw, kw).transpose(1, 3, 5, 0, 2, 4).reshape(c * kh * kw, n * gh * gw)
    assert np.array_equal(cols, expect)


@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_im2col_arange_entries_are_their_own_source_address(oracle, d):
    """With x = 1 + flat index, every non-padding entry of cols names the element it came from."""
    x = (1 + np.arange(d.b * d.c * d.h * d.w, dtype=np.float64)).reshape(d.b, d.c, d.h, d.w)
    cols = oracle.im2col_nchw(x, *d.geom())
    assert cols.shape == (d.c * d.kh * d.kw, d.b * d.ho * d.wo)
    for row in range(cols.shape[0]):
        cc, rem = divmod(row, d.kh * d.kw)
        i, j = divmod(rem, d.kw)
        for col in range(cols.shape[1]):
            nn, rem2 = divmod(col, d.ho * d.wo)
            oy, ox = divmod(rem2, d.wo)
            iy = oy * d.vstride + i * d.vdilation - d.vpadding
            ix = ox * d.hstride + j * d.hdilation - d.hpadding
            inside = 0 <= iy < d.h and 0 <= ix < d.w
            expect = 1 + ((nn * d.c + cc) * d.h + iy) * d.w + ix if inside else 0
            assert cols[row, col] == expect, (row, col)


@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_im2row_nhwc_is_im2col_nchw_transposed(oracle, d):
    """Same gather in the other layout: rows == cols.T once x is permuted (channel-major K in both)."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(np.float32)
    cols = oracle.im2col_nchw(x, *d.geom())
    rows = oracle.im2row_nhwc(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), *d.geom())
    assert np.array_equal(rows, cols.T)


def test_im2col_ones_gives_padding_mask(oracle):
    d = D(1, 1, 6, 5, 1, 3, 3, 1, 1, 1, 1, 1, 1)
    cols = oracle.im2col_nchw(np.ones((1, 1, 6, 5), np.float32), *d.geom())
    # centre tap never touches padding; corner tap (0,0) is padding on the first row and first column
    assert cols[4].sum() == 30
    tap00 = cols[0].reshape(6, 5)
    assert np.array_equal(tap00 == 0, np.add.outer(np.arange(6) == 0, np.arange(5) == 0) > 0)


def test_unsupported_dtype_raises(oracle):
    with pytest.raises(TypeError):
        oracle.im2col_nchw(np.zeros((1, 1, 3, 3), dtype=np.int32), 3, 3, 0, 0, 1, 1, 1, 1)


# ------------------------------------------------------------------ col2im / row2im

@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_col2im_is_the_adjoint_of_im2col(oracle, d):
    """<im2col(x), c> == <x, col2im(c)>, exact on small integers in float64."""
    rng = np.random.default_rng(2)
    x = rng.integers(-8, 9, (d.b, d.c, d.h, d.w)).astype(np.float64)
    cmat = rng.integers(-8, 9, (d.c * d.kh * d.kw, d.b * d.ho * d.wo)).astype(np.float64)
    lhs = np.sum(oracle.im2col_nchw(x, *d.geom()) * cmat)
    rhs = np.sum(x * oracle.col2im_nchw(cmat, d.b, d.c, d.h, d.w, *d.geom()))
    assert lhs == rhs
    xr = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    lhs = np.sum(oracle.im2row_nhwc(xr, *d.geom()) * cmat.T)
    rhs = np.sum(xr * oracle.row2im_nhwc(np.ascontiguousarray(cmat.T), d.b, d.h, d.w, d.c, *d.geom()))
    assert lhs == rhs


@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_col2im_of_ones_counts_taps(oracle, d):
    """col2im(ones)[n,c,y,x] = number of (i,j,oy,ox) whose receptive field covers (y,x)."""
    ones = np.ones((d.c * d.kh * d.kw, d.b * d.ho * d.wo), np.float64)
    got = oracle.col2im_nchw(ones, d.b, d.c, d.h, d.w, *d.geom())
    cnt_v = np.zeros(d.h)
    for oy, i in itertools.product(range(d.ho), range(d.kh)):
        iy = oy * d.vstride + i * d.vdilation - d.vpadding
        if 0 <= iy < d.h:
            cnt_v[iy] += 1
    cnt_h = np.zeros(d.w)
    for ox, j in itertools.product(range(d.wo), range(d.kw)):
        ix = ox * d.hstride + j * d.hdilation - d.hpadding
        if 0 <= ix < d.w:
            cnt_h[ix] += 1
    assert np.array_equal(got, np.broadcast_to(np.outer(cnt_v, cnt_h), got.shape))


def test_col2im_matches_conv_transpose(oracle):
    """W^T dy followed by col2im is the gradient of the convolution w.r.t. x (library routine)."""
    for d in small_grid:
        rng = np.random.default_rng(3)
        w = rng.standard_normal((d.kn, d.c, d.kh, d.kw))
        dy = rng.standard_normal((d.b, d.kn, d.ho, d.wo))
        res = w.reshape(d.kn, -1).T @ dy.transpose(1, 0, 2, 3).reshape(d.kn, -1)
        got = oracle.col2im_nchw(res, d.b, d.c, d.h, d.w, *d.geom())
        xt = torch.zeros(d.b, d.c, d.h, d.w, dtype=torch.float64, requires_grad=True)
        yt = F.conv2d(xt, torch.from_numpy(w), stride=(d.vstride, d.hstride),
                      padding=(d.vpadding, d.hpadding), dilation=(d.vdilation, d.hdilation))
        yt.backward(torch.from_numpy(dy))
        np.testing.assert_allclose(got, xt.grad.numpy(), rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ conv forward

def _fwd_nchw(oracle, x, w, d, b=None):
    y, _ = oracle.conv2d_forward_nchw_i2c(x, w, b, oracle.ConvParams(*d.geom()))
    return y


def test_known_answers_from_reference_hand_arrays(oracle):
    d = D(1, 1, 2, 4, 1, 2, 2, 0, 0)
    y = _fwd_nchw(oracle, x_2x4, w_2x2, d)
    assert y.shape == (1, 1, 1, 3)
    assert np.array_equal(y.ravel(), [51, 102, 204])  # 1+2+16+32, 2+4+32+64, 4+8+64+128
    # the bias *matrix* case of pydtnn/tests/conv_gemm.py:151-155: result + [[1024, 2048, 4196]]
    assert np.array_equal(y.ravel() + np.array([1024, 2048, 4196]), [1075, 2150, 4400])
    d2 = D(1, 2, 2, 4, 1, 2, 2, 0, 0)
    y2 = _fwd_nchw(oracle, x_2x4_c2, w_c2_1234_4567, d2)
    # column 0: 1*1+2*2+3*16+4*32 + 4*128+5*256+6*2048+7*4096
    assert y2.ravel()[0] == 1 + 4 + 48 + 128 + 512 + 1280 + 12288 + 28672


def test_committed_hand_cases(oracle, hand_cases):
    """The oracle's forward routes (NCHW and NHWC) against the committed known answers."""
    assert len(hand_cases) == 10
    for case in hand_cases:
        x, w = case["x"], case["w"]
        p = oracle.ConvParams(w.shape[2], w.shape[3], case["vpadding"], case["hpadding"], case["vstride"],
                              case["hstride"], case["vdilation"], case["hdilation"])
        zero = np.zeros(w.shape[0], np.float32)
        y, _ = oracle.conv2d_forward_nchw_i2c(x, w, zero, p)
        assert np.array_equal(y, case["y"]), case["name"]
        yh, _ = oracle.conv2d_forward_nhwc_i2c(np.ascontiguousarray(x.transpose(0, 2, 3, 1)),
                                               np.ascontiguousarray(w.transpose(1, 2, 3, 0)), zero, p)
        assert np.array_equal(yh.transpose(0, 3, 1, 2), case["y"]), case["name"]
        if "bias_matrix" in case:
            assert np.array_equal(y + case["bias_matrix"], case["y_plus_bias_matrix"])


def test_default_D_ones_interior_and_border(oracle):
    """ones(1,1,128,100) (*) ones(16x10), pad 1: 160 inside, fewer by the clipped taps at the border."""
    d = D()
    y = _fwd_nchw(oracle, np.ones((1, 1, d.h, d.w), np.float32), np.ones((1, 1, d.kh, d.kw), np.float32), d)
    assert y.shape == (1, 1, 115, 93)
    assert np.all(y[0, 0, 1:-1, 1:-1] == 160)
    assert y[0, 0, 0, 0] == 15 * 9 and y[0, 0, 0, 5] == 15 * 10 and y[0, 0, 7, 0] == 16 * 9
    assert y[0, 0, -1, -1] == 15 * 9


@pytest.mark.parametrize("x,w,stride", [
    (x_2x4, w_1x1, 1), (x_2x4, w_1x2, 1), (x_4x4, w_2x2, 2), (x_4x8, w_2x2, (1, 2)),
    (x_8x8, w_3x3, 3), (x_8x8, w_2x2, 1), (x_8x8, w_3x3, 2)])
def test_reference_fixed_arrays_against_direct_convolution(oracle, x, w, stride):
    sv, sh = (stride, stride) if isinstance(stride, int) else stride
    d = D(1, 1, x.shape[2], x.shape[3], 1, w.shape[2], w.shape[3], 1, 1, sv, sh)
    assert np.array_equal(_fwd_nchw(oracle, x, w, d), direct_conv_nchw(x, w, d))  # small integers: exact


@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_forward_against_direct_loop_and_torch_fp64(oracle, d):
    x, w = rng_case(d, dtype=np.float64)
    b = np.random.default_rng(5).standard_normal(d.kn)
    y = _fwd_nchw(oracle, x, w, d, b)
    ref = direct_conv_nchw(x, w, d) + b[None, :, None, None]
    np.testing.assert_allclose(y, ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(y, torch_conv(x, w, d) + b[None, :, None, None], rtol=1e-12, atol=1e-12)


def test_slow_grid_of_the_reference_against_torch(oracle):
    """The sweep of pydtnn/tests/conv2d_conv_gemm_slow.py:35-45, thinned to run in seconds."""
    rng = np.random.default_rng(6)
    count = 0
    for kn, b, c, h, w in itertools.product((1, 3), (1, 2), (1, 3), (8, 10), (8, 9)):
        for kh, kw, pad, stride in itertools.product((1, 2, 3), (1, 3), (0, 1, 3), (1, 2, 3)):
            d = D(b, c, h, w, kn, kh, kw, pad, pad, stride, stride)
            x = rng.standard_normal((b, c, h, w))
            wt = rng.standard_normal((kn, c, kh, kw))
            np.testing.assert_allclose(_fwd_nchw(oracle, x, wt, d), torch_conv(x, wt, d), rtol=1e-11, atol=1e-11)
            count += 1
    assert count > 800


@pytest.mark.parametrize("d", small_grid, ids=repr)
def test_nhwc_forward_equals_nchw_forward(oracle, d):
    """Mapping of pydtnn/tests/check_tensor_format_models.py:70-73: W_nchw = W_nhwc.transpose(3,0,1,2)."""
    x, w = rng_case(d, dtype=np.float64)
    b = np.random.default_rng(7).standard_normal(d.kn)
    p = oracle.ConvParams(*d.geom())
    y_nchw, _ = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
    w_nhwc = np.ascontiguousarray(w.transpose(1, 2, 3, 0))
    assert np.array_equal(w_nhwc.transpose(3, 0, 1, 2), w)
    y_nhwc, _ = oracle.conv2d_forward_nhwc_i2c(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), w_nhwc, b, p)
    np.testing.assert_allclose(y_nhwc.transpose(0, 3, 1, 2), y_nchw, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ conv backward

@pytest.mark.parametrize("d", small_grid, ids=repr)
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_backward_against_torch_autograd_fp64(oracle, d, fmt):
    x, w = rng_case(d, dtype=np.float64)
    dy = np.random.default_rng(8).standard_normal((d.b, d.kn, d.ho, d.wo))
    xt = torch.from_numpy(x).requires_grad_(True)
    wt = torch.from_numpy(w).requires_grad_(True)
    yt = F.conv2d(xt, wt, stride=(d.vstride, d.hstride), padding=(d.vpadding, d.hpadding),
                  dilation=(d.vdilation, d.hdilation))
    yt.backward(torch.from_numpy(dy))
    p = oracle.ConvParams(*d.geom())
    if fmt == "NCHW":
        _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
        dw, db, dx = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
    else:
        xr = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
        wr = np.ascontiguousarray(w.transpose(1, 2, 3, 0))
        _, x_rows = oracle.conv2d_forward_nhwc_i2c(xr, wr, None, p)
        dw, db, dx = oracle.conv2d_backward_nhwc_i2c(np.ascontiguousarray(dy.transpose(0, 2, 3, 1)),
                                                     x_rows, wr, xr.shape, p)
        dw = dw.transpose(3, 0, 1, 2)  # pydtnn/tests/check_tensor_format_models.py:124-129 (inverse map)
        dx = dx.transpose(0, 3, 1, 2)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(db, dy.sum(axis=(0, 2, 3)), rtol=1e-12, atol=1e-12)


def test_dw_finite_difference(oracle):
    d = D(2, 2, 5, 5, 2, 3, 3, 1, 1, 2, 2)
    x, w = rng_case(d, dtype=np.float64)
    dy = np.random.default_rng(9).standard_normal((d.b, d.kn, d.ho, d.wo))
    p = oracle.ConvParams(*d.geom())
    _, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, None, p)
    dw, _, _ = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
    eps = 1e-6
    for idx in [(0, 0, 0, 0), (1, 1, 2, 1), (0, 1, 1, 2)]:
        wp, wm = w.copy(), w.copy()
        wp[idx] += eps
        wm[idx] -= eps
        fd = (np.sum(_fwd_nchw(oracle, x, wp, d) * dy) - np.sum(_fwd_nchw(oracle, x, wm, d) * dy)) / (2 * eps)
        assert abs(fd - dw[idx]) < 1e-6


# ------------------------------------------------------------------ epilogues and small kernels

def test_bias_add_rows_and_columns(oracle):
    x = np.zeros((3, 4), np.float32)
    assert np.array_equal(oracle.add_nchw(x.copy(), np.array([1, 2, 3], np.float32)),
                          np.repeat([[1], [2], [3]], 4, axis=1))
    assert np.array_equal(oracle.add_nhwc(x.copy(), np.array([1, 2, 3, 4], np.float32)),
                          np.tile([1, 2, 3, 4], (3, 1)))


def test_transpose_1023(oracle):
    a = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    assert np.array_equal(oracle.transpose_1023(a), a.transpose(1, 0, 2, 3))


def test_bn_inference_special_cases_and_closed_form(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((50, 7)).astype(np.float32)
    one, zero = np.ones(7, np.float32), np.zeros(7, np.float32)
    assert np.array_equal(oracle.bn_inference(x, zero, one, one, zero), x)  # identity parameters
    mean, var = rng.standard_normal(7).astype(np.float32), rng.uniform(0.5, 1.5, 7).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, 7).astype(np.float32), rng.standard_normal(7).astype(np.float32)
    inv_std = (1.0 / np.sqrt(var + np.float32(1e-5))).astype(np.float32)
    y = oracle.bn_inference(x, mean, inv_std, gamma, beta)
    ref64 = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-5) * gamma + beta
    np.testing.assert_allclose(y, ref64, rtol=2e-6, atol=2e-6)
    # separately rounded steps, as the source states them
    assert np.array_equal(y, ((x - mean) * inv_std) * gamma + beta)
    yr = oracle.bn_inference(x, mean, inv_std, gamma, beta, relu=True)
    assert np.array_equal(yr, np.maximum(y, 0))
    x4 = rng.standard_normal((3, 7, 4, 5)).astype(np.float32)
    y4 = oracle.bn_inference_nchw(x4, mean, inv_std, gamma, beta)
    y2 = oracle.bn_inference(x4.transpose(0, 2, 3, 1).reshape(-1, 7), mean, inv_std, gamma, beta)
    assert np.array_equal(y4, y2.reshape(3, 4, 5, 7).transpose(0, 3, 1, 2))


def test_relu_mask_is_strict(oracle):
    x = np.array([-1.0, -0.0, 0.0, 1e-30, 2.0], np.float32)
    y, m = oracle.relu(x)
    assert np.array_equal(y, np.array([0, 0, 0, 1e-30, 2], np.float32)) and np.array_equal(m, [0, 0, 0, 1, 1])
    assert m.dtype == np.int8


def test_fused_epilogue_is_the_composition(oracle):
    d = small_grid[1]
    x, w = rng_case(d)
    rng = np.random.default_rng(11)
    b = rng.standard_normal(d.kn).astype(np.float32)
    bn = [rng.standard_normal(d.kn).astype(np.float32) for _ in range(4)]
    p = oracle.ConvParams(*d.geom())
    y, _ = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
    fused = oracle.fused_epilogue(y, "NCHW", bn=bn, relu_flag=True)
    mean, inv_std, gamma, beta = [v[None, :, None, None] for v in bn]
    assert np.array_equal(fused, np.maximum(((y - mean) * inv_std) * gamma + beta, 0))


def test_eltw_sum(oracle):
    a = np.arange(6, dtype=np.float32)
    assert np.array_equal(oracle.eltw_sum(a.copy(), np.ones(6, np.float32)), a + 1)


# ------------------------------------------------------------------ FC and the VGG16 tail

def test_fc_against_torch_autograd(oracle):
    rng = np.random.default_rng(12)
    x, w, b = rng.standard_normal((5, 7)), rng.standard_normal((7, 3)), rng.standard_normal(3)
    dy = rng.standard_normal((5, 3))
    xt, wt, bt = [torch.from_numpy(a).requires_grad_(True) for a in (x, w, b)]
    yt = xt @ wt + bt
    yt.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(oracle.fc_forward(x, w, b), yt.detach().numpy(), rtol=1e-13)
    dw, db, dx = oracle.fc_backward(dy, x, w)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC", "2D"])
def test_bn_training_against_torch_batch_norm_and_autograd(oracle, fmt):
    """Pins the TRAIN_MODE restatement with an independent library in fp64: torch's batch_norm in training
    mode uses the same biased variance for normalisation (its running_var is the unbiased one, so the running
    variance is checked against the closed form instead) and autograd supplies dx, dgamma, dbeta."""
    rng = np.random.default_rng(21)
    c = 5
    shape = {"NCHW": (4, c, 3, 6), "NHWC": (4, 3, 6, c), "2D": (9, c)}[fmt]
    x = rng.standard_normal(shape) * 2 + 1
    dy = rng.standard_normal(shape)
    gamma, beta = rng.uniform(0.5, 1.5, c), rng.standard_normal(c)
    rm, rv = rng.standard_normal(c), rng.uniform(0.5, 2, c)
    y, xn, std, new_rm, new_rv = oracle.bn_training_forward(x, gamma, beta, rm, rv, 0.9, 1e-5, tensor_format=fmt)
    to_nc = {"NCHW": lambda a: a, "NHWC": lambda a: a.transpose(0, 3, 1, 2), "2D": lambda a: a}[fmt]
    from_nc = {"NCHW": lambda a: a, "NHWC": lambda a: a.transpose(0, 2, 3, 1), "2D": lambda a: a}[fmt]
    xt = torch.from_numpy(np.ascontiguousarray(to_nc(x))).requires_grad_(True)
    gt, bt = torch.from_numpy(gamma).requires_grad_(True), torch.from_numpy(beta).requires_grad_(True)
    rmt = torch.from_numpy(rm.copy())
    yt = F.batch_norm(xt, rmt, torch.from_numpy(rv.copy()), gt, bt, training=True, momentum=0.1, eps=1e-5)
    np.testing.assert_allclose(y, from_nc(yt.detach().numpy()), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(new_rm, rmt.numpy(), rtol=1e-12)                 # same update rule for the mean
    x2 = np.ascontiguousarray(from_nc(to_nc(x)) if fmt != "NCHW" else x.transpose(0, 2, 3, 1)).reshape(-1, c)
    var = ((x2 - x2.mean(0)) ** 2).mean(0)
    np.testing.assert_allclose(new_rv, 0.9 * rv + 0.1 * var, rtol=1e-12)        # biased variance, closed form
    np.testing.assert_allclose(std, np.sqrt(var + 1e-5), rtol=1e-12)
    np.testing.assert_allclose(xn.mean(0), 0, atol=1e-12)
    np.testing.assert_allclose((xn ** 2).mean(0), var / (var + 1e-5), rtol=1e-10)
    yt.backward(torch.from_numpy(np.ascontiguousarray(to_nc(dy))))
    dgamma, dbeta, dx = oracle.bn_training_backward(dy, xn, std, gamma, tensor_format=fmt)
    np.testing.assert_allclose(dgamma, gt.grad.numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(dbeta, bt.grad.numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(dx, from_nc(xt.grad.numpy()), rtol=1e-9, atol=1e-10)
    assert oracle.bn_training_backward(dy, xn, std, gamma, tensor_format=fmt, need_dx=False)[2] is None


def test_softmax_cce_gradient_is_p_minus_t_over_batch(oracle):
    rng = np.random.default_rng(13)
    z = rng.standard_normal((6, 10))
    t = np.eye(10)[rng.integers(0, 10, 6)]
    y = oracle.softmax_forward(z)
    loss, dx = oracle.categorical_cross_entropy(y, t, global_batch_size=6)
    dz = oracle.softmax_backward(dx, y)
    np.testing.assert_allclose(dz, (y - t) / 6, rtol=1e-10, atol=1e-12)
    zt = torch.from_numpy(z)
    np.testing.assert_allclose(loss, F.cross_entropy(zt, torch.from_numpy(t.argmax(1))).item(), rtol=1e-12)


def test_sgd_momentum_two_steps(oracle):
    w, v = np.array([1.0]), np.array([0.0])
    w, v = oracle.sgd_update(w, np.array([2.0]), v, lr=0.1, momentum=0.9)
    assert np.allclose(w, 0.8) and np.allclose(v, 2.0)
    w, v = oracle.sgd_update(w, np.array([1.0]), v, lr=0.1, momentum=0.9)
    assert np.allclose(v, 2.8) and np.allclose(w, 0.52)


def test_maxpool_against_torch_and_tie_rule(oracle):
    rng = np.random.default_rng(14)
    x = rng.standard_normal((2, 3, 8, 10)).astype(np.float32)
    y, idx = oracle.max_pool_2d_fwd_nchw(x, 2, 2, 0, 0, 2, 2)
    xt = torch.from_numpy(x).requires_grad_(True)
    yt = F.max_pool2d(xt, 2, 2)
    assert np.array_equal(y, yt.detach().numpy())
    dy = rng.standard_normal(y.shape).astype(np.float32)
    yt.backward(torch.from_numpy(dy))
    dx = oracle.max_pool_2d_bwd_nchw(dy, idx, 2, 3, 8, 10, 2, 2, 0, 0, 2, 2)
    assert np.array_equal(dx, xt.grad.numpy())
    # all-equal window: the first tap wins (strict >)
    y1, idx1 = oracle.max_pool_2d_fwd_nchw(np.full((1, 1, 2, 2), 3.0, np.float32), 2, 2, 0, 0, 2, 2)
    assert idx1.item() == 0 and y1.item() == 3.0


def test_maxpool_nhwc_is_the_nchw_pool_in_the_other_layout(oracle):
    """The NHWC pair follows the same rules, so it must equal the (torch-pinned) NCHW pair on the transposed
    tensor, including rectangular windows, padding, dilation and the reference's idx // kh, idx % kw decode."""
    rng = np.random.default_rng(15)
    for (n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh) in [(2, 3, 8, 10, 2, 2, 0, 0, 2, 2, 1, 1),
                                                          (2, 4, 9, 9, 3, 3, 1, 1, 2, 2, 1, 1),
                                                          (1, 5, 7, 11, 3, 2, 1, 0, 1, 2, 1, 1),
                                                          (1, 2, 9, 9, 2, 2, 1, 1, 1, 1, 2, 2)]:
        x = rng.standard_normal((n, c, h, w)).astype(np.float32)
        x[0, 0, :3, :3] = 0.75
        g = (kh, kw, pv, ph, sv, sh, dv, dh)
        y, idx = oracle.max_pool_2d_fwd_nchw(x, *g)
        yh, idxh = oracle.max_pool_2d_fwd_nhwc(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), *g)
        assert np.array_equal(yh, y.transpose(0, 2, 3, 1)) and np.array_equal(idxh, idx.transpose(0, 2, 3, 1))
        dy = rng.standard_normal(y.shape).astype(np.float32)
        dx = oracle.max_pool_2d_bwd_nchw(dy, idx, n, c, h, w, *g)
        dxh = oracle.max_pool_2d_bwd_nhwc(np.ascontiguousarray(dy.transpose(0, 2, 3, 1)), idxh, n, h, w, c, *g)
        assert np.array_equal(dxh, dx.transpose(0, 2, 3, 1))


POOL_GEOMS = [  # (n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh)
    (2, 3, 8, 10, 2, 2, 0, 0, 2, 2, 1, 1),
    (2, 4, 9, 9, 3, 3, 1, 1, 2, 2, 1, 1),      # ResNet's 3x3 / stride 2 / pad 1
    (1, 5, 7, 11, 3, 2, 1, 0, 1, 2, 1, 1),     # rectangular window, padding on one axis, mixed strides
    (1, 2, 9, 9, 2, 2, 1, 1, 1, 1, 2, 2),      # dilated
    (2, 3, 12, 12, 3, 3, 1, 1, 1, 1, 1, 1),    # overlapping windows at stride 1
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("geom", POOL_GEOMS, ids=str)
def test_maxpool_padded_strided_dilated_against_torch(oracle, geom, dtype):
    """torch.nn.functional.max_pool2d pads with -inf, i.e. ignores padding taps like the reference's bound
    tests; distinct random values leave no ties, so values and gradients must agree exactly.  Square windows
    only go through backward: the reference decodes the stored index with kh where kw belongs.  In float64
    (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:46-49) the values are not representable in float32, so
    a pool that computed in float32 on the way would not reproduce them; the NHWC pair is checked against the
    NCHW one in the same dtype."""
    n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh = geom
    rng = np.random.default_rng(21)
    x = rng.permutation(n * c * h * w).astype(dtype).reshape(n, c, h, w) / dtype(7.0)
    y, idx = oracle.max_pool_2d_fwd_nchw(x, kh, kw, pv, ph, sv, sh, dv, dh)
    assert y.dtype == dtype
    xt = torch.from_numpy(x).requires_grad_(True)
    yt = F.max_pool2d(xt, (kh, kw), (sv, sh), (pv, ph), (dv, dh))
    assert np.array_equal(y, yt.detach().numpy())
    yh, idxh = oracle.max_pool_2d_fwd_nhwc(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), kh, kw, pv, ph, sv, sh, dv, dh)
    assert yh.dtype == dtype and np.array_equal(yh, y.transpose(0, 2, 3, 1))
    assert np.array_equal(idxh, idx.transpose(0, 2, 3, 1))
    if kh == kw:
        dy = rng.standard_normal(y.shape).astype(dtype)
        yt.backward(torch.from_numpy(dy))
        dx = oracle.max_pool_2d_bwd_nchw(dy, idx, n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh)
        tol = 1e-6 if dtype == np.float32 else 1e-14
        np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=tol, atol=tol)
        dxh = oracle.max_pool_2d_bwd_nhwc(np.ascontiguousarray(dy.transpose(0, 2, 3, 1)), idxh, n, h, w, c, kh, kw, pv,
                                          ph, sv, sh, dv, dh)
        assert dxh.dtype == dtype and np.array_equal(dxh, dx.transpose(0, 2, 3, 1))


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("geom", [g for g in POOL_GEOMS if g[10] == 1 and g[11] == 1] + [(2, 6, 7, 7, 0, 0, 0, 0, 1, 1, 1, 1)],
                         ids=str)
def test_average_pool_against_torch(oracle, fmt, geom):
    """avg_pool2d(count_include_pad=False) divides by the taps inside the image, as the reference does; the
    last geometry is the global pooling of a 7x7 plane (pool_shape (0, 0))."""
    n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh = geom
    rng = np.random.default_rng(22)
    x = rng.standard_normal((n, c, h, w))
    xt = torch.from_numpy(x).requires_grad_(True)
    yt = F.avg_pool2d(xt, (kh or h, kw or w), (sv, sh), (pv, ph), count_include_pad=False)
    dy = rng.standard_normal(tuple(yt.shape))
    yt.backward(torch.from_numpy(dy))
    to_fmt = (lambda a: a) if fmt == "NCHW" else (lambda a: np.ascontiguousarray(a.transpose(0, 2, 3, 1)))
    y = oracle.average_pool_2d_fwd(to_fmt(x.astype(np.float32)), fmt, kh, kw, pv, ph, sv, sh)
    dx = oracle.average_pool_2d_bwd(to_fmt(dy.astype(np.float32)), fmt, n, c, h, w, kh, kw, pv, ph, sv, sh)
    np.testing.assert_allclose(y, to_fmt(yt.detach().numpy()), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dx, to_fmt(xt.grad.numpy()), rtol=1e-5, atol=1e-6)
    # the float64 pair (the reference's modules dispatch on the dtype) against the same float64 torch result
    y64 = oracle.average_pool_2d_fwd(to_fmt(x), fmt, kh, kw, pv, ph, sv, sh)
    dx64 = oracle.average_pool_2d_bwd(to_fmt(dy), fmt, n, c, h, w, kh, kw, pv, ph, sv, sh)
    assert y64.dtype == np.float64 and dx64.dtype == np.float64
    np.testing.assert_allclose(y64, to_fmt(yt.detach().numpy()), rtol=1e-13, atol=1e-14)
    np.testing.assert_allclose(dx64, to_fmt(xt.grad.numpy()), rtol=1e-13, atol=1e-14)


def test_average_pool_closed_forms(oracle):
    # ones stay ones whatever the padding (the divisor counts inside taps only) ...
    y = oracle.average_pool_2d_fwd(np.ones((1, 2, 5, 5), np.float32), "NCHW", 3, 3, 1, 1, 2, 2)
    assert np.array_equal(y, np.ones_like(y))
    # ... and backward of ones is the sum over covering windows of 1 / (taps inside): corner of a 3x3 / pad 1 /
    # stride 1 pooling of a 3x3 image is covered by the windows at (0,0) [4 taps], (0,1), (1,0) [6] and (1,1) [9]
    dx = oracle.average_pool_2d_bwd(np.ones((1, 1, 3, 3), np.float32), "NCHW", 1, 1, 3, 3, 3, 3, 1, 1, 1, 1)
    assert abs(dx[0, 0, 0, 0] - (1 / 4 + 2 / 6 + 1 / 9)) < 1e-6


def test_sgd_decay_and_nesterov_closed_forms(oracle):
    """pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41 with every term switched on, by hand:
    v' = m v + g;  plain: w' = w - lr (d w + v');  nesterov: w' = w - lr (d w + g + m v')."""
    w0, g, v0, lr, m, d = 2.0, 0.5, 1.0, 0.1, 0.9, 0.01
    w, v = oracle.sgd_update(np.array([w0]), np.array([g]), np.array([v0]), lr=lr, momentum=m, decay=d)
    assert np.allclose(v, 1.4) and np.allclose(w, 2.0 - 0.1 * (0.02 + 1.4))
    w, v = oracle.sgd_update(np.array([w0]), np.array([g]), np.array([v0]), lr=lr, momentum=m, decay=d, nesterov=True)
    assert np.allclose(v, 1.4) and np.allclose(w, 2.0 - 0.1 * (0.02 + 0.5 + 0.9 * 1.4))
    # decay alone shrinks the weight geometrically when there is no gradient and no momentum
    w, v = oracle.sgd_update(np.array([3.0]), np.array([0.0]), np.array([0.0]), lr=0.5, momentum=0.0, decay=0.2)
    assert np.allclose(w, 3.0 * (1 - 0.5 * 0.2))


# ------------------------------------------------------------------ larger library cross-check

@pytest.mark.parametrize("layer", [0, 1, 4, 7], ids=lambda i: f"alexnet{i}")
def test_alexnet_layers_fp32_against_torch(oracle, layer):
    d = alexnet_layers[layer]
    d = D(4, d.c, d.h, d.w, d.kn, d.kh, d.kw, d.vpadding, d.hpadding, d.vstride, d.hstride)
    x, w = rng_case(d)
    y = _fwd_nchw(oracle, x, w, d)
    ref = torch_conv(x, w, d)
    assert np.max(np.abs(y - ref)) / np.max(np.abs(ref)) < 1e-5

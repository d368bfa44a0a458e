"""Operator-level Python API over the C ABI: one function per reference kernel, on GPU tensors.

Names and argument order follow the reference's Cython modules and ``utils.matmul`` so that the
layer code (``layers.py``) reads like PyDTNN's CPU backend.  Every function enqueues work on the
current HIP stream and returns freshly allocated device tensors.
"""
import torch

from . import native
from .native import check, f32, lib, ptr, stream_ptr


def _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    # pydtnn/layers/conv_2d.py:75-76
    ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
    wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
    return ho, wo


def _need_f32(*tensors):
    for t in tensors:
        if t is not None and t.dtype != torch.float32:
            # pydtnn/cython_modules/im2col_nchw_cython.pyx:49-50 raises TypeError for unsupported dtypes
            raise TypeError(f"Type '{t.dtype}' is not supported by the MI355X kernels (float32 only)")


# --------------------------------------------------------------------------- im2col family

def im2col_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:28-52"""
    _need_f32(x)
    n, c, h, w = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    cols = torch.empty((c * kh * kw, n * hh * ww), dtype=x.dtype, device=x.device)
    check(lib().pydtnn_hip_im2col_nchw(f32(x), f32(cols), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "im2col_nchw")
    return cols


def col2im_nchw(cols, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:150-173"""
    _need_f32(cols)
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    if tuple(cols.shape) != (c * kh * kw, n * hh * ww):
        raise ValueError(f"cols has shape {tuple(cols.shape)}, expected {(c * kh * kw, n * hh * ww)}")
    dx = torch.empty((n, c, h, w), dtype=cols.dtype, device=cols.device)
    check(lib().pydtnn_hip_col2im_nchw(f32(cols), f32(dx), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "col2im_nchw")
    return dx


def im2row_nhwc(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49"""
    _need_f32(x)
    n, h, w, c = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    rows = torch.empty((n * hh * ww, c * kh * kw), dtype=x.dtype, device=x.device)
    check(lib().pydtnn_hip_im2row_nhwc(f32(x), f32(rows), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "im2row_nhwc")
    return rows


def row2im_nhwc(rows, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:123-146"""
    _need_f32(rows)
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    if tuple(rows.shape) != (n * hh * ww, c * kh * kw):
        raise ValueError(f"rows has shape {tuple(rows.shape)}, expected {(n * hh * ww, c * kh * kw)}")
    dx = torch.empty((n, h, w, c), dtype=rows.dtype, device=rows.device)
    check(lib().pydtnn_hip_row2im_nhwc(f32(rows), f32(dx), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "row2im_nhwc")
    return dx


# --------------------------------------------------------------------------- GEMM

def _as_gemm_operand(t):
    """Returns (tensor, trans, ld) for a 2-D tensor that is C-contiguous or the .T view of one."""
    if t.dim() != 2:
        raise ValueError("matmul operands must be 2-D")
    if t.is_contiguous():
        return t, 0, t.shape[1]
    if t.t().is_contiguous():
        return t.t(), 1, t.shape[0]
    # pydtnn/utils/__init__.py:175-186 rejects other layouts for the BLAS route
    raise ValueError("Matrix data layout not supported by matmul().")


def matmul(a, b, c=None, bias=None, relu=False):
    """``a @ b`` (pydtnn/utils/__init__.py:148-158) with an optional fused ``+ bias`` / ReLU epilogue.

    Operands may be the ``.T`` view of a contiguous matrix, as in the reference's
    ``x_cols.T`` / ``weights.T`` call sites (conv_2d_cpu.py:454, fc_cpu.py:67,75).
    """
    _need_f32(a, b, c, bias)
    a_, ta, lda = _as_gemm_operand(a)
    b_, tb, ldb = _as_gemm_operand(b)
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise ValueError(f"matmul: shapes {tuple(a.shape)} and {tuple(b.shape)} not aligned")
    if c is None:
        c = torch.empty((m, n), dtype=a.dtype, device=a.device)
    elif tuple(c.shape) != (m, n) or not c.is_contiguous():
        raise ValueError("matmul: output must be a contiguous (m, n) matrix")
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_sgemm_workspace_bytes(m, n, k))
    check(lib().pydtnn_hip_sgemm(ta, tb, m, n, k, ptr(a_), lda, ptr(b_), ldb, ptr(c), n, f32(bias), int(relu),
                                 ws, ws_bytes, stream_ptr()), "sgemm")
    return c


# --------------------------------------------------------------------------- elementwise

def chan_eltwise(x, channels, inner, residual=None, bias=None, bn=None, relu=False, out=None):
    """y = relu?(bn?(x (+ residual) + bias)), channel = (index // inner) % channels."""
    _need_f32(x, residual, bias)
    mean = inv_std = gamma = beta = None
    if bn is not None:
        mean, inv_std, gamma, beta = bn
        _need_f32(mean, inv_std, gamma, beta)
    y = torch.empty_like(x) if out is None else out
    check(lib().pydtnn_hip_chan_eltwise(f32(x), f32(residual), f32(y), x.numel(), inner, channels, f32(bias),
                                        f32(mean), f32(inv_std), f32(gamma), f32(beta), int(relu), stream_ptr()),
          "chan_eltwise")
    return y


def add_nchw(x2d, b):
    """In place x[i, j] += b[i] (pydtnn/cython_modules/add_nchw_cython.pyx:25-41)."""
    return chan_eltwise(x2d, channels=x2d.shape[0], inner=x2d.shape[1], bias=b, out=x2d)


def add_nhwc(x2d, b):
    """In place x[i, j] += b[j] (pydtnn/cython_modules/add_nhwc_cython.pyx:25-41)."""
    return chan_eltwise(x2d, channels=x2d.shape[1], inner=1, bias=b, out=x2d)


def bn_inference(x2d, running_mean, inv_std, gamma, beta):
    """pydtnn/cython_modules/bn_inference_cython.pyx:25-41 on a (rows, C) matrix."""
    return chan_eltwise(x2d, channels=x2d.shape[-1], inner=1, bn=(running_mean, inv_std, gamma, beta))


def bn_relu_inference(x2d, running_mean, inv_std, gamma, beta):
    """pydtnn/cython_modules/bn_relu_inference_cython.pyx:25-40"""
    return chan_eltwise(x2d, channels=x2d.shape[-1], inner=1, bn=(running_mean, inv_std, gamma, beta), relu=True)


def bn_inference_nchw(x, running_mean, inv_std, gamma, beta, relu=False):
    """pydtnn/cython_modules/bn_inference_cython.pyx:88-104"""
    return chan_eltwise(x, channels=x.shape[1], inner=x.shape[2] * x.shape[3],
                        bn=(running_mean, inv_std, gamma, beta), relu=relu)


def eltw_sum(acc, x):
    """In place acc += x (pydtnn/cython_modules/eltw_sum_cython.pyx:25-36)."""
    return chan_eltwise(acc, channels=1, inner=1, residual=x, out=acc)


def _need_gate(gate, dx):
    if gate.dtype != torch.int8 or gate.shape != dx.shape or not gate.is_contiguous():
        raise TypeError("gate must be a contiguous int8 tensor shaped like dx")


def relu(x, with_mask=True):
    """pydtnn/cython_modules/relu_cython.pyx:25-39 -> (max(x, 0), int8 mask)"""
    _need_f32(x)
    y = torch.empty_like(x)
    mask = torch.empty(x.shape, dtype=torch.int8, device=x.device) if with_mask else None
    check(lib().pydtnn_hip_relu_fwd(f32(x), f32(y), ptr(mask), x.numel(), stream_ptr()), "relu_fwd")
    return y, mask


def relu_backward(dy, mask):
    """dy * mask (pydtnn/backends/cpu/activations/relu_cpu.py:38-40)"""
    _need_f32(dy)
    dx = torch.empty_like(dy)
    check(lib().pydtnn_hip_relu_bwd(f32(dy), ptr(mask), f32(dx), dy.numel(), stream_ptr()), "relu_bwd")
    return dx


def bias_grad(dy, channels, inner):
    """Sum of dy over everything but the channel axis; dy viewed as (outer, channels, inner)."""
    _need_f32(dy)
    outer = dy.numel() // (channels * inner)
    db = torch.empty((channels,), dtype=dy.dtype, device=dy.device)
    ws, ws_bytes = native.workspace(2048 * channels)
    check(lib().pydtnn_hip_bias_grad(f32(dy), f32(db), outer, channels, inner, ws, ws_bytes, stream_ptr()),
          "bias_grad")
    return db


def average_pool_2d_fwd(x, nhwc, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:25-52 / average_pool_2d_nhwc_cython.pyx:25-52"""
    _need_f32(x)
    n, c, h, w = (x.shape[0], x.shape[3], x.shape[1], x.shape[2]) if nhwc else x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, hh, ww, c) if nhwc else (n, c, hh, ww), dtype=x.dtype, device=x.device)
    check(lib().pydtnn_hip_average_pool_2d_fwd(int(nhwc), f32(x), f32(y), n, c, h, w, kh, kw, vpadding, hpadding,
                                               vstride, hstride, vdilation, hdilation, stream_ptr()), "avg_pool_fwd")
    return y


def average_pool_2d_bwd(dy, nhwc, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:135-160 / average_pool_2d_nhwc_cython.pyx:135-160"""
    _need_f32(dy)
    dx = torch.empty((n, h, w, c) if nhwc else (n, c, h, w), dtype=dy.dtype, device=dy.device)
    check(lib().pydtnn_hip_average_pool_2d_bwd(int(nhwc), f32(dy), f32(dx), n, c, h, w, kh, kw, vpadding, hpadding,
                                               vstride, hstride, vdilation, hdilation, stream_ptr()), "avg_pool_bwd")
    return dx


def max_pool_2d_fwd_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:25-52 -> (y, idx_max int32)"""
    _need_f32(x)
    n, c, h, w = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, c, hh, ww), dtype=x.dtype, device=x.device)
    idx = torch.empty((n, c, hh, ww), dtype=torch.int32, device=x.device)
    check(lib().pydtnn_hip_max_pool_2d_fwd_nchw(f32(x), f32(y), ptr(idx), n, c, h, w, kh, kw, vpadding, hpadding,
                                                vstride, hstride, vdilation, hdilation, stream_ptr()), "max_pool_fwd")
    return y, idx


def max_pool_2d_bwd_nchw(dy, idx_max, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1, gate=None):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:140-166.  ``gate``: int8 mask of a ReLU layer below
    the pooling layer; dx is stored multiplied by it (that layer's backward, relu_cpu.py:38-40)."""
    _need_f32(dy)
    dx = torch.empty((n, c, h, w), dtype=dy.dtype, device=dy.device)
    if gate is not None:
        _need_gate(gate, dx)
        check(lib().pydtnn_hip_max_pool_2d_bwd_gated(0, f32(dy), ptr(idx_max), f32(dx), ptr(gate), n, c, h, w, kh, kw,
                                                     vpadding, hpadding, vstride, hstride, vdilation, hdilation,
                                                     stream_ptr()), "max_pool_bwd_gated")
        return dx
    check(lib().pydtnn_hip_max_pool_2d_bwd_nchw(f32(dy), ptr(idx_max), f32(dx), n, c, h, w, kh, kw, vpadding,
                                                hpadding, vstride, hstride, vdilation, hdilation, stream_ptr()),
          "max_pool_bwd")
    return dx


def max_pool_2d_fwd_nhwc(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:25-52 -> (y, idx_max int32)"""
    _need_f32(x)
    n, h, w, c = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, hh, ww, c), dtype=x.dtype, device=x.device)
    idx = torch.empty((n, hh, ww, c), dtype=torch.int32, device=x.device)
    check(lib().pydtnn_hip_max_pool_2d_fwd_nhwc(f32(x), f32(y), ptr(idx), n, h, w, c, kh, kw, vpadding, hpadding,
                                                vstride, hstride, vdilation, hdilation, stream_ptr()), "max_pool_fwd")
    return y, idx


def max_pool_2d_bwd_nhwc(dy, idx_max, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1, gate=None):
    """pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:140-166; ``gate`` as in the NCHW twin."""
    _need_f32(dy)
    dx = torch.empty((n, h, w, c), dtype=dy.dtype, device=dy.device)
    if gate is not None:
        _need_gate(gate, dx)
        check(lib().pydtnn_hip_max_pool_2d_bwd_gated(1, f32(dy), ptr(idx_max), f32(dx), ptr(gate), n, c, h, w, kh, kw,
                                                     vpadding, hpadding, vstride, hstride, vdilation, hdilation,
                                                     stream_ptr()), "max_pool_bwd_gated")
        return dx
    check(lib().pydtnn_hip_max_pool_2d_bwd_nhwc(f32(dy), ptr(idx_max), f32(dx), n, h, w, c, kh, kw, vpadding,
                                                hpadding, vstride, hstride, vdilation, hdilation, stream_ptr()),
          "max_pool_bwd")
    return dx


def bn_training_forward(x, gamma, beta, running_mean, running_var, momentum, eps, channels, inner):
    """pydtnn/backends/cpu/layers/batch_normalization_cpu.py:59-82 on x viewed as (outer, channels, inner).
    Updates running_mean / running_var in place; returns (y, xn, std)."""
    _need_f32(x, gamma, beta, running_mean, running_var)
    x = x.contiguous()
    outer = x.numel() // (channels * inner)
    y, xn = torch.empty_like(x), torch.empty_like(x)
    std = torch.empty((channels,), dtype=x.dtype, device=x.device)
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_bn_training_workspace_bytes(channels))
    check(lib().pydtnn_hip_bn_training_fwd(f32(x), f32(y), f32(xn), f32(std), f32(gamma), f32(beta), f32(running_mean),
                                           f32(running_var), float(momentum), float(eps), outer, channels, inner, ws,
                                           ws_bytes, stream_ptr()), "bn_training_fwd")
    return y, xn, std


def bn_training_backward(dy, xn, std, gamma, channels, inner, need_dx=True):
    """batch_normalization_cpu.py:108-129 -> (dgamma, dbeta, dx or None)"""
    _need_f32(dy, xn, std, gamma)
    dy = dy.contiguous()
    outer = dy.numel() // (channels * inner)
    dgamma = torch.empty((channels,), dtype=dy.dtype, device=dy.device)
    dbeta = torch.empty_like(dgamma)
    dx = torch.empty_like(dy) if need_dx else None
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_bn_training_workspace_bytes(channels))
    check(lib().pydtnn_hip_bn_training_bwd(f32(dy), f32(xn), f32(std), f32(gamma), f32(dgamma), f32(dbeta), f32(dx),
                                           outer, channels, inner, ws, ws_bytes, stream_ptr()), "bn_training_bwd")
    return dgamma, dbeta, dx


def softmax(x):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:32-35 on a (batch, classes) matrix."""
    _need_f32(x)
    if x.dim() != 2:
        raise ValueError("softmax expects a (batch, classes) matrix")
    x = x.contiguous()
    y = torch.empty_like(x)
    check(lib().pydtnn_hip_softmax_fwd(f32(x), f32(y), x.shape[0], x.shape[1], stream_ptr()), "softmax_fwd")
    return y


def softmax_backward(dy, y):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:37-39"""
    _need_f32(dy, y)
    dy, y = dy.contiguous(), y.contiguous()
    dx = torch.empty_like(y)
    check(lib().pydtnn_hip_softmax_bwd(f32(dy), f32(y), f32(dx), y.shape[0], y.shape[1], stream_ptr()),
          "softmax_bwd")
    return dx


def categorical_cross_entropy(y_pred, y_targ, global_batch_size, eps=1e-8):
    """pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35.  Returns (loss as a 0-d tensor, dx)."""
    _need_f32(y_pred, y_targ)
    y_pred, y_targ = y_pred.contiguous(), y_targ.contiguous()
    rows, cols = y_pred.shape
    dx = torch.empty_like(y_targ)
    loss = torch.empty(1, dtype=torch.float32, device=y_pred.device)
    ws, ws_bytes = native.workspace(rows * 4)
    check(lib().pydtnn_hip_categorical_cross_entropy(f32(y_pred), f32(y_targ), f32(dx), f32(loss), rows, cols,
                                                     float(eps), int(global_batch_size), ws, ws_bytes,
                                                     stream_ptr()), "categorical_cross_entropy")
    return loss[0], dx


def sgd_momentum(w, dw, velocity, lr, momentum, decay=0.0, nesterov=False):
    """In place SGD step (pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41)."""
    _need_f32(w, dw, velocity)
    check(lib().pydtnn_hip_sgd_momentum(f32(w), f32(dw), f32(velocity), w.numel(), lr, momentum, decay,
                                        int(nesterov), stream_ptr()), "sgd_momentum")


# --------------------------------------------------------------------------- explicit (i2c) conv GEMMs

def _geom13(b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    return (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)


def conv_i2c_forward(nhwc, geom13, weights, mat, y, biases):
    _need_f32(weights, mat, y, biases)
    check(lib().pydtnn_hip_conv_i2c_forward(int(nhwc), *geom13, f32(weights), f32(mat), f32(y), f32(biases),
                                            stream_ptr()), "conv_i2c_forward")
    return y


def conv_i2c_dw(nhwc, geom13, dy, mat, dw):
    _need_f32(dy, mat, dw)
    ws, ws_bytes = native.conv_workspace(native.OP_DW, nhwc, geom13)
    check(lib().pydtnn_hip_conv_i2c_dw(int(nhwc), *geom13, f32(dy), f32(mat), f32(dw), ws, ws_bytes, stream_ptr()),
          "conv_i2c_dw")
    return dw


def conv_i2c_dx(nhwc, geom13, weights, dy, dx):
    _need_f32(weights, dy, dx)
    ws, ws_bytes = native.conv_workspace(native.OP_DX_I2C, nhwc, geom13)
    check(lib().pydtnn_hip_conv_i2c_dx(int(nhwc), *geom13, f32(weights), f32(dy), f32(dx), ws, ws_bytes,
                                       stream_ptr()), "conv_i2c_dx")
    return dx

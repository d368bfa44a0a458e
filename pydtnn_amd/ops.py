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
            raise TypeError(f"Type '{t.dtype}' is not supported by this kernel (float32 only)")


def _is_f64(*tensors):
    """True when the operands are float64 (the explicit route's second dtype, as in the reference's Cython
    modules); every operand must then be float64.  Any dtype other than float32 / float64 raises TypeError."""
    kinds = {t.dtype for t in tensors if t is not None}
    if kinds == {torch.float64}:
        return True
    if kinds - {torch.float32}:
        raise TypeError(f"Type(s) {sorted(str(k) for k in kinds)} not supported (float32, or float64 throughout)")
    return False




# --------------------------------------------------------------------------- im2col family

def im2col_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:28-52"""
    fn = lib().pydtnn_hip_im2col_nchw_f64 if _is_f64(x) else lib().pydtnn_hip_im2col_nchw
    n, c, h, w = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    cols = torch.empty((c * kh * kw, n * hh * ww), dtype=x.dtype, device=x.device)
    check(fn(ptr(x), ptr(cols), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "im2col_nchw")
    return cols


def col2im_nchw(cols, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:150-173"""
    fn = lib().pydtnn_hip_col2im_nchw_f64 if _is_f64(cols) else lib().pydtnn_hip_col2im_nchw
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    if tuple(cols.shape) != (c * kh * kw, n * hh * ww):
        raise ValueError(f"cols has shape {tuple(cols.shape)}, expected {(c * kh * kw, n * hh * ww)}")
    dx = torch.empty((n, c, h, w), dtype=cols.dtype, device=cols.device)
    check(fn(ptr(cols), ptr(dx), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "col2im_nchw")
    return dx


def im2row_nhwc(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49"""
    fn = lib().pydtnn_hip_im2row_nhwc_f64 if _is_f64(x) else lib().pydtnn_hip_im2row_nhwc
    n, h, w, c = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    rows = torch.empty((n * hh * ww, c * kh * kw), dtype=x.dtype, device=x.device)
    check(fn(ptr(x), ptr(rows), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                                       vdilation, hdilation, stream_ptr()), "im2row_nhwc")
    return rows


def row2im_nhwc(rows, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:123-146"""
    fn = lib().pydtnn_hip_row2im_nhwc_f64 if _is_f64(rows) else lib().pydtnn_hip_row2im_nhwc
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    if tuple(rows.shape) != (n * hh * ww, c * kh * kw):
        raise ValueError(f"rows has shape {tuple(rows.shape)}, expected {(n * hh * ww, c * kh * kw)}")
    dx = torch.empty((n, h, w, c), dtype=rows.dtype, device=rows.device)
    check(fn(ptr(rows), ptr(dx), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
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
    f64 = _is_f64(a, b, c, bias)
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
    if f64:
        ws, ws_bytes = native.workspace(lib().pydtnn_hip_dgemm_workspace_bytes(m, n, k))
        check(lib().pydtnn_hip_dgemm(ta, tb, m, n, k, ptr(a_), lda, ptr(b_), ldb, ptr(c), n, ptr(bias), int(relu),
                                     ws, ws_bytes, stream_ptr()), "dgemm")
        return c
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_sgemm_workspace_bytes(m, n, k))
    check(lib().pydtnn_hip_sgemm(ta, tb, m, n, k, ptr(a_), lda, ptr(b_), ldb, ptr(c), n, f32(bias), int(relu),
                                 ws, ws_bytes, stream_ptr()), "sgemm")
    return c


# --------------------------------------------------------------------------- elementwise

def chan_eltwise(x, channels, inner, residual=None, bias=None, bn=None, relu=False, out=None):
    """y = relu?(bn?(x (+ residual) + bias)), channel = (index // inner) % channels."""
    mean = inv_std = gamma = beta = None
    if bn is not None:
        mean, inv_std, gamma, beta = bn
    y = torch.empty_like(x) if out is None else out
    if _is_f64(x, residual, bias, mean, inv_std, gamma, beta, y):
        check(lib().pydtnn_hip_chan_eltwise_f64(ptr(x), ptr(residual), ptr(y), x.numel(), inner, channels, ptr(bias),
                                                ptr(mean), ptr(inv_std), ptr(gamma), ptr(beta), int(relu),
                                                stream_ptr()), "chan_eltwise_f64")
        return y
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
    fn = lib().pydtnn_hip_relu_fwd_f64 if _is_f64(x) else lib().pydtnn_hip_relu_fwd
    y = torch.empty_like(x)
    mask = torch.empty(x.shape, dtype=torch.int8, device=x.device) if with_mask else None
    check(fn(ptr(x), ptr(y), ptr(mask), x.numel(), stream_ptr()), "relu_fwd")
    return y, mask


def relu_backward(dy, mask):
    """dy * mask (pydtnn/backends/cpu/activations/relu_cpu.py:38-40)"""
    fn = lib().pydtnn_hip_relu_bwd_f64 if _is_f64(dy) else lib().pydtnn_hip_relu_bwd
    dx = torch.empty_like(dy)
    check(fn(ptr(dy), ptr(mask), ptr(dx), dy.numel(), stream_ptr()), "relu_bwd")
    return dx


def bias_grad(dy, channels, inner):
    """Sum of dy over everything but the channel axis; dy viewed as (outer, channels, inner)."""
    outer = dy.numel() // (channels * inner)
    db = torch.empty((channels,), dtype=dy.dtype, device=dy.device)
    if _is_f64(dy):
        check(lib().pydtnn_hip_bias_grad_f64(ptr(dy), ptr(db), outer, channels, inner, stream_ptr()), "bias_grad_f64")
        return db
    ws, ws_bytes = native.workspace(2048 * channels)
    check(lib().pydtnn_hip_bias_grad(f32(dy), f32(db), outer, channels, inner, ws, ws_bytes, stream_ptr()),
          "bias_grad")
    return db


def average_pool_2d_fwd(x, nhwc, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:25-52 / average_pool_2d_nhwc_cython.pyx:25-52"""
    fn = lib().pydtnn_hip_average_pool_2d_fwd_f64 if _is_f64(x) else lib().pydtnn_hip_average_pool_2d_fwd
    n, c, h, w = (x.shape[0], x.shape[3], x.shape[1], x.shape[2]) if nhwc else x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, hh, ww, c) if nhwc else (n, c, hh, ww), dtype=x.dtype, device=x.device)
    check(fn(int(nhwc), ptr(x), ptr(y), n, c, h, w, kh, kw, vpadding, hpadding,
                                               vstride, hstride, vdilation, hdilation, stream_ptr()), "avg_pool_fwd")
    return y


def average_pool_2d_bwd(dy, nhwc, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:135-160 / average_pool_2d_nhwc_cython.pyx:135-160"""
    fn = lib().pydtnn_hip_average_pool_2d_bwd_f64 if _is_f64(dy) else lib().pydtnn_hip_average_pool_2d_bwd
    dx = torch.empty((n, h, w, c) if nhwc else (n, c, h, w), dtype=dy.dtype, device=dy.device)
    check(fn(int(nhwc), ptr(dy), ptr(dx), n, c, h, w, kh, kw, vpadding, hpadding,
                                               vstride, hstride, vdilation, hdilation, stream_ptr()), "avg_pool_bwd")
    return dx


def _max_pool_bwd_f64(nhwc, dy, idx_max, dx, gate, n, c, h, w, *geom):
    check(lib().pydtnn_hip_max_pool_2d_bwd_f64(nhwc, ptr(dy), ptr(idx_max), ptr(dx), n, c, h, w, *geom, stream_ptr()),
          "max_pool_bwd_f64")
    if gate is not None:   # the ReLU layer below, as a pass of its own
        _need_gate(gate, dx)
        check(lib().pydtnn_hip_relu_bwd_f64(ptr(dx), ptr(gate), ptr(dx), dx.numel(), stream_ptr()), "relu_bwd_f64")
    return dx


def max_pool_2d_fwd_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:25-52 -> (y, idx_max int32)"""
    n, c, h, w = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, c, hh, ww), dtype=x.dtype, device=x.device)
    idx = torch.empty((n, c, hh, ww), dtype=torch.int32, device=x.device)
    if _is_f64(x):
        check(lib().pydtnn_hip_max_pool_2d_fwd_f64(0, ptr(x), ptr(y), ptr(idx), n, c, h, w, kh, kw, vpadding, hpadding,
                                                   vstride, hstride, vdilation, hdilation, stream_ptr()),
              "max_pool_fwd_f64")
        return y, idx
    check(lib().pydtnn_hip_max_pool_2d_fwd_nchw(f32(x), f32(y), ptr(idx), n, c, h, w, kh, kw, vpadding, hpadding,
                                                vstride, hstride, vdilation, hdilation, stream_ptr()), "max_pool_fwd")
    return y, idx


def max_pool_2d_bwd_nchw(dy, idx_max, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1, gate=None):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:140-166.  ``gate``: int8 mask of a ReLU layer below
    the pooling layer; dx is stored multiplied by it (that layer's backward, relu_cpu.py:38-40)."""
    dx = torch.empty((n, c, h, w), dtype=dy.dtype, device=dy.device)
    if _is_f64(dy):
        return _max_pool_bwd_f64(0, dy, idx_max, dx, gate, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                 vdilation, hdilation)
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
    n, h, w, c = x.shape
    hh, ww = _out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = torch.empty((n, hh, ww, c), dtype=x.dtype, device=x.device)
    idx = torch.empty((n, hh, ww, c), dtype=torch.int32, device=x.device)
    if _is_f64(x):
        check(lib().pydtnn_hip_max_pool_2d_fwd_f64(1, ptr(x), ptr(y), ptr(idx), n, c, h, w, kh, kw, vpadding, hpadding,
                                                   vstride, hstride, vdilation, hdilation, stream_ptr()),
              "max_pool_fwd_f64")
        return y, idx
    check(lib().pydtnn_hip_max_pool_2d_fwd_nhwc(f32(x), f32(y), ptr(idx), n, h, w, c, kh, kw, vpadding, hpadding,
                                                vstride, hstride, vdilation, hdilation, stream_ptr()), "max_pool_fwd")
    return y, idx


def max_pool_2d_bwd_nhwc(dy, idx_max, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1, gate=None):
    """pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:140-166; ``gate`` as in the NCHW twin."""
    dx = torch.empty((n, h, w, c), dtype=dy.dtype, device=dy.device)
    if _is_f64(dy):
        return _max_pool_bwd_f64(1, dy, idx_max, dx, gate, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                                 vdilation, hdilation)
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
    f64 = _is_f64(x, gamma, beta, running_mean, running_var)
    x = x.contiguous()
    outer = x.numel() // (channels * inner)
    y, xn = torch.empty_like(x), torch.empty_like(x)
    std = torch.empty((channels,), dtype=x.dtype, device=x.device)
    if f64:
        check(lib().pydtnn_hip_bn_training_fwd_f64(ptr(x), ptr(y), ptr(xn), ptr(std), ptr(gamma), ptr(beta),
                                                   ptr(running_mean), ptr(running_var), float(momentum), float(eps),
                                                   outer, channels, inner, stream_ptr()), "bn_training_fwd_f64")
        return y, xn, std
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_bn_training_workspace_bytes(channels))
    check(lib().pydtnn_hip_bn_training_fwd(f32(x), f32(y), f32(xn), f32(std), f32(gamma), f32(beta), f32(running_mean),
                                           f32(running_var), float(momentum), float(eps), outer, channels, inner, ws,
                                           ws_bytes, stream_ptr()), "bn_training_fwd")
    return y, xn, std


def bn_training_backward(dy, xn, std, gamma, channels, inner, need_dx=True):
    """batch_normalization_cpu.py:108-129 -> (dgamma, dbeta, dx or None)"""
    f64 = _is_f64(dy, xn, std, gamma)
    dy = dy.contiguous()
    outer = dy.numel() // (channels * inner)
    dgamma = torch.empty((channels,), dtype=dy.dtype, device=dy.device)
    dbeta = torch.empty_like(dgamma)
    dx = torch.empty_like(dy) if need_dx else None
    if f64:
        check(lib().pydtnn_hip_bn_training_bwd_f64(ptr(dy), ptr(xn), ptr(std), ptr(gamma), ptr(dgamma), ptr(dbeta),
                                                   ptr(dx), outer, channels, inner, stream_ptr()), "bn_training_bwd_f64")
        return dgamma, dbeta, dx
    ws, ws_bytes = native.workspace(lib().pydtnn_hip_bn_training_workspace_bytes(channels))
    check(lib().pydtnn_hip_bn_training_bwd(f32(dy), f32(xn), f32(std), f32(gamma), f32(dgamma), f32(dbeta), f32(dx),
                                           outer, channels, inner, ws, ws_bytes, stream_ptr()), "bn_training_bwd")
    return dgamma, dbeta, dx


def softmax(x):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:32-35 on a (batch, classes) matrix."""
    f64 = _is_f64(x)
    if x.dim() != 2:
        raise ValueError("softmax expects a (batch, classes) matrix")
    x = x.contiguous()
    y = torch.empty_like(x)
    if f64:
        check(lib().pydtnn_hip_softmax_fwd_f64(ptr(x), ptr(y), x.shape[0], x.shape[1], stream_ptr()), "softmax_fwd_f64")
        return y
    check(lib().pydtnn_hip_softmax_fwd(f32(x), f32(y), x.shape[0], x.shape[1], stream_ptr()), "softmax_fwd")
    return y


def softmax_backward(dy, y):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:37-39"""
    f64 = _is_f64(dy, y)
    dy, y = dy.contiguous(), y.contiguous()
    dx = torch.empty_like(y)
    if f64:
        check(lib().pydtnn_hip_softmax_bwd_f64(ptr(dy), ptr(y), ptr(dx), y.shape[0], y.shape[1], stream_ptr()),
              "softmax_bwd_f64")
        return dx
    check(lib().pydtnn_hip_softmax_bwd(f32(dy), f32(y), f32(dx), y.shape[0], y.shape[1], stream_ptr()),
          "softmax_bwd")
    return dx


def categorical_cross_entropy(y_pred, y_targ, global_batch_size, eps=1e-8):
    """pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35.  Returns (loss as a 0-d tensor, dx)."""
    f64 = _is_f64(y_pred, y_targ)
    y_pred, y_targ = y_pred.contiguous(), y_targ.contiguous()
    rows, cols = y_pred.shape
    dx = torch.empty_like(y_targ)
    if f64:
        loss = torch.empty(1, dtype=torch.float64, device=y_pred.device)
        ws, ws_bytes = native.workspace(rows * 8)
        check(lib().pydtnn_hip_categorical_cross_entropy_f64(ptr(y_pred), ptr(y_targ), ptr(dx), ptr(loss), rows, cols,
                                                             float(eps), int(global_batch_size), ws, ws_bytes,
                                                             stream_ptr()), "categorical_cross_entropy_f64")
        return loss[0], dx
    loss = torch.empty(1, dtype=torch.float32, device=y_pred.device)
    ws, ws_bytes = native.workspace(rows * 4)
    check(lib().pydtnn_hip_categorical_cross_entropy(f32(y_pred), f32(y_targ), f32(dx), f32(loss), rows, cols,
                                                     float(eps), int(global_batch_size), ws, ws_bytes,
                                                     stream_ptr()), "categorical_cross_entropy")
    return loss[0], dx


def sgd_momentum(w, dw, velocity, lr, momentum, decay=0.0, nesterov=False):
    """In place SGD step (pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41)."""
    if _is_f64(w, dw, velocity):
        check(lib().pydtnn_hip_sgd_momentum_f64(ptr(w), ptr(dw), ptr(velocity), w.numel(), lr, momentum, decay,
                                                int(nesterov), stream_ptr()), "sgd_momentum_f64")
        return
    check(lib().pydtnn_hip_sgd_momentum(f32(w), f32(dw), f32(velocity), w.numel(), lr, momentum, decay,
                                        int(nesterov), stream_ptr()), "sgd_momentum")


def sgd_momentum_multi(tensors, lr, momentum, decay=0.0, nesterov=False):
    """The SGD step of ``sgd_momentum`` for several (w, dw, velocity) triples in one launch (a layer's variables)."""
    import ctypes
    if len(tensors) == 1 or any(_is_f64(*t) for t in tensors):
        for w, dw, velocity in tensors:
            sgd_momentum(w, dw, velocity, lr, momentum, decay, nesterov)
        return
    n = len(tensors)
    ptrs = ctypes.c_void_p * n
    for t in tensors:
        for a in t:
            f32(a)    # float32, contiguous, on the GPU
    check(lib().pydtnn_hip_sgd_momentum_multi(
        n, ptrs(*[t[0].data_ptr() for t in tensors]), ptrs(*[t[1].data_ptr() for t in tensors]),
        ptrs(*[t[2].data_ptr() for t in tensors]), (ctypes.c_long * n)(*[t[0].numel() for t in tensors]), lr, momentum,
        decay, int(nesterov), stream_ptr()), "sgd_momentum_multi")


# --------------------------------------------------------------------------- explicit (i2c) conv GEMMs

def _geom13(b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    return (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)


def transpose_1023(src):
    """(d0, d1, h, w) -> (d1, d0, h, w) copy: pydtnn/utils/best_transpose_1023.py:50-58.  float64 only here: the
    float32 kernels store in the tensor format directly and never need the copy."""
    if not _is_f64(src):
        raise TypeError("transpose_1023 is part of the float64 route only")
    d0, d1 = src.shape[0], src.shape[1]
    inner = src.numel() // (d0 * d1)
    dst = torch.empty((d1, d0) + tuple(src.shape[2:]), dtype=src.dtype, device=src.device)
    check(lib().pydtnn_hip_transpose_1023_f64(ptr(src), ptr(dst), d0, d1, inner, stream_ptr()), "transpose_1023_f64")
    return dst


def _i2c_forward_f64(nhwc, geom13, weights, mat, y, biases):
    """The reference's own steps (conv_2d_cpu.py:183-209, :264-291): matmul, bias pass, and for NCHW the
    (co,N,ho,wo) -> (N,co,ho,wo) copy."""
    b, c, h, w, kn, kh, kw = geom13[:7]
    if nhwc:
        matmul(mat, weights.reshape(-1, kn), c=y.view(-1, kn), bias=biases)
        return y
    ho, wo = y.shape[2], y.shape[3]
    res = matmul(weights.reshape(kn, -1), mat)
    if biases is not None:
        add_nchw(res, biases)
    y.copy_(transpose_1023(res.view(kn, b, ho, wo)))
    return y


def _i2c_dw_f64(nhwc, geom13, dy, mat, dw):
    """conv_2d_cpu.py:370 (x_rows.T @ dy_rows) and :454 (dy_cols @ x_cols.T)."""
    kn = geom13[4]
    if nhwc:
        matmul(mat.t(), dy.reshape(-1, kn), c=dw.view(-1, kn))
    else:
        dy_cols = transpose_1023(dy).reshape(kn, -1)
        matmul(dy_cols, mat.t(), c=dw.view(kn, -1))
    return dw


def _i2c_dx_f64(nhwc, geom13, weights, dy, dx):
    """conv_2d_cpu.py:389-395 (dy_rows @ W.T, row2im) and :473-479 (W.T @ dy_cols, col2im)."""
    b, c, h, w, kn, kh, kw, vp, hp, vs, hs, vd, hd = geom13
    if nhwc:
        res = matmul(dy.reshape(-1, kn), weights.reshape(-1, kn).t())
        dx.copy_(row2im_nhwc(res, b, h, w, c, kh, kw, vp, hp, vs, hs, vd, hd))
    else:
        dy_cols = transpose_1023(dy).reshape(kn, -1)
        res = matmul(weights.reshape(kn, -1).t(), dy_cols)
        dx.copy_(col2im_nchw(res, b, c, h, w, kh, kw, vp, hp, vs, hs, vd, hd))
    return dx


def conv_i2c_forward(nhwc, geom13, weights, mat, y, biases):
    if _is_f64(weights, mat, y, biases):
        return _i2c_forward_f64(nhwc, geom13, weights, mat, y, biases)
    ws, ws_bytes = native.conv_workspace(native.OP_FWD_I2C, nhwc, geom13)
    check(lib().pydtnn_hip_conv_i2c_forward(int(nhwc), *geom13, f32(weights), f32(mat), f32(y), f32(biases), ws,
                                            ws_bytes, stream_ptr()), "conv_i2c_forward")
    return y


def conv_i2c_dw(nhwc, geom13, dy, mat, dw):
    if _is_f64(dy, mat, dw):
        return _i2c_dw_f64(nhwc, geom13, dy, mat, dw)
    ws, ws_bytes = native.conv_workspace(native.OP_DW, nhwc, geom13)
    check(lib().pydtnn_hip_conv_i2c_dw(int(nhwc), *geom13, f32(dy), f32(mat), f32(dw), ws, ws_bytes, stream_ptr()),
          "conv_i2c_dw")
    return dw


def conv_i2c_dx(nhwc, geom13, weights, dy, dx):
    if _is_f64(weights, dy, dx):
        return _i2c_dx_f64(nhwc, geom13, weights, dy, dx)
    ws, ws_bytes = native.conv_workspace(native.OP_DX_I2C, nhwc, geom13)
    check(lib().pydtnn_hip_conv_i2c_dx(int(nhwc), *geom13, f32(weights), f32(dy), f32(dx), ws, ws_bytes,
                                       stream_ptr()), "conv_i2c_dx")
    return dx

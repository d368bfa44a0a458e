"""CPU oracle (TEST INFRASTRUCTURE ONLY): NumPy + C restatement of PyDTNN's CPU conv path.

The C kernels (``pydtnn_oracle.c`` -> ``liboracle.so``) restate the Cython loop
nests; this module restates the Python glue around them: the ``i2c`` Conv2D
forward/backward in both tensor formats, FC, the inference epilogues and the
tail of the VGG16 step.  GEMMs are NumPy ``@`` exactly as in
``pydtnn/utils/__init__.py:148-158``.

Pinning status (see tests/test_oracle.py):
  * im2col/col2im/im2row/row2im, conv forward/backward, FC, bias/BN/ReLU
    epilogues, 1023 transpose, maxpool: pinned by closed forms, adjoint
    identities, brute-force loops, torch.nn.functional CPU fp64 and the
    reference tests' hand-made arrays.
  * fused conv+bias+BN+ReLU through the libconvGemm boundary: the reference has
    no test for those arguments ("parity unpinned" at that boundary); pinned
    here only as the composition conv -> bias -> BN -> ReLU of pinned parts.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def lib():
    """Load liboracle.so (built by ``make -C oracle`` / ``__graft_entry__.build()``)."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            raise ImportError(f"{path} missing: run `make -C oracle`")
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    # pydtnn/cython_modules/im2col_nchw_cython.pyx:49-50
    raise TypeError(f"Type '{dtype}' is not supported by the oracle!")


def out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/layers/conv_2d.py:75-76"""
    ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
    wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
    return ho, wo


# --------------------------------------------------------------------------- kernels

def im2col_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:28-52"""
    x = np.ascontiguousarray(x)
    n, c, h, w = x.shape
    hh, ww = out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    cols = np.zeros((c * kh * kw, n * hh * ww), dtype=x.dtype)
    getattr(lib(), "oracle_im2col_nchw_" + _sfx(x.dtype))(
        _p(cols), _p(x), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return cols


def col2im_nchw(cols, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2col_nchw_cython.pyx:150-173"""
    cols = np.ascontiguousarray(cols)
    x = np.zeros((n, c, h, w), dtype=cols.dtype)
    getattr(lib(), "oracle_col2im_nchw_" + _sfx(cols.dtype))(
        _p(cols), _p(x), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return x


def im2row_nhwc(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49"""
    x = np.ascontiguousarray(x)
    n, h, w, c = x.shape
    hh, ww = out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    rows = np.zeros((n * hh * ww, c * kh * kw), dtype=x.dtype)
    getattr(lib(), "oracle_im2row_nhwc_" + _sfx(x.dtype))(
        _p(rows), _p(x), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return rows


def row2im_nhwc(rows, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation):
    """pydtnn/cython_modules/im2row_nhwc_cython.pyx:123-146"""
    rows = np.ascontiguousarray(rows)
    x = np.zeros((n, h, w, c), dtype=rows.dtype)
    getattr(lib(), "oracle_row2im_nhwc_" + _sfx(rows.dtype))(
        _p(rows), _p(x), n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return x


def add_nchw(x2d, b):
    """In place, pydtnn/cython_modules/add_nchw_cython.pyx:25-41"""
    assert x2d.flags["C_CONTIGUOUS"]
    b = np.ascontiguousarray(b, dtype=x2d.dtype)
    getattr(lib(), "oracle_add_nchw_" + _sfx(x2d.dtype))(
        _p(x2d), _p(b), ctypes.c_long(x2d.shape[0]), ctypes.c_long(x2d.shape[1]))
    return x2d


def add_nhwc(x2d, b):
    """In place, pydtnn/cython_modules/add_nhwc_cython.pyx:25-41"""
    assert x2d.flags["C_CONTIGUOUS"]
    b = np.ascontiguousarray(b, dtype=x2d.dtype)
    getattr(lib(), "oracle_add_nhwc_" + _sfx(x2d.dtype))(
        _p(x2d), _p(b), ctypes.c_long(x2d.shape[0]), ctypes.c_long(x2d.shape[1]))
    return x2d


def transpose_1023(src):
    """pydtnn/utils/best_transpose_1023.py:50-58 -> transpose_cython.pyx:125-141"""
    src = np.ascontiguousarray(src)
    d0, d1, d2, d3 = src.shape
    dst = np.empty((d1, d0, d2, d3), dtype=src.dtype)
    getattr(lib(), "oracle_transpose_1023_" + _sfx(src.dtype))(_p(src), _p(dst), d0, d1, d2, d3)
    return dst


def bn_inference(x2d, running_mean, inv_std, gamma, beta, relu=False):
    """pydtnn/cython_modules/bn_inference_cython.pyx:25-41, bn_relu_inference_cython.pyx:25-40"""
    x2d = np.ascontiguousarray(x2d)
    y = np.empty_like(x2d)
    name = ("oracle_bn_relu_inference_" if relu else "oracle_bn_inference_") + _sfx(x2d.dtype)
    vs = [np.ascontiguousarray(v, dtype=x2d.dtype) for v in (running_mean, inv_std, gamma, beta)]
    getattr(lib(), name)(_p(x2d), *[_p(v) for v in vs], _p(y),
                         ctypes.c_long(x2d.shape[0]), ctypes.c_long(x2d.shape[1]))
    return y


def bn_inference_nchw(x, running_mean, inv_std, gamma, beta):
    """pydtnn/cython_modules/bn_inference_cython.pyx:88-104"""
    x = np.ascontiguousarray(x)
    y = np.empty_like(x)
    vs = [np.ascontiguousarray(v, dtype=x.dtype) for v in (running_mean, inv_std, gamma, beta)]
    getattr(lib(), "oracle_bn_inference_nchw_" + _sfx(x.dtype))(
        _p(x), *[_p(v) for v in vs], _p(y), *x.shape)
    return y


def bn_training_forward(x, gamma, beta, running_mean, running_var, momentum=0.9, eps=1e-5, tensor_format="NHWC"):
    """TRAIN_MODE branch of pydtnn/backends/cpu/layers/batch_normalization_cpu.py:53-82 (sync_stats off).
    x is 2-D (rows, C) or 4-D in ``tensor_format``; the reference moves NCHW to NHWC
    (best_transpose_0231, :54-56), flattens to (rows, C), and restores the format at the end (:101-104).
    Returns (y, xn_2d, std, new_running_mean, new_running_var)."""
    shape = x.shape
    if x.ndim == 4 and tensor_format == "NCHW":
        x = x.transpose(0, 2, 3, 1)
    c = x.shape[-1]
    x2 = np.ascontiguousarray(x).reshape(-1, c)
    mu = np.mean(x2, axis=0)
    xc = (x2 - mu)
    var = np.mean(xc ** 2, axis=0)
    std = np.sqrt(var + eps)
    xn = xc / std
    y = gamma * xn + beta
    new_mean = momentum * running_mean + (1.0 - momentum) * mu
    new_var = momentum * running_var + (1.0 - momentum) * var
    if len(shape) == 4:
        y = y.reshape(x.shape)
        if tensor_format == "NCHW":
            y = np.ascontiguousarray(y.transpose(0, 3, 1, 2))
    return y, xn, std, new_mean, new_var


def bn_training_backward(dy, xn, std, gamma, tensor_format="NHWC", need_dx=True):
    """pydtnn/backends/cpu/layers/batch_normalization_cpu.py:108-129 with the dx formula of
    pydtnn/cython_modules/bn_training_cython.pyx:236-243.  xn is the (rows, C) matrix kept by the forward
    pass.  Returns (dgamma, dbeta, dx in the format of dy or None)."""
    shape = dy.shape
    if dy.ndim == 4 and tensor_format == "NCHW":
        dy = dy.transpose(0, 2, 3, 1)
    c = dy.shape[-1]
    dy2 = np.ascontiguousarray(dy).reshape(-1, c)
    n = dy2.shape[0]
    dgamma = np.sum(dy2 * xn, axis=0)
    dbeta = np.sum(dy2, axis=0)
    dx = None
    if need_dx:
        nf = dy2.dtype.type(n)
        dx = (gamma / (std * nf)) * (nf * dy2 - xn * dgamma - dbeta)
        if len(shape) == 4:
            dx = dx.reshape(dy.shape)
            if tensor_format == "NCHW":
                dx = np.ascontiguousarray(dx.transpose(0, 3, 1, 2))
    return dgamma, dbeta, dx


def relu(x):
    """pydtnn/cython_modules/relu_cython.pyx:25-39 -> (max(x,0), int8 mask)"""
    x = np.ascontiguousarray(x)
    y = np.empty_like(x)
    mask = np.empty(x.shape, dtype=np.int8)
    getattr(lib(), "oracle_relu_" + _sfx(x.dtype))(_p(x), _p(y), _p(mask), ctypes.c_long(x.size))
    return y, mask


def eltw_sum(acc, x):
    """In place acc += x, pydtnn/cython_modules/eltw_sum_cython.pyx:25-36"""
    assert acc.flags["C_CONTIGUOUS"]
    x = np.ascontiguousarray(x, dtype=acc.dtype)
    getattr(lib(), "oracle_eltw_sum_" + _sfx(acc.dtype))(_p(acc), _p(x), ctypes.c_long(acc.size))
    return acc


def _pool_array(a):
    """Pooling runs in the array's own float32 / float64 (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:42-49
    dispatches on the dtype); anything else is taken as float32."""
    a = np.asarray(a)
    return np.ascontiguousarray(a, dtype=a.dtype if a.dtype == np.float64 else np.float32)


def max_pool_2d_fwd_nchw(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:25-52"""
    x = _pool_array(x)
    n, c, h, w = x.shape
    hh, ww = out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = np.zeros((n, c, hh, ww), dtype=x.dtype)
    idx = np.zeros((n, c, hh, ww), dtype=np.int32)
    getattr(lib(), "oracle_max_pool_2d_fwd_nchw_" + _sfx(x.dtype))(_p(x), _p(y), _p(idx), n, c, h, w, kh, kw, vpadding, hpadding,
                                          vstride, hstride, vdilation, hdilation)
    return y, idx


def max_pool_2d_bwd_nchw(dy, idx_max, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:140-166"""
    dy = _pool_array(dy)
    idx_max = np.ascontiguousarray(idx_max, dtype=np.int32)
    dx = np.zeros((n, c, h, w), dtype=dy.dtype)
    getattr(lib(), "oracle_max_pool_2d_bwd_nchw_" + _sfx(dy.dtype))(_p(dy), _p(idx_max), _p(dx), n, c, h, w, kh, kw, vpadding, hpadding,
                                          vstride, hstride, vdilation, hdilation)
    return dx


def average_pool_2d_fwd(x, tensor_format, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:25-52 / average_pool_2d_nhwc_cython.pyx:25-52.
    ``kh`` / ``kw`` of 0 mean the whole extent (pydtnn/layers/abstract_pool_2d_layer.py:44-47)."""
    x = _pool_array(x)
    if tensor_format == "NCHW":
        n, c, h, w = x.shape
    else:
        n, h, w, c = x.shape
    kh, kw = kh or h, kw or w
    hh, ww = out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = np.zeros((n, c, hh, ww) if tensor_format == "NCHW" else (n, hh, ww, c), dtype=x.dtype)
    fn = getattr(lib(), f"oracle_average_pool_2d_{tensor_format.lower()}_fwd_{_sfx(x.dtype)}")
    fn(_p(x), _p(y), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return y


def average_pool_2d_bwd(dy, tensor_format, n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride,
                        vdilation=1, hdilation=1):
    """pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:135-160 / average_pool_2d_nhwc_cython.pyx:135-160"""
    dy = _pool_array(dy)
    kh, kw = kh or h, kw or w
    dx = np.zeros((n, c, h, w) if tensor_format == "NCHW" else (n, h, w, c), dtype=dy.dtype)
    fn = getattr(lib(), f"oracle_average_pool_2d_{tensor_format.lower()}_bwd_{_sfx(dy.dtype)}")
    fn(_p(dy), _p(dx), n, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    return dx


def max_pool_2d_fwd_nhwc(x, kh, kw, vpadding, hpadding, vstride, hstride, vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:25-52"""
    x = _pool_array(x)
    n, h, w, c = x.shape
    hh, ww = out_hw(h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
    y = np.zeros((n, hh, ww, c), dtype=x.dtype)
    idx = np.zeros((n, hh, ww, c), dtype=np.int32)
    getattr(lib(), "oracle_max_pool_2d_fwd_nhwc_" + _sfx(x.dtype))(_p(x), _p(y), _p(idx), n, h, w, c, kh, kw, vpadding, hpadding,
                                          vstride, hstride, vdilation, hdilation)
    return y, idx


def max_pool_2d_bwd_nhwc(dy, idx_max, n, h, w, c, kh, kw, vpadding, hpadding, vstride, hstride,
                         vdilation=1, hdilation=1):
    """pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:140-166"""
    dy = _pool_array(dy)
    idx_max = np.ascontiguousarray(idx_max, dtype=np.int32)
    dx = np.zeros((n, h, w, c), dtype=dy.dtype)
    getattr(lib(), "oracle_max_pool_2d_bwd_nhwc_" + _sfx(dy.dtype))(_p(dy), _p(idx_max), _p(dx), n, h, w, c, kh, kw, vpadding, hpadding,
                                          vstride, hstride, vdilation, hdilation)
    return dx


# --------------------------------------------------------------------------- conv layers (i2c)

class ConvParams:
    """Geometry of one Conv2D, named as in pydtnn/layers/conv_2d.py:31-55."""

    def __init__(self, kh, kw, vpadding=0, hpadding=0, vstride=1, hstride=1, vdilation=1, hdilation=1):
        self.kh, self.kw = kh, kw
        self.vpadding, self.hpadding = vpadding, hpadding
        self.vstride, self.hstride = vstride, hstride
        self.vdilation, self.hdilation = vdilation, hdilation

    def geom(self):
        return (self.kh, self.kw, self.vpadding, self.hpadding, self.vstride, self.hstride,
                self.vdilation, self.hdilation)


def conv2d_forward_nchw_i2c(x, weights, biases, p):
    """pydtnn/backends/cpu/layers/conv_2d_cpu.py:264-291.  weights (co,ci,kh,kw); returns (y, x_cols)."""
    co = weights.shape[0]
    x_cols = im2col_nchw(x, *p.geom())
    w_cols = weights.reshape(co, -1)
    res = w_cols @ x_cols
    if biases is not None:
        res = add_nchw(np.ascontiguousarray(res), biases)
    ho, wo = out_hw(x.shape[2], x.shape[3], *p.geom())
    y = transpose_1023(res.reshape(co, -1, ho, wo))
    return y, x_cols


def conv2d_backward_nchw_i2c(dy, x_cols, weights, x_shape, p, need_dx=True, use_bias=True):
    """pydtnn/backends/cpu/layers/conv_2d_cpu.py:447-481.  Returns (dw, db, dx)."""
    co = weights.shape[0]
    n, ci, hi, wi = x_shape
    dy_cols = transpose_1023(dy).reshape(co, -1)
    dw = (dy_cols @ x_cols.T).reshape(weights.shape)
    db = np.sum(dy, axis=(0, 2, 3)) if use_bias else None
    dx = None
    if need_dx:
        w_cols = weights.reshape(co, -1).T
        res = w_cols @ dy_cols
        dx = col2im_nchw(res, dy.shape[0], ci, hi, wi, *p.geom())
    return dw, db, dx


def conv2d_forward_nhwc_i2c(x, weights, biases, p):
    """pydtnn/backends/cpu/layers/conv_2d_cpu.py:183-209.  weights (ci,kh,kw,co); returns (y, x_rows)."""
    co = weights.shape[3]
    x_rows = im2row_nhwc(x, *p.geom())
    w_cols = weights.reshape(-1, co)
    res = x_rows @ w_cols
    if biases is not None:
        res = add_nhwc(np.ascontiguousarray(res), biases)
    ho, wo = out_hw(x.shape[1], x.shape[2], *p.geom())
    return res.reshape(-1, ho, wo, co), x_rows


def conv2d_backward_nhwc_i2c(dy, x_rows, weights, x_shape, p, need_dx=True, use_bias=True):
    """pydtnn/backends/cpu/layers/conv_2d_cpu.py:363-397.  Returns (dw, db, dx)."""
    co = weights.shape[3]
    n, hi, wi, ci = x_shape
    dy_rows = dy.reshape(-1, co)
    dw = (x_rows.T @ dy_rows).reshape(weights.shape)
    db = np.sum(dy, axis=(0, 1, 2)) if use_bias else None
    dx = None
    if need_dx:
        w_rows = weights.reshape(-1, co)
        res = dy_rows @ w_rows.T
        dx = row2im_nhwc(res, dy.shape[0], hi, wi, ci, *p.geom())
    return dw, db, dx


def fused_epilogue(y, tensor_format, bn=None, relu_flag=False):
    """Order bias -> BN(inference) -> ReLU; the bias is already inside ``y``.

    The order is the one the reference spells out in Python at
    pydtnn/backends/cpu/libs/conv_winograd.py:379-392; BN arithmetic is
    pydtnn/cython_modules/bn_inference_cython.pyx:71-72.
    ``bn`` = (running_mean, inv_std, gamma, beta) or None.
    """
    if bn is not None:
        if tensor_format == "NCHW":
            y = bn_inference_nchw(y, *bn)
        else:
            c = y.shape[-1]
            y = bn_inference(y.reshape(-1, c), *bn).reshape(y.shape)
    if relu_flag:
        y, _ = relu(y)
    return y


# --------------------------------------------------------------------------- FC and the VGG16 tail

def fc_forward(x, weights, biases):
    """pydtnn/backends/cpu/layers/fc_cpu.py:57-63 (use_bias=True branch)."""
    return x @ weights + biases


def fc_backward(dy, x, weights, need_dx=True):
    """pydtnn/backends/cpu/layers/fc_cpu.py:65-77.  Returns (dw, db, dx)."""
    dw = x.T @ dy
    db = np.sum(dy, axis=0)
    dx = dy @ weights.T if need_dx else None
    return dw, db, dx


def softmax_forward(x):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:32-35"""
    y = np.exp(x - np.max(x, axis=1, keepdims=True))
    y /= np.sum(y, axis=1, keepdims=True)
    return y


def softmax_backward(dy, y):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:37-39"""
    return y * (dy - (dy * y).sum(axis=1, keepdims=True))


def categorical_cross_entropy(y_pred, y_targ, global_batch_size, eps=1e-8):
    """pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35"""
    y_pred = np.clip(y_pred, a_min=eps, a_max=(1 - eps))
    b_range = np.arange(y_pred.shape[0])
    loss = -np.sum(np.log(y_pred[b_range, np.argmax(y_targ, axis=1)])) / y_pred.shape[0]
    dx = np.copy(y_targ)
    dx_amax = np.argmax(dx, axis=1)
    dx[b_range, dx_amax] /= (-y_pred[b_range, dx_amax] * global_batch_size)
    return loss, dx


def sgd_update(w, dw, velocity, lr, momentum=0.9, decay=0.0, nesterov=False):
    """pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41.  Returns (w, velocity); w updated in place."""
    velocity = momentum * velocity + dw
    if nesterov:
        w -= lr * (decay * w + dw + momentum * velocity)
    else:
        w -= lr * (decay * w + velocity)
    return w, velocity

"""GPU parity of the float64 route (explicit im2col / im2row + GEMM, FC, the per-channel passes) against the
oracle's float64 functions on the same seeded inputs.

Bar: bit-exact for the index-only kernels (their float64 sums follow the reference's order); max |a - b| / max |b|
<= 1e-10, the float64 tolerance of this path, for everything that goes through a GEMM (measured around 1e-15).
"""
import numpy as np
import pytest
import torch

from gpu_util import announce, dev, host, rel_err
from shapes import D, small_grid

pytestmark = pytest.mark.gpu

F64_REL_TOL = 1e-10

mid64 = [D(3, 5, 20, 17, 70, 3, 3, 1, 1, 1, 1, 1, 1), D(2, 16, 30, 30, 130, 3, 3, 1, 1, 1, 1, 1, 1),
         D(4, 3, 35, 35, 96, 11, 11, 0, 0, 4, 4, 1, 1), D(2, 33, 14, 14, 257, 1, 1, 0, 0, 1, 1, 1, 1),
         D(5, 8, 19, 23, 20, 5, 3, 2, 1, 2, 1, 1, 1), D(2, 12, 16, 16, 24, 3, 3, 2, 2, 1, 1, 2, 2),
         D(9, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1, 1, 1)]
grid64 = small_grid + mid64


@pytest.fixture(scope="module")
def pd():
    import pydtnn_amd
    from pydtnn_amd import native
    native.lib()
    return pydtnn_amd


@pytest.fixture(scope="module")
def ops(pd):
    from pydtnn_amd import ops as _ops
    return _ops


def close64(got, ref, what):
    err = rel_err(got, ref)
    assert err <= F64_REL_TOL, f"{what}: max rel err {err:.3e} > {F64_REL_TOL:.0e}"


def case64(d, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((d.b, d.c, d.h, d.w))
    w = rng.standard_normal((d.kn, d.c, d.kh, d.kw)) * np.sqrt(2.0 / (d.c * d.kh * d.kw))
    b = rng.standard_normal(d.kn)
    dy = rng.standard_normal((d.b, d.kn, d.ho, d.wo))
    return x, w, b, dy


@pytest.mark.parametrize("m,n,k,ta,tb", [(130, 70, 96, 0, 0), (257, 129, 300, 1, 0), (64, 200, 1000, 0, 1),
                                          (5, 3, 17, 1, 1), (256, 2304, 9000, 0, 1), (64, 512, 4096, 0, 0),
                                          (1000, 130, 64, 1, 0)])
def test_dgemm_against_numpy(ops, m, n, k, ta, tb):
    announce("dgemm", m, n, k, ta, tb)
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((k, m) if ta else (m, k))
    b = rng.standard_normal((n, k) if tb else (k, n))
    ad, bd = dev(a), dev(b)
    c = ops.matmul(ad.t() if ta else ad, bd.t() if tb else bd)
    assert c.dtype == torch.float64
    close64(host(c), (a.T if ta else a) @ (b.T if tb else b), "dgemm")
    bias = rng.standard_normal(n)
    c2 = ops.matmul(ad.t() if ta else ad, bd.t() if tb else bd, bias=dev(bias), relu=True)
    close64(host(c2), np.maximum((a.T if ta else a) @ (b.T if tb else b) + bias, 0), "dgemm + bias + relu")


@pytest.mark.parametrize("d", grid64, ids=repr)
def test_gathers_in_float64_equal_the_oracle_bit_for_bit(ops, oracle, d):
    announce("f64 gathers", d)
    x, _, _, _ = case64(d)
    g = d.geom()
    cols = ops.im2col_nchw(dev(x), *g)
    ref_cols = oracle.im2col_nchw(x, *g)
    assert cols.dtype == torch.float64 and np.array_equal(host(cols), ref_cols)
    rng = np.random.default_rng(1)
    c2 = rng.standard_normal(ref_cols.shape)
    assert np.array_equal(host(ops.col2im_nchw(dev(c2), d.b, d.c, d.h, d.w, *g)),
                          oracle.col2im_nchw(c2, d.b, d.c, d.h, d.w, *g))
    xr = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    ref_rows = oracle.im2row_nhwc(xr, *g)
    assert np.array_equal(host(ops.im2row_nhwc(dev(xr), *g)), ref_rows)
    r2 = rng.standard_normal(ref_rows.shape)
    assert np.array_equal(host(ops.row2im_nhwc(dev(r2), d.b, d.h, d.w, d.c, *g)),
                          oracle.row2im_nhwc(r2, d.b, d.h, d.w, d.c, *g))


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("d", grid64, ids=repr)
def test_conv2d_layer_in_float64(pd, oracle, fmt, d):
    """Conv2D under Model(dtype=float64): the explicit route, y / dw / db / dx against the oracle's float64 i2c
    functions (pydtnn/backends/cpu/layers/conv_2d_cpu.py:183-209, :264-291, :363-397, :447-481)."""
    announce("f64 conv layer", fmt, d)
    x, w, b, dy = case64(d)
    model = pd.Model(tensor_format=fmt, dtype="float64")
    assert model.enable_conv_gemm is False
    model.mode = pd.TRAIN_MODE
    conv = pd.Conv2D(nfilters=d.kn, filter_shape=(d.kh, d.kw), padding=(d.vpadding, d.hpadding),
                     stride=(d.vstride, d.hstride), dilation=(d.vdilation, d.hdilation))
    conv.set_model(model)
    p = oracle.ConvParams(*d.geom())
    if fmt == "NCHW":
        conv.initialize(prev_shape=(d.c, d.h, d.w))
        xs, ws, dys = x, w, dy
        fwd, bwd = oracle.conv2d_forward_nchw_i2c, oracle.conv2d_backward_nchw_i2c
    else:
        conv.initialize(prev_shape=(d.h, d.w, d.c))
        xs, ws, dys = (np.ascontiguousarray(a) for a in (x.transpose(0, 2, 3, 1), w.transpose(1, 2, 3, 0),
                                                         dy.transpose(0, 2, 3, 1)))
        fwd, bwd = oracle.conv2d_forward_nhwc_i2c, oracle.conv2d_backward_nhwc_i2c
    assert conv.forward.__name__ == f"_forward_{fmt.lower()}_i2c" and conv.weights.dtype == torch.float64
    conv.weights, conv.biases = dev(ws), dev(b)
    y = conv.forward(dev(xs))
    dx = conv.backward(dev(dys))
    y_ref, mat = fwd(xs, ws, b, p)
    assert y_ref.dtype == np.float64
    dw_ref, db_ref, dx_ref = bwd(dys, mat, ws, xs.shape, p)
    close64(host(y), y_ref, "y")
    close64(host(conv.dw), dw_ref, "dw")
    close64(host(conv.db), db_ref, "db")
    close64(host(dx), dx_ref, "dx")


def test_cfg1_in_float64(pd, oracle):
    import bench_configs
    announce("cfg1 f64")
    x, w, b = (a.astype(np.float64) for a in bench_configs.make_cfg1())
    b = np.random.default_rng(3).standard_normal(32)
    model = pd.Model(tensor_format="NHWC", dtype=torch.float64)
    model.mode = pd.EVALUATE_MODE
    conv = pd.Conv2D(nfilters=32, filter_shape=(3, 3), padding=1)
    conv.set_model(model)
    conv.initialize(prev_shape=(28, 28, 1))
    conv.weights, conv.biases = dev(w), dev(b)
    ref, _ = oracle.conv2d_forward_nhwc_i2c(x, w, b, oracle.ConvParams(3, 3, 1, 1))
    close64(host(conv.forward(dev(x))), ref, "cfg1 y")


def test_fc_relu_bn_and_block_in_float64(pd, oracle):
    """A small inference model in float64: conv - BN - relu, an addition block with a projection, flatten, FC."""
    announce("f64 model")
    rng = np.random.default_rng(5)
    model = pd.Model(tensor_format="NHWC", dtype="float64")
    model.add(pd.Input(shape=(10, 10, 4)))
    model.add(pd.Conv2D(nfilters=6, filter_shape=(3, 3), padding=1))
    model.add(pd.BatchNormalization())
    model.add(pd.Relu())
    model.add(pd.AdditionBlock([pd.Conv2D(nfilters=6, filter_shape=(3, 3), padding=1), pd.BatchNormalization()],
                               [pd.Conv2D(nfilters=6, filter_shape=(1, 1))]))
    model.add(pd.Relu())
    model.add(pd.Flatten())
    model.add(pd.FC(shape=(7,)))
    for layer in model.get_all_layers():
        for key in ("weights", "biases", "gamma", "beta", "running_mean"):
            t = getattr(layer, key, None)
            if t is not None:
                assert t.dtype == torch.float64, (layer, key)
                setattr(layer, key, dev(rng.standard_normal(tuple(t.shape)) * 0.3))
        if layer.canonical_name == "BatchNormalization":
            layer.running_var = dev(rng.uniform(0.5, 1.5, tuple(layer.running_var.shape)))
            layer.updated_running_var = True
    x = rng.standard_normal((3, 10, 10, 4))
    y = model.evaluate_batch(dev(x))
    assert y.dtype == torch.float64
    from test_gpu_models import oracle_forward
    cur = x
    for layer in model.layers[1:]:
        cur = oracle_forward(oracle, layer, cur, "NHWC")
    close64(host(y), cur, "f64 model output")
    # training-mode FC and Relu backward in float64
    model.mode = pd.TRAIN_MODE
    fc, relu = model.layers[-1], model.layers[3]
    xin = rng.standard_normal((3, 600))
    dy = rng.standard_normal((3, 7))
    fc.forward(dev(xin))
    dx = fc.backward(dev(dy))
    dw_ref, db_ref, dx_ref = oracle.fc_backward(dy, xin, host(fc.weights))
    close64(host(fc.dw), dw_ref, "fc dw")
    close64(host(fc.db), db_ref, "fc db")
    close64(host(dx), dx_ref, "fc dx")
    r = rng.standard_normal((3, 10, 10, 6))
    out = relu.forward(dev(r))
    back = relu.backward(dev(r * 2))
    assert np.array_equal(host(out), np.maximum(r, 0)) and np.array_equal(host(back), (r * 2) * (r > 0))


def test_float64_models_take_the_explicit_route_only(pd):
    with pytest.raises(ValueError):
        pd.Model(dtype="float64", enable_conv_gemm=True)
    with pytest.raises(ValueError):
        pd.ConvGemm(dtype=np.float64)     # pydtnn/backends/cpu/libs/conv_gemm.py:101-107

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


def close64(got, ref, what, floor=0.0):
    """``floor``: a lower bound on the scale the error is measured against, for results that are rounding noise
    around zero (the bias gradient of a convolution followed by BatchNormalization is zero in exact arithmetic)."""
    err = rel_err(got, ref)
    if floor > 0.0:
        err = err * np.max(np.abs(ref)) / max(np.max(np.abs(ref)), floor)
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
                                          (1000, 130, 64, 1, 0),
                                          # 2 x 520 = 1040 tiles: two rounds of 512 and a tail of 16, which goes to
                                          # the second launch (split in two along k); ragged last row and column tiles
                                          (200, 66500, 520, 0, 0), (200, 66500, 520, 1, 1),
                                          (130, 66000, 530, 1, 0), (130, 66000, 530, 0, 1)])
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


# ------------------------------------------------------------------ the layers around the convolutions
POOL64 = [  # (n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh)
    (2, 3, 8, 10, 2, 2, 0, 0, 2, 2, 1, 1), (2, 4, 9, 9, 3, 3, 1, 1, 2, 2, 1, 1), (1, 5, 7, 11, 3, 2, 1, 0, 1, 2, 1, 1),
    (1, 2, 9, 9, 2, 2, 1, 1, 1, 1, 2, 2), (2, 3, 12, 12, 3, 3, 1, 1, 1, 1, 1, 1), (3, 7, 13, 9, 2, 3, 0, 1, 2, 1, 1, 1)]


@pytest.mark.parametrize("geom", POOL64, ids=str)
def test_pooling_in_float64_equals_the_oracle_bit_for_bit(ops, oracle, geom):
    """Max-pooling (values, first-maximum indices, the reference's idx // kh, idx % kw decode in backward, ties) and
    average pooling in both tensor formats: index rules and summation orders are the reference's, so every bit
    must agree (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:115-137, :216-233)."""
    announce("pooling f64", geom)
    n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh = geom
    g = (kh, kw, pv, ph, sv, sh, dv, dh)
    rng = np.random.default_rng(33)
    x = rng.standard_normal((n, c, h, w)) + 1e-9 * rng.standard_normal((n, c, h, w))   # not float32-representable
    x[0, 0, :3, :3] = 0.75                                                              # ties: the first tap wins
    xh = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    y_ref, idx_ref = oracle.max_pool_2d_fwd_nchw(x, *g)
    dy = rng.standard_normal(y_ref.shape)
    dyh = np.ascontiguousarray(dy.transpose(0, 2, 3, 1))
    y, idx = ops.max_pool_2d_fwd_nchw(dev(x), *g)
    assert y.dtype == torch.float64
    assert np.array_equal(host(y), y_ref) and np.array_equal(host(idx), idx_ref)
    assert np.array_equal(host(ops.max_pool_2d_bwd_nchw(dev(dy), idx, n, c, h, w, *g)),
                          oracle.max_pool_2d_bwd_nchw(dy, idx_ref, n, c, h, w, *g))
    yh_ref, idxh_ref = oracle.max_pool_2d_fwd_nhwc(xh, *g)
    yh, idxh = ops.max_pool_2d_fwd_nhwc(dev(xh), *g)
    assert np.array_equal(host(yh), yh_ref) and np.array_equal(host(idxh), idxh_ref)
    assert np.array_equal(host(ops.max_pool_2d_bwd_nhwc(dev(dyh), idxh, n, h, w, c, *g)),
                          oracle.max_pool_2d_bwd_nhwc(dyh, idxh_ref, n, h, w, c, *g))
    # a ReLU mask below the pooling layer (the folded training step hands one over): a pass of its own in float64
    gate = (rng.random((n, c, h, w)) < 0.5).astype(np.int8)
    gated = ops.max_pool_2d_bwd_nchw(dev(dy), idx, n, c, h, w, *g, gate=dev(gate))
    assert np.array_equal(host(gated), oracle.max_pool_2d_bwd_nchw(dy, idx_ref, n, c, h, w, *g) * gate)
    if dv == 1 and dh == 1:
        for nhwc, xa, dya in ((False, x, dy), (True, xh, dyh)):
            fmt = "NHWC" if nhwc else "NCHW"
            assert np.array_equal(host(ops.average_pool_2d_fwd(dev(xa), nhwc, *g)), oracle.average_pool_2d_fwd(xa, fmt, *g))
            assert np.array_equal(host(ops.average_pool_2d_bwd(dev(dya), nhwc, n, c, h, w, *g)),
                                  oracle.average_pool_2d_bwd(dya, fmt, n, c, h, w, *g))


@pytest.mark.parametrize("rows,cols", [(64, 1000), (3, 7), (1, 1), (5, 300), (2, 4097)])
def test_softmax_cross_entropy_and_sgd_in_float64(ops, oracle, rows, cols):
    announce("softmax / cce / sgd f64", rows, cols)
    rng = np.random.default_rng(rows * 31 + cols)
    x = rng.standard_normal((rows, cols)) * 3
    y_ref = oracle.softmax_forward(x)
    y = ops.softmax(dev(x))
    assert y.dtype == torch.float64
    close64(host(y), y_ref, "softmax")
    dy = rng.standard_normal((rows, cols))
    close64(host(ops.softmax_backward(dev(dy), dev(y_ref))), oracle.softmax_backward(dy, y_ref), "softmax backward")
    y_targ = np.eye(cols)[rng.integers(0, cols, rows)]
    y_pred = y_ref.copy()
    y_pred[0, np.argmax(y_targ[0])] = 1e-12            # below eps: the clip decides
    loss_ref, dx_ref = oracle.categorical_cross_entropy(y_pred, y_targ, 2 * rows)
    loss, dx = ops.categorical_cross_entropy(dev(y_pred), dev(y_targ), 2 * rows)
    assert loss.dtype == torch.float64 and abs(float(loss) - loss_ref) <= 1e-12 * max(1.0, abs(loss_ref))
    close64(host(dx), dx_ref, "cce dx")
    for nesterov, decay in ((False, 0.0), (True, 1e-3)):
        w, dw, v = rng.standard_normal((rows, cols)), rng.standard_normal((rows, cols)), rng.standard_normal((rows, cols))
        wd, vd = dev(w), dev(v)
        ops.sgd_momentum(wd, dev(dw), vd, 0.01, 0.9, decay, nesterov)
        w_ref, v_ref = oracle.sgd_update(w.copy(), dw, v, 0.01, 0.9, decay, nesterov)
        assert np.array_equal(host(vd), v_ref)
        close64(host(wd), w_ref, "sgd weights")


@pytest.mark.parametrize("fmt,shape", [("NCHW", (8, 6, 5, 7)), ("NCHW", (70, 3, 4, 4)), ("NHWC", (8, 5, 7, 6)),
                                       ("NHWC", (300, 1, 1, 33))])
def test_batch_normalization_training_in_float64(ops, oracle, fmt, shape):
    announce("bn training f64", fmt, shape)
    rng = np.random.default_rng(8)
    c = shape[1] if fmt == "NCHW" else shape[3]
    inner = shape[2] * shape[3] if fmt == "NCHW" else 1
    x, dy = rng.standard_normal(shape) * 3 - 1, rng.standard_normal(shape)
    gamma, beta = rng.uniform(0.5, 1.5, c), rng.standard_normal(c)
    rm, rv = rng.standard_normal(c), rng.uniform(0.5, 1.5, c)
    rmd, rvd = dev(rm), dev(rv)
    y, xn, std = ops.bn_training_forward(dev(x), dev(gamma), dev(beta), rmd, rvd, 0.9, 1e-5, c, inner)
    y_ref, xn_ref, std_ref, rm_ref, rv_ref = oracle.bn_training_forward(x, gamma, beta, rm, rv, 0.9, 1e-5,
                                                                        tensor_format=fmt)
    assert y.dtype == torch.float64
    close64(host(y), y_ref, "y")
    close64(host(std), std_ref, "std")
    close64(host(rmd), rm_ref, "running mean")
    close64(host(rvd), rv_ref, "running var")
    dgamma, dbeta, dx = ops.bn_training_backward(dev(dy), xn, std, dev(gamma), c, inner)
    dgamma_ref, dbeta_ref, dx_ref = oracle.bn_training_backward(dy, xn_ref, std_ref, gamma, tensor_format=fmt)
    close64(host(dgamma), dgamma_ref, "dgamma")
    close64(host(dbeta), dbeta_ref, "dbeta")
    close64(host(dx), dx_ref, "dx")


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_float64_training_steps_match_the_oracle_chain(pd, oracle, fmt):
    """Two training steps of a float64 model, conv-relu-conv-bn-relu-pool-conv-relu-pool-flatten-fc-relu-fc-softmax
    with categorical cross-entropy and SGD with momentum, against the same chain of the oracle's float64 functions:
    loss, every gradient and every updated parameter to 1e-10 (what the reference computes when its model dtype is
    float64: explicit convolutions, pydtnn/backends/cpu/layers/conv_2d_cpu.py:183-209 / :264-291, and the dtype
    dispatch of its Cython modules)."""
    announce("float64 training steps", fmt)
    rng = np.random.default_rng(16)
    n, classes, hw = 6, 10, 12
    nchw = fmt == "NCHW"
    model = pd.Model(tensor_format=fmt, batch_size=n, dtype="float64")
    model.add(pd.Input(shape=(hw, hw, 3)))
    model.add(pd.Conv2D(nfilters=8, filter_shape=(3, 3), padding=1, activation="relu", weights_initializer="he_normal"))
    model.add(pd.Conv2D(nfilters=8, filter_shape=(3, 3), padding=1, weights_initializer="he_normal"))
    model.add(pd.BatchNormalization())
    model.add(pd.Relu())
    model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
    model.add(pd.Conv2D(nfilters=16, filter_shape=(3, 3), padding=1, activation="relu", weights_initializer="he_normal"))
    model.add(pd.MaxPool2D(pool_shape=(3, 3), stride=2, padding=1))
    model.add(pd.Flatten())
    model.add(pd.FC(shape=(32,), activation="relu", weights_initializer="he_normal"))
    model.add(pd.FC(shape=(classes,), activation="softmax", weights_initializer="he_normal"))
    for l in model.layers:   # parameters that float32 cannot hold
        for var in l.grad_vars:
            t = getattr(l, var)
            assert t.dtype == torch.float64
            t += 1e-9 * torch.randn_like(t)
    x = rng.random((n, 3, hw, hw)) if nchw else rng.random((n, hw, hw, 3))
    y_targ = np.eye(classes)[rng.integers(0, classes, n)]
    p3 = oracle.ConvParams(3, 3, 1, 1)
    conv_fwd = oracle.conv2d_forward_nchw_i2c if nchw else oracle.conv2d_forward_nhwc_i2c
    conv_bwd = oracle.conv2d_backward_nchw_i2c if nchw else oracle.conv2d_backward_nhwc_i2c
    pool_fwd = oracle.max_pool_2d_fwd_nchw if nchw else oracle.max_pool_2d_fwd_nhwc
    pool_bwd = oracle.max_pool_2d_bwd_nchw if nchw else oracle.max_pool_2d_bwd_nhwc
    state = {l.id: {v: host(getattr(l, v)).copy() for v in l.grad_vars} for l in model.layers if l.grad_vars}
    velocity = {i: {v: np.zeros_like(a) for v, a in s.items()} for i, s in state.items()}
    running = {l.id: [host(l.running_mean).copy(), host(l.running_var).copy()] for l in model.layers
               if l.canonical_name == "BatchNormalization"}
    opt, loss_fn = pd.SGD(learning_rate=0.05, momentum=0.9), pd.CategoricalCrossEntropy()
    for step in range(2):
        loss = model.train_batch(dev(x), dev(y_targ), loss_fn, opt)
        assert loss.dtype == torch.float64
        acts, cur = [], x
        for l in model.layers[1:]:
            name = l.canonical_name
            if name == "Conv2D":
                y, mat = conv_fwd(cur, state[l.id]["weights"], state[l.id]["biases"], p3)
                acts.append(("conv", l, cur.shape, mat))
                cur = y
            elif name == "BatchNormalization":
                rm, rv = running[l.id]
                cur, xn, std, rm, rv = oracle.bn_training_forward(cur, state[l.id]["gamma"], state[l.id]["beta"], rm, rv,
                                                                  l.momentum, l.epsilon, tensor_format=fmt)
                running[l.id] = [rm, rv]
                acts.append(("bn", l, xn, std))
            elif name == "Relu":
                cur, mask = oracle.relu(cur)
                acts.append(("relu", l, mask))
            elif name == "MaxPool2D":
                shp = cur.shape
                cur, idx = pool_fwd(cur, *l._geom())
                acts.append(("pool", l, shp, idx))
            elif name == "Flatten":
                acts.append(("flat", l, cur.shape))
                cur = cur.reshape(n, -1)
            elif name == "FC":
                acts.append(("fc", l, cur))
                cur = oracle.fc_forward(cur, state[l.id]["weights"], state[l.id]["biases"])
            elif name == "Softmax":
                cur = oracle.softmax_forward(cur)
                acts.append(("softmax", l, cur))
        assert cur.dtype == np.float64
        loss_ref, dcur = oracle.categorical_cross_entropy(cur, y_targ, n)
        assert abs(float(loss) - loss_ref) <= F64_REL_TOL * abs(loss_ref)
        grads = {}
        for kind, l, *saved in reversed(acts):
            if kind == "softmax":
                dcur = oracle.softmax_backward(dcur, saved[0])
            elif kind == "fc":
                dw, db, dcur = oracle.fc_backward(dcur, saved[0], state[l.id]["weights"])
                grads[l.id] = {"weights": dw, "biases": db}
            elif kind == "flat":
                dcur = dcur.reshape(saved[0])
            elif kind == "pool":
                shp, idx = saved
                dcur = pool_bwd(dcur, idx, *shp, *l._geom())
            elif kind == "relu":
                dcur = dcur * saved[0]
            elif kind == "bn":
                dgamma, dbeta, dcur = oracle.bn_training_backward(dcur, saved[0], saved[1], state[l.id]["gamma"],
                                                                  tensor_format=fmt)
                grads[l.id] = {"gamma": dgamma, "beta": dbeta}
            elif kind == "conv":
                shp, mat = saved
                dw, db, dx = conv_bwd(dcur, mat, state[l.id]["weights"], shp, p3, need_dx=l.need_dx)
                grads[l.id] = {"weights": dw, "biases": db}
                dcur = dx
        for l in model.layers:
            for var, grad_name in l.grad_vars.items():
                close64(host(getattr(l, grad_name)).reshape(grads[l.id][var].shape), grads[l.id][var],
                        f"step {step} {l!r} {grad_name}", floor=1e-3)
                w, v = oracle.sgd_update(state[l.id][var], grads[l.id][var].reshape(state[l.id][var].shape),
                                         velocity[l.id][var], 0.05, 0.9)
                state[l.id][var], velocity[l.id][var] = w, v
                close64(host(getattr(l, var)), w, f"step {step} {l!r} {var}", floor=1e-3)
        for l in model.layers:
            if l.id in running:
                close64(host(l.running_mean), running[l.id][0], "running mean")
                close64(host(l.running_var), running[l.id][1], "running var")

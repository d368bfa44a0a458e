"""GPU parity tests at the layer / model level: the PyDTNN layer protocol on top of the kernels.

Pattern follows the reference's own layer tests: build the layer under a model, feed the same
arrays to the CPU path (here: the oracle) and compare y, dw, db, dx
(pydtnn/tests/conv2d_conv_gemm.py:114-200, check_tensor_format_models.py:66-162,
check_conv_gemm_models.py:100-167: the CPU activations are fed to each layer under test).
"""
import numpy as np
import pytest
import torch

from gpu_util import announce, assert_close, dev, host
from shapes import D, small_grid

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pd():
    import pydtnn_amd
    from pydtnn_amd import native
    native.lib()
    return pydtnn_amd


def nhwc(a):
    return np.ascontiguousarray(a.transpose(0, 2, 3, 1))


def make_conv(pd, d, fmt, variant, need_dx=True, use_bias=True):
    model = pd.Model(tensor_format=fmt, enable_conv_gemm=(variant == "cg"), batch_size=d.b)
    model.mode = pd.TRAIN_MODE
    layer = pd.Conv2D(nfilters=d.kn, filter_shape=(d.kh, d.kw), padding=(d.vpadding, d.hpadding),
                      stride=(d.vstride, d.hstride), dilation=(d.vdilation, d.hdilation), use_bias=use_bias)
    layer.set_model(model)
    layer.initialize(prev_shape=(d.c, d.h, d.w) if fmt == "NCHW" else (d.h, d.w, d.c), need_dx=need_dx)
    return model, layer


layer_grid = small_grid[:8] + [D(4, 16, 20, 20, 40, 3, 3, 1, 1, 1, 1), D(3, 8, 17, 17, 12, 3, 3, 1, 1, 2, 2)]


@pytest.mark.parametrize("variant", ["i2c", "cg"])
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("d", layer_grid, ids=repr)
def test_conv2d_layer_forward_backward(pd, oracle, d, fmt, variant):
    announce("Conv2D layer", fmt, variant, d)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(np.float32)
    w = rng.standard_normal((d.kn, d.c, d.kh, d.kw)).astype(np.float32) * 0.2
    b = rng.standard_normal(d.kn).astype(np.float32)
    dy = rng.standard_normal((d.b, d.kn, d.ho, d.wo)).astype(np.float32)
    model, layer = make_conv(pd, d, fmt, variant)
    assert layer.forward.__name__ == f"_forward_{fmt.lower()}_{variant}"
    p = oracle.ConvParams(*d.geom())
    if fmt == "NCHW":
        assert tuple(layer.weights.shape) == w.shape and layer.shape == (d.kn, d.ho, d.wo)
        layer.weights, layer.biases = dev(w), dev(b)
        y_ref, x_cols = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
        dw_ref, db_ref, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
        y = layer.forward(dev(x))
        dx = layer.backward(dev(dy))
        if variant == "i2c":
            assert np.array_equal(host(layer.x_cols), x_cols)  # the stored matrix is the reference's x_cols
    else:
        wr = np.ascontiguousarray(w.transpose(1, 2, 3, 0))
        assert tuple(layer.weights.shape) == wr.shape and layer.shape == (d.ho, d.wo, d.kn)
        layer.weights, layer.biases = dev(wr), dev(b)
        y_ref, x_rows = oracle.conv2d_forward_nhwc_i2c(nhwc(x), wr, b, p)
        dw_ref, db_ref, dx_ref = oracle.conv2d_backward_nhwc_i2c(nhwc(dy), x_rows, wr, nhwc(x).shape, p)
        y = layer.forward(dev(nhwc(x)))
        dx = layer.backward(dev(nhwc(dy)))
        if variant == "i2c":
            assert np.array_equal(host(layer.x_rows), x_rows)
    assert_close(host(y), y_ref, what="y")
    assert_close(host(layer.dw), dw_ref, what="dw")
    assert tuple(layer.dw.shape) == tuple(layer.weights.shape)
    assert_close(host(layer.db), db_ref, tol=1e-5, what="db")
    assert_close(host(dx), dx_ref, what="dx")


def test_first_layer_has_no_dx(pd):
    d = small_grid[1]
    model, layer = make_conv(pd, d, "NCHW", "cg", need_dx=False)
    x = torch.randn((d.b, d.c, d.h, d.w), device="cuda")
    y = layer.forward(x)
    assert layer.backward(torch.ones_like(y)) is None and layer.dw is not None


def test_grouped_convolutions_raise(pd):
    model = pd.Model(tensor_format="NCHW")
    layer = pd.Conv2D(nfilters=4, filter_shape=(3, 3), grouping="depthwise")
    layer.set_model(model)
    with pytest.raises(NotImplementedError):
        layer.initialize(prev_shape=(4, 8, 8))


def test_fc_layer(pd, oracle):
    rng = np.random.default_rng(1)
    for (bsz, nin, nout) in [(64, 300, 100), (5, 4100, 33)]:
        announce("FC", bsz, nin, nout)
        model = pd.Model(tensor_format="NCHW", batch_size=bsz)
        model.mode = pd.TRAIN_MODE
        fc = pd.FC(shape=(nout,))
        fc.set_model(model)
        fc.initialize(prev_shape=(nin,))
        x = rng.standard_normal((bsz, nin)).astype(np.float32)
        w = (rng.standard_normal((nin, nout)) / np.sqrt(nin)).astype(np.float32)
        b = rng.standard_normal(nout).astype(np.float32)
        dy = rng.standard_normal((bsz, nout)).astype(np.float32)
        assert tuple(fc.weights.shape) == (nin, nout)
        fc.weights, fc.biases = dev(w), dev(b)
        y = fc.forward(dev(x))
        dx = fc.backward(dev(dy))
        dw_ref, db_ref, dx_ref = oracle.fc_backward(dy, x, w)
        assert_close(host(y), oracle.fc_forward(x, w, b), what="fc y")
        assert_close(host(fc.dw), dw_ref, what="fc dw")
        assert_close(host(fc.db), db_ref, tol=1e-5, what="fc db")
        assert_close(host(dx), dx_ref, what="fc dx")


# ------------------------------------------------------------------ fusion

def build_conv_bn_relu_model(pd, fmt, flags, shape_hwc=(12, 12, 6), seed=2):
    model = pd.Model(tensor_format=fmt, **flags)
    model.add(pd.Input(shape=shape_hwc))
    model.add(pd.Conv2D(nfilters=10, filter_shape=(3, 3), padding=1))
    model.add(pd.BatchNormalization())
    model.add(pd.Relu())
    model.add(pd.Conv2D(nfilters=7, filter_shape=(1, 1)))
    model.add(pd.BatchNormalization())
    model.add(pd.Conv2D(nfilters=5, filter_shape=(3, 3), stride=2, activation="relu"))
    rng = np.random.default_rng(seed)
    for layer in model.layers:
        if layer.canonical_name == "BatchNormalization":
            c = layer.gamma.numel()
            layer.gamma = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
            layer.beta = dev(rng.normal(0, 0.1, c).astype(np.float32))
            layer.running_mean = dev(rng.normal(0, 0.1, c).astype(np.float32))
            layer.running_var = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
            layer.updated_running_var = True
        elif layer.canonical_name == "Conv2D":
            layer.weights = dev((rng.standard_normal(tuple(layer.weights.shape)) * 0.2).astype(np.float32))
            layer.biases = dev(rng.standard_normal(layer.co).astype(np.float32))
    return model


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_fusion_rewrites_the_graph_and_keeps_the_numbers(pd, oracle, fmt):
    announce("fusion", fmt)
    flags = dict(enable_fused_conv_bn_relu=True, enable_fused_conv_bn=True, enable_fused_conv_relu=True,
                 enable_fused_bn_relu=True)
    plain = build_conv_bn_relu_model(pd, fmt, {})
    fused = build_conv_bn_relu_model(pd, fmt, flags)
    x = np.random.default_rng(3).standard_normal((4, 6, 12, 12)).astype(np.float32)
    xin = dev(x if fmt == "NCHW" else nhwc(x))
    y_plain = plain.evaluate_dataset_batch(xin)
    y_fused = fused.evaluate_dataset_batch(xin)
    names = [layer.canonical_name for layer in fused.layers]
    assert names == ["Input", "Conv2DBatchNormalizationRelu", "Conv2DBatchNormalization", "Conv2DRelu"]
    assert [layer.canonical_name for layer in plain.layers][1:4] == ["Conv2D", "BatchNormalization", "Relu"]
    assert_close(host(y_fused), host(y_plain), tol=1e-6, what="fused vs layer-by-layer")
    # against the oracle: conv -> bias -> BN -> ReLU composed from pinned parts
    p1 = oracle.ConvParams(3, 3, 1, 1)
    p2 = oracle.ConvParams(1, 1)
    p3 = oracle.ConvParams(3, 3, 0, 0, 2, 2)
    convs = [l for l in plain.layers if l.canonical_name == "Conv2D"]
    bns = [l for l in plain.layers if l.canonical_name == "BatchNormalization"]
    cur = x if fmt == "NCHW" else nhwc(x)
    fwd = oracle.conv2d_forward_nchw_i2c if fmt == "NCHW" else oracle.conv2d_forward_nhwc_i2c
    for conv, p, bn, relu in [(convs[0], p1, bns[0], True), (convs[1], p2, bns[1], False), (convs[2], p3, None, True)]:
        cur, _ = fwd(cur, host(conv.weights), host(conv.biases), p)
        bn_args = None
        if bn is not None:
            inv_std = (1.0 / np.sqrt(host(bn.running_var) + np.float32(bn.epsilon))).astype(np.float32)
            bn_args = (host(bn.running_mean), inv_std, host(bn.gamma), host(bn.beta))
        cur = oracle.fused_epilogue(cur, fmt, bn=bn_args, relu_flag=relu)
    assert_close(host(y_fused), cur, what="fused vs oracle")


def test_i2c_convolutions_are_not_fused(pd):
    model = build_conv_bn_relu_model(pd, "NCHW", dict(enable_conv_gemm=False, enable_fused_conv_bn_relu=True))
    model.apply_layer_fusion()
    assert [l.canonical_name for l in model.layers][1:4] == ["Conv2D", "BatchNormalization", "Relu"]


def test_fused_layers_refuse_training_and_backward(pd):
    model = build_conv_bn_relu_model(pd, "NCHW", dict(enable_fused_conv_bn_relu=True))
    model.apply_layer_fusion()
    fused = model.layers[1]
    model.mode = pd.TRAIN_MODE
    with pytest.raises(RuntimeError):
        fused.forward(torch.zeros((1, 6, 12, 12), device="cuda"))
    with pytest.raises(RuntimeError):
        fused.backward(torch.zeros((1, 10, 12, 12), device="cuda"))


def test_residual_block_with_fusion(pd, oracle):
    """A bottleneck shaped like pydtnn/models/resnet50_imagenet.py:41-59, NHWC, all fusions on."""
    announce("bottleneck")
    rng = np.random.default_rng(4)
    cin, mid, hw, n = 16, 8, 10, 3

    def build(flags):
        model = pd.Model(tensor_format="NHWC", **flags)
        model.add(pd.Input(shape=(hw, hw, cin)))
        model.add(pd.AdditionBlock(
            [pd.Conv2D(nfilters=mid, filter_shape=(1, 1)), pd.BatchNormalization(), pd.Relu(),
             pd.Conv2D(nfilters=mid, filter_shape=(3, 3), padding=1), pd.BatchNormalization(), pd.Relu(),
             pd.Conv2D(nfilters=cin, filter_shape=(1, 1)), pd.BatchNormalization()],
            []))
        model.add(pd.Relu())
        return model

    plain, fused = build({}), build(dict(enable_fused_conv_bn_relu=True, enable_fused_conv_bn=True))
    r = np.random.default_rng(5)
    for a, b in zip(plain.get_all_layers(), fused.get_all_layers()):
        if a.canonical_name == "Conv2D":
            a.weights = b.weights = dev((r.standard_normal(tuple(a.weights.shape)) * 0.3).astype(np.float32))
        elif a.canonical_name == "BatchNormalization":
            c = a.gamma.numel()
            a.gamma = b.gamma = dev(r.uniform(0.5, 1.5, c).astype(np.float32))
            a.beta = b.beta = dev(r.normal(0, 0.1, c).astype(np.float32))
            a.running_mean = b.running_mean = dev(r.normal(0, 0.1, c).astype(np.float32))
            a.running_var = b.running_var = dev(r.uniform(0.5, 1.5, c).astype(np.float32))
            a.updated_running_var = b.updated_running_var = True
    x = rng.standard_normal((n, hw, hw, cin)).astype(np.float32)
    xd = dev(x)
    y_plain = plain.evaluate_dataset_batch(xd)
    y_fused = fused.evaluate_dataset_batch(xd)
    block = fused.layers[1]
    assert [l.canonical_name for l in block.paths[0]] == \
        ["Conv2DBatchNormalizationRelu", "Conv2DBatchNormalizationRelu", "Conv2DBatchNormalization"]
    assert np.array_equal(host(xd), x), "the block must not add into its input"
    assert_close(host(y_fused), host(y_plain), tol=1e-6, what="bottleneck fused vs plain")
    # the fused model's block lets its last convolution add the shortcut and do the Relu that follows; the
    # same layers with that hand-over switched off (separate eltw_sum and relu passes) give the same bits
    assert block.relu_above is fused.layers[2] and block._folded_sum_path() == 0
    fused._fused = False
    try:
        assert block._folded_sum_path() is None
        y_separate = fused.evaluate_batch(xd)
    finally:
        fused._fused = True
    assert torch.equal(y_fused, y_separate)
    # oracle: relu(x + bn3(conv3(relu(bn2(conv2(relu(bn1(conv1(x)))))))))
    convs = [l for l in plain.get_all_layers() if l.canonical_name == "Conv2D"]
    bns = [l for l in plain.get_all_layers() if l.canonical_name == "BatchNormalization"]
    cur = x
    for conv, bn, relu, p in zip(convs, bns, (True, True, False),
                                 (oracle.ConvParams(1, 1), oracle.ConvParams(3, 3, 1, 1), oracle.ConvParams(1, 1))):
        cur, _ = oracle.conv2d_forward_nhwc_i2c(cur, host(conv.weights), host(conv.biases), p)
        inv_std = (1.0 / np.sqrt(host(bn.running_var) + np.float32(bn.epsilon))).astype(np.float32)
        cur = oracle.fused_epilogue(cur, "NHWC", bn=(host(bn.running_mean), inv_std, host(bn.gamma), host(bn.beta)),
                                    relu_flag=relu)
    ref, _ = oracle.relu(oracle.eltw_sum(np.ascontiguousarray(cur), x))
    assert_close(host(y_fused), ref, what="bottleneck vs oracle")


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_block_of_one_convolution_adds_its_own_input(pd, oracle, fmt):
    """An AdditionBlock whose one path is a single Conv2D + BN and whose other path is the identity: after the
    fusion pass the convolution's store adds the residual, and the residual is the convolution's own input x
    (the store reads a tile's residual before it writes the tile of y; x is only read).  Same bits as the separate
    sum, x untouched, and the oracle's relu(x + bn(conv(x)))."""
    announce("one-convolution block", fmt)
    rng = np.random.default_rng(8)
    c, hw, n = 12, 9, 4
    shape = (c, hw, hw) if fmt == "NCHW" else (hw, hw, c)

    model = pd.Model(tensor_format=fmt, enable_fused_conv_bn=True)
    model.add(pd.Input(shape=(hw, hw, c)))                     # (h, w, c), encoded into the model's format
    model.add(pd.AdditionBlock([pd.Conv2D(nfilters=c, filter_shape=(3, 3), padding=1), pd.BatchNormalization()], []))
    model.add(pd.Relu())
    conv, bn = [l for l in model.get_all_layers() if l.canonical_name in ("Conv2D", "BatchNormalization")]
    conv.weights = dev((rng.standard_normal(tuple(conv.weights.shape)) * 0.3).astype(np.float32))
    conv.biases = dev(rng.standard_normal(c).astype(np.float32))
    bn.gamma, bn.beta = dev(rng.uniform(0.5, 1.5, c).astype(np.float32)), dev(rng.normal(0, 0.1, c).astype(np.float32))
    bn.running_mean = dev(rng.normal(0, 0.1, c).astype(np.float32))
    bn.running_var = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
    bn.updated_running_var = True
    w_h, b_h = host(conv.weights), host(conv.biases)
    bn_h = (host(bn.running_mean), (1.0 / np.sqrt(host(bn.running_var) + np.float32(bn.epsilon))).astype(np.float32),
            host(bn.gamma), host(bn.beta))
    x = rng.standard_normal((n,) + shape).astype(np.float32)
    xd = dev(x)
    y = model.evaluate_dataset_batch(xd)
    block = model.layers[1]
    assert [l.canonical_name for l in block.paths[0]] == ["Conv2DBatchNormalization"]
    assert block._folded_sum_path() == 0 and block.relu_above is model.layers[2]
    assert np.array_equal(host(xd), x), "the block must not write into its input"
    model._fused = False
    try:
        y_separate = model.evaluate_batch(xd)
    finally:
        model._fused = True
    assert torch.equal(y, y_separate)
    p = oracle.ConvParams(3, 3, 1, 1)
    fwd = oracle.conv2d_forward_nchw_i2c if fmt == "NCHW" else oracle.conv2d_forward_nhwc_i2c
    cur, _ = fwd(x, w_h, b_h, p)
    cur = oracle.fused_epilogue(cur, fmt, bn=bn_h, relu_flag=False)
    ref, _ = oracle.relu(oracle.eltw_sum(np.ascontiguousarray(cur), x))
    assert_close(host(y), ref, what="one-convolution block vs oracle")


# ------------------------------------------------------------------ a small VGG-style training step

@pytest.mark.parametrize("folding", [False, True], ids=["plain", "relu_folding"])
def test_small_vgg_training_step_matches_the_oracle_chain(pd, oracle, folding):
    """conv-relu-conv-relu-pool-conv-relu-pool-flatten-fc-relu-fc-softmax, CCE, SGD momentum: one step,
    every gradient and updated weight compared with the oracle run end to end on the CPU."""
    announce("small vgg step", folding)
    rng = np.random.default_rng(6)
    n, classes = 8, 10
    model = pd.Model(tensor_format="NCHW", batch_size=n, enable_relu_folding=folding)
    model.add(pd.Input(shape=(16, 16, 3)))
    for nf in (8, 8):
        model.add(pd.Conv2D(nfilters=nf, filter_shape=(3, 3), padding=1, activation="relu",
                            weights_initializer="he_normal"))
    model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
    model.add(pd.Conv2D(nfilters=16, filter_shape=(3, 3), padding=1, activation="relu",
                        weights_initializer="he_normal"))
    model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
    model.add(pd.Flatten())
    model.add(pd.FC(shape=(32,), activation="relu", weights_initializer="he_normal"))
    model.add(pd.FC(shape=(classes,), activation="softmax", weights_initializer="he_normal"))
    assert model.layers[1].need_dx is False and model.layers[3].need_dx is True  # pydtnn/model.py:270
    x = rng.random((n, 3, 16, 16)).astype(np.float32)
    labels = rng.integers(0, classes, n)
    y_targ = np.eye(classes, dtype=np.float32)[labels]
    params = {l.id: (host(l.weights).copy(), host(l.biases).copy()) for l in model.layers if l.grad_vars}

    loss = model.train_batch(dev(x), dev(y_targ), pd.CategoricalCrossEntropy(), pd.SGD(learning_rate=0.01, momentum=0.9))

    # ---- oracle chain
    p3 = oracle.ConvParams(3, 3, 1, 1)
    acts, cur = [], x
    for l in model.layers[1:]:
        name = l.canonical_name
        if name == "Conv2D":
            w, b = params[l.id]
            y, cols = oracle.conv2d_forward_nchw_i2c(cur, w, b, p3)
            acts.append(("conv", l, cur.shape, cols))
            cur = y
        elif name == "Relu":
            cur, mask = oracle.relu(cur)
            acts.append(("relu", l, mask))
        elif name == "MaxPool2D":
            shp = cur.shape
            cur, idx = oracle.max_pool_2d_fwd_nchw(cur, 2, 2, 0, 0, 2, 2)
            acts.append(("pool", l, shp, idx))
        elif name == "Flatten":
            acts.append(("flat", l, cur.shape))
            cur = cur.reshape(n, -1)
        elif name == "FC":
            w, b = params[l.id]
            acts.append(("fc", l, cur))
            cur = oracle.fc_forward(cur, w, b)
        elif name == "Softmax":
            cur = oracle.softmax_forward(cur)
            acts.append(("softmax", l, cur))
    loss_ref, dcur = oracle.categorical_cross_entropy(cur, y_targ, n)
    assert abs(float(loss) - loss_ref) <= 1e-4 * abs(loss_ref)
    for kind, l, *saved in reversed(acts):
        if kind == "softmax":
            dcur = oracle.softmax_backward(dcur, saved[0])
        elif kind == "fc":
            w, b = params[l.id]
            dw, db, dcur = oracle.fc_backward(dcur, saved[0], w)
            assert_close(host(l.dw), dw, what=f"{l} dw")
            assert_close(host(l.db), db, tol=1e-5, what=f"{l} db")
            w_new, _ = oracle.sgd_update(w.copy(), dw, np.zeros_like(w), np.float32(0.01), np.float32(0.9))
            assert_close(host(l.weights), w_new, tol=1e-5, what=f"{l} updated weights")
        elif kind == "flat":
            dcur = dcur.reshape(saved[0])
        elif kind == "pool":
            shp, idx = saved
            dcur = oracle.max_pool_2d_bwd_nchw(dcur, idx, *shp, 2, 2, 0, 0, 2, 2)
        elif kind == "relu":
            dcur = dcur * saved[0]
        elif kind == "conv":
            w, b = params[l.id]
            shp, cols = saved
            dw, db, dx = oracle.conv2d_backward_nchw_i2c(dcur, cols, w, shp, p3, need_dx=l.need_dx)
            assert_close(host(l.dw), dw, what=f"{l} dw")
            assert_close(host(l.db), db, tol=1e-5, what=f"{l} db")
            w_new, _ = oracle.sgd_update(w.copy(), dw, np.zeros_like(w), np.float32(0.01), np.float32(0.9))
            assert_close(host(l.weights), w_new, tol=1e-5, what=f"{l} updated weights")
            dcur = dx


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_relu_folding_changes_no_bit_of_a_training_run(pd, fmt, monkeypatch):
    """Two training steps of a small VGG with the Relu layers done by their neighbours' stores (the default) and
    with separate Relu passes: losses, every gradient and every updated weight are identical, and the folded
    run really skips the passes (only the FC layer's Relu calls the stand-alone kernels)."""
    from pydtnn_amd import ops
    announce("relu folding", fmt)
    n, classes = 8, 10
    rng = np.random.default_rng(16)
    x = dev(rng.random((n, 3, 16, 16) if fmt == "NCHW" else (n, 16, 16, 3)).astype(np.float32))
    y_targ = dev(np.eye(classes, dtype=np.float32)[rng.integers(0, classes, n)])
    calls = {"fwd": 0, "bwd": 0}
    relu, relu_backward = ops.relu, ops.relu_backward
    monkeypatch.setattr(ops, "relu", lambda *a, **k: (calls.__setitem__("fwd", calls["fwd"] + 1), relu(*a, **k))[1])
    monkeypatch.setattr(ops, "relu_backward",
                        lambda *a, **k: (calls.__setitem__("bwd", calls["bwd"] + 1), relu_backward(*a, **k))[1])

    def run(folding):
        np.random.seed(5)
        model = pd.Model(tensor_format=fmt, batch_size=n, enable_relu_folding=folding)
        model.add(pd.Input(shape=(16, 16, 3)))
        model.add(pd.Conv2D(nfilters=8, filter_shape=(3, 3), padding=1, activation="relu", weights_initializer="he_normal"))
        model.add(pd.Conv2D(nfilters=8, filter_shape=(3, 3), padding=1, stride=2, weights_initializer="he_normal"))
        model.add(pd.Relu())  # an explicit Relu layer after a strided convolution (dX by GEMM + col2im / row2im)
        model.add(pd.Conv2D(nfilters=12, filter_shape=(3, 3), padding=1, activation="relu", weights_initializer="he_normal"))
        model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
        model.add(pd.Flatten())
        model.add(pd.FC(shape=(32,), activation="relu", weights_initializer="he_normal"))
        model.add(pd.FC(shape=(classes,), activation="softmax", weights_initializer="he_normal"))
        loss_fn, opt = pd.CategoricalCrossEntropy(), pd.SGD(learning_rate=0.05, momentum=0.9)
        calls["fwd"] = calls["bwd"] = 0
        losses = [float(model.train_batch(x, y_targ, loss_fn, opt)) for _ in range(2)]
        state = {}
        for l in model.layers:
            for var, grad in l.grad_vars.items():
                state[f"{l.id}.{var}"] = getattr(l, var).clone()
                state[f"{l.id}.{grad}"] = getattr(l, grad).clone()
        masks = [l.mask.clone() for l in model.layers if l.canonical_name == "Relu"]
        return losses, state, masks, dict(calls)

    losses_a, state_a, masks_a, calls_a = run(True)
    losses_b, state_b, masks_b, calls_b = run(False)
    assert losses_a == losses_b
    assert state_a.keys() == state_b.keys()
    for k in state_a:
        assert torch.equal(state_a[k], state_b[k]), k
    assert all(torch.equal(a, b) for a, b in zip(masks_a, masks_b))
    assert calls_b == {"fwd": 8, "bwd": 8}   # four Relu layers, two steps
    assert calls_a == {"fwd": 2, "bwd": 2}   # only the Relu between the FC layers


@pytest.mark.parametrize("n,hw,c1", [(8, 16, 8), (32, 48, 32)])
@pytest.mark.parametrize("conv_gemm", [True, False])
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_backward_overlap_changes_no_bit_of_a_training_run(pd, fmt, conv_gemm, n, hw, c1):
    """Eight training steps of a small network with a residual block, with the filter / bias gradients on the
    model's second stream (the default) and with everything on the caller's stream: losses, every gradient and
    every updated weight are identical; the second stream is used by the one run only, and nothing of a step is
    left on it when train_batch returns."""
    announce("backward overlap", fmt, conv_gemm, n, hw, c1)
    classes = 10
    rng = np.random.default_rng(23)
    x = dev(rng.random((n, 3, hw, hw) if fmt == "NCHW" else (n, hw, hw, 3)).astype(np.float32))
    y_targ = dev(np.eye(classes, dtype=np.float32)[rng.integers(0, classes, n)])

    def run(overlap):
        np.random.seed(7)
        model = pd.Model(tensor_format=fmt, batch_size=n, enable_backward_overlap=overlap, enable_conv_gemm=conv_gemm)
        model._overlap_min_elements = 0      # problems this small would otherwise stay on one stream
        model.add(pd.Input(shape=(hw, hw, 3)))
        model.add(pd.Conv2D(nfilters=c1, filter_shape=(3, 3), padding=1, activation="relu", weights_initializer="he_normal"))
        model.add(pd.AdditionBlock([pd.Conv2D(nfilters=c1, filter_shape=(3, 3), padding=1, weights_initializer="he_normal"),
                                    pd.BatchNormalization(), pd.Relu(),
                                    pd.Conv2D(nfilters=c1, filter_shape=(1, 1), weights_initializer="he_normal")], []))
        model.add(pd.Relu())
        model.add(pd.Conv2D(nfilters=c1 + 4, filter_shape=(3, 3), padding=1, stride=2, activation="relu",
                            weights_initializer="he_normal"))
        model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
        model.add(pd.Flatten())
        model.add(pd.FC(shape=(32,), activation="relu", weights_initializer="he_normal"))
        model.add(pd.FC(shape=(classes,), activation="softmax", weights_initializer="he_normal"))
        loss_fn, opt = pd.CategoricalCrossEntropy(), pd.SGD(learning_rate=0.05, momentum=0.9)
        losses = []
        for _ in range(8):     # long enough for the caching allocator to hand freed blocks out again
            losses.append(model.train_batch(x, y_targ, loss_fn, opt))    # no synchronization between the steps
            assert not model._side_used
        losses = [float(v) for v in losses]
        state = {}
        for l in model.get_all_layers():
            for var, grad in l.grad_vars.items():
                state[f"{l.id}.{var}"] = getattr(l, var).clone()
                state[f"{l.id}.{grad}"] = getattr(l, grad).clone()
        return losses, state, model._side_launches > 0

    losses_a, state_a, used_a = run(True)
    losses_b, state_b, used_b = run(False)
    assert used_a and not used_b
    assert losses_a == losses_b and len(state_a) >= 12
    assert state_a.keys() == state_b.keys()
    for k in state_a:
        assert torch.equal(state_a[k], state_b[k]), k


def test_backward_overlap_stays_inside_the_training_step(pd):
    """A layer's backward called by hand enqueues everything on the caller's stream."""
    model = pd.Model(tensor_format="NCHW", batch_size=2)
    assert model.enable_backward_overlap
    model.add(pd.Input(shape=(6, 6, 2)))
    model.add(pd.Conv2D(nfilters=3, filter_shape=(3, 3), padding=1))
    model.add(pd.Conv2D(nfilters=3, filter_shape=(3, 3), padding=1))
    model.mode = pd.TRAIN_MODE
    conv = model.layers[2]
    model._overlap_min_elements = 0
    conv.forward(torch.randn(2, 3, 6, 6, device="cuda"))
    conv.backward(torch.randn(2, 3, 6, 6, device="cuda"))
    assert model._side_launches == 0 and not model._side_used


def test_relu_folding_stays_inside_the_training_step(pd):
    """Outside train_batch a convolution's forward returns conv(x) + b as the reference's does, whatever follows
    it in the model; and the hand-over is recognised by tensor identity: a Relu given any other tensor
    computes normally and drops it."""
    model = pd.Model(tensor_format="NCHW", batch_size=2)
    assert model.enable_relu_folding
    model.add(pd.Input(shape=(6, 6, 2)))
    model.add(pd.Conv2D(nfilters=3, filter_shape=(3, 3), padding=1, activation="relu"))
    model.mode = pd.TRAIN_MODE
    conv, relu = model.layers[1], model.layers[2]
    assert conv.relu_above is relu
    x = torch.randn(2, 2, 6, 6, device="cuda")
    y_plain = conv.forward(x)                                      # by hand: not rectified, nothing handed over
    assert bool((y_plain < 0).any()) and relu._folded is None
    model.stepping = True                                          # as train_batch's loop sets it
    try:
        y = conv.forward(x)                                        # hands (y, mask) to relu
    finally:
        model.stepping = False
    assert torch.equal(y, torch.clamp(y_plain, min=0)) and relu._folded is not None
    other = torch.randn(2, 3, 6, 6, device="cuda")
    out = relu.forward(other)                                      # ... which must not use it for `other`
    assert torch.equal(out, torch.clamp(other, min=0)) and torch.equal(relu.mask, (other > 0).to(torch.int8))
    assert relu.forward(y) is not y                                # the hand-over was dropped, not kept


# ------------------------------------------------------------------ BatchNormalization in training mode

@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_batch_normalization_training_layer(pd, oracle, fmt):
    """Forward / backward of the layer in TRAIN_MODE against the restated reference branch, then an
    EVALUATE_MODE forward that must use the running statistics the training step has just updated
    (pydtnn/backends/cpu/layers/batch_normalization_cpu.py:59-82, :92-96, :108-129)."""
    announce("bn layer training", fmt)
    rng = np.random.default_rng(5)
    n, c, h, w = 6, 10, 7, 9
    shape = (n, c, h, w) if fmt == "NCHW" else (n, h, w, c)
    x = (rng.standard_normal(shape) * 3 - 1).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    model = pd.Model(tensor_format=fmt, batch_size=n)
    model.mode = pd.TRAIN_MODE
    bn = pd.BatchNormalization(moving_variance_initializer="ones")
    bn.set_model(model)
    bn.initialize(prev_shape=shape[1:])
    bn.gamma = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
    bn.beta = dev(rng.standard_normal(c).astype(np.float32))
    gamma, beta = host(bn.gamma), host(bn.beta)
    rm0, rv0 = host(bn.running_mean).copy(), host(bn.running_var).copy()
    y = bn.forward(dev(x))
    dx = bn.backward(dev(dy))
    y_ref, xn_ref, std_ref, rm_ref, rv_ref = oracle.bn_training_forward(x, gamma, beta, rm0, rv0, bn.momentum,
                                                                        bn.epsilon, tensor_format=fmt)
    dgamma_ref, dbeta_ref, dx_ref = oracle.bn_training_backward(dy, xn_ref, std_ref, gamma, tensor_format=fmt)
    assert_close(host(y), y_ref, tol=1e-5, what="y")
    assert_close(host(dx), dx_ref, tol=5e-5, what="dx")
    assert_close(host(bn.dgamma), dgamma_ref, tol=1e-5, what="dgamma")
    assert_close(host(bn.dbeta), dbeta_ref, tol=1e-5, what="dbeta")
    assert_close(host(bn.running_mean), rm_ref, tol=1e-5, what="running mean")
    assert_close(host(bn.running_var), rv_ref, tol=1e-5, what="running var")
    model.mode = pd.EVALUATE_MODE
    y_eval = bn.forward(dev(x))
    inv_std = (1.0 / np.sqrt(rv_ref + np.float32(bn.epsilon))).astype(np.float32)
    if fmt == "NCHW":
        ref = oracle.bn_inference_nchw(x, rm_ref.astype(np.float32), inv_std, gamma, beta)
    else:
        ref = oracle.bn_inference(x.reshape(-1, c), rm_ref.astype(np.float32), inv_std, gamma, beta).reshape(shape)
    assert_close(host(y_eval), ref, tol=1e-5, what="y in evaluate mode")


def test_store_and_load_weights_use_the_reference_key_names(pd, tmp_path):
    """pydtnn/model.py:351-387: ``{id}_{Name}_{variable}`` keys, BatchNormalization adds its running statistics."""
    announce("weights file")
    def build():
        model = pd.Model(tensor_format="NHWC", batch_size=2)
        model.add(pd.Input(shape=(8, 8, 3)))
        model.add(pd.Conv2D(nfilters=4, filter_shape=(3, 3), padding=1))
        model.add(pd.BatchNormalization())
        model.add(pd.Relu())
        model.add(pd.AdditionBlock([pd.Conv2D(nfilters=4, filter_shape=(1, 1))], []))
        model.add(pd.Flatten())
        model.add(pd.FC(shape=(5,)))
        return model
    np.random.seed(1)
    a = build()
    a.layers[2].running_mean = dev(np.arange(4, dtype=np.float32))
    path = str(tmp_path / "weights.npz")
    a.store_weights_and_bias(path)
    stored = np.load(path)
    names = sorted(stored.files)
    convs = [l for l in a.get_all_layers() if l.canonical_name == "Conv2D"]
    bn = a.layers[2]
    assert f"{convs[0].id}_Conv2D_weights" in names and f"{convs[0].id}_Conv2D_biases" in names
    assert f"{convs[1].id}_Conv2D_weights" in names                      # inside the AdditionBlock's path
    for key in ("beta", "gamma", "running_mean", "running_var"):
        assert f"{bn.id}_BatchNormalization_{key}" in names
    assert stored[f"{convs[0].id}_Conv2D_weights"].shape == (3, 3, 3, 4)  # NHWC layout (ci, kh, kw, co) as in memory
    np.random.seed(2)
    b = build()
    assert not np.array_equal(host(b.layers[1].weights), host(a.layers[1].weights))
    b.load_weights_and_bias(path)
    for la, lb in zip(a.get_all_layers(), b.get_all_layers()):
        for key in list(la.grad_vars) + (["running_mean", "running_var"] if la.canonical_name == "BatchNormalization" else []):
            assert np.array_equal(host(getattr(la, key)), host(getattr(lb, key))), (la, key)
    assert b.layers[2].updated_running_var
    x = dev(np.random.default_rng(0).standard_normal((2, 8, 8, 3)).astype(np.float32))
    assert np.array_equal(host(a.evaluate_batch(x)), host(b.evaluate_batch(x)))


# ------------------------------------------------------------------ committed known answers

@pytest.mark.parametrize("variant", ["i2c", "cg"])
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_committed_hand_cases_through_the_layer(pd, hand_cases, fmt, variant):
    """Every conv variant against tests/golden/reference_hand_cases.json: small integers, so the GPU result
    must be exact."""
    for case in hand_cases:
        announce("hand case", fmt, variant, case["name"])
        x, w = case["x"], case["w"]
        d = D(x.shape[0], x.shape[1], x.shape[2], x.shape[3], w.shape[0], w.shape[2], w.shape[3],
              case["vpadding"], case["hpadding"], case["vstride"], case["hstride"], case["vdilation"],
              case["hdilation"])
        model, layer = make_conv(pd, d, fmt, variant, use_bias=False)
        model.mode = pd.EVALUATE_MODE
        if fmt == "NCHW":
            layer.weights = dev(w)
            y = host(layer.forward(dev(x)))
        else:
            layer.weights = dev(np.ascontiguousarray(w.transpose(1, 2, 3, 0)))
            y = host(layer.forward(dev(nhwc(x)))).transpose(0, 3, 1, 2)
        assert np.array_equal(y, case["y"]), (case["name"], y, case["y"])


# ------------------------------------------------------------------ BestOf variant

@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_best_of_variant_races_the_two_routes_and_keeps_the_numbers(pd, oracle, fmt):
    """enable_best_of: Conv2D.forward / backward go through BestOf (pydtnn/backends/cpu/layers/conv_2d_cpu.py:95-130,
    :251-262); whichever route is being tried, y / dw / dx must match the oracle, and after the rounds one route
    is chosen for the layer's problem size."""
    announce("best_of", fmt)
    d = D(4, 6, 14, 13, 10, 3, 3, 1, 1, 1, 1)
    x, w, b, dy = (None,) * 4
    rng = np.random.default_rng(8)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(np.float32)
    w = (rng.standard_normal((d.kn, d.c, 3, 3)) * 0.2).astype(np.float32)
    b = rng.standard_normal(d.kn).astype(np.float32)
    dy = rng.standard_normal((d.b, d.kn, d.ho, d.wo)).astype(np.float32)
    model = pd.Model(tensor_format=fmt, batch_size=d.b, enable_best_of=True)
    try:
        model.mode = pd.TRAIN_MODE
        layer = pd.Conv2D(nfilters=d.kn, filter_shape=(3, 3), padding=1)
        layer.set_model(model)
        layer.initialize(prev_shape=(d.c, d.h, d.w) if fmt == "NCHW" else (d.h, d.w, d.c))
        assert layer.forward.__name__ == f"_forward_{fmt.lower()}_best_of"
        p = oracle.ConvParams(3, 3, 1, 1)
        if fmt == "NCHW":
            xin, win, dyin = x, w, dy
            y_ref, cols = oracle.conv2d_forward_nchw_i2c(x, w, b, p)
            dw_ref, db_ref, dx_ref = oracle.conv2d_backward_nchw_i2c(dy, cols, w, x.shape, p)
        else:
            xin, win, dyin = nhwc(x), np.ascontiguousarray(w.transpose(1, 2, 3, 0)), nhwc(dy)
            y_ref, rows = oracle.conv2d_forward_nhwc_i2c(xin, win, b, p)
            dw_ref, db_ref, dx_ref = oracle.conv2d_backward_nhwc_i2c(dyin, rows, win, xin.shape, p)
        layer.weights, layer.biases = dev(win), dev(b)
        pipeline = layer._best_fw_bw_pipeline
        for step in range(pipeline.total_rounds * 2 + 2):
            y = layer.forward(dev(xin))
            dx = layer.backward(dev(dyin))
            assert_close(host(y), y_ref, what=f"y step {step}")
            assert_close(host(layer.dw), dw_ref, what=f"dw step {step}")
            assert_close(host(dx), dx_ref, what=f"dx step {step}")
        assert pipeline.best_method_has_been_found(layer, None)
        assert list(pipeline.best_name.values())[0] in ("i2c", "cg")
        model.mode = pd.EVALUATE_MODE
        for _ in range(layer._best_fw.total_rounds * 2 + 1):
            assert_close(host(layer.forward(dev(xin))), y_ref, what="y eval")
        assert layer._best_fw.best_method_has_been_found(layer, None)
    finally:
        pd.BestOf.use_always_the_first_alternative(True)


# ------------------------------------------------------------------ tracers on a real model

def test_tracers_see_layers_and_operations_of_a_training_step(pd, tmp_path):
    """SimpleTracer on a small model: one Model event per layer and direction, the convolution's operation
    events inside them; RoctxTracer pushes and pops the same regions without error."""
    announce("tracers")
    t = pd.tracers
    model = pd.Model(tensor_format="NCHW", batch_size=2)
    model.add(pd.Input(shape=(8, 8, 3)))                      # (h, w, c), encoded into the model's format
    model.add(pd.Conv2D(nfilters=4, filter_shape=(3, 3), padding=1, activation="relu"))
    model.add(pd.Conv2D(nfilters=4, filter_shape=(3, 3), padding=1))
    model.add(pd.Flatten())
    model.add(pd.FC(shape=(5,), activation="softmax"))
    tracer = t.SimpleTracer(True, str(tmp_path / "trace.csv"))
    model.set_tracer(tracer)
    x = dev(np.random.default_rng(0).standard_normal((2, 3, 8, 8)).astype(np.float32))
    y = dev(np.eye(5, dtype=np.float32)[[1, 3]])
    for _ in range(2):
        model.train_batch(x, y, pd.CategoricalCrossEntropy(), pd.SGD(0.01, 0.9))
    assert not tracer.pending_events
    conv2 = model.layers[3]
    assert conv2.canonical_name == "Conv2D" and conv2.need_dx
    mdl, ops_ = tracer.events[t.PYDTNN_MDL_EVENT], tracer.events[t.PYDTNN_OPS_EVENT]
    for layer in model.layers[1:]:
        assert mdl[layer.id * t.PYDTNN_MDL_EVENTS + t.PYDTNN_MDL_FORWARD][0] == 2
        assert mdl[layer.id * t.PYDTNN_MDL_EVENTS + t.PYDTNN_MDL_BACKWARD][0] == 2
    for kind in (t.PYDTNN_OPS_FORWARD_CONVGEMM, t.PYDTNN_OPS_BACKWARD_CONVGEMM, t.PYDTNN_OPS_BACKWARD_SUM_BIASES,
                 t.PYDTNN_OPS_BACKWARD_DECONV_GEMM):
        assert ops_[conv2.id * t.PYDTNN_OPS_EVENTS + kind][0] == 2
    first = model.layers[1]                                   # no dx for the first layer
    assert first.id * t.PYDTNN_OPS_EVENTS + t.PYDTNN_OPS_BACKWARD_DECONV_GEMM not in ops_
    tracer.write_output()
    text = (tmp_path / "trace.csv").read_text()
    assert f"{conv2.canonical_name_with_id}_forward" in text and "_Conv2D_backward_convgemm" in text
    model.set_tracer(t.RoctxTracer(True))
    model.train_batch(x, y, pd.CategoricalCrossEntropy(), pd.SGD(0.01, 0.9))
    assert not model.tracer._open


# ------------------------------------------------------------------ the call a layer prepares for inference
@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("d", [D(64, 1, 28, 28, 32, 3, 3, 1, 1, 1, 1), D(4, 16, 20, 20, 40, 3, 3, 1, 1, 1, 1),
                               D(3, 8, 17, 17, 12, 3, 3, 1, 1, 2, 2), D(16, 64, 56, 56, 64, 1, 1, 0, 0, 1, 1)], ids=repr)
def test_evaluate_mode_forward_uses_a_prepared_call_with_the_same_bits(pd, oracle, fmt, d):
    """In EVALUATE_MODE a cg convolution goes through a call prepared once (geometry, filter, bias, BN vectors bound in
    the library's plan).  It must give the bits of the ConvGemm shim's call with all arguments, agree with the
    oracle, notice tensors that were replaced or a new batch size, follow in-place updates, and keep its output
    tensor between steps only under Model(enable_memory_cache=True)
    (pydtnn/backends/gpu/layers/conv_2d_gpu.py:89-96 keeps it always)."""
    announce("prepared forward", fmt, d)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((d.b, d.c, d.h, d.w)).astype(np.float32)
    w = (rng.standard_normal((d.kn, d.c, d.kh, d.kw)) * 0.2).astype(np.float32)
    b = rng.standard_normal(d.kn).astype(np.float32)
    p = oracle.ConvParams(*d.geom())
    if fmt == "NCHW":
        xs, ws = dev(x), dev(w)
        ref = lambda w_, b_: oracle.conv2d_forward_nchw_i2c(x, w_, b_, p)[0]
    else:
        xs, ws = dev(nhwc(x)), dev(np.ascontiguousarray(w.transpose(1, 2, 3, 0)))
        ref = lambda w_, b_: nhwc(oracle.conv2d_forward_nchw_i2c(x, w_, b_, p)[0])
    for keep in (False, True):
        model = pd.Model(tensor_format=fmt, batch_size=d.b, enable_memory_cache=keep)
        model.mode = pd.EVALUATE_MODE
        conv = pd.Conv2D(nfilters=d.kn, filter_shape=(d.kh, d.kw), padding=(d.vpadding, d.hpadding),
                         stride=(d.vstride, d.hstride), dilation=(d.vdilation, d.hdilation))
        conv.set_model(model)
        conv.initialize(prev_shape=(d.c, d.h, d.w) if fmt == "NCHW" else (d.h, d.w, d.c))
        conv.weights, conv.biases = ws.clone(), dev(b)
        shim = conv.cg.conv_gemm_nchw if fmt == "NCHW" else conv.cg.conv_gemm_nhwc
        y1 = conv.forward(xs)
        plan = conv._prepared
        assert plan is not None
        assert torch.equal(y1, shim(conv.weights, xs, biases_vector=conv.biases, **conv._cg_kwargs()))
        assert_close(host(y1), ref(w, b), what="prepared forward")
        y2 = conv.forward(xs)
        assert conv._prepared is plan and (y2 is y1) == keep and torch.equal(y2, y1)
        # an update in place is seen by the same plan ...
        conv.weights.mul_(0.5)
        assert_close(host(conv.forward(xs)), ref(w * np.float32(0.5), b), what="after an in-place update")
        assert conv._prepared is plan
        # ... replaced tensors and another batch size make a new one
        conv.biases = dev(b + 1)
        assert_close(host(conv.forward(xs)), ref(w * np.float32(0.5), b + 1), what="after replacing the bias")
        assert conv._prepared is not plan
        half = conv.forward(xs[: max(1, d.b // 2)].contiguous())
        assert half.shape[0] == max(1, d.b // 2)
        # (another batch size may take another launch form: same values, not necessarily the same bits)
        assert_close(host(half), host(conv.forward(xs)[: max(1, d.b // 2)]), what="half the batch")
        with pytest.raises(ValueError):
            conv._prepared(xs.double())
    # the fused inference layers bind their BN vectors and the ReLU as well
    model = pd.Model(tensor_format=fmt, batch_size=d.b, enable_fused_conv_bn_relu=True)
    model.add(pd.Input(shape=(d.h, d.w, d.c)))
    model.add(pd.Conv2D(nfilters=d.kn, filter_shape=(d.kh, d.kw), padding=(d.vpadding, d.hpadding),
                        stride=(d.vstride, d.hstride), dilation=(d.vdilation, d.hdilation)))
    model.add(pd.BatchNormalization())
    model.add(pd.Relu())
    conv, bn = model.layers[1], model.layers[2]
    conv.weights, conv.biases = ws.clone(), dev(b)
    stats = [rng.uniform(0.5, 1.5, d.kn).astype(np.float32) for _ in range(4)]
    bn.running_mean, bn.running_var, bn.gamma, bn.beta = (dev(v) for v in stats)
    bn.updated_running_var = True
    y = model.evaluate_dataset_batch(xs)
    fused = model.layers[1]
    assert type(fused).__name__ == "Conv2DBatchNormalizationRelu" and fused._prepared is not None
    inv_std = (1.0 / np.sqrt(stats[1] + np.float32(bn.epsilon))).astype(np.float32)
    plain = oracle.conv2d_forward_nchw_i2c(x, w, b, p)[0]
    want = oracle.fused_epilogue(plain, "NCHW", bn=[stats[0], inv_std, stats[2], stats[3]], relu_flag=True)
    assert_close(host(y), want if fmt == "NCHW" else nhwc(want), what="fused layer through its prepared call")

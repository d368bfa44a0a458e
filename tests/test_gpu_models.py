"""GPU tests of whole models: ResNet-50 inference through addition blocks and the fusion pass, the weights
file (key names of block models, files written in the other tensor format) and AveragePool2D.

A model is checked layer by layer, the oracle fed the GPU's own input of each top-level layer (the pattern of
pydtnn/tests/check_conv_gemm_models.py:100-167); an addition block is evaluated whole by the oracle.
"""
import numpy as np
import pytest
import torch

from gpu_util import FP32_REL_TOL, announce, assert_close, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pd():
    import pydtnn_amd
    from pydtnn_amd import native
    native.lib()
    return pydtnn_amd


def oracle_forward(oracle, layer, x, fmt):
    """What the reference's CPU layers make of ``x`` (inference), restated with the oracle's functions."""
    name = layer.canonical_name
    if name == "Conv2D":
        p = oracle.ConvParams(layer.kh, layer.kw, layer.vpadding, layer.hpadding, layer.vstride, layer.hstride,
                              layer.vdilation, layer.hdilation)
        fwd = oracle.conv2d_forward_nchw_i2c if fmt == "NCHW" else oracle.conv2d_forward_nhwc_i2c
        return fwd(x, host(layer.weights), host(layer.biases) if layer.use_bias else None, p)[0]
    if name == "BatchNormalization":
        var = host(layer.running_var)
        inv_std = (1.0 / np.sqrt(var + var.dtype.type(layer.epsilon))).astype(var.dtype)
        return oracle.fused_epilogue(x, fmt if x.ndim == 4 else "NHWC",
                                     bn=(host(layer.running_mean), inv_std, host(layer.gamma), host(layer.beta)))
    if name == "Relu":
        return oracle.relu(x)[0]
    if name == "MaxPool2D":
        fwd = oracle.max_pool_2d_fwd_nchw if fmt == "NCHW" else oracle.max_pool_2d_fwd_nhwc
        return fwd(x, layer.kh, layer.kw, layer.vpadding, layer.hpadding, layer.vstride, layer.hstride)[0]
    if name == "AveragePool2D":
        return oracle.average_pool_2d_fwd(x, fmt, layer.kh, layer.kw, layer.vpadding, layer.hpadding, layer.vstride,
                                          layer.hstride)
    if name == "Flatten":
        return x.reshape(x.shape[0], -1)
    if name == "FC":
        return oracle.fc_forward(x, host(layer.weights), host(layer.biases))
    if name == "Softmax":
        return oracle.softmax_forward(x)
    if name == "AdditionBlock":
        outs = []
        for path in layer.paths:
            cur = x
            for sub in path:
                cur = oracle_forward(oracle, sub, cur, fmt)
            outs.append(np.array(cur, copy=True))
        for other in outs[1:]:
            outs[0] = oracle.eltw_sum(outs[0], other)
        return outs[0]
    raise AssertionError(f"no oracle for {name}")


def randomize(model, seed):
    """Weights at their initial scale, non-trivial biases and BatchNormalization statistics."""
    rng = np.random.default_rng(seed)
    for layer in model.get_all_layers():
        if layer.canonical_name in ("Conv2D", "FC"):
            layer.biases = dev(rng.normal(0, 0.05, tuple(layer.biases.shape)).astype(np.float32))
        elif layer.canonical_name == "BatchNormalization":
            c = layer.gamma.numel()
            layer.gamma = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
            layer.beta = dev(rng.normal(0, 0.1, c).astype(np.float32))
            layer.running_mean = dev(rng.normal(0, 0.1, c).astype(np.float32))
            layer.running_var = dev(rng.uniform(0.5, 1.5, c).astype(np.float32))
            layer.updated_running_var = True


POOL_GEOMS = [(2, 3, 8, 10, 2, 2, 0, 0, 2, 2, 1, 1), (2, 4, 9, 9, 3, 3, 1, 1, 2, 2, 1, 1),
              (1, 5, 7, 11, 3, 2, 1, 0, 1, 2, 1, 1), (2, 3, 12, 12, 3, 3, 1, 1, 1, 1, 1, 1),
              (1, 2, 9, 9, 2, 2, 1, 1, 1, 1, 2, 2), (4, 64, 7, 7, 7, 7, 0, 0, 1, 1, 1, 1)]


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("geom", POOL_GEOMS, ids=str)
def test_average_pool_equals_the_oracle_bit_for_bit(pd, oracle, fmt, geom):
    from pydtnn_amd import ops
    n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh = geom
    announce("average pool", fmt, geom)
    rng = np.random.default_rng(31)
    nhwc = fmt == "NHWC"
    x = rng.standard_normal((n, h, w, c) if nhwc else (n, c, h, w)).astype(np.float32)
    y_ref = oracle.average_pool_2d_fwd(x, fmt, kh, kw, pv, ph, sv, sh, dv, dh)
    y = ops.average_pool_2d_fwd(dev(x), nhwc, kh, kw, pv, ph, sv, sh, dv, dh)
    assert np.array_equal(host(y), y_ref)
    dy = rng.standard_normal(y_ref.shape).astype(np.float32)
    dx_ref = oracle.average_pool_2d_bwd(dy, fmt, n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh)
    dx = ops.average_pool_2d_bwd(dev(dy), nhwc, n, c, h, w, kh, kw, pv, ph, sv, sh, dv, dh)
    assert np.array_equal(host(dx), dx_ref)


def test_block_model_keys_follow_the_reference_numbering(pd, tmp_path):
    """pydtnn/model.py:268-283 hands out ids in the order layers are added: a layer, then the activation its
    ``activation=`` argument names; a block layer takes an id and then, while it initialises, so do the layers
    of its paths, path by path (pydtnn/layers/abstract_block_layer.py:35-37).  Keys are
    ``{id}_{class name}_{variable}`` (pydtnn/model.py:351-377).  The list below is derived by hand from those
    rules for this model; nothing in it comes from running the code under test."""
    announce("weights file keys")
    model = pd.Model(tensor_format="NHWC")
    model.add(pd.Input(shape=(8, 8, 3)))                                             # 0
    model.add(pd.Conv2D(nfilters=4, filter_shape=(3, 3), padding=1, activation="relu"))  # 1, its Relu 2
    model.add(pd.AdditionBlock(                                                      # 3
        [pd.Conv2D(nfilters=4, filter_shape=(1, 1)), pd.BatchNormalization(), pd.Relu(),       # 4 5 6
         pd.Conv2D(nfilters=4, filter_shape=(3, 3), padding=1, use_bias=False), pd.BatchNormalization()],  # 7 8
        [pd.Conv2D(nfilters=4, filter_shape=(1, 1)), pd.BatchNormalization()]))                # 9 10
    model.add(pd.Relu())                                                             # 11
    model.add(pd.AveragePool2D(pool_shape=(0, 0)))                                   # 12
    model.add(pd.Flatten())                                                          # 13
    model.add(pd.FC(shape=(5,), activation="softmax"))                               # 14, its Softmax 15
    expected = {"1_Conv2D_weights", "1_Conv2D_biases",
                "4_Conv2D_weights", "4_Conv2D_biases",
                "5_BatchNormalization_beta", "5_BatchNormalization_gamma",
                "5_BatchNormalization_running_var", "5_BatchNormalization_running_mean",
                "7_Conv2D_weights",
                "8_BatchNormalization_beta", "8_BatchNormalization_gamma",
                "8_BatchNormalization_running_var", "8_BatchNormalization_running_mean",
                "9_Conv2D_weights", "9_Conv2D_biases",
                "10_BatchNormalization_beta", "10_BatchNormalization_gamma",
                "10_BatchNormalization_running_var", "10_BatchNormalization_running_mean",
                "14_FC_weights", "14_FC_biases"}
    assert [l.id for l in model.get_all_layers()] == list(range(16))
    path = str(tmp_path / "w.npz")
    model.store_weights_and_bias(path)
    d = np.load(path)
    assert set(d.files) == expected
    # in-memory layout of the model's format: NHWC filters are (ci, kh, kw, co), FC weights (in, out)
    assert d["1_Conv2D_weights"].shape == (3, 3, 3, 4) and d["7_Conv2D_weights"].shape == (4, 3, 3, 4)
    assert d["14_FC_weights"].shape == (4, 5) and d["5_BatchNormalization_running_var"].shape == (4,)


def small_resnet(pd, fmt, **flags):
    model = pd.Model(tensor_format=fmt, **flags)
    pd.models.create_resnet50_imagenet(model, stages=((8, 2, 1), (16, 1, 2)), classes=10, input_shape=(32, 32, 3))
    return model


@pytest.mark.parametrize("src,dst", [("NHWC", "NCHW"), ("NCHW", "NHWC")])
def test_weights_file_written_in_the_other_tensor_format_loads(pd, tmp_path, src, dst):
    """A file stores arrays in its writer's layout (pydtnn/model.py:351-377).  Loading it into a model of the
    other format transposes filters as pydtnn/tests/check_tensor_format_models.py:70-71 does and reorders the
    rows of an FC layer behind a Flatten; the two models then compute the same function."""
    announce("cross-format weights", src, dst)
    rng = np.random.default_rng(41)

    def vgg_like(fmt):
        model = pd.Model(tensor_format=fmt)
        model.add(pd.Input(shape=(12, 12, 3)))
        model.add(pd.Conv2D(nfilters=6, filter_shape=(3, 3), padding=1, activation="relu"))
        model.add(pd.MaxPool2D(pool_shape=(2, 2), stride=2))
        model.add(pd.Conv2D(nfilters=5, filter_shape=(3, 3), padding=1, activation="relu"))
        model.add(pd.Flatten())                       # 6x6x5 image: row order differs between the formats
        model.add(pd.FC(shape=(7,), activation="softmax"))
        return model

    for build in (vgg_like, lambda fmt: small_resnet(pd, fmt)):
        a, b = build(src), build(dst)
        randomize(a, 42)
        path = str(tmp_path / f"{src}.npz")
        a.store_weights_and_bias(path)
        b.load_weights_and_bias(path)
        hw = a.layers[0].shape[1] if src == "NCHW" else a.layers[0].shape[0]
        x = rng.standard_normal((3, hw, hw, 3)).astype(np.float32)     # NHWC on the host
        feed = lambda fmt: dev(x if fmt == "NHWC" else np.ascontiguousarray(x.transpose(0, 3, 1, 2)))
        ya, yb = a.evaluate_batch(feed(src)), b.evaluate_batch(feed(dst))
        assert_close(host(yb), host(ya), tol=1e-5, what=f"{src} file in a {dst} model")


@pytest.mark.parametrize("fmt", ["NHWC", "NCHW"])
def test_resnet50_inference_layer_by_layer_and_fused(pd, oracle, fmt):
    """ResNet-50 (pydtnn/models/resnet50_imagenet.py) at 224x224, batch 2: every top-level layer against the
    oracle on the GPU's own input, then the same weights through the fusion pass (Conv2D+BN(+ReLU) layers,
    block sums done by the last convolution's store) against the unfused result."""
    announce("resnet50", fmt)
    np.random.seed(7)
    n = 2
    plain = pd.Model(tensor_format=fmt, batch_size=n)
    pd.models.create_resnet50_imagenet(plain)
    # parameters counted from the architecture: every convolution has a bias and is followed by a
    # BatchNormalization with gamma, beta and the two running statistics, except the stem (no BN)
    def conv_bn(ci, co, k, bn=True):
        return ci * co * k * k + co + (4 * co if bn else 0)
    count, cin = conv_bn(3, 64, 7, bn=False), 64
    for f, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for i in range(blocks):
            count += conv_bn(cin, f, 1) + conv_bn(f, f, 3) + conv_bn(f, 4 * f, 1)
            count += conv_bn(cin, 4 * f, 1) if i == 0 else 0
            cin = 4 * f
    count += 2048 * 1000 + 1000
    assert plain.nparams == count and sum(l.canonical_name == "Conv2D" for l in plain.get_all_layers()) == 53
    randomize(plain, 8)
    rng = np.random.default_rng(9)
    x = rng.random((n, 224, 224, 3), dtype=np.float32)
    x = x if fmt == "NHWC" else np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    plain.mode = pd.EVALUATE_MODE
    cur = dev(x)
    for layer in plain.layers[1:]:
        out = layer.forward(cur)
        ref = oracle_forward(oracle, layer, host(cur), fmt)
        assert_close(host(out), ref, what=f"{fmt} {layer}")
        cur = out
    y_plain = cur
    assert abs(float(y_plain.sum()) - n) < 1e-3     # softmax rows
    fused = pd.Model(tensor_format=fmt, batch_size=n, enable_fused_conv_bn_relu=True, enable_fused_conv_bn=True)
    np.random.seed(7)
    pd.models.create_resnet50_imagenet(fused)
    for a, b in zip(plain.get_all_layers(), fused.get_all_layers()):
        for key in list(a.grad_vars) + ["running_mean", "running_var"]:
            if getattr(a, key, None) is not None:
                setattr(b, key, getattr(a, key))
        b.updated_running_var = True
    y_fused = fused.evaluate_dataset_batch(dev(x))
    names = [l.canonical_name for l in fused.get_all_layers()]
    assert names.count("Conv2DBatchNormalizationRelu") == 32 and names.count("Conv2DBatchNormalization") == 20
    assert all(b.relu_above is not None and b._folded_sum_path() == 0
               for b in fused.layers if b.canonical_name == "AdditionBlock")
    assert_close(host(y_fused), host(y_plain), tol=1e-5, what="fused vs plain")

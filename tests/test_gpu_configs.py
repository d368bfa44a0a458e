"""GPU parity at the benchmark's configurations.

cfg1, cfg3 and cfg4 are small enough for the CPU oracle to run whole, at the benchmark's batch of 64 (tile
and launch choices depend on the problem size).  At cfg2's full size the
outputs are checked by *sampled direct convolution in float64*: a few thousand randomly chosen
elements of y, dw and dx are recomputed from their defining sums, which needs no column matrix and
is independent of the kernels' tiling.  A VGG16 model (batch 8) is checked layer by layer with the
oracle fed the GPU's own activations, the pattern of pydtnn/tests/check_conv_gemm_models.py:100-167.
"""
import numpy as np
import pytest
import torch

import bench
import bench_configs
from gpu_util import FP32_REL_TOL, announce, assert_close, dev, host, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pd():
    import pydtnn_amd
    from pydtnn_amd import native
    native.lib()
    return pydtnn_amd


def test_cfg1_mnist_layer_nhwc(pd, oracle):
    announce("cfg1")
    x, w, b = bench_configs.make_cfg1()
    y = pd.ConvGemm().conv_gemm_nhwc(dev(w), dev(x), biases_vector=dev(b), vpadding=1, hpadding=1)
    ref, _ = oracle.conv2d_forward_nhwc_i2c(x, w, b, oracle.ConvParams(3, 3, 1, 1))
    assert_close(host(y), ref, what="cfg1 y")


def test_cfg3_alexnet_conv1_bias_relu(pd, oracle):
    announce("cfg3")
    x, w, b = bench_configs.make_cfg3(n=64)
    y = pd.ConvGemm().conv_gemm_nchw(dev(w), dev(x), biases_vector=dev(b), vstride=4, hstride=4, relu=True)
    assert tuple(y.shape) == (64, 96, 55, 55)
    ref, _ = oracle.conv2d_forward_nchw_i2c(x, w, b, oracle.ConvParams(11, 11, 0, 0, 4, 4))
    ref = oracle.fused_epilogue(ref, "NCHW", relu_flag=True)
    assert_close(host(y), ref, what="cfg3 y")
    assert (host(y) == 0).mean() > 0.1, "ReLU must have clipped part of the output"


def test_cfg4_resnet_bottleneck_fused_nhwc(pd, oracle):
    announce("cfg4")
    x, ws, bns = bench_configs.make_cfg4(n=64)
    model = bench_configs.build_cfg4_model(pd, torch, ws, bns, fused=True)
    y = model.evaluate_dataset_batch(dev(x))
    block = model.layers[1]
    assert [l.canonical_name for l in block.paths[0]] == \
        ["Conv2DBatchNormalizationRelu", "Conv2DBatchNormalizationRelu", "Conv2DBatchNormalization"]
    cur = x
    params = [oracle.ConvParams(1, 1), oracle.ConvParams(3, 3, 1, 1), oracle.ConvParams(1, 1)]
    for w, (gamma, beta, mean, var), p, relu in zip(ws, bns, params, (True, True, False)):
        cur, _ = oracle.conv2d_forward_nhwc_i2c(cur, w, np.zeros(w.shape[3], np.float32), p)
        inv_std = (1.0 / np.sqrt(var + np.float32(1e-5))).astype(np.float32)
        cur = oracle.fused_epilogue(cur, "NHWC", bn=(mean, inv_std, gamma, beta), relu_flag=relu)
    ref, _ = oracle.relu(oracle.eltw_sum(np.ascontiguousarray(cur), x))
    assert_close(host(y), ref, what="cfg4 out")


# ------------------------------------------------------------------ cfg2 at full size

def test_cfg2_full_size_sampled_direct_convolution(pd):
    announce("cfg2 full size")
    x, w, b, dy = bench.make_cfg2()
    b = np.random.default_rng(1).standard_normal(256).astype(np.float32)
    n, c, h, wd_ = x.shape
    model = pd.Model(tensor_format="NCHW", batch_size=n)
    model.mode = pd.TRAIN_MODE
    conv = pd.Conv2D(nfilters=256, filter_shape=(3, 3), padding=1)
    conv.set_model(model)
    conv.initialize(prev_shape=(256, 56, 56))
    conv.weights, conv.biases = dev(w), dev(b)
    y = host(conv.forward(dev(x)))
    dx = host(conv.backward(dev(dy)))
    dw, db = host(conv.dw), host(conv.db)
    rng = np.random.default_rng(2)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    dyp = np.pad(dy, ((0, 0), (0, 0), (1, 1), (1, 1)))
    s = 3000
    # y[n,co,oy,ox] = b[co] + sum_{c,i,j} w[co,c,i,j] x[n,c,oy+i-1,ox+j-1]
    ni, co, oy, ox = rng.integers(0, n, s), rng.integers(0, 256, s), rng.integers(0, 56, s), rng.integers(0, 56, s)
    patches = np.stack([xp[ni, :, oy + i, ox + j] for i in range(3) for j in range(3)], axis=-1)  # (s, c, 9)
    ref_y = np.einsum("sck,sck->s", patches.astype(np.float64), w[co].reshape(s, c, 9).astype(np.float64)) + b[co]
    scale = np.abs(y).max()
    assert np.max(np.abs(y[ni, co, oy, ox] - ref_y)) / scale <= FP32_REL_TOL
    # dx[n,c,y,x] = sum_{co,i,j} w[co,c,i,j] dy[n,co,y+1-i,x+1-j]
    cc = rng.integers(0, c, s)
    dpatch = np.stack([dyp[ni, :, oy + 2 - i, ox + 2 - j] for i in range(3) for j in range(3)], axis=-1)  # (s, co, 9)
    ref_dx = np.einsum("sok,sok->s", dpatch.astype(np.float64),
                       w[:, cc].transpose(1, 0, 2, 3).reshape(s, 256, 9).astype(np.float64))
    assert np.max(np.abs(dx[ni, cc, oy, ox] - ref_dx)) / np.abs(dx).max() <= FP32_REL_TOL
    # dw[co,c,i,j] = sum_{n,oy,ox} dy[n,co,oy,ox] x[n,c,oy+i-1,ox+j-1]
    for _ in range(24):
        o, ci, i, j = rng.integers(0, 256), rng.integers(0, c), rng.integers(0, 3), rng.integers(0, 3)
        ref = np.sum(dy[:, o].astype(np.float64) * xp[:, ci, i:i + 56, j:j + 56])
        assert abs(dw[o, ci, i, j] - ref) / np.abs(dw).max() <= FP32_REL_TOL
    assert_close(db, dy.astype(np.float64).sum(axis=(0, 2, 3)), tol=1e-5, what="db")
    # linearity of the forward map at full size: conv(x, 2w) + b == 2 (conv(x, w) + b) - b, exact in fp32
    conv.weights = dev(2 * w)
    model.mode = pd.EVALUATE_MODE
    y2 = host(conv.forward(dev(x)))
    assert np.array_equal(y2 - b[None, :, None, None], 2 * (y - b[None, :, None, None])) or \
        rel_err(y2 - b[None, :, None, None], 2 * (y - b[None, :, None, None])) < 1e-6


# ------------------------------------------------------------------ tensors beyond 2^29 floats

def test_tensors_beyond_the_per_launch_limit(pd):
    """x, y, dy and dx of 40 x 64 x 460 x 460 = 541.7 M floats each (2.17 GB) exceed what one launch can address, so
    the entry points run the batch as groups of images.  Checked by sampled direct convolution in float64."""
    announce("beyond 2^29 floats")
    n, c, hw, kn = 40, 64, 460, 64
    assert n * c * hw * hw > 2 ** 29
    gen = torch.Generator(device="cuda").manual_seed(3)
    xd = torch.randn((n, c, hw, hw), device="cuda", generator=gen)
    dyd = torch.randn((n, kn, hw, hw), device="cuda", generator=gen)
    w = (np.random.default_rng(4).standard_normal((kn, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(np.float32)
    wd = dev(w)
    cg = pd.ConvGemm()
    y = host(cg.conv_gemm_nchw(wd, xd, vpadding=1, hpadding=1))
    dwd = torch.empty_like(wd)
    cg.conv_gemm_nchw(dyd, xd, biases=dwd, trans=True, vpadding=1, hpadding=1)
    dxd = torch.empty_like(xd)
    cg.deconv_gemm_nchw(wd, dyd, dxd, vpadding=1, hpadding=1)
    x, dy, dw = host(xd), host(dyd), host(dwd)
    del xd, dyd
    rng = np.random.default_rng(5)
    s = 1500
    ni, oy, ox = rng.integers(0, n, s), rng.integers(0, hw, s), rng.integers(0, hw, s)
    ni[:8] = n - 1                     # the last image group
    co, cc = rng.integers(0, kn, s), rng.integers(0, c, s)

    def taps(t, ch_axis_len, flip):
        """(s, channels, 9) patches of t around (oy, ox), zero outside the image; flip mirrors the taps."""
        out = np.zeros((s, ch_axis_len, 9))
        for i in range(3):
            for j in range(3):
                yy, xx = (oy + 1 - i, ox + 1 - j) if flip else (oy + i - 1, ox + j - 1)
                ok = (yy >= 0) & (yy < hw) & (xx >= 0) & (xx < hw)
                out[ok, :, i * 3 + j] = t[ni[ok], :, yy[ok], xx[ok]]
        return out

    ref_y = np.einsum("sck,sck->s", taps(x, c, False), w[co].reshape(s, c, 9).astype(np.float64))
    assert np.max(np.abs(y[ni, co, oy, ox] - ref_y)) / np.abs(y).max() <= FP32_REL_TOL
    del y
    dx = host(dxd)
    del dxd
    ref_dx = np.einsum("sok,sok->s", taps(dy, kn, True), w[:, cc].transpose(1, 0, 2, 3).reshape(s, kn, 9).astype(np.float64))
    assert np.max(np.abs(dx[ni, cc, oy, ox] - ref_dx)) / np.abs(dx).max() <= FP32_REL_TOL
    del dx
    for _ in range(6):
        o, ci, i, j = rng.integers(0, kn), rng.integers(0, c), rng.integers(0, 3), rng.integers(0, 3)
        ys, ye = max(0, 1 - i), min(hw, hw + 1 - i)        # output rows whose tap (i, j) lies inside the image
        xs, xe = max(0, 1 - j), min(hw, hw + 1 - j)
        ref = np.sum(dy[:, o, ys:ye, xs:xe].astype(np.float64) * x[:, ci, ys + i - 1:ye + i - 1, xs + j - 1:xe + j - 1])
        assert abs(dw[o, ci, i, j] - ref) / np.abs(dw).max() <= FP32_REL_TOL


# ------------------------------------------------------------------ VGG16, layer by layer

def test_vgg16_step_layer_by_layer_against_oracle(pd, oracle):
    announce("vgg16 layerwise")
    n = 4
    np.random.seed(0)
    model = bench.build_vgg16(pd, n)
    assert model.nparams == 138357544
    rng = np.random.default_rng(0)
    x = rng.random((n, 3, 224, 224), dtype=np.float32)
    y_targ = np.eye(1000, dtype=np.float32)[rng.integers(0, 1000, n)]
    # forward / backward by hand so that every layer's input and upstream gradient can be captured
    model.mode = pd.TRAIN_MODE
    acts = [dev(x)]
    for layer in model.layers[1:]:
        acts.append(layer.forward(acts[-1]))
    loss, dcur = pd.CategoricalCrossEntropy()(acts[-1], dev(y_targ), n)
    grads = {}
    for idx in range(len(model.layers) - 1, 0, -1):
        grads[idx] = dcur
        dcur = model.layers[idx].backward(dcur)
        grads[(idx, "dx")] = dcur
    p3 = oracle.ConvParams(3, 3, 1, 1)
    checked = 0
    for idx, layer in enumerate(model.layers):
        name = layer.canonical_name
        if name not in ("Conv2D", "FC", "MaxPool2D", "Relu"):
            continue
        xin, dy = host(acts[idx - 1]), host(grads[idx])
        if name == "Conv2D":
            w, b = host(layer.weights), host(layer.biases)
            y_ref, cols = oracle.conv2d_forward_nchw_i2c(xin, w, b, p3)
            dw, db, dx = oracle.conv2d_backward_nchw_i2c(dy, cols, w, xin.shape, p3, need_dx=layer.need_dx)
            del cols
        elif name == "FC":
            w, b = host(layer.weights), host(layer.biases)
            y_ref = oracle.fc_forward(xin, w, b)
            dw, db, dx = oracle.fc_backward(dy, xin, w)
        elif name == "MaxPool2D":
            y_ref, idx_ref = oracle.max_pool_2d_fwd_nchw(xin, 2, 2, 0, 0, 2, 2)
            dx = oracle.max_pool_2d_bwd_nchw(dy, idx_ref, *xin.shape, 2, 2, 0, 0, 2, 2)
            dw = None
        else:
            y_ref, mask = oracle.relu(xin)
            dx = dy * mask
            dw = None
        assert_close(host(acts[idx]), y_ref, what=f"{layer} y")
        if dw is not None:
            assert_close(host(layer.dw), dw, what=f"{layer} dw")
            assert_close(host(layer.db), db, tol=1e-5, what=f"{layer} db")
        if layer.need_dx and dx is not None:
            got = host(grads[(idx, "dx")])
            if np.abs(dx).max() > 0:
                assert_close(got, dx, what=f"{layer} dx")
        checked += 1
    assert checked >= 13 + 3 + 5 + 15
    assert np.isfinite(float(loss))

"""``ConvGemm``: the reference's shim over libconvGemm, re-hosted on the MI355X library.

Same class name, method names, keyword arguments, shape asserts and return values as
pydtnn/backends/cpu/libs/conv_gemm.py:39-330, but operands are GPU tensors (``torch.Tensor`` on
``cuda``) and the call goes to the device-pointer C ABI.  The convolution is an implicit GEMM:
the im2col matrix never exists in memory.
"""
import torch

from . import native
from .native import check, f32, lib, ptr, stream_ptr

import ctypes

is_conv_gemm_available = True  # pydtnn/backends/cpu/libs/conv_gemm.py:32-36: probe result of load_library


class ConvGemm:
    """Exposes the implicit-GEMM convolution entry points following the PyDTNN conventions."""

    def __init__(self, dtype=torch.float32, debug=False, parent_layer=None):
        # pydtnn/backends/cpu/libs/conv_gemm.py:79-86 accepts a type or its name
        names = {"float32": torch.float32, "float64": torch.float64}
        if isinstance(dtype, str):
            if dtype not in names:
                raise AttributeError("dtype '{}' not recognized".format(dtype))
            dtype = names[dtype]
        elif not isinstance(dtype, torch.dtype):
            try:
                import numpy as np
                dtype = {np.dtype("float32"): torch.float32, np.dtype("float64"): torch.float64}[np.dtype(dtype)]
            except (KeyError, TypeError):
                raise AttributeError("dtype '{}' not recognized".format(dtype)) from None
        self.dtype = dtype
        if self.dtype != torch.float32:
            # pydtnn/backends/cpu/libs/conv_gemm.py:101-107
            raise ValueError("Type {} not supported by this version of libconvGemm!".format(str(self.dtype)))
        native.lib()  # fail here, loudly, if the HIP library is not built
        self.debug = debug
        self.parent_layer = parent_layer

    # ------------------------------------------------------------------ forward / dW
    def conv_gemm_nchw(self, weights, x, biases=None, vpadding=0, hpadding=0, vstride=1, hstride=1,
                       vdilation=1, hdilation=1, biases_vector=None, trans=False, bn_running_mean=None,
                       bn_inv_std=None, bn_gamma=None, bn_beta=None, relu=False, relu_mask=None, residual=None,
                       relu_after_residual=False):
        """``weights * im2col(x)`` (+ fused bias / BN / ReLU), or with ``trans`` the filter gradient
        ``dy_cols * im2col(x)^T`` written into ``biases`` (pydtnn/backends/cpu/libs/conv_gemm.py:117-207).
        ``relu_mask`` (not in the reference; forward with ``relu`` and no BN only): an int8 tensor shaped
        like the output that receives the mask a separate ReLU layer would keep for its backward.
        ``residual`` (not in the reference; forward only): a tensor shaped like the output that is added
        after the bias / BN / ReLU chain, i.e. the sum an addition block makes of its paths; with
        ``relu_after_residual`` the sum is rectified (the Relu layer that follows the block)."""
        b, c, h, w = x.shape
        if not trans:
            kn, ck, kh, kw = weights.shape
            if biases is None:
                ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
                wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
                biases = torch.empty((b, kn, ho, wo), dtype=weights.dtype, device=weights.device)
            else:
                bb, knb, ho, wo = biases.shape
                assert kn == knb, "Number of filters must be the same!"
                assert b == bb, "Batch size must be the same!"
        else:
            assert biases is not None, "If using the transposed convGemm, the biases matrix must be supplied"
            kn, ck, kh, kw = biases.shape
            bw, knw, ho, wo = weights.shape
            assert kn == knw, "Number of filters must be the same!"
            assert b == bw, "Batch size must be the same!"
        assert ck == c, "Number of channels in weights and x should be the same!"
        assert weights.dtype == x.dtype == biases.dtype, "All the matrices must have the same type of data!"
        assert weights.dtype == self.dtype, \
            "The input matrices must have the same type of data as the one specified when " \
            "this class was instantiated!"
        geom = (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
        ws, ws_bytes = native.conv_workspace(native.OP_DW if trans else native.OP_FWD, 0, geom)
        if relu_mask is not None:
            self._check_relu_mask(relu_mask, biases, trans, relu, bn_running_mean)
            check(lib().pydtnn_hip_sconvGemm_relu_mask(
                0, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, f32(weights),
                f32(x), f32(biases), f32(biases_vector), ptr(relu_mask), ws, ws_bytes, stream_ptr()),
                "sconvGemm_relu_mask")
            return biases
        if residual is not None:
            self._check_residual(residual, biases, trans, relu_mask)
            check(lib().pydtnn_hip_sconvGemm_residual(
                0, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, f32(weights),
                f32(x), f32(biases), f32(biases_vector), f32(bn_running_mean), f32(bn_inv_std), f32(bn_gamma),
                f32(bn_beta), bool(relu), f32(residual), bool(relu_after_residual), ws, ws_bytes, stream_ptr()),
                "sconvGemm_residual")
            return biases
        check(lib().pydtnn_hip_sconvGemmNCHW(
            b'Y' if trans else b'N', b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
            hdilation, f32(weights), f32(x), f32(biases), f32(biases_vector), f32(bn_running_mean), f32(bn_inv_std),
            f32(bn_gamma), f32(bn_beta), bool(relu), ws, ws_bytes, stream_ptr()), "sconvGemmNCHW")
        return biases

    def conv_gemm_nhwc(self, weights, x, biases=None, vpadding=0, hpadding=0, vstride=1, hstride=1,
                       vdilation=1, hdilation=1, biases_vector=None, trans=False, bn_running_mean=None,
                       bn_inv_std=None, bn_gamma=None, bn_beta=None, relu=False, relu_mask=None, residual=None,
                       relu_after_residual=False):
        """NHWC twin (pydtnn/backends/cpu/libs/conv_gemm.py:209-250): weights (c, kh, kw, kn)."""
        b, h, w, c = x.shape
        if not trans:
            ck, kh, kw, kn = weights.shape
            if biases is None:
                ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
                wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
                biases = torch.empty((b, ho, wo, kn), dtype=weights.dtype, device=weights.device)
            else:
                bb, ho, wo, knb = biases.shape
                assert kn == knb, "Number of filters must be the same!"
                assert b == bb, "Batch size must be the same!"
        else:
            assert biases is not None, "If using the transposed convGemm, the output matrix must be supplied"
            ck, kh, kw, kn = biases.shape
            bw, ho, wo, knw = weights.shape
            assert kn == knw, "Number of filters must be the same!"
            assert b == bw, "Batch size must be the same!"
        assert ck == c, "Number of channels in weights and x should be the same!"
        assert weights.dtype == x.dtype == biases.dtype, "All the matrices must have the same type of data!"
        geom = (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
        ws, ws_bytes = native.conv_workspace(native.OP_DW if trans else native.OP_FWD, 1, geom)
        if relu_mask is not None:
            self._check_relu_mask(relu_mask, biases, trans, relu, bn_running_mean)
            check(lib().pydtnn_hip_sconvGemm_relu_mask(
                1, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, f32(weights),
                f32(x), f32(biases), f32(biases_vector), ptr(relu_mask), ws, ws_bytes, stream_ptr()),
                "sconvGemm_relu_mask")
            return biases
        if residual is not None:
            self._check_residual(residual, biases, trans, relu_mask)
            check(lib().pydtnn_hip_sconvGemm_residual(
                1, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, f32(weights),
                f32(x), f32(biases), f32(biases_vector), f32(bn_running_mean), f32(bn_inv_std), f32(bn_gamma),
                f32(bn_beta), bool(relu), f32(residual), bool(relu_after_residual), ws, ws_bytes, stream_ptr()),
                "sconvGemm_residual")
            return biases
        check(lib().pydtnn_hip_sconvGemmNHWC(
            b'Y' if trans else b'N', b, h, w, c, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
            hdilation, f32(weights), f32(x), f32(biases), f32(biases_vector), f32(bn_running_mean), f32(bn_inv_std),
            f32(bn_gamma), f32(bn_beta), bool(relu), ws, ws_bytes, stream_ptr()), "sconvGemmNHWC")
        return biases

    def conv_gemm_pair_nhwc(self, weights, x, weights2, vpadding=0, hpadding=0, vstride=1, hstride=1, vdilation=1,
                            hdilation=1, biases_vector=None, bn_running_mean=None, bn_inv_std=None, bn_gamma=None,
                            bn_beta=None, relu=False, biases_vector2=None, bn_running_mean2=None, bn_inv_std2=None,
                            bn_gamma2=None, bn_beta2=None, relu2=False, residual=None, relu_after_residual=False):
        """Not in the reference: ``conv_gemm_nhwc`` with the first set of arguments followed by a 1 x 1 convolution
        with ``weights2`` (kn, 1, 1, kn2) and the second set, as one launch that never stores the tensor between
        them (the 3 x 3 and the last 1 x 1 layer of a ResNet bottleneck after the fusion pass, with the block's sum
        and ReLU).  Returns the output, or None when the library is not built for the shapes: the caller then makes
        the two calls, which give the same bits."""
        b, h, w, c = x.shape
        ck, kh, kw, kn = weights.shape
        c2, kh2, kw2, kn2 = weights2.shape
        if (ck, c2, kh2, kw2) != (c, kn, 1, 1) or x.dtype != torch.float32:
            return None
        ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
        wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
        y = torch.empty((b, ho, wo, kn2), dtype=x.dtype, device=x.device)
        if residual is not None:
            self._check_residual(residual, y, False, None)
        rc = lib().pydtnn_hip_sconvGemm_pair_nhwc(
            b, h, w, c, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, f32(weights), f32(x),
            f32(biases_vector), f32(bn_running_mean), f32(bn_inv_std), f32(bn_gamma), f32(bn_beta), bool(relu), kn2,
            f32(weights2), f32(y), f32(biases_vector2), f32(bn_running_mean2), f32(bn_inv_std2), f32(bn_gamma2),
            f32(bn_beta2), bool(relu2), f32(residual), bool(relu_after_residual), stream_ptr())
        if rc == native.PYDTNN_HIP_ERR_UNSUPPORTED:
            return None
        check(rc, "sconvGemm_pair_nhwc")
        return y

    @staticmethod
    def _check_relu_mask(relu_mask, out, trans, relu, bn_running_mean):
        assert not trans and relu and bn_running_mean is None, \
            "relu_mask goes with a forward call that applies ReLU and no batch normalization"
        assert relu_mask.dtype == torch.int8 and relu_mask.shape == out.shape and relu_mask.is_contiguous(), \
            "relu_mask must be a contiguous int8 tensor shaped like the output"

    @staticmethod
    def _check_residual(residual, out, trans, relu_mask):
        assert not trans and relu_mask is None, "residual goes with a forward call without relu_mask"
        assert residual.dtype == out.dtype and residual.shape == out.shape and residual.is_contiguous(), \
            "residual must be a contiguous tensor shaped like the output"
        assert residual.data_ptr() != out.data_ptr(), "residual must not be the output tensor"

    @staticmethod
    def _check_gate(gate, dx):
        assert gate.dtype == torch.int8 and gate.shape == dx.shape and gate.is_contiguous(), \
            "gate must be a contiguous int8 tensor shaped like dx"

    # ------------------------------------------------------------------ dX
    def deconv_gemm_nchw(self, weights, dy, dx, vpadding=0, hpadding=0, vstride=1, hstride=1,
                         vdilation=1, hdilation=1, gate=None):
        """dx = col2im(weights_2D^T * dy_2D) (pydtnn/backends/cpu/libs/conv_gemm.py:252-309).
        ``gate`` (not in the reference): the int8 mask of a ReLU layer that sits below this convolution;
        dx is stored multiplied by it, which is that layer's backward."""
        kn, ck, kh, kw = weights.shape
        b2, kn2, ho, wo = dy.shape
        b, c, h, w = dx.shape
        assert kn == kn2, "Number of filters outputs in weights and dy should be the same!"
        assert b == b2, "Different batch size!"
        assert ck == c, "Number of channels in weights and x should be the same!"
        geom = (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
        ws, ws_bytes = native.conv_workspace(native.OP_DX, 0, geom)
        if gate is not None:
            self._check_gate(gate, dx)
            check(lib().pydtnn_hip_sconvGemm_back_gated(
                0, b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation,
                f32(weights), f32(dy), f32(dx), ptr(gate), ws, ws_bytes, stream_ptr()), "sconvGemm_back_gated")
            return dx
        check(lib().pydtnn_hip_sconvGemmNCHW_back(
            b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation,
            f32(weights), f32(dy), f32(dx), ws, ws_bytes, stream_ptr()), "sconvGemmNCHW_back")
        return dx

    def deconv_gemm_nhwc(self, weights, dy, dx, vpadding=0, hpadding=0, vstride=1, hstride=1,
                         vdilation=1, hdilation=1, gate=None):
        """NHWC twin (pydtnn/backends/cpu/libs/conv_gemm.py:311-330)."""
        ck, kh, kw, kn = weights.shape
        b2, ho, wo, kn2 = dy.shape
        b, h, w, c = dx.shape
        assert kn == kn2, "Number of filters outputs in weights and dy should be the same!"
        assert b == b2, "Different batch size!"
        assert ck == c, "Number of channels in weights and x should be the same!"
        geom = (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
        ws, ws_bytes = native.conv_workspace(native.OP_DX, 1, geom)
        if gate is not None:
            self._check_gate(gate, dx)
            check(lib().pydtnn_hip_sconvGemm_back_gated(
                1, b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation,
                f32(weights), f32(dy), f32(dx), ptr(gate), ws, ws_bytes, stream_ptr()), "sconvGemm_back_gated")
            return dx
        check(lib().pydtnn_hip_sconvGemmNHWC_back(
            b, h, w, c, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation,
            f32(weights), f32(dy), f32(dx), ws, ws_bytes, stream_ptr()), "sconvGemmNHWC_back")
        return dx


class PreparedForward:
    """A forward convolution whose geometry, filter and per-channel vectors are bound once (the library's
    ``pydtnn_hip_conv_plan``): what a layer's ``initialize`` prepares so that each inference step passes only the
    activations.  The reference's layers fix the same things in ``initialize``
    (pydtnn/backends/cpu/layers/conv_2d_cpu.py:89-143) and its GPU layers also keep their output tensor between
    steps (pydtnn/backends/gpu/layers/conv_2d_gpu.py:89-96): with ``keep_output`` every call returns the same
    tensor, overwritten; without it a fresh one.

    The tensors are referenced, not copied: they may be updated in place; ``binds(...)`` tells whether a layer's
    current tensors are still the ones bound here."""

    def __init__(self, nhwc, x_shape, weights, geom8, biases_vector=None, bn=None, relu=False, keep_output=False):
        if weights.dtype != torch.float32:
            raise ValueError("Type {} not supported by this version of libconvGemm!".format(weights.dtype))
        kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation = geom8
        if nhwc:
            b, h, w, c = x_shape
            ck, kh_, kw_, kn = weights.shape
        else:
            b, c, h, w = x_shape
            kn, ck, kh_, kw_ = weights.shape
        assert ck == c, "Number of channels in weights and x should be the same!"
        assert (kh_, kw_) == (kh, kw)
        ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) // vstride + 1
        wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) // hstride + 1
        self.nhwc = int(bool(nhwc))
        self.x_shape = tuple(x_shape)
        self.out_shape = (b, ho, wo, kn) if nhwc else (b, kn, ho, wo)
        self.geom13 = (b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation)
        self.bound = (weights, biases_vector) + (tuple(bn) if bn is not None else (None,) * 4)
        self.relu = bool(relu)
        self.device = weights.device
        self.keep_output = keep_output
        self._y = None
        self._ws = {}      # raw stream handle -> (pointer, bytes, key and tensor of the stream's scratch buffer)
        self._run = lib().pydtnn_hip_conv_plan_forward
        self._plan = ctypes.c_void_p()
        check(lib().pydtnn_hip_conv_plan_create(ctypes.byref(self._plan), self.nhwc, *self.geom13,
                                                *[f32(t) for t in self.bound], self.relu), "conv_plan_create")

    def binds(self, weights, biases_vector, bn, relu):
        t = self.bound
        return t[0] is weights and t[1] is biases_vector and self.relu == bool(relu) and \
            ((bn is None and t[2] is None) or
             (bn is not None and t[2] is bn[0] and t[3] is bn[1] and t[4] is bn[2] and t[5] is bn[3]))

    def __call__(self, x):
        if x.shape != self.x_shape or x.dtype != torch.float32 or not x.is_contiguous() or x.device != self.device:
            raise ValueError(f"expected a contiguous float32 tensor of shape {self.x_shape} on {self.device}")
        stream = torch._C._cuda_getCurrentRawStream(self.device.index)
        ws = self._ws.get(stream)
        if ws is None or native.workspace_buffer(ws[2]) is not ws[3]:
            # first call on this stream, or the stream's scratch buffer has been replaced by a larger one
            ptr_, size = native.conv_workspace(native.OP_FWD, self.nhwc, self.geom13, stream)
            key = (self.device.index, stream)
            ws = self._ws[stream] = (ptr_, size, key, native.workspace_buffer(key))
        if self.keep_output:
            y = self._y
            if y is None:
                y = self._y = torch.empty(self.out_shape, dtype=torch.float32, device=self.device)
        else:
            y = torch.empty(self.out_shape, dtype=torch.float32, device=self.device)
        rc = self._run(self._plan, x.data_ptr(), y.data_ptr(), ws[0], ws[1], stream)
        if rc:
            check(rc, "conv_plan_forward")
        return y

    def __del__(self):
        plan, self._plan = getattr(self, "_plan", None), None
        if plan:
            try:
                lib().pydtnn_hip_conv_plan_destroy(plan)
            except Exception:     # interpreter shutdown
                pass

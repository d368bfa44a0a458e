/*
 * C ABI of libpydtnn_hip.so: the MI355X (gfx950) implementation of PyDTNN's conv-as-GEMM path.
 *
 * Two flavours are exported.
 *
 *  (1) Device-pointer entry points, prefixed pydtnn_hip_.  Every pointer is a device address
 *      (for instance torch.Tensor.data_ptr()), `stream` is a hipStream_t passed as void*
 *      (NULL = the default stream), work is enqueued asynchronously and the return value is a
 *      PYDTNN_HIP_* status.  Tensors are dense, C-contiguous fp32.  Entry points that need
 *      scratch memory take `workspace` / `workspace_bytes`; the matching *_workspace_bytes
 *      query says how much.  Nothing here allocates or frees device memory.
 *
 *  (2) Host-pointer entry points with exactly the names and argument lists of the external
 *      libconvGemm that PyDTNN binds with ctypes (pydtnn/backends/cpu/libs/conv_gemm.py:85-107):
 *      alloc_pack_buffs, sconvGemmNCHW, sconvGemmNHWC, sconvGemmNCHW_back, sconvGemmNHWC_back.
 *      They live in libconvGemm.so (same sources plus the shim), copy operands to the GPU, run
 *      the flavour-(1) kernels and copy the result back, so the reference's own ConvGemm class
 *      can load this build through LD_LIBRARY_PATH unchanged.
 *
 * Paths cited below are relative to the PyDTNN source tree.
 */
#ifndef PYDTNN_HIP_H
#define PYDTNN_HIP_H

#include <stddef.h>
#include <stdint.h>
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PYDTNN_HIP_OK 0
#define PYDTNN_HIP_ERR_INVALID 1
#define PYDTNN_HIP_ERR_WORKSPACE 2
#define PYDTNN_HIP_ERR_LAUNCH 3
#define PYDTNN_HIP_ERR_UNSUPPORTED 4

/* Library identification: returns 10000*major + 100*minor + patch. */
int pydtnn_hip_version(void);
/* Human-readable text for a status code (static storage). */
const char *pydtnn_hip_status_string(int status);
/* One launch addresses a tensor with 32-bit byte offsets: at most 2^29 floats.  The implicit
 * convolution entry points (sconvGemm*, *_back) run a larger batch as consecutive groups of whole
 * images, each below that limit; the filter gradient is summed over the groups in order. */

/* ------------------------------------------------------------------------------------------
 * Explicit im2col / col2im.  Replace the Cython modules
 *   im2col_nchw_cython / col2im_nchw_cython   pydtnn/cython_modules/im2col_nchw_cython.pyx:28-52, :150-173
 *   im2row_nhwc_cython / row2im_nhwc_cython   pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49, :123-146
 * with identical index maps.  cols is (c*kh*kw, b*ho*wo); rows is (b*ho*wo, c*kh*kw); the output
 * is fully written (padding positions get 0; col2im/row2im need no pre-zeroed dx).
 * ---------------------------------------------------------------------------------------- */
int pydtnn_hip_im2col_nchw(const float *x, float *cols, int b, int c, int h, int w, int kh, int kw,
                           int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                           void *stream);
int pydtnn_hip_col2im_nchw(const float *cols, float *dx, int b, int c, int h, int w, int kh, int kw,
                           int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                           void *stream);
int pydtnn_hip_im2row_nhwc(const float *x, float *rows, int b, int h, int w, int c, int kh, int kw,
                           int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                           void *stream);
int pydtnn_hip_row2im_nhwc(const float *rows, float *dx, int b, int h, int w, int c, int kh, int kw,
                           int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                           void *stream);

/* ------------------------------------------------------------------------------------------
 * GEMM.  Replaces pydtnn.utils.matmul (pydtnn/utils/__init__.py:148-158: a @ b) for row-major
 * fp32 operands, with the transposed views NumPy would pass to BLAS:
 *     C(m x n) = op(A) * op(B),  op(A) = A (m x k, lda) or A^T (A stored k x m, lda) when transa != 0,
 *                                op(B) = B (k x n, ldb) or B^T (B stored n x k, ldb) when transb != 0.
 * Optional fused epilogue on C: + bias[n] (FC forward, pydtnn/backends/cpu/layers/fc_cpu.py:63), then ReLU.
 * Small m*n with long k is split along k; then `workspace` must hold
 * pydtnn_hip_sgemm_workspace_bytes(m, n, k) bytes (0 means none needed) and C must be dense
 * (ldc == n; PYDTNN_HIP_ERR_UNSUPPORTED otherwise, before anything is launched).
 * ---------------------------------------------------------------------------------------- */
size_t pydtnn_hip_sgemm_workspace_bytes(long m, long n, long k);
int pydtnn_hip_sgemm(int transa, int transb, long m, long n, long k, const float *a, long lda, const float *b,
                     long ldb, float *c, long ldc, const float *bias, int relu, void *workspace,
                     size_t workspace_bytes, void *stream);

/* pydtnn_hip_sgemm for callers that cannot allocate device memory or hold a workspace of their own (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart
 * in PyDTNN.  Same arguments, meaning and results (bit for bit) as pydtnn_hip_sgemm minus the workspace:
 * the partial sums of a split along k go to an array that is part of the library's device image,
 * pydtnn_hip_sgemm_static_scratch_bytes() = 64 MiB on every GPU the library has run on, held until the
 * process ends.  A problem whose pydtnn_hip_sgemm_workspace_bytes(m, n, k) exceeds that returns
 * PYDTNN_HIP_ERR_WORKSPACE and launches nothing.  The call allocates and frees nothing; the first call on a
 * device asks the runtime for the array's address there (make that call before starting a capture).
 * All calls on one GPU share the array: calls that may overlap there (different streams, different
 * threads) race; order them on one stream. */
size_t pydtnn_hip_sgemm_static_scratch_bytes(void);
int pydtnn_hip_sgemm_static(int transa, int transb, long m, long n, long k, const float *a, long lda, const float *b,
                            long ldb, float *c, long ldc, const float *bias, int relu, void *stream);

/* ------------------------------------------------------------------------------------------
 * Implicit-im2col convolution GEMMs: the column matrix is never materialised.
 * Same argument meaning and order as libconvGemm's sconvGemmNCHW / sconvGemmNHWC
 * (call sites pydtnn/backends/cpu/libs/conv_gemm.py:191-205 and :234-248), minus the two CPU
 * packing buffers, plus workspace and stream:
 *   trans == 'N' : forward.  in1 = weights (NCHW: kn,c,kh,kw; NHWC: c,kh,kw,kn), out = y
 *                  (NCHW: b,kn,ho,wo; NHWC: b,ho,wo,kn), then per output channel
 *                  + bias_vector -> ((v - bn_running_mean) * bn_inv_std) * bn_gamma + bn_beta -> ReLU,
 *                  each stage skipped when its pointer is NULL / relu is false.  The BN stage is
 *                  applied when bn_running_mean is non-NULL and then needs all four vectors.
 *                  The workspace is optional here: with
 *                  pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_FWD, ...) bytes the launch is
 *                  balanced over the compute units (tiles that do not fill the chip evenly are
 *                  cut along the reduction axis and summed in a fixed order); with less, or
 *                  NULL, the result is computed by a plain grid of tiles.
 *   trans == 'Y' : filter gradient.  in1 = dy (layout of y), out = dw (layout of weights);
 *                  epilogue arguments must be NULL / false.  Needs a workspace of
 *                  pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DW, ...) bytes.
 * ---------------------------------------------------------------------------------------- */
#define PYDTNN_HIP_OP_FWD 0
#define PYDTNN_HIP_OP_DW 1
#define PYDTNN_HIP_OP_DX 2
#define PYDTNN_HIP_OP_DX_I2C 3 /* explicit GEMM + col2im/row2im variant of dX */
#define PYDTNN_HIP_OP_DB 4     /* bias gradient */
#define PYDTNN_HIP_OP_FWD_I2C 5 /* forward GEMM over a materialised column / row matrix (optional workspace) */

size_t pydtnn_hip_conv_workspace_bytes(int op, int nhwc, int b, int c, int h, int w, int kn, int kh, int kw,
                                       int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation);

int pydtnn_hip_sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float *in1, const float *x, float *out,
                             const float *bias_vector, const float *bn_running_mean, const float *bn_inv_std,
                             const float *bn_gamma, const float *bn_beta, bool relu, void *workspace,
                             size_t workspace_bytes, void *stream);
int pydtnn_hip_sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float *in1, const float *x, float *out,
                             const float *bias_vector, const float *bn_running_mean, const float *bn_inv_std,
                             const float *bn_gamma, const float *bn_beta, bool relu, void *workspace,
                             size_t workspace_bytes, void *stream);

/* Input gradient dx = col2im(W^T dy) without the (K x P) matrix: libconvGemm's sconvGemmNCHW_back /
 * sconvGemmNHWC_back (pydtnn/backends/cpu/libs/conv_gemm.py:299-307, :321-328; note stride comes before
 * padding in this argument list, as in the reference).  dx is fully overwritten (the reference
 * requires the caller to zero it first; here that is not needed).  Workspace:
 * pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DX, ...). */
int pydtnn_hip_sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float *weights,
                                  const float *dy, float *dx, void *workspace, size_t workspace_bytes,
                                  void *stream);
int pydtnn_hip_sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float *weights,
                                  const float *dy, float *dx, void *workspace, size_t workspace_bytes,
                                  void *stream);

/* ------------------------------------------------------------------------------------------
 * Explicit ("i2c") convolution GEMMs over a materialised column / row matrix: the GEMM steps of
 *   Conv2DCPU._forward_nchw_i2c / _backward_nchw_i2c   pydtnn/backends/cpu/layers/conv_2d_cpu.py:264-291, :447-481
 *   Conv2DCPU._forward_nhwc_i2c / _backward_nhwc_i2c   pydtnn/backends/cpu/layers/conv_2d_cpu.py:183-209, :363-397
 * `mat` is x_cols (NCHW: c*kh*kw x b*ho*wo) or x_rows (NHWC: b*ho*wo x c*kh*kw).
 *   forward : y = W * x_cols (+ bias), written straight in the tensor format (the reference's
 *             separate bias pass and 1023 transpose are folded into the store).  Workspace: optional,
 *             OP_FWD_I2C bytes; with it the launch is balanced over the chip like the implicit forward.
 *   dw      : dw = dy_cols * x_cols^T   (NHWC: x_rows^T * dy_rows).  Workspace: OP_DW bytes.
 *   dx      : dx = col2im(W^T * dy_cols) (NHWC: row2im(dy_rows * W^T)); the (K x P) product goes
 *             through the workspace: OP_DX_I2C bytes (the product, then the partial tiles of the balanced
 *             launch; with no more than the product's K*P*4 bytes the GEMM runs as a plain grid).
 * ---------------------------------------------------------------------------------------- */
int pydtnn_hip_conv_i2c_forward(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding,
                                int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                                const float *weights, const float *mat, float *y, const float *bias_vector,
                                void *workspace, size_t workspace_bytes, void *stream);
int pydtnn_hip_conv_i2c_dw(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float *dy, const float *mat,
                           float *dw, void *workspace, size_t workspace_bytes, void *stream);
int pydtnn_hip_conv_i2c_dx(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float *weights,
                           const float *dy, float *dx, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------
 * Stand-alone per-channel epilogue (for layers that are not fused into a convolution):
 *   y = relu?( bn?( x (+ residual) + bias ) )    with channel = (index / inner) % channels.
 * inner = ho*wo for NCHW tensors, 1 for NHWC tensors and (rows, C) matrices.  Covers
 *   add_nchw_cython / add_nhwc_cython            pydtnn/cython_modules/add_nchw_cython.pyx:51-58, add_nhwc_cython.pyx:51-58
 *   bn_inference_cython / bn_inference_nchw      pydtnn/cython_modules/bn_inference_cython.pyx:61-72, :127-140
 *   bn_relu_inference_cython                     pydtnn/cython_modules/bn_relu_inference_cython.pyx:59-70
 *   eltw_sum_cython (residual)                   pydtnn/cython_modules/eltw_sum_cython.pyx:25-36
 * Any of residual, bias, the four BN vectors may be NULL; x and y may alias.
 * ---------------------------------------------------------------------------------------- */
int pydtnn_hip_chan_eltwise(const float *x, const float *residual, float *y, long total, int inner, int channels,
                            const float *bias, const float *bn_running_mean, const float *bn_inv_std,
                            const float *bn_gamma, const float *bn_beta, int relu, void *stream);

/* relu_cython (pydtnn/cython_modules/relu_cython.pyx:25-59): y = x > 0 ? x : 0, mask = x > 0 (int8; may be NULL).
 * Backward dx = dy * mask (pydtnn/backends/cpu/activations/relu_cpu.py:38-40). */
int pydtnn_hip_relu_fwd(const float *x, float *y, int8_t *mask, long total, void *stream);
int pydtnn_hip_relu_bwd(const float *dy, const int8_t *mask, float *dx, long total, void *stream);

/* db = sum of dy over batch and pixels (pydtnn/backends/cpu/layers/conv_2d_cpu.py:377, :463; fc_cpu.py:70).
 * dy is (outer, channels, inner): inner = ho*wo for NCHW, 1 for NHWC / FC.
 * Workspace: pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DB, ...) or 2048*channels bytes. */
int pydtnn_hip_bias_grad(const float *dy, float *db, long outer, int channels, int inner, void *workspace,
                         size_t workspace_bytes, void *stream);

/* MaxPool2D, NCHW (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:25-52, :140-166); idx_max is int32 (b,c,ho,wo). */
int pydtnn_hip_max_pool_2d_fwd_nchw(const float *x, float *y, int32_t *idx_max, int b, int c, int h, int w, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void *stream);
int pydtnn_hip_max_pool_2d_bwd_nchw(const float *dy, const int32_t *idx_max, float *dx, int b, int c, int h, int w,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void *stream);

/* MaxPool2D, NHWC (pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:25-52, :140-166); idx_max is int32 (b,ho,wo,c). */
int pydtnn_hip_max_pool_2d_fwd_nhwc(const float *x, float *y, int32_t *idx_max, int b, int h, int w, int c, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void *stream);
int pydtnn_hip_max_pool_2d_bwd_nhwc(const float *dy, const int32_t *idx_max, float *dx, int b, int h, int w, int c,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void *stream);

/* AveragePool2D in either format (nhwc = 0: pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:25-52 and
 * :135-160; nhwc = 1: average_pool_2d_nhwc_cython.pyx, same lines): the mean over the window's taps that lie
 * inside the image (padding is not counted); backward gives every such tap dy / count.  b, c, h, w name the
 * input's batch, channels, height, width; dx is fully written. */
int pydtnn_hip_average_pool_2d_fwd(int nhwc, const float *x, float *y, int b, int c, int h, int w, int kh, int kw,
                                   int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                   int hdilation, void *stream);
int pydtnn_hip_average_pool_2d_bwd(int nhwc, const float *dy, float *dx, int b, int c, int h, int w, int kh, int kw,
                                   int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                   int hdilation, void *stream);

/* ------------------------------------------------------------------------------------------
 * The ReLU layer between two layers of a training step, done by its neighbours' stores instead of
 * two passes of its own.  Results are those of the separate calls, bit for bit.
 *   pydtnn_hip_sconvGemm_relu_mask: the forward of pydtnn_hip_sconvGemmNCHW / NHWC (nhwc = 0 / 1;
 *       b, c, h, w name the input's batch, channels, height, width in either format) with
 *       y = relu(conv(x) + bias_vector) and mask = (conv(x) + bias_vector) > 0 as int8, shaped like y:
 *       what pydtnn_hip_relu_fwd (relu_cython.pyx:25-59) makes of the convolution's output.
 *   pydtnn_hip_sconvGemm_back_gated: pydtnn_hip_sconvGemmNCHW_back / NHWC_back with dx multiplied by
 *       gate (int8, shaped like dx): what pydtnn_hip_relu_bwd (relu_cpu.py:38-40) makes of dx when
 *       the layer below the convolution is a ReLU whose mask is `gate`.  Same workspace.
 *   pydtnn_hip_max_pool_2d_bwd_gated: the same for pydtnn_hip_max_pool_2d_bwd_nchw / nhwc.
 * ---------------------------------------------------------------------------------------- */
int pydtnn_hip_sconvGemm_relu_mask(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                   unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride,
                                   unsigned hstride, unsigned vdilation, unsigned hdilation, const float *weights,
                                   const float *x, float *y, const float *bias_vector, int8_t *mask, void *workspace,
                                   size_t workspace_bytes, void *stream);
int pydtnn_hip_sconvGemm_back_gated(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                    unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                    unsigned hpadding, unsigned vdilation, unsigned hdilation, const float *weights,
                                    const float *dy, float *dx, const int8_t *gate, void *workspace,
                                    size_t workspace_bytes, void *stream);
int pydtnn_hip_max_pool_2d_bwd_gated(int nhwc, const float *dy, const int32_t *idx_max, float *dx, const int8_t *gate,
                                     int b, int c, int h, int w, int kh, int kw, int vpadding, int hpadding,
                                     int vstride, int hstride, int vdilation, int hdilation, void *stream);

/* Two consecutive convolutions of one path as a single launch, NHWC, inference: the forward of
 * pydtnn_hip_sconvGemmNHWC with the first set of arguments (filter `weights`, its bias / BN vectors and ReLU flag),
 * whose result is never stored but fed, as it leaves the matrix cores, to a 1 x 1 convolution at unit stride
 * without padding with the second set (`weights2` of shape (kn, 1, 1, kn2), its vectors), which stores y
 * (b, ho, wo, kn2) and, with `residual`, adds it and rectifies as pydtnn_hip_sconvGemm_residual does.  This is the
 * tail of a ResNet bottleneck after the fusion pass (pydtnn/model.py:294-349): Conv2DBatchNormalizationRelu 3x3,
 * Conv2DBatchNormalization 1x1, the AdditionBlock's sum (pydtnn/backends/cpu/layers/addition_block_cpu.py:41-45) and
 * the Relu after it.  Results equal the two separate calls bit for bit.  Built for the shapes of the first
 * bottlenecks only (3x3, pad 1, unit stride and dilation, 64 -> 64 filters, then at most 256, BN on the second
 * layer, at least 32768 output pixels in multiples of 32, 16-byte aligned tensors): any other call returns
 * PYDTNN_HIP_ERR_UNSUPPORTED before anything is launched, and the caller makes the two calls.  No workspace. */
int pydtnn_hip_sconvGemm_pair_nhwc(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                                   unsigned vdilation, unsigned hdilation, const float *weights, const float *x,
                                   const float *bias_vector, const float *bn_running_mean, const float *bn_inv_std,
                                   const float *bn_gamma, const float *bn_beta, bool relu, unsigned kn2,
                                   const float *weights2, float *y, const float *bias_vector2,
                                   const float *bn_running_mean2, const float *bn_inv_std2, const float *bn_gamma2,
                                   const float *bn_beta2, bool relu2, const float *residual, bool relu_after_add,
                                   void *stream);

/* A forward convolution with everything but the activations bound once: a layer that calls with the same
 * geometry, filter and per-channel vectors at every step (an inference loop) builds the plan when it is
 * initialised, as the reference's layers build their ConvGemm object and its kernel arguments in initialize()
 * (pydtnn/backends/cpu/layers/conv_2d_cpu.py:89-143; the GPU layers also keep their output tensor,
 * pydtnn/backends/gpu/layers/conv_2d_gpu.py:89-96), and then passes four pointers per call.
 * pydtnn_hip_conv_plan_forward(plan, x, y, ...) computes exactly what pydtnn_hip_sconvGemmNCHW / NHWC
 * (nhwc = 0 / 1; b, c, h, w name the input's extents in either format) computes with trans = 'N' and the plan's
 * arguments; the plan keeps the pointers it was given, not copies, so the filter and the vectors may change in
 * place but must stay where they are.  Creating and destroying a plan touches host memory only. */
typedef struct pydtnn_hip_conv_plan pydtnn_hip_conv_plan;
int pydtnn_hip_conv_plan_create(pydtnn_hip_conv_plan **plan, int nhwc, int b, int c, int h, int w, int kn, int kh,
                                int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                int hdilation, const float *weights, const float *bias_vector,
                                const float *bn_running_mean, const float *bn_inv_std, const float *bn_gamma,
                                const float *bn_beta, bool relu);
int pydtnn_hip_conv_plan_forward(const pydtnn_hip_conv_plan *plan, const float *x, float *y, void *workspace,
                                 size_t workspace_bytes, void *stream);
void pydtnn_hip_conv_plan_destroy(pydtnn_hip_conv_plan *plan);

/* The sum of an addition block done by the store of the convolution that ends one of its two paths
 * (inference).  The forward of pydtnn_hip_sconvGemmNCHW / NHWC (nhwc = 0 / 1; b, c, h, w name the input's
 * batch, channels, height, width in either format) followed by
 *     y = y + residual                      eltw_sum_cython (pydtnn/cython_modules/eltw_sum_cython.pyx:25-36) as
 *                                           AdditionBlockCPU.forward applies it
 *                                           (pydtnn/backends/cpu/layers/addition_block_cpu.py:41-45)
 *     y = y > 0 ? y : 0                     when relu_after_add: the Relu layer that follows the block
 * with `residual` shaped like y.  Results equal the separate calls bit for bit.  residual must not alias y;
 * it may be x itself (both are only read: a block whose folded path is one convolution and whose other path is
 * the identity passes the block input twice).  Same optional workspace as the forward. */
int pydtnn_hip_sconvGemm_residual(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride,
                                  unsigned hstride, unsigned vdilation, unsigned hdilation, const float *weights,
                                  const float *x, float *y, const float *bias_vector, const float *bn_running_mean,
                                  const float *bn_inv_std, const float *bn_gamma, const float *bn_beta, bool relu,
                                  const float *residual, bool relu_after_add, void *workspace, size_t workspace_bytes,
                                  void *stream);

/* BatchNormalization in training mode (pydtnn/backends/cpu/layers/batch_normalization_cpu.py:59-82 and
 * :108-129; dx as pydtnn/cython_modules/bn_training_cython.pyx:236-243).  Tensors are viewed as
 * (outer, channels, inner): NCHW = (N, C, H*W); NHWC and 2-D = (rows, C, 1).  With n = outer * inner:
 *   forward : mu = mean(x); var = mean((x - mu)^2); std = sqrt(var + eps); xn = (x - mu) / std;
 *             y = gamma * xn + beta; running_mean = momentum * running_mean + (1 - momentum) * mu,
 *             running_var likewise with var.  Outputs y, xn (x-shaped) and std (channels).
 *   backward: dgamma = sum(dy * xn); dbeta = sum(dy);
 *             dx = (gamma / (std * n)) * (n * dy - xn * dgamma - dbeta)   (skipped when dx is NULL).
 * Per-channel sums are taken in a fixed order (reproducible run to run).
 * Workspace: pydtnn_hip_bn_training_workspace_bytes(channels). */
size_t pydtnn_hip_bn_training_workspace_bytes(int channels);
int pydtnn_hip_bn_training_fwd(const float *x, float *y, float *xn, float *std_out, const float *gamma,
                               const float *beta, float *running_mean, float *running_var, double momentum, double eps,
                               long outer, int channels, int inner, void *workspace, size_t workspace_bytes,
                               void *stream);
int pydtnn_hip_bn_training_bwd(const float *dy, const float *xn, const float *std_in, const float *gamma,
                               float *dgamma, float *dbeta, float *dx, long outer, int channels, int inner,
                               void *workspace, size_t workspace_bytes, void *stream);

/* Softmax over the rows of a (rows, cols) matrix and its backward
 * (pydtnn/backends/cpu/activations/softmax_cpu.py:32-39):
 *   y = exp(x - max(x, axis=1)) / sum(...);   dx = y * (dy - sum(dy * y, axis=1)). */
int pydtnn_hip_softmax_fwd(const float *x, float *y, int rows, int cols, void *stream);
int pydtnn_hip_softmax_bwd(const float *dy, const float *y, float *dx, int rows, int cols, void *stream);

/* Categorical cross-entropy and its gradient
 * (pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35): with a = first argmax of
 * y_targ[row] and p = clip(y_pred[row, a], eps, 1 - eps) (bounds rounded to float32),
 *   loss[0] = -sum_rows log(p) / rows;   dx = y_targ except dx[row, a] = y_targ[row, a] / (-p * global_batch).
 * Workspace: rows * 4 bytes. */
int pydtnn_hip_categorical_cross_entropy(const float *y_pred, const float *y_targ, float *dx, float *loss, int rows,
                                         int cols, double eps, int global_batch, void *workspace,
                                         size_t workspace_bytes, void *stream);

/* SGD with momentum, in place (pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41). */
int pydtnn_hip_sgd_momentum(float *w, const float *dw, float *velocity, long total, float lr, float momentum,
                            float decay, int nesterov, void *stream);
/* The same step for `count` tensors in one pass (a layer's weights and biases: SGDCPU.update walks
 * layer.grad_vars, pydtnn/backends/cpu/optimizers/sgd_cpu.py:30-41).  w, dw, velocity and total are host arrays of
 * `count` device pointers / element counts; every element gets what pydtnn_hip_sgd_momentum gives it. */
int pydtnn_hip_sgd_momentum_multi(int count, float *const *w, const float *const *dw, float *const *velocity,
                                  const long *total, float lr, float momentum, float decay, int nesterov,
                                  void *stream);

/* ------------------------------------------------------------------------------------------
 * The float64 route.  The reference computes in float64 through its explicit path only: the im2col / im2row /
 * col2im / row2im, add, ReLU and BN-inference modules dispatch on float64
 * (pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49, im2col_nchw_cython.pyx:28-52) and utils.matmul is a plain
 * a @ b (pydtnn/utils/__init__.py:148-158); libconvGemm is float32 only (conv_gemm.py:101-107).  Same index
 * maps, summation orders and argument meaning as the float32 entry points of the same name.
 *   pydtnn_hip_dgemm: C = op(A) op(B) (+ bias[n], ReLU) on v_mfma_f64_16x16x4_f64, operands row-major or the
 *       transposed view of a row-major matrix.  `workspace` (pydtnn_hip_dgemm_workspace_bytes, 0 = not needed)
 *       serves two cases: a small C with a long reduction is split along k into it (required then:
 *       PYDTNN_HIP_ERR_WORKSPACE without it); a C of many tiles whose last round would leave most of the chip
 *       idle gets those tiles from a second launch split along k (optional: without the workspace the call runs
 *       the one grid of whole tiles).  lda, ldb < 2^22 (PYDTNN_HIP_ERR_UNSUPPORTED beyond).
 *   pydtnn_hip_transpose_1023_f64: dst[d1][d0][inner] = src[d0][d1][inner], the (co,N,ho,wo) <-> (N,co,ho,wo)
 *       copy of pydtnn/utils/best_transpose_1023.py:50-58.
 *   pydtnn_hip_bias_grad_f64: db[ch] = sum of dy over (outer, inner); needs no workspace.
 * ---------------------------------------------------------------------------------------- */
size_t pydtnn_hip_dgemm_workspace_bytes(long m, long n, long k);
int pydtnn_hip_dgemm(int transa, int transb, long m, long n, long k, const double *a, long lda, const double *b,
                     long ldb, double *c, long ldc, const double *bias, int relu, void *workspace,
                     size_t workspace_bytes, void *stream);
int pydtnn_hip_im2col_nchw_f64(const double *x, double *cols, int b, int c, int h, int w, int kh, int kw,
                               int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                               void *stream);
int pydtnn_hip_col2im_nchw_f64(const double *cols, double *dx, int b, int c, int h, int w, int kh, int kw,
                               int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                               void *stream);
int pydtnn_hip_im2row_nhwc_f64(const double *x, double *rows, int b, int h, int w, int c, int kh, int kw,
                               int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                               void *stream);
int pydtnn_hip_row2im_nhwc_f64(const double *rows, double *dx, int b, int h, int w, int c, int kh, int kw,
                               int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                               void *stream);
int pydtnn_hip_chan_eltwise_f64(const double *x, const double *residual, double *y, long total, long inner,
                                int channels, const double *bias, const double *bn_running_mean,
                                const double *bn_inv_std, const double *bn_gamma, const double *bn_beta, int relu,
                                void *stream);
int pydtnn_hip_relu_fwd_f64(const double *x, double *y, int8_t *mask, long total, void *stream);
int pydtnn_hip_relu_bwd_f64(const double *dy, const int8_t *mask, double *dx, long total, void *stream);
int pydtnn_hip_bias_grad_f64(const double *dy, double *db, long outer, int channels, long inner, void *stream);
int pydtnn_hip_transpose_1023_f64(const double *src, double *dst, int d0, int d1, long inner, void *stream);

/* The layers around the convolutions in float64, so that a float64 model runs a whole training step as it does in
 * the reference: its pooling and BN-training modules dispatch on float64
 * (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:42-49 and :157-164, max_pool_2d_nhwc_cython.pyx,
 * average_pool_2d_nchw_cython.pyx / _nhwc_cython.pyx, bn_training_cython.pyx), and softmax
 * (pydtnn/backends/cpu/activations/softmax_cpu.py:32-39), categorical cross-entropy
 * (pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35) and SGD
 * (pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41) are NumPy expressions in the model's dtype.  Same rules as the
 * float32 entry points above (first maximum wins; stored index ii*kw + jj decoded as idx / kh, idx % kw; sums in
 * the reference's order); nhwc = 0 / 1 selects the tensor format, b, c, h, w name the input's extents in either.
 * The cross-entropy needs rows * 8 bytes of workspace, the others none. */
int pydtnn_hip_max_pool_2d_fwd_f64(int nhwc, const double *x, double *y, int32_t *idx_max, int b, int c, int h, int w,
                                   int kh, int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                   int hdilation, void *stream);
int pydtnn_hip_max_pool_2d_bwd_f64(int nhwc, const double *dy, const int32_t *idx_max, double *dx, int b, int c, int h,
                                   int w, int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                   int vdilation, int hdilation, void *stream);
int pydtnn_hip_average_pool_2d_fwd_f64(int nhwc, const double *x, double *y, int b, int c, int h, int w, int kh, int kw,
                                       int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation, void *stream);
int pydtnn_hip_average_pool_2d_bwd_f64(int nhwc, const double *dy, double *dx, int b, int c, int h, int w, int kh,
                                       int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation, void *stream);
int pydtnn_hip_softmax_fwd_f64(const double *x, double *y, int rows, int cols, void *stream);
int pydtnn_hip_softmax_bwd_f64(const double *dy, const double *y, double *dx, int rows, int cols, void *stream);
int pydtnn_hip_categorical_cross_entropy_f64(const double *y_pred, const double *y_targ, double *dx, double *loss,
                                             int rows, int cols, double eps, int global_batch, void *workspace,
                                             size_t workspace_bytes, void *stream);
int pydtnn_hip_sgd_momentum_f64(double *w, const double *dw, double *velocity, long total, double lr, double momentum,
                                double decay, int nesterov, void *stream);
int pydtnn_hip_bn_training_fwd_f64(const double *x, double *y, double *xn, double *std_out, const double *gamma,
                                   const double *beta, double *running_mean, double *running_var, double momentum,
                                   double eps, long outer, int channels, long inner, void *stream);
int pydtnn_hip_bn_training_bwd_f64(const double *dy, const double *xn, const double *std_in, const double *gamma,
                                   double *dgamma, double *dbeta, double *dx, long outer, int channels, long inner,
                                   void *stream);

/* ------------------------------------------------------------------------------------------
 * Host-pointer compatibility flavour (exported by libconvGemm.so only).  Signatures are those
 * PyDTNN's ctypes shim calls (pydtnn/backends/cpu/libs/conv_gemm.py:91-92, :191-205, :234-248,
 * :299-307, :321-328).  ac_pack / bc_pack are accepted and ignored; alloc_pack_buffs hands out two
 * small malloc() blocks because the reference free()s them with libc (:109-115, :332-349).
 * The operands are pageable host arrays: a call moves them in groups of whole images through pinned bounce
 * buffers (worker threads copy, the DMA engines transfer, the kernels of the group between run, all at once).
 * Errors cannot be returned through this ABI (the reference has no error channel): a failure is reported on
 * stderr, the call returns, and pydtnn_convgemm_last_status() gives the PYDTNN_HIP_* status of the most recent of
 * the four compute calls in this process (PYDTNN_HIP_OK after a good one).  Arguments are checked before anything
 * is copied, so a call rejected as invalid or unsupported leaves its output array untouched; after a run-time
 * failure (status PYDTNN_HIP_ERR_LAUNCH) the output holds the groups that had already come back.  This status
 * function has no counterpart in the reference's libconvGemm: a shim that never calls it behaves as before.
 * ---------------------------------------------------------------------------------------- */
int pydtnn_convgemm_last_status(void);
int alloc_pack_buffs(float **ac_pack, float **bc_pack);
void sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float *in1, const float *x, float *out, const float *bias_vector,
                   const float *bn_running_mean, const float *bn_inv_std, const float *bn_gamma,
                   const float *bn_beta, bool relu, float *ac_pack, float *bc_pack);
void sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float *in1, const float *x, float *out, const float *bias_vector,
                   const float *bn_running_mean, const float *bn_inv_std, const float *bn_gamma,
                   const float *bn_beta, bool relu, float *ac_pack, float *bc_pack);
void sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float *weights, const float *dy, float *dx, float *ac_pack,
                        float *bc_pack);
void sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float *weights, const float *dy, float *dx, float *ac_pack,
                        float *bc_pack);

#ifdef __cplusplus
}
#endif
#endif /* PYDTNN_HIP_H */

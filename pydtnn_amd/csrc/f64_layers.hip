// The layers around the convolutions in float64: max-pooling, average pooling, softmax, categorical
// cross-entropy, SGD with momentum and BatchNormalization in training mode.  The reference's Cython modules
// dispatch on float64 (pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:42-49, average_pool_2d_nchw_cython.pyx,
// bn_training_cython.pyx) and its NumPy layers compute in the model's dtype (softmax_cpu.py, sgd_cpu.py,
// categorical_cross_entropy_cpu.py), so a float64 model runs a whole training step there.
//
// These are the float32 kernels' index rules and summation orders restated one thread per element (per row, per
// channel for the reductions): a float64 model is a precision reference, not a throughput path.
#include "conv_internal.h"
#include <cfloat>

// NumPy rounds after every operation: no multiply-add is fused here, so that elementwise results (SGD, the
// normalisation) carry the reference's roundings
#pragma clang fp contract(off)

namespace {

constexpr int kT = 256;
inline unsigned blocks_for(long total) { return (unsigned)((total + kT - 1) / kT); }

// element (n, ch, y, x) of a tensor of extents (n, c, h, w) stored NCHW or NHWC
template <bool NHWC>
__device__ __forceinline__ long at(int n, int ch, int y, int x, int c, int h, int w)
{
    return NHWC ? (((long)n * h + y) * w + x) * c + ch : (((long)n * c + ch) * h + y) * w + x;
}

// decomposes a linear index of the same tensor
template <bool NHWC>
__device__ __forceinline__ void split(long idx, int c, int h, int w, int* n, int* ch, int* y, int* x)
{
    if (NHWC) {
        *ch = (int)(idx % c); idx /= c;
        *x = (int)(idx % w); idx /= w;
        *y = (int)(idx % h);
        *n = (int)(idx / h);
    } else {
        *x = (int)(idx % w); idx /= w;
        *y = (int)(idx % h); idx /= h;
        *ch = (int)(idx % c);
        *n = (int)(idx / c);
    }
}

// pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:115-137 (NHWC: max_pool_2d_nhwc_cython.pyx): the first
// maximum wins (strict >), start value the lowest finite double, stored index ii*kw + jj.
template <bool NHWC>
__global__ void __launch_bounds__(kT) max_pool_fwd_f64_kernel(const double* __restrict__ x, double* __restrict__ y,
                                                             int32_t* __restrict__ idx_max, ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * kT + threadIdx.x;
    if (idx >= total) return;
    int n, ch, yy, xx;
    split<NHWC>(idx, g.c, g.ho, g.wo, &n, &ch, &yy, &xx);
    double maxval = -DBL_MAX;
    int best = 0;
    for (int ii = 0; ii < g.kh; ++ii) {
        const int ih = g.vstride * yy + g.vdilation * ii - g.vpadding;
        if ((unsigned)ih >= (unsigned)g.h) continue;
        for (int jj = 0; jj < g.kw; ++jj) {
            const int iw = g.hstride * xx + g.hdilation * jj - g.hpadding;
            if ((unsigned)iw >= (unsigned)g.w) continue;
            const double v = x[at<NHWC>(n, ch, ih, iw, g.c, g.h, g.w)];
            if (v > maxval) { maxval = v; best = ii * g.kw + jj; }
        }
    }
    y[idx] = maxval;
    idx_max[idx] = best;
}

// pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:216-233, gather form: an input element collects the dy of
// the windows that point at it, in the order the reference's loop visits them (ascending output row, then
// column).  The stored index is decoded as the reference writes it, ii = idx / kh and jj = idx % kw.
template <bool NHWC>
__global__ void __launch_bounds__(kT) max_pool_bwd_f64_kernel(const double* __restrict__ dy,
                                                             const int32_t* __restrict__ idx_max,
                                                             double* __restrict__ dx, ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * kT + threadIdx.x;
    if (idx >= total) return;
    int n, ch, ih, iw;
    split<NHWC>(idx, g.c, g.h, g.w, &n, &ch, &ih, &iw);
    // windows whose decoded tap can reach (ih, iw): the decoded row index runs up to (kh*kw - 1) / kh
    const int ii_max = (g.kh * g.kw - 1) / g.kh, jj_max = g.kw - 1;
    const int y_hi = min(g.ho - 1, (ih + g.vpadding) / g.vstride);
    const int x_hi = min(g.wo - 1, (iw + g.hpadding) / g.hstride);
    const int y_num = ih + g.vpadding - g.vdilation * ii_max, x_num = iw + g.hpadding - g.hdilation * jj_max;
    const int y_lo = y_num <= 0 ? 0 : (y_num + g.vstride - 1) / g.vstride;
    const int x_lo = x_num <= 0 ? 0 : (x_num + g.hstride - 1) / g.hstride;
    double acc = 0.0;
    for (int yy = y_lo; yy <= y_hi; ++yy)
        for (int xx = x_lo; xx <= x_hi; ++xx) {
            const long o = at<NHWC>(n, ch, yy, xx, g.c, g.ho, g.wo);
            const int code = idx_max[o];
            const int ii = code / g.kh, jj = code % g.kw;
            if (g.vstride * yy + g.vdilation * ii - g.vpadding == ih &&
                g.hstride * xx + g.hdilation * jj - g.hpadding == iw)
                acc += dy[o];
        }
    dx[idx] = acc;
}

// pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:83-108: the taps inside the image, summed in (ii, jj)
// order and divided by their number.
template <bool NHWC>
__global__ void __launch_bounds__(kT) avg_pool_fwd_f64_kernel(const double* __restrict__ x, double* __restrict__ y,
                                                             ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * kT + threadIdx.x;
    if (idx >= total) return;
    int n, ch, yy, xx;
    split<NHWC>(idx, g.c, g.ho, g.wo, &n, &ch, &yy, &xx);
    double accum = 0.0;
    int items = 0;
    for (int ii = 0; ii < g.kh; ++ii) {
        const int ih = g.vstride * yy + g.vdilation * ii - g.vpadding;
        if ((unsigned)ih >= (unsigned)g.h) continue;
        for (int jj = 0; jj < g.kw; ++jj) {
            const int iw = g.hstride * xx + g.hdilation * jj - g.hpadding;
            if ((unsigned)iw >= (unsigned)g.w) continue;
            accum = accum + x[at<NHWC>(n, ch, ih, iw, g.c, g.h, g.w)];
            ++items;
        }
    }
    y[idx] = accum / items;
}

__device__ __forceinline__ int taps_inside(const ConvGeom& g, int yy, int xx)
{
    int rows = 0, cols = 0;
    for (int ii = 0; ii < g.kh; ++ii) rows += (unsigned)(g.vstride * yy + g.vdilation * ii - g.vpadding) < (unsigned)g.h;
    for (int jj = 0; jj < g.kw; ++jj) cols += (unsigned)(g.hstride * xx + g.hdilation * jj - g.hpadding) < (unsigned)g.w;
    return rows * cols;
}

// :198-227, gather form: dy / items of every window that covers the element, windows in ascending (yy, xx) order
// (a window reaches an element through at most one tap per axis).
template <bool NHWC>
__global__ void __launch_bounds__(kT) avg_pool_bwd_f64_kernel(const double* __restrict__ dy, double* __restrict__ dx,
                                                             ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * kT + threadIdx.x;
    if (idx >= total) return;
    int n, ch, ih, iw;
    split<NHWC>(idx, g.c, g.h, g.w, &n, &ch, &ih, &iw);
    double acc = 0.0;
    for (int ii = g.kh - 1; ii >= 0; --ii) {
        const int nv = ih + g.vpadding - g.vdilation * ii;
        if (nv < 0 || nv % g.vstride != 0 || nv / g.vstride >= g.ho) continue;
        const int yy = nv / g.vstride;
        for (int jj = g.kw - 1; jj >= 0; --jj) {
            const int nh = iw + g.hpadding - g.hdilation * jj;
            if (nh < 0 || nh % g.hstride != 0 || nh / g.hstride >= g.wo) continue;
            const int xx = nh / g.hstride;
            acc += dy[at<NHWC>(n, ch, yy, xx, g.c, g.ho, g.wo)] / taps_inside(g, yy, xx);
        }
    }
    dx[idx] = acc;
}

// ---------------------------------------------------------------- row reductions: a workgroup per row
__device__ __forceinline__ double block_sum(double v, double* part)
{
    part[threadIdx.x] = v;
    __syncthreads();
    for (int step = kT / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) part[threadIdx.x] += part[threadIdx.x + step];
        __syncthreads();
    }
    const double r = part[0];
    __syncthreads();
    return r;
}

__device__ __forceinline__ double block_max(double v, double* part)
{
    part[threadIdx.x] = v;
    __syncthreads();
    for (int step = kT / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) part[threadIdx.x] = fmax(part[threadIdx.x], part[threadIdx.x + step]);
        __syncthreads();
    }
    const double r = part[0];
    __syncthreads();
    return r;
}

// pydtnn/backends/cpu/activations/softmax_cpu.py:32-35
__global__ void __launch_bounds__(kT) softmax_fwd_f64_kernel(const double* __restrict__ x, double* __restrict__ y, int cols)
{
    __shared__ double part[kT];
    const double* xr = x + (long)blockIdx.x * cols;
    double* yr = y + (long)blockIdx.x * cols;
    double m = -DBL_MAX;
    for (int i = threadIdx.x; i < cols; i += kT) m = fmax(m, xr[i]);
    m = block_max(m, part);
    double s = 0.0;
    for (int i = threadIdx.x; i < cols; i += kT) {
        const double e = exp(xr[i] - m);
        yr[i] = e;
        s += e;
    }
    s = block_sum(s, part);
    for (int i = threadIdx.x; i < cols; i += kT) yr[i] = yr[i] / s;
}

// softmax_cpu.py:37-39: dx = y * (dy - sum(dy * y))
__global__ void __launch_bounds__(kT) softmax_bwd_f64_kernel(const double* __restrict__ dy, const double* __restrict__ y,
                                                            double* __restrict__ dx, int cols)
{
    __shared__ double part[kT];
    const long r0 = (long)blockIdx.x * cols;
    double s = 0.0;
    for (int i = threadIdx.x; i < cols; i += kT) s += dy[r0 + i] * y[r0 + i];
    s = block_sum(s, part);
    for (int i = threadIdx.x; i < cols; i += kT) dx[r0 + i] = y[r0 + i] * (dy[r0 + i] - s);
}

// pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35, one workgroup per row: a = first argmax of
// y_targ[row], p = clip(y_pred[row, a], eps, 1 - eps); row_loss = log(p); dx = y_targ with dx[row, a] divided by
// (-p * global_batch).
__global__ void __launch_bounds__(kT) cce_rows_f64_kernel(const double* __restrict__ y_pred,
                                                         const double* __restrict__ y_targ, double* __restrict__ dx,
                                                         double* __restrict__ row_loss, int cols, double eps,
                                                         double global_batch)
{
    __shared__ double vals[kT];
    __shared__ int args[kT];
    const long r0 = (long)blockIdx.x * cols;
    double best = -DBL_MAX;
    int arg = cols;
    for (int i = threadIdx.x; i < cols; i += kT) {
        const double t = y_targ[r0 + i];
        dx[r0 + i] = t;
        if (t > best) { best = t; arg = i; }   // ascending i per thread: the first maximum of its subset
    }
    vals[threadIdx.x] = best;
    args[threadIdx.x] = arg;
    __syncthreads();
    for (int step = kT / 2; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) {
            const double ov = vals[threadIdx.x + step];
            const int oa = args[threadIdx.x + step];
            if (ov > vals[threadIdx.x] || (ov == vals[threadIdx.x] && oa < args[threadIdx.x])) {
                vals[threadIdx.x] = ov;
                args[threadIdx.x] = oa;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const int a = args[0];
        double p = y_pred[r0 + a];
        p = p < eps ? eps : (p > 1.0 - eps ? 1.0 - eps : p);
        row_loss[blockIdx.x] = log(p);
        dx[r0 + a] = vals[0] / (-p * global_batch);
    }
}

__global__ void cce_loss_f64_kernel(const double* __restrict__ row_loss, double* __restrict__ loss, int rows)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    double s = 0.0;
    for (int r = 0; r < rows; ++r) s += row_loss[r];
    loss[0] = -s / rows;
}

// pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41
__global__ void __launch_bounds__(kT) sgd_momentum_f64_kernel(double* __restrict__ w, const double* __restrict__ dw,
                                                             double* __restrict__ velocity, long total, double lr,
                                                             double momentum, double decay, int nesterov)
{
    const long idx = (long)blockIdx.x * kT + threadIdx.x;
    if (idx >= total) return;
    const double g = dw[idx];
    const double v = momentum * velocity[idx] + g;
    const double wv = w[idx];
    const double upd = nesterov ? (decay * wv + g + momentum * v) : (decay * wv + v);
    w[idx] = wv - lr * upd;
    velocity[idx] = v;
}

// ---------------------------------------------------------------- BatchNormalization, training
// pydtnn/backends/cpu/layers/batch_normalization_cpu.py:59-82 on x viewed as (outer, channels, inner): one
// workgroup per channel takes the mean, then the mean of the squared deviations (two passes, as the reference),
// then normalises.
__device__ __forceinline__ long chan_elem(long i, int ch, int channels, long inner)
{
    const long o = i / inner, p = i - o * inner;
    return (o * channels + ch) * inner + p;
}

__global__ void __launch_bounds__(kT) bn_train_fwd_f64_kernel(const double* __restrict__ x, double* __restrict__ y,
                                                             double* __restrict__ xn, double* __restrict__ std_out,
                                                             const double* __restrict__ gamma,
                                                             const double* __restrict__ beta, double* running_mean,
                                                             double* running_var, double momentum, double eps,
                                                             long outer, int channels, long inner)
{
    __shared__ double part[kT];
    const int ch = blockIdx.x;
    const long count = outer * inner;
    double s = 0.0;
    for (long i = threadIdx.x; i < count; i += kT) s += x[chan_elem(i, ch, channels, inner)];
    const double mu = block_sum(s, part) / (double)count;
    double q = 0.0;
    for (long i = threadIdx.x; i < count; i += kT) {
        const double d = x[chan_elem(i, ch, channels, inner)] - mu;
        q += d * d;
    }
    const double var = block_sum(q, part) / (double)count;
    const double sd = sqrt(var + eps);
    const double gm = gamma[ch], bt = beta[ch];
    for (long i = threadIdx.x; i < count; i += kT) {
        const long e = chan_elem(i, ch, channels, inner);
        const double n = (x[e] - mu) / sd;
        xn[e] = n;
        y[e] = gm * n + bt;
    }
    if (threadIdx.x == 0) {
        std_out[ch] = sd;
        running_mean[ch] = momentum * running_mean[ch] + (1.0 - momentum) * mu;
        running_var[ch] = momentum * running_var[ch] + (1.0 - momentum) * var;
    }
}

// :108-129 with dx of pydtnn/cython_modules/bn_training_cython.pyx:236-243
__global__ void __launch_bounds__(kT) bn_train_bwd_f64_kernel(const double* __restrict__ dy, const double* __restrict__ xn,
                                                             const double* __restrict__ std_in,
                                                             const double* __restrict__ gamma, double* __restrict__ dgamma,
                                                             double* __restrict__ dbeta, double* __restrict__ dx,
                                                             long outer, int channels, long inner)
{
    __shared__ double part[kT];
    const int ch = blockIdx.x;
    const long count = outer * inner;
    double sg = 0.0, sb = 0.0;
    for (long i = threadIdx.x; i < count; i += kT) {
        const long e = chan_elem(i, ch, channels, inner);
        sg += dy[e] * xn[e];
        sb += dy[e];
    }
    const double dg = block_sum(sg, part);
    const double db = block_sum(sb, part);
    if (threadIdx.x == 0) {
        dgamma[ch] = dg;
        dbeta[ch] = db;
    }
    if (!dx) return;
    const double nf = (double)count;
    const double scale = gamma[ch] / (std_in[ch] * nf);
    for (long i = threadIdx.x; i < count; i += kT) {
        const long e = chan_elem(i, ch, channels, inner);
        dx[e] = scale * (nf * dy[e] - xn[e] * dg - db);
    }
}

int pool_geom(ConvGeom* g, int b, int c, int h, int w, int kh, int kw, int vpadding, int hpadding, int vstride,
              int hstride, int vdilation, int hdilation)
{
    return make_conv_geom(g, b, c, h, w, 1, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
}

#define POOL64_ARGS b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation

}  // namespace

extern "C" {

int pydtnn_hip_max_pool_2d_fwd_f64(int nhwc, const double* x, double* y, int32_t* idx_max, int b, int c, int h, int w,
                                   int kh, int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                   int hdilation, void* stream)
{
    if (!x || !y || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = pool_geom(&g, POOL64_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.ho * g.wo;
    const hipStream_t st = convint::as_stream(stream);
    if (nhwc) hipLaunchKernelGGL(max_pool_fwd_f64_kernel<true>, dim3(blocks_for(total)), dim3(kT), 0, st, x, y, idx_max, g, total);
    else hipLaunchKernelGGL(max_pool_fwd_f64_kernel<false>, dim3(blocks_for(total)), dim3(kT), 0, st, x, y, idx_max, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_max_pool_2d_bwd_f64(int nhwc, const double* dy, const int32_t* idx_max, double* dx, int b, int c, int h,
                                   int w, int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                   int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = pool_geom(&g, POOL64_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.h * g.w;
    const hipStream_t st = convint::as_stream(stream);
    if (nhwc) hipLaunchKernelGGL(max_pool_bwd_f64_kernel<true>, dim3(blocks_for(total)), dim3(kT), 0, st, dy, idx_max, dx, g, total);
    else hipLaunchKernelGGL(max_pool_bwd_f64_kernel<false>, dim3(blocks_for(total)), dim3(kT), 0, st, dy, idx_max, dx, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_average_pool_2d_fwd_f64(int nhwc, const double* x, double* y, int b, int c, int h, int w, int kh, int kw,
                                       int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = pool_geom(&g, POOL64_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.ho * g.wo;
    const hipStream_t st = convint::as_stream(stream);
    if (nhwc) hipLaunchKernelGGL(avg_pool_fwd_f64_kernel<true>, dim3(blocks_for(total)), dim3(kT), 0, st, x, y, g, total);
    else hipLaunchKernelGGL(avg_pool_fwd_f64_kernel<false>, dim3(blocks_for(total)), dim3(kT), 0, st, x, y, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_average_pool_2d_bwd_f64(int nhwc, const double* dy, double* dx, int b, int c, int h, int w, int kh,
                                       int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation, void* stream)
{
    if (!dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = pool_geom(&g, POOL64_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.h * g.w;
    const hipStream_t st = convint::as_stream(stream);
    if (nhwc) hipLaunchKernelGGL(avg_pool_bwd_f64_kernel<true>, dim3(blocks_for(total)), dim3(kT), 0, st, dy, dx, g, total);
    else hipLaunchKernelGGL(avg_pool_bwd_f64_kernel<false>, dim3(blocks_for(total)), dim3(kT), 0, st, dy, dx, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_softmax_fwd_f64(const double* x, double* y, int rows, int cols, void* stream)
{
    if (!x || !y || rows <= 0 || cols <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(softmax_fwd_f64_kernel, dim3((unsigned)rows), dim3(kT), 0, convint::as_stream(stream), x, y, cols);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_softmax_bwd_f64(const double* dy, const double* y, double* dx, int rows, int cols, void* stream)
{
    if (!dy || !y || !dx || rows <= 0 || cols <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(softmax_bwd_f64_kernel, dim3((unsigned)rows), dim3(kT), 0, convint::as_stream(stream), dy, y, dx,
                       cols);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_categorical_cross_entropy_f64(const double* y_pred, const double* y_targ, double* dx, double* loss,
                                             int rows, int cols, double eps, int global_batch, void* workspace,
                                             size_t workspace_bytes, void* stream)
{
    if (!y_pred || !y_targ || !dx || !loss || rows <= 0 || cols <= 0 || global_batch <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < (size_t)rows * 8) return PYDTNN_HIP_ERR_WORKSPACE;
    double* row_loss = static_cast<double*>(workspace);
    const hipStream_t st = convint::as_stream(stream);
    hipLaunchKernelGGL(cce_rows_f64_kernel, dim3((unsigned)rows), dim3(kT), 0, st, y_pred, y_targ, dx, row_loss, cols, eps,
                       (double)global_batch);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(cce_loss_f64_kernel, dim3(1), dim3(64), 0, st, row_loss, loss, rows);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_sgd_momentum_f64(double* w, const double* dw, double* velocity, long total, double lr, double momentum,
                                double decay, int nesterov, void* stream)
{
    if (!w || !dw || !velocity || total <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(sgd_momentum_f64_kernel, dim3(blocks_for(total)), dim3(kT), 0, convint::as_stream(stream), w, dw,
                       velocity, total, lr, momentum, decay, nesterov);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_bn_training_fwd_f64(const double* x, double* y, double* xn, double* std_out, const double* gamma,
                                   const double* beta, double* running_mean, double* running_var, double momentum,
                                   double eps, long outer, int channels, long inner, void* stream)
{
    if (!x || !y || !xn || !std_out || !gamma || !beta || !running_mean || !running_var) return PYDTNN_HIP_ERR_INVALID;
    if (outer <= 0 || channels <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(bn_train_fwd_f64_kernel, dim3((unsigned)channels), dim3(kT), 0, convint::as_stream(stream), x, y,
                       xn, std_out, gamma, beta, running_mean, running_var, momentum, eps, outer, channels, inner);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_bn_training_bwd_f64(const double* dy, const double* xn, const double* std_in, const double* gamma,
                                   double* dgamma, double* dbeta, double* dx, long outer, int channels, long inner,
                                   void* stream)
{
    if (!dy || !xn || !std_in || !gamma || !dgamma || !dbeta) return PYDTNN_HIP_ERR_INVALID;
    if (outer <= 0 || channels <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(bn_train_bwd_f64_kernel, dim3((unsigned)channels), dim3(kT), 0, convint::as_stream(stream), dy, xn,
                       std_in, gamma, dgamma, dbeta, dx, outer, channels, inner);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

}  // extern "C"

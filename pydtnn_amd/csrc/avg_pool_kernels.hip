// AveragePool2D forward / backward for both tensor formats
// (pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:83-108, :198-227 and the NHWC twins).
// One thread per output element (forward) or per input element (backward, gather form: the windows that
// cover an input pixel are visited in ascending (row, column) order, which is the order in which the
// reference's scatter adds them, so the fp32 sums are the same bits).  These layers move a few megabytes
// (ResNet's global pooling of 7x7 planes); nothing here is tuned beyond coalesced indexing.
#include "conv_internal.h"

namespace {

// Taps of a window along one axis that lie inside the image.
__device__ __forceinline__ int taps_inside(int first, int taps, int dilation, int extent)
{
    int n = 0;
    for (int t = 0; t < taps; ++t) n += (unsigned)(first + t * dilation) < (unsigned)extent;
    return n;
}

template <bool NHWC>
__global__ void __launch_bounds__(256) avg_pool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                           ConvGeom g, long total)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int nn, cc, xx, yy;
    long r = i;
    if (NHWC) {
        cc = (int)(r % g.c); r /= g.c;
        yy = (int)(r % g.wo); r /= g.wo;
        xx = (int)(r % g.ho); nn = (int)(r / g.ho);
    } else {
        yy = (int)(r % g.wo); r /= g.wo;
        xx = (int)(r % g.ho); r /= g.ho;
        cc = (int)(r % g.c); nn = (int)(r / g.c);
    }
    float accum = 0.0f;
    int items = 0;
    for (int ii = 0; ii < g.kh; ++ii) {
        const int x_x = g.vstride * xx + g.vdilation * ii - g.vpadding;
        if ((unsigned)x_x >= (unsigned)g.h) continue;
        for (int jj = 0; jj < g.kw; ++jj) {
            const int x_y = g.hstride * yy + g.hdilation * jj - g.hpadding;
            if ((unsigned)x_y >= (unsigned)g.w) continue;
            const long src = NHWC ? (((long)nn * g.h + x_x) * g.w + x_y) * g.c + cc
                                  : (((long)nn * g.c + cc) * g.h + x_x) * g.w + x_y;
            accum = accum + x[src];
            ++items;
        }
    }
    y[i] = accum / (float)items;
}

template <bool NHWC>
__global__ void __launch_bounds__(256) avg_pool_bwd_kernel(const float* __restrict__ dy, float* __restrict__ dx,
                                                           ConvGeom g, long total)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int nn, cc, ih, iw;
    long r = i;
    if (NHWC) {
        cc = (int)(r % g.c); r /= g.c;
        iw = (int)(r % g.w); r /= g.w;
        ih = (int)(r % g.h); nn = (int)(r / g.h);
    } else {
        iw = (int)(r % g.w); r /= g.w;
        ih = (int)(r % g.h); r /= g.h;
        cc = (int)(r % g.c); nn = (int)(r / g.c);
    }
    // window (xx, yy) covers the pixel through tap (ii, jj) when vstride*xx + vdilation*ii - vpadding == ih;
    // descending taps give ascending windows
    float acc = 0.0f;
    for (int ii = g.kh - 1; ii >= 0; --ii) {
        const int num_v = ih + g.vpadding - g.vdilation * ii;
        if (num_v < 0 || num_v % g.vstride != 0) continue;
        const int xx = num_v / g.vstride;
        if (xx >= g.ho) continue;
        const int cnt_v = taps_inside(g.vstride * xx - g.vpadding, g.kh, g.vdilation, g.h);
        for (int jj = g.kw - 1; jj >= 0; --jj) {
            const int num_h = iw + g.hpadding - g.hdilation * jj;
            if (num_h < 0 || num_h % g.hstride != 0) continue;
            const int yy = num_h / g.hstride;
            if (yy >= g.wo) continue;
            const int items = cnt_v * taps_inside(g.hstride * yy - g.hpadding, g.kw, g.hdilation, g.w);
            const long src = NHWC ? (((long)nn * g.ho + xx) * g.wo + yy) * g.c + cc
                                  : (((long)nn * g.c + cc) * g.ho + xx) * g.wo + yy;
            acc += dy[src] / (float)items;
        }
    }
    dx[i] = acc;
}

}  // namespace

int launch_avg_pool_fwd(int nhwc, const float* x, float* y, const ConvGeom& g, hipStream_t stream)
{
    const long total = (long)g.n * g.c * g.ho * g.wo;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (nhwc)
        hipLaunchKernelGGL(avg_pool_fwd_kernel<true>, dim3(blocks), dim3(256), 0, stream, x, y, g, total);
    else
        hipLaunchKernelGGL(avg_pool_fwd_kernel<false>, dim3(blocks), dim3(256), 0, stream, x, y, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_avg_pool_bwd(int nhwc, const float* dy, float* dx, const ConvGeom& g, hipStream_t stream)
{
    const long total = (long)g.n * g.c * g.h * g.w;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (nhwc)
        hipLaunchKernelGGL(avg_pool_bwd_kernel<true>, dim3(blocks), dim3(256), 0, stream, dy, dx, g, total);
    else
        hipLaunchKernelGGL(avg_pool_bwd_kernel<false>, dim3(blocks), dim3(256), 0, stream, dy, dx, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

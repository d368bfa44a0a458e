// im2col / col2im (NCHW) and im2row / row2im (NHWC) for gfx950.
//
// Index contract (bit-exact with PyDTNN's Cython modules):
//   NCHW  cols[c*kh*kw + i*kw + j, n*ho*wo + y*wo + x] = X[n, c, sv*y + dv*i - pv, sh*x + dh*j - ph]
//         (pydtnn/cython_modules/im2col_nchw_cython.pyx:104-124), zero outside the image.
//   NHWC  rows[n*ho*wo + y*wo + x, c*kh*kw + i*kw + j] = X[n, sv*y + dv*i - pv, sh*x + dh*j - ph, c]
//         (pydtnn/cython_modules/im2row_nhwc_cython.pyx:77-97): K stays channel-major in NHWC.
// The adjoints (col2im :224-244, row2im :174-194) are written in gather form: one thread owns one
// image element and adds its taps in the order in which the reference's scatter loop reaches that
// element (col2im: taps (i, j) ascending, its outer loops; row2im: output pixels (y, x) ascending,
// i.e. taps descending), so fp32 results are reproducible and equal to the reference's sums; no
// atomics, no pre-zeroed output needed.
//
// All four are HBM-bound streams: every matrix element is written (or read) once, lanes run along
// the contiguous axis of the matrix, and padding zeros are produced in the same pass.
#include "common.h"

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------- im2col NCHW
// grid.y = matrix row (c,i,j); grid.x * 256 threads * 4 columns walk the row.
template <bool VEC4>
__global__ void __launch_bounds__(kThreads) im2col_nchw_kernel(const float* __restrict__ x,
                                                              float* __restrict__ cols, ConvGeom g)
{
    const int row = blockIdx.y;
    const int cc = row / g.khw;
    const int rem = row - cc * g.khw;
    const int ii = rem / g.kw;
    const int jj = rem - ii * g.kw;
    const int di = g.vdilation * ii - g.vpadding;
    const int dj = g.hdilation * jj - g.hpadding;

    const long col0 = ((long)blockIdx.x * kThreads + threadIdx.x) * 4;
    if (col0 >= g.p) return;
    int nn = (int)(col0 / g.howo);
    int pp = (int)(col0 - (long)nn * g.howo);
    int yy = pp / g.wo;
    int xx = pp - yy * g.wo;

    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float val = 0.0f;
        if (col0 + e < g.p) {
            const int x_x = g.vstride * yy + di;
            const int x_y = g.hstride * xx + dj;
            if ((unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w)
                val = x[(((long)nn * g.c + cc) * g.h + x_x) * g.w + x_y];
        }
        v[e] = val;
        if (++xx == g.wo) {
            xx = 0;
            if (++yy == g.ho) { yy = 0; ++nn; }
        }
    }
    float* dst = cols + (long)row * g.p + col0;
    if (VEC4) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col0 + e < g.p) dst[e] = v[e];
    }
}

// ---------------------------------------------------------------- col2im NCHW (gather form)
// One thread per dx element; lanes along w.
__global__ void __launch_bounds__(kThreads) col2im_nchw_kernel(const float* __restrict__ cols,
                                                              float* __restrict__ dx, ConvGeom g)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    const long total = (long)g.n * g.c * g.h * g.w;
    if (idx >= total) return;
    const int ww = (int)(idx % g.w);
    long t = idx / g.w;
    const int hh = (int)(t % g.h);
    t /= g.h;
    const int cc = (int)(t % g.c);
    const int nn = (int)(t / g.c);

    float acc = 0.0f;
    for (int ii = 0; ii < g.kh; ++ii) {
        const int ty = hh + g.vpadding - g.vdilation * ii;
        if (ty < 0) continue;
        const int oy = ty / g.vstride;
        if (oy * g.vstride != ty || oy >= g.ho) continue;
        for (int jj = 0; jj < g.kw; ++jj) {
            const int tx = ww + g.hpadding - g.hdilation * jj;
            if (tx < 0) continue;
            const int ox = tx / g.hstride;
            if (ox * g.hstride != tx || ox >= g.wo) continue;
            const long row = (long)cc * g.khw + ii * g.kw + jj;
            const long col = (long)nn * g.howo + oy * g.wo + ox;
            acc += cols[row * g.p + col];
        }
    }
    dx[idx] = acc;
}

// ---------------------------------------------------------------- im2row NHWC
// One thread per matrix element; lanes along the K axis (c,i,j) of one pixel row.
__global__ void __launch_bounds__(kThreads) im2row_nhwc_kernel(const float* __restrict__ x,
                                                              float* __restrict__ rows, ConvGeom g)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    const long total = g.p * g.k;
    if (idx >= total) return;
    const int col = (int)(idx % g.k);
    const long row = idx / g.k;
    const int cc = col / g.khw;
    const int rem = col - cc * g.khw;
    const int ii = rem / g.kw;
    const int jj = rem - ii * g.kw;
    const int nn = (int)(row / g.howo);
    const int pp = (int)(row - (long)nn * g.howo);
    const int yy = pp / g.wo;
    const int xx = pp - yy * g.wo;
    const int x_x = g.vstride * yy + g.vdilation * ii - g.vpadding;
    const int x_y = g.hstride * xx + g.hdilation * jj - g.hpadding;
    float val = 0.0f;
    if ((unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w)
        val = x[(((long)nn * g.h + x_x) * g.w + x_y) * g.c + cc];
    rows[idx] = val;
}

// ---------------------------------------------------------------- row2im NHWC (gather form)
// One thread per dx element; lanes along c.
__global__ void __launch_bounds__(kThreads) row2im_nhwc_kernel(const float* __restrict__ rows,
                                                              float* __restrict__ dx, ConvGeom g)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    const long total = (long)g.n * g.h * g.w * g.c;
    if (idx >= total) return;
    const int cc = (int)(idx % g.c);
    long t = idx / g.c;
    const int ww = (int)(t % g.w);
    t /= g.w;
    const int hh = (int)(t % g.h);
    const int nn = (int)(t / g.h);

    float acc = 0.0f;
    // ascending output pixel (oy, ox) == descending tap (ii, jj): the order of the reference's n,y,x-major loop
    for (int ii = g.kh - 1; ii >= 0; --ii) {
        const int ty = hh + g.vpadding - g.vdilation * ii;
        if (ty < 0) continue;
        const int oy = ty / g.vstride;
        if (oy * g.vstride != ty || oy >= g.ho) continue;
        for (int jj = g.kw - 1; jj >= 0; --jj) {
            const int tx = ww + g.hpadding - g.hdilation * jj;
            if (tx < 0) continue;
            const int ox = tx / g.hstride;
            if (ox * g.hstride != tx || ox >= g.wo) continue;
            const long row = (long)nn * g.howo + oy * g.wo + ox;
            const long col = (long)cc * g.khw + ii * g.kw + jj;
            acc += rows[row * g.k + col];
        }
    }
    dx[idx] = acc;
}

inline unsigned blocks_for(long total) { return (unsigned)((total + kThreads - 1) / kThreads); }

}  // namespace

int make_conv_geom(ConvGeom* g, int n, int c, int h, int w, int kn, int kh, int kw,
                   int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation)
{
    if (n <= 0 || c <= 0 || h <= 0 || w <= 0 || kn <= 0 || kh <= 0 || kw <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (vpadding < 0 || hpadding < 0 || vstride <= 0 || hstride <= 0 || vdilation <= 0 || hdilation <= 0)
        return PYDTNN_HIP_ERR_INVALID;
    g->n = n; g->c = c; g->h = h; g->w = w;
    g->kn = kn; g->kh = kh; g->kw = kw;
    g->vpadding = vpadding; g->hpadding = hpadding;
    g->vstride = vstride; g->hstride = hstride;
    g->vdilation = vdilation; g->hdilation = hdilation;
    g->ho = conv_out_dim(h, vpadding, vdilation, kh, vstride);
    g->wo = conv_out_dim(w, hpadding, hdilation, kw, hstride);
    if (g->ho <= 0 || g->wo <= 0) return PYDTNN_HIP_ERR_INVALID;
    g->khw = kh * kw;
    const long k = (long)c * g->khw;
    const long howo = (long)g->ho * g->wo;
    g->p = (long)n * howo;
    // The kernels index x, y and one image's pixels with 32-bit ints and divide k, pixel and
    // channel indices with FastDiv; refuse extents those do not cover.
    // Tensors are addressed through buffer descriptors of less than 2 GiB (2^29 floats), and the
    // loaders pack tap / pixel offsets into 16-bit fields.
    const long lim = 1l << 29;
    if (k >= (1l << 24) || howo >= (1l << 24) || (long)n * c * h * w >= lim || g->p * kn >= lim ||
        (long)kn * k >= lim)
        return PYDTNN_HIP_ERR_UNSUPPORTED;
    if (h + 2 * vpadding >= 8192 || w + 2 * hpadding >= 8192 || (kh - 1) * vdilation >= 8192 ||
        (kw - 1) * hdilation >= 8192)
        return PYDTNN_HIP_ERR_UNSUPPORTED;
    g->k = (int)k;
    g->howo = (int)howo;
    const unsigned long two32 = 1ul << 32;
    if ((unsigned long)(k + 256) * g->khw >= two32 || (unsigned long)(g->khw + 256) * kw >= two32 ||
        (unsigned long)(howo + 256) * g->wo >= two32 || (unsigned long)(k + 256) * c >= two32)
        return PYDTNN_HIP_ERR_UNSUPPORTED;
    g->fd_khw = make_fastdiv((uint32_t)g->khw);
    g->fd_kw = make_fastdiv((uint32_t)kw);
    g->fd_wo = make_fastdiv((uint32_t)g->wo);
    g->fd_c = make_fastdiv((uint32_t)c);
    g->fd_howo = make_fastdiv((uint32_t)g->howo);
    return PYDTNN_HIP_OK;
}

int launch_im2col_nchw(const float* x, float* cols, const ConvGeom& g, hipStream_t stream)
{
    if (g.k > 65535) return PYDTNN_HIP_ERR_UNSUPPORTED;
    dim3 grid((unsigned)((g.p + (long)kThreads * 4 - 1) / ((long)kThreads * 4)), (unsigned)g.k);
    const bool vec = (g.p % 4 == 0) && ((reinterpret_cast<uintptr_t>(cols) & 15) == 0);
    if (vec)
        hipLaunchKernelGGL(im2col_nchw_kernel<true>, grid, dim3(kThreads), 0, stream, x, cols, g);
    else
        hipLaunchKernelGGL(im2col_nchw_kernel<false>, grid, dim3(kThreads), 0, stream, x, cols, g);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_col2im_nchw(const float* cols, float* dx, const ConvGeom& g, hipStream_t stream)
{
    const long total = (long)g.n * g.c * g.h * g.w;
    hipLaunchKernelGGL(col2im_nchw_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, cols, dx, g);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_im2row_nhwc(const float* x, float* rows, const ConvGeom& g, hipStream_t stream)
{
    const long total = g.p * g.k;
    if ((total + kThreads - 1) / kThreads >= (1l << 31)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(im2row_nhwc_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, x, rows, g);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_row2im_nhwc(const float* rows, float* dx, const ConvGeom& g, hipStream_t stream)
{
    const long total = (long)g.n * g.h * g.w * g.c;
    hipLaunchKernelGGL(row2im_nhwc_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, rows, dx, g);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

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
#include "gemm_engine.h"

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------- im2col NCHW
// The matrix is kh*kw times larger than the image, so the kernel is a store stream and anything
// it re-reads from L2 competes with that stream for the same fabric.  A block therefore stages
// the input rows its pixels need in LDS once (coalesced loads of one contiguous piece of an
// (n, c) plane) and produces all kh*kw matrix rows of its channel from there.
//   grid.x = image * chunks + chunk (a chunk is `chunk_px` consecutive output pixels of one image)
//   grid.y = input channel;  256 threads * 4 consecutive pixels each.
// Index arithmetic is 32-bit (tensors hold fewer than 2^29 floats) with multiply-high divisions.
template <bool VEC4>
__global__ void __launch_bounds__(kThreads) im2col_nchw_lds_kernel(const float* __restrict__ x,
                                                                  float* __restrict__ cols, ConvGeom g,
                                                                  int chunks, int chunk_px)
{
    extern __shared__ float win[];
    const uint32_t cc = blockIdx.y;
    const uint32_t nn = blockIdx.x / (uint32_t)chunks;
    const uint32_t chunk = blockIdx.x - nn * chunks;
    const uint32_t pp_begin = chunk * (uint32_t)chunk_px;
    const uint32_t pp_stop = pp_begin + chunk_px;
    const uint32_t pp_end = pp_stop < (uint32_t)g.howo ? pp_stop : (uint32_t)g.howo;
    if (pp_begin >= pp_end) return;  // uniform

    // Input rows touched by output rows y0..y1, clipped to the image.
    const int y0 = (int)(pp_begin / (uint32_t)g.wo), y1 = (int)((pp_end - 1) / (uint32_t)g.wo);
    int r0 = g.vstride * y0 - g.vpadding;
    int r1 = g.vstride * y1 + g.vdilation * (g.kh - 1) - g.vpadding;
    r0 = r0 < 0 ? 0 : r0;
    r1 = r1 > g.h - 1 ? g.h - 1 : r1;
    const float* plane = x + (size_t)(nn * g.c + cc) * g.h * g.w;
    const int start = r0 * g.w, end = (r1 + 1) * g.w;
    // eight loads in flight per thread before the first LDS store
    for (int i0 = start + (int)threadIdx.x; i0 < end; i0 += 8 * kThreads) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kThreads;
            v[u] = plane[i < end ? i : start];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kThreads;
            if (i < end) win[i - start] = v[u];
        }
    }
    __syncthreads();

    const uint32_t pp = pp_begin + threadIdx.x * 4;
    if (pp >= pp_end) return;
    uint32_t yy = fd_div(pp, g.fd_wo);
    uint32_t xx = pp - yy * g.wo;
    int iy0[4], ix0[4];
    bool live[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        iy0[e] = g.vstride * (int)yy - g.vpadding;
        ix0[e] = g.hstride * (int)xx - g.hpadding;
        live[e] = pp + e < pp_end;
        if (++xx == (uint32_t)g.wo) { xx = 0; ++yy; }
    }
    float* dst = cols + (size_t)cc * g.khw * g.p + (size_t)nn * g.howo + pp;
    for (int ii = 0; ii < g.kh; ++ii) {
        for (int jj = 0; jj < g.kw; ++jj) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int x_x = iy0[e] + g.vdilation * ii;
                const int x_y = ix0[e] + g.hdilation * jj;
                const bool ok = live[e] && (unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w;
                const float val = win[ok ? (x_x - r0) * g.w + x_y : 0];
                v[e] = ok ? val : 0.0f;
            }
            if (VEC4) {
                // the matrix is written once and read by a later kernel: a streaming store
                const gemm::floatx4 quad = {v[0], v[1], v[2], v[3]};
                __builtin_nontemporal_store(quad, reinterpret_cast<gemm::floatx4*>(dst));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (live[e]) dst[e] = v[e];
            }
            dst += g.p;
        }
    }
}

// Fallback without staging, for windows that do not fit in LDS (large strides or filters on wide
// images): grid.y = matrix row (c,i,j); grid.x * 256 threads * 4 columns walk the row.
template <bool VEC4>
__global__ void __launch_bounds__(kThreads) im2col_nchw_direct_kernel(const float* __restrict__ x,
                                                                     float* __restrict__ cols, ConvGeom g,
                                                                     int p_exact)
{
    const uint32_t row = blockIdx.y;
    const uint32_t cc = fd_div(row, g.fd_khw);
    const uint32_t rem = row - cc * g.khw;
    const uint32_t ii = fd_div(rem, g.fd_kw);
    const uint32_t jj = rem - ii * g.kw;
    const int di = g.vdilation * (int)ii - g.vpadding;
    const int dj = g.hdilation * (int)jj - g.hpadding;

    const uint32_t p = (uint32_t)g.p;
    const uint32_t col0 = (blockIdx.x * kThreads + threadIdx.x) * 4;
    if (col0 >= p) return;
    uint32_t nn = fd_div_checked(col0, g.fd_howo, p_exact);
    const uint32_t pp = col0 - nn * g.howo;
    uint32_t yy = fd_div(pp, g.fd_wo);
    uint32_t xx = pp - yy * g.wo;

    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int x_x = g.vstride * (int)yy + di;
        const int x_y = g.hstride * (int)xx + dj;
        const bool ok = col0 + e < p && (unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w;
        const float val = x[ok ? ((nn * g.c + cc) * g.h + x_x) * g.w + x_y : 0u];
        v[e] = ok ? val : 0.0f;
        if (++xx == (uint32_t)g.wo) {
            xx = 0;
            if (++yy == (uint32_t)g.ho) { yy = 0; ++nn; }
        }
    }
    float* dst = cols + (long)row * g.p + col0;
    if (VEC4) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col0 + e < p) dst[e] = v[e];
    }
}

// Output coordinate reached from input coordinate t = in + pad - dil*tap: t / stride when that is
// exact and inside [0, limit).  UNIT skips the division for stride 1.
template <bool UNIT>
__device__ __forceinline__ bool out_coord(int t, int stride, const FastDiv fd, int limit, int* out)
{
    int o = t;
    bool ok = t >= 0;
    if (!UNIT) {
        o = (int)fd_div((uint32_t)(ok ? t : 0), fd);
        ok = ok && o * stride == t;
    }
    *out = o;
    return ok && o < limit;
}

// ---------------------------------------------------------------- col2im NCHW (gather form)
// grid.x * 256 threads walk one (n, c) plane of dx, grid.y walks the planes; lanes along w.
// Every tap is a clamped load followed by a select, so the loads of one element do not wait for
// each other; adding +0 for a tap outside the matrix leaves the sum unchanged (the accumulator
// starts at +0 and can therefore never hold -0).  KH, KW > 0 fix the filter at compile time so
// that the tap loops unroll; 0 keeps them as run-time loops.
template <bool UNIT, int KH, int KW>
__global__ void __launch_bounds__(kThreads) col2im_nchw_kernel(const float* __restrict__ cols,
                                                              float* __restrict__ dx, ConvGeom g, int remap)
{
    const uint32_t hw = (uint32_t)(g.h * g.w);
    // Workgroups are dealt to the 8 XCDs in turn; renumbered so that each XCD gets a contiguous run of them, the
    // workgroups of one plane (which share the lines of the matrix where their pixel rows meet) fetch through one
    // L2 (FETCH_SIZE 1.14 x the matrix with a plane's workgroups spread over all eight).
    uint32_t bx = blockIdx.x, by = blockIdx.y;
    if (remap) {
        const uint32_t seq = (uint32_t)gemm::xcd_remap((int)(blockIdx.y * gridDim.x + blockIdx.x),
                                                       (int)(gridDim.x * gridDim.y));
        by = seq / gridDim.x;
        bx = seq - by * gridDim.x;
    }
    const uint32_t pix = bx * kThreads + threadIdx.x;
    if (pix >= hw) return;
    const int hh = (int)fd_div(pix, g.fd_w);
    const int ww = (int)pix - hh * g.w;
    const int kh = KH > 0 ? KH : g.kh, kw = KW > 0 ? KW : g.kw;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    for (uint32_t plane = by; plane < planes; plane += gridDim.y) {
        const uint32_t nn = plane / (uint32_t)g.c;
        const uint32_t cc = plane - nn * g.c;
        const float* src = cols + (long)cc * (kh * kw) * g.p + (long)nn * g.howo;
        float acc = 0.0f;
#pragma unroll
        for (int ii = 0; ii < kh; ++ii) {
            int oy = 0;
            const bool row_ok = out_coord<UNIT>(hh + g.vpadding - g.vdilation * ii, g.vstride, g.fd_vs, g.ho, &oy);
#pragma unroll
            for (int jj = 0; jj < kw; ++jj) {
                int ox = 0;
                const bool ok =
                    out_coord<UNIT>(ww + g.hpadding - g.hdilation * jj, g.hstride, g.fd_hs, g.wo, &ox) && row_ok;
                // (a streaming load here measured 4.57 against 5.17 TB/s: neighbouring rows of dx share lines of the
                // matrix through the caches; four pixels per thread with unaligned 128-bit loads 5.09 against 5.24,
                // with 36 scalar loads in flight over chunks of 800 pixels 4.80; planes taken with the image index
                // fastest 5.13)
                const float val = src[(long)(ii * kw + jj) * g.p + (ok ? oy * g.wo + ox : 0)];
                acc += ok ? val : 0.0f;
            }
        }
        dx[(long)plane * hw + pix] = acc;
    }
}

// ---------------------------------------------------------------- im2row NHWC
// One block owns `rpb`
// consecutive pixel rows of the matrix (a contiguous run of rpb*k floats) and its threads walk that
// run, so stores are fully coalesced; the block's first pixel is decomposed once with scalar
// arithmetic and each element only needs multiply-high divisions.
__global__ void __launch_bounds__(kThreads) im2row_nhwc_kernel(const float* __restrict__ x,
                                                              float* __restrict__ rows, ConvGeom g, int rpb,
                                                              FastDiv fd_k)
{
    const uint32_t row0 = blockIdx.x * (uint32_t)rpb;
    const uint32_t left = (uint32_t)g.p - row0;
    const uint32_t nrows = left < (uint32_t)rpb ? left : (uint32_t)rpb;
    const uint32_t n0 = row0 / (uint32_t)g.howo;
    const uint32_t pp0 = row0 - n0 * g.howo;
    const uint32_t count = nrows * (uint32_t)g.k;
    float* dst = rows + (long)row0 * g.k;
    // four elements per trip: their loads are issued together (clamped index, then select)
    for (uint32_t e0 = threadIdx.x; e0 < count; e0 += 4 * kThreads) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t e = e0 + u * kThreads;
            const uint32_t ec = e < count ? e : 0u;
            const uint32_t r = rpb > 1 ? fd_div(ec, fd_k) : 0u;
            const uint32_t col = ec - r * g.k;
            uint32_t pp = pp0 + r, nn = n0;
            if (pp >= (uint32_t)g.howo) { pp -= g.howo; ++nn; }  // rpb <= howo: at most one wrap
            const uint32_t yy = fd_div(pp, g.fd_wo);
            const uint32_t xx = pp - yy * g.wo;
            const uint32_t cc = fd_div(col, g.fd_khw);
            const uint32_t rem = col - cc * g.khw;
            const uint32_t ii = fd_div(rem, g.fd_kw);
            const uint32_t jj = rem - ii * g.kw;
            const int x_x = g.vstride * (int)yy + g.vdilation * (int)ii - g.vpadding;
            const int x_y = g.hstride * (int)xx + g.hdilation * (int)jj - g.hpadding;
            const bool ok = e < count && (unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w;
            const float val = x[ok ? ((nn * g.h + x_x) * g.w + x_y) * g.c + cc : 0u];
            v[u] = ok ? val : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t e = e0 + u * kThreads;
            if (e < count) dst[e] = v[u];
        }
    }
}

// The same matrix for channel counts 4, 8, ..., 1024 and KHW taps, by quads of channels: a thread owns
// (pixel, 4 channels), fetches the quad of every tap with one 128-bit load each (a wavefront reads 1 KB
// runs of x), turns its KHW x 4 values into the row's (channel, tap) order in registers, and the
// workgroup's rows, which are one contiguous run of the matrix, go out through LDS with full-width
// 128-bit stores.  256 / (c/4) pixels per workgroup; LDS 4096 * KHW bytes.
template <int KHW>
__global__ void __launch_bounds__(kThreads) im2row_nhwc_quads_kernel(const float* __restrict__ x,
                                                                    float* __restrict__ rows, ConvGeom g)
{
    __shared__ float4 staged[kThreads * KHW];
    const int c4n = g.c >> 2, rows_per_block = kThreads / c4n;
    const int r = threadIdx.x / c4n, q = threadIdx.x - r * c4n;
    // each XCD takes one contiguous run of pixels, so the taps its workgroups share come from its own L2
    const long p0 = (long)gemm::xcd_remap((int)blockIdx.x, (int)gridDim.x) * rows_per_block;
    const long p = p0 + r;
    float4 v[KHW];
#pragma unroll
    for (int t = 0; t < KHW; ++t) v[t] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (p < g.p) {
        const uint32_t nn = (uint32_t)(p / g.howo);
        const uint32_t pp = (uint32_t)(p - (long)nn * g.howo);
        const uint32_t yy = fd_div(pp, g.fd_wo);
        const uint32_t xx = pp - yy * g.wo;
        const int ih0 = g.vstride * (int)yy - g.vpadding, iw0 = g.hstride * (int)xx - g.hpadding;
        const float* src = x + ((size_t)nn * g.h * g.w) * g.c + 4 * q;
#pragma unroll
        for (int t = 0; t < KHW; ++t) {
            const int ii = (int)fd_div((uint32_t)t, g.fd_kw), jj = t - ii * g.kw;
            const int x_x = ih0 + g.vdilation * ii, x_y = iw0 + g.hdilation * jj;
            if ((unsigned)x_x < (unsigned)g.h && (unsigned)x_y < (unsigned)g.w)
                v[t] = *reinterpret_cast<const float4*>(src + (size_t)(x_x * g.w + x_y) * g.c);
        }
    }
    // (tap, channel) -> (channel, tap): element u*KHW + t of the thread's run is channel u of tap t
    float run[4 * KHW];
#pragma unroll
    for (int t = 0; t < KHW; ++t) {
        run[0 * KHW + t] = v[t].x;
        run[1 * KHW + t] = v[t].y;
        run[2 * KHW + t] = v[t].z;
        run[3 * KHW + t] = v[t].w;
    }
    float4* mine = staged + (size_t)threadIdx.x * KHW;  // thread (r, q) owns floats [(r*c4n + q) * 4*KHW, +4*KHW)
#pragma unroll
    for (int t = 0; t < KHW; ++t) mine[t] = make_float4(run[4 * t], run[4 * t + 1], run[4 * t + 2], run[4 * t + 3]);
    __syncthreads();
    const long left = g.p - p0;
    const long valid4 = (left < rows_per_block ? left : (long)rows_per_block) * c4n * KHW;  // float4s of this block
    gemm::floatx4* dst = reinterpret_cast<gemm::floatx4*>(rows + p0 * g.k);
#pragma unroll
    for (int t = 0; t < KHW; ++t) {
        const int f4 = t * kThreads + threadIdx.x;
        if (f4 < valid4) {
            const float4 q = staged[f4];
            const gemm::floatx4 quad = {q.x, q.y, q.z, q.w};
            __builtin_nontemporal_store(quad, dst + f4);   // written once, read by a later kernel
        }
    }
}

// ---------------------------------------------------------------- row2im NHWC (gather form)
// grid.x * 256 threads walk one image of dx (h*w*c floats, lanes along c), grid.y walks
// the images.
template <bool UNIT>
__global__ void __launch_bounds__(kThreads) row2im_nhwc_kernel(const float* __restrict__ rows,
                                                              float* __restrict__ dx, ConvGeom g, int c_exact)
{
    const uint32_t hwc = (uint32_t)(g.h * g.w * g.c);
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= hwc) return;
    const uint32_t t = fd_div_checked(e, g.fd_c, c_exact);
    const uint32_t cc = e - t * g.c;
    const int hh = (int)fd_div(t, g.fd_w);
    const int ww = (int)t - hh * g.w;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const float* src = rows + (long)nn * g.howo * g.k + cc * g.khw;
        float acc = 0.0f;
        // ascending output pixel (oy, ox) == descending tap (ii, jj): the order of the reference's n,y,x-major loop
        for (int ii = g.kh - 1; ii >= 0; --ii) {
            int oy;
            if (!out_coord<UNIT>(hh + g.vpadding - g.vdilation * ii, g.vstride, g.fd_vs, g.ho, &oy)) continue;
            for (int jj = g.kw - 1; jj >= 0; --jj) {
                int ox;
                if (!out_coord<UNIT>(ww + g.hpadding - g.hdilation * jj, g.hstride, g.fd_hs, g.wo, &ox)) continue;
                acc += src[(long)(oy * g.wo + ox) * g.k + ii * g.kw + jj];
            }
        }
        dx[(long)nn * hwc + e] = acc;
    }
}

inline unsigned blocks_for(long total) { return (unsigned)((total + kThreads - 1) / kThreads); }
inline unsigned grid_y_for(long count) { return (unsigned)(count < 65535 ? count : 65535); }
// fd_div(n, d) is exact for every n below `bound` when bound * d < 2^32.
inline int fd_exact(unsigned long bound, unsigned long d) { return bound * d < (1ul << 32); }

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
    // Streaming kernels: pixel index of one input plane by w; pool index by kh; coordinates by the strides.
    if ((unsigned long)((long)h * w + 1024) * w >= two32 || vstride >= 65536 || hstride >= 65536)
        return PYDTNN_HIP_ERR_UNSUPPORTED;
    g->fd_w = make_fastdiv((uint32_t)w);
    g->fd_kh = make_fastdiv((uint32_t)kh);
    g->fd_vs = make_fastdiv((uint32_t)vstride);
    g->fd_hs = make_fastdiv((uint32_t)hstride);
    return PYDTNN_HIP_OK;
}

int launch_im2col_nchw(const float* x, float* cols, const ConvGeom& g, hipStream_t stream)
{
    const bool aligned = (reinterpret_cast<uintptr_t>(cols) & 15) == 0;
    // Staged form: chunks of at most 1024 pixels, about equal within an image and a multiple of 32 long, so that
    // (with images that are a multiple of 32 pixels) every chunk's run of a matrix row starts on a 128-byte line.
    const int chunks = (g.howo + 1023) / 1024;
    const int chunk_px = ((g.howo + chunks - 1) / chunks + 31) & ~31;
    const long rows_out = (chunk_px + g.wo - 2) / g.wo + 1;  // output rows a chunk can straddle
    const long rows_in = (long)g.vstride * (rows_out - 1) + (long)g.vdilation * (g.kh - 1) + 1;
    const long lds_bytes = (rows_in < g.h ? rows_in : g.h) * g.w * 4;
    if (lds_bytes <= 48 * 1024 && g.c <= 65535) {
        dim3 grid((unsigned)((long)g.n * chunks), (unsigned)g.c);
        if (aligned && g.howo % 4 == 0)
            hipLaunchKernelGGL(im2col_nchw_lds_kernel<true>, grid, dim3(kThreads), (size_t)lds_bytes, stream, x, cols,
                               g, chunks, chunk_px);
        else
            hipLaunchKernelGGL(im2col_nchw_lds_kernel<false>, grid, dim3(kThreads), (size_t)lds_bytes, stream, x, cols,
                               g, chunks, chunk_px);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    if (g.k > 65535) return PYDTNN_HIP_ERR_UNSUPPORTED;
    dim3 grid((unsigned)((g.p + (long)kThreads * 4 - 1) / ((long)kThreads * 4)), (unsigned)g.k);
    const int p_exact = fd_exact((unsigned long)g.p + 4 * kThreads, (unsigned long)g.howo);
    if (aligned && g.p % 4 == 0)
        hipLaunchKernelGGL(im2col_nchw_direct_kernel<true>, grid, dim3(kThreads), 0, stream, x, cols, g, p_exact);
    else
        hipLaunchKernelGGL(im2col_nchw_direct_kernel<false>, grid, dim3(kThreads), 0, stream, x, cols, g, p_exact);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_col2im_nchw(const float* cols, float* dx, const ConvGeom& g, hipStream_t stream)
{
    dim3 grid(blocks_for((long)g.h * g.w), grid_y_for((long)g.n * g.c));
    const bool unit = g.vstride == 1 && g.hstride == 1;
    const int remap = (long)grid.x * grid.y < (1l << 31) ? 1 : 0;
    if (unit && g.kh == 3 && g.kw == 3)
        hipLaunchKernelGGL((col2im_nchw_kernel<true, 3, 3>), grid, dim3(kThreads), 0, stream, cols, dx, g, remap);
    else if (unit)
        hipLaunchKernelGGL((col2im_nchw_kernel<true, 0, 0>), grid, dim3(kThreads), 0, stream, cols, dx, g, remap);
    else
        hipLaunchKernelGGL((col2im_nchw_kernel<false, 0, 0>), grid, dim3(kThreads), 0, stream, cols, dx, g, remap);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_im2row_nhwc(const float* x, float* rows, const ConvGeom& g, hipStream_t stream)
{
    // channel quads: c a power of two in 4..1024 (c/4 divides the workgroup), 9 taps, aligned tensors
    const bool pow2 = g.c >= 4 && g.c <= 1024 && (g.c & (g.c - 1)) == 0;
    if (pow2 && g.khw == 9 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(rows)) & 15) == 0) {
        const int rows_per_block = kThreads / (g.c / 4);
        const long blocks = (g.p + rows_per_block - 1) / rows_per_block;
        if (blocks < (1l << 31)) {
            hipLaunchKernelGGL(im2row_nhwc_quads_kernel<9>, dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, rows,
                               g);
            HIP_RETURN_IF_LAUNCH_FAILED();
            return PYDTNN_HIP_OK;
        }
    }
    // About 2048 matrix elements per block, never more rows than one image holds.
    int rpb = 2048 / g.k;
    if (rpb > g.howo) rpb = g.howo;
    if (rpb < 1) rpb = 1;
    if (rpb > 1 && !fd_exact((unsigned long)rpb * g.k + kThreads, (unsigned long)g.k)) rpb = 1;
    const long blocks = (g.p + rpb - 1) / rpb;
    hipLaunchKernelGGL(im2row_nhwc_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, rows, g, rpb,
                       make_fastdiv((uint32_t)g.k));
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

namespace {
// The same sums with the work laid out for the caches: a workgroup owns 8 neighbouring pixels x 32
// channels, so the 1152-byte runs of `rows` it touches (32 channels x 9 taps of one output pixel) are
// shared by its pixels through L1, and the channel chunk is the fastest-running part of the workgroup
// index, so that (workgroups being dealt to the 8 XCDs in turn) a chunk's runs are re-read, for the rows
// of dx above and below, from the same L2.  Needs c % 32 == 0.
template <bool UNIT, int CB>
__global__ void __launch_bounds__(kThreads) row2im_nhwc_patch_kernel(const float* __restrict__ rows,
                                                                    float* __restrict__ dx, ConvGeom g, int chunks)
{
    constexpr int PX = kThreads / CB;
    const uint32_t cb = blockIdx.x % (uint32_t)chunks, pg = blockIdx.x / (uint32_t)chunks;
    const uint32_t t = pg * PX + (threadIdx.x / CB);
    const uint32_t hw = (uint32_t)(g.h * g.w);
    if (t >= hw) return;
    const uint32_t cc = cb * CB + (threadIdx.x % CB);
    const int hh = (int)fd_div(t, g.fd_w);
    const int ww = (int)t - hh * g.w;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const float* src = rows + (long)nn * g.howo * g.k + cc * g.khw;
        float acc = 0.0f;
        for (int ii = g.kh - 1; ii >= 0; --ii) {
            int oy;
            if (!out_coord<UNIT>(hh + g.vpadding - g.vdilation * ii, g.vstride, g.fd_vs, g.ho, &oy)) continue;
            for (int jj = g.kw - 1; jj >= 0; --jj) {
                int ox;
                if (!out_coord<UNIT>(ww + g.hpadding - g.hdilation * jj, g.hstride, g.fd_hs, g.wo, &ox)) continue;
                acc += src[(long)(oy * g.wo + ox) * g.k + ii * g.kw + jj];
            }
        }
        dx[((long)nn * hw + t) * g.c + cc] = acc;
    }
}


// 3x3 taps, unit strides and dilations, c % 32 == 0: the matrix is read once, in full cache lines.
// A workgroup owns (image, band of dx rows, strip of at most 8*S dx columns, chunk of 32 channels) and
// walks down the output rows that feed its band.  The 32 x 9 floats a pixel of the matrix holds for the
// chunk are one 1152-byte run (nine 128-byte lines when the matrix is so aligned); the runs of one output
// row go to LDS through 128-bit loads, next row's loads in flight while this row is consumed.  Thread
// (channel, slot) owns dx columns slot, slot + 8, ...; an output row gives taps i = 2, 1, 0 to the dx rows
// one below, at and one above it (for vpadding 1), so each column keeps three running sums that rotate
// as the walk advances, and a dx element receives its taps in descending (i, j) order as above.  Runs
// outside the matrix read as zeros, which leaves a sum that starts at +0 unchanged.
template <int S>
__global__ void __launch_bounds__(kThreads) row2im_nhwc_walk_kernel(const float* __restrict__ rows,
                                                                   float* __restrict__ dx, ConvGeom g, int strips,
                                                                   int tw, int bands, int band_rows)
{
    constexpr int CB = 32, RUN4 = CB * 9 / 4;              // 72 float4 per (pixel, chunk)
    constexpr int NLD = ((8 * S + 2) * RUN4 + kThreads - 1) / kThreads;
    extern __shared__ float4 walk_lds[];
    const int chunks = g.c / CB;
    uint32_t bid = (uint32_t)gemm::xcd_remap((int)blockIdx.x, (int)gridDim.x);
    const uint32_t cb = bid % (uint32_t)chunks; bid /= (uint32_t)chunks;
    const uint32_t strip = bid % (uint32_t)strips; bid /= (uint32_t)strips;
    const uint32_t band = bid % (uint32_t)bands;
    const uint32_t nn = bid / (uint32_t)bands;
    const int w0 = (int)strip * tw, wn = min(tw, g.w - w0);
    const int h0 = (int)band * band_rows, hn = min(band_rows, g.h - h0);
    const int ox0 = w0 + g.hpadding - 2;                  // output column of LDS column 0
    const int ncols = wn + 2;
    const gemm::rsrc_t src = gemm::make_rsrc(rows + (size_t)nn * g.howo * g.k + cb * (CB * 9), (long)g.howo * g.k - cb * (CB * 9));

    // byte offset of this thread's j-th float4 of an output row, less the row's own offset
    uint32_t off[NLD];
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
        const int f4 = (int)threadIdx.x + j * kThreads;
        const int lc = f4 / RUN4, f = f4 - lc * RUN4;
        const int ox = ox0 + lc;
        off[j] = (lc < ncols && (unsigned)ox < (unsigned)g.wo) ? ((uint32_t)ox * g.k * 4u + (uint32_t)f * 16u) : gemm::kOob;
    }
    auto fetch = [&](int oy, gemm::floatx4* v) {
        const bool row_ok = (unsigned)oy < (unsigned)g.ho;
        const uint32_t soff = row_ok ? (uint32_t)oy * g.wo * g.k * 4u : 0u;
#pragma unroll
        for (int j = 0; j < NLD; ++j)   // streaming loads (cache policy nt): each line of the matrix is read once
            v[j] = __builtin_bit_cast(gemm::floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                src, (int)(row_ok ? off[j] : gemm::kOob), (int)soff, 2));
    };

    const int cc = threadIdx.x & (CB - 1), slot = threadIdx.x / CB;
    const float* mine = reinterpret_cast<const float*>(walk_lds) + (slot * CB + cc) * 9;
    float* out = dx + ((size_t)nn * g.h * g.w + w0 + slot) * g.c + cb * CB + cc;
    float a0[S], a1[S], a2[S];
#pragma unroll
    for (int s = 0; s < S; ++s) a0[s] = a1[s] = a2[s] = 0.0f;

    const int oy_first = h0 + g.vpadding - 2, oy_last = h0 + hn - 1 + g.vpadding;
    gemm::floatx4 v[NLD];
    fetch(oy_first, v);
    for (int oy = oy_first; oy <= oy_last; ++oy) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int f4 = (int)threadIdx.x + j * kThreads;
            if (f4 < (8 * S + 2) * RUN4) walk_lds[f4] = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
        }
        __syncthreads();
        fetch(oy + 1 <= oy_last ? oy + 1 : -1, v);
        // LDS column of tap j for dx column q is q + 2 - j
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const float* px = mine + s * 8 * CB * 9;
            a2[s] = ((a2[s] + px[0 * CB * 9 + 8]) + px[1 * CB * 9 + 7]) + px[2 * CB * 9 + 6];
            a1[s] = ((a1[s] + px[0 * CB * 9 + 5]) + px[1 * CB * 9 + 4]) + px[2 * CB * 9 + 3];
            a0[s] = ((a0[s] + px[0 * CB * 9 + 2]) + px[1 * CB * 9 + 1]) + px[2 * CB * 9 + 0];
        }
        const int hh = oy - g.vpadding;  // the dx row whose last taps this output row held
        if (hh >= h0) {
            float* orow = out + (size_t)hh * g.w * g.c;
#pragma unroll
            for (int s = 0; s < S; ++s)
                if (slot + 8 * s < wn) orow[(size_t)(8 * s) * g.c] = a0[s];
        }
#pragma unroll
        for (int s = 0; s < S; ++s) { a0[s] = a1[s]; a1[s] = a2[s]; a2[s] = 0.0f; }
    }
}

template <int S>
int launch_row2im_walk(const float* rows, float* dx, const ConvGeom& g, int strips, int tw, int bands, int band_rows,
                       hipStream_t stream)
{
    const size_t lds = (size_t)(8 * S + 2) * 32 * 9 * sizeof(float);
    static std::atomic<unsigned> raised{0};
    if (lds > 64 * 1024) {
        const int rc = gemm::raise_lds_limit(reinterpret_cast<const void*>(&row2im_nhwc_walk_kernel<S>), raised, (int)lds);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    const long blocks = (long)g.n * bands * strips * (g.c / 32);
    hipLaunchKernelGGL(row2im_nhwc_walk_kernel<S>, dim3((unsigned)blocks), dim3(kThreads), lds, stream, rows, dx, g,
                       strips, tw, bands, band_rows);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

// 0 when the walk kernel does not cover the geometry.
bool row2im_walk_plan(const ConvGeom& g, const float* rows, int* strips, int* tw, int* bands, int* band_rows)
{
    if (g.kh != 3 || g.kw != 3 || g.vstride != 1 || g.hstride != 1 || g.vdilation != 1 || g.hdilation != 1) return false;
    if (g.c % 32 != 0 || (reinterpret_cast<uintptr_t>(rows) & 15) != 0) return false;
    if ((long)g.howo * g.k >= (1l << 29) || g.vpadding > 2 || g.hpadding > 2) return false;
    *strips = (g.w + 63) / 64;
    *tw = (g.w + *strips - 1) / *strips;
    // whole images while they fill the chip; else bands of rows (each re-reads two output rows)
    const long per_band = (long)g.n * *strips * (g.c / 32);
    int b = 1;
    while (per_band * b < 512 && g.h / (b * 2) >= 8) b *= 2;
    *band_rows = (g.h + b - 1) / b;
    *bands = (g.h + *band_rows - 1) / *band_rows;
    return per_band * *bands < (1l << 31);
}

}  // namespace

int launch_row2im_nhwc(const float* rows, float* dx, const ConvGeom& g, hipStream_t stream)
{
    constexpr int CB = 32;
    int strips, tw, bands, band_rows;
    if (row2im_walk_plan(g, rows, &strips, &tw, &bands, &band_rows)) {
        if (tw <= 8) return launch_row2im_walk<1>(rows, dx, g, strips, tw, bands, band_rows, stream);
        if (tw <= 16) return launch_row2im_walk<2>(rows, dx, g, strips, tw, bands, band_rows, stream);
        if (tw <= 32) return launch_row2im_walk<4>(rows, dx, g, strips, tw, bands, band_rows, stream);
        if (tw <= 56) return launch_row2im_walk<7>(rows, dx, g, strips, tw, bands, band_rows, stream);
        return launch_row2im_walk<8>(rows, dx, g, strips, tw, bands, band_rows, stream);
    }
    if (g.c % CB == 0) {
        const int chunks = g.c / CB;
        const long groups = ((long)g.h * g.w + (kThreads / CB) - 1) / (kThreads / CB);
        if (groups * chunks < (1l << 31)) {
            dim3 pgrid((unsigned)(groups * chunks), grid_y_for(g.n));
            if (g.vstride == 1 && g.hstride == 1)
                hipLaunchKernelGGL((row2im_nhwc_patch_kernel<true, CB>), pgrid, dim3(kThreads), 0, stream, rows, dx, g,
                                   chunks);
            else
                hipLaunchKernelGGL((row2im_nhwc_patch_kernel<false, CB>), pgrid, dim3(kThreads), 0, stream, rows, dx, g,
                                   chunks);
            HIP_RETURN_IF_LAUNCH_FAILED();
            return PYDTNN_HIP_OK;
        }
    }
    const long hwc = (long)g.h * g.w * g.c;
    dim3 grid(blocks_for(hwc), grid_y_for(g.n));
    const int c_exact = fd_exact((unsigned long)hwc + kThreads, (unsigned long)g.c);
    if (g.vstride == 1 && g.hstride == 1)
        hipLaunchKernelGGL(row2im_nhwc_kernel<true>, grid, dim3(kThreads), 0, stream, rows, dx, g, c_exact);
    else
        hipLaunchKernelGGL(row2im_nhwc_kernel<false>, grid, dim3(kThreads), 0, stream, rows, dx, g, c_exact);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

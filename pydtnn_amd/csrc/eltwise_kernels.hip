// HBM-bound helper kernels around the GEMMs: stand-alone bias / BatchNorm-inference / ReLU /
// residual epilogue, ReLU with mask, bias gradient, split-K reduction, filter re-layouts,
// MaxPool2D (NCHW) and the SGD-momentum update.  Each is a single streaming pass with lanes on
// the contiguous axis; algorithmic bytes are stated at each launcher.
#include "common.h"

namespace {

constexpr int kThreads = 256;
inline unsigned blocks_for(long total, int per_block = kThreads)
{
    return (unsigned)((total + per_block - 1) / per_block);
}

// ---------------------------------------------------------------- channel-wise epilogue
// y[idx] = epilogue(ch, x[idx] (+ residual[idx])), ch = (idx / inner) % channels.
// inner = ho*wo for NCHW tensors, 1 for NHWC tensors and 2-D (rows, C) matrices.
// Order: residual add first (pydtnn/cython_modules/eltw_sum_cython.pyx:25-36 is a separate,
// earlier layer in the reference), then bias -> BN -> ReLU as in chan_epilogue_apply.
__global__ void __launch_bounds__(kThreads) chan_eltwise_kernel(const float* __restrict__ x,
                                                               const float* __restrict__ residual,
                                                               float* __restrict__ y, long total, int inner,
                                                               int channels, ChanEpilogue epi)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int ch = (int)((idx / inner) % channels);
    float v = x[idx];
    if (residual) v += residual[idx];
    y[idx] = chan_epilogue_apply(epi, ch, v);
}

// Four consecutive elements per thread; valid when either all four share a channel
// (inner % 4 == 0) or they are four consecutive channels (inner == 1, channels % 4 == 0).
__global__ void __launch_bounds__(kThreads) chan_eltwise_vec4_kernel(const float4* __restrict__ x,
                                                                    const float4* __restrict__ residual,
                                                                    float4* __restrict__ y, long total4, int inner,
                                                                    int channels, ChanEpilogue epi)
{
    const long i4 = (long)blockIdx.x * kThreads + threadIdx.x;
    if (i4 >= total4) return;
    const long idx = i4 * 4;
    const int ch0 = (int)((idx / inner) % channels);
    const int step = inner == 1 ? 1 : 0;
    float4 v = x[i4];
    if (residual) {
        const float4 r = residual[i4];
        v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
    }
    v.x = chan_epilogue_apply(epi, ch0, v.x);
    v.y = chan_epilogue_apply(epi, ch0 + step, v.y);
    v.z = chan_epilogue_apply(epi, ch0 + 2 * step, v.z);
    v.w = chan_epilogue_apply(epi, ch0 + 3 * step, v.w);
    y[i4] = v;
}

// The two layouts that matter, without a division per element and with the per-channel parameters fetched
// once per workgroup / thread instead of once per element.
//
// Planes (NCHW, inner % 4 == 0): grid.y walks the (image, channel) planes, so the channel is uniform in a
// workgroup; grid.x * 256 threads walk one plane's float4s.
__global__ void __launch_bounds__(kThreads) chan_eltwise_planes_kernel(const float4* __restrict__ x,
                                                                      const float4* __restrict__ residual,
                                                                      float4* __restrict__ y, int inner4, int planes,
                                                                      int channels, ChanEpilogue epi)
{
    const int i = blockIdx.x * kThreads + threadIdx.x;
    if (i >= inner4) return;
    for (int plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const int ch = plane % channels;
        const size_t at = (size_t)plane * inner4 + i;
        float4 v = x[at];
        if (residual) {
            const float4 r = residual[at];
            v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
        }
        v.x = chan_epilogue_apply(epi, ch, v.x);
        v.y = chan_epilogue_apply(epi, ch, v.y);
        v.z = chan_epilogue_apply(epi, ch, v.z);
        v.w = chan_epilogue_apply(epi, ch, v.w);
        y[at] = v;
    }
}

// Rows (NHWC and (rows, C) matrices, inner == 1) with C/4 a divisor of 256: a thread keeps one quad of
// channels for all its rows, so its parameters live in registers; 256 / (C/4) rows per pass.
__global__ void __launch_bounds__(kThreads) chan_eltwise_rows_kernel(const float4* __restrict__ x,
                                                                    const float4* __restrict__ residual,
                                                                    float4* __restrict__ y, long rows, int c4,
                                                                    ChanEpilogue epi)
{
    const int q = threadIdx.x % c4, r0 = threadIdx.x / c4, rows_per_pass = kThreads / c4;
    float bias[4] = {0, 0, 0, 0}, mean[4] = {0, 0, 0, 0}, inv_std[4] = {0, 0, 0, 0}, gamma[4] = {0, 0, 0, 0},
          beta[4] = {0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (epi.bias) bias[t] = epi.bias[4 * q + t];
        if (epi.mean) {
            mean[t] = epi.mean[4 * q + t];
            inv_std[t] = epi.inv_std[4 * q + t];
            gamma[t] = epi.gamma[4 * q + t];
            beta[t] = epi.beta[4 * q + t];
        }
    }
    for (long row = (long)blockIdx.x * rows_per_pass + r0; row < rows; row += (long)gridDim.x * rows_per_pass) {
        const size_t at = (size_t)row * c4 + q;
        float4 v4 = x[at];
        float v[4] = {v4.x, v4.y, v4.z, v4.w};
        if (residual) {
            const float4 r = residual[at];
            v[0] += r.x; v[1] += r.y; v[2] += r.z; v[3] += r.w;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (epi.bias) v[t] += bias[t];
            if (epi.mean) {
                const float u = (v[t] - mean[t]) * inv_std[t];
                v[t] = u * gamma[t] + beta[t];
            }
            if (epi.relu) v[t] = v[t] > 0.0f ? v[t] : 0.0f;
        }
        y[at] = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// ---------------------------------------------------------------- ReLU with mask
// pydtnn/cython_modules/relu_cython.pyx:52-59 (strict x > 0); pydtnn/backends/cpu/activations/relu_cpu.py:38-40.
// Four elements per thread (one 16-byte load, one 16-byte store, one 4-byte mask store) when the
// pointers allow it; the last thread finishes a tail of up to three elements.
template <bool VEC4>
__global__ void __launch_bounds__(kThreads) relu_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                           int8_t* __restrict__ mask, long total)
{
    const long idx = ((long)blockIdx.x * kThreads + threadIdx.x) * (VEC4 ? 4 : 1);
    if (idx >= total) return;
    if (VEC4 && idx + 4 <= total) {
        const float4 v = *reinterpret_cast<const float4*>(x + idx);
        const bool p0 = v.x > 0.0f, p1 = v.y > 0.0f, p2 = v.z > 0.0f, p3 = v.w > 0.0f;
        *reinterpret_cast<float4*>(y + idx) =
            make_float4(p0 ? v.x : 0.0f, p1 ? v.y : 0.0f, p2 ? v.z : 0.0f, p3 ? v.w : 0.0f);
        if (mask)
            *reinterpret_cast<uint32_t*>(mask + idx) =
                (uint32_t)p0 | ((uint32_t)p1 << 8) | ((uint32_t)p2 << 16) | ((uint32_t)p3 << 24);
        return;
    }
    const long end = VEC4 ? total : idx + 1;
    for (long i = idx; i < end; ++i) {
        const float v = x[i];
        const bool pos = v > 0.0f;
        y[i] = pos ? v : 0.0f;
        if (mask) mask[i] = pos ? 1 : 0;
    }
}

template <bool VEC4>
__global__ void __launch_bounds__(kThreads) relu_bwd_kernel(const float* __restrict__ dy,
                                                           const int8_t* __restrict__ mask,
                                                           float* __restrict__ dx, long total)
{
    const long idx = ((long)blockIdx.x * kThreads + threadIdx.x) * (VEC4 ? 4 : 1);
    if (idx >= total) return;
    if (VEC4 && idx + 4 <= total) {
        const float4 v = *reinterpret_cast<const float4*>(dy + idx);
        const uint32_t m = *reinterpret_cast<const uint32_t*>(mask + idx);
        *reinterpret_cast<float4*>(dx + idx) =
            make_float4(v.x * (float)(int8_t)(m & 0xff), v.y * (float)(int8_t)((m >> 8) & 0xff),
                        v.z * (float)(int8_t)((m >> 16) & 0xff), v.w * (float)(int8_t)(m >> 24));
        return;
    }
    const long end = VEC4 ? total : idx + 1;
    for (long i = idx; i < end; ++i) dx[i] = dy[i] * (float)mask[i];
}

// ---------------------------------------------------------------- bias gradient
// db[c] = sum over batch and pixels of dy (pydtnn/backends/cpu/layers/conv_2d_cpu.py:463 NCHW, :377 NHWC;
// fc_cpu.py:70).  Two deterministic stages: per-(channel, slice) partial sums, then a sum over slices.
__device__ __forceinline__ float block_sum(float v)
{
    __shared__ float red[kThreads / 64];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = 0.0f;
    if (threadIdx.x == 0)
        for (int i = 0; i < kThreads / 64; ++i) s += red[i];
    return s;  // valid on thread 0
}

// NCHW: grid (C, S); slice s covers images [s*per, (s+1)*per).  VEC4: planes are read 16 bytes per lane
// (hw % 4 == 0 and a 16-byte aligned tensor).
template <bool VEC4>
__global__ void __launch_bounds__(kThreads) bias_grad_nchw_stage1(const float* __restrict__ dy,
                                                                 float* __restrict__ partial, int n, int c,
                                                                 int hw, int per)
{
    const int ch = blockIdx.x, s = blockIdx.y;
    const int n0 = s * per, n1 = min(n, n0 + per);
    float acc = 0.0f;
    if (!VEC4 && hw < kThreads) {
        // planes smaller than the workgroup: its threads walk the (image, pixel) pairs of the slice together
        const uint32_t count = (uint32_t)(n1 - n0) * (uint32_t)hw;
        for (uint32_t e = threadIdx.x; e < count; e += kThreads) {
            const uint32_t nn = e / (uint32_t)hw, i = e - nn * (uint32_t)hw;
            acc += dy[((long)(n0 + (int)nn) * c + ch) * hw + i];
        }
    } else {
        for (int nn = n0; nn < n1; ++nn) {
            const float* plane = dy + ((long)nn * c + ch) * hw;
            if (VEC4) {
                const float4* p4 = reinterpret_cast<const float4*>(plane);
                float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
                for (int i = threadIdx.x; i < hw / 4; i += kThreads) {
                    const float4 v = p4[i];
                    a0 += v.x; a1 += v.y; a2 += v.z; a3 += v.w;
                }
                acc += (a0 + a1) + (a2 + a3);
            } else {
                for (int i = threadIdx.x; i < hw; i += kThreads) acc += plane[i];
            }
        }
    }
    const float tot = block_sum(acc);
    if (threadIdx.x == 0) partial[(long)s * c + ch] = tot;
}

// (rows, C) matrix: grid (S, ceil(C/64)); block = 64 channels x 4 row lanes.
__global__ void __launch_bounds__(kThreads) bias_grad_rows_stage1(const float* __restrict__ dy,
                                                                 float* __restrict__ partial, long rows, int c,
                                                                 long per)
{
    __shared__ float red[4][64];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const int ch = blockIdx.y * 64 + cl;
    const long r0 = (long)blockIdx.x * per;
    const long r1 = r0 + per < rows ? r0 + per : rows;
    float acc = 0.0f;
    if (ch < c)
        for (long r = r0 + rl; r < r1; r += 4) acc += dy[r * c + ch];
    red[rl][cl] = acc;
    __syncthreads();
    if (rl == 0 && ch < c) partial[(long)blockIdx.x * c + ch] = (red[0][cl] + red[1][cl]) + (red[2][cl] + red[3][cl]);
}

// (rows, C) matrix whose row is `lanes` = C/4 quads with lanes a power of two <= kThreads, 16-byte aligned:
// one workgroup reads kThreads/lanes whole rows per load, eight loads in flight per lane, and covers the row
// slice [blockIdx.x*per, +per).  HBM-bound: 4*rows*C bytes read once.
__global__ void __launch_bounds__(kThreads) bias_grad_rows_quads_stage1(const float4* __restrict__ dy,
                                                                       float* __restrict__ partial, long rows,
                                                                       int lanes, long per)
{
    constexpr int kInFlight = 8;
    __shared__ float4 red[kThreads];
    const int cl = threadIdx.x & (lanes - 1);
    const int row_lanes = kThreads / lanes, rl = threadIdx.x / lanes;
    const long r0 = (long)blockIdx.x * per;
    const long r1 = r0 + per < rows ? r0 + per : rows;
    float4 acc[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc[u] = float4{0.0f, 0.0f, 0.0f, 0.0f};
    const float4* p = dy + cl;
    for (long r = r0 + rl; r < r1; r += (long)row_lanes * kInFlight) {
        float4 v[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            const long rr = r + (long)u * row_lanes;
            v[u] = rr < r1 ? p[rr * lanes] : float4{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            acc[u].x += v[u].x; acc[u].y += v[u].y; acc[u].z += v[u].z; acc[u].w += v[u].w;
        }
    }
    float4 t = acc[0];
#pragma unroll
    for (int u = 1; u < kInFlight; ++u) { t.x += acc[u].x; t.y += acc[u].y; t.z += acc[u].z; t.w += acc[u].w; }
    red[threadIdx.x] = t;
    __syncthreads();
    if (rl == 0) {
        for (int i = 1; i < row_lanes; ++i) {
            const float4 o = red[i * lanes + cl];
            t.x += o.x; t.y += o.y; t.z += o.z; t.w += o.w;
        }
        reinterpret_cast<float4*>(partial + (long)blockIdx.x * lanes * 4)[cl] = t;
    }
}

// db[ch] = sum over slices of partial[s*c + ch]: 16 channels x 16 slice lanes per workgroup, each lane adding
// its slices in order, the lanes' sums added in lane order.
__global__ void __launch_bounds__(kThreads) bias_grad_stage2(const float* __restrict__ partial,
                                                            float* __restrict__ db, int c, int slices)
{
    __shared__ float red[16][17];
    const int cl = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int ch = blockIdx.x * 16 + cl;
    float acc = 0.0f;
    if (ch < c)
        for (int s = sl; s < slices; s += 16) acc += partial[(long)s * c + ch];
    red[sl][cl] = acc;
    __syncthreads();
    if (sl == 0 && ch < c) {
        float t = red[0][cl];
        for (int i = 1; i < 16; ++i) t += red[i][cl];
        db[ch] = t;
    }
}

// ---------------------------------------------------------------- split-K reduction
// out[map(r, col)] = epilogue(col, sum_s partial[s*stride + r*ncols + col]), or with `accumulate` that value
// added to what out already holds (a filter gradient built up over several launches).
// perm_c > 0 re-orders rows from the kernels' internal (i, j, c) order to the reference's
// (c, i, j) weight rows: r = ij*perm_c + c  ->  c*khw + ij.
__global__ void __launch_bounds__(kThreads) splitk_reduce_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ out, long total, long stride,
                                                                int slices, int ncols, int perm_c, int khw,
                                                                ChanEpilogue epi, int accumulate)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    // eight loads in flight, then added in slice order (the sum is the same as one load at a time)
    float acc = 0.0f;
    int s = 0;
    for (; s + 8 <= slices; s += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = partial[(long)(s + u) * stride + idx];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; s < slices; ++s) acc += partial[(long)s * stride + idx];
    const int col = (int)(idx % ncols);
    long r = idx / ncols;
    if (perm_c > 0) {
        const long ij = r / perm_c;
        const long cc = r - ij * perm_c;
        r = cc * khw + ij;
    }
    const float v = chan_epilogue_apply(epi, col, acc);
    out[r * ncols + col] = accumulate ? out[r * ncols + col] + v : v;
}

// ---------------------------------------------------------------- filter re-layouts for dX
// Stride-1 dX is a forward convolution of dy with the spatially flipped, channel-swapped filter.
// NCHW: wf[c][co][i][j] = w[co][c][kh-1-i][kw-1-j]
__global__ void __launch_bounds__(kThreads) flip_filter_nchw_kernel(const float* __restrict__ w,
                                                                   float* __restrict__ wf, int kn, int c, int kh,
                                                                   int kw)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    const long total = (long)kn * c * kh * kw;
    if (idx >= total) return;
    const int j = (int)(idx % kw);
    long t = idx / kw;
    const int i = (int)(t % kh);
    t /= kh;
    const int co = (int)(t % kn);
    const int cc = (int)(t / kn);
    wf[idx] = w[(((long)co * c + cc) * kh + (kh - 1 - i)) * kw + (kw - 1 - j)];
}

// NHWC: wf[co][i][j][c] = w[c][kh-1-i][kw-1-j][co]
__global__ void __launch_bounds__(kThreads) flip_filter_nhwc_kernel(const float* __restrict__ w,
                                                                   float* __restrict__ wf, int kn, int c, int kh,
                                                                   int kw)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    const long total = (long)kn * c * kh * kw;
    if (idx >= total) return;
    const int cc = (int)(idx % c);
    long t = idx / c;
    const int j = (int)(t % kw);
    t /= kw;
    const int i = (int)(t % kh);
    const int co = (int)(t / kh);
    wf[idx] = w[(((long)cc * kh + (kh - 1 - i)) * kw + (kw - 1 - j)) * kn + co];
}

// ---------------------------------------------------------------- MaxPool2D NCHW
// Forward: pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:86-110 (first maximum wins, index ii*kw+jj).
// grid.x * 256 threads walk one (n, c) plane of the output, grid.y walks the planes.
__global__ void __launch_bounds__(kThreads) max_pool_fwd_nchw_kernel(const float* __restrict__ x,
                                                                    float* __restrict__ y,
                                                                    int32_t* __restrict__ idx_max, ConvGeom g)
{
    const uint32_t pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= (uint32_t)g.howo) return;
    const int oy = (int)fd_div(pix, g.fd_wo);
    const int ox = (int)pix - oy * g.wo;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    const int y0 = g.vstride * oy - g.vpadding, x0 = g.hstride * ox - g.hpadding;
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const float* src = x + (long)plane * g.h * g.w;
        float maxval = -3.402823466e+38f;
        int best = 0;
        for (int ii = 0; ii < g.kh; ++ii) {
            const int x_x = y0 + g.vdilation * ii;
            if ((unsigned)x_x >= (unsigned)g.h) continue;
            for (int jj = 0; jj < g.kw; ++jj) {
                const int x_y = x0 + g.hdilation * jj;
                if ((unsigned)x_y >= (unsigned)g.w) continue;
                const float val = src[x_x * g.w + x_y];
                if (val > maxval) { maxval = val; best = ii * g.kw + jj; }
            }
        }
        y[(long)plane * g.howo + pix] = maxval;
        idx_max[(long)plane * g.howo + pix] = best;
    }
}

// Forward for K x K windows without dilation (any stride and padding): the K*K taps of a window are loaded
// without conditions (taps outside the plane from a clamped address, masked out afterwards), their offsets and
// masks worked out once per thread; the taps are then compared in the reference's order (first maximum wins).
template <int K>
__global__ void __launch_bounds__(kThreads) max_pool_fwd_square_nchw_kernel(const float* __restrict__ x,
                                                                           float* __restrict__ y,
                                                                           int32_t* __restrict__ idx_max, ConvGeom g)
{
    const uint32_t pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= (uint32_t)g.howo) return;
    const int oy = (int)fd_div(pix, g.fd_wo);
    const int ox = (int)pix - oy * g.wo;
    const int y0 = g.vstride * oy - g.vpadding, x0 = g.hstride * ox - g.hpadding;
    int off[K * K];
    bool live[K * K];
#pragma unroll
    for (int ii = 0; ii < K; ++ii)
#pragma unroll
        for (int jj = 0; jj < K; ++jj) {
            const bool ok = (unsigned)(y0 + ii) < (unsigned)g.h && (unsigned)(x0 + jj) < (unsigned)g.w;
            live[ii * K + jj] = ok;
            off[ii * K + jj] = ok ? (y0 + ii) * g.w + x0 + jj : 0;
        }
    const uint32_t planes = (uint32_t)(g.n * g.c);
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const float* src = x + (long)plane * g.h * g.w;
        float v[K * K];
#pragma unroll
        for (int t = 0; t < K * K; ++t) v[t] = src[off[t]];
        float maxval = -3.402823466e+38f;
        int best = 0;
#pragma unroll
        for (int t = 0; t < K * K; ++t)
            if (live[t] && v[t] > maxval) { maxval = v[t]; best = t; }
        y[(long)plane * g.howo + pix] = maxval;
        idx_max[(long)plane * g.howo + pix] = best;
    }
}

// The NHWC twin: lanes along the channels.
template <int K>
__global__ void __launch_bounds__(kThreads) max_pool_fwd_square_nhwc_kernel(const float* __restrict__ x,
                                                                           float* __restrict__ y,
                                                                           int32_t* __restrict__ idx_max, ConvGeom g,
                                                                           int c_exact)
{
    const uint32_t per_image = (uint32_t)(g.howo * g.c);
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t pix = fd_div_checked(e, g.fd_c, c_exact);
    const uint32_t cc = e - pix * g.c;
    const int oy = (int)fd_div(pix, g.fd_wo);
    const int ox = (int)pix - oy * g.wo;
    const int y0 = g.vstride * oy - g.vpadding, x0 = g.hstride * ox - g.hpadding;
    size_t off[K * K];
    bool live[K * K];
#pragma unroll
    for (int ii = 0; ii < K; ++ii)
#pragma unroll
        for (int jj = 0; jj < K; ++jj) {
            const bool ok = (unsigned)(y0 + ii) < (unsigned)g.h && (unsigned)(x0 + jj) < (unsigned)g.w;
            live[ii * K + jj] = ok;
            off[ii * K + jj] = (ok ? (size_t)((y0 + ii) * g.w + x0 + jj) * g.c : 0) + cc;
        }
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const float* src = x + (size_t)nn * g.h * g.w * g.c;
        float v[K * K];
#pragma unroll
        for (int t = 0; t < K * K; ++t) v[t] = src[off[t]];
        float maxval = -3.402823466e+38f;
        int best = 0;
#pragma unroll
        for (int t = 0; t < K * K; ++t)
            if (live[t] && v[t] > maxval) { maxval = v[t]; best = t; }
        y[(size_t)nn * per_image + e] = maxval;
        idx_max[(size_t)nn * per_image + e] = best;
    }
}

// Forward for 2x2 windows that tile the plane exactly (stride 2, no padding or dilation, h == 2*ho, w == 2*wo,
// 8-byte aligned x): a thread reads its window as two 64-bit loads and tests the four values in the reference's
// order (first maximum wins).
__global__ void __launch_bounds__(kThreads) max_pool_fwd_windows2_nchw_kernel(const float* __restrict__ x,
                                                                             float* __restrict__ y,
                                                                             int32_t* __restrict__ idx_max,
                                                                             ConvGeom g)
{
    const uint32_t win = blockIdx.x * kThreads + threadIdx.x;
    if (win >= (uint32_t)g.howo) return;
    const int oy = (int)fd_div(win, g.fd_wo);
    const int ox = (int)win - oy * g.wo;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    const size_t first = (size_t)(2 * oy) * g.w + 2 * ox;
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const float* src = x + (size_t)plane * g.h * g.w + first;
        const float2 r0 = *reinterpret_cast<const float2*>(src);
        const float2 r1 = *reinterpret_cast<const float2*>(src + g.w);
        float maxval = -3.402823466e+38f;
        int best = 0;
        if (r0.x > maxval) { maxval = r0.x; best = 0; }
        if (r0.y > maxval) { maxval = r0.y; best = 1; }
        if (r1.x > maxval) { maxval = r1.x; best = 2; }
        if (r1.y > maxval) { maxval = r1.y; best = 3; }
        y[(size_t)plane * g.howo + win] = maxval;
        idx_max[(size_t)plane * g.howo + win] = best;
    }
}

// Backward when square windows tile the plane exactly (kh == kw == both strides, no padding or
// dilation, h == ho*kh, w == wo*kw): one thread owns one window, reads its index and gradient once
// and writes the window's kh x kw elements of dx (the decoded element gets 0 + dy, the others 0).
// The decode is the reference's own (ii = idx / kh, jj = idx % kw, max_pool_2d_nchw_cython.pyx:204-205).
template <int KW>
__global__ void __launch_bounds__(kThreads) max_pool_bwd_windows_nchw_kernel(const float* __restrict__ dy,
                                                                            const int32_t* __restrict__ idx_max,
                                                                            float* __restrict__ dx, ConvGeom g,
                                                                            const int8_t* __restrict__ gate)
{
    const uint32_t win = blockIdx.x * kThreads + threadIdx.x;
    if (win >= (uint32_t)g.howo) return;
    const int oy = (int)fd_div(win, g.fd_wo);
    const int ox = (int)win - oy * g.wo;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    const int kw = KW > 0 ? KW : g.kw;
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const uint32_t rec = (uint32_t)idx_max[(size_t)plane * g.howo + win];
        const float grad = 0.0f + dy[(size_t)plane * g.howo + win];
        const int ri = (int)fd_div(rec, g.fd_kh);
        const int rj = (int)(rec - fd_div(rec, g.fd_kw) * g.kw);
        const size_t first = (size_t)plane * g.h * g.w + (size_t)(oy * g.kh) * g.w + ox * kw;
        float* dst = dx + first;
        const int8_t* gt = gate ? gate + first : nullptr;
        for (int ii = 0; ii < g.kh; ++ii) {
            if (KW == 2) {
                float2 v = make_float2(ii == ri && rj == 0 ? grad : 0.0f, ii == ri && rj == 1 ? grad : 0.0f);
                if (gt) { v.x *= (float)gt[0]; v.y *= (float)gt[1]; }
                *reinterpret_cast<float2*>(dst) = v;
            } else {
                for (int jj = 0; jj < kw; ++jj) {
                    const float v = ii == ri && jj == rj ? grad : 0.0f;
                    dst[jj] = gt ? v * (float)gt[jj] : v;
                }
            }
            dst += g.w;
            if (gt) gt += g.w;
        }
    }
}

// The same for 2 x 2 windows with an even number of windows per row: one thread owns two neighbouring windows
// and writes their four columns of both rows as one 128-bit store each (indices and gradients arrive as 64-bit
// loads, gate bytes as one 32-bit load per row).
__global__ void __launch_bounds__(kThreads) max_pool_bwd_window_pairs_nchw_kernel(const float2* __restrict__ dy,
                                                                                 const int2* __restrict__ idx_max,
                                                                                 float4* __restrict__ dx, ConvGeom g,
                                                                                 const uint32_t* __restrict__ gate)
{
    const uint32_t pairs = (uint32_t)g.howo >> 1, half_wo = (uint32_t)g.wo >> 1;
    const uint32_t pr = blockIdx.x * kThreads + threadIdx.x;
    if (pr >= pairs) return;
    const uint32_t oy = pr / half_wo, px = pr - oy * half_wo;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    const size_t plane_quads = (size_t)g.h * g.w / 4, row_quads = (size_t)g.w / 4;
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const int2 rec = idx_max[(size_t)plane * pairs + pr];
        const float2 gr = dy[(size_t)plane * pairs + pr];
        const float g0 = 0.0f + gr.x, g1 = 0.0f + gr.y;
        const size_t first = (size_t)plane * plane_quads + (size_t)(2 * oy) * row_quads + px;
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
            // the reference's decode for 2 x 2 windows: row = idx / 2, column = idx % 2
            float4 v = make_float4(rec.x == 2 * ii ? g0 : 0.0f, rec.x == 2 * ii + 1 ? g0 : 0.0f,
                                   rec.y == 2 * ii ? g1 : 0.0f, rec.y == 2 * ii + 1 ? g1 : 0.0f);
            if (gate) {
                const uint32_t gt = gate[first + ii * row_quads];
                v.x *= (float)(int8_t)(gt & 0xff); v.y *= (float)(int8_t)((gt >> 8) & 0xff);
                v.z *= (float)(int8_t)((gt >> 16) & 0xff); v.w *= (float)(int8_t)(gt >> 24);
            }
            dx[first + ii * row_quads] = v;
        }
    }
}

// Output rows (or columns) whose window covers input coordinate `t = coord + padding`, for windows of `k` taps at
// stride `stride` without dilation: [lo, hi], empty when lo > hi.
__device__ __forceinline__ void pool_window_range(int t, int k, int stride, const FastDiv fd_stride, int extent,
                                                  int* lo, int* hi)
{
    const int first = t - (k - 1);
    *hi = min((int)fd_div((uint32_t)t, fd_stride), extent - 1);
    *lo = first <= 0 ? 0 : (int)fd_div((uint32_t)(first + stride - 1), fd_stride);
}

// Backward for square windows without dilation that overlap or leave gaps (any stride and padding): the windows
// that cover an element form a small rectangle of outputs (at most ceil(k/stride) per axis), worked out directly
// instead of testing all k*k taps; visited in ascending (oy, ox) like the reference's scatter loop.  With
// kh == kw the reference's decode (idx / kh, idx % kw) is the plain one, so a window's maximum lies on this
// element exactly when its index equals ii*kw + jj.
// PER_AXIS = 2: at most two windows per axis cover an element (k <= 2*stride): the four candidates are loaded
// without conditions (out-of-range ones from a clamped address, masked out afterwards) so that no load waits for
// a comparison; adding 0.0f for a window whose maximum lies elsewhere leaves the sum's bits unchanged.
template <int PER_AXIS>
__global__ void __launch_bounds__(kThreads) max_pool_bwd_ranges_nchw_kernel(const float* __restrict__ dy,
                                                                           const int32_t* __restrict__ idx_max,
                                                                           float* __restrict__ dx, ConvGeom g,
                                                                           const int8_t* __restrict__ gate)
{
    const uint32_t hw = (uint32_t)(g.h * g.w);
    const uint32_t pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= hw) return;
    const int hh = (int)fd_div(pix, g.fd_w);
    const int ww = (int)pix - hh * g.w;
    const int ty = hh + g.vpadding, tx = ww + g.hpadding;
    int oy0, oy1, ox0, ox1;
    pool_window_range(ty, g.kh, g.vstride, g.fd_vs, g.ho, &oy0, &oy1);
    pool_window_range(tx, g.kw, g.hstride, g.fd_hs, g.wo, &ox0, &ox1);
    const uint32_t planes = (uint32_t)(g.n * g.c);
    if (PER_AXIS == 2) {
        int at[4], code[4];
        bool live[4];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int oy = oy0 + a, ox = ox0 + b;
                live[a * 2 + b] = oy <= oy1 && ox <= ox1;
                at[a * 2 + b] = live[a * 2 + b] ? oy * g.wo + ox : 0;
                code[a * 2 + b] = (ty - oy * g.vstride) * g.kw + (tx - ox * g.hstride);
            }
        for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
            const float* gy = dy + (long)plane * g.howo;
            const int32_t* gi = idx_max + (long)plane * g.howo;
            int rec[4];
            float grad[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) { rec[q] = gi[at[q]]; grad[q] = gy[at[q]]; }
            float acc = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) acc += live[q] && rec[q] == code[q] ? grad[q] : 0.0f;
            if (gate) acc *= (float)gate[(long)plane * hw + pix];
            dx[(long)plane * hw + pix] = acc;
        }
        return;
    }
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const float* gy = dy + (long)plane * g.howo;
        const int32_t* gi = idx_max + (long)plane * g.howo;
        float acc = 0.0f;
        for (int oy = oy0; oy <= oy1; ++oy) {
            const int ii = ty - oy * g.vstride;
            for (int ox = ox0; ox <= ox1; ++ox) {
                const int jj = tx - ox * g.hstride;
                const float grad = gy[oy * g.wo + ox];
                acc += gi[oy * g.wo + ox] == ii * g.kw + jj ? grad : 0.0f;
            }
        }
        if (gate) acc *= (float)gate[(long)plane * hw + pix];
        dx[(long)plane * hw + pix] = acc;
    }
}

// Backward in gather form: one thread per dx element sums dy of every window whose recorded
// maximum decodes to this element.  The decode is the reference's own
// (ii = idx / kh, jj = idx % kw, max_pool_2d_nchw_cython.pyx:204-205).  Windows are visited in
// ascending (oy, ox), the order of the reference's scatter loop.
// TILED: square windows that do not overlap and have no padding or dilation (kh == kw == both strides),
// so each element lies in at most one window and the tap loops collapse to one lookup.
template <bool TILED>
__global__ void __launch_bounds__(kThreads) max_pool_bwd_nchw_kernel(const float* __restrict__ dy,
                                                                    const int32_t* __restrict__ idx_max,
                                                                    float* __restrict__ dx, ConvGeom g,
                                                                    const int8_t* __restrict__ gate)
{
    const uint32_t hw = (uint32_t)(g.h * g.w);
    const uint32_t pix = blockIdx.x * kThreads + threadIdx.x;
    if (pix >= hw) return;
    const int hh = (int)fd_div(pix, g.fd_w);
    const int ww = (int)pix - hh * g.w;
    const uint32_t planes = (uint32_t)(g.n * g.c);
    if (TILED) {
        const int oy = (int)fd_div((uint32_t)hh, g.fd_vs), ox = (int)fd_div((uint32_t)ww, g.fd_hs);
        const int ii = hh - oy * g.vstride, jj = ww - ox * g.hstride;
        const bool inside = oy < g.ho && ox < g.wo;
        const int win = oy * g.wo + ox;
        for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
            float acc = 0.0f;
            if (inside) {
                const uint32_t rec = (uint32_t)idx_max[(long)plane * g.howo + win];
                const uint32_t ri = fd_div(rec, g.fd_kh);
                const uint32_t rj = rec - fd_div(rec, g.fd_kw) * g.kw;
                if ((int)ri == ii && (int)rj == jj) acc = 0.0f + dy[(long)plane * g.howo + win];
            }
            if (gate) acc *= (float)gate[(long)plane * hw + pix];
            dx[(long)plane * hw + pix] = acc;
        }
        return;
    }
    for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
        const float* gy = dy + (long)plane * g.howo;
        const int32_t* gi = idx_max + (long)plane * g.howo;
        float acc = 0.0f;
        // decoded rows run up to (kh*kw - 1) / kh, which exceeds kh - 1 when kw > kh
        for (int ii = (g.khw - 1) / g.kh; ii >= 0; --ii) {
            const int ty = hh + g.vpadding - g.vdilation * ii;
            if (ty < 0) continue;
            const int oy = (int)fd_div((uint32_t)ty, g.fd_vs);
            if (oy * g.vstride != ty || oy >= g.ho) continue;
            for (int jj = g.kw - 1; jj >= 0; --jj) {
                const int tx = ww + g.hpadding - g.hdilation * jj;
                if (tx < 0) continue;
                const int ox = (int)fd_div((uint32_t)tx, g.fd_hs);
                if (ox * g.hstride != tx || ox >= g.wo) continue;
                const uint32_t rec = (uint32_t)gi[oy * g.wo + ox];
                const uint32_t ri = fd_div(rec, g.fd_kh);
                const uint32_t rj = rec - fd_div(rec, g.fd_kw) * g.kw;
                if ((int)ri == ii && (int)rj == jj) acc += gy[oy * g.wo + ox];
            }
        }
        if (gate) acc *= (float)gate[(long)plane * hw + pix];
        dx[(long)plane * hw + pix] = acc;
    }
}

// ---------------------------------------------------------------- MaxPool2D NHWC
// pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:86-110 and :194-212: the rules of the NCHW pair.
// grid.x * 256 threads walk the (pixel, channel) elements of one image, lanes along c; grid.y walks the images.
__global__ void __launch_bounds__(kThreads) max_pool_fwd_nhwc_kernel(const float* __restrict__ x,
                                                                    float* __restrict__ y,
                                                                    int32_t* __restrict__ idx_max, ConvGeom g,
                                                                    int c_exact)
{
    const uint32_t per_image = (uint32_t)(g.howo * g.c);
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t pix = fd_div_checked(e, g.fd_c, c_exact);
    const uint32_t cc = e - pix * g.c;
    const int oy = (int)fd_div(pix, g.fd_wo);
    const int ox = (int)pix - oy * g.wo;
    const int y0 = g.vstride * oy - g.vpadding, x0 = g.hstride * ox - g.hpadding;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const float* src = x + (size_t)nn * g.h * g.w * g.c + cc;
        float maxval = -3.402823466e+38f;
        int best = 0;
        for (int ii = 0; ii < g.kh; ++ii) {
            const int x_x = y0 + g.vdilation * ii;
            if ((unsigned)x_x >= (unsigned)g.h) continue;
            for (int jj = 0; jj < g.kw; ++jj) {
                const int x_y = x0 + g.hdilation * jj;
                if ((unsigned)x_y >= (unsigned)g.w) continue;
                const float val = src[(size_t)(x_x * g.w + x_y) * g.c];
                if (val > maxval) { maxval = val; best = ii * g.kw + jj; }
            }
        }
        y[(size_t)nn * per_image + e] = maxval;
        idx_max[(size_t)nn * per_image + e] = best;
    }
}

// NHWC forward for 2x2 windows that tile the image exactly, c % 4 == 0 and 16-byte aligned tensors: a thread owns
// four channels of a window and reads each of its four pixels with one 128-bit load.
__global__ void __launch_bounds__(kThreads) max_pool_fwd_windows2_nhwc_kernel(const float4* __restrict__ x,
                                                                             float4* __restrict__ y,
                                                                             int4* __restrict__ idx_max, ConvGeom g)
{
    const uint32_t cq = (uint32_t)g.c / 4;
    const uint32_t per_image = (uint32_t)g.howo * cq;
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t win = e / cq, q = e - win * cq;
    const int oy = (int)fd_div(win, g.fd_wo);
    const int ox = (int)win - oy * g.wo;
    const size_t first = ((size_t)(2 * oy) * g.w + (size_t)(2 * ox)) * cq + q;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const float4* src = x + (size_t)nn * g.h * g.w * cq + first;
        const float4 v[4] = {src[0], src[cq], src[(size_t)g.w * cq], src[(size_t)g.w * cq + cq]};
        float m[4] = {-3.402823466e+38f, -3.402823466e+38f, -3.402823466e+38f, -3.402823466e+38f};
        int b[4] = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float c4[4] = {v[t].x, v[t].y, v[t].z, v[t].w};
#pragma unroll
            for (int l = 0; l < 4; ++l)
                if (c4[l] > m[l]) { m[l] = c4[l]; b[l] = t; }
        }
        y[(size_t)nn * per_image + e] = float4{m[0], m[1], m[2], m[3]};
        idx_max[(size_t)nn * per_image + e] = int4{b[0], b[1], b[2], b[3]};
    }
}

// Gather form of the backward scatter: windows visited in ascending (oy, ox), i.e. descending taps.
__global__ void __launch_bounds__(kThreads) max_pool_bwd_nhwc_kernel(const float* __restrict__ dy,
                                                                    const int32_t* __restrict__ idx_max,
                                                                    float* __restrict__ dx, ConvGeom g, int c_exact,
                                                                    const int8_t* __restrict__ gate)
{
    const uint32_t per_image = (uint32_t)(g.h * g.w * g.c);
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t pix = fd_div_checked(e, g.fd_c, c_exact);
    const uint32_t cc = e - pix * g.c;
    const int hh = (int)fd_div(pix, g.fd_w);
    const int ww = (int)pix - hh * g.w;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const size_t base = (size_t)nn * g.howo * g.c + cc;
        float acc = 0.0f;
        // decoded rows run up to (kh*kw - 1) / kh, which exceeds kh - 1 when kw > kh
        for (int ii = (g.khw - 1) / g.kh; ii >= 0; --ii) {
            const int ty = hh + g.vpadding - g.vdilation * ii;
            if (ty < 0) continue;
            const int oy = (int)fd_div((uint32_t)ty, g.fd_vs);
            if (oy * g.vstride != ty || oy >= g.ho) continue;
            for (int jj = g.kw - 1; jj >= 0; --jj) {
                const int tx = ww + g.hpadding - g.hdilation * jj;
                if (tx < 0) continue;
                const int ox = (int)fd_div((uint32_t)tx, g.fd_hs);
                if (ox * g.hstride != tx || ox >= g.wo) continue;
                const size_t at = base + (size_t)(oy * g.wo + ox) * g.c;
                const uint32_t rec = (uint32_t)idx_max[at];
                const uint32_t ri = fd_div(rec, g.fd_kh);
                const uint32_t rj = rec - fd_div(rec, g.fd_kw) * g.kw;
                if ((int)ri == ii && (int)rj == jj) acc += dy[at];
            }
        }
        if (gate) acc *= (float)gate[(size_t)nn * per_image + e];
        dx[(size_t)nn * per_image + e] = acc;
    }
}

// The NHWC twin of max_pool_bwd_ranges_nchw_kernel: lanes along the channels.
template <int PER_AXIS>
__global__ void __launch_bounds__(kThreads) max_pool_bwd_ranges_nhwc_kernel(const float* __restrict__ dy,
                                                                           const int32_t* __restrict__ idx_max,
                                                                           float* __restrict__ dx, ConvGeom g,
                                                                           int c_exact,
                                                                           const int8_t* __restrict__ gate)
{
    const uint32_t per_image = (uint32_t)(g.h * g.w * g.c);
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t pix = fd_div_checked(e, g.fd_c, c_exact);
    const uint32_t cc = e - pix * g.c;
    const int hh = (int)fd_div(pix, g.fd_w);
    const int ww = (int)pix - hh * g.w;
    const int ty = hh + g.vpadding, tx = ww + g.hpadding;
    int oy0, oy1, ox0, ox1;
    pool_window_range(ty, g.kh, g.vstride, g.fd_vs, g.ho, &oy0, &oy1);
    pool_window_range(tx, g.kw, g.hstride, g.fd_hs, g.wo, &ox0, &ox1);
    if (PER_AXIS == 2) {
        size_t at[4];
        int code[4];
        bool live[4];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int oy = oy0 + a, ox = ox0 + b;
                live[a * 2 + b] = oy <= oy1 && ox <= ox1;
                at[a * 2 + b] = (live[a * 2 + b] ? (size_t)(oy * g.wo + ox) * g.c : 0) + cc;
                code[a * 2 + b] = (ty - oy * g.vstride) * g.kw + (tx - ox * g.hstride);
            }
        for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
            const size_t base = (size_t)nn * g.howo * g.c;
            int rec[4];
            float grad[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) { rec[q] = idx_max[base + at[q]]; grad[q] = dy[base + at[q]]; }
            float acc = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) acc += live[q] && rec[q] == code[q] ? grad[q] : 0.0f;
            if (gate) acc *= (float)gate[(size_t)nn * per_image + e];
            dx[(size_t)nn * per_image + e] = acc;
        }
        return;
    }
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const size_t base = (size_t)nn * g.howo * g.c + cc;
        float acc = 0.0f;
        for (int oy = oy0; oy <= oy1; ++oy) {
            const int ii = ty - oy * g.vstride;
            for (int ox = ox0; ox <= ox1; ++ox) {
                const int jj = tx - ox * g.hstride;
                const size_t at = base + (size_t)(oy * g.wo + ox) * g.c;
                const float grad = dy[at];
                acc += idx_max[at] == ii * g.kw + jj ? grad : 0.0f;
            }
        }
        if (gate) acc *= (float)gate[(size_t)nn * per_image + e];
        dx[(size_t)nn * per_image + e] = acc;
    }
}

// NHWC backward when square windows tile the image exactly (same conditions as the NCHW windows kernel) and
// c % 4 == 0 with 16-byte aligned tensors: one thread owns four channels of one window, reads their indices
// and gradients once and writes the window's kh x kw quads of dx.  Decode as in
// max_pool_2d_nhwc_cython.pyx (ii = idx / kh, jj = idx % kw).
template <int K>
__global__ void __launch_bounds__(kThreads) max_pool_bwd_windows_nhwc_kernel(const float4* __restrict__ dy,
                                                                            const int4* __restrict__ idx_max,
                                                                            float4* __restrict__ dx, ConvGeom g,
                                                                            const uint32_t* __restrict__ gate)
{
    const uint32_t cq = (uint32_t)g.c / 4;
    const uint32_t per_image = (uint32_t)g.howo * cq;
    const uint32_t e = blockIdx.x * kThreads + threadIdx.x;
    if (e >= per_image) return;
    const uint32_t win = e / cq, q = e - win * cq;
    const int oy = (int)fd_div(win, g.fd_wo);
    const int ox = (int)win - oy * g.wo;
    const int kh = K > 0 ? K : g.kh, kw = K > 0 ? K : g.kw;
    for (uint32_t nn = blockIdx.y; nn < (uint32_t)g.n; nn += gridDim.y) {
        const int4 rec = idx_max[(size_t)nn * per_image + e];
        const float4 grad = dy[(size_t)nn * per_image + e];
        const int ri[4] = {(int)fd_div((uint32_t)rec.x, g.fd_kh), (int)fd_div((uint32_t)rec.y, g.fd_kh),
                           (int)fd_div((uint32_t)rec.z, g.fd_kh), (int)fd_div((uint32_t)rec.w, g.fd_kh)};
        const int rj[4] = {(int)((uint32_t)rec.x - fd_div((uint32_t)rec.x, g.fd_kw) * g.kw),
                           (int)((uint32_t)rec.y - fd_div((uint32_t)rec.y, g.fd_kw) * g.kw),
                           (int)((uint32_t)rec.z - fd_div((uint32_t)rec.z, g.fd_kw) * g.kw),
                           (int)((uint32_t)rec.w - fd_div((uint32_t)rec.w, g.fd_kw) * g.kw)};
        const float gr[4] = {0.0f + grad.x, 0.0f + grad.y, 0.0f + grad.z, 0.0f + grad.w};
        const size_t first = (((size_t)nn * g.h + (size_t)(oy * kh)) * g.w + (size_t)(ox * kw)) * cq + q;
#pragma unroll
        for (int ii = 0; ii < kh; ++ii)
#pragma unroll
            for (int jj = 0; jj < kw; ++jj) {
                const size_t at = first + ((size_t)ii * g.w + jj) * cq;
                float v[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) v[t] = ri[t] == ii && rj[t] == jj ? gr[t] : 0.0f;
                if (gate) {
                    const uint32_t gt = gate[at];
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] *= (float)(int8_t)(gt >> (8 * t));
                }
                dx[at] = float4{v[0], v[1], v[2], v[3]};
            }
    }
}

// ---------------------------------------------------------------- SGD with momentum
// pydtnn/backends/cpu/optimizers/sgd_cpu.py:28-41: velocity = momentum * velocity + dw;
// w -= lr * (decay * w + velocity)   (Nesterov: w -= lr * (decay * w + dw + momentum * velocity)).
// One launch updates up to kSgdTensors tensors (a layer's weights and biases, or more): every workgroup of
// kSgdBlock elements belongs to one tensor (first_block[] is the running sum of the tensors' workgroup counts)
// and a thread moves four consecutive elements with 128-bit accesses where the tensor allows it.
constexpr int kSgdTensors = 8;
constexpr int kSgdBlock = kThreads * 4;
struct SgdBatch {
    float* w[kSgdTensors];
    const float* dw[kSgdTensors];
    float* velocity[kSgdTensors];
    long total[kSgdTensors];
    unsigned first_block[kSgdTensors + 1];
    int count;
};

__device__ __forceinline__ float sgd_step(float wv, float g, float* v, float lr, float momentum, float decay, int nesterov)
{
    *v = momentum * *v + g;
    const float upd = nesterov ? (decay * wv + g + momentum * *v) : (decay * wv + *v);
    return wv - lr * upd;
}

__global__ void __launch_bounds__(kThreads) sgd_momentum_kernel(SgdBatch b, float lr, float momentum, float decay,
                                                               int nesterov)
{
    int t = 0;
#pragma unroll
    for (int i = 1; i < kSgdTensors; ++i)
        if (i < b.count && blockIdx.x >= b.first_block[i]) t = i;
    float* __restrict__ w = b.w[t];
    const float* __restrict__ dw = b.dw[t];
    float* __restrict__ velocity = b.velocity[t];
    const long total = b.total[t];
    const long idx = ((long)(blockIdx.x - b.first_block[t]) * kThreads + threadIdx.x) * 4;
    if (idx >= total) return;
    const bool vec = idx + 4 <= total &&
                     (((uintptr_t)w | (uintptr_t)dw | (uintptr_t)velocity) & 15) == 0;   // wave-uniform but for the tail
    if (vec) {
        const float4 g = *reinterpret_cast<const float4*>(dw + idx);
        float4 v = *reinterpret_cast<const float4*>(velocity + idx);
        float4 wv = *reinterpret_cast<const float4*>(w + idx);
        wv.x = sgd_step(wv.x, g.x, &v.x, lr, momentum, decay, nesterov);
        wv.y = sgd_step(wv.y, g.y, &v.y, lr, momentum, decay, nesterov);
        wv.z = sgd_step(wv.z, g.z, &v.z, lr, momentum, decay, nesterov);
        wv.w = sgd_step(wv.w, g.w, &v.w, lr, momentum, decay, nesterov);
        *reinterpret_cast<float4*>(w + idx) = wv;
        *reinterpret_cast<float4*>(velocity + idx) = v;
        return;
    }
    for (long i = idx; i < total && i < idx + 4; ++i) {
        float v = velocity[i];
        w[i] = sgd_step(w[i], dw[i], &v, lr, momentum, decay, nesterov);
        velocity[i] = v;
    }
}

// ---------------------------------------------------------------- BatchNormalization, training
// pydtnn/backends/cpu/layers/batch_normalization_cpu.py:59-82 (forward) and :108-129 (backward), on
// tensors viewed as (outer, channels, inner): NCHW is (N, C, H*W), NHWC and 2-D inputs are
// (rows, C, 1), so no transposed copy is made.  Per-channel sums are taken in two deterministic
// stages (slices of the outer axis, then a sum over slices in ascending order).
// What is summed: MODE 0  a = x
//                 MODE 1  a = (x - p0[ch])^2
//                 MODE 2  a = x, b = x * q          (x = dy, q = xn)
template <int MODE>
__device__ __forceinline__ void bn_term(float x, float q, float p0, float* a, float* b)
{
    if (MODE == 0) {
        *a += x;
    } else if (MODE == 1) {
        const float d = x - p0;
        *a += d * d;
    } else {
        *a += x;
        *b += x * q;
    }
}

// NCHW: grid (C, S); slice s covers images [s*per, (s+1)*per).  partial[(which*slices + s)*c + ch]
template <int MODE>
__global__ void __launch_bounds__(kThreads) bn_reduce_nchw_stage1(const float* __restrict__ x,
                                                                 const float* __restrict__ q,
                                                                 const float* __restrict__ p0,
                                                                 float* __restrict__ partial, int n, int c, int hw,
                                                                 int per, int slices)
{
    __shared__ float red[2][kThreads / 64];
    const int ch = blockIdx.x, s = blockIdx.y;
    const int n0 = s * per, n1 = min(n, n0 + per);
    const float shift = MODE == 1 ? p0[ch] : 0.0f;
    float a = 0.0f, b = 0.0f;
    if (hw >= kThreads) {
        for (int nn = n0; nn < n1; ++nn) {
            const long base = ((long)nn * c + ch) * hw;
            for (int i = threadIdx.x; i < hw; i += kThreads)
                bn_term<MODE>(x[base + i], MODE == 2 ? q[base + i] : 0.0f, shift, &a, &b);
        }
    } else {
        // planes smaller than the workgroup: its threads walk the (image, pixel) pairs of the slice together
        const uint32_t count = (uint32_t)(n1 - n0) * (uint32_t)hw;
        for (uint32_t e = threadIdx.x; e < count; e += kThreads) {
            const uint32_t nn = e / (uint32_t)hw, i = e - nn * (uint32_t)hw;
            const long at = ((long)(n0 + (int)nn) * c + ch) * hw + i;
            bn_term<MODE>(x[at], MODE == 2 ? q[at] : 0.0f, shift, &a, &b);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_down(a, off, 64);
        b += __shfl_down(b, off, 64);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { red[0][wave] = a; red[1][wave] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float sa = 0.0f, sb = 0.0f;
        for (int i = 0; i < kThreads / 64; ++i) { sa += red[0][i]; sb += red[1][i]; }
        partial[(long)s * c + ch] = sa;
        if (MODE == 2) partial[((long)slices + s) * c + ch] = sb;
    }
}

// (rows, C): grid (S, ceil(C/64)); block = 64 channels x 4 row lanes.
template <int MODE>
__global__ void __launch_bounds__(kThreads) bn_reduce_rows_stage1(const float* __restrict__ x,
                                                                 const float* __restrict__ q,
                                                                 const float* __restrict__ p0,
                                                                 float* __restrict__ partial, long rows, int c,
                                                                 long per, int slices)
{
    __shared__ float red[2][4][64];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const int ch = blockIdx.y * 64 + cl;
    const long r0 = (long)blockIdx.x * per;
    const long r1 = r0 + per < rows ? r0 + per : rows;
    float a = 0.0f, b = 0.0f;
    if (ch < c) {
        const float shift = MODE == 1 ? p0[ch] : 0.0f;
        for (long r = r0 + rl; r < r1; r += 4)
            bn_term<MODE>(x[r * c + ch], MODE == 2 ? q[r * c + ch] : 0.0f, shift, &a, &b);
    }
    red[0][rl][cl] = a;
    red[1][rl][cl] = b;
    __syncthreads();
    if (rl == 0 && ch < c) {
        partial[(long)blockIdx.x * c + ch] = (red[0][0][cl] + red[0][1][cl]) + (red[0][2][cl] + red[0][3][cl]);
        if (MODE == 2)
            partial[((long)slices + blockIdx.x) * c + ch] =
                (red[1][0][cl] + red[1][1][cl]) + (red[1][2][cl] + red[1][3][cl]);
    }
}

// (rows, C) with a row of `lanes` = C/4 quads, lanes a power of two <= kThreads, 16-byte aligned tensors: as
// bias_grad_rows_quads_stage1, whole rows per 128-bit load and several loads in flight per lane; up to
// kBnSlices row slices.  A row beyond the slice reads as the value that adds nothing (0, or p0 for MODE 1).
template <int MODE>
__global__ void __launch_bounds__(kThreads) bn_reduce_rows_quads_stage1(const float4* __restrict__ x,
                                                                       const float4* __restrict__ q,
                                                                       const float4* __restrict__ p0,
                                                                       float* __restrict__ partial, long rows,
                                                                       int lanes, long per, int slices)
{
    constexpr int kInFlight = MODE == 2 ? 4 : 8;
    __shared__ float4 red[MODE == 2 ? 2 : 1][kThreads];
    const int cl = threadIdx.x & (lanes - 1);
    const int row_lanes = kThreads / lanes, rl = threadIdx.x / lanes;
    const long r0 = (long)blockIdx.x * per;
    const long r1 = r0 + per < rows ? r0 + per : rows;
    const float4 zero = float4{0.0f, 0.0f, 0.0f, 0.0f};
    const float4 shift = MODE == 1 ? p0[cl] : zero;
    float4 a[kInFlight], b[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) a[u] = b[u] = zero;
    for (long r = r0 + rl; r < r1; r += (long)row_lanes * kInFlight) {
        float4 v[kInFlight], w[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            const long rr = r + (long)u * row_lanes;
            v[u] = rr < r1 ? x[rr * lanes + cl] : shift;
            w[u] = MODE == 2 && rr < r1 ? q[rr * lanes + cl] : zero;
        }
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            bn_term<MODE>(v[u].x, w[u].x, shift.x, &a[u].x, &b[u].x);
            bn_term<MODE>(v[u].y, w[u].y, shift.y, &a[u].y, &b[u].y);
            bn_term<MODE>(v[u].z, w[u].z, shift.z, &a[u].z, &b[u].z);
            bn_term<MODE>(v[u].w, w[u].w, shift.w, &a[u].w, &b[u].w);
        }
    }
    float4 ta = a[0], tb = b[0];
#pragma unroll
    for (int u = 1; u < kInFlight; ++u) {
        ta.x += a[u].x; ta.y += a[u].y; ta.z += a[u].z; ta.w += a[u].w;
        tb.x += b[u].x; tb.y += b[u].y; tb.z += b[u].z; tb.w += b[u].w;
    }
    red[0][threadIdx.x] = ta;
    if (MODE == 2) red[MODE == 2 ? 1 : 0][threadIdx.x] = tb;
    __syncthreads();
    if (rl == 0) {
        for (int i = 1; i < row_lanes; ++i) {
            const float4 oa = red[0][i * lanes + cl];
            ta.x += oa.x; ta.y += oa.y; ta.z += oa.z; ta.w += oa.w;
            if (MODE == 2) {
                const float4 ob = red[MODE == 2 ? 1 : 0][i * lanes + cl];
                tb.x += ob.x; tb.y += ob.y; tb.z += ob.z; tb.w += ob.w;
            }
        }
        reinterpret_cast<float4*>(partial + (long)blockIdx.x * lanes * 4)[cl] = ta;
        if (MODE == 2) reinterpret_cast<float4*>(partial + ((long)slices + blockIdx.x) * lanes * 4)[cl] = tb;
    }
}

// Sum over slices of partial[s*c + ch] for the second stages: 16 channels x 16 slice lanes per workgroup, each
// lane adding its slices in ascending order, then the lanes' sums in lane order (thread sl == 0 gets the total).
__device__ __forceinline__ float bn_sum_slices(const float* __restrict__ partial, int c, int slices, int ch, int sl,
                                               float (*red)[17])
{
    float acc = 0.0f;
    if (ch < c)
        for (int s = sl; s < slices; s += 16) acc += partial[(long)s * c + ch];
    __syncthreads();  // red may still be read from a previous call
    red[sl][threadIdx.x & 15] = acc;
    __syncthreads();
    float t = red[0][threadIdx.x & 15];
    for (int i = 1; i < 16; ++i) t += red[i][threadIdx.x & 15];
    return t;
}

// Second stage of the forward statistics.  PASS 0: mu = sum / count.  PASS 1: var = sum / count,
// std = sqrt(var + eps), running statistics updated as momentum*running + (1-momentum)*new.
template <int PASS>
__global__ void __launch_bounds__(kThreads) bn_stats_stage2(const float* __restrict__ partial, int c, int slices,
                                                           float count, float* __restrict__ mu,
                                                           float* __restrict__ std_out, float eps,
                                                           float* __restrict__ running_mean,
                                                           float* __restrict__ running_var, float momentum,
                                                           float one_minus_momentum)
{
    __shared__ float red[16][17];
    const int ch = blockIdx.x * 16 + (threadIdx.x & 15), sl = threadIdx.x >> 4;
    const float acc = bn_sum_slices(partial, c, slices, ch, sl, red);
    if (sl != 0 || ch >= c) return;
    const float mean = acc / count;
    if (PASS == 0) {
        mu[ch] = mean;
    } else {
        std_out[ch] = sqrtf(mean + eps);
        running_mean[ch] = __fadd_rn(__fmul_rn(momentum, running_mean[ch]), __fmul_rn(one_minus_momentum, mu[ch]));
        running_var[ch] = __fadd_rn(__fmul_rn(momentum, running_var[ch]), __fmul_rn(one_minus_momentum, mean));
    }
}

// Second stage of the backward sums: dbeta = sum dy, dgamma = sum dy*xn.
__global__ void __launch_bounds__(kThreads) bn_grads_stage2(const float* __restrict__ partial, int c, int slices,
                                                           float* __restrict__ dgamma, float* __restrict__ dbeta)
{
    __shared__ float red[16][17];
    const int ch = blockIdx.x * 16 + (threadIdx.x & 15), sl = threadIdx.x >> 4;
    const float a = bn_sum_slices(partial, c, slices, ch, sl, red);
    const float b = bn_sum_slices(partial + (long)slices * c, c, slices, ch, sl, red);
    if (sl != 0 || ch >= c) return;
    dbeta[ch] = a;
    dgamma[ch] = b;
}

// xn = (x - mu) / std;  y = gamma * xn + beta   (two roundings in the last step, as NumPy evaluates it)
__global__ void __launch_bounds__(kThreads) bn_train_apply_kernel(const float* __restrict__ x,
                                                                 float* __restrict__ y, float* __restrict__ xn,
                                                                 long total, int inner, int channels,
                                                                 const float* __restrict__ mu,
                                                                 const float* __restrict__ std_in,
                                                                 const float* __restrict__ gamma,
                                                                 const float* __restrict__ beta)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int ch = (int)((idx / inner) % channels);
    const float v = (x[idx] - mu[ch]) / std_in[ch];
    xn[idx] = v;
    y[idx] = __fadd_rn(__fmul_rn(gamma[ch], v), beta[ch]);
}

// dx = (gamma / (std * n)) * (n * dy - xn * dgamma - dbeta)   (bn_training_cython.pyx:236-243)
__global__ void __launch_bounds__(kThreads) bn_train_bwd_kernel(const float* __restrict__ dy,
                                                               const float* __restrict__ xn,
                                                               float* __restrict__ dx, long total, int inner,
                                                               int channels, float n,
                                                               const float* __restrict__ std_in,
                                                               const float* __restrict__ gamma,
                                                               const float* __restrict__ dgamma,
                                                               const float* __restrict__ dbeta)
{
    const long idx = (long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int ch = (int)((idx / inner) % channels);
    const float scale = gamma[ch] / (std_in[ch] * n);
    dx[idx] = scale * (n * dy[idx] - xn[idx] * dgamma[ch] - dbeta[ch]);
}

// ---------------------------------------------------------------- softmax and categorical cross-entropy
// Rows of a (rows, cols) matrix, one workgroup per row.
template <class Op>
__device__ __forceinline__ float block_reduce(float v, Op op, float* red)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();  // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < kThreads / 64; ++i) r = op(r, red[i]);
    return r;  // the same value in every thread
}

struct MaxOp { __device__ float operator()(float a, float b) const { return a > b ? a : b; } };
struct SumOp { __device__ float operator()(float a, float b) const { return a + b; } };

// pydtnn/backends/cpu/activations/softmax_cpu.py:32-35: y = exp(x - max(x)); y /= sum(y)
__global__ void __launch_bounds__(kThreads) softmax_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int cols)
{
    __shared__ float red[kThreads / 64];
    const float* xr = x + (long)blockIdx.x * cols;
    float* yr = y + (long)blockIdx.x * cols;
    float m = -3.402823466e+38f;
    for (int c = threadIdx.x; c < cols; c += kThreads) m = fmaxf(m, xr[c]);
    m = block_reduce(m, MaxOp(), red);
    float sum = 0.0f;
    for (int c = threadIdx.x; c < cols; c += kThreads) {
        const float e = expf(xr[c] - m);
        yr[c] = e;
        sum += e;
    }
    sum = block_reduce(sum, SumOp(), red);
    for (int c = threadIdx.x; c < cols; c += kThreads) yr[c] = yr[c] / sum;
}

// softmax_cpu.py:37-39: dx = y * (dy - sum(dy * y))
__global__ void __launch_bounds__(kThreads) softmax_bwd_kernel(const float* __restrict__ dy,
                                                              const float* __restrict__ y, float* __restrict__ dx,
                                                              int cols)
{
    __shared__ float red[kThreads / 64];
    const long base = (long)blockIdx.x * cols;
    float dot = 0.0f;
    for (int c = threadIdx.x; c < cols; c += kThreads) dot += dy[base + c] * y[base + c];
    dot = block_reduce(dot, SumOp(), red);
    for (int c = threadIdx.x; c < cols; c += kThreads) dx[base + c] = y[base + c] * (dy[base + c] - dot);
}

// pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:28-35, one row per workgroup:
//   a = first argmax of y_targ[row];  p = clip(y_pred[row, a], lo, hi);  row_loss[row] = log(p);
//   dx[row] = y_targ[row] except dx[row, a] = y_targ[row, a] / (-p * global_batch)
__global__ void __launch_bounds__(kThreads) cce_rows_kernel(const float* __restrict__ y_pred,
                                                           const float* __restrict__ y_targ, float* __restrict__ dx,
                                                           float* __restrict__ row_loss, int cols, float lo, float hi,
                                                           float global_batch)
{
    __shared__ float best_v[kThreads];
    __shared__ int best_i[kThreads];
    const long base = (long)blockIdx.x * cols;
    float bv = -3.402823466e+38f;
    int bi = 0x7fffffff;
    for (int c = threadIdx.x; c < cols; c += kThreads) {
        const float v = y_targ[base + c];
        dx[base + c] = v;
        if (bi == 0x7fffffff || v > bv) { bv = v; bi = c; }
    }
    best_v[threadIdx.x] = bv;
    best_i[threadIdx.x] = bi;
    __syncthreads();
    for (int off = kThreads / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            const float ov = best_v[threadIdx.x + off];
            const int oi = best_i[threadIdx.x + off];
            const float mv = best_v[threadIdx.x];
            const int mi = best_i[threadIdx.x];
            // larger value wins; on a tie the smaller column (numpy.argmax returns the first maximum)
            if (oi != 0x7fffffff && (mi == 0x7fffffff || ov > mv || (ov == mv && oi < mi))) {
                best_v[threadIdx.x] = ov;
                best_i[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const int a = best_i[0];
        float p = y_pred[base + a];
        p = p < lo ? lo : (p > hi ? hi : p);
        row_loss[blockIdx.x] = logf(p);
        dx[base + a] = best_v[0] / (-p * global_batch);
    }
}

// loss = -sum(row_loss) / rows, rows added in ascending order by one thread.
__global__ void cce_loss_kernel(const float* __restrict__ row_loss, float* __restrict__ loss, int rows)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float acc = 0.0f;
    for (int r = 0; r < rows; ++r) acc += row_loss[r];
    loss[0] = -acc / (float)rows;
}

}  // namespace

// Algorithmic bytes: 2 * 4 * total (+ 4 * total when a residual is read).
int launch_chan_eltwise(const float* x, const float* residual, float* y, long total, int inner, int channels,
                        const ChanEpilogue& epi, hipStream_t stream)
{
    if (total <= 0 || inner <= 0 || channels <= 0) return PYDTNN_HIP_ERR_INVALID;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) |
                           reinterpret_cast<uintptr_t>(residual)) & 15) == 0;
    const bool no_params = !epi.bias && !epi.mean;
    if (aligned && inner % 4 == 0 && total % inner == 0 && total / inner < (1l << 31) && !no_params) {
        const long planes = total / inner;
        const int inner4 = inner / 4;
        dim3 grid(blocks_for(inner4), (unsigned)(planes < 65535 ? planes : 65535));
        hipLaunchKernelGGL(chan_eltwise_planes_kernel, grid, dim3(kThreads), 0, stream,
                           reinterpret_cast<const float4*>(x), reinterpret_cast<const float4*>(residual),
                           reinterpret_cast<float4*>(y), inner4, (int)planes, channels, epi);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    if (aligned && inner == 1 && channels % 4 == 0 && kThreads % (channels / 4) == 0 && total % channels == 0 &&
        !no_params) {
        const long rows = total / channels;
        const int c4 = channels / 4, rows_per_pass = kThreads / c4;
        // a few passes per thread amortise the parameter fetch
        long blocks = (rows + (long)rows_per_pass * 8 - 1) / ((long)rows_per_pass * 8);
        if (blocks < 1) blocks = 1;
        if (blocks > (1l << 30)) blocks = 1l << 30;
        hipLaunchKernelGGL(chan_eltwise_rows_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                           reinterpret_cast<const float4*>(x), reinterpret_cast<const float4*>(residual),
                           reinterpret_cast<float4*>(y), rows, c4, epi);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    // without per-channel parameters (residual add, ReLU only) the channel of an element does not matter
    const bool vec = aligned && total % 4 == 0 &&
                     (no_params || inner % 4 == 0 || (inner == 1 && channels % 4 == 0));
    if (vec)
        hipLaunchKernelGGL(chan_eltwise_vec4_kernel, dim3(blocks_for(total / 4)), dim3(kThreads), 0, stream,
                           reinterpret_cast<const float4*>(x), reinterpret_cast<const float4*>(residual),
                           reinterpret_cast<float4*>(y), total / 4, inner, channels, epi);
    else
        hipLaunchKernelGGL(chan_eltwise_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, x, residual, y,
                           total, inner, channels, epi);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

// Algorithmic bytes: 4 * total read + 4 * total + total written.
int launch_relu_fwd(const float* x, float* y, int8_t* mask, long total, hipStream_t stream)
{
    if (total <= 0) return PYDTNN_HIP_ERR_INVALID;
    const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(mask) & 3) == 0;
    if (vec)
        hipLaunchKernelGGL(relu_fwd_kernel<true>, dim3(blocks_for((total + 3) / 4)), dim3(kThreads), 0, stream, x, y,
                           mask, total);
    else
        hipLaunchKernelGGL(relu_fwd_kernel<false>, dim3(blocks_for(total)), dim3(kThreads), 0, stream, x, y, mask,
                           total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_relu_bwd(const float* dy, const int8_t* mask, float* dx, long total, hipStream_t stream)
{
    if (total <= 0) return PYDTNN_HIP_ERR_INVALID;
    const bool vec = ((reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(dx)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(mask) & 3) == 0;
    if (vec)
        hipLaunchKernelGGL(relu_bwd_kernel<true>, dim3(blocks_for((total + 3) / 4)), dim3(kThreads), 0, stream, dy,
                           mask, dx, total);
    else
        hipLaunchKernelGGL(relu_bwd_kernel<false>, dim3(blocks_for(total)), dim3(kThreads), 0, stream, dy, mask, dx,
                           total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

constexpr int kBiasGradSlices = 512;

size_t bias_grad_workspace_floats(long outer, int channels)
{
    (void)outer;
    return (size_t)kBiasGradSlices * channels;
}

// inner > 1: dy is (outer, channels, inner) [NCHW]; inner == 1: dy is (outer, channels) rows.
// Algorithmic bytes: 4 * outer * channels * inner read.
int launch_bias_grad(const float* dy, float* db, long outer, int channels, int inner, float* workspace,
                     hipStream_t stream)
{
    if (outer <= 0 || channels <= 0 || inner <= 0 || !workspace) return PYDTNN_HIP_ERR_INVALID;
    int slices;
    if (inner > 1) {
        const int n = (int)outer;
        slices = n < 64 ? n : 64;
        // small planes: a slice holds at least 2048 elements of a channel
        const long by_size = outer * inner / 2048;
        if (inner < kThreads && slices > by_size) slices = by_size < 1 ? 1 : (int)by_size;
        const int per = (n + slices - 1) / slices;
        slices = (n + per - 1) / per;
        if (inner >= kThreads && inner % 4 == 0 && (reinterpret_cast<uintptr_t>(dy) & 15) == 0)
            hipLaunchKernelGGL(bias_grad_nchw_stage1<true>, dim3(channels, slices), dim3(kThreads), 0, stream, dy,
                               workspace, n, channels, inner, per);
        else
            hipLaunchKernelGGL(bias_grad_nchw_stage1<false>, dim3(channels, slices), dim3(kThreads), 0, stream, dy,
                               workspace, n, channels, inner, per);
    } else {
        const int lanes = channels / 4;
        const bool quads = channels % 4 == 0 && lanes <= kThreads && (lanes & (lanes - 1)) == 0 &&
                           (reinterpret_cast<uintptr_t>(dy) & 15) == 0;
        if (quads) {
            // a slice is at least 32 rows per row lane; at most kBiasGradSlices of them
            const long rows_per_load = kThreads / lanes;
            const long want = (outer + rows_per_load * 32 - 1) / (rows_per_load * 32);
            slices = (int)(want < kBiasGradSlices ? want : kBiasGradSlices);
            const long per = (outer + slices - 1) / slices;
            slices = (int)((outer + per - 1) / per);
            hipLaunchKernelGGL(bias_grad_rows_quads_stage1, dim3(slices), dim3(kThreads), 0, stream,
                               reinterpret_cast<const float4*>(dy), workspace, outer, lanes, per);
        } else {
            slices = outer < 64 * 4 ? (int)((outer + 3) / 4) : 64;
            const long per = (outer + slices - 1) / slices;
            slices = (int)((outer + per - 1) / per);
            hipLaunchKernelGGL(bias_grad_rows_stage1, dim3(slices, (channels + 63) / 64), dim3(kThreads), 0, stream,
                               dy, workspace, outer, channels, per);
        }
    }
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(bias_grad_stage2, dim3((channels + 15) / 16), dim3(kThreads), 0, stream, workspace, db,
                       channels, slices);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_splitk_reduce(const float* partial, float* out, long rows, int ncols, long stride, int slices, int perm_c,
                         int khw, const ChanEpilogue& epi, int accumulate, hipStream_t stream)
{
    const long total = rows * ncols;
    if (total <= 0 || slices <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, partial, out, total,
                       stride, slices, ncols, perm_c, khw, epi, accumulate);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_flip_filter(const float* w, float* wf, int nhwc, int kn, int c, int kh, int kw, hipStream_t stream)
{
    const long total = (long)kn * c * kh * kw;
    if (nhwc)
        hipLaunchKernelGGL(flip_filter_nhwc_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, w, wf, kn, c,
                           kh, kw);
    else
        hipLaunchKernelGGL(flip_filter_nchw_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, w, wf, kn, c,
                           kh, kw);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_max_pool_fwd_nchw(const float* x, float* y, int32_t* idx_max, const ConvGeom& g, hipStream_t stream)
{
    const long planes = (long)g.n * g.c;
    dim3 grid(blocks_for(g.howo), (unsigned)(planes < 65535 ? planes : 65535));
    const bool windows2 = g.kh == 2 && g.kw == 2 && g.vstride == 2 && g.hstride == 2 && g.vpadding == 0 &&
                          g.hpadding == 0 && g.vdilation == 1 && g.hdilation == 1 && g.h == 2 * g.ho &&
                          g.w == 2 * g.wo;
    if (windows2 && (reinterpret_cast<uintptr_t>(x) & 7) == 0) {
        hipLaunchKernelGGL(max_pool_fwd_windows2_nchw_kernel, grid, dim3(kThreads), 0, stream, x, y, idx_max, g);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    if (g.kh == 3 && g.kw == 3 && g.vdilation == 1 && g.hdilation == 1) {
        hipLaunchKernelGGL(max_pool_fwd_square_nchw_kernel<3>, grid, dim3(kThreads), 0, stream, x, y, idx_max, g);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    hipLaunchKernelGGL(max_pool_fwd_nchw_kernel, grid, dim3(kThreads), 0, stream, x, y, idx_max, g);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

// `gate` (optional, shaped like dx): dx is stored multiplied by it, ReLU's backward of the layer below.
int launch_max_pool_bwd_nchw(const float* dy, const int32_t* idx_max, float* dx, const ConvGeom& g,
                             hipStream_t stream, const int8_t* gate)
{
    const long planes = (long)g.n * g.c;
    dim3 grid(blocks_for((long)g.h * g.w), (unsigned)(planes < 65535 ? planes : 65535));
    // square windows only: with kh != kw the reference's decode can leave the window it came from and land
    // in a neighbour's, which only the general gather follows
    const bool tiled = g.kh == g.kw && g.kh == g.vstride && g.kw == g.hstride && g.vpadding == 0 &&
                       g.hpadding == 0 && g.vdilation == 1 && g.hdilation == 1;
    if (tiled && g.h == g.ho * g.kh && g.w == g.wo * g.kw) {
        dim3 wgrid(blocks_for(g.howo), (unsigned)(planes < 65535 ? planes : 65535));
        const uintptr_t all = reinterpret_cast<uintptr_t>(dx) | reinterpret_cast<uintptr_t>(dy) |
                              reinterpret_cast<uintptr_t>(idx_max) | reinterpret_cast<uintptr_t>(gate);
        if (g.kw == 2 && g.wo % 2 == 0 && (all & 15) == 0 && g.howo / 2 < (1 << 30)) {
            dim3 pgrid(blocks_for(g.howo / 2), wgrid.y);
            hipLaunchKernelGGL(max_pool_bwd_window_pairs_nchw_kernel, pgrid, dim3(kThreads), 0, stream,
                               reinterpret_cast<const float2*>(dy), reinterpret_cast<const int2*>(idx_max),
                               reinterpret_cast<float4*>(dx), g, reinterpret_cast<const uint32_t*>(gate));
        } else if (g.kw == 2 && (reinterpret_cast<uintptr_t>(dx) & 7) == 0)
            hipLaunchKernelGGL(max_pool_bwd_windows_nchw_kernel<2>, wgrid, dim3(kThreads), 0, stream, dy, idx_max, dx,
                               g, gate);
        else
            hipLaunchKernelGGL(max_pool_bwd_windows_nchw_kernel<0>, wgrid, dim3(kThreads), 0, stream, dy, idx_max, dx,
                               g, gate);
    } else if (tiled)
        hipLaunchKernelGGL(max_pool_bwd_nchw_kernel<true>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g, gate);
    else if (g.kh == g.kw && g.vdilation == 1 && g.hdilation == 1 && g.kh <= 2 * g.vstride && g.kw <= 2 * g.hstride)
        hipLaunchKernelGGL(max_pool_bwd_ranges_nchw_kernel<2>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g, gate);
    else if (g.kh == g.kw && g.vdilation == 1 && g.hdilation == 1)
        hipLaunchKernelGGL(max_pool_bwd_ranges_nchw_kernel<0>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g, gate);
    else
        hipLaunchKernelGGL(max_pool_bwd_nchw_kernel<false>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g, gate);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_max_pool_fwd_nhwc(const float* x, float* y, int32_t* idx_max, const ConvGeom& g, hipStream_t stream)
{
    const long per_image = (long)g.howo * g.c;
    if (per_image >= (1l << 31) - kThreads) return PYDTNN_HIP_ERR_UNSUPPORTED;
    const bool windows2 = g.kh == 2 && g.kw == 2 && g.vstride == 2 && g.hstride == 2 && g.vpadding == 0 &&
                          g.hpadding == 0 && g.vdilation == 1 && g.hdilation == 1 && g.h == 2 * g.ho &&
                          g.w == 2 * g.wo;
    if (windows2 && g.c % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(idx_max)) & 15) ==
            0) {
        dim3 wgrid(blocks_for(per_image / 4), (unsigned)(g.n < 65535 ? g.n : 65535));
        hipLaunchKernelGGL(max_pool_fwd_windows2_nhwc_kernel, wgrid, dim3(kThreads), 0, stream,
                           reinterpret_cast<const float4*>(x), reinterpret_cast<float4*>(y),
                           reinterpret_cast<int4*>(idx_max), g);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    const int c_exact = (unsigned long)(per_image + kThreads) * (unsigned long)g.c < (1ul << 32);
    dim3 grid(blocks_for(per_image), (unsigned)(g.n < 65535 ? g.n : 65535));
    if (g.kh == 3 && g.kw == 3 && g.vdilation == 1 && g.hdilation == 1) {
        hipLaunchKernelGGL(max_pool_fwd_square_nhwc_kernel<3>, grid, dim3(kThreads), 0, stream, x, y, idx_max, g,
                           c_exact);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    hipLaunchKernelGGL(max_pool_fwd_nhwc_kernel, grid, dim3(kThreads), 0, stream, x, y, idx_max, g, c_exact);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_max_pool_bwd_nhwc(const float* dy, const int32_t* idx_max, float* dx, const ConvGeom& g,
                             hipStream_t stream, const int8_t* gate)
{
    const long per_image = (long)g.h * g.w * g.c;
    if (per_image >= (1l << 31) - kThreads) return PYDTNN_HIP_ERR_UNSUPPORTED;
    const bool tiled = g.kh == g.kw && g.kh == g.vstride && g.kw == g.hstride && g.vpadding == 0 &&
                       g.hpadding == 0 && g.vdilation == 1 && g.hdilation == 1 && g.h == g.ho * g.kh &&
                       g.w == g.wo * g.kw;
    const auto aligned = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    if (tiled && g.c % 4 == 0 && aligned(dy, 16) && aligned(idx_max, 16) && aligned(dx, 16) &&
        (!gate || aligned(gate, 4))) {
        dim3 wgrid(blocks_for((long)g.howo * (g.c / 4)), (unsigned)(g.n < 65535 ? g.n : 65535));
        const auto dy4 = reinterpret_cast<const float4*>(dy);
        const auto idx4 = reinterpret_cast<const int4*>(idx_max);
        const auto dx4 = reinterpret_cast<float4*>(dx);
        const auto gate4 = reinterpret_cast<const uint32_t*>(gate);
        if (g.kh == 2)
            hipLaunchKernelGGL(max_pool_bwd_windows_nhwc_kernel<2>, wgrid, dim3(kThreads), 0, stream, dy4, idx4, dx4, g,
                               gate4);
        else
            hipLaunchKernelGGL(max_pool_bwd_windows_nhwc_kernel<0>, wgrid, dim3(kThreads), 0, stream, dy4, idx4, dx4, g,
                               gate4);
        HIP_RETURN_IF_LAUNCH_FAILED();
        return PYDTNN_HIP_OK;
    }
    const int c_exact = (unsigned long)(per_image + kThreads) * (unsigned long)g.c < (1ul << 32);
    dim3 grid(blocks_for(per_image), (unsigned)(g.n < 65535 ? g.n : 65535));
    if (g.kh == g.kw && g.vdilation == 1 && g.hdilation == 1 && g.kh <= 2 * g.vstride && g.kw <= 2 * g.hstride)
        hipLaunchKernelGGL(max_pool_bwd_ranges_nhwc_kernel<2>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g,
                           c_exact, gate);
    else if (g.kh == g.kw && g.vdilation == 1 && g.hdilation == 1)
        hipLaunchKernelGGL(max_pool_bwd_ranges_nhwc_kernel<0>, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g,
                           c_exact, gate);
    else
        hipLaunchKernelGGL(max_pool_bwd_nhwc_kernel, grid, dim3(kThreads), 0, stream, dy, idx_max, dx, g, c_exact,
                           gate);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_sgd_momentum_multi(int count, float* const* w, const float* const* dw, float* const* velocity,
                              const long* total, float lr, float momentum, float decay, int nesterov, hipStream_t stream)
{
    if (count <= 0 || !w || !dw || !velocity || !total) return PYDTNN_HIP_ERR_INVALID;
    for (int i0 = 0; i0 < count; i0 += kSgdTensors) {
        SgdBatch b;
        b.count = count - i0 < kSgdTensors ? count - i0 : kSgdTensors;
        unsigned blocks = 0;
        for (int i = 0; i < kSgdTensors; ++i) {
            const int j = i < b.count ? i0 + i : i0;
            if (!w[j] || !dw[j] || !velocity[j] || total[j] <= 0) return PYDTNN_HIP_ERR_INVALID;
            const long nb = (total[j] + kSgdBlock - 1) / kSgdBlock;
            if (nb + blocks >= (1l << 31)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            b.w[i] = w[j]; b.dw[i] = dw[j]; b.velocity[i] = velocity[j]; b.total[i] = total[j];
            b.first_block[i] = blocks;
            if (i < b.count) blocks += (unsigned)nb;
        }
        b.first_block[kSgdTensors] = blocks;
        hipLaunchKernelGGL(sgd_momentum_kernel, dim3(blocks), dim3(kThreads), 0, stream, b, lr, momentum, decay, nesterov);
        HIP_RETURN_IF_LAUNCH_FAILED();
    }
    return PYDTNN_HIP_OK;
}

int launch_sgd_momentum(float* w, const float* dw, float* velocity, long total, float lr, float momentum, float decay,
                        int nesterov, hipStream_t stream)
{
    return launch_sgd_momentum_multi(1, &w, &dw, &velocity, &total, lr, momentum, decay, nesterov, stream);
}

int launch_softmax_fwd(const float* x, float* y, int rows, int cols, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(softmax_fwd_kernel, dim3(rows), dim3(kThreads), 0, stream, x, y, cols);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_softmax_bwd(const float* dy, const float* y, float* dx, int rows, int cols, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(softmax_bwd_kernel, dim3(rows), dim3(kThreads), 0, stream, dy, y, dx, cols);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int launch_cce(const float* y_pred, const float* y_targ, float* dx, float* loss, float* row_loss, int rows, int cols,
               float lo, float hi, float global_batch, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(cce_rows_kernel, dim3(rows), dim3(kThreads), 0, stream, y_pred, y_targ, dx, row_loss, cols, lo,
                       hi, global_batch);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(cce_loss_kernel, dim3(1), dim3(64), 0, stream, row_loss, loss, rows);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

// Slices of the outer axis for a two-stage channel reduction; at most 64 (kBnSlices for the 16-byte row kernel).
constexpr int kBnSlices = 512;

static int bn_slices(long outer, int inner, long* per)
{
    long slices;
    if (inner > 1) {
        slices = outer < 64 ? outer : 64;
        // small planes: a slice holds at least 2048 elements of a channel
        const long by_size = outer * inner / 2048;
        if (inner < kThreads && slices > by_size) slices = by_size < 1 ? 1 : by_size;
    } else {
        slices = outer < 64 * 4 ? (outer + 3) / 4 : 64;
    }
    *per = (outer + slices - 1) / slices;
    return (int)((outer + *per - 1) / *per);
}

template <int MODE>
static void bn_reduce_stage1(const float* x, const float* q, const float* p0, float* partial, long outer, int channels,
                             int inner, hipStream_t stream, int* slices_out)
{
    long per;
    int slices = bn_slices(outer, inner, &per);
    const int lanes = channels / 4;
    const auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (inner > 1) {
        hipLaunchKernelGGL(bn_reduce_nchw_stage1<MODE>, dim3(channels, slices), dim3(kThreads), 0, stream, x, q, p0,
                           partial, (int)outer, channels, inner, (int)per, slices);
    } else if (channels % 4 == 0 && lanes <= kThreads && (lanes & (lanes - 1)) == 0 && aligned16(x) &&
               (MODE != 2 || aligned16(q)) && (MODE != 1 || aligned16(p0)) && aligned16(partial)) {
        // a slice is at least 32 rows per row lane
        const long rows_per_load = kThreads / lanes;
        const long want = (outer + rows_per_load * 32 - 1) / (rows_per_load * 32);
        slices = (int)(want < kBnSlices ? want : kBnSlices);
        per = (outer + slices - 1) / slices;
        slices = (int)((outer + per - 1) / per);
        hipLaunchKernelGGL(bn_reduce_rows_quads_stage1<MODE>, dim3(slices), dim3(kThreads), 0, stream,
                           reinterpret_cast<const float4*>(x), reinterpret_cast<const float4*>(q),
                           reinterpret_cast<const float4*>(p0), partial, outer, lanes, per, slices);
    } else {
        hipLaunchKernelGGL(bn_reduce_rows_stage1<MODE>, dim3(slices, (channels + 63) / 64), dim3(kThreads), 0, stream,
                           x, q, p0, partial, outer, channels, per, slices);
    }
    *slices_out = slices;
}

// floats: two sets of kBnSlices partial sums per channel, then mu (16-byte aligned when the workspace is)
size_t bn_training_workspace_floats(int channels) { return (size_t)(2 * kBnSlices + 4) * channels; }

// Algorithmic bytes: x read three times (mean, variance, normalise), y and xn written: 20 bytes per element.
int launch_bn_training_fwd(const float* x, float* y, float* xn, float* std_out, const float* gamma, const float* beta,
                           float* running_mean, float* running_var, float momentum, float one_minus_momentum, float eps,
                           long outer, int channels, int inner, float* workspace, hipStream_t stream)
{
    if (outer <= 0 || channels <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (inner > 1 && outer >= (1l << 31)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    float* partial = workspace;
    float* mu = workspace + (size_t)2 * kBnSlices * channels;
    const float count = (float)(outer * inner);
    const long total = outer * channels * inner;
    int slices = 0;
    bn_reduce_stage1<0>(x, nullptr, nullptr, partial, outer, channels, inner, stream, &slices);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(bn_stats_stage2<0>, dim3((channels + 15) / 16), dim3(kThreads), 0, stream, partial, channels,
                       slices, count, mu, std_out, eps, running_mean, running_var, momentum, one_minus_momentum);
    HIP_RETURN_IF_LAUNCH_FAILED();
    bn_reduce_stage1<1>(x, nullptr, mu, partial, outer, channels, inner, stream, &slices);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(bn_stats_stage2<1>, dim3((channels + 15) / 16), dim3(kThreads), 0, stream, partial, channels,
                       slices, count, mu, std_out, eps, running_mean, running_var, momentum, one_minus_momentum);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(bn_train_apply_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, x, y, xn, total,
                       inner, channels, mu, std_out, gamma, beta);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

// Algorithmic bytes: dy and xn read twice, dx written: 20 bytes per element (16 without dx).
int launch_bn_training_bwd(const float* dy, const float* xn, const float* std_in, const float* gamma, float* dgamma,
                           float* dbeta, float* dx, long outer, int channels, int inner, float* workspace,
                           hipStream_t stream)
{
    if (outer <= 0 || channels <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (inner > 1 && outer >= (1l << 31)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    const long total = outer * channels * inner;
    int slices = 0;
    bn_reduce_stage1<2>(dy, xn, nullptr, workspace, outer, channels, inner, stream, &slices);
    HIP_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(bn_grads_stage2, dim3((channels + 15) / 16), dim3(kThreads), 0, stream, workspace, channels,
                       slices, dgamma, dbeta);
    HIP_RETURN_IF_LAUNCH_FAILED();
    if (dx) {
        hipLaunchKernelGGL(bn_train_bwd_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, stream, dy, xn, dx, total,
                           inner, channels, (float)(outer * inner), std_in, gamma, dgamma, dbeta);
        HIP_RETURN_IF_LAUNCH_FAILED();
    }
    return PYDTNN_HIP_OK;
}

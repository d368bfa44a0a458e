// The float64 route of the path: the explicit (im2col / im2row + GEMM) convolution and the FC layer, which is
// what the reference runs in float64 (its im2col / im2row / col2im / row2im, add, ReLU and BN-inference
// modules dispatch on float64, pydtnn/cython_modules/im2row_nhwc_cython.pyx:25-49, and utils.matmul is a plain
// a @ b, pydtnn/utils/__init__.py:148-158; libconvGemm, the implicit route, is float32 only,
// pydtnn/backends/cpu/libs/conv_gemm.py:101-107).
//
// GEMM: v_mfma_f64_16x16x4_f64.  A workgroup of four wavefronts owns a 128 x 128 tile of C, a wavefront 64 x 64
// = 4 x 4 blocks of 16 x 16 (lane l holds C[4v + l/16][l%16] of a block in register pair v; the A operand wants
// A[l%16][l/16] and B wants B[l/16][l%16]).  The reduction axis is walked in steps of 16: both tiles go
// through LDS k-major ([k][m], row pitch 130 doubles so that stores along k and operand fetches along m
// spread over the banks), double buffered with the next step's tiles prefetched into registers, one barrier per
// step.  Operands may be the transposed view of a row-major matrix (NumPy hands such views to BLAS for
// x_rows.T and weights.T).  Small C with a long reduction (the filter gradient, an FC layer at batch 64) is
// split along k into a workspace and summed in a fixed order.
//
// The streaming kernels beside it (gathers, per-channel epilogue, ReLU, bias gradient, the (1,0,2,3)
// transpose) are one thread per element with the reference's index maps and summation orders.
#include "conv_internal.h"

namespace {

typedef double doublex4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128, kBN = 128, kBK64 = 16, kPitch = 130;

struct Dgemm {
    const double* a;
    const double* b;
    double* c;          // C, or the workspace when splits > 1
    long lda, ldb, ldc;
    int m, n, k;
    int transa, transb;
    int chunk;          // reduction elements per split (a multiple of 16)
    const double* bias; // per column, applied when splits == 1
    int relu;
    int tiles_m;        // tiles along m; a workgroup's tile is blockIdx.x + tile0, m fastest
    int tile0;
    int compact;        // partial tiles go to c as [split][blockIdx.x][128][128] (the tail launch)
};

typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));

// A descriptor over "everything from p on": the loads below only use offsets of elements that exist (rows and
// columns beyond the matrix are clamped, reduction indices beyond the chunk are not loaded), so no range check
// is wanted from it.
__device__ __forceinline__ gemm::rsrc_t open_rsrc(const double* p)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<double*>(p), 0, -1, 0x00020000);
}
__device__ __forceinline__ double load64(gemm::rsrc_t r, uint32_t byte_offset)
{
    return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_offset, 0, 0));
}

template <bool TA, bool TB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) dgemm_kernel(Dgemm g)
{
    __shared__ double As[2][kBK64 * kPitch];
    __shared__ double Bs[2][kBK64 * kPitch];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile = (int)blockIdx.x + g.tile0;
    const int m0 = (tile % g.tiles_m) * kBM, n0 = (tile / g.tiles_m) * kBN;
    const int split = blockIdx.y;
    const int kbeg = split * g.chunk;
    const int kend = min(g.k, kbeg + g.chunk);
    const int wm0 = (wave & 1) * 64, wn0 = (wave >> 1) * 64;
    const int fi = lane & 15, fk = lane >> 4;

    // thread -> tile element maps for the global loads: lanes run along the operand's contiguous axis
    //   k contiguous: (kk = tid % 16, mn = tid / 16 + 16 e);  mn contiguous: (mn = tid % 128, kk = tid / 128 + 2 e)
    // A step's elements are fetched with buffer loads from the step's corner of the operand (a scalar pointer
    // that moves with k) at per-thread byte offsets that are computed once: no vector arithmetic per load.  Rows
    // of A / columns of B beyond the matrix are clamped to the last one (they only feed rows / columns of C that
    // are never stored); the one step that may reach beyond the chunk's end tests each element.
    uint32_t offa[8], offb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        if (TA) offa[e] = (uint32_t)(((long)((tid >> 7) + 2 * e) * g.lda + (min(m0 + (tid & 127), g.m - 1) - m0)) * 8);
        else offa[e] = (uint32_t)(((long)(min(m0 + (tid >> 4) + 16 * e, g.m - 1) - m0) * g.lda + (tid & 15)) * 8);
        if (TB) offb[e] = (uint32_t)(((long)(min(n0 + (tid >> 4) + 16 * e, g.n - 1) - n0) * g.ldb + (tid & 15)) * 8);
        else offb[e] = (uint32_t)(((long)((tid >> 7) + 2 * e) * g.ldb + (min(n0 + (tid & 127), g.n - 1) - n0)) * 8);
    }
    double ra[8], rb[8];
    auto fetch = [&](int k0) {
        const gemm::rsrc_t wa = open_rsrc(TA ? g.a + (long)k0 * g.lda + m0 : g.a + (long)m0 * g.lda + k0);
        const gemm::rsrc_t wb = open_rsrc(TB ? g.b + (long)n0 * g.ldb + k0 : g.b + (long)k0 * g.ldb + n0);
        if (k0 + kBK64 <= kend) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ra[e] = load64(wa, offa[e]);
                rb[e] = load64(wb, offb[e]);
            }
        } else {
            // the reduction index of element e within the step, and the element's offset with that index set to 0
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ka = TA ? (tid >> 7) + 2 * e : (tid & 15);
                const int kb = TB ? (tid & 15) : (tid >> 7) + 2 * e;
                const bool oka = k0 + ka < kend, okb = k0 + kb < kend;
                const uint32_t za = offa[e] - (uint32_t)((TA ? (long)ka * g.lda : (long)ka) * 8);
                const uint32_t zb = offb[e] - (uint32_t)((TB ? (long)kb : (long)kb * g.ldb) * 8);
                const double va = load64(wa, oka ? offa[e] : za), vb = load64(wb, okb ? offb[e] : zb);
                ra[e] = oka ? va : 0.0;
                rb[e] = okb ? vb : 0.0;
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (TA) As[buf][((tid >> 7) + 2 * e) * kPitch + (tid & 127)] = ra[e];
            else As[buf][(tid & 15) * kPitch + (tid >> 4) + 16 * e] = ra[e];
            if (TB) Bs[buf][(tid & 15) * kPitch + (tid >> 4) + 16 * e] = rb[e];
            else Bs[buf][((tid >> 7) + 2 * e) * kPitch + (tid & 127)] = rb[e];
        }
    };

    doublex4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = doublex4{0.0, 0.0, 0.0, 0.0};

    fetch(kbeg);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = kbeg; k0 < kend; k0 += kBK64) {
        const bool more = k0 + kBK64 < kend;
        if (more) fetch(k0 + kBK64);
#pragma unroll
        for (int kg = 0; kg < kBK64 / 4; ++kg) {
            double af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) af[i] = As[buf][(kg * 4 + fk) * kPitch + wm0 + i * 16 + fi];
#pragma unroll
            for (int j = 0; j < 4; ++j) bf[j] = Bs[buf][(kg * 4 + fk) * kPitch + wn0 + j * 16 + fi];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    if (g.compact) {
        double* part = g.c + ((long)split * gridDim.x + blockIdx.x) * (kBM * kBN);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    part[(wm0 + i * 16 + 4 * v + fk) * kBN + wn0 + j * 16 + fi] = acc[i][j][v];
        return;
    }
    double* out = g.c + (long)split * g.m * g.ldc;  // split > 0 only with the workspace, whose ldc is n
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = n0 + wn0 + j * 16 + fi;
        if (col >= g.n) continue;
        const double bias = g.bias ? g.bias[col] : 0.0;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int row = m0 + wm0 + i * 16 + 4 * v + fk;
                if (row >= g.m) continue;
                double val = acc[i][j][v];
                if (g.bias) val += bias;
                if (g.relu) val = val > 0.0 ? val : 0.0;
                out[(long)row * g.ldc + col] = val;
            }
    }
}

// C[i] = relu?(sum over splits of ws[s][i] (+ bias[col])), splits added in ascending order
__global__ void __launch_bounds__(256) dgemm_reduce_kernel(const double* ws, double* c, long ldc, long m, int n,
                                                           int splits, const double* bias, int relu)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= m * n) return;
    double s = 0.0;
    for (int z = 0; z < splits; ++z) s += ws[(long)z * m * n + i];
    const long row = i / n;
    const int col = (int)(i - row * n);
    if (bias) s += bias[col];
    if (relu) s = s > 0.0 ? s : 0.0;
    c[row * ldc + col] = s;
}

// The tiles of the tail launch: C[tile] = relu?(sum over splits of part[s][t] (+ bias[col])), ascending splits
__global__ void __launch_bounds__(256) dgemm_tail_reduce_kernel(const double* ws, double* c, long ldc, int m, int n,
                                                                int tiles_m, int tile0, int tail, int splits,
                                                                const double* bias, int relu)
{
    const int t = blockIdx.x / (kBM * kBN / 256);
    const int e = (blockIdx.x % (kBM * kBN / 256)) * 256 + threadIdx.x;
    const int tile = tile0 + t;
    const int row = (tile % tiles_m) * kBM + e / kBN, col = (tile / tiles_m) * kBN + e % kBN;
    if (row >= m || col >= n) return;
    double s = 0.0;
    for (int z = 0; z < splits; ++z) s += ws[((long)z * tail + t) * (kBM * kBN) + e];
    if (bias) s += bias[col];
    if (relu) s = s > 0.0 ? s : 0.0;
    c[(long)row * ldc + col] = s;
}

// What the chip holds at once: two workgroups on each of 256 compute units.
constexpr long kDgemmResident = 512;

struct DgemmPlan {
    int splits;
    int chunk;
    // Many whole tiles: the grid runs as rounds of kDgemmResident tiles and a last, partly empty round costs as
    // much as a full one (3136 tiles = 6.125 rounds take the time of 7).  The tiles of a last round that fills at
    // most half the chip go to a second launch instead, split along k so that they fill it once, into a
    // workspace of partial tiles that dgemm_tail_reduce_kernel sums.
    int tail;          // tiles of the second launch (0: none)
    int tail_splits;
    int tail_chunk;
};

DgemmPlan plan_dgemm(long m, long n, long k)
{
    const long tiles = ((m + kBM - 1) / kBM) * ((n + kBN - 1) / kBN);
    // as many chunks as fill the 512 resident workgroups (two per CU) once: a few more would run alone in a second round
    long want = tiles >= 256 ? 1 : 512 / tiles;
    long chunk = ((k + want - 1) / want + 15) / 16 * 16;
    if (chunk < 256) chunk = 256;
    if (chunk > k) chunk = (k + 15) / 16 * 16;
    DgemmPlan p;
    p.chunk = (int)chunk;
    p.splits = (int)((k + chunk - 1) / chunk);
    p.tail = 0; p.tail_splits = 1; p.tail_chunk = p.chunk;
    const long tail = tiles % kDgemmResident;
    if (p.splits == 1 && tiles >= 2 * kDgemmResident && tail > 0 && 2 * tail <= kDgemmResident && k >= 512) {
        long ts = kDgemmResident / tail;
        if (ts > k / 256) ts = k / 256;
        const long tc = ((k + ts - 1) / ts + 15) / 16 * 16;
        p.tail = (int)tail;
        p.tail_chunk = (int)tc;
        p.tail_splits = (int)((k + tc - 1) / tc);
    }
    return p;
}

size_t dgemm_plan_bytes(const DgemmPlan& p, long m, long n)
{
    if (p.splits > 1) return (size_t)p.splits * m * n * 8;
    return (size_t)p.tail * p.tail_splits * kBM * kBN * 8;
}

// ---------------------------------------------------------------- streaming kernels
// im2col (NCHW): cols[(c*kh + i)*kw + j][(n*ho + y)*wo + x] = X[n, c, sv*y + dv*i - pv, sh*x + dh*j - ph] or 0
// (pydtnn/cython_modules/im2col_nchw_cython.pyx:104-124).  One thread per element of cols, lanes along pixels.
__global__ void __launch_bounds__(256) im2col_nchw_f64_kernel(const double* __restrict__ x, double* __restrict__ cols,
                                                              ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const long row = idx / g.p, col = idx - row * g.p;
    const int cc = (int)(row / g.khw), rem = (int)(row - (long)cc * g.khw), ii = rem / g.kw, jj = rem - ii * g.kw;
    const int nn = (int)(col / g.howo), pp = (int)(col - (long)nn * g.howo), yy = pp / g.wo, xx = pp - yy * g.wo;
    const int ih = g.vstride * yy + g.vdilation * ii - g.vpadding, iw = g.hstride * xx + g.hdilation * jj - g.hpadding;
    const bool ok = (unsigned)ih < (unsigned)g.h && (unsigned)iw < (unsigned)g.w;
    cols[idx] = ok ? x[(((long)nn * g.c + cc) * g.h + ih) * g.w + iw] : 0.0;
}

// col2im (NCHW), gather form: dx[n, c, ih, iw] = sum over (i, j) ascending of the cols entries that map to it
// (pydtnn/cython_modules/im2col_nchw_cython.pyx:224-244 adds them in that order).
__global__ void __launch_bounds__(256) col2im_nchw_f64_kernel(const double* __restrict__ cols, double* __restrict__ dx,
                                                              ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    long r = idx;
    const int iw = (int)(r % g.w); r /= g.w;
    const int ih = (int)(r % g.h); r /= g.h;
    const int cc = (int)(r % g.c);
    const int nn = (int)(r / g.c);
    double acc = 0.0;
    for (int ii = 0; ii < g.kh; ++ii) {
        const int nv = ih + g.vpadding - g.vdilation * ii;
        if (nv < 0 || nv % g.vstride != 0 || nv / g.vstride >= g.ho) continue;
        const int yy = nv / g.vstride;
        for (int jj = 0; jj < g.kw; ++jj) {
            const int nh = iw + g.hpadding - g.hdilation * jj;
            if (nh < 0 || nh % g.hstride != 0 || nh / g.hstride >= g.wo) continue;
            const int xx = nh / g.hstride;
            acc += cols[((long)(cc * g.kh + ii) * g.kw + jj) * g.p + ((long)nn * g.ho + yy) * g.wo + xx];
        }
    }
    dx[idx] = acc;
}

// im2row (NHWC): rows[(n*ho + y)*wo + x][(c*kh + i)*kw + j] = X[n, ih, iw, c] or 0
// (pydtnn/cython_modules/im2row_nhwc_cython.pyx:77-97).  One thread per (pixel, tap, channel), lanes along the
// channels: reads are contiguous, a wavefront's writes fall into one row of `rows`, kh*kw doubles apart.
__global__ void __launch_bounds__(256) im2row_nhwc_f64_kernel(const double* __restrict__ x, double* __restrict__ rows,
                                                              ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    long r = idx;
    const int cc = (int)(r % g.c); r /= g.c;
    const int t = (int)(r % g.khw);
    const long pix = r / g.khw;
    const int ii = t / g.kw, jj = t - ii * g.kw;
    const int nn = (int)(pix / g.howo), pp = (int)(pix - (long)nn * g.howo), yy = pp / g.wo, xx = pp - yy * g.wo;
    const int ih = g.vstride * yy + g.vdilation * ii - g.vpadding, iw = g.hstride * xx + g.hdilation * jj - g.hpadding;
    const bool ok = (unsigned)ih < (unsigned)g.h && (unsigned)iw < (unsigned)g.w;
    rows[pix * g.k + (long)cc * g.khw + t] = ok ? x[(((long)nn * g.h + ih) * g.w + iw) * g.c + cc] : 0.0;
}

// row2im (NHWC), gather form.  The reference walks the rows of the matrix in order and scatters
// (pydtnn/cython_modules/im2row_nhwc_cython.pyx:174-194): an input pixel receives its contributions by
// ascending output pixel (y, x), which is descending tap (i, j).
__global__ void __launch_bounds__(256) row2im_nhwc_f64_kernel(const double* __restrict__ rows, double* __restrict__ dx,
                                                              ConvGeom g, long total)
{
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    long r = idx;
    const int cc = (int)(r % g.c); r /= g.c;
    const int iw = (int)(r % g.w); r /= g.w;
    const int ih = (int)(r % g.h);
    const int nn = (int)(r / g.h);
    double acc = 0.0;
    for (int ii = g.kh - 1; ii >= 0; --ii) {
        const int nv = ih + g.vpadding - g.vdilation * ii;
        if (nv < 0 || nv % g.vstride != 0 || nv / g.vstride >= g.ho) continue;
        const int yy = nv / g.vstride;
        for (int jj = g.kw - 1; jj >= 0; --jj) {
            const int nh = iw + g.hpadding - g.hdilation * jj;
            if (nh < 0 || nh % g.hstride != 0 || nh / g.hstride >= g.wo) continue;
            const int xx = nh / g.hstride;
            acc += rows[(((long)nn * g.ho + yy) * g.wo + xx) * g.k + (long)(cc * g.kh + ii) * g.kw + jj];
        }
    }
    dx[idx] = acc;
}

// y = relu?(bn?(x (+ residual) + bias)) with channel = (index / inner) % channels: add_nchw / add_nhwc,
// bn_inference, bn_relu_inference, eltw_sum in float64 (the float32 entry point cites the modules).
struct ChanEpilogue64 {
    const double *bias, *mean, *inv_std, *gamma, *beta;
    int relu;
};
__global__ void __launch_bounds__(256) chan_eltwise_f64_kernel(const double* __restrict__ x,
                                                               const double* __restrict__ residual, double* y,
                                                               long total, long inner, int channels, ChanEpilogue64 e)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int ch = (int)((i / inner) % channels);
    double v = x[i];
    if (residual) v += residual[i];
    if (e.bias) v += e.bias[ch];
    if (e.mean) {
        const double t = (v - e.mean[ch]) * e.inv_std[ch];
        v = t * e.gamma[ch] + e.beta[ch];
    }
    if (e.relu) v = v > 0.0 ? v : 0.0;
    y[i] = v;
}

__global__ void __launch_bounds__(256) relu_fwd_f64_kernel(const double* x, double* y, int8_t* mask, long total)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const double v = x[i];
    y[i] = v > 0.0 ? v : 0.0;
    if (mask) mask[i] = v > 0.0 ? 1 : 0;
}

__global__ void __launch_bounds__(256) relu_bwd_f64_kernel(const double* dy, const int8_t* mask, double* dx, long total)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) dx[i] = dy[i] * (double)mask[i];
}

// db[ch] = sum over (outer, inner) of dy[(o*channels + ch)*inner + p]: one workgroup per channel, every thread
// sums a strided subset in ascending order, then a tree over the 256 partial sums (a fixed order).
__global__ void __launch_bounds__(256) bias_grad_f64_kernel(const double* __restrict__ dy, double* __restrict__ db,
                                                            long outer, int channels, long inner)
{
    __shared__ double part[256];
    const int ch = blockIdx.x;
    double s = 0.0;
    const long count = outer * inner;
    for (long i = threadIdx.x; i < count; i += 256) {
        const long o = i / inner, p = i - o * inner;
        s += dy[(o * channels + ch) * inner + p];
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int step = 128; step > 0; step >>= 1) {
        if ((int)threadIdx.x < step) part[threadIdx.x] += part[threadIdx.x + step];
        __syncthreads();
    }
    if (threadIdx.x == 0) db[ch] = part[0];
}

// dst[d1][d0][inner] = src[d0][d1][inner]: best_transpose_1023 (pydtnn/cython_modules/transpose_cython.pyx:125-141)
__global__ void __launch_bounds__(256) transpose_1023_f64_kernel(const double* __restrict__ src,
                                                                 double* __restrict__ dst, int d0, int d1, long inner,
                                                                 long total)
{
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long p = i % inner;
    const long r = i / inner;
    const int b = (int)(r % d0), a = (int)(r / d0);  // destination index (a in d1, b in d0)
    dst[i] = src[((long)b * d1 + a) * inner + p];
}

inline unsigned blocks_for(long total) { return (unsigned)((total + 255) / 256); }

int geom64(ConvGeom* g, int b, int c, int h, int w, int kh, int kw, int vpadding, int hpadding, int vstride,
           int hstride, int vdilation, int hdilation)
{
    return make_conv_geom(g, b, c, h, w, 1, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
}

}  // namespace

extern "C" {

size_t pydtnn_hip_dgemm_workspace_bytes(long m, long n, long k)
{
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    return dgemm_plan_bytes(plan_dgemm(m, n, k), m, n);
}

int pydtnn_hip_dgemm(int transa, int transb, long m, long n, long k, const double* a, long lda, const double* b,
                     long ldb, double* c, long ldc, const double* bias, int relu, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    if (!a || !b || !c || m <= 0 || n <= 0 || k <= 0) return PYDTNN_HIP_ERR_INVALID;
    const long lim = 1l << 31;
    if (m >= lim || n >= lim || k >= lim) return PYDTNN_HIP_ERR_UNSUPPORTED;
    if (lda < (transa ? m : k) || ldb < (transb ? k : n) || ldc < n) return PYDTNN_HIP_ERR_INVALID;
    // a thread's byte offsets inside a step's window of an operand (up to 128 rows) are 32-bit
    if (lda >= (1l << 22) || ldb >= (1l << 22)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    DgemmPlan p = plan_dgemm(m, n, k);
    const long tiles_m = (m + kBM - 1) / kBM, tiles_n = (n + kBN - 1) / kBN;
    const long tiles = tiles_m * tiles_n;
    if (tiles >= (1l << 31) || p.splits > 65535) return PYDTNN_HIP_ERR_UNSUPPORTED;
    // the tail launch is an optimisation: without the workspace for it the one grid of whole tiles runs
    if (p.tail > 0 && (!workspace || workspace_bytes < dgemm_plan_bytes(p, m, n))) p.tail = 0;
    Dgemm g;
    g.a = a; g.b = b; g.lda = lda; g.ldb = ldb; g.m = (int)m; g.n = (int)n; g.k = (int)k;
    g.transa = transa ? 1 : 0; g.transb = transb ? 1 : 0; g.chunk = p.chunk;
    g.tiles_m = (int)tiles_m; g.tile0 = 0; g.compact = 0;
    if (p.splits > 1) {
        if (!workspace || workspace_bytes < (size_t)p.splits * m * n * 8) return PYDTNN_HIP_ERR_WORKSPACE;
        g.c = static_cast<double*>(workspace); g.ldc = n; g.bias = nullptr; g.relu = 0;
    } else {
        g.c = c; g.ldc = ldc; g.bias = bias; g.relu = relu ? 1 : 0;
    }
    const hipStream_t st = convint::as_stream(stream);
    auto run = [&](const Dgemm& d, long count, int splits) {
        const dim3 grid((unsigned)count, (unsigned)splits);
        if (d.transa && d.transb) hipLaunchKernelGGL((dgemm_kernel<true, true>), grid, dim3(256), 0, st, d);
        else if (d.transa) hipLaunchKernelGGL((dgemm_kernel<true, false>), grid, dim3(256), 0, st, d);
        else if (d.transb) hipLaunchKernelGGL((dgemm_kernel<false, true>), grid, dim3(256), 0, st, d);
        else hipLaunchKernelGGL((dgemm_kernel<false, false>), grid, dim3(256), 0, st, d);
    };
    run(g, tiles - p.tail, p.splits);
    HIP_RETURN_IF_LAUNCH_FAILED();
    if (p.splits > 1) {
        hipLaunchKernelGGL(dgemm_reduce_kernel, dim3(blocks_for(m * n)), dim3(256), 0, st,
                           static_cast<const double*>(workspace), c, ldc, m, (int)n, p.splits, bias, relu ? 1 : 0);
        HIP_RETURN_IF_LAUNCH_FAILED();
    }
    if (p.tail > 0) {
        Dgemm t = g;
        t.c = static_cast<double*>(workspace); t.bias = nullptr; t.relu = 0;
        t.tile0 = (int)(tiles - p.tail); t.compact = 1; t.chunk = p.tail_chunk;
        run(t, p.tail, p.tail_splits);
        HIP_RETURN_IF_LAUNCH_FAILED();
        hipLaunchKernelGGL(dgemm_tail_reduce_kernel, dim3((unsigned)(p.tail * (kBM * kBN / 256))), dim3(256), 0, st,
                           static_cast<const double*>(workspace), c, ldc, (int)m, (int)n, (int)tiles_m, t.tile0, p.tail,
                           p.tail_splits, bias, relu ? 1 : 0);
        HIP_RETURN_IF_LAUNCH_FAILED();
    }
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_im2col_nchw_f64(const double* x, double* cols, int b, int c, int h, int w, int kh, int kw, int vpadding,
                               int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom64(&g, b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.k * g.p;
    hipLaunchKernelGGL(im2col_nchw_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), x,
                       cols, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_col2im_nchw_f64(const double* cols, double* dx, int b, int c, int h, int w, int kh, int kw, int vpadding,
                               int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom64(&g, b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.h * g.w;
    hipLaunchKernelGGL(col2im_nchw_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), cols,
                       dx, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_im2row_nhwc_f64(const double* x, double* rows, int b, int h, int w, int c, int kh, int kw, int vpadding,
                               int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom64(&g, b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.k * g.p;
    hipLaunchKernelGGL(im2row_nhwc_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), x,
                       rows, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_row2im_nhwc_f64(const double* rows, double* dx, int b, int h, int w, int c, int kh, int kw, int vpadding,
                               int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom64(&g, b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    const long total = (long)g.n * g.c * g.h * g.w;
    hipLaunchKernelGGL(row2im_nhwc_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), rows,
                       dx, g, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_chan_eltwise_f64(const double* x, const double* residual, double* y, long total, long inner,
                                int channels, const double* bias, const double* bn_running_mean,
                                const double* bn_inv_std, const double* bn_gamma, const double* bn_beta, int relu,
                                void* stream)
{
    if (!x || !y || total < 0 || inner <= 0 || channels <= 0) return PYDTNN_HIP_ERR_INVALID;
    const int set = (bn_running_mean != nullptr) + (bn_inv_std != nullptr) + (bn_gamma != nullptr) + (bn_beta != nullptr);
    if (set != 0 && set != 4) return PYDTNN_HIP_ERR_INVALID;
    if (total == 0) return PYDTNN_HIP_OK;
    const ChanEpilogue64 e = {bias, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu ? 1 : 0};
    hipLaunchKernelGGL(chan_eltwise_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), x,
                       residual, y, total, inner, channels, e);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_relu_fwd_f64(const double* x, double* y, int8_t* mask, long total, void* stream)
{
    if (!x || !y || total < 0) return PYDTNN_HIP_ERR_INVALID;
    if (total == 0) return PYDTNN_HIP_OK;
    hipLaunchKernelGGL(relu_fwd_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), x, y,
                       mask, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_relu_bwd_f64(const double* dy, const int8_t* mask, double* dx, long total, void* stream)
{
    if (!dy || !mask || !dx || total < 0) return PYDTNN_HIP_ERR_INVALID;
    if (total == 0) return PYDTNN_HIP_OK;
    hipLaunchKernelGGL(relu_bwd_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), dy, mask,
                       dx, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_bias_grad_f64(const double* dy, double* db, long outer, int channels, long inner, void* stream)
{
    if (!dy || !db || outer <= 0 || channels <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    hipLaunchKernelGGL(bias_grad_f64_kernel, dim3((unsigned)channels), dim3(256), 0, convint::as_stream(stream), dy, db,
                       outer, channels, inner);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_transpose_1023_f64(const double* src, double* dst, int d0, int d1, long inner, void* stream)
{
    if (!src || !dst || d0 <= 0 || d1 <= 0 || inner <= 0) return PYDTNN_HIP_ERR_INVALID;
    const long total = (long)d0 * d1 * inner;
    hipLaunchKernelGGL(transpose_1023_f64_kernel, dim3(blocks_for(total)), dim3(256), 0, convint::as_stream(stream), src,
                       dst, d0, d1, inner, total);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

}  // extern "C"

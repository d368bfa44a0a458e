/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the conv-as-GEMM hot path.
 *
 * Plain-C restatement of the loop nests of PyDTNN's Cython CPU kernels.  It is
 * the checker for the HIP kernels and the timed "reference CPU backend" leg of
 * the benchmark; the product library never links or calls it.
 *
 * Every function keeps the reference's loop order, index arithmetic, bounds
 * predicates, accumulation order and OpenMP parallel axis, and cites the
 * reference lines it follows (paths relative to the PyDTNN source tree).
 *
 * Build: make -C oracle   (gcc -O3 -fopenmp -shared -fPIC)
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <float.h>

#define IDX4(a, b, c, d, B, C, D) ((((size_t)(a) * (B) + (b)) * (C) + (c)) * (D) + (d))

static inline int out_dim(int in, int pad, int dil, int k, int stride)
{
    /* pydtnn/cython_modules/im2col_nchw_cython.pyx:35-36 */
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

/* ---------------------------------------------------------------------------
 * im2col / col2im, NCHW
 * pydtnn/cython_modules/im2col_nchw_cython.pyx:104-124 (gather, fp32)
 * pydtnn/cython_modules/im2col_nchw_cython.pyx:224-244 (scatter-add, fp32)
 * row = c*kh*kw + i*kw + j ; col = n*hh*ww + y*ww + x ; parallel over c.
 * The caller passes cols zero-filled (np.zeros at :38) for im2col and x
 * zero-filled (:161) for col2im, exactly as the reference allocates them.
 * ------------------------------------------------------------------------- */
#define DEF_IM2COL_NCHW(NAME, T)                                                               \
void NAME(T *cols, const T *x, int n, int c, int h, int w, int kh, int kw,                     \
          int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation)  \
{                                                                                              \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                               \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                               \
    const size_t ncols = (size_t)n * hh * ww;                                                  \
    _Pragma("omp parallel for")                                                                \
    for (int cc = 0; cc < c; cc++)                                                             \
        for (int ii = 0; ii < kh; ii++)                                                        \
            for (int jj = 0; jj < kw; jj++) {                                                  \
                const size_t row = (size_t)cc * kh * kw + ii * kw + jj;                        \
                for (int nn = 0; nn < n; nn++)                                                 \
                    for (int xx = 0; xx < hh; xx++) {                                          \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;              \
                        if (0 <= x_x && x_x < h)                                               \
                            for (int yy = 0; yy < ww; yy++) {                                  \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;      \
                                if (0 <= x_y && x_y < w) {                                     \
                                    const size_t col = (size_t)nn * hh * ww + xx * ww + yy;    \
                                    cols[row * ncols + col] = x[IDX4(nn, cc, x_x, x_y, c, h, w)]; \
                                }                                                              \
                            }                                                                  \
                    }                                                                          \
            }                                                                                  \
}

#define DEF_COL2IM_NCHW(NAME, T)                                                               \
void NAME(const T *cols, T *x, int n, int c, int h, int w, int kh, int kw,                     \
          int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation)  \
{                                                                                              \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                               \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                               \
    const size_t ncols = (size_t)n * hh * ww;                                                  \
    _Pragma("omp parallel for")                                                                \
    for (int cc = 0; cc < c; cc++)                                                             \
        for (int ii = 0; ii < kh; ii++)                                                        \
            for (int jj = 0; jj < kw; jj++) {                                                  \
                const size_t row = (size_t)cc * kh * kw + ii * kw + jj;                        \
                for (int nn = 0; nn < n; nn++)                                                 \
                    for (int xx = 0; xx < hh; xx++) {                                          \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;              \
                        if (0 <= x_x && x_x < h)                                               \
                            for (int yy = 0; yy < ww; yy++) {                                  \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;      \
                                if (0 <= x_y && x_y < w) {                                     \
                                    const size_t col = (size_t)nn * hh * ww + xx * ww + yy;    \
                                    x[IDX4(nn, cc, x_x, x_y, c, h, w)] += cols[row * ncols + col]; \
                                }                                                              \
                            }                                                                  \
                    }                                                                          \
            }                                                                                  \
}

DEF_IM2COL_NCHW(oracle_im2col_nchw_f32, float)
DEF_IM2COL_NCHW(oracle_im2col_nchw_f64, double)
DEF_COL2IM_NCHW(oracle_col2im_nchw_f32, float)
DEF_COL2IM_NCHW(oracle_col2im_nchw_f64, double)

/* ---------------------------------------------------------------------------
 * im2row / row2im, NHWC
 * pydtnn/cython_modules/im2row_nhwc_cython.pyx:77-97 (gather, fp32)
 * pydtnn/cython_modules/im2row_nhwc_cython.pyx:174-194 (scatter-add, fp32)
 * row = n*hh*ww + y*ww + x ; col = c*kh*kw + i*kw + j (channel-major K also in
 * NHWC) ; parallel over n.
 * ------------------------------------------------------------------------- */
#define DEF_IM2ROW_NHWC(NAME, T)                                                               \
void NAME(T *rows, const T *x, int n, int h, int w, int c, int kh, int kw,                     \
          int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation)  \
{                                                                                              \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                               \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                               \
    const size_t nk = (size_t)c * kh * kw;                                                     \
    _Pragma("omp parallel for")                                                                \
    for (int nn = 0; nn < n; nn++)                                                             \
        for (int xx = 0; xx < hh; xx++)                                                        \
            for (int yy = 0; yy < ww; yy++) {                                                  \
                const size_t row = (size_t)nn * hh * ww + xx * ww + yy;                        \
                for (int cc = 0; cc < c; cc++)                                                 \
                    for (int ii = 0; ii < kh; ii++) {                                          \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;              \
                        if (0 <= x_x && x_x < h)                                               \
                            for (int jj = 0; jj < kw; jj++) {                                  \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;      \
                                if (0 <= x_y && x_y < w) {                                     \
                                    const size_t col = (size_t)cc * kh * kw + ii * kw + jj;    \
                                    rows[row * nk + col] = x[IDX4(nn, x_x, x_y, cc, h, w, c)]; \
                                }                                                              \
                            }                                                                  \
                    }                                                                          \
            }                                                                                  \
}

#define DEF_ROW2IM_NHWC(NAME, T)                                                               \
void NAME(const T *rows, T *x, int n, int h, int w, int c, int kh, int kw,                     \
          int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation)  \
{                                                                                              \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                               \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                               \
    const size_t nk = (size_t)c * kh * kw;                                                     \
    _Pragma("omp parallel for")                                                                \
    for (int nn = 0; nn < n; nn++)                                                             \
        for (int xx = 0; xx < hh; xx++)                                                        \
            for (int yy = 0; yy < ww; yy++) {                                                  \
                const size_t row = (size_t)nn * hh * ww + xx * ww + yy;                        \
                for (int cc = 0; cc < c; cc++)                                                 \
                    for (int ii = 0; ii < kh; ii++) {                                          \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;              \
                        if (0 <= x_x && x_x < h)                                               \
                            for (int jj = 0; jj < kw; jj++) {                                  \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;      \
                                if (0 <= x_y && x_y < w) {                                     \
                                    const size_t col = (size_t)cc * kh * kw + ii * kw + jj;    \
                                    x[IDX4(nn, x_x, x_y, cc, h, w, c)] += rows[row * nk + col]; \
                                }                                                              \
                            }                                                                  \
                    }                                                                          \
            }                                                                                  \
}

DEF_IM2ROW_NHWC(oracle_im2row_nhwc_f32, float)
DEF_IM2ROW_NHWC(oracle_im2row_nhwc_f64, double)
DEF_ROW2IM_NHWC(oracle_row2im_nhwc_f32, float)
DEF_ROW2IM_NHWC(oracle_row2im_nhwc_f64, double)

/* ---------------------------------------------------------------------------
 * Bias add on the 2-D GEMM result (in place).
 * pydtnn/cython_modules/add_nchw_cython.pyx:51-58  x[i,j] += b[i]
 * pydtnn/cython_modules/add_nhwc_cython.pyx:51-58  x[i,j] += b[j]
 * ------------------------------------------------------------------------- */
#define DEF_ADD(NAME, T, BIDX)                                                  \
void NAME(T *x, const T *b, long rows, long cols)                               \
{                                                                               \
    _Pragma("omp parallel for")                                                 \
    for (long i = 0; i < rows; i++)                                             \
        for (long j = 0; j < cols; j++)                                         \
            x[i * cols + j] += b[BIDX];                                         \
}
DEF_ADD(oracle_add_nchw_f32, float, i)
DEF_ADD(oracle_add_nchw_f64, double, i)
DEF_ADD(oracle_add_nhwc_f32, float, j)
DEF_ADD(oracle_add_nhwc_f64, double, j)

/* ---------------------------------------------------------------------------
 * (co, N, ho, wo) <-> (N, co, ho, wo): the "1023" permute.
 * pydtnn/cython_modules/transpose_cython.pyx:125-141 ; dst[d1,d0,d2,d3] = src[d0,d1,d2,d3]
 * ------------------------------------------------------------------------- */
#define DEF_T1023(NAME, T)                                                      \
void NAME(const T *src, T *dst, int d0, int d1, int d2, int d3)                 \
{                                                                               \
    const size_t inner = (size_t)d2 * d3;                                       \
    _Pragma("omp parallel for")                                                 \
    for (int a = 0; a < d0; a++)                                                \
        for (int b = 0; b < d1; b++)                                            \
            memcpy(dst + ((size_t)b * d0 + a) * inner,                          \
                   src + ((size_t)a * d1 + b) * inner, inner * sizeof(T));      \
}
DEF_T1023(oracle_transpose_1023_f32, float)
DEF_T1023(oracle_transpose_1023_f64, double)

/* ---------------------------------------------------------------------------
 * BatchNorm inference and BN+ReLU inference on a (rows, C) matrix, and the
 * NCHW 4-D form.  tmp and y are rounded separately, in this order:
 *     tmp = (x - mean[c]) * inv_std[c];  y = tmp * gamma[c] + beta[c]
 * pydtnn/cython_modules/bn_inference_cython.pyx:61-72 (2-D), :127-140 (NCHW)
 * pydtnn/cython_modules/bn_relu_inference_cython.pyx:59-70
 * The source states three separately rounded operations.  Whether the
 * reference's own build fuses tmp*gamma+beta into one FMA depends on its
 * compiler flags (-O3 -march=native, settings.py:85-93), so its result is only
 * defined to within one rounding of the last step; this oracle takes the
 * source literally (volatile temporaries stop gcc from contracting), and
 * comparisons against it allow that one-ulp slack.
 * ------------------------------------------------------------------------- */
#define DEF_BN2D(NAME, T, RELU)                                                          \
void NAME(const T *x, const T *mean, const T *inv_std, const T *gamma, const T *beta,    \
          T *y, long rows, long c)                                                       \
{                                                                                        \
    _Pragma("omp parallel for schedule(static)")                                         \
    for (long i = 0; i < rows; i++)                                                      \
        for (long j = 0; j < c; j++) {                                                   \
            volatile T tmp = (x[i * c + j] - mean[j]) * inv_std[j];                      \
            volatile T prod = tmp * gamma[j];                                            \
            T v = prod + beta[j];                                                        \
            if (RELU) v = v > (T)0 ? v : (T)0;                                           \
            y[i * c + j] = v;                                                            \
        }                                                                                \
}
DEF_BN2D(oracle_bn_inference_f32, float, 0)
DEF_BN2D(oracle_bn_inference_f64, double, 0)
DEF_BN2D(oracle_bn_relu_inference_f32, float, 1)
DEF_BN2D(oracle_bn_relu_inference_f64, double, 1)

#define DEF_BN_NCHW(NAME, T)                                                             \
void NAME(const T *x, const T *mean, const T *inv_std, const T *gamma, const T *beta,    \
          T *y, int n, int c, int h, int w)                                              \
{                                                                                        \
    const size_t hw = (size_t)h * w;                                                     \
    _Pragma("omp parallel for schedule(static)")                                         \
    for (int i = 0; i < n; i++)                                                          \
        for (int j = 0; j < c; j++)                                                      \
            for (size_t p = 0; p < hw; p++) {                                            \
                const size_t o = ((size_t)i * c + j) * hw + p;                           \
                volatile T tmp = (x[o] - mean[j]) * inv_std[j];                          \
                volatile T prod = tmp * gamma[j];                                        \
                y[o] = prod + beta[j];                                                   \
            }                                                                            \
}
DEF_BN_NCHW(oracle_bn_inference_nchw_f32, float)
DEF_BN_NCHW(oracle_bn_inference_nchw_f64, double)

/* ---------------------------------------------------------------------------
 * ReLU forward with int8 mask: strict x > 0.
 * pydtnn/cython_modules/relu_cython.pyx:52-59
 * ------------------------------------------------------------------------- */
#define DEF_RELU(NAME, T)                                                       \
void NAME(const T *x, T *y, int8_t *mask, long n)                               \
{                                                                               \
    _Pragma("omp parallel for")                                                 \
    for (long i = 0; i < n; i++) {                                              \
        if (x[i] > (T)0) { y[i] = x[i]; mask[i] = 1; }                          \
        else             { y[i] = (T)0; mask[i] = 0; }                          \
    }                                                                           \
}
DEF_RELU(oracle_relu_f32, float)
DEF_RELU(oracle_relu_f64, double)

/* ---------------------------------------------------------------------------
 * Residual add: acc += x.   pydtnn/cython_modules/eltw_sum_cython.pyx:25-59
 * ------------------------------------------------------------------------- */
#define DEF_ELTW(NAME, T)                                                       \
void NAME(T *acc, const T *x, long n)                                           \
{                                                                               \
    _Pragma("omp parallel for")                                                 \
    for (long i = 0; i < n; i++) acc[i] += x[i];                                \
}
DEF_ELTW(oracle_eltw_sum_f32, float)
DEF_ELTW(oracle_eltw_sum_f64, double)

/* ---------------------------------------------------------------------------
 * MaxPool2D NCHW forward / backward.
 * pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:86-110 : first maximum
 * wins (strict val > maxval), start value = lowest finite float, stored index
 * = ii*kw + jj.
 * pydtnn/cython_modules/max_pool_2d_nchw_cython.pyx:194-212 : the index is
 * decoded as ii = idx / kh, jj = idx % kw (as written in the reference; equal
 * to the encoding only for kh == kw).
 * ------------------------------------------------------------------------- */
#define DEF_MAX_POOL_NCHW(T, SFX, LOWEST)                                                            \
void oracle_max_pool_2d_fwd_nchw_##SFX(const T *x, T *y, int32_t *idx_max,                           \
                                     int n, int c, int h, int w, int kh, int kw,                     \
                                     int vpadding, int hpadding, int vstride, int hstride,           \
                                     int vdilation, int hdilation)                                   \
{                                                                                                    \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                     \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                     \
    _Pragma("omp parallel for")                                                                      \
    for (int nn = 0; nn < n; nn++)                                                                   \
        for (int cc = 0; cc < c; cc++)                                                               \
            for (int xx = 0; xx < hh; xx++)                                                          \
                for (int yy = 0; yy < ww; yy++) {                                                    \
                    T maxval = LOWEST;                                                               \
                    int idx_maxval = 0;                                                              \
                    for (int ii = 0; ii < kh; ii++) {                                                \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;                    \
                        if (0 <= x_x && x_x < h)                                                     \
                            for (int jj = 0; jj < kw; jj++) {                                        \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;            \
                                if (0 <= x_y && x_y < w) {                                           \
                                    const T val = x[IDX4(nn, cc, x_x, x_y, c, h, w)];                \
                                    if (val > maxval) { maxval = val; idx_maxval = ii * kw + jj; }   \
                                }                                                                    \
                            }                                                                        \
                    }                                                                                \
                    y[IDX4(nn, cc, xx, yy, c, hh, ww)] = maxval;                                     \
                    idx_max[IDX4(nn, cc, xx, yy, c, hh, ww)] = idx_maxval;                           \
                }                                                                                    \
}                                                                                                    \
                                                                                                     \
void oracle_max_pool_2d_bwd_nchw_##SFX(const T *dy, const int32_t *idx_max, T *dx,                   \
                                     int n, int c, int h, int w, int kh, int kw,                     \
                                     int vpadding, int hpadding, int vstride, int hstride,           \
                                     int vdilation, int hdilation)                                   \
{                                                                                                    \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                     \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                     \
    _Pragma("omp parallel for")                                                                      \
    for (int nn = 0; nn < n; nn++)                                                                   \
        for (int cc = 0; cc < c; cc++)                                                               \
            for (int xx = 0; xx < hh; xx++)                                                          \
                for (int yy = 0; yy < ww; yy++) {                                                    \
                    const int idx_maxval = idx_max[IDX4(nn, cc, xx, yy, c, hh, ww)];                 \
                    const int ii = idx_maxval / kh, jj = idx_maxval % kw;                            \
                    const int x_x = vstride * xx + vdilation * ii - vpadding;                        \
                    const int x_y = hstride * yy + hdilation * jj - hpadding;                        \
                    if (0 <= x_x && x_x < h && 0 <= x_y && x_y < w)                                  \
                        dx[IDX4(nn, cc, x_x, x_y, c, h, w)] += dy[IDX4(nn, cc, xx, yy, c, hh, ww)];  \
                }                                                                                    \
}
DEF_MAX_POOL_NCHW(float, f32, -FLT_MAX)
DEF_MAX_POOL_NCHW(double, f64, -DBL_MAX)

/* ---------------------------------------------------------------------------
 * MaxPool2D NHWC forward / backward.
 * pydtnn/cython_modules/max_pool_2d_nhwc_cython.pyx:86-110 and :194-212: the
 * same rules as the NCHW pair (first maximum, index ii*kw + jj, decoded as
 * ii = idx / kh, jj = idx % kw), loop order n, output row, output column, c.
 * ------------------------------------------------------------------------- */
#define IDX_NHWC(n_, y_, x_, c_, H, W, C) ((((long)(n_) * (H) + (y_)) * (W) + (x_)) * (C) + (c_))

#define DEF_MAX_POOL_NHWC(T, SFX, LOWEST)                                                                    \
                                                                                                             \
void oracle_max_pool_2d_fwd_nhwc_##SFX(const T *x, T *y, int32_t *idx_max,                                   \
                                     int n, int h, int w, int c, int kh, int kw,                             \
                                     int vpadding, int hpadding, int vstride, int hstride,                   \
                                     int vdilation, int hdilation)                                           \
{                                                                                                            \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                             \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                             \
    _Pragma("omp parallel for")                                                                              \
    for (int nn = 0; nn < n; nn++)                                                                           \
        for (int xx = 0; xx < hh; xx++)                                                                      \
            for (int yy = 0; yy < ww; yy++)                                                                  \
                for (int cc = 0; cc < c; cc++) {                                                             \
                    T maxval = LOWEST;                                                                       \
                    int idx_maxval = 0;                                                                      \
                    for (int ii = 0; ii < kh; ii++) {                                                        \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;                            \
                        if (0 <= x_x && x_x < h)                                                             \
                            for (int jj = 0; jj < kw; jj++) {                                                \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;                    \
                                if (0 <= x_y && x_y < w) {                                                   \
                                    const T val = x[IDX_NHWC(nn, x_x, x_y, cc, h, w, c)];                    \
                                    if (val > maxval) { maxval = val; idx_maxval = ii * kw + jj; }           \
                                }                                                                            \
                            }                                                                                \
                    }                                                                                        \
                    y[IDX_NHWC(nn, xx, yy, cc, hh, ww, c)] = maxval;                                         \
                    idx_max[IDX_NHWC(nn, xx, yy, cc, hh, ww, c)] = idx_maxval;                               \
                }                                                                                            \
}                                                                                                            \
                                                                                                             \
void oracle_max_pool_2d_bwd_nhwc_##SFX(const T *dy, const int32_t *idx_max, T *dx,                           \
                                     int n, int h, int w, int c, int kh, int kw,                             \
                                     int vpadding, int hpadding, int vstride, int hstride,                   \
                                     int vdilation, int hdilation)                                           \
{                                                                                                            \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                             \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                             \
    _Pragma("omp parallel for")                                                                              \
    for (int nn = 0; nn < n; nn++)                                                                           \
        for (int xx = 0; xx < hh; xx++)                                                                      \
            for (int yy = 0; yy < ww; yy++)                                                                  \
                for (int cc = 0; cc < c; cc++) {                                                             \
                    const int idx_maxval = idx_max[IDX_NHWC(nn, xx, yy, cc, hh, ww, c)];                     \
                    const int ii = idx_maxval / kh, jj = idx_maxval % kw;                                    \
                    const int x_x = vstride * xx + vdilation * ii - vpadding;                                \
                    const int x_y = hstride * yy + hdilation * jj - hpadding;                                \
                    if (0 <= x_x && x_x < h && 0 <= x_y && x_y < w)                                          \
                        dx[IDX_NHWC(nn, x_x, x_y, cc, h, w, c)] += dy[IDX_NHWC(nn, xx, yy, cc, hh, ww, c)];  \
                }                                                                                            \
}
DEF_MAX_POOL_NHWC(float, f32, -FLT_MAX)
DEF_MAX_POOL_NHWC(double, f64, -DBL_MAX)

/* ---------------------------------------------------------------------------
 * AveragePool2D forward / backward, both tensor formats.
 * pydtnn/cython_modules/average_pool_2d_nchw_cython.pyx:83-108 and :198-227,
 * average_pool_2d_nhwc_cython.pyx:83-108 and :198-227: the window's taps that
 * lie inside the image are summed in (ii, jj) order and divided by their
 * number (padding is not counted); backward adds dy / items to every such
 * tap, windows visited in ascending (xx, yy) order.
 * ------------------------------------------------------------------------- */
#define DEF_AVG_POOL(NAME, NHWC, T, SFX)                                                                        \
void NAME##_fwd_##SFX(const T *x, T *y, int n, int c, int h, int w, int kh, int kw,               \
                    int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation) \
{                                                                                                        \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                         \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                         \
    _Pragma("omp parallel for")                                                                          \
    for (int nn = 0; nn < n; nn++)                                                                       \
        for (int cc = 0; cc < c; cc++)                                                                   \
            for (int xx = 0; xx < hh; xx++)                                                              \
                for (int yy = 0; yy < ww; yy++) {                                                        \
                    T accum = 0;                                                                         \
                    int items = 0;                                                                       \
                    for (int ii = 0; ii < kh; ii++) {                                                    \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;                        \
                        if (0 <= x_x && x_x < h)                                                         \
                            for (int jj = 0; jj < kw; jj++) {                                            \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;                \
                                if (0 <= x_y && x_y < w) {                                               \
                                    accum = accum + (NHWC ? x[IDX4(nn, x_x, x_y, cc, h, w, c)]           \
                                                          : x[IDX4(nn, cc, x_x, x_y, c, h, w)]);         \
                                    items = items + 1;                                                   \
                                }                                                                        \
                            }                                                                            \
                    }                                                                                    \
                    y[NHWC ? IDX4(nn, xx, yy, cc, hh, ww, c) : IDX4(nn, cc, xx, yy, c, hh, ww)] =        \
                        accum / items;                                                                   \
                }                                                                                        \
}                                                                                                        \
void NAME##_bwd_##SFX(const T *dy, T *dx, int n, int c, int h, int w, int kh, int kw,             \
                    int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation) \
{                                                                                                        \
    const int hh = out_dim(h, vpadding, vdilation, kh, vstride);                                         \
    const int ww = out_dim(w, hpadding, hdilation, kw, hstride);                                         \
    _Pragma("omp parallel for")                                                                          \
    for (int nn = 0; nn < n; nn++)                                                                       \
        for (int cc = 0; cc < c; cc++)                                                                   \
            for (int xx = 0; xx < hh; xx++)                                                              \
                for (int yy = 0; yy < ww; yy++) {                                                        \
                    int items = 0;                                                                       \
                    for (int ii = 0; ii < kh; ii++) {                                                    \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;                        \
                        if (0 <= x_x && x_x < h)                                                         \
                            for (int jj = 0; jj < kw; jj++) {                                            \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;                \
                                if (0 <= x_y && x_y < w) items = items + 1;                              \
                            }                                                                            \
                    }                                                                                    \
                    const T avgval =                                                                     \
                        dy[NHWC ? IDX4(nn, xx, yy, cc, hh, ww, c) : IDX4(nn, cc, xx, yy, c, hh, ww)] / items; \
                    for (int ii = 0; ii < kh; ii++) {                                                    \
                        const int x_x = vstride * xx + vdilation * ii - vpadding;                        \
                        if (0 <= x_x && x_x < h)                                                         \
                            for (int jj = 0; jj < kw; jj++) {                                            \
                                const int x_y = hstride * yy + hdilation * jj - hpadding;                \
                                if (0 <= x_y && x_y < w)                                                 \
                                    dx[NHWC ? IDX4(nn, x_x, x_y, cc, h, w, c)                            \
                                            : IDX4(nn, cc, x_x, x_y, c, h, w)] += avgval;                \
                            }                                                                            \
                    }                                                                                    \
                }                                                                                        \
}
DEF_AVG_POOL(oracle_average_pool_2d_nchw, 0, float, f32)
DEF_AVG_POOL(oracle_average_pool_2d_nhwc, 1, float, f32)
DEF_AVG_POOL(oracle_average_pool_2d_nchw, 0, double, f64)
DEF_AVG_POOL(oracle_average_pool_2d_nhwc, 1, double, f64)

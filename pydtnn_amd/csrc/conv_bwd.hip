// Filter-gradient launches and the explicit (GEMM + col2im / row2im) input gradient.
#include "conv_internal.h"

namespace convint {

// ---------------------------------------------------------------- filter gradient
// cols / rows == nullptr: implicit (x gathered on the fly); otherwise the materialised x_cols / x_rows.
// With at most 64 filters the filter gradient is one tile wide and kh*kw*c long; where 256-long tiles would
// be padding for a tenth or more of their length (576 = 2.25 x 256 = 3 x 192) the implicit launches use
// 192-long tiles instead.
typedef Tile<192, 64, 2, 2> T192x64;
typedef Tile<64, 192, 2, 2> T64x192;

static bool dw_tile_192(const ConvGeom& g, int nhwc)
{
    const long m = nhwc ? g.k : g.kn, n = nhwc ? g.kn : g.k;
    if (g.kn > 64 || pick_tile(m, n) != (nhwc ? SEL_256x64 : SEL_64x256)) return false;
    return round_up(g.k, 192) * 10 <= round_up(g.k, 256) * 9;
}

// A filter matrix that 256x128 tiles cover without padding rows (NCHW: a multiple of 256 filters; NHWC: kh*kw*c a
// multiple of 256 and a multiple of 128 filters) and that is at least 1152 long: those tiles, two workgroups per
// CU, so the reduction is split for 512 of them.  The loaders' per-element vector and scalar instructions are
// spread over twice the MFMAs.
static bool dw_tile_big(const ConvGeom& g, int nhwc)
{
    if (g.k < 1152) return false;
    return nhwc ? g.k % 256 == 0 && g.kn % 128 == 0 : g.kn % 256 == 0;
}

// A multiple of 128 filters (that the 256x128 tile does not serve) and kh*kw*c a multiple of 192, at least 1152:
// tiles of 128 filters x 192, six MFMA blocks per wavefront, also two workgroups per CU (1152 is 6 times 192: no
// padding columns and a third fewer tiles than 9 times 128; measured +6.5 % there in both formats, but -13 % at
// 576 = 3 x 192, which therefore stays on the 128x128 tile).
typedef Tile<128, 192, 2, 2> T128x192;
typedef Tile<192, 128, 2, 2> T192x128;

static bool dw_tile_192x128(const ConvGeom& g, int nhwc)
{
    return !dw_tile_big(g, nhwc) && g.kn % 128 == 0 && g.k % 192 == 0 && g.k >= 1152;
}

SplitPlan plan_dw(const ConvGeom& g, int nhwc)
{
    if (dw_tile_192x128(g, nhwc))
        return plan_pixel_split((long)(g.kn / 128) * (g.k / 192), g.n, g.howo, (long)g.kn * g.k, 512);
    if (dw_tile_big(g, nhwc)) {
        const long tiles = nhwc ? (g.k / 256) * (g.kn / 128) : (g.kn / 256) * ((g.k + 127) / 128);
        return plan_pixel_split(tiles, g.n, g.howo, (long)g.kn * g.k, 512);
    }
    const long m = nhwc ? g.k : g.kn, n = nhwc ? g.kn : g.k;
    const TileSel sel = pick_tile(m, n);
    const long tiles = dw_tile_192(g, nhwc) ? (g.k + 191) / 192 : tiles_of(sel, m, n);
    return plan_pixel_split(tiles, g.n, g.howo, (long)g.kn * g.k);
}

// One implicit NCHW launch with tile T: partial sums of the split into the workspace.
// A(m = filter, k = (image, pixel)) = dy[image][filter][pixel]; B = the column matrix gathered from x.
template <class T>
static int dw_nchw_implicit(const ConvGeom& g, const SplitPlan& sp, const float* dy, const float* x, float* ws,
                            hipStream_t stream)
{
    const long dy_img = (long)g.kn * g.howo;
    if (!span_ok_k(T::BM, g.howo, sp.si.ips, dy_img)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    auto al = plain_k<T::BM, true>(dy, g.p * g.kn, g.howo, dy_img, g.kn, g.howo);
    al.fd_seg = group_div(g.howo, sp.si.ips);
    Im2colNchwK<T::BN> bl;
    bl.x = x; bl.g = g;
    bl.g.fd_howo = group_div(g.howo, sp.si.ips);
    const EpiPlain ep = epi_plain(ws, g.k, (long)g.kn * g.k, g.kn, g.k, no_epilogue(), no_masks(), sp.splits);
    return launch<T>(al, bl, ep, g.kn, g.k, sp.si, sp.splits, stream);
}

// The NHWC twin: A(m = (i,j,c), k = (image, pixel)) gathered from x; B(k, n = filter) = dy[(image*howo + pixel)*kn + n].
template <class T>
static int dw_nhwc_implicit(const ConvGeom& g, const SplitPlan& sp, const float* dy, const float* x, float* ws,
                            hipStream_t stream)
{
    auto bl = plain_mn<T::BN>(dy, g.p * g.kn, g.kn, (long)g.howo * g.kn, g.kn);
    Im2rowNhwcMN<T::BM> al;
    al.x = x; al.g = g;
    al.g.fd_howo = group_div(g.howo, sp.si.ips);
    const EpiPlain ep = epi_plain(ws, g.kn, (long)g.kn * g.k, g.k, g.kn, no_epilogue(), no_masks(), sp.splits);
    return launch<T>(al, bl, ep, g.k, g.kn, sp.si, sp.splits, stream);
}

int conv_dw_nchw(const ConvGeom& g, const float* dy, const float* x, const float* cols, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate)
{
    const SplitPlan sp = plan_dw(g, 0);
    const long out_elems = (long)g.kn * g.k;
    if (!ws || ws_bytes < (size_t)sp.splits * out_elems * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    const TileSel sel = pick_tile(g.kn, g.k);
    const bool special_tile = dw_tile_big(g, 0) || dw_tile_192x128(g, 0) || dw_tile_192(g, 0);
    int rc = PYDTNN_HIP_OK;
    // The equal chunks of the split leave part of the chip idle when tiles * chunks misses what it holds
    // (144 tiles x 5 chunks = 720 of 768).  With all images in one reduction group the balanced launch deals
    // the reduction units of all tiles evenly instead and writes dw directly.  Measured: 5 % faster at 144
    // tiles (512 filters, 28x28), 3 % slower at 72, hence the tile bound.
    const long tiles = tiles_of(sel, g.kn, g.k);
    const long split_blocks = (long)sp.splits * tiles;
    if (!cols && !accumulate && !special_tile && sp.si.ips == g.n && tiles >= 96 &&
        split_blocks * 100 < kTargetBlocks * 97 && ws_bytes >= kBalanceBytes && g.p < (1l << 31)) {
        WITH_TILE(sel, {
            const long dy_img = (long)g.kn * g.howo;
            if (!span_ok_k(T::BM, g.howo, g.n, dy_img)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            auto al = plain_k<T::BM, true>(dy, g.p * g.kn, g.howo, dy_img, g.kn, g.howo);
            al.fd_seg = group_div(g.howo, g.n);
            Im2colNchwK<T::BN> bl;
            bl.x = x; bl.g = g;
            bl.g.fd_howo = group_div(g.howo, g.n);
            rc = launch_balanced<T>(al, bl, epi_plain(dw, g.k, 0, g.kn, g.k, no_epilogue()), g.kn, g.k, (int)g.p, ws,
                                    ws_bytes, stream, true);
        })
        if (rc != kNotBalanced) return rc;
        rc = PYDTNN_HIP_OK;
    }
    if (cols) {
        WITH_TILE(sel, {
            // A as in the implicit form; B(k = (image, pixel), n = row of cols) = cols[n][image*howo + pixel]
            const long dy_img = (long)g.kn * g.howo;
            if (!span_ok_k(T::BM, g.howo, sp.si.ips, dy_img) || !span_ok_k(T::BN, g.p, sp.si.ips, g.howo))
                return PYDTNN_HIP_ERR_UNSUPPORTED;
            auto al = plain_k<T::BM, true>(dy, g.p * g.kn, g.howo, dy_img, g.kn, g.howo);
            al.fd_seg = group_div(g.howo, sp.si.ips);
            auto bl = plain_k<T::BN, true>(cols, (long)g.k * g.p, g.p, g.howo, g.k, g.howo);
            bl.fd_seg = group_div(g.howo, sp.si.ips);
            rc = launch<T>(al, bl, epi_plain(ws, g.k, out_elems, g.kn, g.k, no_epilogue(), no_masks(), sp.splits), g.kn,
                           g.k, sp.si, sp.splits, stream);
        })
    } else if (dw_tile_big(g, 0)) {
        rc = dw_nchw_implicit<T256x128>(g, sp, dy, x, ws, stream);
    } else if (dw_tile_192x128(g, 0)) {
        rc = dw_nchw_implicit<T128x192>(g, sp, dy, x, ws, stream);
    } else if (dw_tile_192(g, 0)) {
        rc = dw_nchw_implicit<T64x192>(g, sp, dy, x, ws, stream);
    } else {
        WITH_TILE(sel, { rc = dw_nchw_implicit<T>(g, sp, dy, x, ws, stream); })
    }
    if (rc != PYDTNN_HIP_OK) return rc;
    return launch_splitk_reduce(ws, dw, g.kn, g.k, out_elems, sp.splits, 0, 0, no_epilogue(), accumulate, stream);
}

int conv_dw_nhwc(const ConvGeom& g, const float* dy, const float* x, const float* rows, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate)
{
    const SplitPlan sp = plan_dw(g, 1);
    const long out_elems = (long)g.kn * g.k;
    if (!ws || ws_bytes < (size_t)sp.splits * out_elems * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    const TileSel sel = pick_tile(g.k, g.kn);
    int rc = PYDTNN_HIP_OK;
    if (rows) {
        WITH_TILE(sel, {
            // A(m = column of rows, k) = rows[(image*howo + pixel)*K + m]; B as in the implicit form
            auto al = plain_mn<T::BM>(rows, g.p * g.k, g.k, (long)g.howo * g.k, g.k);
            auto bl = plain_mn<T::BN>(dy, g.p * g.kn, g.kn, (long)g.howo * g.kn, g.kn);
            rc = launch<T>(al, bl, epi_plain(ws, g.kn, out_elems, g.k, g.kn, no_epilogue(), no_masks(), sp.splits), g.k,
                           g.kn, sp.si, sp.splits, stream);
        })
    } else if (dw_tile_big(g, 1)) {
        rc = dw_nhwc_implicit<T256x128>(g, sp, dy, x, ws, stream);
    } else if (dw_tile_192x128(g, 1)) {
        rc = dw_nhwc_implicit<T192x128>(g, sp, dy, x, ws, stream);
    } else if (dw_tile_192(g, 1)) {
        rc = dw_nhwc_implicit<T192x64>(g, sp, dy, x, ws, stream);
    } else {
        WITH_TILE(sel, { rc = dw_nhwc_implicit<T>(g, sp, dy, x, ws, stream); })
    }
    if (rc != PYDTNN_HIP_OK) return rc;
    // implicit rows come out in (i, j, c) order; materialised x_rows already has the (c, i, j) order
    const int perm_c = rows ? 0 : g.c;
    return launch_splitk_reduce(ws, dw, g.k, g.kn, out_elems, sp.splits, perm_c, g.khw, no_epilogue(), accumulate,
                                stream);
}

// `gate` (optional, shaped like dx): dx is stored as gate ? dx : 0; after the scatter-add kernels this is
// one more pass over dx.
int conv_dx_i2c(const ConvGeom& g, int nhwc, const float* w, const float* dy, float* dx, float* ws, size_t ws_bytes,
                hipStream_t stream, const int8_t* gate)
{
    const size_t need = (size_t)g.k * g.p * 4;
    if (!ws || ws_bytes < need) return PYDTNN_HIP_ERR_WORKSPACE;
    if ((long)g.k * g.p >= (1l << 33)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    // what lies behind the product balances the GEMM's launch
    const size_t product = i2c_product_bytes(g);
    float* balance = ws_bytes >= product + kBalanceBytes ? ws + product / 4 : nullptr;
    const size_t balance_bytes = balance ? ws_bytes - product : 0;
    int rc = PYDTNN_HIP_OK;
    if (!nhwc) {
        // res(K x P) = W^T (A(m = k, kk = filter) = w[kk*K + m]) * dy_cols (dy seen as a 1x1 im2col)
        ConvGeom g1;
        rc = make_conv_geom(&g1, g.n, g.kn, g.ho, g.wo, 1, 1, 1, 0, 0, 1, 1, 1, 1);
        if (rc != PYDTNN_HIP_OK) return rc;
        const TileSel sel = pick_tile_fwd(g.k, g.p, g.kn);
        if (sel == SEL_256x128) {
            typedef T256x128 T;
            Im2colNchwMN<T::BN> bl;
            bl.x = dy; bl.g = g1;
            rc = launch_balanced<T>(plain_mn<T::BM>(w, (long)g.kn * g.k, g.k, 0, g.k), bl,
                                    epi_plain(ws, g.p, 0, g.k, g.p, no_epilogue()), g.k, g.p, g.kn, balance,
                                    balance_bytes, stream);
        } else {
            WITH_TILE(sel, {
                auto al = plain_mn<T::BM>(w, (long)g.kn * g.k, g.k, 0, g.k);
                Im2colNchwMN<T::BN> bl;
                bl.x = dy; bl.g = g1;
                rc = launch_balanced<T>(al, bl, epi_plain(ws, g.p, 0, g.k, g.p, no_epilogue()), g.k, g.p, g.kn, balance,
                                        balance_bytes, stream);
            })
        }
        if (rc != PYDTNN_HIP_OK) return rc;
        rc = launch_col2im_nchw(ws, dx, g, stream);
        if (rc != PYDTNN_HIP_OK || !gate) return rc;
        return launch_relu_bwd(dx, gate, dx, (long)g.n * g.c * g.h * g.w, stream);
    }
    // res(P x K) = dy_rows (P x kn) * W_rows^T : B(kk = filter, n = k) = w[n*kn + kk]
    const TileSel sel = pick_tile(g.p, g.k);
    WITH_TILE(sel, {
        auto al = plain_k<T::BM, false>(dy, g.p * g.kn, g.kn, 0, g.p, 0);
        auto bl = plain_k<T::BN, false>(w, (long)g.k * g.kn, g.kn, 0, g.k, 0);
        rc = launch_balanced<T>(al, bl, epi_plain(ws, g.k, 0, g.p, g.k, no_epilogue()), g.p, g.k, g.kn, balance,
                                balance_bytes, stream);
    })
    if (rc != PYDTNN_HIP_OK) return rc;
    rc = launch_row2im_nhwc(ws, dx, g, stream);
    if (rc != PYDTNN_HIP_OK || !gate) return rc;
    return launch_relu_bwd(dx, gate, dx, (long)g.n * g.c * g.h * g.w, stream);
}


}  // namespace convint

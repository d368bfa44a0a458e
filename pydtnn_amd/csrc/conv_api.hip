// Device-pointer C ABI: argument checks, tile / split selection and kernel launches.
#include "../../include/pydtnn_hip.h"
#include "gemm_engine.h"

// launchers defined in gather_kernels.hip / eltwise_kernels.hip
int launch_im2col_nchw(const float*, float*, const ConvGeom&, hipStream_t);
int launch_col2im_nchw(const float*, float*, const ConvGeom&, hipStream_t);
int launch_im2row_nhwc(const float*, float*, const ConvGeom&, hipStream_t);
int launch_row2im_nhwc(const float*, float*, const ConvGeom&, hipStream_t);
int launch_chan_eltwise(const float*, const float*, float*, long, int, int, const ChanEpilogue&, hipStream_t);
int launch_relu_fwd(const float*, float*, int8_t*, long, hipStream_t);
int launch_relu_bwd(const float*, const int8_t*, float*, long, hipStream_t);
size_t bias_grad_workspace_floats(long, int);
int launch_bias_grad(const float*, float*, long, int, int, float*, hipStream_t);
int launch_splitk_reduce(const float*, float*, long, int, long, int, int, int, const ChanEpilogue&, int, hipStream_t);
int launch_flip_filter(const float*, float*, int, int, int, int, int, hipStream_t);
size_t bn_training_workspace_floats(int);
int launch_bn_training_fwd(const float*, float*, float*, float*, const float*, const float*, float*, float*, float, float,
                           float, long, int, int, float*, hipStream_t);
int launch_bn_training_bwd(const float*, const float*, const float*, const float*, float*, float*, float*, long, int,
                           int, float*, hipStream_t);
int launch_softmax_fwd(const float*, float*, int, int, hipStream_t);
int launch_softmax_bwd(const float*, const float*, float*, int, int, hipStream_t);
int launch_cce(const float*, const float*, float*, float*, float*, int, int, float, float, float, hipStream_t);
int launch_max_pool_fwd_nchw(const float*, float*, int32_t*, const ConvGeom&, hipStream_t);
int launch_max_pool_bwd_nchw(const float*, const int32_t*, float*, const ConvGeom&, hipStream_t, const int8_t* gate);
int launch_max_pool_fwd_nhwc(const float*, float*, int32_t*, const ConvGeom&, hipStream_t);
int launch_max_pool_bwd_nhwc(const float*, const int32_t*, float*, const ConvGeom&, hipStream_t, const int8_t* gate);
int launch_sgd_momentum(float*, const float*, float*, long, float, float, float, int, hipStream_t);

namespace {

using namespace gemm;

typedef Tile<128, 128, 2, 2> T128x128;
typedef Tile<64, 256, 1, 4> T64x256;
typedef Tile<256, 64, 4, 1> T256x64;
typedef Tile<64, 64, 2, 2> T64x64;

enum TileSel { SEL_128x128, SEL_64x256, SEL_256x64, SEL_64x64, SEL_COUNT };

struct TileShape {
    long bm, bn;
    double efficiency;  // matrix-core rate of the shape relative to 128x128 (fewer MFMAs per load and barrier)
};
constexpr TileShape kTileShapes[SEL_COUNT] = {{128, 128, 1.0}, {64, 256, 0.93}, {256, 64, 0.93}, {64, 64, 0.6}};

inline long tiles_of(TileSel sel, long m, long n)
{
    const TileShape& t = kTileShapes[sel];
    return ((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn);
}

// The shape that computes the fewest padded products, weighted by what the shape achieves.  A
// reduction of a step or two is all set-up (per-row tap masks, prologue): then the small tile, which
// has a quarter of the rows per thread and fills the chip with more workgroups, unless the
// problem already makes plenty of large ones.
inline TileSel pick_tile(long m, long n, long k = 1l << 30)
{
    if (k <= 2 * BK && tiles_of(SEL_128x128, m, n) < 2048) return SEL_64x64;
    TileSel best = SEL_128x128;
    double best_cost = 0.0;
    for (int s = 0; s < SEL_COUNT; ++s) {
        const TileShape& t = kTileShapes[s];
        const double cost = (double)tiles_of((TileSel)s, m, n) * (double)(t.bm * t.bn) / t.efficiency;
        if (s == 0 || cost < best_cost) { best = (TileSel)s; best_cost = cost; }
    }
    return best;
}

#define WITH_TILE(sel, ...)                                                 \
    switch (sel) {                                                          \
        case SEL_64x256: { typedef T64x256 T; __VA_ARGS__; } break;         \
        case SEL_256x64: { typedef T256x64 T; __VA_ARGS__; } break;         \
        case SEL_64x64: { typedef T64x64 T; __VA_ARGS__; } break;           \
        default: { typedef T128x128 T; __VA_ARGS__; } break;                \
    }

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline long round_up(long v, long m) { return (v + m - 1) / m * m; }

// Target number of workgroups for a launch that has to be split along the reduction axis: what the
// chip holds at once (three per CU on a 256-CU part).  A few more would run as a second, nearly
// empty round, so the split rounds down.
constexpr long kTargetBlocks = 768;
constexpr long kMinChunk = 256;
constexpr size_t kMaxPartialBytes = (size_t)768 << 20;

struct SplitPlan {
    SplitInfo si;
    int splits;
};

// Reduction over `images` segments of `seg` elements (pixels of one image): equal chunks of the whole
// run of images where the index arithmetic allows it, else groups of whole images.
SplitPlan plan_pixel_split(long tiles, int images, int seg, long out_elems)
{
    const long total = (long)images * seg;
    long want = tiles >= kTargetBlocks ? 1 : kTargetBlocks / tiles;
    const long max_by_ws = (long)(kMaxPartialBytes / ((size_t)out_elems * 4));
    if (want > max_by_ws) want = max_by_ws < 1 ? 1 : max_by_ws;
    long chunk = round_up((total + want - 1) / want, BK);
    if (chunk < kMinChunk) chunk = kMinChunk;
    SplitPlan p;
    // A group of several images finds the image of a reduction index with a multiply-high division by
    // seg, exact while (ips*seg + 256) * seg < 2^32; a group of one image needs no division
    // (group_div below).
    const long ips_cap = (((1l << 32) - 1) / seg - 256) / seg;
    if (images <= ips_cap) {
        const int cpg = (int)((total + chunk - 1) / chunk);
        p.si = make_split(seg, images, images, cpg, (int)chunk);
        p.splits = cpg;
    } else if (chunk >= seg && ips_cap >= 2) {
        long ips = chunk / seg;
        if (ips > images) ips = images;
        if (ips > ips_cap) ips = ips_cap;
        p.si = make_split(seg, images, (int)ips, 1, (int)(ips * seg));
        p.splits = (int)((images + ips - 1) / ips);
    } else {
        if (chunk > seg) chunk = seg;
        int cpg = (int)((seg + chunk - 1) / chunk);
        chunk = round_up((seg + cpg - 1) / cpg, BK);
        cpg = (int)((seg + chunk - 1) / chunk);
        p.si = make_split(seg, images, 1, cpg, (int)chunk);
        p.splits = images * cpg;
    }
    return p;
}

// Divider that maps a reduction index of a group to its image: a real one for groups of several
// images, "always image 0" for groups of one (exact for any image size).
inline FastDiv group_div(int seg, int ips)
{
    if (ips > 1) return make_fastdiv((uint32_t)seg);
    FastDiv f = {0u, (uint32_t)seg, 0u};
    return f;
}

// Plain GEMM: one segment of length k.
SplitPlan plan_plain_split(long tiles, long k, long out_elems)
{
    SplitPlan p;
    long want = tiles >= 256 ? 1 : (kTargetBlocks + tiles - 1) / tiles;
    const long max_by_ws = (long)(kMaxPartialBytes / ((size_t)out_elems * 4));
    if (want > max_by_ws) want = max_by_ws < 1 ? 1 : max_by_ws;
    long chunk = round_up((k + want - 1) / want, BK);
    if (chunk < kMinChunk) chunk = kMinChunk;
    if (chunk > k) chunk = k;
    const int splits = (int)((k + chunk - 1) / chunk);
    p.si = make_split((int)k, 1, 1, splits, (int)chunk);
    p.splits = splits;
    return p;
}

inline ChanEpilogue make_chan(const float* bias, const float* mean, const float* inv_std, const float* gamma,
                              const float* beta, int relu)
{
    ChanEpilogue e = {bias, mean, inv_std, gamma, beta, relu};
    return e;
}

inline bool bn_args_consistent(const float* mean, const float* inv_std, const float* gamma, const float* beta)
{
    const int set = (mean != nullptr) + (inv_std != nullptr) + (gamma != nullptr) + (beta != nullptr);
    return set == 0 || set == 4;
}

template <int BMN, bool SEG>
inline PlainK<BMN, SEG> plain_k(const float* base, long total, long ld, long image_stride, long extent, int seg_len)
{
    PlainK<BMN, SEG> l;
    l.base = base; l.total = total; l.ld = ld; l.image_stride = image_stride; l.extent = (int)extent;
    l.seg_len = seg_len; l.fd_seg = make_fastdiv((uint32_t)(seg_len > 0 ? seg_len : 1));
    return l;
}

template <int BMN>
inline PlainMN<BMN> plain_mn(const float* base, long total, long ld, long image_stride, long extent)
{
    PlainMN<BMN> l;
    l.base = base; l.total = total; l.ld = ld; l.image_stride = image_stride; l.extent = (int)extent;
    return l;
}

// Buffer descriptors span less than 2 GiB: a K-major operand needs its tile rows (plus the images of
// one reduction group) inside that span, an MN-major operand one step of BK rows.
inline bool span_ok_k(long tile_rows, long ld, long group_images, long image_stride)
{
    return (tile_rows * ld + group_images * image_stride) * 4 < kMaxSpanBytes;
}
inline bool span_ok_mn(long ld) { return (long)BK * ld * 4 < kMaxSpanBytes; }

template <int MASKS = kNoMasks>
inline EpiPlainT<MASKS> epi_plain(float* out, long ldc, long split_stride, long m, long n, const ChanEpilogue& chan,
                                  const ElemMasks& masks = no_masks(), int splits = 1)
{
    EpiPlainT<MASKS> e;
    e.out = out; e.ldc = ldc; e.split_stride = split_stride; e.m_extent = (int)m; e.n_extent = (int)n; e.chan = chan;
    e.masks = masks;
    // the branch-free tile store addresses the destination with 32-bit byte offsets
    const long span = (long)(splits - 1) * split_stride + (m - 1) * ldc + n;
    e.span = span < (1l << 29) && ldc < (1l << 24) ? span : 0;
    return e;
}

template <int MASKS = kNoMasks>
inline EpiNchwT<MASKS> epi_nchw(float* out, int channels, int howo, long p, const ChanEpilogue& chan,
                                const ElemMasks& masks = no_masks())
{
    EpiNchwT<MASKS> e;
    e.out = out; e.m_extent = channels; e.howo = howo; e.p = p; e.chan = chan; e.masks = masks;
    return e;
}

// at most one of the two is ever set: the forward writes a ReLU mask, dX reads a gate
inline int mask_kind(const ElemMasks& m) { return m.gate ? kGate : m.relu_mask ? kReluMask : kNoMasks; }

// ---------------------------------------------------------------- forward (implicit)
// The padding test works on tap masks of 31 usable bits: one word over i*kw + j when kh*kw <= 31,
// otherwise one word per axis.
inline bool taps_supported(const ConvGeom& g) { return g.kh <= 31 && g.kw <= 31; }
inline bool taps_wide(const ConvGeom& g) { return g.khw > 31; }

// Workspace of the balanced launch (gemm::launch_balanced): two accumulator tiles per resident
// workgroup, sized for the most this part can hold (4 per CU on 256 CUs) so that the query needs no device.
constexpr int kMaxResident = 1024;
constexpr size_t kBalanceBytes = (size_t)2 * kMaxResident * 128 * 128 * 4;

template <bool WIDE>
int conv_fwd_nchw_t(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                    size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    const TileSel sel = pick_tile(g.kn, g.p, g.k);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        if (!span_ok_k(T::BM, g.k, 0, 0)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        auto al = plain_k<T::BM, false>(w, (long)g.kn * g.k, g.k, 0, g.kn, 0);
        Im2colNchwMN<T::BN, WIDE> bl;
        bl.x = x; bl.g = g;
        switch (mask_kind(masks)) {
        case kGate:
            rc = launch_balanced<T>(al, bl, epi_nchw<kGate>(y, g.kn, g.howo, g.p, chan, masks), g.kn, g.p, g.k, ws,
                                    ws_bytes, stream);
            break;
        case kReluMask:
            rc = launch_balanced<T>(al, bl, epi_nchw<kReluMask>(y, g.kn, g.howo, g.p, chan, masks), g.kn, g.p, g.k, ws,
                                    ws_bytes, stream);
            break;
        default:
            rc = launch_balanced<T>(al, bl, epi_nchw(y, g.kn, g.howo, g.p, chan), g.kn, g.p, g.k, ws, ws_bytes, stream);
        }
    })
    return rc;
}

// `ws` is optional: without it (or with less than kBalanceBytes) the launch is a plain grid of tiles.
int conv_fwd_nchw(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks = no_masks())
{
    if (!taps_supported(g)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    return taps_wide(g) ? conv_fwd_nchw_t<true>(g, w, x, y, chan, ws, ws_bytes, stream, masks)
                        : conv_fwd_nchw_t<false>(g, w, x, y, chan, ws, ws_bytes, stream, masks);
}

template <bool WIDE>
int conv_fwd_nhwc_t(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                    size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    const TileSel sel = pick_tile(g.p, g.kn, g.k);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        Im2rowNhwcK<T::BM, WIDE> al;
        al.x = x; al.g = g;
        FilterNhwcMN<T::BN> bl;
        bl.w = w; bl.g = g;
        switch (mask_kind(masks)) {
        case kGate:
            rc = launch_balanced<T>(al, bl, epi_plain<kGate>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn, g.k, ws,
                                    ws_bytes, stream);
            break;
        case kReluMask:
            rc = launch_balanced<T>(al, bl, epi_plain<kReluMask>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn, g.k,
                                    ws, ws_bytes, stream);
            break;
        default:
            rc = launch_balanced<T>(al, bl, epi_plain(y, g.kn, 0, g.p, g.kn, chan), g.p, g.kn, g.k, ws, ws_bytes,
                                    stream);
        }
    })
    return rc;
}

// A 1x1 filter at stride 1 without padding makes x itself the (P x C) row matrix and the filter the
// (C x kn) matrix: a plain GEMM, whose loaders carry no per-pixel offsets or tap masks.
inline bool pointwise_nhwc(const ConvGeom& g)
{
    return g.khw == 1 && g.vstride == 1 && g.hstride == 1 && g.vpadding == 0 && g.hpadding == 0;
}

int conv_fwd_nhwc_pointwise(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                            float* ws, size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    const TileSel sel = pick_tile(g.p, g.kn, g.k);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        if (!span_ok_k(T::BM, g.c, 0, 0) || !span_ok_mn(g.kn)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        auto al = plain_k<T::BM, false>(x, g.p * g.c, g.c, 0, g.p, 0);
        auto bl = plain_mn<T::BN>(w, (long)g.c * g.kn, g.kn, 0, g.kn);
        switch (mask_kind(masks)) {
        case kGate:
            rc = launch_balanced<T>(al, bl, epi_plain<kGate>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn, g.k, ws,
                                    ws_bytes, stream);
            break;
        case kReluMask:
            rc = launch_balanced<T>(al, bl, epi_plain<kReluMask>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn, g.k,
                                    ws, ws_bytes, stream);
            break;
        default:
            rc = launch_balanced<T>(al, bl, epi_plain(y, g.kn, 0, g.p, g.kn, chan), g.p, g.kn, g.k, ws, ws_bytes,
                                    stream);
        }
    })
    return rc;
}

int conv_fwd_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks = no_masks())
{
    if (pointwise_nhwc(g)) return conv_fwd_nhwc_pointwise(g, w, x, y, chan, ws, ws_bytes, stream, masks);
    if (!taps_supported(g)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    return taps_wide(g) ? conv_fwd_nhwc_t<true>(g, w, x, y, chan, ws, ws_bytes, stream, masks)
                        : conv_fwd_nhwc_t<false>(g, w, x, y, chan, ws, ws_bytes, stream, masks);
}

// ---------------------------------------------------------------- filter gradient
// mat == nullptr: implicit (x gathered on the fly); otherwise the materialised x_cols / x_rows.
SplitPlan plan_dw(const ConvGeom& g, int nhwc)
{
    const long m = nhwc ? g.k : g.kn, n = nhwc ? g.kn : g.k;
    const TileSel sel = pick_tile(m, n);
    return plan_pixel_split(tiles_of(sel, m, n), g.n, g.howo, (long)g.kn * g.k);
}

int conv_dw_nchw(const ConvGeom& g, const float* dy, const float* x, const float* cols, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate = 0)
{
    const SplitPlan sp = plan_dw(g, 0);
    const long out_elems = (long)g.kn * g.k;
    if (!ws || ws_bytes < (size_t)sp.splits * out_elems * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    const TileSel sel = pick_tile(g.kn, g.k);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        // A(m = filter, k = (image, pixel)) = dy[image][filter][pixel]
        const long dy_img = (long)g.kn * g.howo;
        if (!span_ok_k(T::BM, g.howo, sp.si.ips, dy_img)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        auto al = plain_k<T::BM, true>(dy, g.p * g.kn, g.howo, dy_img, g.kn, g.howo);
        al.fd_seg = group_div(g.howo, sp.si.ips);
        const EpiPlain ep = epi_plain(ws, g.k, out_elems, g.kn, g.k, no_epilogue(), no_masks(), sp.splits);
        if (cols) {
            // B(k = (image, pixel), n = row of cols) = cols[n][image*howo + pixel]
            if (!span_ok_k(T::BN, g.p, sp.si.ips, g.howo)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            auto bl = plain_k<T::BN, true>(cols, (long)g.k * g.p, g.p, g.howo, g.k, g.howo);
            bl.fd_seg = group_div(g.howo, sp.si.ips);
            rc = launch<T>(al, bl, ep, g.kn, g.k, sp.si, sp.splits, stream);
        } else {
            Im2colNchwK<T::BN> bl;
            bl.x = x; bl.g = g;
            bl.g.fd_howo = group_div(g.howo, sp.si.ips);
            rc = launch<T>(al, bl, ep, g.kn, g.k, sp.si, sp.splits, stream);
        }
    })
    if (rc != PYDTNN_HIP_OK) return rc;
    return launch_splitk_reduce(ws, dw, g.kn, g.k, out_elems, sp.splits, 0, 0, no_epilogue(), accumulate, stream);
}

int conv_dw_nhwc(const ConvGeom& g, const float* dy, const float* x, const float* rows, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate = 0)
{
    const SplitPlan sp = plan_dw(g, 1);
    const long out_elems = (long)g.kn * g.k;
    if (!ws || ws_bytes < (size_t)sp.splits * out_elems * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    const TileSel sel = pick_tile(g.k, g.kn);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        // B(k = (image, pixel), n = filter) = dy[(image*howo + pixel)*kn + n]
        auto bl = plain_mn<T::BN>(dy, g.p * g.kn, g.kn, (long)g.howo * g.kn, g.kn);
        const EpiPlain ep = epi_plain(ws, g.kn, out_elems, g.k, g.kn, no_epilogue(), no_masks(), sp.splits);
        if (rows) {
            // A(m = column of rows, k) = rows[(image*howo + pixel)*K + m]
            auto al = plain_mn<T::BM>(rows, g.p * g.k, g.k, (long)g.howo * g.k, g.k);
            rc = launch<T>(al, bl, ep, g.k, g.kn, sp.si, sp.splits, stream);
        } else {
            Im2rowNhwcMN<T::BM> al;
            al.x = x; al.g = g;
            al.g.fd_howo = group_div(g.howo, sp.si.ips);
            rc = launch<T>(al, bl, ep, g.k, g.kn, sp.si, sp.splits, stream);
        }
    })
    if (rc != PYDTNN_HIP_OK) return rc;
    // implicit rows come out in (i, j, c) order; materialised x_rows already has the (c, i, j) order
    const int perm_c = rows ? 0 : g.c;
    return launch_splitk_reduce(ws, dw, g.k, g.kn, out_elems, sp.splits, perm_c, g.khw, no_epilogue(), accumulate,
                                stream);
}

// ---------------------------------------------------------------- input gradient
// Stride 1: dx = forward convolution of dy with the flipped, channel-swapped filter and padding
// dilation*(k-1) - padding.  Otherwise: the reference's own route, W^T dy then col2im / row2im.
inline bool dx_as_forward(const ConvGeom& g)
{
    return g.vstride == 1 && g.hstride == 1 && g.vdilation * (g.kh - 1) >= g.vpadding &&
           g.hdilation * (g.kw - 1) >= g.hpadding;
}

// `gate` (optional, shaped like dx): dx is stored as gate ? dx : 0; after the scatter-add kernels this is
// one more pass over dx.
int conv_dx_i2c(const ConvGeom& g, int nhwc, const float* w, const float* dy, float* dx, float* ws, size_t ws_bytes,
                hipStream_t stream, const int8_t* gate = nullptr)
{
    const size_t need = (size_t)g.k * g.p * 4;
    if (!ws || ws_bytes < need) return PYDTNN_HIP_ERR_WORKSPACE;
    if ((long)g.k * g.p >= (1l << 33)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    int rc = PYDTNN_HIP_OK;
    if (!nhwc) {
        // res(K x P) = W^T (A(m = k, kk = filter) = w[kk*K + m]) * dy_cols (dy seen as a 1x1 im2col)
        ConvGeom g1;
        rc = make_conv_geom(&g1, g.n, g.kn, g.ho, g.wo, 1, 1, 1, 0, 0, 1, 1, 1, 1);
        if (rc != PYDTNN_HIP_OK) return rc;
        const TileSel sel = pick_tile(g.k, g.p);
        WITH_TILE(sel, {
            auto al = plain_mn<T::BM>(w, (long)g.kn * g.k, g.k, 0, g.k);
            Im2colNchwMN<T::BN> bl;
            bl.x = dy; bl.g = g1;
            rc = launch<T>(al, bl, epi_plain(ws, g.p, 0, g.k, g.p, no_epilogue()), g.k, g.p, no_split(g.kn), 1,
                           stream);
        })
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
        rc = launch<T>(al, bl, epi_plain(ws, g.k, 0, g.p, g.k, no_epilogue()), g.p, g.k, no_split(g.kn), 1, stream);
    })
    if (rc != PYDTNN_HIP_OK) return rc;
    rc = launch_row2im_nhwc(ws, dx, g, stream);
    if (rc != PYDTNN_HIP_OK || !gate) return rc;
    return launch_relu_bwd(dx, gate, dx, (long)g.n * g.c * g.h * g.w, stream);
}

int conv_dx(const ConvGeom& g, int nhwc, const float* w, const float* dy, float* dx, float* ws, size_t ws_bytes,
            hipStream_t stream, const int8_t* gate = nullptr)
{
    if (!dx_as_forward(g)) return conv_dx_i2c(g, nhwc, w, dy, dx, ws, ws_bytes, stream, gate);
    const size_t need = (size_t)g.kn * g.k * 4;
    if (!ws || ws_bytes < need) return PYDTNN_HIP_ERR_WORKSPACE;
    int rc = launch_flip_filter(w, ws, nhwc, g.kn, g.c, g.kh, g.kw, stream);
    if (rc != PYDTNN_HIP_OK) return rc;
    ConvGeom gb;  // input = dy (kn channels, ho x wo), filters = c, output = (h, w)
    rc = make_conv_geom(&gb, g.n, g.kn, g.ho, g.wo, g.c, g.kh, g.kw, g.vdilation * (g.kh - 1) - g.vpadding,
                        g.hdilation * (g.kw - 1) - g.hpadding, 1, 1, g.vdilation, g.hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    if (gb.ho != g.h || gb.wo != g.w) return PYDTNN_HIP_ERR_INVALID;
    // what is left of the workspace after the flipped filter balances the launch
    const size_t used = (need + 255) & ~(size_t)255;
    float* rest = ws_bytes > used ? ws + used / 4 : nullptr;
    const size_t rest_bytes = ws_bytes > used ? ws_bytes - used : 0;
    const ElemMasks masks = {gate, nullptr};
    return nhwc ? conv_fwd_nhwc(gb, ws, dy, dx, no_epilogue(), rest, rest_bytes, stream, masks)
                : conv_fwd_nchw(gb, ws, dy, dx, no_epilogue(), rest, rest_bytes, stream, masks);
}

int geom_from_args(ConvGeom* g, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                   long hpadding, long vstride, long hstride, long vdilation, long hdilation)
{
    const long lim = 1l << 30;
    if (b >= lim || c >= lim || h >= lim || w >= lim || kn >= lim || kh >= lim || kw >= lim || vpadding >= lim ||
        hpadding >= lim || vstride >= lim || hstride >= lim || vdilation >= lim || hdilation >= lim)
        return PYDTNN_HIP_ERR_INVALID;
    return make_conv_geom(g, (int)b, (int)c, (int)h, (int)w, (int)kn, (int)kh, (int)kw, (int)vpadding, (int)hpadding,
                          (int)vstride, (int)hstride, (int)vdilation, (int)hdilation);
}

int sconv_gemm(int nhwc, char trans, const ConvGeom& g, const float* in1, const float* x, float* out,
               const float* bias, const float* mean, const float* inv_std, const float* gamma, const float* beta,
               bool relu, void* ws, size_t ws_bytes, hipStream_t stream, int accumulate = 0,
               int8_t* relu_mask = nullptr)
{
    if (!in1 || !x || !out) return PYDTNN_HIP_ERR_INVALID;
    if (relu_mask && !relu) return PYDTNN_HIP_ERR_INVALID;
    if (trans == 'N') {
        if (!bn_args_consistent(mean, inv_std, gamma, beta)) return PYDTNN_HIP_ERR_INVALID;
        const ChanEpilogue chan = make_chan(bias, mean, inv_std, gamma, beta, relu ? 1 : 0);
        const ElemMasks masks = {nullptr, relu_mask};
        return nhwc ? conv_fwd_nhwc(g, in1, x, out, chan, (float*)ws, ws_bytes, stream, masks)
                    : conv_fwd_nchw(g, in1, x, out, chan, (float*)ws, ws_bytes, stream, masks);
    }
    if (trans == 'Y') {
        if (bias || mean || inv_std || gamma || beta || relu) return PYDTNN_HIP_ERR_INVALID;
        return nhwc ? conv_dw_nhwc(g, in1, x, nullptr, out, (float*)ws, ws_bytes, stream, accumulate)
                    : conv_dw_nchw(g, in1, x, nullptr, out, (float*)ws, ws_bytes, stream, accumulate);
    }
    return PYDTNN_HIP_ERR_INVALID;
}

#define GEOM_ARGS b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation

// ---------------------------------------------------------------- batches beyond the addressing limit
// One launch addresses every tensor through 32-bit byte offsets (fewer than 2^29 floats per tensor).
// Larger batches are run as consecutive groups of whole images: forward and dX are independent per
// image; the filter gradient of the second and later groups is added to the first's (in that order).
long g_tensor_floats_limit = 1l << 29;

struct ImageGroups {
    long per_image_in, per_image_out;  // floats of x and of y per image
    long images;                       // images per launch
};

inline int plan_image_groups(ImageGroups* ig, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                             long hpadding, long vstride, long hstride, long vdilation, long hdilation)
{
    if (b <= 0 || c <= 0 || h <= 0 || w <= 0 || kn <= 0 || kh <= 0 || kw <= 0 || vstride <= 0 || hstride <= 0 ||
        vdilation <= 0 || hdilation <= 0 || h >= (1l << 20) || w >= (1l << 20) || c >= (1l << 24) || kn >= (1l << 24))
        return PYDTNN_HIP_ERR_INVALID;
    const long ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) / vstride + 1;
    const long wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) / hstride + 1;
    if (ho <= 0 || wo <= 0) return PYDTNN_HIP_ERR_INVALID;
    ig->per_image_in = c * h * w;
    ig->per_image_out = kn * ho * wo;
    const long largest = ig->per_image_in > ig->per_image_out ? ig->per_image_in : ig->per_image_out;
    long images = (g_tensor_floats_limit - 1) / largest;
    if (images < 1) images = 1;  // a single image beyond the limit is refused by make_conv_geom
    ig->images = images < b ? images : b;
    return PYDTNN_HIP_OK;
}

int sconv_gemm_batched(int nhwc, char trans, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                       long hpadding, long vstride, long hstride, long vdilation, long hdilation, const float* in1,
                       const float* x, float* out, const float* bias, const float* mean, const float* inv_std,
                       const float* gamma, const float* beta, bool relu, void* ws, size_t ws_bytes, hipStream_t stream,
                       int8_t* relu_mask = nullptr)
{
    if (!in1 || !x || !out) return PYDTNN_HIP_ERR_INVALID;
    ImageGroups ig;
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    for (long n0 = 0; n0 < b; n0 += ig.images) {
        ConvGeom g;
        const long nb = b - n0 < ig.images ? b - n0 : ig.images;
        rc = geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
        if (rc != PYDTNN_HIP_OK) return rc;
        const float* xg = x + n0 * ig.per_image_in;
        if (trans == 'Y')  // in1 = dy, out = dw
            rc = sconv_gemm(nhwc, trans, g, in1 + n0 * ig.per_image_out, xg, out, bias, mean, inv_std, gamma, beta,
                            relu, ws, ws_bytes, stream, n0 > 0);
        else               // in1 = weights, out = y
            rc = sconv_gemm(nhwc, trans, g, in1, xg, out + n0 * ig.per_image_out, bias, mean, inv_std, gamma, beta,
                            relu, ws, ws_bytes, stream, 0, relu_mask ? relu_mask + n0 * ig.per_image_out : nullptr);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return PYDTNN_HIP_OK;
}

int conv_dx_batched(int nhwc, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding, long hpadding,
                    long vstride, long hstride, long vdilation, long hdilation, const float* weights, const float* dy,
                    float* dx, float* ws, size_t ws_bytes, hipStream_t stream, const int8_t* gate = nullptr)
{
    if (!weights || !dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    ImageGroups ig;
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    for (long n0 = 0; n0 < b; n0 += ig.images) {
        ConvGeom g;
        const long nb = b - n0 < ig.images ? b - n0 : ig.images;
        rc = geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
        if (rc != PYDTNN_HIP_OK) return rc;
        rc = conv_dx(g, nhwc, weights, dy + n0 * ig.per_image_out, dx + n0 * ig.per_image_in, ws, ws_bytes, stream,
                     gate ? gate + n0 * ig.per_image_in : nullptr);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return PYDTNN_HIP_OK;
}

}  // namespace

extern "C" {

long pydtnn_hip_debug_set_tensor_floats_limit(long floats)
{
    const long before = g_tensor_floats_limit;
    if (floats > 0 && floats <= (1l << 29)) g_tensor_floats_limit = floats;
    return before;
}

int pydtnn_hip_version(void) { return 10000 * 0 + 100 * 1 + 0; }

const char* pydtnn_hip_status_string(int status)
{
    switch (status) {
        case PYDTNN_HIP_OK: return "ok";
        case PYDTNN_HIP_ERR_INVALID: return "invalid argument";
        case PYDTNN_HIP_ERR_WORKSPACE: return "workspace missing or too small";
        case PYDTNN_HIP_ERR_LAUNCH: return "HIP launch/runtime error";
        case PYDTNN_HIP_ERR_UNSUPPORTED: return "extents not supported by the index arithmetic";
        default: return "unknown status";
    }
}


int pydtnn_hip_im2col_nchw(const float* x, float* cols, int b, int c, int h, int w, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_im2col_nchw(x, cols, g, as_stream(stream));
}

int pydtnn_hip_col2im_nchw(const float* cols, float* dx, int b, int c, int h, int w, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_col2im_nchw(cols, dx, g, as_stream(stream));
}

int pydtnn_hip_im2row_nhwc(const float* x, float* rows, int b, int h, int w, int c, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_im2row_nhwc(x, rows, g, as_stream(stream));
}

int pydtnn_hip_row2im_nhwc(const float* rows, float* dx, int b, int h, int w, int c, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_row2im_nhwc(rows, dx, g, as_stream(stream));
}

// ---------------------------------------------------------------- GEMM
size_t pydtnn_hip_sgemm_workspace_bytes(long m, long n, long k)
{
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const TileSel sel = pick_tile(m, n);
    const SplitPlan sp = plan_plain_split(tiles_of(sel, m, n), k, m * n);
    return sp.splits > 1 ? (size_t)sp.splits * m * n * 4 : 0;
}

int pydtnn_hip_sgemm(int transa, int transb, long m, long n, long k, const float* a, long lda, const float* b,
                     long ldb, float* c, long ldc, const float* bias, int relu, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    if (!a || !b || !c || m <= 0 || n <= 0 || k <= 0) return PYDTNN_HIP_ERR_INVALID;
    const long lim = 1l << 31;
    if (m >= lim || n >= lim || k >= lim) return PYDTNN_HIP_ERR_UNSUPPORTED;
    if (lda < (transa ? m : k) || ldb < (transb ? k : n) || ldc < n) return PYDTNN_HIP_ERR_INVALID;
    const TileSel sel = pick_tile(m, n);
    const SplitPlan sp = plan_plain_split(tiles_of(sel, m, n), k, m * n);
    const ChanEpilogue chan = make_chan(bias, nullptr, nullptr, nullptr, nullptr, relu);
    float* dst = c;
    long dst_ld = ldc;
    ChanEpilogue gemm_chan = chan;
    if (sp.splits > 1) {
        if (!workspace || workspace_bytes < (size_t)sp.splits * m * n * 4) return PYDTNN_HIP_ERR_WORKSPACE;
        dst = (float*)workspace;
        dst_ld = n;
        gemm_chan = no_epilogue();
    }
    const hipStream_t st = as_stream(stream);
    int rc = PYDTNN_HIP_OK;
    // floats reachable from each base pointer (last row may be shorter than its leading dimension)
    const long a_total = transa ? (k - 1) * lda + m : (m - 1) * lda + k;
    const long b_total = transb ? (n - 1) * ldb + k : (k - 1) * ldb + n;
    WITH_TILE(sel, {
        const EpiPlain ep = epi_plain(dst, dst_ld, m * n, m, n, gemm_chan, no_masks(), sp.splits);
        if ((!transa && !span_ok_k(T::BM, lda, 0, 0)) || (transa && !span_ok_mn(lda)) ||
            (transb && !span_ok_k(T::BN, ldb, 0, 0)) || (!transb && !span_ok_mn(ldb)))
            return PYDTNN_HIP_ERR_UNSUPPORTED;
        if (!transa && !transb)
            rc = launch<T>(plain_k<T::BM, false>(a, a_total, lda, 0, m, 0), plain_mn<T::BN>(b, b_total, ldb, 0, n), ep,
                           m, n, sp.si, sp.splits, st);
        else if (!transa && transb)
            rc = launch<T>(plain_k<T::BM, false>(a, a_total, lda, 0, m, 0),
                           plain_k<T::BN, false>(b, b_total, ldb, 0, n, 0), ep, m, n, sp.si, sp.splits, st);
        else if (transa && !transb)
            rc = launch<T>(plain_mn<T::BM>(a, a_total, lda, 0, m), plain_mn<T::BN>(b, b_total, ldb, 0, n), ep, m, n,
                           sp.si, sp.splits, st);
        else
            rc = launch<T>(plain_mn<T::BM>(a, a_total, lda, 0, m), plain_k<T::BN, false>(b, b_total, ldb, 0, n, 0), ep,
                           m, n, sp.si, sp.splits, st);
    })
    if (rc != PYDTNN_HIP_OK || sp.splits == 1) return rc;
    if (ldc != n) return PYDTNN_HIP_ERR_UNSUPPORTED;  // the split reduction writes a dense C
    return launch_splitk_reduce((const float*)workspace, c, m, (int)n, m * n, sp.splits, 0, 0, chan, 0, st);
}

// ---------------------------------------------------------------- convolution
size_t pydtnn_hip_conv_workspace_bytes(int op, int nhwc, int b, int c, int h, int w, int kn, int kh, int kw,
                                       int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation)
{
    // the implicit routes run a large batch as groups of images: their workspace is that of one group
    ConvGeom g;
    ImageGroups ig;
    long nb = b;
    if (op != PYDTNN_HIP_OP_DX_I2C && plan_image_groups(&ig, GEOM_ARGS) == PYDTNN_HIP_OK) nb = ig.images;
    if (geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation) !=
        PYDTNN_HIP_OK)
        return 0;
    switch (op) {
        case PYDTNN_HIP_OP_DW: return (size_t)plan_dw(g, nhwc).splits * g.kn * g.k * 4;
        case PYDTNN_HIP_OP_FWD: return kBalanceBytes;  // optional: a smaller or absent workspace only costs speed
        case PYDTNN_HIP_OP_DX:
            return dx_as_forward(g) ? (((size_t)g.kn * g.k * 4 + 255) & ~(size_t)255) + kBalanceBytes
                                    : (size_t)g.k * g.p * 4;
        case PYDTNN_HIP_OP_DX_I2C: return (size_t)g.k * g.p * 4;
        case PYDTNN_HIP_OP_DB: return bias_grad_workspace_floats(g.n, g.kn) * 4;
        default: return 0;
    }
}

int pydtnn_hip_sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float* in1, const float* x, float* out,
                             const float* bias_vector, const float* bn_running_mean, const float* bn_inv_std,
                             const float* bn_gamma, const float* bn_beta, bool relu, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return sconv_gemm_batched(0, trans, GEOM_ARGS, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma,
                              bn_beta, relu, workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float* in1, const float* x, float* out,
                             const float* bias_vector, const float* bn_running_mean, const float* bn_inv_std,
                             const float* bn_gamma, const float* bn_beta, bool relu, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return sconv_gemm_batched(1, trans, GEOM_ARGS, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma,
                              bn_beta, relu, workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                  const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    return conv_dx_batched(0, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                  const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    return conv_dx_batched(1, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

// ---------------------------------------------------------------- explicit (i2c) GEMM steps
int pydtnn_hip_conv_i2c_forward(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding,
                                int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                                const float* weights, const float* mat, float* y, const float* bias_vector,
                                void* stream)
{
    if (!weights || !mat || !y) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const ChanEpilogue chan = make_chan(bias_vector, nullptr, nullptr, nullptr, nullptr, 0);
    const hipStream_t st = as_stream(stream);
    if (!nhwc) {
        const TileSel sel = pick_tile(g.kn, g.p, g.k);
        WITH_TILE(sel, {
            if (!span_ok_mn(g.p)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            rc = launch<T>(plain_k<T::BM, false>(weights, (long)g.kn * g.k, g.k, 0, g.kn, 0),
                           plain_mn<T::BN>(mat, (long)g.k * g.p, g.p, 0, g.p),
                           epi_nchw(y, g.kn, g.howo, g.p, chan), g.kn, g.p, no_split(g.k), 1, st);
        })
    } else {
        const TileSel sel = pick_tile(g.p, g.kn, g.k);
        WITH_TILE(sel, {
            rc = launch<T>(plain_k<T::BM, false>(mat, g.p * g.k, g.k, 0, g.p, 0),
                           plain_mn<T::BN>(weights, (long)g.k * g.kn, g.kn, 0, g.kn),
                           epi_plain(y, g.kn, 0, g.p, g.kn, chan), g.p, g.kn, no_split(g.k), 1, st);
        })
    }
    return rc;
}

int pydtnn_hip_conv_i2c_dw(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float* dy, const float* mat,
                           float* dw, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!dy || !mat || !dw) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    return nhwc ? conv_dw_nhwc(g, dy, nullptr, mat, dw, (float*)workspace, workspace_bytes, as_stream(stream))
                : conv_dw_nchw(g, dy, nullptr, mat, dw, (float*)workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_conv_i2c_dx(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float* weights,
                           const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!weights || !dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    return conv_dx_i2c(g, nhwc, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

// ---------------------------------------------------------------- elementwise and friends
int pydtnn_hip_chan_eltwise(const float* x, const float* residual, float* y, long total, int inner, int channels,
                            const float* bias, const float* bn_running_mean, const float* bn_inv_std,
                            const float* bn_gamma, const float* bn_beta, int relu, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    if (!bn_args_consistent(bn_running_mean, bn_inv_std, bn_gamma, bn_beta)) return PYDTNN_HIP_ERR_INVALID;
    return launch_chan_eltwise(x, residual, y, total, inner, channels,
                               make_chan(bias, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu),
                               as_stream(stream));
}

int pydtnn_hip_relu_fwd(const float* x, float* y, int8_t* mask, long total, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    return launch_relu_fwd(x, y, mask, total, as_stream(stream));
}

int pydtnn_hip_relu_bwd(const float* dy, const int8_t* mask, float* dx, long total, void* stream)
{
    if (!dy || !mask || !dx) return PYDTNN_HIP_ERR_INVALID;
    return launch_relu_bwd(dy, mask, dx, total, as_stream(stream));
}

int pydtnn_hip_bias_grad(const float* dy, float* db, long outer, int channels, int inner, void* workspace,
                         size_t workspace_bytes, void* stream)
{
    if (!dy || !db) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < bias_grad_workspace_floats(outer, channels) * 4)
        return PYDTNN_HIP_ERR_WORKSPACE;
    return launch_bias_grad(dy, db, outer, channels, inner, (float*)workspace, as_stream(stream));
}

int pydtnn_hip_max_pool_2d_fwd_nchw(const float* x, float* y, int32_t* idx_max, int b, int c, int h, int w, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void* stream)
{
    if (!x || !y || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_max_pool_fwd_nchw(x, y, idx_max, g, as_stream(stream));
}

int pydtnn_hip_max_pool_2d_bwd_nchw(const float* dy, const int32_t* idx_max, float* dx, int b, int c, int h, int w,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_max_pool_bwd_nchw(dy, idx_max, dx, g, as_stream(stream), nullptr);
}

int pydtnn_hip_max_pool_2d_fwd_nhwc(const float* x, float* y, int32_t* idx_max, int b, int h, int w, int c, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void* stream)
{
    if (!x || !y || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_max_pool_fwd_nhwc(x, y, idx_max, g, as_stream(stream));
}

int pydtnn_hip_max_pool_2d_bwd_nhwc(const float* dy, const int32_t* idx_max, float* dx, int b, int h, int w, int c,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_max_pool_bwd_nhwc(dy, idx_max, dx, g, as_stream(stream), nullptr);
}

int pydtnn_hip_max_pool_2d_bwd_gated(int nhwc, const float* dy, const int32_t* idx_max, float* dx, const int8_t* gate,
                                     int b, int c, int h, int w, int kh, int kw, int vpadding, int hpadding,
                                     int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max || !gate) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    return nhwc ? launch_max_pool_bwd_nhwc(dy, idx_max, dx, g, as_stream(stream), gate)
                : launch_max_pool_bwd_nchw(dy, idx_max, dx, g, as_stream(stream), gate);
}

int pydtnn_hip_sconvGemm_relu_mask(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                   unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride,
                                   unsigned hstride, unsigned vdilation, unsigned hdilation, const float* weights,
                                   const float* x, float* y, const float* bias_vector, int8_t* mask, void* workspace,
                                   size_t workspace_bytes, void* stream)
{
    if (!mask) return PYDTNN_HIP_ERR_INVALID;
    return sconv_gemm_batched(nhwc, 'N', GEOM_ARGS, weights, x, y, bias_vector, nullptr, nullptr, nullptr, nullptr,
                              true, workspace, workspace_bytes, as_stream(stream), mask);
}

int pydtnn_hip_sconvGemm_back_gated(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                    unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                    unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                    const float* dy, float* dx, const int8_t* gate, void* workspace,
                                    size_t workspace_bytes, void* stream)
{
    if (!gate) return PYDTNN_HIP_ERR_INVALID;
    return conv_dx_batched(nhwc, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream),
                           gate);
}

size_t pydtnn_hip_bn_training_workspace_bytes(int channels)
{
    return channels > 0 ? bn_training_workspace_floats(channels) * 4 : 0;
}

int pydtnn_hip_bn_training_fwd(const float* x, float* y, float* xn, float* std_out, const float* gamma,
                               const float* beta, float* running_mean, float* running_var, double momentum, double eps,
                               long outer, int channels, int inner, void* workspace, size_t workspace_bytes,
                               void* stream)
{
    if (!x || !y || !xn || !std_out || !gamma || !beta || !running_mean || !running_var)
        return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < pydtnn_hip_bn_training_workspace_bytes(channels))
        return PYDTNN_HIP_ERR_WORKSPACE;
    // NumPy multiplies float32 arrays by the Python floats momentum and (1.0 - momentum) rounded to float32
    return launch_bn_training_fwd(x, y, xn, std_out, gamma, beta, running_mean, running_var, (float)momentum,
                                  (float)(1.0 - momentum), (float)eps, outer, channels, inner, (float*)workspace,
                                  as_stream(stream));
}

int pydtnn_hip_bn_training_bwd(const float* dy, const float* xn, const float* std_in, const float* gamma,
                               float* dgamma, float* dbeta, float* dx, long outer, int channels, int inner,
                               void* workspace, size_t workspace_bytes, void* stream)
{
    if (!dy || !xn || !std_in || !gamma || !dgamma || !dbeta) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < pydtnn_hip_bn_training_workspace_bytes(channels))
        return PYDTNN_HIP_ERR_WORKSPACE;
    return launch_bn_training_bwd(dy, xn, std_in, gamma, dgamma, dbeta, dx, outer, channels, inner, (float*)workspace,
                                  as_stream(stream));
}

int pydtnn_hip_softmax_fwd(const float* x, float* y, int rows, int cols, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    return launch_softmax_fwd(x, y, rows, cols, as_stream(stream));
}

int pydtnn_hip_softmax_bwd(const float* dy, const float* y, float* dx, int rows, int cols, void* stream)
{
    if (!dy || !y || !dx) return PYDTNN_HIP_ERR_INVALID;
    return launch_softmax_bwd(dy, y, dx, rows, cols, as_stream(stream));
}

int pydtnn_hip_categorical_cross_entropy(const float* y_pred, const float* y_targ, float* dx, float* loss, int rows,
                                         int cols, double eps, int global_batch, void* workspace,
                                         size_t workspace_bytes, void* stream)
{
    if (!y_pred || !y_targ || !dx || !loss || global_batch <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < (size_t)(rows > 0 ? rows : 0) * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    // the reference clips a float32 array with float64 bounds: the bounds are rounded to float32 first
    return launch_cce(y_pred, y_targ, dx, loss, (float*)workspace, rows, cols, (float)eps, (float)(1.0 - eps),
                      (float)global_batch, as_stream(stream));
}

int pydtnn_hip_sgd_momentum(float* w, const float* dw, float* velocity, long total, float lr, float momentum,
                            float decay, int nesterov, void* stream)
{
    if (!w || !dw || !velocity) return PYDTNN_HIP_ERR_INVALID;
    return launch_sgd_momentum(w, dw, velocity, total, lr, momentum, decay, nesterov, as_stream(stream));
}

}  // extern "C"

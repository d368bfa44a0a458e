// Shared by the translation units that hold the GEMM launches: tile / split selection, loader and
// epilogue builders, and the entry points each unit defines for the others.
#pragma once
#include "../../include/pydtnn_hip.h"
#include "gemm_engine.h"
#include <atomic>

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
int launch_avg_pool_fwd(int nhwc, const float*, float*, const ConvGeom&, hipStream_t);
int launch_avg_pool_bwd(int nhwc, const float*, float*, const ConvGeom&, hipStream_t);
int launch_sgd_momentum(float*, const float*, float*, long, float, float, float, int, hipStream_t);
int launch_sgd_momentum_multi(int, float* const*, const float* const*, float* const*, const long*, float, float, float,
                              int, hipStream_t);

namespace convint {


using namespace gemm;

typedef Tile<128, 128, 2, 2> T128x128;
typedef Tile<64, 256, 1, 4> T64x256;
typedef Tile<256, 64, 4, 1> T256x64;
typedef Tile<64, 64, 2, 2> T64x64;

// eight MFMA blocks per wavefront, two workgroups per CU: NCHW forward / dX launches with long reductions
// (pick_tile_fwd) and the filter gradients whose matrix the tile covers without padding rows.
// (The 128x256 twin measured 2-4 % slower than 128x128 on VGG16's 128-filter layers and is not built.)
typedef Tile<256, 128, 4, 1> T256x128;

enum TileSel { SEL_128x128, SEL_64x256, SEL_256x64, SEL_64x64, SEL_COUNT, SEL_256x128 = SEL_COUNT, SEL_ALL };

struct TileShape {
    long bm, bn;
    double efficiency;  // matrix-core rate of the shape relative to 128x128 (fewer MFMAs per load and barrier)
};
constexpr TileShape kTileShapes[SEL_ALL] = {{128, 128, 1.0}, {64, 256, 0.93}, {256, 64, 0.93}, {64, 64, 0.6},
                                           {256, 128, 1.02}};

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

// Forward / dX: as pick_tile, but a choice of 128x128 moves up to the 256x128 tile when the reduction is long
// (its prologue and tile store are twice as long) and there are enough of them to fill the chip, which holds
// 512 at once.
constexpr long kBigTileMinTiles = 512;
inline TileSel pick_tile_fwd(long m, long n, long k)
{
    TileSel best = pick_tile(m, n, k);
    if (best != SEL_128x128 || k < 16 * BK) return best;
    double best_cost = (double)tiles_of(best, m, n) * 128.0 * 128.0;
    for (int s = SEL_256x128; s < SEL_ALL; ++s) {
        const TileShape& t = kTileShapes[s];
        const long tiles = tiles_of((TileSel)s, m, n);
        const double cost = (double)tiles * (double)(t.bm * t.bn) / t.efficiency;
        if (tiles >= kBigTileMinTiles && cost < best_cost) { best = (TileSel)s; best_cost = cost; }
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
inline SplitPlan plan_pixel_split(long tiles, int images, int seg, long out_elems, long target_blocks = kTargetBlocks)
{
    const long total = (long)images * seg;
    long want = tiles >= target_blocks ? 1 : target_blocks / tiles;
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
inline SplitPlan plan_plain_split(long tiles, long k, long out_elems)
{
    SplitPlan p;
    // as many chunks as fill one resident round of workgroups: a few more would run alone in a second round
    long want = tiles >= 256 ? 1 : kTargetBlocks / tiles;
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
inline PlainK4<BMN> plain_k4(const float* base, long total, long ld, long extent)
{
    PlainK4<BMN> l;
    l.base = base; l.total = total; l.ld = ld; l.extent = (int)extent;
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

// at most one of them is ever set: a training forward writes a ReLU mask, dX reads a gate, an inference
// forward at the end of an addition block's path adds the other path
inline int mask_kind(const ElemMasks& m)
{
    return m.gate ? kGate : m.relu_mask ? kReluMask : m.residual ? kResidual : kNoMasks;
}

// ---------------------------------------------------------------- forward (implicit)
// The padding test works on tap masks of 31 usable bits: one word over i*kw + j when kh*kw <= 31,
// otherwise one word per axis.
inline bool taps_supported(const ConvGeom& g) { return g.kh <= 31 && g.kw <= 31; }
inline bool taps_wide(const ConvGeom& g) { return g.khw > 31; }

// Workspace of the balanced launch (gemm::launch_balanced): two accumulator tiles per resident
// workgroup, sized for the most this part can hold (4 per CU on 256 CUs) so that the query needs no device.
constexpr int kMaxResident = 1024;
constexpr size_t kBalanceBytes = (size_t)2 * kMaxResident * 128 * 128 * 4;

// ---------------------------------------------------------------- input gradient
// Stride 1: dx = forward convolution of dy with the flipped, channel-swapped filter and padding
// dilation*(k-1) - padding.  Otherwise: the reference's own route, W^T dy then col2im / row2im.
inline bool dx_as_forward(const ConvGeom& g)
{
    return g.vstride == 1 && g.hstride == 1 && g.vdilation * (g.kh - 1) >= g.vpadding &&
           g.hdilation * (g.kw - 1) >= g.hpadding;
}

// A 1x1 filter at stride 1 without padding makes x itself the (P x C) row matrix and the filter the
// (C x kn) matrix: a plain GEMM, whose loaders carry no per-pixel offsets or tap masks.
inline bool pointwise_nhwc(const ConvGeom& g)
{
    return g.khw == 1 && g.vstride == 1 && g.hstride == 1 && g.vpadding == 0 && g.hpadding == 0;
}

// bytes of the (K x P) product of the explicit input gradient, rounded so that what follows it stays aligned
inline size_t i2c_product_bytes(const ConvGeom& g) { return ((size_t)g.k * g.p * 4 + 255) & ~(size_t)255; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Row-major forward launch (y is P x kn) with the epilogue variant the masks ask for.
template <class T, class AL, class BL>
inline int launch_rows_forward(const AL& al, const BL& bl, const ConvGeom& g, float* y, const ChanEpilogue& chan,
                               float* ws, size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    switch (mask_kind(masks)) {
    case kGate:
        return gemm::launch_balanced<T>(al, bl, epi_plain<kGate>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn, g.k, ws,
                                        ws_bytes, stream);
    case kReluMask:
        return gemm::launch_balanced<T>(al, bl, epi_plain<kReluMask>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn,
                                        g.k, ws, ws_bytes, stream);
    case kResidual:
        return gemm::launch_balanced<T>(al, bl, epi_plain<kResidual>(y, g.kn, 0, g.p, g.kn, chan, masks), g.p, g.kn,
                                        g.k, ws, ws_bytes, stream);
    default:
        return gemm::launch_balanced<T>(al, bl, epi_plain(y, g.kn, 0, g.p, g.kn, chan), g.p, g.kn, g.k, ws, ws_bytes,
                                        stream);
    }
}

// ---------------------------------------------------------------- defined in the conv_*.hip units
// conv_fwd_nchw.hip / conv_fwd_nhwc.hip.  `ws` is optional: without it (or with less than kBalanceBytes)
// the launch is a plain grid of tiles.
int conv_fwd_nchw(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks = no_masks());
int conv_fwd_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks = no_masks());
// conv_fwd_nhwc_pointwise.hip
int conv_fwd_nhwc_pointwise(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                            float* ws, size_t ws_bytes, hipStream_t stream, const ElemMasks& masks);
// conv_stream.hip: small filter matrices (whole in LDS), activations straight from memory into MFMA operands
bool conv_stream_nhwc_eligible(const ConvGeom& g, const float* w, const float* x);
int conv_stream_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                     hipStream_t stream, const ElemMasks& masks);
// conv_stream_nchw.hip: the same idea for first layers (few channels, large filters, any stride), both formats
bool conv_stream_first_eligible(int nhwc, const ConvGeom& g, const ElemMasks& masks);
int conv_stream_first(int nhwc, const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                      hipStream_t stream, const ElemMasks& masks);
// conv_bwd.hip
SplitPlan plan_dw(const ConvGeom& g, int nhwc);
int conv_dw_nchw(const ConvGeom& g, const float* dy, const float* x, const float* cols, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate = 0);
int conv_dw_nhwc(const ConvGeom& g, const float* dy, const float* x, const float* rows, float* dw, float* ws,
                 size_t ws_bytes, hipStream_t stream, int accumulate = 0);
int conv_dx_i2c(const ConvGeom& g, int nhwc, const float* w, const float* dy, float* dx, float* ws, size_t ws_bytes,
                hipStream_t stream, const int8_t* gate = nullptr);

}  // namespace convint

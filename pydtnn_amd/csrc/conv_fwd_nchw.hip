// Implicit-GEMM forward (and stride-1 dX) launches, NCHW.
#include "conv_internal.h"

namespace convint {

template <class T, class AL, class BL>
int launch_planes_forward(const AL& al, const BL& bl, const ConvGeom& g, float* y, const ChanEpilogue& chan, float* ws,
                          size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    switch (mask_kind(masks)) {
    case kGate:
        return launch_balanced<T>(al, bl, epi_nchw<kGate>(y, g.kn, g.howo, g.p, chan, masks), g.kn, g.p, g.k, ws,
                                  ws_bytes, stream);
    case kReluMask:
        return launch_balanced<T>(al, bl, epi_nchw<kReluMask>(y, g.kn, g.howo, g.p, chan, masks), g.kn, g.p, g.k, ws,
                                  ws_bytes, stream);
    case kResidual:
        return launch_balanced<T>(al, bl, epi_nchw<kResidual>(y, g.kn, g.howo, g.p, chan, masks), g.kn, g.p, g.k, ws,
                                  ws_bytes, stream);
    default:
        return launch_balanced<T>(al, bl, epi_nchw(y, g.kn, g.howo, g.p, chan), g.kn, g.p, g.k, ws, ws_bytes, stream);
    }
}

template <bool WIDE>
int conv_fwd_nchw_t(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                    size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    // filter rows of a multiple of 4 floats from an aligned tensor: 128-bit loads along the reduction axis
    const bool quads = !WIDE && g.k % 4 == 0 && aligned16(w);
    const TileSel sel = quads ? pick_tile_fwd(g.kn, g.p, g.k) : pick_tile(g.kn, g.p, g.k);
    int rc = PYDTNN_HIP_OK;
    if constexpr (!WIDE) {
        if (sel == SEL_256x128) {
            typedef T256x128 T;
            if (!span_ok_k(T::BM, g.k, 0, 0)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            Im2colNchwMN<T::BN, false> bl;
            bl.x = x; bl.g = g;
            return launch_planes_forward<T>(plain_k4<T::BM>(w, (long)g.kn * g.k, g.k, g.kn), bl, g, y, chan, ws,
                                            ws_bytes, stream, masks);
        }
    }
    if (g.kn % 96 == 0 && g.kn % 64 != 0) {
        // 96, 288, ... filters (AlexNet's first layer): 96-row tiles instead of 128-row ones that are a quarter padding
        typedef Tile<96, 256, 1, 4> T;
        if (!span_ok_k(T::BM, g.k, 0, 0)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        Im2colNchwMN<T::BN, WIDE> bl;
        bl.x = x; bl.g = g;
        return launch_planes_forward<T>(plain_k<T::BM, false>(w, (long)g.kn * g.k, g.k, 0, g.kn, 0), bl, g, y, chan, ws,
                                        ws_bytes, stream, masks);
    }
    WITH_TILE(sel, {
        if (!span_ok_k(T::BM, g.k, 0, 0)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        Im2colNchwMN<T::BN, WIDE> bl;
        bl.x = x; bl.g = g;
        if constexpr (!WIDE) {
            if (quads)
                return launch_planes_forward<T>(plain_k4<T::BM>(w, (long)g.kn * g.k, g.k, g.kn), bl, g, y, chan, ws,
                                                ws_bytes, stream, masks);
        }
        rc = launch_planes_forward<T>(plain_k<T::BM, false>(w, (long)g.kn * g.k, g.k, 0, g.kn, 0), bl, g, y, chan, ws,
                                      ws_bytes, stream, masks);
    })
    return rc;
}

// `ws` is optional: without it (or with less than kBalanceBytes) the launch is a plain grid of tiles.
int conv_fwd_nchw(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    if (!taps_supported(g)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    if (conv_stream_first_eligible(0, g, masks)) return conv_stream_first(0, g, w, x, y, chan, stream, masks);
    return taps_wide(g) ? conv_fwd_nchw_t<true>(g, w, x, y, chan, ws, ws_bytes, stream, masks)
                        : conv_fwd_nchw_t<false>(g, w, x, y, chan, ws, ws_bytes, stream, masks);
}


}  // namespace convint

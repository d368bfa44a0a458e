// Implicit-GEMM forward (and stride-1 dX) launches, NHWC.
#include "conv_internal.h"

namespace convint {

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

int conv_fwd_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    if (pointwise_nhwc(g)) return conv_fwd_nhwc_pointwise(g, w, x, y, chan, ws, ws_bytes, stream, masks);
    if (!taps_supported(g)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    return taps_wide(g) ? conv_fwd_nhwc_t<true>(g, w, x, y, chan, ws, ws_bytes, stream, masks)
                        : conv_fwd_nhwc_t<false>(g, w, x, y, chan, ws, ws_bytes, stream, masks);
}


}  // namespace convint

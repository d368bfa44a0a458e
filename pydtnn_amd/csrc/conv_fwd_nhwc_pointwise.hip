// NHWC 1x1 convolutions as plain GEMMs.
#include "conv_internal.h"

namespace convint {

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


}  // namespace convint

// NHWC 1x1 convolutions as plain GEMMs.
#include "conv_internal.h"

namespace convint {

int conv_fwd_nhwc_pointwise(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                            float* ws, size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    // A reduction of four steps or fewer is all loads and stores: with tiles as wide as 256 filters a workgroup
    // reads its rows of x once for all of them (64 -> 256 channels at 56x56: 95 us against 105 us on 128x128 tiles).
    const TileSel sel = g.k <= 64 && g.kn % 256 == 0 ? SEL_64x256 : pick_tile(g.p, g.kn, g.k);
    const bool quads = g.c % 4 == 0 && aligned16(x);
    int rc = PYDTNN_HIP_OK;
    WITH_TILE(sel, {
        if (!span_ok_k(T::BM, g.c, 0, 0) || !span_ok_mn(g.kn)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        auto bl = plain_mn<T::BN>(w, (long)g.c * g.kn, g.kn, 0, g.kn);
        if (quads)
            rc = launch_rows_forward<T>(plain_k4<T::BM>(x, g.p * g.c, g.c, g.p), bl, g, y, chan, ws, ws_bytes, stream,
                                        masks);
        else
            rc = launch_rows_forward<T>(plain_k<T::BM, false>(x, g.p * g.c, g.c, 0, g.p, 0), bl, g, y, chan, ws,
                                        ws_bytes, stream, masks);
    })
    return rc;
}

}  // namespace convint

// Implicit-GEMM forward (and stride-1 dX) launches, NHWC.
#include "conv_internal.h"

namespace convint {

template <bool WIDE>
int conv_fwd_nhwc_t(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                    size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    // channels in multiples of 16 from an aligned tensor: 128-bit loads along the channel axis
    const bool quads = !WIDE && g.c % 16 == 0 && aligned16(x);
    // (the 256x128 tile of the NCHW forward measured level or up to 6 % slower here and is not used)
    const TileSel sel = pick_tile(g.p, g.kn, g.k);
    int rc = PYDTNN_HIP_OK;
    if (g.c <= 4) {
        // a first layer: lanes along the pixels (3 floats apart for RGB) and the reduction index in the filter's own
        // (c, i, j) row order; with lanes along 27 reduction indices the loads of a tile are a chain of latencies
        WITH_TILE(sel, {
            Im2colNchwMN<T::BM, WIDE, true> al;
            al.x = x; al.g = g;
            auto bl = plain_mn<T::BN>(w, (long)g.k * g.kn, g.kn, 0, g.kn);
            rc = launch_rows_forward<T>(al, bl, g, y, chan, ws, ws_bytes, stream, masks);
        })
        return rc;
    }
    WITH_TILE(sel, {
        FilterNhwcMN<T::BN> bl;
        bl.w = w; bl.g = g;
        if constexpr (!WIDE) {
            if (quads) {
                Im2rowNhwcK4<T::BM> al;
                al.x = x; al.g = g;
                return launch_rows_forward<T>(al, bl, g, y, chan, ws, ws_bytes, stream, masks);
            }
        }
        Im2rowNhwcK<T::BM, WIDE> al;
        al.x = x; al.g = g;
        rc = launch_rows_forward<T>(al, bl, g, y, chan, ws, ws_bytes, stream, masks);
    })
    return rc;
}

int conv_fwd_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan, float* ws,
                  size_t ws_bytes, hipStream_t stream, const ElemMasks& masks)
{
    if (conv_stream_first_eligible(1, g, masks)) return conv_stream_first(1, g, w, x, y, chan, stream, masks);
    if (conv_stream_nhwc_eligible(g, w, x)) return conv_stream_nhwc(g, w, x, y, chan, stream, masks);
    if (pointwise_nhwc(g)) return conv_fwd_nhwc_pointwise(g, w, x, y, chan, ws, ws_bytes, stream, masks);
    if (!taps_supported(g)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    return taps_wide(g) ? conv_fwd_nhwc_t<true>(g, w, x, y, chan, ws, ws_bytes, stream, masks)
                        : conv_fwd_nhwc_t<false>(g, w, x, y, chan, ws, ws_bytes, stream, masks);
}


}  // namespace convint

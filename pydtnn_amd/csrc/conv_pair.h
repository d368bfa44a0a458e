// Entry points of the streaming kernels that other translation units call beside those of conv_internal.h.
#pragma once
#include "conv_internal.h"

namespace convint {

// The direction (0 forwards, 1 backwards) in which the next streaming launch on `stream` should walk the pixel
// blocks of x: the opposite of the launch that last walked its residual (or else its input).  Notes the walk.
int conv_stream_choose_direction(hipStream_t stream, const void* x, const void* residual, const void* y);

// A 3x3 convolution over 64 channels with 64 filters followed by a 1x1 convolution of its rectified, normalised
// output to `kn2` filters, NHWC, as one launch: the 64-channel tensor between them never exists in memory.
// g1 is the geometry of the first convolution.
bool conv_stream_pair_eligible(const ConvGeom& g1, int kn2, const float* w1, const float* w2, const float* x,
                               const ChanEpilogue& chan2, const ElemMasks& masks);
int conv_stream_pair(const ConvGeom& g1, int kn2, const float* w1, const float* w2, const float* x, float* y,
                     const ChanEpilogue& chan1, const ChanEpilogue& chan2, const ElemMasks& masks, hipStream_t stream);

}  // namespace convint

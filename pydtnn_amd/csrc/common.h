// Shared declarations for the gfx950 conv-as-GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

// Status codes returned by every device-pointer entry point.
#define PYDTNN_HIP_OK 0
#define PYDTNN_HIP_ERR_INVALID 1      // bad argument (null pointer, zero extent, unknown flag)
#define PYDTNN_HIP_ERR_WORKSPACE 2    // workspace missing or too small
#define PYDTNN_HIP_ERR_LAUNCH 3       // HIP reported a launch/runtime error
#define PYDTNN_HIP_ERR_UNSUPPORTED 4  // extents beyond what the index arithmetic covers

// Division of a small unsigned by a run-time constant as one mul-hi, branch-free.
// Exact for every n with n * div < 2^32 (checked on the host before a launch).
// div == 1 has no 32-bit multiplier; it is handled by mul = 0 and pass = all ones (q = 0 + n).
struct FastDiv {
    uint32_t mul;
    uint32_t div;
    uint32_t pass;
};

static inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.div = d;
    f.mul = d <= 1 ? 0u : (uint32_t)(((1ull << 32) + d - 1) / d);
    f.pass = d <= 1 ? 0xffffffffu : 0u;
    return f;
}

__device__ __forceinline__ uint32_t fd_div(uint32_t n, const FastDiv f)
{
    return __umulhi(n, f.mul) + (n & f.pass);
}

// The same quotient where the host could not prove n * div < 2^32: `exact` is a launch-wide flag,
// so the branch is uniform and the hardware division is only paid by shapes that need it.
__device__ __forceinline__ uint32_t fd_div_checked(uint32_t n, const FastDiv f, int exact)
{
    return exact ? fd_div(n, f) : n / f.div;
}

// Geometry of one convolution. Names follow PyDTNN's Conv2D (vpadding = vertical padding, ...).
// Output extent: ho = (h + 2*vpadding - vdilation*(kh-1) - 1) / vstride + 1 (pydtnn/layers/conv_2d.py:75-76).
struct ConvGeom {
    int n, c, h, w;     // input batch, channels, height, width
    int kn, kh, kw;     // filters, filter height, filter width
    int vpadding, hpadding, vstride, hstride, vdilation, hdilation;
    int ho, wo;         // output height, width
    int k;              // c*kh*kw  (reduction length of the forward GEMM)
    int khw;            // kh*kw
    int howo;           // ho*wo
    long p;             // n*ho*wo  (pixels = GEMM columns in NCHW, rows in NHWC)
    FastDiv fd_khw, fd_kw, fd_wo, fd_c, fd_howo;
    FastDiv fd_w, fd_kh, fd_vs, fd_hs;  // used by the streaming kernels (input-plane pixel, pool index, strides)
};

static inline int conv_out_dim(int in, int pad, int dil, int k, int stride)
{
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

// Fills a ConvGeom; returns a PYDTNN_HIP_* status.
int make_conv_geom(ConvGeom* g, int n, int c, int h, int w, int kn, int kh, int kw,
                   int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation);

// Per-channel epilogue applied to an accumulator before the single store:
//   v += bias[ch];  v = ((v - mean[ch]) * inv_std[ch]) * gamma[ch] + beta[ch];  v = v > 0 ? v : 0
// in that order (bias -> BN inference -> ReLU), each stage optional.
struct ChanEpilogue {
    const float* bias;
    const float* mean;
    const float* inv_std;
    const float* gamma;
    const float* beta;
    int relu;
};

__device__ __forceinline__ float chan_epilogue_apply(const ChanEpilogue& e, int ch, float v)
{
    if (e.bias) v += e.bias[ch];
    if (e.mean) {
        float t = (v - e.mean[ch]) * e.inv_std[ch];
        v = t * e.gamma[ch] + e.beta[ch];
    }
    if (e.relu) v = v > 0.0f ? v : 0.0f;
    return v;
}

static inline ChanEpilogue no_epilogue()
{
    ChanEpilogue e = {nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    return e;
}

// Per-element companions a GEMM store can read or write beside its output, all indexed like the output:
//   gate      (input)  the value is stored as v * gate[i], i.e. ReLU's backward dx = dy * mask
//                      (pydtnn/backends/cpu/activations/relu_cpu.py:38-40) applied by the producer of dy;
//   relu_mask (output) relu_mask[i] = v > 0, the mask ReLU's forward keeps for its backward
//                      (pydtnn/cython_modules/relu_cython.pyx:25-59), written by a store that also rectifies;
//   residual  (input)  the value is stored as v + residual[i], the sum an addition block makes of its paths
//                      (pydtnn/backends/cpu/layers/addition_block_cpu.py:41-45, eltw_sum_cython.pyx:25-36),
//                      then rectified when relu_after_add is set (the Relu layer that follows the block).
struct ElemMasks {
    const int8_t* gate;
    int8_t* relu_mask;
    const float* residual;
    int relu_after_add;
};

static inline ElemMasks no_masks()
{
    ElemMasks m = {nullptr, nullptr, nullptr, 0};
    return m;
}

// Which of them a store handles is a compile-time choice, so that no store tests a pointer per element.
constexpr int kNoMasks = 0, kGate = 1, kReluMask = 2, kResidual = 3;

template <int MASKS>
__device__ __forceinline__ float elem_masks_apply(const ElemMasks& mk, long i, float v)
{
    if (MASKS == kGate) v *= (float)mk.gate[i];
    if (MASKS == kReluMask) mk.relu_mask[i] = v > 0.0f ? 1 : 0;
    if (MASKS == kResidual) {
        v += mk.residual[i];
        if (mk.relu_after_add) v = v > 0.0f ? v : 0.0f;
    }
    return v;
}

// The form of the calling thread's most recent GEMM or streaming-convolution launch, kept for the test-only
// query pydtnn_hip_debug_last_launch: a benchmark that quotes counters taken for one kernel form checks with it
// that the library still picks that form.
enum { kLaunchNone = 0, kLaunchTiles = 1, kLaunchBalanced = 2, kLaunchStreamNhwc = 3, kLaunchStreamNchw = 4,
       kLaunchPair = 5 };
struct LaunchNote {
    int kind, tile_m, tile_n, workgroups, cut_tiles, splits;
};
inline thread_local LaunchNote g_last_launch = {};
inline void note_launch(int kind, int tile_m, int tile_n, long workgroups, int cut_tiles, int splits)
{
    g_last_launch = LaunchNote{kind, tile_m, tile_n, (int)workgroups, cut_tiles, splits};
}

#define HIP_RETURN_IF_LAUNCH_FAILED()                         \
    do {                                                      \
        hipError_t e__ = hipGetLastError();                   \
        if (e__ != hipSuccess) return PYDTNN_HIP_ERR_LAUNCH;  \
    } while (0)

// Host-pointer flavour of the convolution entry points, with the names and signatures of the
// external libconvGemm that PyDTNN binds through ctypes
// (pydtnn/backends/cpu/libs/conv_gemm.py:85-107).  Operands are copied to the GPU, the
// device-pointer entry points do the work, and the result is copied back.  The reference's ABI has no error
// channel (void functions): a failure is reported on stderr and the process aborts instead of continuing with
// numbers that were never computed.
#include "../../include/pydtnn_hip.h"
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <mutex>

namespace {

[[noreturn]] void die(const char* what, const char* detail)
{
    fprintf(stderr, "libconvGemm (pydtnn_hip): %s failed: %s\n", what, detail);
    abort();
}

void check_hip(hipError_t e, const char* what)
{
    if (e != hipSuccess) die(what, hipGetErrorString(e));
}

void check_rc(int rc, const char* what)
{
    if (rc != PYDTNN_HIP_OK) die(what, pydtnn_hip_status_string(rc));
}

// Device buffers live in a grow-only cache, one slot per role, kept for the life of the process: a layer
// calls with the same shapes again and again, and a hipMalloc / hipFree pair per operand and call costs more
// than a small kernel.  The slots are never freed explicitly (at process exit the HIP runtime may already be
// gone when static destructors run; the driver reclaims the memory).  One call at a time: the reference calls
// from a single thread, but ctypes releases the GIL, so a mutex keeps two callers from sharing the slots.
enum Slot { SLOT_IN1, SLOT_X, SLOT_OUT, SLOT_WS, SLOT_BIAS, SLOT_MEAN, SLOT_ISTD, SLOT_GAMMA, SLOT_BETA, SLOT_COUNT };

struct Cache {
    void* p[SLOT_COUNT] = {};
    size_t bytes[SLOT_COUNT] = {};
    int device = -1;
    std::mutex lock;
};
Cache g_cache;

void* slot(Slot s, size_t n)
{
    if (n == 0) return nullptr;
    int dev = 0;
    check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (dev != g_cache.device) {  // buffers belong to the device they were allocated on
        for (int i = 0; i < SLOT_COUNT; ++i) {
            if (g_cache.p[i]) (void)hipFree(g_cache.p[i]);
            g_cache.p[i] = nullptr;
            g_cache.bytes[i] = 0;
        }
        g_cache.device = dev;
    }
    if (g_cache.bytes[s] < n) {
        if (g_cache.p[s]) check_hip(hipFree(g_cache.p[s]), "hipFree");
        g_cache.p[s] = nullptr;
        g_cache.bytes[s] = 0;
        const size_t want = n + n / 8;  // a little head room: batch sizes wobble
        check_hip(hipMalloc(&g_cache.p[s], want), "hipMalloc");
        g_cache.bytes[s] = want;
    }
    return g_cache.p[s];
}

float* upload(Slot s, const void* src, size_t n)
{
    if (!src || n == 0) return nullptr;
    void* d = slot(s, n);
    check_hip(hipMemcpy(d, src, n, hipMemcpyHostToDevice), "hipMemcpy H2D");
    return static_cast<float*>(d);
}

inline unsigned out_dim(unsigned in, unsigned pad, unsigned dil, unsigned k, unsigned stride)
{
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

void conv_host(int nhwc, char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
               unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
               unsigned vdilation, unsigned hdilation, const float* in1, const float* x, float* out,
               const float* bias_vector, const float* mean, const float* inv_std, const float* gamma,
               const float* beta, bool relu)
{
    const size_t ho = out_dim(h, vpadding, vdilation, kh, vstride), wo = out_dim(w, hpadding, hdilation, kw, hstride);
    const size_t x_elems = (size_t)b * c * h * w, y_elems = (size_t)b * kn * ho * wo, w_elems = (size_t)kn * c * kh * kw;
    const bool fwd = trans == 'N';
    std::lock_guard<std::mutex> hold(g_cache.lock);
    float* d_in1 = upload(SLOT_IN1, in1, (fwd ? w_elems : y_elems) * 4);
    float* d_x = upload(SLOT_X, x, x_elems * 4);
    const size_t out_bytes = (fwd ? y_elems : w_elems) * 4;
    float* d_out = static_cast<float*>(slot(SLOT_OUT, out_bytes));
    const size_t vec = (size_t)kn * 4;
    float* d_bias = upload(SLOT_BIAS, bias_vector, vec);
    float* d_mean = upload(SLOT_MEAN, mean, vec);
    float* d_istd = upload(SLOT_ISTD, inv_std, vec);
    float* d_gamma = upload(SLOT_GAMMA, gamma, vec);
    float* d_beta = upload(SLOT_BETA, beta, vec);
    // forward: the optional workspace that balances the launch; filter gradient: the partial sums of its split
    const size_t ws_bytes = pydtnn_hip_conv_workspace_bytes(fwd ? PYDTNN_HIP_OP_FWD : PYDTNN_HIP_OP_DW, nhwc, b, c, h, w,
                                                            kn, kh, kw, vpadding, hpadding, vstride, hstride,
                                                            vdilation, hdilation);
    void* d_ws = slot(SLOT_WS, ws_bytes);
    int rc;
    if (nhwc)
        rc = pydtnn_hip_sconvGemmNHWC(trans, b, h, w, c, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
                                      hdilation, d_in1, d_x, d_out, d_bias, d_mean, d_istd, d_gamma, d_beta, relu,
                                      d_ws, ws_bytes, nullptr);
    else
        rc = pydtnn_hip_sconvGemmNCHW(trans, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
                                      hdilation, d_in1, d_x, d_out, d_bias, d_mean, d_istd, d_gamma, d_beta, relu,
                                      d_ws, ws_bytes, nullptr);
    check_rc(rc, nhwc ? "sconvGemmNHWC" : "sconvGemmNCHW");
    // the copy back is ordered after the kernels on the null stream and returns when the data is on the host
    check_hip(hipMemcpy(out, d_out, out_bytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
}

void deconv_host(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                 unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                 unsigned hdilation, const float* weights, const float* dy, float* dx)
{
    const size_t ho = out_dim(h, vpadding, vdilation, kh, vstride), wo = out_dim(w, hpadding, hdilation, kw, hstride);
    const size_t x_elems = (size_t)b * c * h * w, y_elems = (size_t)b * kn * ho * wo, w_elems = (size_t)kn * c * kh * kw;
    std::lock_guard<std::mutex> hold(g_cache.lock);
    float* d_w = upload(SLOT_IN1, weights, w_elems * 4);
    float* d_dy = upload(SLOT_X, dy, y_elems * 4);
    float* d_dx = static_cast<float*>(slot(SLOT_OUT, x_elems * 4));
    const size_t ws_bytes = pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DX, nhwc, b, c, h, w, kn, kh, kw, vpadding,
                                                            hpadding, vstride, hstride, vdilation, hdilation);
    void* d_ws = slot(SLOT_WS, ws_bytes);
    int rc;
    if (nhwc)
        rc = pydtnn_hip_sconvGemmNHWC_back(b, h, w, c, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation,
                                           hdilation, d_w, d_dy, d_dx, d_ws, ws_bytes, nullptr);
    else
        rc = pydtnn_hip_sconvGemmNCHW_back(b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation,
                                           hdilation, d_w, d_dy, d_dx, d_ws, ws_bytes, nullptr);
    check_rc(rc, nhwc ? "sconvGemmNHWC_back" : "sconvGemmNCHW_back");
    check_hip(hipMemcpy(dx, d_dx, x_elems * 4, hipMemcpyDeviceToHost), "hipMemcpy D2H");
}

}  // namespace

extern "C" {

int alloc_pack_buffs(float** ac_pack, float** bc_pack)
{
    // The reference releases both blocks with libc free(); the GPU path has no use for them.
    *ac_pack = static_cast<float*>(malloc(64));
    *bc_pack = static_cast<float*>(malloc(64));
    if (!*ac_pack || !*bc_pack) {
        free(*ac_pack);
        free(*bc_pack);
        *ac_pack = *bc_pack = nullptr;
        return 1;
    }
    return 0;
}

void sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float* in1, const float* x, float* out, const float* bias_vector,
                   const float* bn_running_mean, const float* bn_inv_std, const float* bn_gamma,
                   const float* bn_beta, bool relu, float* /*ac_pack*/, float* /*bc_pack*/)
{
    conv_host(0, trans, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, in1, x,
              out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu);
}

void sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float* in1, const float* x, float* out, const float* bias_vector,
                   const float* bn_running_mean, const float* bn_inv_std, const float* bn_gamma,
                   const float* bn_beta, bool relu, float* /*ac_pack*/, float* /*bc_pack*/)
{
    conv_host(1, trans, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, in1, x,
              out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu);
}

void sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float* weights, const float* dy, float* dx, float* /*ac_pack*/,
                        float* /*bc_pack*/)
{
    deconv_host(0, b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation, weights, dy,
                dx);
}

void sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float* weights, const float* dy, float* dx, float* /*ac_pack*/,
                        float* /*bc_pack*/)
{
    deconv_host(1, b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation, hdilation, weights, dy,
                dx);
}

}  // extern "C"

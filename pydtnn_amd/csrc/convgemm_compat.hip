// Host-pointer flavour of the convolution entry points, with the names and signatures of the
// external libconvGemm that PyDTNN binds through ctypes
// (pydtnn/backends/cpu/libs/conv_gemm.py:85-107).  Operands are copied to the GPU, the
// device-pointer entry points do the work, and the result is copied back.
#include "../../include/pydtnn_hip.h"
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

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

struct DeviceBuf {
    void* p = nullptr;
    size_t bytes = 0;
    explicit DeviceBuf(size_t n) : bytes(n)
    {
        if (n) check_hip(hipMalloc(&p, n), "hipMalloc");
    }
    ~DeviceBuf()
    {
        if (p) (void)hipFree(p);
    }
    float* f() const { return static_cast<float*>(p); }
    void upload(const void* src) const
    {
        if (src && bytes) check_hip(hipMemcpy(p, src, bytes, hipMemcpyHostToDevice), "hipMemcpy H2D");
    }
    void download(void* dst) const
    {
        if (dst && bytes) check_hip(hipMemcpy(dst, p, bytes, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    }
    DeviceBuf(const DeviceBuf&) = delete;
    DeviceBuf& operator=(const DeviceBuf&) = delete;
};

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
    DeviceBuf d_in1((fwd ? w_elems : y_elems) * 4), d_x(x_elems * 4), d_out((fwd ? y_elems : w_elems) * 4);
    d_in1.upload(in1);
    d_x.upload(x);
    const size_t vec = (size_t)kn * 4;
    DeviceBuf d_bias(bias_vector ? vec : 0), d_mean(mean ? vec : 0), d_istd(inv_std ? vec : 0),
        d_gamma(gamma ? vec : 0), d_beta(beta ? vec : 0);
    d_bias.upload(bias_vector);
    d_mean.upload(mean);
    d_istd.upload(inv_std);
    d_gamma.upload(gamma);
    d_beta.upload(beta);
    const size_t ws_bytes =
        fwd ? 0
            : pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DW, nhwc, b, c, h, w, kn, kh, kw, vpadding, hpadding,
                                              vstride, hstride, vdilation, hdilation);
    DeviceBuf d_ws(ws_bytes);
    int rc;
    if (nhwc)
        rc = pydtnn_hip_sconvGemmNHWC(trans, b, h, w, c, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
                                      hdilation, d_in1.f(), d_x.f(), d_out.f(), d_bias.f(), d_mean.f(), d_istd.f(),
                                      d_gamma.f(), d_beta.f(), relu, d_ws.p, ws_bytes, nullptr);
    else
        rc = pydtnn_hip_sconvGemmNCHW(trans, b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation,
                                      hdilation, d_in1.f(), d_x.f(), d_out.f(), d_bias.f(), d_mean.f(), d_istd.f(),
                                      d_gamma.f(), d_beta.f(), relu, d_ws.p, ws_bytes, nullptr);
    check_rc(rc, nhwc ? "sconvGemmNHWC" : "sconvGemmNCHW");
    check_hip(hipDeviceSynchronize(), "kernel execution");
    d_out.download(out);
}

void deconv_host(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                 unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                 unsigned hdilation, const float* weights, const float* dy, float* dx)
{
    const size_t ho = out_dim(h, vpadding, vdilation, kh, vstride), wo = out_dim(w, hpadding, hdilation, kw, hstride);
    const size_t x_elems = (size_t)b * c * h * w, y_elems = (size_t)b * kn * ho * wo, w_elems = (size_t)kn * c * kh * kw;
    DeviceBuf d_w(w_elems * 4), d_dy(y_elems * 4), d_dx(x_elems * 4);
    d_w.upload(weights);
    d_dy.upload(dy);
    const size_t ws_bytes = pydtnn_hip_conv_workspace_bytes(PYDTNN_HIP_OP_DX, nhwc, b, c, h, w, kn, kh, kw, vpadding,
                                                            hpadding, vstride, hstride, vdilation, hdilation);
    DeviceBuf d_ws(ws_bytes);
    int rc;
    if (nhwc)
        rc = pydtnn_hip_sconvGemmNHWC_back(b, h, w, c, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation,
                                           hdilation, d_w.f(), d_dy.f(), d_dx.f(), d_ws.p, ws_bytes, nullptr);
    else
        rc = pydtnn_hip_sconvGemmNCHW_back(b, c, h, w, kn, kh, kw, vstride, hstride, vpadding, hpadding, vdilation,
                                           hdilation, d_w.f(), d_dy.f(), d_dx.f(), d_ws.p, ws_bytes, nullptr);
    check_rc(rc, nhwc ? "sconvGemmNHWC_back" : "sconvGemmNCHW_back");
    check_hip(hipDeviceSynchronize(), "kernel execution");
    d_dx.download(dx);
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

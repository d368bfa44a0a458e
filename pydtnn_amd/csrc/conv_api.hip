// Device-pointer C ABI: argument checks, batching over image groups, and the launches that are not
// convolutions (GEMM, explicit-path GEMMs, streaming kernels).
#include "conv_internal.h"
#include "conv_pair.h"
#include "../../include/pydtnn_hip_test.h"
#include <mutex>
#include <new>

namespace {

using namespace convint;

int conv_dx(const ConvGeom& g, int nhwc, const float* w, const float* dy, float* dx, float* ws, size_t ws_bytes,
            hipStream_t stream, const int8_t* gate = nullptr)
{
    if (!dx_as_forward(g)) return conv_dx_i2c(g, nhwc, w, dy, dx, ws, ws_bytes, stream, gate);
    const size_t need = (size_t)g.kn * g.k * 4;
    if (!ws || ws_bytes < need) return PYDTNN_HIP_ERR_WORKSPACE;
    int rc = launch_flip_filter(w, ws, nhwc, g.kn, g.c, g.kh, g.kw, stream);
    if (rc != PYDTNN_HIP_OK) return rc;
    ConvGeom gb;  // input = dy (kn channels, ho x wo), filters = c, output = (h, w)
    rc = make_conv_geom(&gb, g.n, g.kn, g.ho, g.wo, g.c, g.kh, g.kw, g.vdilation * (g.kh - 1) - g.vpadding,
                        g.hdilation * (g.kw - 1) - g.hpadding, 1, 1, g.vdilation, g.hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    if (gb.ho != g.h || gb.wo != g.w) return PYDTNN_HIP_ERR_INVALID;
    // what is left of the workspace after the flipped filter balances the launch
    const size_t used = (need + 255) & ~(size_t)255;
    float* rest = ws_bytes > used ? ws + used / 4 : nullptr;
    const size_t rest_bytes = ws_bytes > used ? ws_bytes - used : 0;
    const ElemMasks masks = {gate, nullptr, nullptr, 0};
    return nhwc ? conv_fwd_nhwc(gb, ws, dy, dx, no_epilogue(), rest, rest_bytes, stream, masks)
                : conv_fwd_nchw(gb, ws, dy, dx, no_epilogue(), rest, rest_bytes, stream, masks);
}

int geom_from_args(ConvGeom* g, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                   long hpadding, long vstride, long hstride, long vdilation, long hdilation)
{
    const long lim = 1l << 30;
    if (b >= lim || c >= lim || h >= lim || w >= lim || kn >= lim || kh >= lim || kw >= lim || vpadding >= lim ||
        hpadding >= lim || vstride >= lim || hstride >= lim || vdilation >= lim || hdilation >= lim)
        return PYDTNN_HIP_ERR_INVALID;
    return make_conv_geom(g, (int)b, (int)c, (int)h, (int)w, (int)kn, (int)kh, (int)kw, (int)vpadding, (int)hpadding,
                          (int)vstride, (int)hstride, (int)vdilation, (int)hdilation);
}

int sconv_gemm(int nhwc, char trans, const ConvGeom& g, const float* in1, const float* x, float* out,
               const float* bias, const float* mean, const float* inv_std, const float* gamma, const float* beta,
               bool relu, void* ws, size_t ws_bytes, hipStream_t stream, int accumulate = 0,
               int8_t* relu_mask = nullptr, const float* residual = nullptr, int relu_after_add = 0)
{
    if (!in1 || !x || !out) return PYDTNN_HIP_ERR_INVALID;
    if (relu_mask && !relu) return PYDTNN_HIP_ERR_INVALID;
    if (residual && (relu_mask || trans != 'N')) return PYDTNN_HIP_ERR_INVALID;
    if (trans == 'N') {
        if (!bn_args_consistent(mean, inv_std, gamma, beta)) return PYDTNN_HIP_ERR_INVALID;
        const ChanEpilogue chan = make_chan(bias, mean, inv_std, gamma, beta, relu ? 1 : 0);
        const ElemMasks masks = {nullptr, relu_mask, residual, relu_after_add};
        return nhwc ? conv_fwd_nhwc(g, in1, x, out, chan, (float*)ws, ws_bytes, stream, masks)
                    : conv_fwd_nchw(g, in1, x, out, chan, (float*)ws, ws_bytes, stream, masks);
    }
    if (trans == 'Y') {
        if (bias || mean || inv_std || gamma || beta || relu) return PYDTNN_HIP_ERR_INVALID;
        return nhwc ? conv_dw_nhwc(g, in1, x, nullptr, out, (float*)ws, ws_bytes, stream, accumulate)
                    : conv_dw_nchw(g, in1, x, nullptr, out, (float*)ws, ws_bytes, stream, accumulate);
    }
    return PYDTNN_HIP_ERR_INVALID;
}

#define GEOM_ARGS b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation

// ---------------------------------------------------------------- batches beyond the addressing limit
// One launch addresses every tensor through 32-bit byte offsets (fewer than 2^29 floats per tensor).
// Larger batches are run as consecutive groups of whole images: forward and dX are independent per
// image; the filter gradient of the second and later groups is added to the first's (in that order).
long g_tensor_floats_limit = 1l << 29;

struct ImageGroups {
    long per_image_in, per_image_out;  // floats of x and of y per image
    long images;                       // images per launch
};

inline int plan_image_groups(ImageGroups* ig, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                             long hpadding, long vstride, long hstride, long vdilation, long hdilation)
{
    if (b <= 0 || c <= 0 || h <= 0 || w <= 0 || kn <= 0 || kh <= 0 || kw <= 0 || vstride <= 0 || hstride <= 0 ||
        vdilation <= 0 || hdilation <= 0 || h >= (1l << 20) || w >= (1l << 20) || c >= (1l << 24) || kn >= (1l << 24))
        return PYDTNN_HIP_ERR_INVALID;
    const long ho = (h + 2 * vpadding - vdilation * (kh - 1) - 1) / vstride + 1;
    const long wo = (w + 2 * hpadding - hdilation * (kw - 1) - 1) / hstride + 1;
    if (ho <= 0 || wo <= 0) return PYDTNN_HIP_ERR_INVALID;
    ig->per_image_in = c * h * w;
    ig->per_image_out = kn * ho * wo;
    const long largest = ig->per_image_in > ig->per_image_out ? ig->per_image_in : ig->per_image_out;
    long images = (g_tensor_floats_limit - 1) / largest;
    if (images < 1) images = 1;  // a single image beyond the limit is refused by make_conv_geom
    ig->images = images < b ? images : b;
    return PYDTNN_HIP_OK;
}

int sconv_gemm_batched(int nhwc, char trans, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding,
                       long hpadding, long vstride, long hstride, long vdilation, long hdilation, const float* in1,
                       const float* x, float* out, const float* bias, const float* mean, const float* inv_std,
                       const float* gamma, const float* beta, bool relu, void* ws, size_t ws_bytes, hipStream_t stream,
                       int8_t* relu_mask = nullptr, const float* residual = nullptr, int relu_after_add = 0)
{
    if (!in1 || !x || !out) return PYDTNN_HIP_ERR_INVALID;
    ImageGroups ig;
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    for (long n0 = 0; n0 < b; n0 += ig.images) {
        ConvGeom g;
        const long nb = b - n0 < ig.images ? b - n0 : ig.images;
        rc = geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
        if (rc != PYDTNN_HIP_OK) return rc;
        const float* xg = x + n0 * ig.per_image_in;
        if (trans == 'Y')  // in1 = dy, out = dw
            rc = sconv_gemm(nhwc, trans, g, in1 + n0 * ig.per_image_out, xg, out, bias, mean, inv_std, gamma, beta,
                            relu, ws, ws_bytes, stream, n0 > 0);
        else               // in1 = weights, out = y
            rc = sconv_gemm(nhwc, trans, g, in1, xg, out + n0 * ig.per_image_out, bias, mean, inv_std, gamma, beta,
                            relu, ws, ws_bytes, stream, 0, relu_mask ? relu_mask + n0 * ig.per_image_out : nullptr,
                            residual ? residual + n0 * ig.per_image_out : nullptr, relu_after_add);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return PYDTNN_HIP_OK;
}

int conv_dx_batched(int nhwc, long b, long c, long h, long w, long kn, long kh, long kw, long vpadding, long hpadding,
                    long vstride, long hstride, long vdilation, long hdilation, const float* weights, const float* dy,
                    float* dx, float* ws, size_t ws_bytes, hipStream_t stream, const int8_t* gate = nullptr)
{
    if (!weights || !dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    ImageGroups ig;
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    for (long n0 = 0; n0 < b; n0 += ig.images) {
        ConvGeom g;
        const long nb = b - n0 < ig.images ? b - n0 : ig.images;
        rc = geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
        if (rc != PYDTNN_HIP_OK) return rc;
        rc = conv_dx(g, nhwc, weights, dy + n0 * ig.per_image_out, dx + n0 * ig.per_image_in, ws, ws_bytes, stream,
                     gate ? gate + n0 * ig.per_image_in : nullptr);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return PYDTNN_HIP_OK;
}

// ---------------------------------------------------------------- GEMM (shared by the two entry points)
int sgemm_impl(int transa, int transb, long m, long n, long k, const float* a, long lda, const float* b, long ldb,
               float* c, long ldc, const float* bias, int relu, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!a || !b || !c || m <= 0 || n <= 0 || k <= 0) return PYDTNN_HIP_ERR_INVALID;
    const long lim = 1l << 31;
    if (m >= lim || n >= lim || k >= lim) return PYDTNN_HIP_ERR_UNSUPPORTED;
    if (lda < (transa ? m : k) || ldb < (transb ? k : n) || ldc < n) return PYDTNN_HIP_ERR_INVALID;
    const TileSel sel = pick_tile(m, n);
    const SplitPlan sp = plan_plain_split(tiles_of(sel, m, n), k, m * n);
    const ChanEpilogue chan = make_chan(bias, nullptr, nullptr, nullptr, nullptr, relu);
    float* dst = c;
    long dst_ld = ldc;
    ChanEpilogue gemm_chan = chan;
    if (sp.splits > 1) {
        if (ldc != n) return PYDTNN_HIP_ERR_UNSUPPORTED;  // the sum over the split writes a dense C
        if (!workspace || workspace_bytes < (size_t)sp.splits * m * n * 4) return PYDTNN_HIP_ERR_WORKSPACE;
        dst = (float*)workspace;
        dst_ld = n;
        gemm_chan = no_epilogue();
    }
    const hipStream_t st = as_stream(stream);
    int rc = PYDTNN_HIP_OK;
    // floats reachable from each base pointer (last row may be shorter than its leading dimension)
    const long a_total = transa ? (k - 1) * lda + m : (m - 1) * lda + k;
    const long b_total = transb ? (n - 1) * ldb + k : (k - 1) * ldb + n;
    WITH_TILE(sel, {
        const EpiPlain ep = epi_plain(dst, dst_ld, m * n, m, n, gemm_chan, no_masks(), sp.splits);
        if ((!transa && !span_ok_k(T::BM, lda, 0, 0)) || (transa && !span_ok_mn(lda)) ||
            (transb && !span_ok_k(T::BN, ldb, 0, 0)) || (!transb && !span_ok_mn(ldb)))
            return PYDTNN_HIP_ERR_UNSUPPORTED;
        if (!transa && !transb)
            rc = launch<T>(plain_k<T::BM, false>(a, a_total, lda, 0, m, 0), plain_mn<T::BN>(b, b_total, ldb, 0, n), ep,
                           m, n, sp.si, sp.splits, st);
        else if (!transa && transb)
            rc = launch<T>(plain_k<T::BM, false>(a, a_total, lda, 0, m, 0),
                           plain_k<T::BN, false>(b, b_total, ldb, 0, n, 0), ep, m, n, sp.si, sp.splits, st);
        else if (transa && !transb)
            rc = launch<T>(plain_mn<T::BM>(a, a_total, lda, 0, m), plain_mn<T::BN>(b, b_total, ldb, 0, n), ep, m, n,
                           sp.si, sp.splits, st);
        else
            rc = launch<T>(plain_mn<T::BM>(a, a_total, lda, 0, m), plain_k<T::BN, false>(b, b_total, ldb, 0, n, 0), ep,
                           m, n, sp.si, sp.splits, st);
    })
    if (rc != PYDTNN_HIP_OK || sp.splits == 1) return rc;
    return launch_splitk_reduce((const float*)workspace, c, m, (int)n, m * n, sp.splits, 0, 0, chan, 0, st);
}

// ---------------------------------------------------------------- scratch that no call allocates
// Partial sums of pydtnn_hip_sgemm_static's split along k.  Every GPU the library runs on holds its own
// copy of this array, at its own address, until the process ends.  In host code the name `scratch` is
// only a handle for hipGetSymbolAddress: kernels get the address that call returns for the current
// device.  Nothing in it has to start at zero: a split GEMM writes every partial sum it later reads.
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_address[kMaxDevices] = {};

// Address of `scratch` on the current device, asked once per device (the first call on a device loads
// the library's code object there, which is the only set-up work).
int static_scratch_address(void** out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return PYDTNN_HIP_ERR_LAUNCH;
    if (dev < 0 || dev >= kMaxDevices) return PYDTNN_HIP_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_address[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return PYDTNN_HIP_ERR_LAUNCH;
        g_scratch_address[dev] = p;
    }
    *out = g_scratch_address[dev];
    return PYDTNN_HIP_OK;
}

// Pooling layers work plane by plane, so a batch whose tensors exceed the addressing limit of one launch runs
// as consecutive groups of whole images, like the convolutions.  `launch(geometry of the group, first image)`.
template <class Launch>
int pool_batched(long b, long c, long h, long w, long kh, long kw, long vpadding, long hpadding, long vstride,
                 long hstride, long vdilation, long hdilation, Launch launch)
{
    ImageGroups ig;
    const long kn = c;  // the output has the input's channels
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    for (long n0 = 0; n0 < b; n0 += ig.images) {
        ConvGeom g;
        const long nb = b - n0 < ig.images ? b - n0 : ig.images;
        rc = geom_from_args(&g, nb, c, h, w, 1, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
        if (rc != PYDTNN_HIP_OK) return rc;
        rc = launch(g, n0 * ig.per_image_in, n0 * ig.per_image_out);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return PYDTNN_HIP_OK;
}

#define POOL_ARGS b, c, h, w, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation

}  // namespace

extern "C" {

long pydtnn_hip_debug_set_tensor_floats_limit(long floats)
{
    const long before = g_tensor_floats_limit;
    if (floats > 0 && floats <= (1l << 29)) g_tensor_floats_limit = floats;
    return before;
}

void pydtnn_hip_debug_last_launch(int out[6])
{
    const LaunchNote n = g_last_launch;
    out[0] = n.kind; out[1] = n.tile_m; out[2] = n.tile_n; out[3] = n.workgroups; out[4] = n.cut_tiles; out[5] = n.splits;
}

int pydtnn_hip_version(void) { return 10000 * 0 + 100 * 1 + 0; }

const char* pydtnn_hip_status_string(int status)
{
    switch (status) {
        case PYDTNN_HIP_OK: return "ok";
        case PYDTNN_HIP_ERR_INVALID: return "invalid argument";
        case PYDTNN_HIP_ERR_WORKSPACE: return "workspace missing or too small";
        case PYDTNN_HIP_ERR_LAUNCH: return "HIP launch/runtime error";
        case PYDTNN_HIP_ERR_UNSUPPORTED: return "extents not supported by the index arithmetic";
        default: return "unknown status";
    }
}


int pydtnn_hip_im2col_nchw(const float* x, float* cols, int b, int c, int h, int w, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_im2col_nchw(x, cols, g, as_stream(stream));
}

int pydtnn_hip_col2im_nchw(const float* cols, float* dx, int b, int c, int h, int w, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !cols) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_col2im_nchw(cols, dx, g, as_stream(stream));
}

int pydtnn_hip_im2row_nhwc(const float* x, float* rows, int b, int h, int w, int c, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!x || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_im2row_nhwc(x, rows, g, as_stream(stream));
}

int pydtnn_hip_row2im_nhwc(const float* rows, float* dx, int b, int h, int w, int c, int kh, int kw, int vpadding,
                           int hpadding, int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dx || !rows) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int kn = 1;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    return rc != PYDTNN_HIP_OK ? rc : launch_row2im_nhwc(rows, dx, g, as_stream(stream));
}

// ---------------------------------------------------------------- GEMM
size_t pydtnn_hip_sgemm_workspace_bytes(long m, long n, long k)
{
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const TileSel sel = pick_tile(m, n);
    const SplitPlan sp = plan_plain_split(tiles_of(sel, m, n), k, m * n);
    return sp.splits > 1 ? (size_t)sp.splits * m * n * 4 : 0;
}

int pydtnn_hip_sgemm(int transa, int transb, long m, long n, long k, const float* a, long lda, const float* b,
                     long ldb, float* c, long ldc, const float* bias, int relu, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    return sgemm_impl(transa, transb, m, n, k, a, lda, b, ldb, c, ldc, bias, relu, workspace, workspace_bytes, stream);
}

size_t pydtnn_hip_sgemm_static_scratch_bytes(void) { return kStaticScratchBytes; }

int pydtnn_hip_sgemm_static(int transa, int transb, long m, long n, long k, const float* a, long lda, const float* b,
                            long ldb, float* c, long ldc, const float* bias, int relu, void* stream)
{
    const size_t need = pydtnn_hip_sgemm_workspace_bytes(m, n, k);
    if (need > kStaticScratchBytes) return PYDTNN_HIP_ERR_WORKSPACE;
    void* ws = nullptr;
    if (need > 0) {
        const int rc = static_scratch_address(&ws);
        if (rc != PYDTNN_HIP_OK) return rc;
    }
    return sgemm_impl(transa, transb, m, n, k, a, lda, b, ldb, c, ldc, bias, relu, ws, need ? kStaticScratchBytes : 0,
                      stream);
}

// ---------------------------------------------------------------- convolution
size_t pydtnn_hip_conv_workspace_bytes(int op, int nhwc, int b, int c, int h, int w, int kn, int kh, int kw,
                                       int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                       int hdilation)
{
    // the implicit routes run a large batch as groups of images: their workspace is that of one group
    ConvGeom g;
    ImageGroups ig;
    long nb = b;
    if (op != PYDTNN_HIP_OP_DX_I2C && op != PYDTNN_HIP_OP_FWD_I2C && plan_image_groups(&ig, GEOM_ARGS) == PYDTNN_HIP_OK) nb = ig.images;
    if (geom_from_args(&g, nb, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation) !=
        PYDTNN_HIP_OK)
        return 0;
    switch (op) {
        case PYDTNN_HIP_OP_DW: {
            // partial sums of the split, or the partial tiles of the balanced launch
            const size_t split = (size_t)plan_dw(g, nhwc).splits * g.kn * g.k * 4;
            return split > kBalanceBytes ? split : kBalanceBytes;
        }
        case PYDTNN_HIP_OP_FWD: return kBalanceBytes;  // optional: a smaller or absent workspace only costs speed
        case PYDTNN_HIP_OP_DX:
            return dx_as_forward(g) ? (((size_t)g.kn * g.k * 4 + 255) & ~(size_t)255) + kBalanceBytes
                                    : i2c_product_bytes(g) + kBalanceBytes;
        case PYDTNN_HIP_OP_DX_I2C: return i2c_product_bytes(g) + kBalanceBytes;  // the (K x P) product, then partial tiles
        case PYDTNN_HIP_OP_FWD_I2C: return kBalanceBytes;                       // optional, as for the implicit forward
        case PYDTNN_HIP_OP_DB: return bias_grad_workspace_floats(g.n, g.kn) * 4;
        default: return 0;
    }
}

int pydtnn_hip_sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float* in1, const float* x, float* out,
                             const float* bias_vector, const float* bn_running_mean, const float* bn_inv_std,
                             const float* bn_gamma, const float* bn_beta, bool relu, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return sconv_gemm_batched(0, trans, GEOM_ARGS, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma,
                              bn_beta, relu, workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                             unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                             unsigned vdilation, unsigned hdilation, const float* in1, const float* x, float* out,
                             const float* bias_vector, const float* bn_running_mean, const float* bn_inv_std,
                             const float* bn_gamma, const float* bn_beta, bool relu, void* workspace,
                             size_t workspace_bytes, void* stream)
{
    return sconv_gemm_batched(1, trans, GEOM_ARGS, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma,
                              bn_beta, relu, workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                  const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    return conv_dx_batched(0, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                  unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                  const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    return conv_dx_batched(1, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

// ---------------------------------------------------------------- two convolutions of a bottleneck in one launch
int pydtnn_hip_sconvGemm_pair_nhwc(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride,
                                   unsigned vdilation, unsigned hdilation, const float* weights, const float* x,
                                   const float* bias_vector, const float* bn_running_mean, const float* bn_inv_std,
                                   const float* bn_gamma, const float* bn_beta, bool relu, unsigned kn2,
                                   const float* weights2, float* y, const float* bias_vector2,
                                   const float* bn_running_mean2, const float* bn_inv_std2, const float* bn_gamma2,
                                   const float* bn_beta2, bool relu2, const float* residual, bool relu_after_add,
                                   void* stream)
{
    if (!weights || !x || !weights2 || !y) return PYDTNN_HIP_ERR_INVALID;
    if (!bn_args_consistent(bn_running_mean, bn_inv_std, bn_gamma, bn_beta) ||
        !bn_args_consistent(bn_running_mean2, bn_inv_std2, bn_gamma2, bn_beta2))
        return PYDTNN_HIP_ERR_INVALID;
    if (kn2 == 0 || kn2 >= (1u << 24)) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const ChanEpilogue chan1 = make_chan(bias_vector, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu ? 1 : 0);
    const ChanEpilogue chan2 = make_chan(bias_vector2, bn_running_mean2, bn_inv_std2, bn_gamma2, bn_beta2, relu2 ? 1 : 0);
    const ElemMasks masks = {nullptr, nullptr, residual, relu_after_add ? 1 : 0};
    return conv_stream_pair(g, (int)kn2, weights, weights2, x, y, chan1, chan2, masks, as_stream(stream));
}

// ---------------------------------------------------------------- a forward call with its arguments bound
struct pydtnn_hip_conv_plan {
    int nhwc;
    long geom[13];
    const float *weights, *bias, *mean, *inv_std, *gamma, *beta;
    bool relu;
};

int pydtnn_hip_conv_plan_create(pydtnn_hip_conv_plan** plan, int nhwc, int b, int c, int h, int w, int kn, int kh,
                                int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                int hdilation, const float* weights, const float* bias_vector,
                                const float* bn_running_mean, const float* bn_inv_std, const float* bn_gamma,
                                const float* bn_beta, bool relu)
{
    if (!plan) return PYDTNN_HIP_ERR_INVALID;
    *plan = nullptr;
    if (!weights || !bn_args_consistent(bn_running_mean, bn_inv_std, bn_gamma, bn_beta)) return PYDTNN_HIP_ERR_INVALID;
    ImageGroups ig;
    int rc = plan_image_groups(&ig, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    ConvGeom g;   // refuses here what the call would refuse: extents the index arithmetic does not cover
    rc = geom_from_args(&g, ig.images, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation);
    if (rc != PYDTNN_HIP_OK) return rc;
    pydtnn_hip_conv_plan* p = new (std::nothrow) pydtnn_hip_conv_plan;
    if (!p) return PYDTNN_HIP_ERR_INVALID;
    p->nhwc = nhwc ? 1 : 0;
    const long geom[13] = {GEOM_ARGS};
    for (int i = 0; i < 13; ++i) p->geom[i] = geom[i];
    p->weights = weights; p->bias = bias_vector; p->mean = bn_running_mean; p->inv_std = bn_inv_std;
    p->gamma = bn_gamma; p->beta = bn_beta; p->relu = relu;
    *plan = p;
    return PYDTNN_HIP_OK;
}

int pydtnn_hip_conv_plan_forward(const pydtnn_hip_conv_plan* plan, const float* x, float* y, void* workspace,
                                 size_t workspace_bytes, void* stream)
{
    if (!plan) return PYDTNN_HIP_ERR_INVALID;
    const long* q = plan->geom;
    return sconv_gemm_batched(plan->nhwc, 'N', q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], q[8], q[9], q[10], q[11],
                              q[12], plan->weights, x, y, plan->bias, plan->mean, plan->inv_std, plan->gamma, plan->beta,
                              plan->relu, workspace, workspace_bytes, as_stream(stream));
}

void pydtnn_hip_conv_plan_destroy(pydtnn_hip_conv_plan* plan) { delete plan; }

// ---------------------------------------------------------------- explicit (i2c) GEMM steps
int pydtnn_hip_conv_i2c_forward(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding,
                                int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                                const float* weights, const float* mat, float* y, const float* bias_vector,
                                void* workspace, size_t workspace_bytes, void* stream)
{
    if (!weights || !mat || !y) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    const ChanEpilogue chan = make_chan(bias_vector, nullptr, nullptr, nullptr, nullptr, 0);
    const hipStream_t st = as_stream(stream);
    float* ws = (float*)workspace;   // optional: without it the launch is a plain grid of tiles
    // rows of k floats read with 128-bit loads when k is a multiple of 4 and the matrix is aligned
    if (!nhwc) {
        // y (kn x P, stored as N,kn,ho,wo) = weights (kn x K) * x_cols (K x P)
        if (!span_ok_mn(g.p)) return PYDTNN_HIP_ERR_UNSUPPORTED;
        const bool quads = g.k % 4 == 0 && aligned16(weights);
        const TileSel sel = quads ? pick_tile_fwd(g.kn, g.p, g.k) : pick_tile(g.kn, g.p, g.k);
        if (sel == SEL_256x128) {
            typedef T256x128 T;
            return launch_balanced<T>(plain_k4<T::BM>(weights, (long)g.kn * g.k, g.k, g.kn),
                                      plain_mn<T::BN>(mat, (long)g.k * g.p, g.p, 0, g.p),
                                      epi_nchw(y, g.kn, g.howo, g.p, chan), g.kn, g.p, g.k, ws, workspace_bytes, st);
        }
        WITH_TILE(sel, {
            rc = launch_balanced<T>(plain_k<T::BM, false>(weights, (long)g.kn * g.k, g.k, 0, g.kn, 0),
                                    plain_mn<T::BN>(mat, (long)g.k * g.p, g.p, 0, g.p),
                                    epi_nchw(y, g.kn, g.howo, g.p, chan), g.kn, g.p, g.k, ws, workspace_bytes, st);
        })
    } else {
        // y (P x kn) = x_rows (P x K) * weights (K x kn)
        const TileSel sel = pick_tile(g.p, g.kn, g.k);
        const bool quads = g.k % 4 == 0 && aligned16(mat);
        WITH_TILE(sel, {
            if (!span_ok_k(T::BM, g.k, 0, 0) || !span_ok_mn(g.kn)) return PYDTNN_HIP_ERR_UNSUPPORTED;
            auto bl = plain_mn<T::BN>(weights, (long)g.k * g.kn, g.kn, 0, g.kn);
            const EpiPlain ep = epi_plain(y, g.kn, 0, g.p, g.kn, chan);
            if (quads)
                rc = launch_balanced<T>(plain_k4<T::BM>(mat, g.p * g.k, g.k, g.p), bl, ep, g.p, g.kn, g.k, ws,
                                        workspace_bytes, st);
            else
                rc = launch_balanced<T>(plain_k<T::BM, false>(mat, g.p * g.k, g.k, 0, g.p, 0), bl, ep, g.p, g.kn, g.k, ws,
                                        workspace_bytes, st);
        })
    }
    return rc;
}

int pydtnn_hip_conv_i2c_dw(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float* dy, const float* mat,
                           float* dw, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!dy || !mat || !dw) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    return nhwc ? conv_dw_nhwc(g, dy, nullptr, mat, dw, (float*)workspace, workspace_bytes, as_stream(stream))
                : conv_dw_nchw(g, dy, nullptr, mat, dw, (float*)workspace, workspace_bytes, as_stream(stream));
}

int pydtnn_hip_conv_i2c_dx(int nhwc, int b, int c, int h, int w, int kn, int kh, int kw, int vpadding, int hpadding,
                           int vstride, int hstride, int vdilation, int hdilation, const float* weights,
                           const float* dy, float* dx, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!weights || !dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    ConvGeom g;
    const int rc = geom_from_args(&g, GEOM_ARGS);
    if (rc != PYDTNN_HIP_OK) return rc;
    return conv_dx_i2c(g, nhwc, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream));
}

// ---------------------------------------------------------------- elementwise and friends
int pydtnn_hip_chan_eltwise(const float* x, const float* residual, float* y, long total, int inner, int channels,
                            const float* bias, const float* bn_running_mean, const float* bn_inv_std,
                            const float* bn_gamma, const float* bn_beta, int relu, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    if (!bn_args_consistent(bn_running_mean, bn_inv_std, bn_gamma, bn_beta)) return PYDTNN_HIP_ERR_INVALID;
    return launch_chan_eltwise(x, residual, y, total, inner, channels,
                               make_chan(bias, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu),
                               as_stream(stream));
}

int pydtnn_hip_relu_fwd(const float* x, float* y, int8_t* mask, long total, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    return launch_relu_fwd(x, y, mask, total, as_stream(stream));
}

int pydtnn_hip_relu_bwd(const float* dy, const int8_t* mask, float* dx, long total, void* stream)
{
    if (!dy || !mask || !dx) return PYDTNN_HIP_ERR_INVALID;
    return launch_relu_bwd(dy, mask, dx, total, as_stream(stream));
}

int pydtnn_hip_bias_grad(const float* dy, float* db, long outer, int channels, int inner, void* workspace,
                         size_t workspace_bytes, void* stream)
{
    if (!dy || !db) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < bias_grad_workspace_floats(outer, channels) * 4)
        return PYDTNN_HIP_ERR_WORKSPACE;
    return launch_bias_grad(dy, db, outer, channels, inner, (float*)workspace, as_stream(stream));
}

int pydtnn_hip_max_pool_2d_fwd_nchw(const float* x, float* y, int32_t* idx_max, int b, int c, int h, int w, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void* stream)
{
    if (!x || !y || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_max_pool_fwd_nchw(x + in0, y + out0, idx_max + out0, g, as_stream(stream));
    });
}

int pydtnn_hip_max_pool_2d_bwd_nchw(const float* dy, const int32_t* idx_max, float* dx, int b, int c, int h, int w,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_max_pool_bwd_nchw(dy + out0, idx_max + out0, dx + in0, g, as_stream(stream), nullptr);
    });
}

int pydtnn_hip_max_pool_2d_fwd_nhwc(const float* x, float* y, int32_t* idx_max, int b, int h, int w, int c, int kh,
                                    int kw, int vpadding, int hpadding, int vstride, int hstride, int vdilation,
                                    int hdilation, void* stream)
{
    if (!x || !y || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_max_pool_fwd_nhwc(x + in0, y + out0, idx_max + out0, g, as_stream(stream));
    });
}

int pydtnn_hip_max_pool_2d_bwd_nhwc(const float* dy, const int32_t* idx_max, float* dx, int b, int h, int w, int c,
                                    int kh, int kw, int vpadding, int hpadding, int vstride, int hstride,
                                    int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_max_pool_bwd_nhwc(dy + out0, idx_max + out0, dx + in0, g, as_stream(stream), nullptr);
    });
}

int pydtnn_hip_average_pool_2d_fwd(int nhwc, const float* x, float* y, int b, int c, int h, int w, int kh, int kw,
                                   int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                                   void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_avg_pool_fwd(nhwc, x + in0, y + out0, g, as_stream(stream));
    });
}

int pydtnn_hip_average_pool_2d_bwd(int nhwc, const float* dy, float* dx, int b, int c, int h, int w, int kh, int kw,
                                   int vpadding, int hpadding, int vstride, int hstride, int vdilation, int hdilation,
                                   void* stream)
{
    if (!dy || !dx) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return launch_avg_pool_bwd(nhwc, dy + out0, dx + in0, g, as_stream(stream));
    });
}

int pydtnn_hip_max_pool_2d_bwd_gated(int nhwc, const float* dy, const int32_t* idx_max, float* dx, const int8_t* gate,
                                     int b, int c, int h, int w, int kh, int kw, int vpadding, int hpadding,
                                     int vstride, int hstride, int vdilation, int hdilation, void* stream)
{
    if (!dy || !dx || !idx_max || !gate) return PYDTNN_HIP_ERR_INVALID;
    return pool_batched(POOL_ARGS, [&](const ConvGeom& g, long in0, long out0) {
        return nhwc ? launch_max_pool_bwd_nhwc(dy + out0, idx_max + out0, dx + in0, g, as_stream(stream), gate + in0)
                    : launch_max_pool_bwd_nchw(dy + out0, idx_max + out0, dx + in0, g, as_stream(stream), gate + in0);
    });
}

int pydtnn_hip_sconvGemm_relu_mask(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                   unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride,
                                   unsigned hstride, unsigned vdilation, unsigned hdilation, const float* weights,
                                   const float* x, float* y, const float* bias_vector, int8_t* mask, void* workspace,
                                   size_t workspace_bytes, void* stream)
{
    if (!mask) return PYDTNN_HIP_ERR_INVALID;
    return sconv_gemm_batched(nhwc, 'N', GEOM_ARGS, weights, x, y, bias_vector, nullptr, nullptr, nullptr, nullptr,
                              true, workspace, workspace_bytes, as_stream(stream), mask);
}

int pydtnn_hip_sconvGemm_residual(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                  unsigned kw, unsigned vpadding, unsigned hpadding, unsigned vstride,
                                  unsigned hstride, unsigned vdilation, unsigned hdilation, const float* weights,
                                  const float* x, float* y, const float* bias_vector, const float* bn_running_mean,
                                  const float* bn_inv_std, const float* bn_gamma, const float* bn_beta, bool relu,
                                  const float* residual, bool relu_after_add, void* workspace, size_t workspace_bytes,
                                  void* stream)
{
    if (!residual) return PYDTNN_HIP_ERR_INVALID;
    return sconv_gemm_batched(nhwc, 'N', GEOM_ARGS, weights, x, y, bias_vector, bn_running_mean, bn_inv_std, bn_gamma,
                              bn_beta, relu, workspace, workspace_bytes, as_stream(stream), nullptr, residual,
                              relu_after_add ? 1 : 0);
}

int pydtnn_hip_sconvGemm_back_gated(int nhwc, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh,
                                    unsigned kw, unsigned vstride, unsigned hstride, unsigned vpadding,
                                    unsigned hpadding, unsigned vdilation, unsigned hdilation, const float* weights,
                                    const float* dy, float* dx, const int8_t* gate, void* workspace,
                                    size_t workspace_bytes, void* stream)
{
    if (!gate) return PYDTNN_HIP_ERR_INVALID;
    return conv_dx_batched(nhwc, GEOM_ARGS, weights, dy, dx, (float*)workspace, workspace_bytes, as_stream(stream),
                           gate);
}

size_t pydtnn_hip_bn_training_workspace_bytes(int channels)
{
    return channels > 0 ? bn_training_workspace_floats(channels) * 4 : 0;
}

int pydtnn_hip_bn_training_fwd(const float* x, float* y, float* xn, float* std_out, const float* gamma,
                               const float* beta, float* running_mean, float* running_var, double momentum, double eps,
                               long outer, int channels, int inner, void* workspace, size_t workspace_bytes,
                               void* stream)
{
    if (!x || !y || !xn || !std_out || !gamma || !beta || !running_mean || !running_var)
        return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < pydtnn_hip_bn_training_workspace_bytes(channels))
        return PYDTNN_HIP_ERR_WORKSPACE;
    // NumPy multiplies float32 arrays by the Python floats momentum and (1.0 - momentum) rounded to float32
    return launch_bn_training_fwd(x, y, xn, std_out, gamma, beta, running_mean, running_var, (float)momentum,
                                  (float)(1.0 - momentum), (float)eps, outer, channels, inner, (float*)workspace,
                                  as_stream(stream));
}

int pydtnn_hip_bn_training_bwd(const float* dy, const float* xn, const float* std_in, const float* gamma,
                               float* dgamma, float* dbeta, float* dx, long outer, int channels, int inner,
                               void* workspace, size_t workspace_bytes, void* stream)
{
    if (!dy || !xn || !std_in || !gamma || !dgamma || !dbeta) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < pydtnn_hip_bn_training_workspace_bytes(channels))
        return PYDTNN_HIP_ERR_WORKSPACE;
    return launch_bn_training_bwd(dy, xn, std_in, gamma, dgamma, dbeta, dx, outer, channels, inner, (float*)workspace,
                                  as_stream(stream));
}

int pydtnn_hip_softmax_fwd(const float* x, float* y, int rows, int cols, void* stream)
{
    if (!x || !y) return PYDTNN_HIP_ERR_INVALID;
    return launch_softmax_fwd(x, y, rows, cols, as_stream(stream));
}

int pydtnn_hip_softmax_bwd(const float* dy, const float* y, float* dx, int rows, int cols, void* stream)
{
    if (!dy || !y || !dx) return PYDTNN_HIP_ERR_INVALID;
    return launch_softmax_bwd(dy, y, dx, rows, cols, as_stream(stream));
}

int pydtnn_hip_categorical_cross_entropy(const float* y_pred, const float* y_targ, float* dx, float* loss, int rows,
                                         int cols, double eps, int global_batch, void* workspace,
                                         size_t workspace_bytes, void* stream)
{
    if (!y_pred || !y_targ || !dx || !loss || global_batch <= 0) return PYDTNN_HIP_ERR_INVALID;
    if (!workspace || workspace_bytes < (size_t)(rows > 0 ? rows : 0) * 4) return PYDTNN_HIP_ERR_WORKSPACE;
    // the reference clips a float32 array with float64 bounds: the bounds are rounded to float32 first
    return launch_cce(y_pred, y_targ, dx, loss, (float*)workspace, rows, cols, (float)eps, (float)(1.0 - eps),
                      (float)global_batch, as_stream(stream));
}

int pydtnn_hip_sgd_momentum(float* w, const float* dw, float* velocity, long total, float lr, float momentum,
                            float decay, int nesterov, void* stream)
{
    if (!w || !dw || !velocity) return PYDTNN_HIP_ERR_INVALID;
    return launch_sgd_momentum(w, dw, velocity, total, lr, momentum, decay, nesterov, as_stream(stream));
}

int pydtnn_hip_sgd_momentum_multi(int count, float* const* w, const float* const* dw, float* const* velocity,
                                  const long* total, float lr, float momentum, float decay, int nesterov, void* stream)
{
    return launch_sgd_momentum_multi(count, w, dw, velocity, total, lr, momentum, decay, nesterov, as_stream(stream));
}

}  // extern "C"

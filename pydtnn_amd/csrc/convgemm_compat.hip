// Host-pointer flavour of the convolution entry points, with the names and signatures of the
// external libconvGemm that PyDTNN binds through ctypes
// (pydtnn/backends/cpu/libs/conv_gemm.py:85-107).  Operands are copied to the GPU, the
// device-pointer entry points do the work, and the result is copied back.
//
// The reference hands over NumPy arrays, i.e. pageable host memory, and one synchronous copy of such memory runs
// at about 20 GB/s: 205 MB in and 205 MB out around a 1.8 ms kernel.  The calls here therefore work on groups of
// whole images and keep three things going at once: worker threads copy the next group from the caller's array
// into a pinned bounce buffer (and the group before last out of one), the DMA engines move the previous group's
// buffers, and the kernel of the group between runs on its own stream.  Forward and input gradient are independent
// per image; the filter gradient streams both of its inputs in the same way and then runs once over the whole
// batch, so that its sum has the order of the device-pointer call.
//
// The reference's ABI has no error channel (void functions).  A failure is reported on stderr, the call returns,
// and pydtnn_convgemm_last_status() tells: arguments are checked before anything is copied, so a rejected call
// leaves the output untouched.
#include "../../include/pydtnn_hip.h"
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

namespace {

std::atomic<int> g_last_status{PYDTNN_HIP_OK};

int fail(int status, const char* what, const char* detail)
{
    fprintf(stderr, "libconvGemm (pydtnn_hip): %s failed: %s\n", what, detail);
    g_last_status.store(status, std::memory_order_relaxed);
    return status;
}

#define HIP_TRY(expr, what)                                                                       \
    do {                                                                                          \
        const hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess) return fail(PYDTNN_HIP_ERR_LAUNCH, what, hipGetErrorString(e_));    \
    } while (0)
// a helper that has already reported its failure
#define PASS(expr)                                                                                \
    do {                                                                                          \
        const int rc_ = (expr);                                                                   \
        if (rc_ != PYDTNN_HIP_OK) return rc_;                                                     \
    } while (0)
#define RC_TRY(expr, what)                                                                        \
    do {                                                                                          \
        const int rc_ = (expr);                                                                   \
        if (rc_ != PYDTNN_HIP_OK) return fail(rc_, what, pydtnn_hip_status_string(rc_));          \
    } while (0)

// ---------------------------------------------------------------- host copies on worker threads
// One memcpy thread moves 10-15 GB/s; a handful of them keep up with the PCIe link.  The pool lives for the
// life of the process (its threads are never joined: they sleep between calls).
class CopyPool {
public:
    explicit CopyPool(int n)
    {
        for (int i = 0; i < n; ++i) std::thread([this] { run(); }).detach();
        workers_ = n;
    }
    // copies [src, src + bytes) to dst in pieces of at least 1 MiB, one per worker at most
    void submit(void* dst, const void* src, size_t bytes)
    {
        if (bytes == 0) return;
        size_t pieces = bytes / (1u << 20);
        pieces = pieces < 1 ? 1 : (pieces > (size_t)workers_ ? (size_t)workers_ : pieces);
        const size_t step = ((bytes + pieces - 1) / pieces + 63) & ~(size_t)63;
        std::lock_guard<std::mutex> hold(m_);
        for (size_t off = 0; off < bytes; off += step) {
            jobs_.push_back(Job{static_cast<char*>(dst) + off, static_cast<const char*>(src) + off,
                                bytes - off < step ? bytes - off : step});
            ++pending_;
        }
        cv_.notify_all();
    }
    void wait()
    {
        std::unique_lock<std::mutex> hold(m_);
        done_.wait(hold, [this] { return pending_ == 0; });
    }

private:
    struct Job {
        char* dst;
        const char* src;
        size_t n;
    };
    void run()
    {
        for (;;) {
            Job j;
            {
                std::unique_lock<std::mutex> hold(m_);
                cv_.wait(hold, [this] { return !jobs_.empty(); });
                j = jobs_.front();
                jobs_.pop_front();
            }
            memcpy(j.dst, j.src, j.n);
            std::lock_guard<std::mutex> hold(m_);
            if (--pending_ == 0) done_.notify_all();
        }
    }
    std::mutex m_;
    std::condition_variable cv_, done_;
    std::deque<Job> jobs_;
    int pending_ = 0;
    int workers_ = 0;
};

CopyPool& pool()
{
    static CopyPool* p = [] {
        int n = 8;
        if (const char* env = getenv("PYDTNN_CONVGEMM_COPY_THREADS")) n = atoi(env);
        const int hw = (int)std::thread::hardware_concurrency();
        if (hw > 0 && n > hw) n = hw;
        return new CopyPool(n < 1 ? 1 : n);
    }();
    return *p;
}

// ---------------------------------------------------------------- device and pinned buffers
// A grow-only cache, one slot per role, kept for the life of the process: a layer calls with the same shapes
// again and again.  The slots are never freed explicitly (at process exit the HIP runtime may already be gone
// when static destructors run; the driver reclaims the memory).  One call at a time: the reference calls from a
// single thread, but ctypes releases the GIL, so a mutex keeps two callers from sharing the slots.
enum Slot { SLOT_IN1, SLOT_X, SLOT_OUT, SLOT_WS, SLOT_BIAS, SLOT_MEAN, SLOT_ISTD, SLOT_GAMMA, SLOT_BETA, SLOT_COUNT };
enum Pinned { PIN_IN0, PIN_IN1, PIN_OUT0, PIN_OUT1, PIN_COUNT };

struct Cache {
    void* p[SLOT_COUNT] = {};
    size_t bytes[SLOT_COUNT] = {};
    void* pin[PIN_COUNT] = {};
    size_t pin_bytes[PIN_COUNT] = {};
    hipStream_t s_in = nullptr, s_run = nullptr, s_out = nullptr;
    hipEvent_t up[2] = {}, ran = nullptr, down[2] = {};
    int device = -1;
    std::mutex lock;
};
Cache g_cache;

int prepare_device()
{
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    if (dev == g_cache.device) return PYDTNN_HIP_OK;
    // buffers, streams and events belong to the device they were made on
    for (int i = 0; i < SLOT_COUNT; ++i) {
        if (g_cache.p[i]) (void)hipFree(g_cache.p[i]);
        g_cache.p[i] = nullptr;
        g_cache.bytes[i] = 0;
    }
    if (g_cache.s_in) {
        (void)hipStreamDestroy(g_cache.s_in); (void)hipStreamDestroy(g_cache.s_run); (void)hipStreamDestroy(g_cache.s_out);
        for (int i = 0; i < 2; ++i) { (void)hipEventDestroy(g_cache.up[i]); (void)hipEventDestroy(g_cache.down[i]); }
        (void)hipEventDestroy(g_cache.ran);
        g_cache.s_in = nullptr;
    }
    g_cache.device = -1;
    // three streams of the default priority: uploads, kernels, downloads
    HIP_TRY(hipStreamCreateWithFlags(&g_cache.s_in, hipStreamNonBlocking), "hipStreamCreate");
    HIP_TRY(hipStreamCreateWithFlags(&g_cache.s_run, hipStreamNonBlocking), "hipStreamCreate");
    HIP_TRY(hipStreamCreateWithFlags(&g_cache.s_out, hipStreamNonBlocking), "hipStreamCreate");
    for (int i = 0; i < 2; ++i) {
        HIP_TRY(hipEventCreateWithFlags(&g_cache.up[i], hipEventDisableTiming), "hipEventCreate");
        HIP_TRY(hipEventCreateWithFlags(&g_cache.down[i], hipEventDisableTiming), "hipEventCreate");
    }
    HIP_TRY(hipEventCreateWithFlags(&g_cache.ran, hipEventDisableTiming), "hipEventCreate");
    g_cache.device = dev;
    return PYDTNN_HIP_OK;
}

int slot(Slot s, size_t n, void** out)
{
    *out = nullptr;
    if (n == 0) return PYDTNN_HIP_OK;
    if (g_cache.bytes[s] < n) {
        if (g_cache.p[s]) HIP_TRY(hipFree(g_cache.p[s]), "hipFree");
        g_cache.p[s] = nullptr;
        g_cache.bytes[s] = 0;
        const size_t want = n + n / 8;  // a little head room: batch sizes wobble
        HIP_TRY(hipMalloc(&g_cache.p[s], want), "hipMalloc");
        g_cache.bytes[s] = want;
    }
    *out = g_cache.p[s];
    return PYDTNN_HIP_OK;
}

int pinned(Pinned s, size_t n, void** out)
{
    if (g_cache.pin_bytes[s] < n) {
        if (g_cache.pin[s]) HIP_TRY(hipHostFree(g_cache.pin[s]), "hipHostFree");
        g_cache.pin[s] = nullptr;
        g_cache.pin_bytes[s] = 0;
        HIP_TRY(hipHostMalloc(&g_cache.pin[s], n, hipHostMallocDefault), "hipHostMalloc");
        g_cache.pin_bytes[s] = n;
    }
    *out = g_cache.pin[s];
    return PYDTNN_HIP_OK;
}

// a per-channel vector (a few KB): one synchronous copy
int upload_small(Slot s, const void* src, size_t n, float** out)
{
    *out = nullptr;
    if (!src || n == 0) return PYDTNN_HIP_OK;
    void* d = nullptr;
    PASS(slot(s, n, &d));
    HIP_TRY(hipMemcpy(d, src, n, hipMemcpyHostToDevice), "hipMemcpy H2D");
    *out = static_cast<float*>(d);
    return PYDTNN_HIP_OK;
}

// Pieces of at most this many bytes travel through the bounce buffers (two per direction).
constexpr size_t kPieceBytes = (size_t)16 << 20;

// Streams a host array to the device in pieces: the workers fill one bounce buffer while the DMA engine drains
// the other.  Returns with the last piece enqueued on s_in (event up[] recorded after every piece).
int upload_streamed(const void* src, void* dst, size_t bytes, int* turn)
{
    for (size_t off = 0; off < bytes; off += kPieceBytes) {
        const size_t n = bytes - off < kPieceBytes ? bytes - off : kPieceBytes;
        const int b = (*turn)++ & 1;
        void* bounce = nullptr;
        PASS(pinned(b ? PIN_IN1 : PIN_IN0, kPieceBytes, &bounce));
        HIP_TRY(hipEventSynchronize(g_cache.up[b]), "hipEventSynchronize");   // its previous contents have left
        pool().submit(bounce, static_cast<const char*>(src) + off, n);
        pool().wait();
        HIP_TRY(hipMemcpyAsync(static_cast<char*>(dst) + off, bounce, n, hipMemcpyHostToDevice, g_cache.s_in),
                "hipMemcpyAsync H2D");
        HIP_TRY(hipEventRecord(g_cache.up[b], g_cache.s_in), "hipEventRecord");
    }
    return PYDTNN_HIP_OK;
}

inline size_t out_dim(size_t in, size_t pad, size_t dil, size_t k, size_t stride)
{
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

struct Geometry {
    unsigned b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation;
    size_t ho, wo;
};

// What the device entry points would refuse for its extents, refused here before anything is copied.
int check_geometry(Geometry* g, const char* what)
{
    if (!g->b || !g->c || !g->h || !g->w || !g->kn || !g->kh || !g->kw || !g->vstride || !g->hstride ||
        !g->vdilation || !g->hdilation)
        return fail(PYDTNN_HIP_ERR_INVALID, what, "an extent, stride or dilation of zero");
    if ((size_t)g->h + 2 * (size_t)g->vpadding < (size_t)g->vdilation * (g->kh - 1) + 1 ||
        (size_t)g->w + 2 * (size_t)g->hpadding < (size_t)g->hdilation * (g->kw - 1) + 1)
        return fail(PYDTNN_HIP_ERR_INVALID, what, "the filter does not fit the padded image");
    g->ho = out_dim(g->h, g->vpadding, g->vdilation, g->kh, g->vstride);
    g->wo = out_dim(g->w, g->hpadding, g->hdilation, g->kw, g->hstride);
    const size_t limit = (size_t)1 << 29;   // floats of one image that one launch can address
    if ((size_t)g->c * g->h * g->w >= limit || (size_t)g->kn * g->ho * g->wo >= limit ||
        (size_t)g->kn * g->c * g->kh * g->kw >= limit)
        return fail(PYDTNN_HIP_ERR_UNSUPPORTED, what, "one image or the filter exceeds 2^29 floats");
    return PYDTNN_HIP_OK;
}

size_t workspace_bytes(int op, int nhwc, const Geometry& g, unsigned b)
{
    return pydtnn_hip_conv_workspace_bytes(op, nhwc, (int)b, (int)g.c, (int)g.h, (int)g.w, (int)g.kn, (int)g.kh,
                                           (int)g.kw, (int)g.vpadding, (int)g.hpadding, (int)g.vstride,
                                           (int)g.hstride, (int)g.vdilation, (int)g.hdilation);
}

// Images per group: about kPieceBytes of the larger of the two per-image tensors, at least one image.
unsigned images_per_group(const Geometry& g, size_t in_per_image, size_t out_per_image)
{
    const size_t big = (in_per_image > out_per_image ? in_per_image : out_per_image) * 4;
    size_t n = kPieceBytes / (big ? big : 1);
    n = n < 1 ? 1 : n;
    return (unsigned)(n > g.b ? g.b : n);
}

// `launch(first image, images)` enqueues the kernels of one group on s_run.  `in` (in_per_image floats per image)
// is streamed up group by group and `out` (out_per_image floats per image) comes back the same way, in lockstep:
// step t copies group t into a bounce buffer and group t - 2 out of one on the worker threads, then enqueues
// upload, kernels and download of group t, each waiting for the one before.
template <class Launch>
int pipelined(const Geometry& g, const float* in, float* d_in, size_t in_per_image, float* out, float* d_out,
              size_t out_per_image, Launch launch)
{
    const unsigned per = images_per_group(g, in_per_image, out_per_image);
    const unsigned groups = (g.b + per - 1) / per;
    const size_t in_bounce = (size_t)per * in_per_image * 4, out_bounce = (size_t)per * out_per_image * 4;
    void *bin[2], *bout[2];
    PASS(pinned(PIN_IN0, in_bounce > kPieceBytes ? in_bounce : kPieceBytes, &bin[0]));
    PASS(pinned(PIN_IN1, in_bounce > kPieceBytes ? in_bounce : kPieceBytes, &bin[1]));
    PASS(pinned(PIN_OUT0, out_bounce, &bout[0]));
    PASS(pinned(PIN_OUT1, out_bounce, &bout[1]));
    auto first = [&](unsigned grp) { return (size_t)grp * per; };
    auto count = [&](unsigned grp) { return (size_t)(g.b - first(grp) < per ? g.b - first(grp) : per); };
    for (unsigned t = 0; t < groups + 2; ++t) {
        const int b = t & 1;
        if (t < groups) {
            HIP_TRY(hipEventSynchronize(g_cache.up[b]), "hipEventSynchronize");   // bounce buffer b has been uploaded
            pool().submit(bin[b], in + first(t) * in_per_image, count(t) * in_per_image * 4);
        }
        if (t >= 2) {
            HIP_TRY(hipEventSynchronize(g_cache.down[b]), "hipEventSynchronize");  // group t - 2 has arrived
            pool().submit(out + first(t - 2) * out_per_image, bout[b], count(t - 2) * out_per_image * 4);
        }
        pool().wait();
        if (t >= groups) continue;
        HIP_TRY(hipMemcpyAsync(d_in + first(t) * in_per_image, bin[b], count(t) * in_per_image * 4,
                               hipMemcpyHostToDevice, g_cache.s_in), "hipMemcpyAsync H2D");
        HIP_TRY(hipEventRecord(g_cache.up[b], g_cache.s_in), "hipEventRecord");
        HIP_TRY(hipStreamWaitEvent(g_cache.s_run, g_cache.up[b], 0), "hipStreamWaitEvent");
        RC_TRY(launch(first(t), count(t)), "convolution");
        HIP_TRY(hipEventRecord(g_cache.ran, g_cache.s_run), "hipEventRecord");
        HIP_TRY(hipStreamWaitEvent(g_cache.s_out, g_cache.ran, 0), "hipStreamWaitEvent");
        HIP_TRY(hipMemcpyAsync(bout[b], d_out + first(t) * out_per_image, count(t) * out_per_image * 4,
                               hipMemcpyDeviceToHost, g_cache.s_out), "hipMemcpyAsync D2H");
        HIP_TRY(hipEventRecord(g_cache.down[b], g_cache.s_out), "hipEventRecord");
    }
    return PYDTNN_HIP_OK;
}

// After a failure in the middle of a call nothing may still be in flight when the caller's arrays go away.
void drain()
{
    pool().wait();
    if (g_cache.s_in) {
        (void)hipStreamSynchronize(g_cache.s_in);
        (void)hipStreamSynchronize(g_cache.s_run);
        (void)hipStreamSynchronize(g_cache.s_out);
    }
}

int conv_host(int nhwc, char trans, Geometry g, const float* in1, const float* x, float* out,
              const float* bias_vector, const float* mean, const float* inv_std, const float* gamma,
              const float* beta, bool relu)
{
    const char* what = nhwc ? "sconvGemmNHWC" : "sconvGemmNCHW";
    if (trans != 'N' && trans != 'Y') return fail(PYDTNN_HIP_ERR_INVALID, what, "trans must be 'N' or 'Y'");
    if (!in1 || !x || !out) return fail(PYDTNN_HIP_ERR_INVALID, what, "a null operand");
    const int set = (mean != nullptr) + (inv_std != nullptr) + (gamma != nullptr) + (beta != nullptr);
    if (set != 0 && set != 4) return fail(PYDTNN_HIP_ERR_INVALID, what, "the four BN vectors come together");
    PASS(check_geometry(&g, what));
    const size_t x_img = (size_t)g.c * g.h * g.w, y_img = (size_t)g.kn * g.ho * g.wo;
    const size_t w_elems = (size_t)g.kn * g.c * g.kh * g.kw;
    const bool fwd = trans == 'N';
    std::lock_guard<std::mutex> hold(g_cache.lock);
    PASS(prepare_device());
    void *d_x = nullptr, *d_in1 = nullptr, *d_out = nullptr, *d_ws = nullptr;
    PASS(slot(SLOT_X, g.b * x_img * 4, &d_x));
    PASS(slot(SLOT_IN1, (fwd ? w_elems : g.b * y_img) * 4, &d_in1));
    PASS(slot(SLOT_OUT, (fwd ? g.b * y_img : w_elems) * 4, &d_out));
    const size_t vec = (size_t)g.kn * 4;
    float *d_bias, *d_mean, *d_istd, *d_gamma, *d_beta;
    PASS(upload_small(SLOT_BIAS, bias_vector, vec, &d_bias));
    PASS(upload_small(SLOT_MEAN, mean, vec, &d_mean));
    PASS(upload_small(SLOT_ISTD, inv_std, vec, &d_istd));
    PASS(upload_small(SLOT_GAMMA, gamma, vec, &d_gamma));
    PASS(upload_small(SLOT_BETA, beta, vec, &d_beta));
    auto run = [&](const float* a, const float* xs, float* o, unsigned images, void* ws, size_t ws_bytes) {
        return nhwc ? pydtnn_hip_sconvGemmNHWC(trans, images, g.h, g.w, g.c, g.kn, g.kh, g.kw, g.vpadding, g.hpadding,
                                               g.vstride, g.hstride, g.vdilation, g.hdilation, a, xs, o, d_bias, d_mean,
                                               d_istd, d_gamma, d_beta, relu, ws, ws_bytes, g_cache.s_run)
                    : pydtnn_hip_sconvGemmNCHW(trans, images, g.c, g.h, g.w, g.kn, g.kh, g.kw, g.vpadding, g.hpadding,
                                               g.vstride, g.hstride, g.vdilation, g.hdilation, a, xs, o, d_bias, d_mean,
                                               d_istd, d_gamma, d_beta, relu, ws, ws_bytes, g_cache.s_run);
    };
    int rc;
    if (fwd) {
        // the filter first (small), then x in and y out group by group
        HIP_TRY(hipMemcpy(d_in1, in1, w_elems * 4, hipMemcpyHostToDevice), "hipMemcpy H2D");
        const unsigned per = images_per_group(g, x_img, y_img);
        const size_t ws_bytes = workspace_bytes(PYDTNN_HIP_OP_FWD, nhwc, g, per);
        PASS(slot(SLOT_WS, ws_bytes, &d_ws));
        rc = pipelined(g, x, static_cast<float*>(d_x), x_img, out, static_cast<float*>(d_out), y_img,
                       [&](size_t n0, size_t images) {
                           return run(static_cast<const float*>(d_in1), static_cast<const float*>(d_x) + n0 * x_img,
                                      static_cast<float*>(d_out) + n0 * y_img, (unsigned)images, d_ws, ws_bytes);
                       });
    } else {
        // both inputs stream up, then one launch over the whole batch (the sum keeps the order of the
        // device-pointer call) and a small copy back
        const size_t ws_bytes = workspace_bytes(PYDTNN_HIP_OP_DW, nhwc, g, g.b);
        PASS(slot(SLOT_WS, ws_bytes, &d_ws));
        auto filter_gradient = [&]() -> int {
            int turn = 0;
            PASS(upload_streamed(in1, d_in1, g.b * y_img * 4, &turn));
            PASS(upload_streamed(x, d_x, g.b * x_img * 4, &turn));
            HIP_TRY(hipStreamSynchronize(g_cache.s_in), "hipStreamSynchronize");
            RC_TRY(run(static_cast<const float*>(d_in1), static_cast<const float*>(d_x), static_cast<float*>(d_out), g.b,
                       d_ws, ws_bytes), what);
            HIP_TRY(hipMemcpyAsync(out, d_out, w_elems * 4, hipMemcpyDeviceToHost, g_cache.s_run), "hipMemcpyAsync D2H");
            HIP_TRY(hipStreamSynchronize(g_cache.s_run), "hipStreamSynchronize");
            return PYDTNN_HIP_OK;
        };
        rc = filter_gradient();
    }
    if (rc != PYDTNN_HIP_OK) drain();
    return rc;
}

int deconv_host(int nhwc, Geometry g, const float* weights, const float* dy, float* dx)
{
    const char* what = nhwc ? "sconvGemmNHWC_back" : "sconvGemmNCHW_back";
    if (!weights || !dy || !dx) return fail(PYDTNN_HIP_ERR_INVALID, what, "a null operand");
    PASS(check_geometry(&g, what));
    const size_t x_img = (size_t)g.c * g.h * g.w, y_img = (size_t)g.kn * g.ho * g.wo;
    const size_t w_elems = (size_t)g.kn * g.c * g.kh * g.kw;
    std::lock_guard<std::mutex> hold(g_cache.lock);
    PASS(prepare_device());
    void *d_w = nullptr, *d_dy = nullptr, *d_dx = nullptr, *d_ws = nullptr;
    PASS(slot(SLOT_IN1, w_elems * 4, &d_w));
    PASS(slot(SLOT_X, g.b * y_img * 4, &d_dy));
    PASS(slot(SLOT_OUT, g.b * x_img * 4, &d_dx));
    HIP_TRY(hipMemcpy(d_w, weights, w_elems * 4, hipMemcpyHostToDevice), "hipMemcpy H2D");
    const unsigned per = images_per_group(g, y_img, x_img);
    const size_t ws_bytes = workspace_bytes(PYDTNN_HIP_OP_DX, nhwc, g, per);
    PASS(slot(SLOT_WS, ws_bytes, &d_ws));
    const int rc = pipelined(
        g, dy, static_cast<float*>(d_dy), y_img, dx, static_cast<float*>(d_dx), x_img, [&](size_t n0, size_t images) {
            const float* dyg = static_cast<const float*>(d_dy) + n0 * y_img;
            float* dxg = static_cast<float*>(d_dx) + n0 * x_img;
            return nhwc ? pydtnn_hip_sconvGemmNHWC_back((unsigned)images, g.h, g.w, g.c, g.kn, g.kh, g.kw, g.vstride,
                                                        g.hstride, g.vpadding, g.hpadding, g.vdilation, g.hdilation,
                                                        static_cast<const float*>(d_w), dyg, dxg, d_ws, ws_bytes,
                                                        g_cache.s_run)
                        : pydtnn_hip_sconvGemmNCHW_back((unsigned)images, g.c, g.h, g.w, g.kn, g.kh, g.kw, g.vstride,
                                                        g.hstride, g.vpadding, g.hpadding, g.vdilation, g.hdilation,
                                                        static_cast<const float*>(d_w), dyg, dxg, d_ws, ws_bytes,
                                                        g_cache.s_run);
        });
    if (rc != PYDTNN_HIP_OK) drain();
    return rc;
}

}  // namespace

extern "C" {

int pydtnn_convgemm_last_status(void) { return g_last_status.load(std::memory_order_relaxed); }

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

#define GEOMETRY Geometry{b, c, h, w, kn, kh, kw, vpadding, hpadding, vstride, hstride, vdilation, hdilation, 0, 0}

void sconvGemmNCHW(char trans, unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float* in1, const float* x, float* out, const float* bias_vector,
                   const float* bn_running_mean, const float* bn_inv_std, const float* bn_gamma,
                   const float* bn_beta, bool relu, float* /*ac_pack*/, float* /*bc_pack*/)
{
    g_last_status.store(PYDTNN_HIP_OK, std::memory_order_relaxed);
    (void)conv_host(0, trans, GEOMETRY, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu);
}

void sconvGemmNHWC(char trans, unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                   unsigned vpadding, unsigned hpadding, unsigned vstride, unsigned hstride, unsigned vdilation,
                   unsigned hdilation, const float* in1, const float* x, float* out, const float* bias_vector,
                   const float* bn_running_mean, const float* bn_inv_std, const float* bn_gamma,
                   const float* bn_beta, bool relu, float* /*ac_pack*/, float* /*bc_pack*/)
{
    g_last_status.store(PYDTNN_HIP_OK, std::memory_order_relaxed);
    (void)conv_host(1, trans, GEOMETRY, in1, x, out, bias_vector, bn_running_mean, bn_inv_std, bn_gamma, bn_beta, relu);
}

void sconvGemmNCHW_back(unsigned b, unsigned c, unsigned h, unsigned w, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float* weights, const float* dy, float* dx, float* /*ac_pack*/,
                        float* /*bc_pack*/)
{
    g_last_status.store(PYDTNN_HIP_OK, std::memory_order_relaxed);
    (void)deconv_host(0, GEOMETRY, weights, dy, dx);
}

void sconvGemmNHWC_back(unsigned b, unsigned h, unsigned w, unsigned c, unsigned kn, unsigned kh, unsigned kw,
                        unsigned vstride, unsigned hstride, unsigned vpadding, unsigned hpadding, unsigned vdilation,
                        unsigned hdilation, const float* weights, const float* dy, float* dx, float* /*ac_pack*/,
                        float* /*bc_pack*/)
{
    g_last_status.store(PYDTNN_HIP_OK, std::memory_order_relaxed);
    (void)deconv_host(1, GEOMETRY, weights, dy, dx);
}

}  // extern "C"

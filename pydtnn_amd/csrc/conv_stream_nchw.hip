// Forward convolutions whose whole filter matrix fits LDS and whose reduction is short (the first layer of a
// network: few input channels, any filter size and stride), as a streaming kernel; written for NCHW, with NHWC as a
// variant of the offset tables and the store.
//
// On the tile engine such a layer is tiles of 2 to 23 reduction steps: filling the pipeline and storing the tile
// take as long as the steps between them, and every workgroup does so at the same time.  Here, as in the NHWC
// streaming kernel, nothing is tiled through LDS and there is no barrier after set-up:
//   * one workgroup per compute unit keeps the filter matrix in LDS for its lifetime, laid out so that one
//     128-bit LDS read is the A operand (filter rows) of four MFMAs;
//   * a wavefront owns a unit of 32 consecutive output pixels of one image x all filters.  The B operand of
//     v_mfma_f32_32x32x2_f32 wants pixel l%32 and reduction index l/32 in lane l: lane (p, h) loads
//     x[image][c][sv*oy + dv*i][sh*ox + dh*j] for the taps (c, i, j) of parity class h straight from memory into
//     the registers the MFMAs read, one 32-bit load per tap at the lane's pixel offset plus the tap's offset
//     (a table in LDS, read four taps at a time);
//   * the reduction axis is cut into chunks of 8 MFMA steps (16 taps); a unit is straight-line code over its
//     chunks, and while the MFMAs of a chunk run the loads of the next chunk (or of the first chunk of the
//     wavefront's next unit) are in flight.  Every path issues the same memory instructions (a prefetch without a
//     next unit, the pixels beyond the end of an image and the taps beyond the reduction length are aimed beyond
//     the descriptor and read as zero), so the waits the compiler places are exact counts;
//   * accumulator rows are filters and columns pixels, so a store instruction writes two runs of 32 consecutive
//     pixels of y; bias -> BN -> ReLU are applied on the way, optionally with the int8 ReLU mask.
// Units are dealt to the wavefronts of a workgroup from a counter in LDS; which wavefront computes a unit does
// not change a bit of it.
#include "conv_internal.h"
#include <type_traits>

namespace convint {

namespace {

constexpr uint32_t kDead = 0x40000000u;      // byte offset beyond every descriptor this kernel builds (< 1 GiB)

struct StreamNchwArgs {
    const float* x;
    const float* w;
    float* y;
    ConvGeom g;
    ChanEpilogue chan;
    ElemMasks masks;
    int units_per_image;  // ceil(howo / 32)
    int units;            // n * units_per_image
};

typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));

// MB: filters / 32;  CHUNKS: chunks of 16 reduction indices (kh*kw*c rounded up);  WAVES: wavefronts of the
// workgroup, 12 (168 registers) or 16 (128 registers; same code, no spills).
// NHWC: x is (n, h, w, c), the filter (c, kh, kw, kn) and y (n, ho, wo, kn); the taps keep their (c, i, j) order.
template <int MB, int CHUNKS, int MASKS, int WAVES, bool PAD, bool NHWC>
__global__ void __launch_bounds__(64 * WAVES) conv_stream_nchw_kernel(StreamNchwArgs a)
{
    constexpr int KN = 32 * MB, GROUPS = CHUNKS * 2, SLOTS = CHUNKS * 16;
    constexpr int kWaves = WAVES, kThreadsNchw = 64 * WAVES;
    extern __shared__ __align__(16) float lds[];
    const ConvGeom& g = a.g;
    // filter: quad [(group*2 + h)*KN + f] holds w[f][tap 2*(4*group + i) + h], i = 0..3
    floatx4* wl = reinterpret_cast<floatx4*>(lds);
    // tap offsets in bytes: quad [group*2 + h] holds those of the same four taps
    uintx4* toff = reinterpret_cast<uintx4*>(lds + (size_t)GROUPS * 2 * KN * 4);
    // with padding: the taps' row / column bits (1 << i) | (1 << (16 + j)), laid out like the offsets
    [[maybe_unused]] uintx4* tbits = toff + GROUPS * 2;
    float* params = lds + (size_t)GROUPS * 2 * KN * 4 + GROUPS * 2 * 4 * 2;  // [5][KN]
    int* counter = reinterpret_cast<int*>(params + 5 * KN);

    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6);
    const int lp = lane & 31, lh = lane >> 5;

    // this workgroup's range of units
    const int u0 = (int)((long)blockIdx.x * a.units / gridDim.x);
    const int u1 = (int)((long)(blockIdx.x + 1) * a.units / gridDim.x);
    const int units = u1 - u0;

    // ---- set-up
    {
        float* wf = lds;
        constexpr int kBatch = 8;  // loads in flight per thread
        for (int e0 = 0; e0 < KN * SLOTS; e0 += kThreadsNchw * kBatch) {
            float v[kBatch];
            int dst[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int e = e0 + u * kThreadsNchw + tid;
                // consecutive threads walk along the tensor's contiguous axis: taps in NCHW, filters in NHWC
                const int f = NHWC ? e % KN : e / SLOTS, s = NHWC ? e / KN : e - f * SLOTS;
                const bool real = e < KN * SLOTS && s < g.k;
                v[u] = a.w[real ? (NHWC ? (size_t)s * KN + f : (size_t)f * g.k + s) : 0];
                if (!real) v[u] = 0.0f;
                const int m = s >> 1, h = s & 1;
                dst[u] = e < KN * SLOTS ? (((m >> 2) * 2 + h) * KN + f) * 4 + (m & 3) : -1;
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (dst[u] >= 0) wf[dst[u]] = v[u];
        }
        uint32_t* tf = reinterpret_cast<uint32_t*>(toff);
        for (int s = tid; s < SLOTS; s += kThreadsNchw) {
            uint32_t off = kOob, bits = 0;
            if (s < g.k) {
                const int cc = (int)fd_div((uint32_t)s, g.fd_khw), rem = s - cc * g.khw;
                const int ti = (int)fd_div((uint32_t)rem, g.fd_kw), tj = rem - ti * g.kw;
                off = NHWC ? (uint32_t)(((long)ti * g.vdilation * g.w + tj * g.hdilation) * g.c + cc) * 4u
                           : (uint32_t)(((long)cc * g.h + ti * g.vdilation) * g.w + tj * g.hdilation) * 4u;
                bits = (1u << ti) | (1u << (16 + tj));
            }
            const int m = s >> 1, h = s & 1;
            tf[((m >> 2) * 2 + h) * 4 + (m & 3)] = off;
            if constexpr (PAD) tf[GROUPS * 2 * 4 + ((m >> 2) * 2 + h) * 4 + (m & 3)] = bits;
        }
        for (int i = tid; i < KN; i += kThreadsNchw) {
            params[i] = a.chan.bias ? a.chan.bias[i] : 0.0f;
            params[KN + i] = a.chan.mean ? a.chan.mean[i] : 0.0f;
            params[2 * KN + i] = a.chan.mean ? a.chan.inv_std[i] : 1.0f;
            params[3 * KN + i] = a.chan.mean ? a.chan.gamma[i] : 1.0f;
            params[4 * KN + i] = a.chan.mean ? a.chan.beta[i] : 0.0f;
        }
        if (tid == 0) *counter = kWaves;  // the first unit of each wavefront is its own index
    }
    __syncthreads();

    const long x_floats = (long)g.n * g.c * g.h * g.w;
    const rsrc_t x_rsrc = make_rsrc(a.x, x_floats);
    const long y_floats = g.p * KN;
    const rsrc_t y_rsrc = make_rsrc(a.y, y_floats);
    [[maybe_unused]] rsrc_t mask_rsrc;
    if constexpr (MASKS == kReluMask) mask_rsrc = make_rsrc_bytes(a.masks.relu_mask, y_floats);

    // Per-lane data of a unit.  Without padding: `base` is the byte offset of the lane's pixel at tap (0, 0, 0), or
    // kDead when the plane ends before it.  With padding: the same offset (which may be "negative", i.e. wrap), and
    // `bad` holds bit i for every filter row i and bit 16 + j for every filter column j that falls outside the
    // image for this pixel (all ones beyond the end of the plane): a tap is read when bad & its bits == 0.
    struct Lane {
        uint32_t base;
        uint32_t bad;
    };
    auto pixel_lane = [&](int unit) __attribute__((always_inline)) -> Lane {
        const int gu = u0 + unit;
        const int img = gu / a.units_per_image;
        const int p = (gu - img * a.units_per_image) * 32 + lp;
        const uint32_t oy = fd_div((uint32_t)p, g.fd_wo), ox = (uint32_t)p - oy * (uint32_t)g.wo;
        const int ih0 = (int)oy * g.vstride - g.vpadding, iw0 = (int)ox * g.hstride - g.hpadding;
        Lane l;
        l.base = NHWC ? (uint32_t)((((long)img * g.h + ih0) * g.w + iw0) * g.c) * 4u
                      : (uint32_t)(((long)img * g.c * g.h + ih0) * g.w + iw0) * 4u;
        l.bad = 0;
        if constexpr (PAD) {
            for (int t = 0; t < g.kh; ++t)
                if ((unsigned)(ih0 + t * g.vdilation) >= (unsigned)g.h) l.bad |= 1u << t;
            for (int t = 0; t < g.kw; ++t)
                if ((unsigned)(iw0 + t * g.hdilation) >= (unsigned)g.w) l.bad |= 1u << (16 + t);
            if (p >= g.howo) l.bad = 0xffffffffu;
        } else {
            if (p >= g.howo) l.base = kDead;
        }
        return l;
    };
    const Lane dead_lane = {kDead, 0xffffffffu};
    auto load_chunk = [&](const Lane& l, int chunk, float (&r)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
            const uintx4 t = toff[(chunk * 2 + gg) * 2 + lh];
            [[maybe_unused]] uintx4 tb;
            if constexpr (PAD) tb = tbits[(chunk * 2 + gg) * 2 + lh];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t voff = l.base + t[i];
                // a reduction slot beyond the last tap has no bits and the offset kOob, which stays beyond the
                // descriptor for every base (|base| < 2^30)
                if constexpr (PAD) voff = (l.bad & tb[i]) != 0 ? kOob : voff;
                r[gg * 4 + i] = buf_load(x_rsrc, voff, 0);
            }
        }
    };
    auto claim = [&]() __attribute__((always_inline)) -> int {
        int u = 0;
        if (lane == 0) u = atomicAdd(counter, 1);
        u = uniform(u);
        return u < units ? u : -1;
    };
    auto relu_of = [](float v) __attribute__((always_inline)) {
        float r;
        asm("v_max_f32 %0, 0, %1" : "=v"(r) : "v"(v));
        return r;
    };
    constexpr int kEpiBias = 1, kEpiBn = 2, kEpiRelu = 4;
    const int epi_flags = (a.chan.bias ? kEpiBias : 0) | (a.chan.mean ? kEpiBn : 0) | (a.chan.relu ? kEpiRelu : 0);

    auto store_unit = [&](auto flags_tag, const floatx16 (&ac)[MB], int unit) __attribute__((always_inline)) {
        constexpr int F = decltype(flags_tag)::value;
        const int gu = u0 + unit;
        const int img = gu / a.units_per_image;
        const int p0 = (gu - img * a.units_per_image) * 32;
        // lane (p, h) holds filters 32*mb + 8*(v/4) + 4*h + v%4 of pixel p0 + p
        const float* pl = params + 4 * lh;
        if constexpr (NHWC) {
            // a lane's registers 4q .. 4q+3 are four consecutive filters of its pixel: stored as two pairs, and the
            // mask bytes of the four as one word
            const uint32_t e4 = p0 + lp < g.howo ? (uint32_t)(lp * KN + 4 * lh) : kDead;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int f = 32 * mb + 8 * q;
                    const uint32_t soff = (uint32_t)(((long)img * g.howo + p0) * KN + f);
                    uintx4 out;
                    uint32_t bytes = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float val = ac[mb][4 * q + i];
                        if constexpr ((F & kEpiBias) != 0) val += pl[f + i];
                        if constexpr ((F & kEpiBn) != 0) {
                            const float t = (val - pl[KN + f + i]) * pl[2 * KN + f + i];
                            val = t * pl[3 * KN + f + i] + pl[4 * KN + f + i];
                        }
                        if constexpr ((F & kEpiRelu) != 0) val = val > 0.0f ? val : 0.0f;
                        out[i] = __builtin_bit_cast(uint32_t, val);
                        bytes |= (val > 0.0f ? 1u : 0u) << (8 * i);
                    }
                    // two 64-bit stores: a 128-bit buffer store with a register offset, followed at once by an
                    // instruction that overwrites its data registers, stored the new values for some lanes on this
                    // part (the compiler inserts the wait state only for a constant offset)
                    typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));
                    const uintx2 lo = {out[0], out[1]}, hi = {out[2], out[3]};
                    const int voff = (int)(e4 == kDead ? kOob : e4 * 4u);
                    __builtin_amdgcn_raw_buffer_store_b64(lo, y_rsrc, voff, (int)(soff * 4u), 0);
                    __builtin_amdgcn_raw_buffer_store_b64(hi, y_rsrc, voff, (int)(soff * 4u + 8u), 0);
                    if constexpr (MASKS == kReluMask)
                        __builtin_amdgcn_raw_buffer_store_b32(bytes, mask_rsrc, (int)(e4 == kDead ? kOob : e4),
                                                              (int)soff, 0);
                }
            return;
        }
        const uint32_t e = p0 + lp < g.howo ? (uint32_t)(4 * lh * g.howo + lp) : kDead;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int f = 32 * mb + 8 * (v / 4) + (v % 4);
                const uint32_t soff = (uint32_t)(((long)img * KN + f) * g.howo + p0);
                float val = ac[mb][v];
                if constexpr ((F & kEpiBias) != 0) val += pl[f];
                if constexpr ((F & kEpiBn) != 0) {
                    const float t = (val - pl[KN + f]) * pl[2 * KN + f];
                    val = t * pl[3 * KN + f] + pl[4 * KN + f];
                }
                if constexpr ((F & kEpiRelu) != 0) val = relu_of(val);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), y_rsrc,
                                                      (int)(e == kDead ? kOob : e * 4u), (int)(soff * 4u), 0);
                if constexpr (MASKS == kReluMask)
                    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(val > 0.0f ? 1 : 0), mask_rsrc,
                                                         (int)(e == kDead ? kOob : e), (int)soff, 0);
            }
    };

    float bbuf[2][8];
    floatx16 acc[MB];
    int cur = wave < units ? wave : -1;
    if (cur < 0) return;
    Lane ln = pixel_lane(cur);
    load_chunk(ln, 0, bbuf[0]);
    const floatx4* wq0 = wl + (size_t)lh * KN + lp;

    // One unit, straight-line: chunk ch is consumed from bbuf[(P0 + ch) & 1] while the next chunk (of this unit, or
    // the first of the wavefront's next unit) is in flight into the other buffer.
    auto unit_body = [&](auto parity_tag) __attribute__((always_inline)) {
        constexpr int P0 = decltype(parity_tag)::value;
        const int next = claim();
        const Lane ln_next = next >= 0 ? pixel_lane(next) : dead_lane;
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) {
            const int B = (P0 + ch) & 1;
            if (ch + 1 < CHUNKS)
                load_chunk(ln, ch + 1, bbuf[B ^ 1]);
            else
                load_chunk(ln_next, 0, bbuf[B ^ 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int gg = 0; gg < 2; ++gg) {
                const floatx4* wq = wq0 + (size_t)((ch * 2 + gg) * 2) * KN;
                floatx4 aq[MB];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) aq[mb] = wq[32 * mb];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const floatx16 zero = {};
                        acc[mb] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            aq[mb][i], bbuf[B][gg * 4 + i], ch == 0 && gg == 0 && i == 0 ? zero : acc[mb], 0, 0, 0);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        switch (epi_flags) {
        case 0: store_unit(std::integral_constant<int, 0>{}, acc, cur); break;
        case 1: store_unit(std::integral_constant<int, 1>{}, acc, cur); break;
        case 2: store_unit(std::integral_constant<int, 2>{}, acc, cur); break;
        case 3: store_unit(std::integral_constant<int, 3>{}, acc, cur); break;
        case 4: store_unit(std::integral_constant<int, 4>{}, acc, cur); break;
        case 5: store_unit(std::integral_constant<int, 5>{}, acc, cur); break;
        case 6: store_unit(std::integral_constant<int, 6>{}, acc, cur); break;
        default: store_unit(std::integral_constant<int, 7>{}, acc, cur); break;
        }
        ln = ln_next;
        cur = next;
    };

    if constexpr (CHUNKS % 2 == 0) {
        while (cur >= 0) unit_body(std::integral_constant<int, 0>{});
    } else {
        for (;;) {
            unit_body(std::integral_constant<int, 0>{});
            if (cur < 0) break;
            unit_body(std::integral_constant<int, 1>{});
            if (cur < 0) break;
        }
    }
}

template <int MB, int CHUNKS>
constexpr size_t stream_nchw_lds_bytes()
{
    return ((size_t)CHUNKS * 2 * 2 * 32 * MB * 4 + CHUNKS * 2 * 2 * 4 * 2 + 5 * 32 * MB) * 4 + 16;
}

template <int MB, int CHUNKS, int MASKS, int WAVES, bool PAD, bool NHWC>
int launch_stream_nchw_waves(const StreamNchwArgs& a, int grid, hipStream_t stream)
{
    static std::atomic<unsigned> raised{0};
    constexpr size_t lds_bytes = stream_nchw_lds_bytes<MB, CHUNKS>();
    static_assert(lds_bytes <= 160 * 1024, "filter matrix must fit LDS");
    auto kernel = conv_stream_nchw_kernel<MB, CHUNKS, MASKS, WAVES, PAD, NHWC>;
    const int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), raised, 160 * 1024);
    if (rc != PYDTNN_HIP_OK) return rc;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * WAVES), lds_bytes, stream, a);
    HIP_RETURN_IF_LAUNCH_FAILED();
    note_launch(kLaunchStreamNchw, MB, 32, grid, 0, 1);
    return PYDTNN_HIP_OK;
}

template <int MB, int CHUNKS, int MASKS, bool PAD, bool NHWC>
int launch_stream_nchw(const StreamNchwArgs& a, hipStream_t stream)
{
    int cus = 0;
    const int rc = device_compute_units(&cus);
    if (rc != PYDTNN_HIP_OK) return rc;
    const int grid = a.units < cus ? a.units : cus;
    // A workgroup's units are taken by its wavefronts in rounds: sixteen wavefronts unless twelve leave fewer
    // idle slots in the last round (24 units: two full rounds of 12, but 32 slots of 16).
    const int per_wg = (a.units + grid - 1) / grid;
    const int slots16 = (per_wg + 15) / 16 * 16, slots12 = (per_wg + 11) / 12 * 12;
    if (slots12 < slots16) return launch_stream_nchw_waves<MB, CHUNKS, MASKS, 12, PAD, NHWC>(a, grid, stream);
    return launch_stream_nchw_waves<MB, CHUNKS, MASKS, 16, PAD, NHWC>(a, grid, stream);
}

// The (format, filters, chunks of 16 reduction indices, padded?) combinations that are built.  NCHW: AlexNet's first
// layer (96 filters, 3 x 11 x 11 = 363 taps, no padding), VGG's (64 filters, 3 x 3 x 3 = 27 taps, padded) and
// ResNet's (64 filters, 3 x 7 x 7 = 147 taps, padded).  NHWC: VGG's and ResNet's, and 32 filters over at most 16
// taps (a 3 x 3 layer on one channel).
bool stream_first_shape_built(int nhwc, int kn, int k, bool padded)
{
    const int chunks = (k + 15) / 16;
    if (nhwc) return padded && ((kn == 64 && (chunks == 2 || chunks == 10)) || (kn == 32 && chunks == 1));
    if (!padded) return kn == 96 && chunks == 23;
    return kn == 64 && (chunks == 2 || chunks == 10);
}

}  // namespace

bool conv_stream_first_eligible(int nhwc, const ConvGeom& g, const ElemMasks& masks)
{
    const bool padded = g.vpadding != 0 || g.hpadding != 0;
    if (!stream_first_shape_built(nhwc, g.kn, g.k, padded)) return false;
    if (padded && (g.kh > 16 || g.kw > 16)) return false;  // row and column bits share one word
    const int mk = mask_kind(masks);
    if (mk != kNoMasks && mk != kReluMask) return false;
    if (g.p < 32 * 1024) return false;                      // enough units for every compute unit
    // every byte offset the kernel forms stays below 2^30 in magnitude, and so do the descriptors
    const long reach = (long)g.n * g.c * g.h * g.w + (((long)g.vpadding + 1) * g.w + g.hpadding) * (nhwc ? g.c : 1);
    return reach < (1l << 28) && g.p * g.kn < (1l << 28);
}

int conv_stream_first(int nhwc, const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                      hipStream_t stream, const ElemMasks& masks)
{
    StreamNchwArgs a;
    a.x = x; a.w = w; a.y = y; a.g = g; a.chan = chan; a.masks = masks;
    a.units_per_image = (g.howo + 31) / 32;
    a.units = g.n * a.units_per_image;
    const int chunks = (g.k + 15) / 16;
    const bool mask = mask_kind(masks) == kReluMask;
    const bool padded = g.vpadding != 0 || g.hpadding != 0;
#define STREAM_FIRST_CASE(FMT, KN, CH, PAD)                                                        \
    if ((nhwc != 0) == FMT && g.kn == KN && chunks == CH && padded == PAD)                         \
        return mask ? launch_stream_nchw<KN / 32, CH, kReluMask, PAD, FMT>(a, stream)              \
                    : launch_stream_nchw<KN / 32, CH, kNoMasks, PAD, FMT>(a, stream)
    STREAM_FIRST_CASE(false, 96, 23, false);
    STREAM_FIRST_CASE(false, 64, 2, true);
    STREAM_FIRST_CASE(false, 64, 10, true);
    STREAM_FIRST_CASE(true, 64, 2, true);
    STREAM_FIRST_CASE(true, 64, 10, true);
    STREAM_FIRST_CASE(true, 32, 1, true);
#undef STREAM_FIRST_CASE
    return PYDTNN_HIP_ERR_UNSUPPORTED;
}

}  // namespace convint

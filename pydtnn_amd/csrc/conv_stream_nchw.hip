// NCHW forward convolutions whose whole filter matrix fits LDS and whose reduction is short (the first layer
// of a network: few input channels, any filter size and stride), as a streaming kernel.
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
template <int MB, int CHUNKS, int MASKS, int WAVES>
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
    float* params = lds + (size_t)GROUPS * 2 * KN * 4 + GROUPS * 2 * 4;  // [5][KN]
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
                const int f = e / SLOTS, s = e - f * SLOTS;
                const bool real = e < KN * SLOTS && s < g.k;
                v[u] = a.w[real ? (size_t)f * g.k + s : 0];
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
            uint32_t off = kOob;
            if (s < g.k) {
                const int cc = (int)fd_div((uint32_t)s, g.fd_khw), rem = s - cc * g.khw;
                const int ti = (int)fd_div((uint32_t)rem, g.fd_kw), tj = rem - ti * g.kw;
                off = (uint32_t)(((long)cc * g.h + ti * g.vdilation) * g.w + tj * g.hdilation) * 4u;
            }
            const int m = s >> 1, h = s & 1;
            tf[((m >> 2) * 2 + h) * 4 + (m & 3)] = off;
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

    // byte offset of this lane's pixel of a unit at tap (0, 0, 0), or kDead when the unit ends before it
    auto pixel_base = [&](int unit) __attribute__((always_inline)) -> uint32_t {
        const int gu = u0 + unit;
        const int img = gu / a.units_per_image;
        const int p = (gu - img * a.units_per_image) * 32 + lp;
        const uint32_t oy = fd_div((uint32_t)p, g.fd_wo), ox = (uint32_t)p - oy * (uint32_t)g.wo;
        const uint32_t off = (uint32_t)(((long)img * g.c * g.h + oy * g.vstride) * g.w + ox * g.hstride) * 4u;
        return p < g.howo ? off : kDead;
    };
    auto load_chunk = [&](uint32_t base, int chunk, float (&r)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
            const uintx4 t = toff[(chunk * 2 + gg) * 2 + lh];
#pragma unroll
            for (int i = 0; i < 4; ++i) r[gg * 4 + i] = buf_load(x_rsrc, base + t[i], 0);
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
        const uint32_t e = p0 + lp < g.howo ? (uint32_t)(4 * lh * g.howo + lp) : kDead;
        const float* pl = params + 4 * lh;
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
    uint32_t base = pixel_base(cur);
    load_chunk(base, 0, bbuf[0]);
    const floatx4* wq0 = wl + (size_t)lh * KN + lp;

    // One unit, straight-line: chunk ch is consumed from bbuf[(P0 + ch) & 1] while the next chunk (of this unit, or
    // the first of the wavefront's next unit) is in flight into the other buffer.
    auto unit_body = [&](auto parity_tag) __attribute__((always_inline)) {
        constexpr int P0 = decltype(parity_tag)::value;
        const int next = claim();
        const uint32_t base_next = next >= 0 ? pixel_base(next) : kDead;
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) {
            const int B = (P0 + ch) & 1;
            if (ch + 1 < CHUNKS)
                load_chunk(base, ch + 1, bbuf[B ^ 1]);
            else
                load_chunk(base_next, 0, bbuf[B ^ 1]);
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
        base = base_next;
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
    return ((size_t)CHUNKS * 2 * 2 * 32 * MB * 4 + CHUNKS * 2 * 2 * 4 + 5 * 32 * MB) * 4 + 16;
}

template <int MB, int CHUNKS, int MASKS, int WAVES>
int launch_stream_nchw_waves(const StreamNchwArgs& a, int grid, hipStream_t stream)
{
    static bool attr_set = false;
    constexpr size_t lds_bytes = stream_nchw_lds_bytes<MB, CHUNKS>();
    static_assert(lds_bytes <= 160 * 1024, "filter matrix must fit LDS");
    auto kernel = conv_stream_nchw_kernel<MB, CHUNKS, MASKS, WAVES>;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024) != hipSuccess)
            return PYDTNN_HIP_ERR_LAUNCH;
        attr_set = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * WAVES), lds_bytes, stream, a);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

template <int MB, int CHUNKS, int MASKS>
int launch_stream_nchw(const StreamNchwArgs& a, hipStream_t stream)
{
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            return PYDTNN_HIP_ERR_LAUNCH;
    }
    const int grid = a.units < cus ? a.units : cus;
    // A workgroup's units are taken by its wavefronts in rounds: sixteen wavefronts unless twelve leave fewer
    // idle slots in the last round (24 units: two full rounds of 12, but 32 slots of 16).
    const int per_wg = (a.units + grid - 1) / grid;
    const int slots16 = (per_wg + 15) / 16 * 16, slots12 = (per_wg + 11) / 12 * 12;
    if (slots12 < slots16) return launch_stream_nchw_waves<MB, CHUNKS, MASKS, 12>(a, grid, stream);
    return launch_stream_nchw_waves<MB, CHUNKS, MASKS, 16>(a, grid, stream);
}

// The (filters / 32, chunks of 16 reduction indices) pairs that are built: AlexNet's first layer
// (96 filters, 3 x 11 x 11 = 363 taps).
bool stream_nchw_shape_built(int kn, int k)
{
    const int chunks = (k + 15) / 16;
    return kn == 96 && chunks == 23;
}

}  // namespace

bool conv_stream_nchw_eligible(const ConvGeom& g, const ElemMasks& masks)
{
    if (!stream_nchw_shape_built(g.kn, g.k)) return false;
    if (g.vpadding != 0 || g.hpadding != 0) return false;  // taps never leave the image
    const int mk = mask_kind(masks);
    if (mk != kNoMasks && mk != kReluMask) return false;
    if (g.p < 32 * 1024) return false;                      // enough units for every compute unit
    // offsets of valid loads stay below kDead, and the descriptors below 1 GiB
    return (long)g.n * g.c * g.h * g.w < (1l << 28) && g.p * g.kn < (1l << 28);
}

int conv_stream_nchw(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                     hipStream_t stream, const ElemMasks& masks)
{
    StreamNchwArgs a;
    a.x = x; a.w = w; a.y = y; a.g = g; a.chan = chan; a.masks = masks;
    a.units_per_image = (g.howo + 31) / 32;
    a.units = g.n * a.units_per_image;
    const int chunks = (g.k + 15) / 16;
    const bool mask = mask_kind(masks) == kReluMask;
#define STREAM_NCHW_CASE(KN, CH)                                                              \
    if (g.kn == KN && chunks == CH)                                                           \
        return mask ? launch_stream_nchw<KN / 32, CH, kReluMask>(a, stream)                   \
                    : launch_stream_nchw<KN / 32, CH, kNoMasks>(a, stream)
    STREAM_NCHW_CASE(96, 23);
#undef STREAM_NCHW_CASE
    return PYDTNN_HIP_ERR_UNSUPPORTED;
}

}  // namespace convint

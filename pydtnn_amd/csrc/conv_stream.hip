// NHWC forward convolutions with a small filter matrix (1x1 and 3x3 layers of a bottleneck's first stage:
// kh*kw*c*kn <= 36864 floats, c a multiple of 64, 64 / 128 / 256 filters) as a streaming kernel.
//
// Such layers move 20-40 bytes per 1000 FLOP through a reduction of only 4 to 36 steps: on the tile engine every
// workgroup of the (one-round) launch is in its prologue or its tile store at the same time.  Here nothing is
// tiled through LDS and there is no barrier after set-up:
//   * the whole filter matrix lives in LDS for the lifetime of the workgroup (one workgroup of 8, 12 or 16
//     wavefronts per compute unit), laid out so that one 128-bit LDS read is the B operand of four MFMAs;
//   * a wavefront owns a unit of 32 output pixels x 64 filters.  The A operand of
//     v_mfma_f32_32x32x2_f32 wants pixel l%32 and reduction index l/32 in lane l, and a sum over the
//     reduction axis does not care about its order: lane (r, h) takes the channels 8q+4h .. 8q+4h+3 of a
//     64-channel chunk as its q-th quad, i.e. eight 128-bit loads straight from x into the registers the
//     MFMAs read.  Padding taps get an offset beyond the descriptor and read as zero;
//   * a unit is straight-line code over its chunks (their number is a template parameter): while the MFMAs
//     of a chunk run, the loads of the next chunk (the next tap, or the first chunk of the wavefront's next
//     unit) are in flight, and so are the unit's residual / gate values.  Every path issues the same memory
//     instructions (a prefetch without a next unit is aimed beyond the descriptor), so the waits the compiler
//     places are exact counts, not "everything";
//   * the wavefronts of a compute unit are at different points of their units, so stores, loads and MFMAs
//     of different wavefronts overlap;
//   * units are dealt to the wavefronts of a workgroup from a counter in LDS (each workgroup owns a contiguous
//     range of pixel blocks); which wavefront computes a unit does not change a bit of it;
//   * a launch walks the pixel blocks from the first to the last or the other way round, whichever starts with
//     the part of its largest input that an earlier launch on the stream touched last: a 1x1 layer on 205 MB is
//     bound by memory, and the end of what the previous kernel wrote (or read) is still in the memory-side cache.
// The store applies bias -> BN -> ReLU and one of: gate, ReLU mask, residual (+ ReLU), like the tile engine's.
#include "conv_internal.h"
#include "conv_pair.h"
#include <mutex>
#include <type_traits>

namespace convint {

namespace {

// Wavefronts per workgroup (one workgroup per compute unit): sixteen, four per SIMD, where the kernel fits 128
// registers (no side values to hold), twelve where it fits 168; the nine-chunk kernel (a 3x3 layer) needs
// more and runs eight.
constexpr int stream_waves(int chunks, int masks)
{
    return chunks > 4 ? 8 : (masks == kNoMasks || masks == kReluMask) ? 16 : 12;
}
constexpr size_t kStreamMaxFilterFloats = 36864;  // 144 KiB of the 160 KiB of LDS

struct StreamArgs {
    const float* x;
    const float* w;
    float* y;
    ConvGeom g;
    ChanEpilogue chan;
    ElemMasks masks;
    int chunks;          // reduction chunks of 64: kh*kw * (c / 64)
    int cchunks;         // c / 64
    int row_blocks;      // p / 32
    int reverse;         // workgroups and their units take the pixel blocks from the last to the first
    int n_total;         // filters of the layer (SPLIT kernels: a workgroup computes N of them)
};

typedef float floatx4s __attribute__((ext_vector_type(4)));

// SPLIT: the layer has more filters than fit LDS beside each other (n_total = a multiple of N); workgroup b
// computes filters (b % parts) * N .. + N - 1 of the pixel blocks of workgroup b / parts.
template <int N, int NB, int CHUNKS, int MASKS, bool SPLIT = false>
__global__ void __launch_bounds__(64 * stream_waves(CHUNKS, MASKS)) conv_stream_nhwc_kernel(StreamArgs a)
{
    constexpr int kStreamWaves = stream_waves(CHUNKS, MASKS), kStreamThreads = 64 * kStreamWaves;
    static_assert(N % (32 * NB) == 0, "filters per wavefront");
    constexpr int CG = N / (32 * NB);  // column groups of a pixel block
    extern __shared__ __align__(16) float lds[];
    const ConvGeom& g = a.g;
    const int k_total = g.k;
    float* wl = lds;                          // [k/4][N][4], reduction index in (tap, channel) order
    float* params = lds + (size_t)k_total * N;  // [5][N]
    int* counter = reinterpret_cast<int*>(params + 5 * N);

    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6);
    const int ln = lane & 31, lh = lane >> 5;

    // this workgroup's range of pixel blocks
    const int NT = SPLIT ? a.n_total : N;                  // row length of w, y and the side tensor
    const int parts = SPLIT ? NT / N : 1;
    const int wgs = (int)gridDim.x / parts, wgi = (int)blockIdx.x / parts;
    const int nbase = SPLIT ? ((int)blockIdx.x - wgi * parts) * N : 0;
    const int wg = a.reverse ? wgs - 1 - wgi : wgi;
    const int rb0 = (int)((long)wg * a.row_blocks / wgs);
    const int rb1 = (int)((long)(wg + 1) * a.row_blocks / wgs);
    const int units = (rb1 - rb0) * CG;

    // ---- set-up: filter matrix and per-channel parameters into LDS
    {
        const int quads = k_total * N / 4;  // float4 along the filter axis
        const floatx4s* w4 = reinterpret_cast<const floatx4s*>(a.w);
        for (int q0 = 0; q0 < quads; q0 += kStreamThreads * 6) {
            floatx4s v[6];
            int kp[6], n4[6];
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                const int q = q0 + u * kStreamThreads + tid;
                const int qc = q < quads ? q : quads - 1;
                const int kk = qc / (N / 4);       // reduction index in (tap, channel) order
                n4[u] = (qc - kk * (N / 4)) * 4;
                const int t = kk / g.c, cc = kk - t * g.c;
                kp[u] = q < quads ? kk : -1;
                v[u] = w4[((size_t)(cc * g.khw + t) * NT + nbase + n4[u]) / 4];  // the tensor's rows are (c, i, j)
            }
#pragma unroll
            for (int u = 0; u < 6; ++u)
                if (kp[u] >= 0) {
                    float* dst = wl + ((size_t)(kp[u] >> 2) * N + n4[u]) * 4 + (kp[u] & 3);
                    dst[0] = v[u][0]; dst[4] = v[u][1]; dst[8] = v[u][2]; dst[12] = v[u][3];
                }
        }
        for (int i = tid; i < N; i += kStreamThreads) {
            params[i] = a.chan.bias ? a.chan.bias[nbase + i] : 0.0f;
            params[N + i] = a.chan.mean ? a.chan.mean[nbase + i] : 0.0f;
            params[2 * N + i] = a.chan.mean ? a.chan.inv_std[nbase + i] : 1.0f;
            params[3 * N + i] = a.chan.mean ? a.chan.gamma[nbase + i] : 1.0f;
            params[4 * N + i] = a.chan.mean ? a.chan.beta[nbase + i] : 0.0f;
        }
        if (tid == 0) *counter = kStreamWaves;  // the first unit of each wavefront is its own index
    }
    __syncthreads();

    const long x_floats = (long)g.n * g.c * g.h * g.w;
    const long lead = (long)(g.vpadding * g.w + g.hpadding) * g.c;  // keeps every lane's base offset >= 0
    const rsrc_t x_rsrc = make_rsrc(a.x - lead, x_floats + lead);
    const long y_floats = g.p * NT;
    const rsrc_t y_rsrc = make_rsrc(a.y, y_floats);
    [[maybe_unused]] rsrc_t side_rsrc;  // gate bytes / mask bytes / residual floats, indexed like y
    if constexpr (MASKS == kGate) side_rsrc = make_rsrc_bytes(a.masks.gate, y_floats);
    if constexpr (MASKS == kReluMask) side_rsrc = make_rsrc_bytes(a.masks.relu_mask, y_floats);
    if constexpr (MASKS == kResidual) side_rsrc = make_rsrc(a.masks.residual, y_floats);

    // ---- per-lane data of the unit whose chunks are being loaded
    struct LoadSide {
        uint32_t base;   // byte offset of (img, ih0, iw0, channel 4h) from the shifted start
        uint32_t inv;    // tap mask: bit t set when tap t lies in the padding (bit 31 always set)
    };
    auto unit_block = [&](int unit) { return a.reverse ? rb1 - 1 - unit / CG : rb0 + unit / CG; };
    auto unit_group = [&](int unit) { return unit - (unit / CG) * CG; };
    auto setup_load = [&](int unit, LoadSide& ls) {
        const long m = (long)unit_block(unit) * 32 + ln;
        const uint32_t img = fd_div_checked((uint32_t)m, g.fd_howo, g.p < (1l << 31) && (long)g.p * g.howo < (1l << 32));
        const uint32_t pp = (uint32_t)m - img * (uint32_t)g.howo;
        const uint32_t oy = fd_div(pp, g.fd_wo), ox = pp - oy * (uint32_t)g.wo;
        const int ih0 = (int)oy * g.vstride - g.vpadding, iw0 = (int)ox * g.hstride - g.hpadding;
        ls.base = (uint32_t)((((long)img * g.h + ih0) * g.w + iw0) * g.c + lead + 4 * lh) * 4u;
        uint32_t inv = 0xffffffffu;
        for (int t = 0; t < g.khw; ++t) {
            const int ti = (int)fd_div((uint32_t)t, g.fd_kw), tj = t - ti * g.kw;
            const bool ok = (unsigned)(ih0 + ti * g.vdilation) < (unsigned)g.h &&
                            (unsigned)(iw0 + tj * g.hdilation) < (unsigned)g.w;
            if (ok) inv &= ~(1u << t);
        }
        ls.inv = inv;
    };
    // the eight quads of chunk `chunk` of that unit; with `live` false nothing is read (every offset lies
    // beyond the descriptor) but the same instructions are issued, so that the number of memory operations
    // between a load and its use is the same on every path and the waits can be exact
    auto load_chunk = [&](const LoadSide& l, int chunk, bool live, floatx4 (&r)[8]) {
        const int t = chunk / a.cchunks, c0 = (chunk - t * a.cchunks) * 64;
        const int ti = (int)fd_div((uint32_t)t, g.fd_kw), tj = t - ti * g.kw;
        const uint32_t soff = (uint32_t)((ti * g.vdilation * g.w + tj * g.hdilation) * g.c + c0) * 4u;
        const uint32_t voff = ((l.inv << (31u - (uint32_t)t)) & kOob) | l.base | (live ? 0u : kOob);
#pragma unroll
        for (int q = 0; q < 8; ++q) r[q] = buf_load4(x_rsrc, voff + (uint32_t)q * 32u, soff);
    };
    // side values (residual floats or gate bytes) of a unit, in accumulator order
    auto load_side = [&](int unit, bool live, float (&sd)[NB][16]) {
        const int m0 = unit_block(unit) * 32, n0 = unit_group(unit) * 32 * NB;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v / 4) + (v % 4);
                const uint32_t e = (uint32_t)((4 * lh) * NT + nbase + n0 + 32 * nb + ln);
                const uint32_t soff = (uint32_t)(m0 + row) * NT;
                if constexpr (MASKS == kResidual)
                    sd[nb][v] = buf_load(side_rsrc, live ? e * 4u : kOob, soff * 4u);
                if constexpr (MASKS == kGate)
                    sd[nb][v] = (float)(int8_t)__builtin_amdgcn_raw_buffer_load_b8(
                        side_rsrc, (int)(live ? e : kOob), (int)soff, 0);
            }
    };
    auto claim = [&]() -> int {
        int u = 0;
        if (lane == 0) u = atomicAdd(counter, 1);
        u = uniform(u);
        return u < units ? u : -1;
    };
    constexpr bool kSide = MASKS == kResidual || MASKS == kGate;

    floatx4 abuf[2][8];
    [[maybe_unused]] float side[NB][16];
    floatx16 acc[NB];
    LoadSide ls;
    int cur = wave < units ? wave : -1;
    if (cur < 0) return;
    setup_load(cur, ls);
    load_chunk(ls, 0, true, abuf[0]);

    // max(v, 0) as one instruction; equal to v > 0 ? v : 0 for every value an accumulator can hold (a quiet
    // NaN and -0 both give +0)
    auto relu_of = [](float v) {
        float r;
        asm("v_max_f32 %0, 0, %1" : "=v"(r) : "v"(v));
        return r;
    };
    constexpr int kEpiBias = 1, kEpiBn = 2, kEpiRelu = 4, kEpiReluAfterAdd = 8;
    const int epi_flags = (a.chan.bias ? kEpiBias : 0) | (a.chan.mean ? kEpiBn : 0) | (a.chan.relu ? kEpiRelu : 0) |
                          (MASKS == kResidual && a.masks.relu_after_add ? kEpiReluAfterAdd : 0);
    auto store_unit = [&](auto flags_tag, const floatx16 (&ac)[NB], [[maybe_unused]] const float (&sd)[NB][16], int m0,
                          int n0) {
        constexpr int F = decltype(flags_tag)::value;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int col = n0 + 32 * nb + ln;
            [[maybe_unused]] float bias, mean, inv_std, gamma, beta;
            if constexpr ((F & kEpiBias) != 0) bias = params[col];
            if constexpr ((F & kEpiBn) != 0) {
                mean = params[N + col]; inv_std = params[2 * N + col];
                gamma = params[3 * N + col]; beta = params[4 * N + col];
            }
            const uint32_t e = (uint32_t)((4 * lh) * NT + nbase + col);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v / 4) + (v % 4);
                const uint32_t soff = (uint32_t)(m0 + row) * NT;
                float val = ac[nb][v];
                if constexpr ((F & kEpiBias) != 0) val += bias;
                if constexpr ((F & kEpiBn) != 0) {
                    const float t = (val - mean) * inv_std;
                    val = t * gamma + beta;
                }
                if constexpr ((F & kEpiRelu) != 0) val = relu_of(val);
                if constexpr (MASKS == kGate) val *= sd[nb][v];
                if constexpr (MASKS == kResidual) {
                    val += sd[nb][v];
                    if constexpr ((F & kEpiReluAfterAdd) != 0) val = relu_of(val);
                }
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), y_rsrc, (int)(e * 4u),
                                                      (int)(soff * 4u), 0);
                if constexpr (MASKS == kReluMask)
                    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(val > 0.0f ? 1 : 0), side_rsrc, (int)e, (int)soff,
                                                         0);
            }
        }
    };

    // One unit, straight-line: chunk ch is consumed from abuf[(P0 + ch) & 1] while the next chunk (of this
    // unit, or the first of the wavefront's next unit) is in flight into the other buffer.
    auto unit_body = [&](auto parity_tag) {
        constexpr int P0 = decltype(parity_tag)::value;
        const int next = claim();
        const bool more = next >= 0;
        LoadSide lsn;
        setup_load(more ? next : cur, lsn);
        // the unit's side values have its MFMAs (and those of the wavefronts sharing the SIMD) to arrive
        if constexpr (kSide) load_side(cur, true, side);
        const int n0 = unit_group(cur) * 32 * NB;
        const floatx4* wq0 = reinterpret_cast<const floatx4*>(wl) + ((size_t)lh * N + n0 + ln);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) {
            const int B = (P0 + ch) & 1;
            if (ch + 1 < CHUNKS)
                load_chunk(ls, ch + 1, true, abuf[B ^ 1]);
            else
                load_chunk(lsn, 0, more, abuf[B ^ 1]);
            __builtin_amdgcn_sched_barrier(0);
            // B operands: quad q of the chunk holds reduction indices 8q + 4h .. + 3 for filter n0 + 32 nb + n
            const floatx4* wq = wq0 + (size_t)(ch * 16) * N;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                floatx4 bq[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) bq[nb] = wq[(size_t)(2 * q) * N + 32 * nb];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        // the unit's first MFMA of each block starts from a constant zero: no registers to clear
                        const floatx16 zero = {};
                        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(abuf[B][q][i], bq[nb][i],
                                                                       ch == 0 && q == 0 && i == 0 ? zero : acc[nb], 0, 0, 0);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- the unit's store (every block is whole: the pixel count is a multiple of 32), in the variant
        // the launch's epilogue flags select: a store loop carries no test or select per element
        const int m0 = unit_block(cur) * 32;
        switch (epi_flags) {
        case 0: store_unit(std::integral_constant<int, 0>{}, acc, side, m0, n0); break;
        case 1: store_unit(std::integral_constant<int, 1>{}, acc, side, m0, n0); break;
        case 2: store_unit(std::integral_constant<int, 2>{}, acc, side, m0, n0); break;
        case 3: store_unit(std::integral_constant<int, 3>{}, acc, side, m0, n0); break;
        case 4: store_unit(std::integral_constant<int, 4>{}, acc, side, m0, n0); break;
        case 5: store_unit(std::integral_constant<int, 5>{}, acc, side, m0, n0); break;
        case 6: store_unit(std::integral_constant<int, 6>{}, acc, side, m0, n0); break;
        case 7: store_unit(std::integral_constant<int, 7>{}, acc, side, m0, n0); break;
        case 8: store_unit(std::integral_constant<int, 8>{}, acc, side, m0, n0); break;
        case 9: store_unit(std::integral_constant<int, 9>{}, acc, side, m0, n0); break;
        case 10: store_unit(std::integral_constant<int, 10>{}, acc, side, m0, n0); break;
        case 11: store_unit(std::integral_constant<int, 11>{}, acc, side, m0, n0); break;
        case 12: store_unit(std::integral_constant<int, 12>{}, acc, side, m0, n0); break;
        case 13: store_unit(std::integral_constant<int, 13>{}, acc, side, m0, n0); break;
        case 14: store_unit(std::integral_constant<int, 14>{}, acc, side, m0, n0); break;
        default: store_unit(std::integral_constant<int, 15>{}, acc, side, m0, n0); break;
        }
        ls = lsn;
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

// The same kernel on v_mfma_f32_16x16x4_f32, for layers over many channels whose loads, not their MFMAs, set the
// time (a 1x1 layer over 256 channels: pixels are 1 KB apart).  A unit is 16 pixels x 64 filters.  The A operand
// wants pixel l%16 and reduction index l/16 in lane l: lane (r, kq) takes channels 16q + 4kq .. + 3 of a 64-channel
// chunk as its q-th quad (four 128-bit loads per chunk), so the four lanes of a pixel fetch 64 consecutive bytes
// and a load instruction touches 16 lines instead of the 32 of the 32-pixel form (the rate at which addresses are
// accepted is what limits that form), and the last, partly filled round of units is half as long.  The filter
// matrix lies in LDS exactly as above ([k/4][N][4]: one 128-bit read is the B operand of four MFMAs for filter n).
// Accumulator register v of lane (g, n) holds pixel 4g + v, filter n of a 16 x 16 block.
template <int N, int CHUNKS, int MASKS>
__global__ void __launch_bounds__(64 * stream_waves(CHUNKS, MASKS)) conv_stream_nhwc16_kernel(StreamArgs a)
{
    constexpr int kStreamWaves = stream_waves(CHUNKS, MASKS), kStreamThreads = 64 * kStreamWaves;
    constexpr int NB = 4;              // 16-filter blocks of a unit
    constexpr int CG = N / 64;         // column groups of a pixel block
    extern __shared__ __align__(16) float lds[];
    const ConvGeom& g = a.g;
    const int k_total = g.k;
    float* wl = lds;
    float* params = lds + (size_t)k_total * N;
    int* counter = reinterpret_cast<int*>(params + 5 * N);

    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6);
    const int ln = lane & 15, lk = lane >> 4;

    const int row_blocks = a.row_blocks * 2;   // of 16 pixels
    const int wg = a.reverse ? (int)(gridDim.x - 1 - blockIdx.x) : (int)blockIdx.x;
    const int rb0 = (int)((long)wg * row_blocks / gridDim.x);
    const int rb1 = (int)((long)(wg + 1) * row_blocks / gridDim.x);
    const int units = (rb1 - rb0) * CG;

    {
        const int quads = k_total * N / 4;
        const floatx4s* w4 = reinterpret_cast<const floatx4s*>(a.w);
        for (int q0 = 0; q0 < quads; q0 += kStreamThreads * 6) {
            floatx4s v[6];
            int kp[6], n4[6];
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                const int q = q0 + u * kStreamThreads + tid;
                const int qc = q < quads ? q : quads - 1;
                const int kk = qc / (N / 4);
                n4[u] = (qc - kk * (N / 4)) * 4;
                const int t = kk / g.c, cc = kk - t * g.c;
                kp[u] = q < quads ? kk : -1;
                v[u] = w4[((size_t)(cc * g.khw + t) * N + n4[u]) / 4];
            }
#pragma unroll
            for (int u = 0; u < 6; ++u)
                if (kp[u] >= 0) {
                    float* dst = wl + ((size_t)(kp[u] >> 2) * N + n4[u]) * 4 + (kp[u] & 3);
                    dst[0] = v[u][0]; dst[4] = v[u][1]; dst[8] = v[u][2]; dst[12] = v[u][3];
                }
        }
        for (int i = tid; i < N; i += kStreamThreads) {
            params[i] = a.chan.bias ? a.chan.bias[i] : 0.0f;
            params[N + i] = a.chan.mean ? a.chan.mean[i] : 0.0f;
            params[2 * N + i] = a.chan.mean ? a.chan.inv_std[i] : 1.0f;
            params[3 * N + i] = a.chan.mean ? a.chan.gamma[i] : 1.0f;
            params[4 * N + i] = a.chan.mean ? a.chan.beta[i] : 0.0f;
        }
        if (tid == 0) *counter = kStreamWaves;
    }
    __syncthreads();

    const long x_floats = (long)g.n * g.c * g.h * g.w;
    const long lead = (long)(g.vpadding * g.w + g.hpadding) * g.c;
    const rsrc_t x_rsrc = make_rsrc(a.x - lead, x_floats + lead);
    const long y_floats = g.p * N;
    const rsrc_t y_rsrc = make_rsrc(a.y, y_floats);
    [[maybe_unused]] rsrc_t side_rsrc;
    if constexpr (MASKS == kGate) side_rsrc = make_rsrc_bytes(a.masks.gate, y_floats);
    if constexpr (MASKS == kReluMask) side_rsrc = make_rsrc_bytes(a.masks.relu_mask, y_floats);
    if constexpr (MASKS == kResidual) side_rsrc = make_rsrc(a.masks.residual, y_floats);

    struct LoadSide {
        uint32_t base;   // byte offset of (img, ih0, iw0, channel 4 kq) from the shifted start
        uint32_t inv;    // tap mask: bit t set when tap t lies in the padding (bit 31 always set)
    };
    auto unit_block = [&](int unit) { return a.reverse ? rb1 - 1 - unit / CG : rb0 + unit / CG; };
    auto unit_group = [&](int unit) { return unit - (unit / CG) * CG; };
    auto setup_load = [&](int unit, LoadSide& ls) {
        const long m = (long)unit_block(unit) * 16 + ln;
        const uint32_t img = fd_div_checked((uint32_t)m, g.fd_howo, g.p < (1l << 31) && (long)g.p * g.howo < (1l << 32));
        const uint32_t pp = (uint32_t)m - img * (uint32_t)g.howo;
        const uint32_t oy = fd_div(pp, g.fd_wo), ox = pp - oy * (uint32_t)g.wo;
        const int ih0 = (int)oy * g.vstride - g.vpadding, iw0 = (int)ox * g.hstride - g.hpadding;
        ls.base = (uint32_t)((((long)img * g.h + ih0) * g.w + iw0) * g.c + lead + 4 * lk) * 4u;
        uint32_t inv = 0xffffffffu;
        for (int t = 0; t < g.khw; ++t) {
            const int ti = (int)fd_div((uint32_t)t, g.fd_kw), tj = t - ti * g.kw;
            const bool ok = (unsigned)(ih0 + ti * g.vdilation) < (unsigned)g.h &&
                            (unsigned)(iw0 + tj * g.hdilation) < (unsigned)g.w;
            if (ok) inv &= ~(1u << t);
        }
        ls.inv = inv;
    };
    auto load_chunk = [&](const LoadSide& l, int chunk, bool live, floatx4 (&r)[4]) {
        const int t = chunk / a.cchunks, c0 = (chunk - t * a.cchunks) * 64;
        const int ti = (int)fd_div((uint32_t)t, g.fd_kw), tj = t - ti * g.kw;
        const uint32_t soff = (uint32_t)((ti * g.vdilation * g.w + tj * g.hdilation) * g.c + c0) * 4u;
        const uint32_t voff = ((l.inv << (31u - (uint32_t)t)) & kOob) | l.base | (live ? 0u : kOob);
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = buf_load4(x_rsrc, voff + (uint32_t)q * 64u, soff);
    };
    auto load_side = [&](int unit, bool live, float (&sd)[NB][4]) {
        const int m0 = unit_block(unit) * 16, n0 = unit_group(unit) * 64;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t e = (uint32_t)((4 * lk) * N + n0 + 16 * nb + ln);
                const uint32_t soff = (uint32_t)(m0 + v) * N;
                if constexpr (MASKS == kResidual)
                    sd[nb][v] = buf_load(side_rsrc, live ? e * 4u : kOob, soff * 4u);
                if constexpr (MASKS == kGate)
                    sd[nb][v] = (float)(int8_t)__builtin_amdgcn_raw_buffer_load_b8(
                        side_rsrc, (int)(live ? e : kOob), (int)soff, 0);
            }
    };
    auto claim = [&]() -> int {
        int u = 0;
        if (lane == 0) u = atomicAdd(counter, 1);
        u = uniform(u);
        return u < units ? u : -1;
    };
    constexpr bool kSide = MASKS == kResidual || MASKS == kGate;

    floatx4 abuf[2][4];
    [[maybe_unused]] float side[NB][4];
    floatx4 acc[NB];
    LoadSide ls;
    int cur = wave < units ? wave : -1;
    if (cur < 0) return;
    setup_load(cur, ls);
    load_chunk(ls, 0, true, abuf[0]);

    auto relu_of = [](float v) {
        float r;
        asm("v_max_f32 %0, 0, %1" : "=v"(r) : "v"(v));
        return r;
    };
    constexpr int kEpiBias = 1, kEpiBn = 2, kEpiRelu = 4, kEpiReluAfterAdd = 8;
    const int epi_flags = (a.chan.bias ? kEpiBias : 0) | (a.chan.mean ? kEpiBn : 0) | (a.chan.relu ? kEpiRelu : 0) |
                          (MASKS == kResidual && a.masks.relu_after_add ? kEpiReluAfterAdd : 0);
    auto store_unit = [&](auto flags_tag, const floatx4 (&ac)[NB], [[maybe_unused]] const float (&sd)[NB][4], int m0,
                          int n0) {
        constexpr int F = decltype(flags_tag)::value;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int col = n0 + 16 * nb + ln;
            [[maybe_unused]] float bias, mean, inv_std, gamma, beta;
            if constexpr ((F & kEpiBias) != 0) bias = params[col];
            if constexpr ((F & kEpiBn) != 0) {
                mean = params[N + col]; inv_std = params[2 * N + col];
                gamma = params[3 * N + col]; beta = params[4 * N + col];
            }
            const uint32_t e = (uint32_t)((4 * lk) * N + col);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t soff = (uint32_t)(m0 + v) * N;
                float val = ac[nb][v];
                if constexpr ((F & kEpiBias) != 0) val += bias;
                if constexpr ((F & kEpiBn) != 0) {
                    const float t = (val - mean) * inv_std;
                    val = t * gamma + beta;
                }
                if constexpr ((F & kEpiRelu) != 0) val = relu_of(val);
                if constexpr (MASKS == kGate) val *= sd[nb][v];
                if constexpr (MASKS == kResidual) {
                    val += sd[nb][v];
                    if constexpr ((F & kEpiReluAfterAdd) != 0) val = relu_of(val);
                }
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), y_rsrc, (int)(e * 4u),
                                                      (int)(soff * 4u), 0);
                if constexpr (MASKS == kReluMask)
                    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(val > 0.0f ? 1 : 0), side_rsrc, (int)e, (int)soff,
                                                         0);
            }
        }
    };

    auto unit_body = [&](auto parity_tag) {
        constexpr int P0 = decltype(parity_tag)::value;
        const int next = claim();
        const bool more = next >= 0;
        LoadSide lsn;
        setup_load(more ? next : cur, lsn);
        if constexpr (kSide) load_side(cur, true, side);
        const int n0 = unit_group(cur) * 64;
        const floatx4* wq0 = reinterpret_cast<const floatx4*>(wl) + ((size_t)lk * N + n0 + ln);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) {
            const int B = (P0 + ch) & 1;
            if (ch + 1 < CHUNKS)
                load_chunk(ls, ch + 1, true, abuf[B ^ 1]);
            else
                load_chunk(lsn, 0, more, abuf[B ^ 1]);
            __builtin_amdgcn_sched_barrier(0);
            // B operands: quad q of the chunk holds reduction indices 16q + 4kq .. + 3 for filter n0 + 16 nb + n
            const floatx4* wq = wq0 + (size_t)(ch * 16) * N;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                floatx4 bq[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) bq[nb] = wq[(size_t)(4 * q) * N + 16 * nb];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const floatx4 zero = {};
                        acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(abuf[B][q][i], bq[nb][i],
                                                                       ch == 0 && q == 0 && i == 0 ? zero : acc[nb], 0, 0, 0);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        const int m0 = unit_block(cur) * 16;
        switch (epi_flags) {
        case 0: store_unit(std::integral_constant<int, 0>{}, acc, side, m0, n0); break;
        case 1: store_unit(std::integral_constant<int, 1>{}, acc, side, m0, n0); break;
        case 2: store_unit(std::integral_constant<int, 2>{}, acc, side, m0, n0); break;
        case 3: store_unit(std::integral_constant<int, 3>{}, acc, side, m0, n0); break;
        case 4: store_unit(std::integral_constant<int, 4>{}, acc, side, m0, n0); break;
        case 5: store_unit(std::integral_constant<int, 5>{}, acc, side, m0, n0); break;
        case 6: store_unit(std::integral_constant<int, 6>{}, acc, side, m0, n0); break;
        case 7: store_unit(std::integral_constant<int, 7>{}, acc, side, m0, n0); break;
        case 8: store_unit(std::integral_constant<int, 8>{}, acc, side, m0, n0); break;
        case 9: store_unit(std::integral_constant<int, 9>{}, acc, side, m0, n0); break;
        case 10: store_unit(std::integral_constant<int, 10>{}, acc, side, m0, n0); break;
        case 11: store_unit(std::integral_constant<int, 11>{}, acc, side, m0, n0); break;
        case 12: store_unit(std::integral_constant<int, 12>{}, acc, side, m0, n0); break;
        case 13: store_unit(std::integral_constant<int, 13>{}, acc, side, m0, n0); break;
        case 14: store_unit(std::integral_constant<int, 14>{}, acc, side, m0, n0); break;
        default: store_unit(std::integral_constant<int, 15>{}, acc, side, m0, n0); break;
        }
        ls = lsn;
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

template <int N, int CHUNKS, int MASKS>
int launch_stream16(const StreamArgs& a, hipStream_t stream)
{
    static std::atomic<unsigned> raised{0};
    const size_t lds_bytes = ((size_t)a.g.k * N + 5 * N) * 4 + 16;
    auto kernel = conv_stream_nhwc16_kernel<N, CHUNKS, MASKS>;
    int cus = 0;
    int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), raised, 160 * 1024);
    if (rc == PYDTNN_HIP_OK) rc = device_compute_units(&cus);
    if (rc != PYDTNN_HIP_OK) return rc;
    const int grid = 2 * a.row_blocks < cus ? 2 * a.row_blocks : cus;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * stream_waves(CHUNKS, MASKS)), lds_bytes, stream, a);
    HIP_RETURN_IF_LAUNCH_FAILED();
    note_launch(kLaunchStreamNhwc, 16, N, grid, 0, 1);
    return PYDTNN_HIP_OK;
}

template <int N, int CHUNKS>
int launch_stream16_masks(const StreamArgs& a, hipStream_t stream)
{
    switch (mask_kind(a.masks)) {
    case kGate: return launch_stream16<N, CHUNKS, kGate>(a, stream);
    case kReluMask: return launch_stream16<N, CHUNKS, kReluMask>(a, stream);
    case kResidual: return launch_stream16<N, CHUNKS, kResidual>(a, stream);
    default: return launch_stream16<N, CHUNKS, kNoMasks>(a, stream);
    }
}

template <int N, int NB, int CHUNKS, int MASKS, bool SPLIT = false>
int launch_stream(const StreamArgs& a, hipStream_t stream)
{
    static std::atomic<unsigned> raised{0};
    const size_t lds_bytes = ((size_t)a.g.k * N + 5 * N) * 4 + 16;
    auto kernel = conv_stream_nhwc_kernel<N, NB, CHUNKS, MASKS, SPLIT>;
    int cus = 0;
    int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), raised, 160 * 1024);
    if (rc == PYDTNN_HIP_OK) rc = device_compute_units(&cus);
    if (rc != PYDTNN_HIP_OK) return rc;
    // one workgroup per compute unit; SPLIT: that many shared out between the parts of every pixel range
    const int parts = SPLIT ? a.n_total / N : 1;
    int ranges = cus / parts;
    if (ranges > a.row_blocks) ranges = a.row_blocks;
    if (ranges < 1) ranges = 1;
    const int grid = ranges * parts;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * stream_waves(CHUNKS, MASKS)), lds_bytes, stream, a);
    HIP_RETURN_IF_LAUNCH_FAILED();
    note_launch(kLaunchStreamNhwc, 32, N, grid, 0, 1);
    return PYDTNN_HIP_OK;
}

template <int N, int CHUNKS, bool SPLIT = false>
int launch_stream_masks(const StreamArgs& a, hipStream_t stream)
{
    switch (mask_kind(a.masks)) {
    case kGate: return launch_stream<N, 2, CHUNKS, kGate, SPLIT>(a, stream);
    case kReluMask: return launch_stream<N, 2, CHUNKS, kReluMask, SPLIT>(a, stream);
    case kResidual: return launch_stream<N, 2, CHUNKS, kResidual, SPLIT>(a, stream);
    default: return launch_stream<N, 2, CHUNKS, kNoMasks, SPLIT>(a, stream);
    }
}

// The (filters, chunks of 64 reduction indices) pairs that are built: 1x1 layers over 64, 128 and 256 channels
// and the 3x3 layer over 64.
bool stream_shape_built(int kn, int chunks)
{
    switch (kn) {
    case 64: return chunks == 1 || chunks == 2 || chunks == 4 || chunks == 9;
    case 128: return chunks == 1 || chunks == 2 || chunks == 4;
    case 256: return chunks == 1 || chunks == 2;
    // more filters than fit LDS beside each other, in parts of 256 (a bottleneck's last 1x1 layer over 128 channels)
    case 512: return chunks == 2;
    default: return false;
    }
}
constexpr int stream_part_filters(int kn) { return kn > 256 ? 256 : kn; }

// The direction of a launch.  Per stream, the tensors the last few launches walked and the direction they walked
// them in; a new launch goes the other way than the launch that last touched its residual (if it has one: that is
// its largest input) or else its input, so that it begins where that one ended, and forwards when neither is
// known.  Results do not depend on the direction; the table only has to be consistent, hence the mutex.
struct Walk {
    const void* tensor;
    int reverse;
};
struct StreamWalks {
    hipStream_t stream;
    bool used;
    int next;
    Walk walks[6];
};
std::mutex walks_mutex;
StreamWalks stream_walks[8];
int next_stream_slot = 0;

}  // namespace

int conv_stream_choose_direction(hipStream_t stream, const void* x, const void* residual, const void* y)
{
    std::lock_guard<std::mutex> lock(walks_mutex);
    StreamWalks* sw = nullptr;
    for (StreamWalks& c : stream_walks)
        if (c.used && c.stream == stream) sw = &c;
    if (!sw) {
        sw = &stream_walks[next_stream_slot];
        next_stream_slot = (next_stream_slot + 1) % 8;
        *sw = StreamWalks{};
        sw->stream = stream;
        sw->used = true;
    }
    auto last_walk = [&](const void* t) {
        if (t)
            for (const Walk& wk : sw->walks)
                if (wk.tensor == t) return wk.reverse;
        return -1;
    };
    int seen = last_walk(residual);
    if (seen < 0) seen = last_walk(x);
    const int reverse = seen < 0 ? 0 : !seen;
    auto note = [&](const void* t) {
        if (!t) return;
        for (Walk& wk : sw->walks)
            if (wk.tensor == t) { wk.reverse = reverse; return; }
        sw->walks[sw->next] = Walk{t, reverse};
        sw->next = (sw->next + 1) % 6;
    };
    note(x);
    note(residual);
    note(y);
    return reverse;
}

// Shapes the streaming kernel takes: the filter matrix fits LDS, channels come in chunks of 64 floats that
// 128-bit loads can fetch, and there is enough work for every compute unit.
bool conv_stream_nhwc_eligible(const ConvGeom& g, const float* w, const float* x)
{
    if (g.c % 64 != 0 || !stream_shape_built(g.kn, g.khw * (g.c / 64))) return false;
    if ((size_t)g.k * stream_part_filters(g.kn) > kStreamMaxFilterFloats || g.khw > 31) return false;
    if (!aligned16(w) || !aligned16(x)) return false;
    if (g.p < 32 * 1024 || g.p % 32 != 0) return false;
    return (long)g.n * g.c * g.h * g.w + (long)(g.vpadding * g.w + g.hpadding) * g.c < (1l << 29) &&
           g.p * g.kn < (1l << 29);
}

int conv_stream_nhwc(const ConvGeom& g, const float* w, const float* x, float* y, const ChanEpilogue& chan,
                     hipStream_t stream, const ElemMasks& masks)
{
    StreamArgs a;
    a.x = x; a.w = w; a.y = y; a.g = g; a.chan = chan; a.masks = masks;
    a.cchunks = g.c / 64;
    a.chunks = g.khw * a.cchunks;
    a.row_blocks = (int)(g.p / 32);
    a.reverse = conv_stream_choose_direction(stream, x, masks.residual, y);
    a.n_total = g.kn;
    if (g.kn == 512 && a.chunks == 2) return launch_stream_masks<256, 2, true>(a, stream);
    // 64 filters over 256 channels (a bottleneck's first 1x1 layer): units of 16 pixels
    if (g.kn == 64 && a.chunks == 4 && g.khw == 1) return launch_stream16_masks<64, 4>(a, stream);
#define STREAM_CASE(KN, CH) \
    if (g.kn == KN && a.chunks == CH) return launch_stream_masks<KN, CH>(a, stream)
    STREAM_CASE(64, 1); STREAM_CASE(64, 2); STREAM_CASE(64, 4); STREAM_CASE(64, 9);
    STREAM_CASE(128, 1); STREAM_CASE(128, 2); STREAM_CASE(128, 4);
    STREAM_CASE(256, 1); STREAM_CASE(256, 2);
#undef STREAM_CASE
    return PYDTNN_HIP_ERR_UNSUPPORTED;
}

}  // namespace convint

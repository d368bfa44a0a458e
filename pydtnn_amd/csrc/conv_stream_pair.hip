// Two convolutions of a ResNet bottleneck as one launch, NHWC: the 3x3 layer over 64 channels with 64 filters
// (bias -> BN -> ReLU in registers) and the 1x1 layer that takes its output to 256 filters (bias -> BN, the block's
// residual sum and the ReLU after it in the store).  The 64-channel tensor between them is never written or read:
// 51 MB each way at batch 64, and one launch with its set-up and drain less.
//
// The kernel is the streaming kernel of conv_stream.hip (3x3 filter matrix in LDS for the life of the workgroup,
// activations loaded straight into MFMA operand registers, units of 32 pixels dealt from an LDS counter, every
// path issuing the same memory instructions) with two changes:
//   * the first product is computed transposed.  v_mfma_f32_32x32x2_f32 takes A[row = lane % 32][k = lane / 32] and
//     B[k = lane / 32][col = lane % 32]: the registers that hold x as an A operand (row = pixel) are a B operand
//     with col = pixel just as well, and the filter quads from LDS an A operand with row = filter.  The
//     accumulators then hold, in lane (pixel, h), register v: filter 8*(v/4) + 4h + v%4 of that pixel, which is
//     the A operand (row = pixel, k chosen by h) of the second product as it lies: step (nb, v) of the second
//     product multiplies the first product's accumulator nb, register v.  That is also the order in which the
//     1x1 streaming kernel walks its 64 channels, so the fused result has the bits of the two launches;
//   * the second filter (64 x 256 floats) does not fit beside the first (147 KB of the 160 KB of LDS).  Its B
//     operands come straight from memory (it stays in L2): lane (col, h) needs W2[that k][32*piece + col],
//     a row of 128 contiguous bytes per half wavefront, requested one piece (32 MFMAs) ahead of its use.
// A unit: 576 MFMAs of the first product, then eight times (32 MFMAs for 32 of the 256 output filters, the next
// piece's filter values and residual in flight meanwhile, store).  The next unit's first activations are requested
// inside the last piece.
#include "conv_pair.h"
#include <type_traits>

namespace convint {

namespace {

constexpr int kN1 = 64;            // filters of the first convolution = channels of the second
constexpr int kChunks = 9;         // taps of the first convolution (64 channels each)
constexpr int kWaves = 8, kPairThreads = 64 * kWaves;
constexpr int kMaxN2 = 256;

struct PairArgs {
    const float* x;
    const float* w1;
    const float* w2;
    float* y;
    ConvGeom g;            // the first convolution
    ChanEpilogue chan1, chan2;
    ElemMasks masks;       // of the second convolution's store: residual (+ ReLU) or nothing
    int n2;                // filters of the second convolution, a multiple of 64, at most kMaxN2
    int row_blocks;        // p / 32
    int reverse;
};

typedef float floatx4s __attribute__((ext_vector_type(4)));

// flags of the second store's variants (the first epilogue works on 32 values a unit and tests its flags)
constexpr int kEpiBias = 1, kEpiBn = 2, kEpiRelu = 4, kEpiReluAfterAdd = 8;

template <int MASKS>
__global__ void __launch_bounds__(kPairThreads) conv_stream_pair_kernel(PairArgs a)
{
    constexpr int N = kN1, NB = 2;
    extern __shared__ __align__(16) float lds[];
    const ConvGeom& g = a.g;
    const int k_total = g.k;                      // 576
    const int n2 = a.n2;
    float* wl = lds;                              // [k/4][N][4], reduction index in (tap, channel) order
    float* params1 = lds + (size_t)k_total * N;   // [5][N]
    float* params2 = params1 + 5 * N;             // [5][kMaxN2]
    int* counter = reinterpret_cast<int*>(params2 + 5 * kMaxN2);

    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6);
    const int ln = lane & 31, lh = lane >> 5;

    const int wg = a.reverse ? (int)(gridDim.x - 1 - blockIdx.x) : (int)blockIdx.x;
    const int rb0 = (int)((long)wg * a.row_blocks / gridDim.x);
    const int rb1 = (int)((long)(wg + 1) * a.row_blocks / gridDim.x);
    const int units = rb1 - rb0;

    // ---- set-up: first filter matrix and both layers' per-channel parameters into LDS
    {
        const int quads = k_total * N / 4;
        const floatx4s* w4 = reinterpret_cast<const floatx4s*>(a.w1);
        for (int q0 = 0; q0 < quads; q0 += kPairThreads * 6) {
            floatx4s v[6];
            int kp[6], n4[6];
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                const int q = q0 + u * kPairThreads + tid;
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
        for (int i = tid; i < N; i += kPairThreads) {
            params1[i] = a.chan1.bias ? a.chan1.bias[i] : 0.0f;
            params1[N + i] = a.chan1.mean ? a.chan1.mean[i] : 0.0f;
            params1[2 * N + i] = a.chan1.mean ? a.chan1.inv_std[i] : 1.0f;
            params1[3 * N + i] = a.chan1.mean ? a.chan1.gamma[i] : 1.0f;
            params1[4 * N + i] = a.chan1.mean ? a.chan1.beta[i] : 0.0f;
        }
        for (int i = tid; i < n2; i += kPairThreads) {
            params2[i] = a.chan2.bias ? a.chan2.bias[i] : 0.0f;
            params2[kMaxN2 + i] = a.chan2.mean ? a.chan2.mean[i] : 0.0f;
            params2[2 * kMaxN2 + i] = a.chan2.mean ? a.chan2.inv_std[i] : 1.0f;
            params2[3 * kMaxN2 + i] = a.chan2.mean ? a.chan2.gamma[i] : 1.0f;
            params2[4 * kMaxN2 + i] = a.chan2.mean ? a.chan2.beta[i] : 0.0f;
        }
        if (tid == 0) *counter = kWaves;
    }
    __syncthreads();

    const long x_floats = (long)g.n * g.c * g.h * g.w;
    const long lead = (long)(g.vpadding * g.w + g.hpadding) * g.c;
    const rsrc_t x_rsrc = make_rsrc(a.x - lead, x_floats + lead);
    const long y_floats = g.p * n2;
    const rsrc_t y_rsrc = make_rsrc(a.y, y_floats);
    const rsrc_t w2_rsrc = make_rsrc(a.w2, (long)N * n2);
    [[maybe_unused]] rsrc_t side_rsrc;
    if constexpr (MASKS == kResidual) side_rsrc = make_rsrc(a.masks.residual, y_floats);

    struct LoadSide {
        uint32_t base;
        uint32_t inv;
    };
    auto unit_block = [&](int unit) __attribute__((always_inline)) { return a.reverse ? rb1 - 1 - unit : rb0 + unit; };
    auto setup_load = [&](int unit, LoadSide& ls) __attribute__((always_inline)) {
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
    // the eight quads of tap `chunk` (64 channels) of that unit; with `live` false nothing is read
    auto load_chunk = [&](const LoadSide& l, int chunk, bool live, floatx4 (&r)[8]) __attribute__((always_inline)) {
        const int ti = (int)fd_div((uint32_t)chunk, g.fd_kw), tj = chunk - ti * g.kw;
        const uint32_t soff = (uint32_t)((ti * g.vdilation * g.w + tj * g.hdilation) * g.c) * 4u;
        const uint32_t voff = ((l.inv << (31u - (uint32_t)chunk)) & kOob) | l.base | (live ? 0u : kOob);
#pragma unroll
        for (int q = 0; q < 8; ++q) r[q] = buf_load4(x_rsrc, voff + (uint32_t)q * 32u, soff);
    };
    // B operands of one piece of the second product (32 of its filters, all 32 steps): step t = (nb, v) wants
    // W2[32 nb + 8 (v / 4) + 4 h + v % 4][32 piece + col]
    const uint32_t w2_lane = (uint32_t)((4 * lh) * n2 + ln) * 4u;
    auto load_w2 = [&](int piece, float (&wb)[32]) __attribute__((always_inline)) {
        const uint32_t voff = w2_lane + (uint32_t)piece * 128u;
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const int nb = t / 16, v = t % 16;
            const int f = 32 * nb + 8 * (v / 4) + (v % 4);
            wb[t] = buf_load(w2_rsrc, voff, (uint32_t)(f * n2) * 4u);
        }
    };
    auto load_side = [&](int unit, int piece, float (&sd)[16]) __attribute__((always_inline)) {
        const int m0 = unit_block(unit) * 32;
        const uint32_t e = (uint32_t)((4 * lh) * n2 + 32 * piece + ln);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v / 4) + (v % 4);
            const uint32_t soff = (uint32_t)(m0 + row) * (uint32_t)n2;
            sd[v] = buf_load(side_rsrc, e * 4u, soff * 4u);
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

    floatx4 abuf[2][8];
    float wbuf[2][32];
    [[maybe_unused]] float side[2][16];
    floatx16 acc1[NB], acc2;
    LoadSide ls;
    int cur = wave < units ? wave : -1;
    if (cur < 0) return;
    setup_load(cur, ls);
    load_chunk(ls, 0, true, abuf[0]);

    const bool bias1 = a.chan1.bias != nullptr, bn1 = a.chan1.mean != nullptr, relu1 = a.chan1.relu != 0;
    const int epi_flags2 = (a.chan2.bias ? kEpiBias : 0) | (a.chan2.mean ? kEpiBn : 0) | (a.chan2.relu ? kEpiRelu : 0) |
                           (MASKS == kResidual && a.masks.relu_after_add ? kEpiReluAfterAdd : 0);
    const int pieces = n2 / 32;

    // the store of one piece: 32 pixels x 32 of the second convolution's filters
    auto store_piece = [&](auto flags_tag, const floatx16& ac, [[maybe_unused]] const float (&sd)[16], int m0,
                           int piece) __attribute__((always_inline)) {
        constexpr int F = decltype(flags_tag)::value;
        const int col = 32 * piece + ln;
        [[maybe_unused]] float bias, mean, inv_std, gamma, beta;
        if constexpr ((F & kEpiBias) != 0) bias = params2[col];
        if constexpr ((F & kEpiBn) != 0) {
            mean = params2[kMaxN2 + col]; inv_std = params2[2 * kMaxN2 + col];
            gamma = params2[3 * kMaxN2 + col]; beta = params2[4 * kMaxN2 + col];
        }
        const uint32_t e = (uint32_t)((4 * lh) * n2 + col);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v / 4) + (v % 4);
            const uint32_t soff = (uint32_t)(m0 + row) * (uint32_t)n2;
            float val = ac[v];
            if constexpr ((F & kEpiBias) != 0) val += bias;
            if constexpr ((F & kEpiBn) != 0) {
                const float t = (val - mean) * inv_std;
                val = t * gamma + beta;
            }
            if constexpr ((F & kEpiRelu) != 0) val = relu_of(val);
            if constexpr (MASKS == kResidual) {
                val += sd[v];
                if constexpr ((F & kEpiReluAfterAdd) != 0) val = relu_of(val);
            }
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), y_rsrc, (int)(e * 4u),
                                                  (int)(soff * 4u), 0);
        }
    };

    // One piece of the second product: 32 MFMAs on the operands requested during the piece before, while the next
    // piece's operands and residual (or, in the unit's last piece, the next unit's first activations) are
    // requested.  Loads return in the order of their issue: the filter values (from L2) go before the residual
    // (from memory), so that waiting for the former never waits for the latter.
    auto piece_body = [&](auto last_tag, auto buf_tag, int piece, int m0, const LoadSide& lsn, bool more,
                          auto next_buf_tag) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_tag)::value;
        constexpr int B = decltype(buf_tag)::value;
        if constexpr (!LAST) {
            load_w2(piece + 1, wbuf[B ^ 1]);
            if constexpr (MASKS == kResidual) load_side(cur, piece + 1, side[B ^ 1]);
        } else {
            load_chunk(lsn, 0, more, abuf[decltype(next_buf_tag)::value]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const floatx16 zero = {};
            const float mid = acc1[t / 16][t % 16];
            acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(mid, wbuf[B][t], t == 0 ? zero : acc2, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        switch (epi_flags2) {
        case 2: store_piece(std::integral_constant<int, 2>{}, acc2, side[B], m0, piece); break;
        case 3: store_piece(std::integral_constant<int, 3>{}, acc2, side[B], m0, piece); break;
        case 10: store_piece(std::integral_constant<int, 10>{}, acc2, side[B], m0, piece); break;
        default: store_piece(std::integral_constant<int, 11>{}, acc2, side[B], m0, piece); break;   // 11
        }
    };

    auto unit_body = [&](auto parity_tag) __attribute__((always_inline)) {
        constexpr int P0 = decltype(parity_tag)::value;
        const int next = claim();
        const bool more = next >= 0;
        LoadSide lsn;
        setup_load(more ? next : cur, lsn);
        const floatx4* wq0 = reinterpret_cast<const floatx4*>(wl) + ((size_t)lh * N + ln);
        // ---- first product, transposed: accumulator rows are filters, columns pixels
#pragma unroll
        for (int ch = 0; ch < kChunks; ++ch) {
            const int B = (P0 + ch) & 1;
            if (ch + 1 < kChunks)
                load_chunk(ls, ch + 1, true, abuf[B ^ 1]);
            else {
                load_w2(0, wbuf[0]);
                if constexpr (MASKS == kResidual) load_side(cur, 0, side[0]);
            }
            __builtin_amdgcn_sched_barrier(0);
            const floatx4* wq = wq0 + (size_t)(ch * 16) * N;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                floatx4 fq[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) fq[nb] = wq[(size_t)(2 * q) * N + 32 * nb];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const floatx16 zero = {};
                        acc1[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(fq[nb][i], abuf[B][q][i],
                                                                        ch == 0 && q == 0 && i == 0 ? zero : acc1[nb], 0, 0, 0);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- the first layer's bias -> BN -> ReLU, in place: register v of block nb is filter
        // 32 nb + 8 (v / 4) + 4 h + v % 4 of the lane's pixel
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                const int f0 = 32 * nb + 8 * vq + 4 * lh;
                const floatx4 b4 = *reinterpret_cast<const floatx4*>(params1 + f0);
                const floatx4 m4 = *reinterpret_cast<const floatx4*>(params1 + N + f0);
                const floatx4 s4 = *reinterpret_cast<const floatx4*>(params1 + 2 * N + f0);
                const floatx4 g4 = *reinterpret_cast<const floatx4*>(params1 + 3 * N + f0);
                const floatx4 t4 = *reinterpret_cast<const floatx4*>(params1 + 4 * N + f0);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float val = acc1[nb][4 * vq + i];
                    if (bias1) val += b4[i];
                    if (bn1) {
                        const float t = (val - m4[i]) * s4[i];
                        val = t * g4[i] + t4[i];
                    }
                    if (relu1) val = relu_of(val);
                    acc1[nb][4 * vq + i] = val;
                }
            }
        // ---- second product, 32 of its filters at a time (an even number of pieces)
        const int m0 = unit_block(cur) * 32;
        constexpr int kNextBuf = (P0 + kChunks) & 1;
        for (int piece = 0; piece + 2 < pieces; piece += 2) {
            piece_body(std::false_type{}, std::integral_constant<int, 0>{}, piece, m0, lsn, more,
                       std::integral_constant<int, 0>{});
            piece_body(std::false_type{}, std::integral_constant<int, 1>{}, piece + 1, m0, lsn, more,
                       std::integral_constant<int, 0>{});
        }
        piece_body(std::false_type{}, std::integral_constant<int, 0>{}, pieces - 2, m0, lsn, more,
                   std::integral_constant<int, 0>{});
        piece_body(std::true_type{}, std::integral_constant<int, 1>{}, pieces - 1, m0, lsn, more,
                   std::integral_constant<int, kNextBuf>{});
        ls = lsn;
        cur = next;
    };

    // nine chunks: the activations' double buffer changes parity from one unit to the next
    for (;;) {
        unit_body(std::integral_constant<int, 0>{});
        if (cur < 0) break;
        unit_body(std::integral_constant<int, 1>{});
        if (cur < 0) break;
    }
}

template <int MASKS>
int launch_pair(const PairArgs& a, hipStream_t stream)
{
    static std::atomic<unsigned> raised{0};
    const size_t lds_bytes = ((size_t)a.g.k * kN1 + 5 * kN1 + 5 * kMaxN2) * 4 + 16;
    auto kernel = conv_stream_pair_kernel<MASKS>;
    int cus = 0;
    int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), raised, 160 * 1024);
    if (rc == PYDTNN_HIP_OK) rc = device_compute_units(&cus);
    if (rc != PYDTNN_HIP_OK) return rc;
    const int grid = a.row_blocks < cus ? a.row_blocks : cus;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kPairThreads), lds_bytes, stream, a);
    HIP_RETURN_IF_LAUNCH_FAILED();
    note_launch(kLaunchPair, 32, kN1, grid, 0, 1);
    return PYDTNN_HIP_OK;
}

}  // namespace

// What the fused launch is built for: the 3x3, 64 -> 64 layer at unit stride and dilation with padding 1 (the
// middle layer of the first bottlenecks), followed by a 1x1 layer to 64, 128, 192 or 256 filters whose store
// normalises (BN, with or without bias, no ReLU of its own) and either adds a residual or does not.
bool conv_stream_pair_eligible(const ConvGeom& g, int kn2, const float* w1, const float* w2, const float* x,
                               const ChanEpilogue& chan2, const ElemMasks& masks)
{
    if (g.c != 64 || g.kn != kN1 || g.kh != 3 || g.kw != 3) return false;
    if (g.vstride != 1 || g.hstride != 1 || g.vdilation != 1 || g.hdilation != 1 || g.vpadding != 1 || g.hpadding != 1)
        return false;
    if (kn2 <= 0 || kn2 % 64 != 0 || kn2 > kMaxN2) return false;
    if (!chan2.mean || chan2.relu) return false;                       // the store variants that are built
    if (masks.gate || masks.relu_mask) return false;
    if (!aligned16(w1) || !aligned16(x) || !aligned16(w2)) return false;
    if (g.p < 32 * 1024 || g.p % 32 != 0) return false;
    return (long)g.n * g.c * g.h * g.w + (long)(g.vpadding * g.w + g.hpadding) * g.c < (1l << 29) &&
           g.p * kn2 < (1l << 29);
}

int conv_stream_pair(const ConvGeom& g, int kn2, const float* w1, const float* w2, const float* x, float* y,
                     const ChanEpilogue& chan1, const ChanEpilogue& chan2, const ElemMasks& masks, hipStream_t stream)
{
    if (!conv_stream_pair_eligible(g, kn2, w1, w2, x, chan2, masks)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    PairArgs a;
    a.x = x; a.w1 = w1; a.w2 = w2; a.y = y; a.g = g; a.chan1 = chan1; a.chan2 = chan2; a.masks = masks;
    a.n2 = kn2;
    a.row_blocks = (int)(g.p / 32);
    a.reverse = conv_stream_choose_direction(stream, x, masks.residual, y);
    return masks.residual ? launch_pair<kResidual>(a, stream) : launch_pair<kNoMasks>(a, stream);
}

}  // namespace convint

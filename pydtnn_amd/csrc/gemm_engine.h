// fp32 GEMM tile engine for gfx950 (CDNA4) on v_mfma_f32_32x32x2_f32.
//
// One workgroup = 256 threads = 4 wavefronts of 64 lanes.  It owns a BM x BN tile of C and walks
// the reduction axis in steps of BK = 16.  A and B tiles are staged through LDS, double-buffered:
// while the matrix cores consume tile t out of LDS, the global loads of tile t+1 are issued
// *between* the MFMA groups of the same wavefront (a few loads after every four MFMAs), land in
// registers, and are written to the other LDS buffer after the last MFMA, so there is one barrier
// per step and a wavefront keeps the matrix pipe fed on its own.  Every wavefront owns a 64 x 64
// sub-tile = 2 x 2 MFMA blocks of 32 x 32 (64 accumulator registers).
//
// What A(m, k) and B(k, n) *are* is decided by loader policies: plain strided matrices, or an
// implicit im2col / im2row view of an activation tensor that is never materialised.  What
// happens to C(m, n) is decided by an epilogue policy: plain row-major store, or a direct store
// into an NCHW tensor, both with the optional per-channel bias -> BN(inference) -> ReLU chain.
//
// Loads are raw buffer loads (buffer_load_dword through a 128-bit resource descriptor):
//   * an element that must read as zero (padding, reduction tail) gets the offset kOob, which is
//     beyond every descriptor's size, and the hardware returns 0: no branches in the loop;
//   * rows of A / columns of B beyond the matrix are *clamped* to the last valid one instead of
//     predicated: they only feed rows / columns of C that the epilogue never stores;
//   * a descriptor never spans more than 2 GiB and its size is the true number of bytes left in
//     the tensor, so a wrong offset reads 0 instead of faulting.
// The loop body exists in a fast form (every reduction index of the step is valid) and a tail
// form (predicated on k < kend); only the last step of a tile takes the tail form.
//
// LDS tiles are kept as [k][m] and [k][n] with rows padded by 4 floats, so that an MFMA operand
// fetch - lane l reads element (row l%32, k l/32) - is a conflict-free read of 32 consecutive
// floats per half-wave, and stores from loaders whose lanes run along k (row stride = 4 banks)
// spread over all banks.
#pragma once
#include "common.h"

namespace gemm {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int kThreads = 256;
constexpr int BK = 16;
constexpr int kPad = 4;
constexpr uint32_t kOob = 0x80000000u;       // byte offset beyond any descriptor (sizes are < 2 GiB)
constexpr long kMaxSpanBytes = 0x7fffffffl;  // largest descriptor size

template <int BM_, int BN_, int WGM_, int WGN_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 MFMA blocks");
};

// Reduction range of one workgroup.  The reduction axis is a run of `images` segments of
// `seg_len` elements each (one segment for a plain GEMM; one per image when the reduction runs
// over pixels, as in dW).  Segments are bundled into groups of `ips` consecutive images and each
// group is cut into `cpg` chunks of `chunk` elements; blockIdx.y enumerates (group, chunk) and
// partial sums of different blockIdx.y go to different slices of a workspace (split-K).
struct SplitInfo {
    int seg_len;
    int images;
    int ips;    // images per group
    int cpg;    // chunks per group
    int chunk;  // reduction elements per workgroup
};

static inline SplitInfo make_split(int seg_len, int images, int ips, int cpg, int chunk)
{
    SplitInfo s;
    s.seg_len = seg_len; s.images = images; s.ips = ips; s.cpg = cpg; s.chunk = chunk;
    return s;
}

static inline SplitInfo no_split(int k) { return make_split(k, 1, 1, 1, k); }

// ---------------------------------------------------------------- buffer access
// `p` must be wave-uniform.  `avail_elems` = floats between p and the end of the tensor.
__device__ __forceinline__ rsrc_t make_rsrc(const float* p, long avail_elems)
{
    long bytes = avail_elems * 4;
    bytes = bytes < 0 ? 0 : (bytes > kMaxSpanBytes ? kMaxSpanBytes : bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float buf_load(rsrc_t r, uint32_t voff_bytes, uint32_t soff_bytes)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff_bytes, (int)soff_bytes, 0));
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// ---------------------------------------------------------------- thread -> element maps
// MapMN: lanes run along the m (or n) axis of the tile; the k row is uniform per wavefront.
template <int BMN>
struct MapMN {
    static_assert(BMN % 64 == 0 && BMN <= kThreads, "tile extent");
    static constexpr int kRowsPerPass = kThreads / BMN;
    static constexpr int NLD = BK / kRowsPerPass;
    static __device__ __forceinline__ int mn(int tid) { return tid % BMN; }
    static __device__ __forceinline__ int krow(int tid) { return uniform(tid / BMN); }
    static __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid)
    {
        const int m = tid % BMN, k0 = tid / BMN;
#pragma unroll
        for (int e = 0; e < NLD; ++e) lds[(k0 + e * kRowsPerPass) * (BMN + kPad) + m] = r[e];
    }
};

// MapK: lanes run along k; each thread owns NLD different m (or n) positions.
template <int BMN>
struct MapK {
    static constexpr int kMnPerPass = kThreads / BK;
    static constexpr int NLD = BMN / kMnPerPass;
    static __device__ __forceinline__ int kk(int tid) { return tid % BK; }
    static __device__ __forceinline__ int mn(int tid, int e) { return tid / BK + e * kMnPerPass; }
    static __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid)
    {
        const int k = tid % BK, m0 = tid / BK;
#pragma unroll
        for (int e = 0; e < NLD; ++e) lds[k * (BMN + kPad) + m0 + e * kMnPerPass] = r[e];
    }
};

// Every loader exposes
//   State            per-thread data fixed for the whole tile
//   Iter             per-thread / per-wave data of one reduction step
//   init(State&, origin, image0, tid)
//   begin<TAIL>(State, Iter&, k0, kend)      prepare the step that starts at reduction index k0
//   elem<TAIL, E>(State, Iter, k0, kend)     value of this thread's E-th element of that step
//   store(lds, regs, tid)

// ---------------------------------------------------------------- plain strided loaders
// elem(mn, k) = base[(image0 + k / seg)*image_stride + mn*ld + k % seg]   (k contiguous inside a segment)
// With SEG == false the reduction axis is one segment: elem = base[image0*image_stride + mn*ld + k].
// Needs BMN*ld*4 (+ ips*image_stride*4 when SEG) < 2 GiB, checked on the host.
template <int BMN, bool SEG = false>
struct PlainK {
    using Map = MapK<BMN>;
    static constexpr int NLD = Map::NLD;
    const float* base;
    long total;  // floats in the tensor
    long ld;
    long image_stride;
    int extent;  // valid mn range
    int seg_len;
    FastDiv fd_seg;
    struct State {
        rsrc_t rsrc;
        uint32_t rowoff[NLD];  // byte offset of (row e, this thread's k lane)
    };
    struct Iter {
        uint32_t voff;  // per-thread byte offset of the step (or kOob)
        uint32_t soff;  // uniform byte offset of the step
    };
    __device__ __forceinline__ void init(State& s, int origin, int image0, int tid) const
    {
        const long first = (long)image0 * image_stride + (long)origin * ld;
        s.rsrc = make_rsrc(base + first, total - first);
        const int rows = min(BMN, extent - origin);
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int row = min(Map::mn(tid, e), rows - 1);
            s.rowoff[e] = (uint32_t)(row * ld + Map::kk(tid)) * 4u;
        }
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        const int k = k0 + Map::kk(threadIdx.x);
        if (SEG) {
            const uint32_t img = fd_div((uint32_t)k, fd_seg);
            it.voff = (uint32_t)((long)img * image_stride - (long)img * seg_len) * 4u;
        } else {
            it.voff = 0;
        }
        it.soff = (uint32_t)k0 * 4u;
        if (TAIL && k >= kend) it.voff = kOob;
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        return buf_load(s.rsrc, s.rowoff[E] + it.voff, it.soff);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// elem(mn, k) = base[image*image_stride + k*ld + mn]   (mn contiguous).  The descriptor is re-based to
// row k0 at every step, so only BK*ld*4 < 2 GiB is needed (checked on the host).
template <int BMN>
struct PlainMN {
    using Map = MapMN<BMN>;
    static constexpr int NLD = Map::NLD;
    const float* base;
    long total;
    long ld;
    long image_stride;
    int extent;
    struct State {
        long first;     // float index of (image, row 0, column 0)
        uint32_t voff;  // byte offset of this thread's (clamped) column
        int krow;
    };
    struct Iter {
        rsrc_t rsrc;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image, int tid) const
    {
        s.first = (long)image * image_stride;
        s.voff = (uint32_t)min(origin + Map::mn(tid), extent - 1) * 4u;
        s.krow = Map::krow(tid);
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State& s, Iter& it, int k0, int) const
    {
        const long row0 = s.first + (long)(k0 + s.krow) * ld;
        it.rsrc = make_rsrc(base + row0, total - row0);
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int k0, int kend) const
    {
        const uint32_t soff = (uint32_t)(E * Map::kRowsPerPass) * (uint32_t)ld * 4u;
        uint32_t voff = s.voff;
        if (TAIL && k0 + s.krow + E * Map::kRowsPerPass >= kend) voff = kOob;
        return buf_load(it.rsrc, voff, soff);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// ---------------------------------------------------------------- implicit im2col, NCHW
// Taps of one reduction step, decomposed by the lanes of a wavefront in parallel: lane l holds the
// tap with reduction index k0 + (l % 16); a wave-uniform tap is then fetched with v_readlane.
struct TapLanes {
    int off;  // c*h*w + (i*dv)*w + j*dh  (float offset of the tap inside one image)
    int dij;  // (i*dv) << 16 | (j*dh)
};

template <bool TAIL>
__device__ __forceinline__ TapLanes nchw_taps(const ConvGeom& g, int k0, int kend)
{
    const uint32_t k = (uint32_t)(k0 + (threadIdx.x & (BK - 1)));
    const uint32_t cc = fd_div(k, g.fd_khw);
    const uint32_t rem = k - cc * g.khw;
    const uint32_t ii = fd_div(rem, g.fd_kw);
    const uint32_t jj = rem - ii * g.kw;
    int di = (int)ii * g.vdilation;
    const int dj = (int)jj * g.hdilation;
    TapLanes t;
    t.off = ((int)cc * g.h + di) * g.w + dj;
    if (TAIL && (int)k >= kend) di = 0x4000;  // fails every row bound test (h + padding < 8192)
    t.dij = (di << 16) | dj;
    return t;
}

// B(k = (c,i,j), n = (img,y,x)) = X[img, c, sv*y + dv*i - pv, sh*x + dh*j - ph]: the column matrix of
// pydtnn/cython_modules/im2col_nchw_cython.pyx:104-124, never written to memory.
// Lanes run along the pixel axis (contiguous in x for a fixed tap); the tap (c,i,j) is wave-uniform.
template <int BN>
struct Im2colNchwMN {
    using Map = MapMN<BN>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        int base;  // float index of (img, c=0, ih0, iw0); may be negative, only used with an in-range tap
        int ih0, iw0;
        int krow;
    };
    struct Iter {
        TapLanes taps;
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        s.rsrc = make_rsrc(x, (long)g.n * g.c * g.h * g.w);
        long n = (long)origin + Map::mn(tid);
        n = n < g.p ? n : g.p - 1;
        const int img = (int)(n / g.howo);
        const int pp = (int)(n - (long)img * g.howo);
        const int yy = pp / g.wo, xx = pp - yy * g.wo;
        s.ih0 = yy * g.vstride - g.vpadding;
        s.iw0 = xx * g.hstride - g.hpadding;
        s.krow = Map::krow(tid);
        s.base = (img * g.c * g.h + s.ih0) * g.w + s.iw0;
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        it.taps = nchw_taps<TAIL>(g, k0, kend);
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        const int lane = s.krow + E * Map::kRowsPerPass;
        const int off = __builtin_amdgcn_readlane(it.taps.off, lane);
        const int dij = __builtin_amdgcn_readlane(it.taps.dij, lane);
        const int di = dij >> 16, dj = dij & 0xffff;
        const bool ok = (unsigned)(s.ih0 + di) < (unsigned)g.h && (unsigned)(s.iw0 + dj) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(s.base + off) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// dW view of the same matrix: B(k = (image, pixel), n = (c,i,j)).  Lanes run along the pixel (reduction)
// axis; each thread owns NLD fixed taps.
template <int BN>
struct Im2colNchwK {
    using Map = MapK<BN>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        int image0;
        int coff[NLD];  // c*h*w + i*dv*w + j*dh
        int di[NLD], dj[NLD];
    };
    struct Iter {
        int base;  // float index of (img, c=0, ih0, iw0)
        int ih0, iw0;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image0, int tid) const
    {
        s.rsrc = make_rsrc(x, (long)g.n * g.c * g.h * g.w);
        s.image0 = image0;
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int n = min(origin + Map::mn(tid, e), g.k - 1);
            const int cc = n / g.khw, rem = n - cc * g.khw;
            const int ii = rem / g.kw, jj = rem - ii * g.kw;
            s.di[e] = ii * g.vdilation;
            s.dj[e] = jj * g.hdilation;
            s.coff[e] = (cc * g.h + s.di[e]) * g.w + s.dj[e];
        }
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State& s, Iter& it, int k0, int kend) const
    {
        const int k = k0 + Map::kk(threadIdx.x);  // (image within the group, pixel)
        const uint32_t img = fd_div((uint32_t)k, g.fd_howo);
        const uint32_t pp = (uint32_t)k - img * g.howo;
        const uint32_t yy = fd_div(pp, g.fd_wo);
        const uint32_t xx = pp - yy * g.wo;
        it.ih0 = (int)yy * g.vstride - g.vpadding;
        it.iw0 = (int)xx * g.hstride - g.hpadding;
        it.base = ((s.image0 + (int)img) * g.c * g.h + it.ih0) * g.w + it.iw0;
        if (TAIL && k >= kend) it.ih0 = -(1 << 20);  // fails every bound test
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        const bool ok = (unsigned)(it.ih0 + s.di[E]) < (unsigned)g.h && (unsigned)(it.iw0 + s.dj[E]) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(it.base + s.coff[E]) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// ---------------------------------------------------------------- implicit im2row, NHWC
// A(m = (img,y,x), k) = X[img, sv*y + dv*i - pv, sh*x + dh*j - ph, c] with the reduction index walked
// in (i, j, c) order so that lanes along k read consecutive channels.  The reference orders K as
// (c, i, j) (pydtnn/cython_modules/im2row_nhwc_cython.pyx:96); a sum over K does not depend on the
// order, and the filter loader below applies the same permutation to the rows of W.
template <int BM>
struct Im2rowNhwcK {
    using Map = MapK<BM>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        int base[NLD];  // ((img*h + ih0)*w + iw0)*c, may be negative when padding reaches outside
        int ih0[NLD], iw0[NLD];
    };
    struct Iter {
        int koff;  // (di*w + dj)*c + channel
        int di, dj;
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        s.rsrc = make_rsrc(x, (long)g.n * g.c * g.h * g.w);
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            long m = (long)origin + Map::mn(tid, e);
            m = m < g.p ? m : g.p - 1;
            const int img = (int)(m / g.howo);
            const int pp = (int)(m - (long)img * g.howo);
            const int yy = pp / g.wo, xx = pp - yy * g.wo;
            s.ih0[e] = yy * g.vstride - g.vpadding;
            s.iw0[e] = xx * g.hstride - g.hpadding;
            s.base[e] = ((img * g.h + s.ih0[e]) * g.w + s.iw0[e]) * g.c;
        }
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        const uint32_t k = (uint32_t)(k0 + Map::kk(threadIdx.x));
        const uint32_t ij = fd_div(k, g.fd_c);
        const uint32_t cc = k - ij * g.c;
        const uint32_t ii = fd_div(ij, g.fd_kw);
        const uint32_t jj = ij - ii * g.kw;
        it.di = (int)ii * g.vdilation;
        it.dj = (int)jj * g.hdilation;
        it.koff = (it.di * g.w + it.dj) * g.c + (int)cc;
        if (TAIL && (int)k >= kend) it.di = 1 << 20;
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        const bool ok = (unsigned)(s.ih0[E] + it.di) < (unsigned)g.h && (unsigned)(s.iw0[E] + it.dj) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(s.base[E] + it.koff) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// Filter in NHWC layout (c, kh, kw, kn) read as B(k in (i,j,c) order, n = filter).
template <int BN>
struct FilterNhwcMN {
    using Map = MapMN<BN>;
    static constexpr int NLD = Map::NLD;
    const float* w;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        uint32_t voff;
        int krow;
    };
    struct Iter {
        int row;  // per lane: filter row c*kh*kw + i*kw + j of reduction index k0 + lane%16
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        s.rsrc = make_rsrc(w, (long)g.k * g.kn);
        s.voff = (uint32_t)min(origin + Map::mn(tid), g.kn - 1) * 4u;
        s.krow = Map::krow(tid);
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int) const
    {
        const uint32_t k = (uint32_t)(k0 + (threadIdx.x & (BK - 1)));
        const uint32_t ij = fd_div(k, g.fd_c);
        const uint32_t cc = k - ij * g.c;
        it.row = (int)(cc * g.khw + ij);
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int k0, int kend) const
    {
        const int lane = s.krow + E * Map::kRowsPerPass;
        const uint32_t row = (uint32_t)__builtin_amdgcn_readlane(it.row, lane);
        uint32_t voff = s.voff;
        if (TAIL && k0 + lane >= kend) voff = kOob;
        return buf_load(s.rsrc, voff, row * (uint32_t)g.kn * 4u);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// dW view in NHWC: A(m = (i,j,c), k = (image, pixel)).  Lanes run along m (consecutive channels);
// the pixel is wave-uniform and decomposed by the lanes in parallel.
template <int BM>
struct Im2rowNhwcMN {
    using Map = MapMN<BM>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        int moff;  // (di*w + dj)*c + channel
        int di, dj;
        int krow;
        int image0;
    };
    struct Iter {
        int pix;  // per lane: (img*h + ih0)*w + iw0 of reduction index k0 + lane%16 (may be negative)
        int ihw;  // per lane: (ih0 + 0x4000) << 16 | (iw0 + 0x4000)
    };
    __device__ __forceinline__ void init(State& s, int origin, int image0, int tid) const
    {
        s.rsrc = make_rsrc(x, (long)g.n * g.c * g.h * g.w);
        const int m = min(origin + Map::mn(tid), g.k - 1);
        const int ij = m / g.c, cc = m - ij * g.c;
        const int ii = ij / g.kw, jj = ij - ii * g.kw;
        s.di = ii * g.vdilation;
        s.dj = jj * g.hdilation;
        s.moff = (s.di * g.w + s.dj) * g.c + cc;
        s.krow = Map::krow(tid);
        s.image0 = image0;
    }
    template <bool TAIL>
    __device__ __forceinline__ void begin(const State& s, Iter& it, int k0, int kend) const
    {
        const uint32_t k = (uint32_t)(k0 + (threadIdx.x & (BK - 1)));  // (image within the group, pixel)
        const uint32_t img = fd_div(k, g.fd_howo);
        const uint32_t pp = k - img * g.howo;
        const uint32_t yy = fd_div(pp, g.fd_wo);
        const uint32_t xx = pp - yy * g.wo;
        int ih0 = (int)yy * g.vstride - g.vpadding;
        const int iw0 = (int)xx * g.hstride - g.hpadding;
        it.pix = ((s.image0 + (int)img) * g.h + ih0) * g.w + iw0;
        if (TAIL && (int)k >= kend) ih0 = 0x2000;  // fails every row bound test (h < 8192)
        it.ihw = ((ih0 + 0x4000) << 16) | (iw0 + 0x4000);
    }
    template <bool TAIL, int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        const int lane = s.krow + E * Map::kRowsPerPass;
        const int pix = __builtin_amdgcn_readlane(it.pix, lane);
        const int ihw = __builtin_amdgcn_readlane(it.ihw, lane);
        const int ih0 = (ihw >> 16) - 0x4000, iw0 = (ihw & 0xffff) - 0x4000;
        const bool ok = (unsigned)(ih0 + s.di) < (unsigned)g.h && (unsigned)(iw0 + s.dj) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(pix * g.c + s.moff) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// ---------------------------------------------------------------- epilogues
// Row-major store C[split*split_stride + m*ldc + n]; the per-channel chain uses the column index
// (NHWC convolution, FC forward).
struct EpiPlain {
    float* out;
    long ldc;
    long split_stride;
    int m_extent, n_extent;
    ChanEpilogue chan;
    struct Col {
        float* ptr;
        int n;
        bool ok;
    };
    __device__ __forceinline__ Col column(int n, int split) const
    {
        Col c;
        c.n = n;
        c.ok = n < n_extent;
        c.ptr = out + (long)split * split_stride + n;
        return c;
    }
    __device__ __forceinline__ void store(const Col& c, int m, float v) const
    {
        if (c.ok && m < m_extent) c.ptr[(long)m * ldc] = chan_epilogue_apply(chan, c.n, v);
    }
};

// Direct store into an NCHW tensor: row m = output channel, column n = (img, pixel):
// out[(img*m_extent + m)*howo + pixel].  This folds the reference's bias pass
// (add_nchw_cython.pyx:57-58) and its (co,N,ho,wo)->(N,co,ho,wo) copy
// (conv_2d_cpu.py:288) into the GEMM's only store.  Channel = row.
struct EpiNchw {
    float* out;
    int m_extent;  // output channels
    int howo;
    long p;        // images * howo
    ChanEpilogue chan;
    struct Col {
        float* ptr;
        bool ok;
    };
    __device__ __forceinline__ Col column(int n, int /*split*/) const
    {
        Col c;
        c.ok = n < p;
        const int nc = c.ok ? n : 0;
        const int img = nc / howo;
        const int pp = nc - img * howo;
        c.ptr = out + (long)img * m_extent * howo + pp;
        return c;
    }
    __device__ __forceinline__ void store(const Col& c, int m, float v) const
    {
        if (c.ok && m < m_extent) c.ptr[(long)m * howo] = chan_epilogue_apply(chan, m, v);
    }
};

// ---------------------------------------------------------------- the kernel
// Workgroups of one launch are handed to the 8 XCDs round-robin; remap the linear id so that each
// XCD works on one contiguous run of tiles (neighbouring tiles share A or B rows in that XCD's L2).
__device__ __forceinline__ int xcd_remap(int bid, int nblocks)
{
    const int q = nblocks >> 3, r = nblocks & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    return xcd < r ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
}

// Loads of one reduction step are spread over the BK/2 MFMA groups of the step: group J issues the
// elements E with E*(BK/2)/NLD == J.
template <bool TAIL, int J, int E, class L>
__device__ __forceinline__ void group_load(const L& l, const typename L::State& s, const typename L::Iter& it,
                                           float (&r)[L::NLD], int k0, int kend)
{
    if constexpr (E < L::NLD) {
        if constexpr (E * (BK / 2) / L::NLD == J) r[E] = l.template elem<TAIL, E>(s, it, k0, kend);
        group_load<TAIL, J, E + 1, L>(l, s, it, r, k0, kend);
    }
}

template <bool TAIL, int E, class L>
__device__ __forceinline__ void load_all(const L& l, const typename L::State& s, const typename L::Iter& it,
                                         float (&r)[L::NLD], int k0, int kend)
{
    if constexpr (E < L::NLD) {
        r[E] = l.template elem<TAIL, E>(s, it, k0, kend);
        load_all<TAIL, E + 1, L>(l, s, it, r, k0, kend);
    }
}

// One MFMA group (k-step J of the LDS tile) and everything scheduled around it.
// LOADS: 0 = last step of the tile (nothing to prefetch), 1 = prefetch a full step, 2 = prefetch the tail step
template <class T, int LOADS, int J, class AL, class BL>
__device__ __forceinline__ void mfma_groups(const AL& al, const BL& bl, const typename AL::State& as,
                                            const typename BL::State& bs, const typename AL::Iter& ai,
                                            const typename BL::Iter& bi, float (&ra)[AL::NLD], float (&rb)[BL::NLD],
                                            const float* a_lds, const float* b_lds, floatx16 (&acc)[T::TM][T::TN],
                                            float (&af)[2][T::TM], float (&bf)[2][T::TN], int knext, int kend)
{
    constexpr int G = BK / 2;
    if constexpr (J < G) {
        if constexpr (J + 1 < G) {  // operands of the next group are fetched before this group's MFMAs issue
#pragma unroll
            for (int i = 0; i < T::TM; ++i) af[(J + 1) & 1][i] = a_lds[2 * (J + 1) * (T::BM + kPad) + i * 32];
#pragma unroll
            for (int j = 0; j < T::TN; ++j) bf[(J + 1) & 1][j] = b_lds[2 * (J + 1) * (T::BN + kPad) + j * 32];
        }
        if constexpr (LOADS == 1) {
            group_load<false, J, 0, AL>(al, as, ai, ra, knext, kend);
            group_load<false, J, 0, BL>(bl, bs, bi, rb, knext, kend);
        } else if constexpr (LOADS == 2) {
            group_load<true, J, 0, AL>(al, as, ai, ra, knext, kend);
            group_load<true, J, 0, BL>(bl, bs, bi, rb, knext, kend);
        }
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
            for (int j = 0; j < T::TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[J & 1][i], bf[J & 1][j], acc[i][j], 0, 0, 0);
        // keep this group's LDS fetches, global loads and MFMAs together: the instruction scheduler
        // must not sink the loads to the end of the step
        __builtin_amdgcn_sched_barrier(0);
        mfma_groups<T, LOADS, J + 1, AL, BL>(al, bl, as, bs, ai, bi, ra, rb, a_lds, b_lds, acc, af, bf, knext, kend);
    }
}

template <class T, int LOADS, class AL, class BL>
__device__ __forceinline__ void step(const AL& al, const BL& bl, const typename AL::State& as,
                                     const typename BL::State& bs, float (&ra)[AL::NLD], float (&rb)[BL::NLD],
                                     const float* a_lds, const float* b_lds, floatx16 (&acc)[T::TM][T::TN], int knext,
                                     int kend)
{
    typename AL::Iter ai;
    typename BL::Iter bi;
    if constexpr (LOADS == 1) {
        al.template begin<false>(as, ai, knext, kend);
        bl.template begin<false>(bs, bi, knext, kend);
    } else if constexpr (LOADS == 2) {
        al.template begin<true>(as, ai, knext, kend);
        bl.template begin<true>(bs, bi, knext, kend);
    }
    float af[2][T::TM], bf[2][T::TN];
#pragma unroll
    for (int i = 0; i < T::TM; ++i) af[0][i] = a_lds[i * 32];
#pragma unroll
    for (int j = 0; j < T::TN; ++j) bf[0][j] = b_lds[j * 32];
    mfma_groups<T, LOADS, 0, AL, BL>(al, bl, as, bs, ai, bi, ra, rb, a_lds, b_lds, acc, af, bf, knext, kend);
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) gemm_kernel(AL al, BL bl, EP ep, int tiles_m, SplitInfo si)
{
    __shared__ float As[2][BK * (T::BM + kPad)];
    __shared__ float Bs[2][BK * (T::BN + kPad)];

    const int tid = threadIdx.x;
    const int tile = xcd_remap(blockIdx.x, gridDim.x);
    const int tm_idx = tile % tiles_m, tn_idx = tile / tiles_m;
    const int m0 = tm_idx * T::BM, n0 = tn_idx * T::BN;
    const int split = blockIdx.y;
    const int group = split / si.cpg;
    const int chunk_idx = split - group * si.cpg;
    const int image = group * si.ips;  // first image of this workgroup's group
    const int k_total = min(si.ips, si.images - image) * si.seg_len;
    const int kbeg = chunk_idx * si.chunk;
    const int kend = min(k_total, kbeg + si.chunk);

    typename AL::State as;
    typename BL::State bs;
    al.init(as, m0, image, tid);
    bl.init(bs, n0, image, tid);

    float ra[AL::NLD], rb[BL::NLD];
    floatx16 acc[T::TM][T::TN];
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;

    {   // first tile: tail form (correct for any kend, including an empty range)
        typename AL::Iter ai;
        typename BL::Iter bi;
        al.template begin<true>(as, ai, kbeg, kend);
        bl.template begin<true>(bs, bi, kbeg, kend);
        load_all<true, 0, AL>(al, as, ai, ra, kbeg, kend);
        load_all<true, 0, BL>(bl, bs, bi, rb, kbeg, kend);
    }
    al.store(As[0], ra, tid);
    bl.store(Bs[0], rb, tid);
    __syncthreads();

    // Steady state: the step being prefetched is a full one, so the loop body exists in one form.
    int cur = 0;
    int k0 = kbeg;
    for (; k0 + 2 * BK <= kend; k0 += BK) {
        const float* a_lds = As[cur] + frag_k * (T::BM + kPad) + wm0 + frag_r;
        const float* b_lds = Bs[cur] + frag_k * (T::BN + kPad) + wn0 + frag_r;
        step<T, 1>(al, bl, as, bs, ra, rb, a_lds, b_lds, acc, k0 + BK, kend);
        al.store(As[cur ^ 1], ra, tid);
        bl.store(Bs[cur ^ 1], rb, tid);
        __syncthreads();
        cur ^= 1;
    }
    if (k0 + BK < kend) {  // the next step is the partial one at the end of the reduction range
        const float* a_lds = As[cur] + frag_k * (T::BM + kPad) + wm0 + frag_r;
        const float* b_lds = Bs[cur] + frag_k * (T::BN + kPad) + wn0 + frag_r;
        step<T, 2>(al, bl, as, bs, ra, rb, a_lds, b_lds, acc, k0 + BK, kend);
        al.store(As[cur ^ 1], ra, tid);
        bl.store(Bs[cur ^ 1], rb, tid);
        __syncthreads();
        cur ^= 1;
        k0 += BK;
    }
    if (k0 < kend) {  // last step: nothing left to prefetch
        const float* a_lds = As[cur] + frag_k * (T::BM + kPad) + wm0 + frag_r;
        const float* b_lds = Bs[cur] + frag_k * (T::BN + kPad) + wn0 + frag_r;
        step<T, 0>(al, bl, as, bs, ra, rb, a_lds, b_lds, acc, k0 + BK, kend);
    }

    // Accumulator layout of v_mfma_f32_32x32x2_f32: register v of lane l holds
    // C[8*(v/4) + 4*(l/32) + v%4][l%32] of the 32x32 block.
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
        const typename EP::Col col = ep.column(n0 + wn0 + j * 32 + frag_r, split);
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm0 + i * 32 + 8 * (v / 4) + 4 * frag_k + (v % 4);
                ep.store(col, m, acc[i][j][v]);
            }
    }
}

template <class T, class AL, class BL, class EP>
inline int launch(const AL& al, const BL& bl, const EP& ep, long m, long n, const SplitInfo& si, int splits,
                  hipStream_t stream)
{
    const long tiles_m = (m + T::BM - 1) / T::BM, tiles_n = (n + T::BN - 1) / T::BN;
    if (tiles_m * tiles_n >= (1l << 31) || splits > 65535 || splits < 1) return PYDTNN_HIP_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)splits);
    hipLaunchKernelGGL((gemm_kernel<T, AL, BL, EP>), grid, dim3(kThreads), 0, stream, al, bl, ep, (int)tiles_m, si);
    HIP_RETURN_IF_LAUNCH_FAILED();
    return PYDTNN_HIP_OK;
}

}  // namespace gemm

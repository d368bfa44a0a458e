// fp32 GEMM tile engine for gfx950 (CDNA4) on v_mfma_f32_32x32x2_f32.
//
// One workgroup = 256 threads = 4 wavefronts of 64 lanes.  It owns a BM x BN tile of C and walks
// the reduction axis in steps of BK = 16.  A and B tiles are staged through LDS, double-buffered:
// while the matrix cores consume tile t out of LDS, the global loads of tile t+1 are in flight in
// registers and are written to the other LDS buffer after the MFMA block, so there is one barrier
// per step.  Every wavefront owns a 64 x 64 sub-tile = 2 x 2 MFMA blocks of 32 x 32 (64
// accumulator registers), which keeps 2-3 workgroups resident per CU.
//
// What A(m, k) and B(k, n) *are* is decided by loader policies: plain strided matrices, or an
// implicit im2col / im2row view of an activation tensor that is never materialised.  What
// happens to C(m, n) is decided by an epilogue policy: plain row-major store, or a direct store
// into an NCHW tensor, both with the optional per-channel bias -> BN(inference) -> ReLU chain.
//
// LDS tiles are kept as [k][m] and [k][n] (row length padded by 2 floats) so that an MFMA
// operand fetch - lane l reads element (row l%32, k l/32) - is a conflict-free ds_read_b32 of 32
// consecutive floats per half-wave, and so that stores from loaders whose lanes run along k hit
// distinct banks.
#pragma once
#include "common.h"

namespace gemm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BK = 16;
constexpr int kPad = 2;

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
    FastDiv fd_seg;
};

static inline SplitInfo make_split(int seg_len, int images, int ips, int cpg, int chunk)
{
    SplitInfo s;
    s.seg_len = seg_len; s.images = images; s.ips = ips; s.cpg = cpg; s.chunk = chunk;
    s.fd_seg = make_fastdiv((uint32_t)seg_len);
    return s;
}

static inline SplitInfo no_split(int k) { return make_split(k, 1, 1, 1, k); }

// ---------------------------------------------------------------- thread -> element maps
// MapMN: lanes run along the m (or n) axis of the tile; k row is uniform per wavefront.
template <int BMN>
struct MapMN {
    static_assert(BMN % 64 == 0 && BMN <= kThreads, "tile extent");
    static constexpr int kRowsPerPass = kThreads / BMN;
    static constexpr int NLD = BK / kRowsPerPass;
    static __device__ __forceinline__ int mn(int tid) { return tid % BMN; }
    // wave-uniform, held in an SGPR
    static __device__ __forceinline__ int krow(int tid) { return __builtin_amdgcn_readfirstlane(tid / BMN); }
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

// ---------------------------------------------------------------- plain strided loaders
// elem(mn, k) = base[(image0 + k / seg)*image_stride + mn*ld + k % seg]   (k contiguous inside a segment)
// With SEG == false the reduction axis is one segment: elem = base[image0*image_stride + mn*ld + k].
template <int BMN, bool SEG = false>
struct PlainK {
    using Map = MapK<BMN>;
    static constexpr int NLD = Map::NLD;
    const float* base;
    long ld;
    long image_stride;
    int extent;  // valid mn range
    int seg_len;
    FastDiv fd_seg;
    struct State {
        const float* ptr;  // element (first mn of this thread, kk of this thread, k = 0)
        int mn0;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image0, int tid) const
    {
        s.mn0 = origin + Map::mn(tid, 0);
        s.ptr = base + (long)image0 * image_stride + (long)s.mn0 * ld + Map::kk(tid);
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
        const int k = k0 + Map::kk(threadIdx.x);
        const bool kok = k < kend;
        long koff = k0;
        if (SEG) {
            const uint32_t img = fd_div((uint32_t)k, fd_seg);
            koff = (long)img * image_stride + (k0 - (int)(img * (uint32_t)seg_len));
        }
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const bool ok = kok && (s.mn0 + e * Map::kMnPerPass) < extent;
            r[e] = ok ? s.ptr[(long)e * Map::kMnPerPass * ld + koff] : 0.0f;
        }
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// elem(mn, k) = base[image*image_stride + k*ld + mn]   (mn contiguous)
template <int BMN>
struct PlainMN {
    using Map = MapMN<BMN>;
    static constexpr int NLD = Map::NLD;
    const float* base;
    long ld;
    long image_stride;
    int extent;
    struct State {
        const float* ptr;
        int krow;
        bool ok;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image, int tid) const
    {
        const int mn = origin + Map::mn(tid);
        s.ok = mn < extent;
        s.krow = Map::krow(tid);
        s.ptr = base + (long)image * image_stride + mn;
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int k = k0 + s.krow + e * Map::kRowsPerPass;
            r[e] = (s.ok && k < kend) ? s.ptr[(long)k * ld] : 0.0f;
        }
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// ---------------------------------------------------------------- implicit im2col, NCHW
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
        const float* ptr;  // x + offset of (img, c=0, ih0, iw0); only dereferenced with an in-range tap
        int ih0, iw0;
        int krow;
        bool ok;
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        const long n = (long)origin + Map::mn(tid);
        s.ok = n < g.p;
        const long nc = s.ok ? n : 0;
        const int img = (int)(nc / g.howo);
        const int pp = (int)(nc - (long)img * g.howo);
        const int yy = pp / g.wo, xx = pp - yy * g.wo;
        s.ih0 = yy * g.vstride - g.vpadding;
        s.iw0 = xx * g.hstride - g.hpadding;
        s.krow = Map::krow(tid);
        s.ptr = x + (long)img * g.c * g.h * g.w + (long)s.ih0 * g.w + s.iw0;
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const uint32_t k = (uint32_t)(k0 + s.krow + e * Map::kRowsPerPass);
            const uint32_t cc = fd_div(k, g.fd_khw);
            const uint32_t rem = k - cc * g.khw;
            const uint32_t ii = fd_div(rem, g.fd_kw);
            const uint32_t jj = rem - ii * g.kw;
            const int di = (int)ii * g.vdilation, dj = (int)jj * g.hdilation;
            const int koff = ((int)cc * g.h + di) * g.w + dj;
            const bool ok = s.ok && (int)k < kend && (unsigned)(s.ih0 + di) < (unsigned)g.h &&
                            (unsigned)(s.iw0 + dj) < (unsigned)g.w;
            r[e] = ok ? s.ptr[koff] : 0.0f;
        }
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// dW view of the same matrix: B(k = pixel (y,x) of one image, n = (c,i,j)).  Lanes run along the
// pixel (reduction) axis; each thread owns NLD fixed taps.
template <int BN>
struct Im2colNchwK {
    using Map = MapK<BN>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        const float* img;
        int coff[NLD];  // c*h*w + i*dv*w + j*dh
        int dij[NLD];   // (i*dv) << 16 | (j*dh)
        unsigned vmask;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image, int tid) const
    {
        s.img = x + (long)image * g.c * g.h * g.w;
        s.vmask = 0;
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int n = origin + Map::mn(tid, e);
            const bool ok = n < g.k;
            const int nc = ok ? n : 0;
            const int cc = nc / g.khw, rem = nc - cc * g.khw;
            const int ii = rem / g.kw, jj = rem - ii * g.kw;
            const int di = ii * g.vdilation, dj = jj * g.hdilation;
            s.coff[e] = (cc * g.h + di) * g.w + dj;
            s.dij[e] = (di << 16) | dj;
            if (ok) s.vmask |= 1u << e;
        }
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
        const int k = k0 + Map::kk(threadIdx.x);  // (image within the group, pixel)
        const bool pok = k < kend;
        const uint32_t img = fd_div((uint32_t)k, g.fd_howo);
        const uint32_t pp = (uint32_t)k - img * g.howo;
        const uint32_t yy = fd_div(pp, g.fd_wo);
        const uint32_t xx = pp - yy * g.wo;
        const int ih0 = (int)yy * g.vstride - g.vpadding;
        const int iw0 = (int)xx * g.hstride - g.hpadding;
        const float* p0 = s.img + (long)img * g.c * g.h * g.w + (long)ih0 * g.w + iw0;
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int di = s.dij[e] >> 16, dj = s.dij[e] & 0xffff;
            const bool ok = pok && ((s.vmask >> e) & 1u) && (unsigned)(ih0 + di) < (unsigned)g.h &&
                            (unsigned)(iw0 + dj) < (unsigned)g.w;
            r[e] = ok ? p0[s.coff[e]] : 0.0f;
        }
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
        int base[NLD];  // ((img*h + ih0)*w + iw0)*c, may be negative when padding reaches outside
        int ih0[NLD], iw0[NLD];
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const long m = (long)origin + Map::mn(tid, e);
            const bool ok = m < g.p;
            const long mc = ok ? m : 0;
            const int img = (int)(mc / g.howo);
            const int pp = (int)(mc - (long)img * g.howo);
            const int yy = pp / g.wo, xx = pp - yy * g.wo;
            const int ih0 = yy * g.vstride - g.vpadding, iw0 = xx * g.hstride - g.hpadding;
            s.ih0[e] = ok ? ih0 : -(1 << 28);  // fails every bounds test
            s.iw0[e] = iw0;
            s.base[e] = ((img * g.h + ih0) * g.w + iw0) * g.c;
        }
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
        const uint32_t k = (uint32_t)(k0 + Map::kk(threadIdx.x));
        const bool kok = (int)k < kend;
        const uint32_t ij = fd_div(k, g.fd_c);
        const uint32_t cc = k - ij * g.c;
        const uint32_t ii = fd_div(ij, g.fd_kw);
        const uint32_t jj = ij - ii * g.kw;
        const int di = (int)ii * g.vdilation, dj = (int)jj * g.hdilation;
        const int koff = (di * g.w + dj) * g.c + (int)cc;
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const bool ok = kok && (unsigned)(s.ih0[e] + di) < (unsigned)g.h && (unsigned)(s.iw0[e] + dj) < (unsigned)g.w;
            r[e] = ok ? x[(long)s.base[e] + koff] : 0.0f;
        }
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
        const float* ptr;
        int krow;
        bool ok;
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        const int n = origin + Map::mn(tid);
        s.ok = n < g.kn;
        s.krow = Map::krow(tid);
        s.ptr = w + n;
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const uint32_t k = (uint32_t)(k0 + s.krow + e * Map::kRowsPerPass);
            const uint32_t ij = fd_div(k, g.fd_c);
            const uint32_t cc = k - ij * g.c;
            const uint32_t row = cc * g.khw + ij;
            r[e] = (s.ok && (int)k < kend) ? s.ptr[(long)row * g.kn] : 0.0f;
        }
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
};

// dW view in NHWC: A(m = (i,j,c), k = pixel (y,x) of one image).  Lanes run along m (consecutive
// channels); the pixel is wave-uniform.
template <int BM>
struct Im2rowNhwcMN {
    using Map = MapMN<BM>;
    static constexpr int NLD = Map::NLD;
    const float* x;
    ConvGeom g;
    struct State {
        const float* ptr;  // image base + (di*w + dj)*c + c
        int di, dj;
        int krow;
        bool ok;
    };
    __device__ __forceinline__ void init(State& s, int origin, int image, int tid) const
    {
        const int m = origin + Map::mn(tid);
        s.ok = m < g.k;
        const int mc = s.ok ? m : 0;
        const int ij = mc / g.c, cc = mc - ij * g.c;
        const int ii = ij / g.kw, jj = ij - ii * g.kw;
        s.di = ii * g.vdilation;
        s.dj = jj * g.hdilation;
        s.krow = Map::krow(tid);
        s.ptr = x + (long)image * g.h * g.w * g.c + (long)(s.di * g.w + s.dj) * g.c + cc;
    }
    __device__ __forceinline__ void load(const State& s, float (&r)[NLD], int k0, int kend) const
    {
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const uint32_t k = (uint32_t)(k0 + s.krow + e * Map::kRowsPerPass);  // (image within the group, pixel)
            const uint32_t img = fd_div(k, g.fd_howo);
            const uint32_t pp = k - img * g.howo;
            const uint32_t yy = fd_div(pp, g.fd_wo);
            const uint32_t xx = pp - yy * g.wo;
            const int ih0 = (int)yy * g.vstride - g.vpadding, iw0 = (int)xx * g.hstride - g.hpadding;
            const bool ok = s.ok && (int)k < kend && (unsigned)(ih0 + s.di) < (unsigned)g.h &&
                            (unsigned)(iw0 + s.dj) < (unsigned)g.w;
            r[e] = ok ? s.ptr[(long)(((int)img * g.h + ih0) * g.w + iw0) * g.c] : 0.0f;
        }
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

    al.load(as, ra, kbeg, kend);
    bl.load(bs, rb, kbeg, kend);
    al.store(As[0], ra, tid);
    bl.store(Bs[0], rb, tid);
    __syncthreads();

    int cur = 0;
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        const bool more = k0 + BK < kend;
        if (more) {
            al.load(as, ra, k0 + BK, kend);
            bl.load(bs, rb, k0 + BK, kend);
        }
        const float* a_lds = As[cur] + frag_k * (T::BM + kPad) + wm0 + frag_r;
        const float* b_lds = Bs[cur] + frag_k * (T::BN + kPad) + wn0 + frag_r;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float af[T::TM], bf[T::TN];
#pragma unroll
            for (int i = 0; i < T::TM; ++i) af[i] = a_lds[kk * (T::BM + kPad) + i * 32];
#pragma unroll
            for (int j = 0; j < T::TN; ++j) bf[j] = b_lds[kk * (T::BN + kPad) + j * 32];
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
#pragma unroll
                for (int j = 0; j < T::TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            al.store(As[cur ^ 1], ra, tid);
            bl.store(Bs[cur ^ 1], rb, tid);
        }
        __syncthreads();
        cur ^= 1;
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

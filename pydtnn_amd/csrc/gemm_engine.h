// fp32 GEMM tile engine for gfx950 (CDNA4) on v_mfma_f32_32x32x2_f32.
//
// One workgroup = 256 threads = 4 wavefronts of 64 lanes.  It owns a BM x BN tile of C and walks
// the reduction axis in steps of BK = 16.  A and B tiles are staged through LDS, double-buffered,
// and through two register sets, so three tiles are in flight: while the matrix cores consume
// tile t out of LDS, the global loads of tile t+2 are issued *between* the MFMA groups of the same
// wavefront (a few loads after every four MFMAs) into one register set, and the other set -
// tile t+1, loaded a whole step earlier - is written to the second LDS buffer after the last
// MFMA.  There is one barrier per step, a load has a full step to arrive, and a wavefront keeps
// the matrix pipe fed on its own.  Every wavefront owns a 64 x 64 sub-tile = 2 x 2 MFMA blocks of
// 32 x 32 (64 accumulator registers).
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
// On this hardware a VALU instruction is not free next to MFMAs: each one takes matrix-pipe time
// (8 per MFMA cost a quarter of the throughput), while scalar-ALU, LDS and memory instructions issue
// beside them.  The loop is therefore written to need very few VALU instructions per step:
//   * wave-uniform index arithmetic (tap decomposition of a reduction index) is done on the scalar ALU;
//   * the padding test of an element is one bit-field extract from a per-thread tap mask that is
//     computed once per tile, and invalid elements get their offset's top bit set with one more op;
//   * MFMA operands are fetched from LDS with ds_read_b64 and 16-bit immediate offsets from one base
//     register per operand (explicit instructions: the compiler would re-add a base per k-step).
//
// LDS tiles are k-major ([k][m] and [k][n], rows padded by 4 floats) with reduction rows k and k+2 of a
// column interleaved, so that an MFMA operand fetch - lane l needs element (row l%32, k = 2J + l/32) for
// k-step J - is one conflict-free 64-bit read per two k-steps, stores from loaders whose lanes run
// along k spread over all banks, and loaders whose lanes run along m / n store two rows at once.
#pragma once
#include "common.h"
#include <atomic>

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

// ---------------------------------------------------------------- host helpers
// A kernel's dynamic LDS limit belongs to the device's copy of the kernel: raised once per device (bit `device` of
// `done`), from any thread.
inline int raise_lds_limit(const void* kernel, std::atomic<unsigned>& done, int bytes)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return PYDTNN_HIP_ERR_LAUNCH;
    const unsigned bit = 1u << (dev & 31);
    if (done.load(std::memory_order_acquire) & bit) return PYDTNN_HIP_OK;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
        return PYDTNN_HIP_ERR_LAUNCH;
    done.fetch_or(bit, std::memory_order_release);
    return PYDTNN_HIP_OK;
}

// Compute units of the current device (cached for the first 32 devices).
inline int device_compute_units(int* cus)
{
    static std::atomic<int> cached[32];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return PYDTNN_HIP_ERR_LAUNCH;
    int v = dev < 32 ? cached[dev].load(std::memory_order_relaxed) : 0;
    if (v <= 0) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            return PYDTNN_HIP_ERR_LAUNCH;
        if (dev < 32) cached[dev].store(v, std::memory_order_relaxed);
    }
    *cus = v;
    return PYDTNN_HIP_OK;
}

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

typedef float floatx4 __attribute__((ext_vector_type(4)));

// Four consecutive floats (each dword is range-checked against the descriptor on its own).
__device__ __forceinline__ floatx4 buf_load4(rsrc_t r, uint32_t voff_bytes, uint32_t soff_bytes)
{
    return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff_bytes, (int)soff_bytes, 0));
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Byte offset for buf_load, pushed beyond every descriptor when `invalid_bit` is 1.
__device__ __forceinline__ uint32_t guarded_offset(uint32_t invalid_bit, uint32_t byte_offset)
{
    return (invalid_bit << 31) | byte_offset;
}

// LDS byte address of a __shared__ object, and a read at a compile-time byte offset from it.  The
// result may only be used after lds_wait().
__device__ __forceinline__ uint32_t lds_addr(const float* p)
{
    return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const float*)p);
}

typedef float floatx2 __attribute__((ext_vector_type(2)));

template <int OFF>
__device__ __forceinline__ floatx2 lds_read2(uint32_t addr)
{
    static_assert(OFF >= 0 && OFF < 65536 && OFF % 8 == 0, "ds_read_b64 takes a 16-bit byte offset");
    floatx2 v;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

// Waits for every outstanding LDS read; the registers are passed through so that their uses cannot be
// scheduled above the wait.
template <int N>
__device__ __forceinline__ void lds_wait(floatx2 (&a)[N])
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]));
#pragma unroll
    for (int i = 1; i < N; ++i) asm volatile("" : "+v"(a[i]));
}

// LDS tile layout.  Reduction rows k and k+2 of the same column sit next to each other, so that one
// 64-bit read serves two consecutive MFMA k-steps (lane (r, h) needs k = 2J + h for step J):
//   float index of (k, mn) = ((k >> 2) * 2 + (k & 1)) * kRowPitch + mn * 2 + ((k >> 1) & 1)
// with kRowPitch = 2 * (BMN + kPad) floats; the tile takes BK * (BMN + kPad) floats as before.
template <int BMN>
struct LdsTile {
    static constexpr int kRowPitch = 2 * (BMN + kPad);
    static constexpr int kFloats = BK * (BMN + kPad);
    static __device__ __forceinline__ int index(int k, int mn)
    {
        return ((k >> 2) * 2 + (k & 1)) * kRowPitch + mn * 2 + ((k >> 1) & 1);
    }
};

// Tap masks for the padding test.  Bit t of the returned word is 1 when tap t must read as zero.
// Narrow form (kh*kw <= 31): one word over the combined tap index i*kw + j.  Wide form: one word over
// i and one over j (kh, kw <= 31).  Bit 31 is always 1: reduction indices >= kend select it.
__device__ __forceinline__ uint32_t tap_mask_combined(const ConvGeom& g, int ih0, int iw0)
{
    uint32_t inv = 0xffffffffu;
    for (int t = 0; t < g.khw; ++t) {
        const int ii = t / g.kw, jj = t - ii * g.kw;
        const bool ok = (unsigned)(ih0 + ii * g.vdilation) < (unsigned)g.h &&
                        (unsigned)(iw0 + jj * g.hdilation) < (unsigned)g.w;
        if (ok) inv &= ~(1u << t);
    }
    return inv;
}

__device__ __forceinline__ uint32_t tap_mask_axis(int first, int taps, int dilation, int extent)
{
    uint32_t inv = 0xffffffffu;
    for (int t = 0; t < taps; ++t)
        if ((unsigned)(first + t * dilation) < (unsigned)extent) inv &= ~(1u << t);
    return inv;
}

// ---------------------------------------------------------------- thread -> element maps
// MapMN: lanes run along the m (or n) axis of the tile; the k row is uniform per wavefront.
template <int BMN>
struct MapMN {
    static_assert(BMN % 64 == 0 && BMN <= kThreads, "tile extent");
    static constexpr int kRowsPerPass = kThreads / BMN;
    static constexpr int NLD = BK / kRowsPerPass;
    static __device__ __forceinline__ int mn(int tid) { return tid % BMN; }
    static __device__ __forceinline__ int krow(int tid) { return uniform(tid / BMN); }
    // This thread's rows are k0 + e * kRowsPerPass.  With one or two rows per pass it holds both rows
    // of every (k, k+2) pair and writes them with one 64-bit store; with four (BMN = 64) it does not.
    // Stores the elements e with e*PARTS/NLD == PART (a pair goes with its first element).
    template <int PART, int PARTS>
    static __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid)
    {
        const int m = tid % BMN, k0 = tid / BMN;
        float* base = lds + LdsTile<BMN>::index(k0, m);
        constexpr int P = LdsTile<BMN>::kRowPitch;
        if constexpr (kRowsPerPass == 2) {
#pragma unroll
            for (int e = 0; e < NLD; e += 2)  // k = k0 + 2e and k + 2
                if (e * PARTS / NLD == PART)
                    *reinterpret_cast<floatx2*>(base + (e >> 1) * 2 * P) = floatx2{r[e], r[e + 1]};
        } else if constexpr (kRowsPerPass == 1) {
#pragma unroll
            for (int e = 0; e < NLD; ++e)  // k = e (k0 = 0); pairs (e, e + 2) for e % 4 in {0, 1}
                if ((e & 2) == 0 && e * PARTS / NLD == PART)
                    *reinterpret_cast<floatx2*>(base + ((e >> 2) * 2 + (e & 1)) * P) = floatx2{r[e], r[e + 2]};
        } else {
            static_assert(kRowsPerPass == 4, "tile extents are 64, 128 or 256");
#pragma unroll
            for (int e = 0; e < NLD; ++e)
                if (e * PARTS / NLD == PART) base[e * 2 * P] = r[e];  // k = k0 + 4e
        }
    }
    static __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid)
    {
        store_part<0, 1>(lds, r, tid);
    }
};

// MapMNW: lanes run along m like MapMN, but a wavefront owns four consecutive k rows of the step
// (k = 4*wave + row) and visits the BMN/64 groups of 64 columns in turn.  Element e is (row e / kPasses,
// column group e % kPasses), so whatever a loader derives from the row alone (wave-uniform, scalar) is worked
// out for four rows per wavefront and step, not for every element.
template <int BMN>
struct MapMNW {
    static_assert(BMN % 64 == 0 && kThreads == 256 && BK == 16, "four wavefronts with four rows each");
    static constexpr int kPasses = BMN / 64;
    static constexpr int NLD = 4 * kPasses;
    static constexpr int row_of(int e) { return e / kPasses; }
    static constexpr int pass_of(int e) { return e % kPasses; }
    static __device__ __forceinline__ int mn(int tid, int pass) { return (tid & 63) + 64 * pass; }
    static __device__ __forceinline__ int krow0(int tid) { return uniform(tid >> 6) * 4; }
    // Rows (0, 2) of the wavefront share the 64-bit words of one pitch, rows (1, 3) those of the next.
    template <int PART, int PARTS>
    static __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid)
    {
        constexpr int P = LdsTile<BMN>::kRowPitch;
        float* base = lds + (2 * (tid >> 6)) * P + (tid & 63) * 2;
#pragma unroll
        for (int j = 0; j < kPasses; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                if ((j * 2 + h) * PARTS / (NLD / 2) == PART)
                    *reinterpret_cast<floatx2*>(base + h * P + j * 128) =
                        floatx2{r[h * kPasses + j], r[(h + 2) * kPasses + j]};
    }
    static __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid)
    {
        store_part<0, 1>(lds, r, tid);
    }
};

// MapK: lanes run along k; each thread owns NLD different m (or n) positions.
template <int BMN>
struct MapK {
    static constexpr int kMnPerPass = kThreads / BK;
    static constexpr int NLD = BMN / kMnPerPass;
    static __device__ __forceinline__ int kk(int tid) { return tid % BK; }
    static __device__ __forceinline__ int mn(int tid, int e) { return tid / BK + e * kMnPerPass; }
    template <int PART, int PARTS>
    static __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid)
    {
        const int k = tid % BK, m0 = tid / BK;
        float* base = lds + LdsTile<BMN>::index(k, m0);
#pragma unroll
        for (int e = 0; e < NLD; ++e)
            if (e * PARTS / NLD == PART) base[e * kMnPerPass * 2] = r[e];
    }
    static __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid)
    {
        store_part<0, 1>(lds, r, tid);
    }
};

// MapK4: four lanes cover the 16 reduction indices of a step with one 128-bit load each (k = 4q .. 4q+3,
// q = tid % 4); 64 rows per pass.  For operands whose reduction axis is contiguous and 16-byte aligned.
template <int BMN>
struct MapK4 {
    static_assert(BK == 16, "four lanes of four floats per step");
    static constexpr int kMnPerPass = kThreads / 4;
    static constexpr int NLD = BMN / kMnPerPass;
    static __device__ __forceinline__ int kq(int tid) { return tid % 4; }
    static __device__ __forceinline__ int mn(int tid, int e) { return tid / 4 + e * kMnPerPass; }
    // In the tile layout (k, k+2) share a 64-bit word: the quad goes out as {k0, k2} and {k1, k3}.
    template <int PART, int PARTS>
    static __device__ __forceinline__ void store_part(float* lds, const floatx4 (&r)[NLD], int tid)
    {
        constexpr int P = LdsTile<BMN>::kRowPitch;
        float* base = lds + (2 * (tid % 4)) * P + (tid / 4) * 2;
#pragma unroll
        for (int e = 0; e < NLD; ++e)
            if (e * PARTS / NLD == PART) {
                float* p = base + e * kMnPerPass * 2;
                *reinterpret_cast<floatx2*>(p) = floatx2{r[e][0], r[e][2]};
                *reinterpret_cast<floatx2*>(p + P) = floatx2{r[e][1], r[e][3]};
            }
    }
    static __device__ __forceinline__ void store(float* lds, const floatx4 (&r)[NLD], int tid)
    {
        store_part<0, 1>(lds, r, tid);
    }
};

// Every loader exposes
//   State            per-thread data fixed for the whole tile
//   Iter             per-thread / per-wave data of one reduction step
//   init(State&, origin, image0, tid)
//   begin(State, Iter&, k0, kend)            prepare the step that starts at reduction index k0
//   elem<E>(State, Iter, k0, kend)           value of this thread's E-th element of that step
//   store(lds, regs, tid)
// Reduction indices >= kend read as zero.  That test is made once per step (it is folded into the
// step's tap / offset computation or into the size of the step's descriptor), never per element, so
// the loop body has a single form for full and partial steps.

// ---------------------------------------------------------------- plain strided loaders
// elem(mn, k) = base[(image0 + k / seg)*image_stride + mn*ld + k % seg]   (k contiguous inside a segment)
// With SEG == false the reduction axis is one segment: elem = base[image0*image_stride + mn*ld + k].
// Needs BMN*ld*4 (+ ips*image_stride*4 when SEG) < 2 GiB, checked on the host.
template <int BMN, bool SEG = false>
struct PlainK {
    using Map = MapK<BMN>;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    using Reg = float;
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
        if (k >= kend) it.voff = kOob;
    }
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        return buf_load(s.rsrc, s.rowoff[E] + it.voff, it.soff);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// elem(mn, k) = base[image*image_stride + k*ld + mn]   (mn contiguous).  The descriptor is re-based to
// row k0 at every step and sized to end with row kend-1, so rows of a partial step beyond the
// reduction range read as zero; only BK*ld*4 < 2 GiB is needed (checked on the host).
// PlainK with 128-bit loads: elem(mn, k) = base[mn*ld + k], one segment.  Needs ld % 4 == 0, a 16-byte
// aligned base and reduction ranges that end on multiples of 4 (checked on the host).
template <int BMN>
struct PlainK4 {
    using Map = MapK4<BMN>;
    using Reg = floatx4;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    const float* base;
    long total;  // floats in the tensor
    long ld;
    int extent;  // valid mn range
    struct State {
        rsrc_t rsrc;
        uint32_t rowoff[NLD];  // byte offset of (row e, this thread's quad)
    };
    struct Iter {
        uint32_t voff;  // 0, or kOob when this thread's quad lies beyond kend
        uint32_t soff;  // uniform byte offset of the step
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image0*/, int tid) const
    {
        const long first = (long)origin * ld;
        s.rsrc = make_rsrc(base + first, total - first);
        const int rows = min(BMN, extent - origin);
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            const int row = min(Map::mn(tid, e), rows - 1);
            s.rowoff[e] = (uint32_t)(row * ld + 4 * Map::kq(tid)) * 4u;
        }
    }
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        it.voff = k0 + 4 * Map::kq(threadIdx.x) >= kend ? kOob : 0u;
        it.soff = (uint32_t)k0 * 4u;
    }
    template <int E>
    __device__ __forceinline__ floatx4 elem(const State& s, const Iter& it, int, int) const
    {
        return buf_load4(s.rsrc, s.rowoff[E] + it.voff, it.soff);
    }
    __device__ __forceinline__ void store(float* lds, const floatx4 (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const floatx4 (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

template <int BMN>
struct PlainMN {
    using Map = MapMN<BMN>;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    using Reg = float;
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
    __device__ __forceinline__ void begin(const State& s, Iter& it, int k0, int kend) const
    {
        const int krow0 = k0 + s.krow;
        const long row0 = s.first + (long)krow0 * ld;
        const long in_range = (long)(kend - krow0) * ld;  // <= 0 when the whole step lies beyond kend
        const long in_tensor = total - row0;
        it.rsrc = make_rsrc(base + row0, in_range < in_tensor ? in_range : in_tensor);
    }
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        return buf_load(it.rsrc, s.voff + (uint32_t)(E * Map::kRowsPerPass) * (uint32_t)ld * 4u, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// ---------------------------------------------------------------- implicit im2col, NCHW
// B(k = (c,i,j), n = (img,y,x)) = X[img, c, sv*y + dv*i - pv, sh*x + dh*j - ph]: the column matrix of
// pydtnn/cython_modules/im2col_nchw_cython.pyx:104-124, never written to memory.
// Lanes run along the pixel axis (contiguous in x for a fixed tap); the tap (c,i,j) of an element is
// wave-uniform and is decomposed on the scalar ALU.  WIDE selects the two-word tap mask.
// NHWC: the same matrix read from an (N,H,W,C) tensor, X[img, ih, iw, c]; lanes are then c floats apart, which
// only pays for very few channels (a first layer), where the rows of one tap's channels share cache lines.
template <int BN, bool WIDE = false, bool NHWC = false>
struct Im2colNchwMN {
    using Map = MapMNW<BN>;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    using Reg = float;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;                  // starts `lead` floats before x, so that every thread's base offset is >= 0
        uint32_t base[Map::kPasses];  // byte offset of (img, c=0, ih0, iw0) from there, per column group
        uint32_t inv0[Map::kPasses];  // narrow: combined tap mask; wide: mask over i
        uint32_t inv1[Map::kPasses];  // wide: mask over j
        int krow0;
    };
    struct Iter {};
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        // ih0*w + iw0 >= -(vpadding*w + hpadding): shifting the descriptor back by that much keeps the
        // per-thread offset unsigned, and the tap's own offset (>= 0) can then ride in the scalar offset
        // operand of the load, which the hardware adds after its range check of the vector offset.
        const int lead = (g.vpadding * g.w + g.hpadding) * (NHWC ? g.c : 1);
        s.rsrc = make_rsrc(x - lead, (long)g.n * g.c * g.h * g.w + lead);
        s.krow0 = Map::krow0(tid);
#pragma unroll
        for (int j = 0; j < Map::kPasses; ++j) {
            long n = (long)origin + Map::mn(tid, j);
            n = n < g.p ? n : g.p - 1;
            // 32-bit division whenever the pixel count allows it (a launch-wide condition): a third of the
            // instructions of the 64-bit one, which counts for tiles with only a few reduction steps
            const int img = g.p < (1l << 31) ? (int)((uint32_t)n / (uint32_t)g.howo) : (int)(n / g.howo);
            const int pp = (int)(n - (long)img * g.howo);
            const int yy = (int)((uint32_t)pp / (uint32_t)g.wo), xx = pp - yy * g.wo;
            const int ih0 = yy * g.vstride - g.vpadding;
            const int iw0 = xx * g.hstride - g.hpadding;
            s.base[j] = NHWC ? (uint32_t)(((img * g.h + ih0) * g.w + iw0) * g.c + lead) * 4u
                             : (uint32_t)((img * g.c * g.h + ih0) * g.w + iw0 + lead) * 4u;
            if (WIDE) {
                s.inv0[j] = tap_mask_axis(ih0, g.kh, g.vdilation, g.h);
                s.inv1[j] = tap_mask_axis(iw0, g.kw, g.hdilation, g.w);
            } else {
                s.inv0[j] = tap_mask_combined(g, ih0, iw0);
                s.inv1[j] = 0;
            }
        }
    }
    __device__ __forceinline__ void begin(const State&, Iter&, int, int) const {}
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter&, int k0, int kend) const
    {
        constexpr int R = Map::row_of(E), J = Map::pass_of(E);
        // scalar, once per row: reduction index -> (c, i, j) -> byte offset of the tap inside one image
        const uint32_t k = (uint32_t)(k0 + s.krow0 + R);
        const uint32_t cc = fd_div(k, g.fd_khw);
        const uint32_t rem = k - cc * g.khw;
        const uint32_t ii = fd_div(rem, g.fd_kw);
        const uint32_t jj = rem - ii * g.kw;
        const uint32_t off =
            NHWC ? (uint32_t)(((int)ii * g.vdilation * g.w + (int)jj * g.hdilation) * g.c + (int)cc) * 4u
                 : (uint32_t)(((int)cc * g.h + (int)ii * g.vdilation) * g.w + (int)jj * g.hdilation) * 4u;
        const bool live = (int)k < kend;
        if (WIDE) {
            const uint32_t invalid =
                __builtin_amdgcn_ubfe(s.inv0[J], live ? ii : 31u, 1) | __builtin_amdgcn_ubfe(s.inv1[J], jj, 1);
            return buf_load(s.rsrc, guarded_offset(invalid, s.base[J]), off);
        }
        // two vector instructions per element: move the tap's mask bit to bit 31, merge it into the offset
        const uint32_t bit = live ? rem : 31u;
        return buf_load(s.rsrc, ((s.inv0[J] << (31u - bit)) & kOob) | s.base[J], off);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// dW view of the same matrix: B(k = (image, pixel), n = (c,i,j)).  Lanes run along the pixel (reduction)
// axis; each thread owns NLD fixed taps.
template <int BN>
struct Im2colNchwK {
    using Map = MapK<BN>;
    static constexpr int NLD = Map::NLD;
    // three precomputed words for each of 12 or 16 elements: built without the three-per-CU register limit
    static constexpr bool kLargeState = BN >= 192;
    using Reg = float;
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
        if (k >= kend) it.ih0 = -(1 << 20);  // fails every bound test
    }
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        const bool ok = (unsigned)(it.ih0 + s.di[E]) < (unsigned)g.h && (unsigned)(it.iw0 + s.dj[E]) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(it.base + s.coff[E]) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// ---------------------------------------------------------------- implicit im2row, NHWC
// A(m = (img,y,x), k) = X[img, sv*y + dv*i - pv, sh*x + dh*j - ph, c] with the reduction index walked
// in (i, j, c) order so that lanes along k read consecutive channels.  The reference orders K as
// (c, i, j) (pydtnn/cython_modules/im2row_nhwc_cython.pyx:96); a sum over K does not depend on the
// order, and the filter loader below applies the same permutation to the rows of W.
template <int BM, bool WIDE = false>
struct Im2rowNhwcK {
    using Map = MapK<BM>;
    static constexpr int NLD = Map::NLD;
    // offset and tap mask(s) for each of 16 pixels: too much for three workgroups per CU
    static constexpr bool kLargeState = BM >= 256;
    using Reg = float;
    static constexpr int NMASK1 = WIDE ? NLD : 1;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        uint32_t base[NLD];    // byte offset of ((img*h + ih0)*w + iw0)*c, modulo 2^32
        uint32_t inv0[NLD];    // narrow: combined tap mask of the row's pixel; wide: mask over i
        uint32_t inv1[NMASK1]; // wide: mask over j
    };
    struct Iter {
        uint32_t koff;  // byte offset of (di*w + dj)*c + channel
        uint32_t bit0;  // narrow: combined tap index (31 beyond kend); wide: i (31 beyond kend)
        uint32_t bit1;  // wide: j
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
            const int ih0 = yy * g.vstride - g.vpadding;
            const int iw0 = xx * g.hstride - g.hpadding;
            s.base[e] = (uint32_t)(((img * g.h + ih0) * g.w + iw0) * g.c) * 4u;
            if (WIDE) {
                s.inv0[e] = tap_mask_axis(ih0, g.kh, g.vdilation, g.h);
                s.inv1[e] = tap_mask_axis(iw0, g.kw, g.hdilation, g.w);
            } else {
                s.inv0[e] = tap_mask_combined(g, ih0, iw0);
            }
        }
    }
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        const uint32_t k = (uint32_t)(k0 + Map::kk(threadIdx.x));
        const uint32_t ij = fd_div(k, g.fd_c);
        const uint32_t cc = k - ij * g.c;
        const uint32_t ii = fd_div(ij, g.fd_kw);
        const uint32_t jj = ij - ii * g.kw;
        it.koff = (uint32_t)(((int)ii * g.vdilation * g.w + (int)jj * g.hdilation) * g.c + (int)cc) * 4u;
        const bool live = (int)k < kend;
        it.bit0 = live ? (WIDE ? ii : ij) : 31u;
        it.bit1 = jj;
    }
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter& it, int, int) const
    {
        uint32_t invalid = __builtin_amdgcn_ubfe(s.inv0[E], it.bit0, 1);
        if (WIDE) invalid |= __builtin_amdgcn_ubfe(s.inv1[E], it.bit1, 1);
        return buf_load(s.rsrc, guarded_offset(invalid, s.base[E] + it.koff), 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// Im2rowNhwcK with 128-bit loads, for c % 16 == 0 and kh*kw <= 31: the reduction index is (tap, channel)
// with the channel fastest, so a step of 16 lies inside one tap; that tap is decomposed once per step on
// the scalar ALU and its offset rides in the load's scalar operand, and a thread keeps the pixel offset
// and tap mask of BM/64 rows instead of BM/16.  The descriptor starts `lead` floats before x so that the
// per-thread offset is never negative.
template <int BM>
struct Im2rowNhwcK4 {
    using Map = MapK4<BM>;
    using Reg = floatx4;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        uint32_t base[NLD];  // byte offset of ((img*h + ih0)*w + iw0)*c + 4q from the shifted start
        uint32_t inv0[NLD];  // combined tap mask of the row's pixel (bit 31 always set)
    };
    struct Iter {
        uint32_t soff;  // byte offset of (di*w + dj)*c + first channel of the step
        uint32_t sh;    // 31 - tap index (0 beyond kend: selects the always-set bit)
    };
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        const long lead = (long)(g.vpadding * g.w + g.hpadding) * g.c;
        s.rsrc = make_rsrc(x - lead, (long)g.n * g.c * g.h * g.w + lead);
#pragma unroll
        for (int e = 0; e < NLD; ++e) {
            long m = (long)origin + Map::mn(tid, e);
            m = m < g.p ? m : g.p - 1;
            const int img = (int)(m / g.howo);
            const int pp = (int)(m - (long)img * g.howo);
            const int yy = pp / g.wo, xx = pp - yy * g.wo;
            const int ih0 = yy * g.vstride - g.vpadding;
            const int iw0 = xx * g.hstride - g.hpadding;
            s.base[e] = (uint32_t)((((long)img * g.h + ih0) * g.w + iw0) * g.c + lead + 4 * Map::kq(tid)) * 4u;
            s.inv0[e] = tap_mask_combined(g, ih0, iw0);
        }
    }
    __device__ __forceinline__ void begin(const State&, Iter& it, int k0, int kend) const
    {
        const uint32_t ij = fd_div((uint32_t)k0, g.fd_c);
        const uint32_t c0 = (uint32_t)k0 - ij * g.c;
        const uint32_t ii = fd_div(ij, g.fd_kw);
        const uint32_t jj = ij - ii * g.kw;
        it.soff = (uint32_t)(((int)ii * g.vdilation * g.w + (int)jj * g.hdilation) * g.c + (int)c0) * 4u;
        it.sh = k0 < kend ? 31u - ij : 0u;
    }
    template <int E>
    __device__ __forceinline__ floatx4 elem(const State& s, const Iter& it, int, int) const
    {
        return buf_load4(s.rsrc, ((s.inv0[E] << it.sh) & kOob) | s.base[E], it.soff);
    }
    __device__ __forceinline__ void store(float* lds, const floatx4 (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const floatx4 (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// Filter in NHWC layout (c, kh, kw, kn) read as B(k in (i,j,c) order, n = filter).
template <int BN>
struct FilterNhwcMN {
    using Map = MapMNW<BN>;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    using Reg = float;
    const float* w;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        uint32_t voff[Map::kPasses];
        int krow0;
    };
    struct Iter {};
    __device__ __forceinline__ void init(State& s, int origin, int /*image*/, int tid) const
    {
        s.rsrc = make_rsrc(w, (long)g.k * g.kn);
#pragma unroll
        for (int j = 0; j < Map::kPasses; ++j) s.voff[j] = (uint32_t)min(origin + Map::mn(tid, j), g.kn - 1) * 4u;
        s.krow0 = Map::krow0(tid);
    }
    __device__ __forceinline__ void begin(const State&, Iter&, int, int) const {}
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter&, int k0, int kend) const
    {
        constexpr int R = Map::row_of(E), J = Map::pass_of(E);
        // scalar, once per row: reduction index in (i,j,c) order -> filter row c*kh*kw + i*kw + j
        const uint32_t k = (uint32_t)(k0 + s.krow0 + R);
        const uint32_t ij = fd_div(k, g.fd_c);
        const uint32_t cc = k - ij * g.c;
        const uint32_t rowoff = (int)k < kend ? (cc * g.khw + ij) * (uint32_t)g.kn * 4u : kOob;
        return buf_load(s.rsrc, s.voff[J] + rowoff, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// dW view in NHWC: A(m = (i,j,c), k = (image, pixel)).  Lanes run along m (consecutive channels); the
// pixel of a row is wave-uniform and decomposed on the scalar unit, once per row for all column groups.
template <int BM>
struct Im2rowNhwcMN {
    using Map = MapMNW<BM>;
    static constexpr int NLD = Map::NLD;
    static constexpr bool kLargeState = false;
    using Reg = float;
    const float* x;
    ConvGeom g;
    struct State {
        rsrc_t rsrc;
        int moff[Map::kPasses];  // (di*w + dj)*c + channel, per column group
        int di[Map::kPasses], dj[Map::kPasses];
        int krow0;
        int image0;
    };
    struct Iter {};
    __device__ __forceinline__ void init(State& s, int origin, int image0, int tid) const
    {
        s.rsrc = make_rsrc(x, (long)g.n * g.c * g.h * g.w);
#pragma unroll
        for (int j = 0; j < Map::kPasses; ++j) {
            const int m = min(origin + Map::mn(tid, j), g.k - 1);
            const int ij = m / g.c, cc = m - ij * g.c;
            const int ii = ij / g.kw, jj = ij - ii * g.kw;
            s.di[j] = ii * g.vdilation;
            s.dj[j] = jj * g.hdilation;
            s.moff[j] = (s.di[j] * g.w + s.dj[j]) * g.c + cc;
        }
        s.krow0 = Map::krow0(tid);
        s.image0 = image0;
    }
    __device__ __forceinline__ void begin(const State&, Iter&, int, int) const {}
    template <int E>
    __device__ __forceinline__ float elem(const State& s, const Iter&, int k0, int kend) const
    {
        constexpr int R = Map::row_of(E), J = Map::pass_of(E);
        // scalar: reduction index -> (image within the group, y, x) -> first input row / column of the window
        const uint32_t k = (uint32_t)(k0 + s.krow0 + R);
        const uint32_t img = fd_div(k, g.fd_howo);
        const uint32_t pp = k - img * g.howo;
        const uint32_t yy = fd_div(pp, g.fd_wo);
        const uint32_t xx = pp - yy * g.wo;
        const int ih0 = (int)k < kend ? (int)yy * g.vstride - g.vpadding : 0x2000;  // beyond kend: fails the row test
        const int iw0 = (int)xx * g.hstride - g.hpadding;
        const int pixc = (((s.image0 + (int)img) * g.h + ih0) * g.w + iw0) * g.c;
        const bool ok = (unsigned)(ih0 + s.di[J]) < (unsigned)g.h && (unsigned)(iw0 + s.dj[J]) < (unsigned)g.w;
        return buf_load(s.rsrc, ok ? (uint32_t)(pixc + s.moff[J]) * 4u : kOob, 0);
    }
    __device__ __forceinline__ void store(float* lds, const float (&r)[NLD], int tid) const { Map::store(lds, r, tid); }
    template <int PART, int PARTS>
    __device__ __forceinline__ void store_part(float* lds, const float (&r)[NLD], int tid) const
    {
        Map::template store_part<PART, PARTS>(lds, r, tid);
    }
};

// ---------------------------------------------------------------- epilogues
// Row-major store C[split*split_stride + m*ldc + n]; the per-channel chain uses the column index
// (NHWC convolution, FC forward).
// MASKS (kNoMasks, kGate, kReluMask, kResidual): the store also applies the gate, writes the ReLU mask or adds
// the residual (separate instantiations, so that no case carries a test per stored element).
template <int MASKS>
struct EpiPlainT {
    using Unmasked = EpiPlainT<kNoMasks>;
    float* out;
    long ldc;
    long split_stride;
    int m_extent, n_extent;
    ChanEpilogue chan;
    ElemMasks masks;  // only with a single split
    long span;        // floats from `out` to the end of the last split if that is below 2^29, else 0
    struct Col {
        long off;
        int n;
        bool ok;
    };
    __device__ __forceinline__ Col column(int n, int split) const
    {
        Col c;
        c.n = n;
        c.ok = n < n_extent;
        c.off = (long)split * split_stride + n;
        return c;
    }
    __device__ __forceinline__ void store(const Col& c, int m, float v) const
    {
        if (c.ok && m < m_extent) {
            const long i = c.off + (long)m * ldc;
            const float r = chan_epilogue_apply(chan, c.n, v);
            out[i] = elem_masks_apply<MASKS>(masks, i, r);
        }
    }
};
using EpiPlain = EpiPlainT<kNoMasks>;

template <int MASKS>
struct EpiNchwT {
    using Unmasked = EpiNchwT<kNoMasks>;
    float* out;
    int m_extent;  // output channels
    int howo;
    long p;        // images * howo
    ChanEpilogue chan;
    ElemMasks masks;
    struct Col {
        long off;
        bool ok;
    };
    __device__ __forceinline__ Col column(int n, int /*split*/) const
    {
        Col c;
        c.ok = n < p;
        const int nc = c.ok ? n : 0;
        const int img = nc / howo;
        const int pp = nc - img * howo;
        c.off = (long)img * m_extent * howo + pp;
        return c;
    }
    __device__ __forceinline__ void store(const Col& c, int m, float v) const
    {
        if (c.ok && m < m_extent) {
            const long i = c.off + (long)m * howo;
            const float r = chan_epilogue_apply(chan, m, v);
            out[i] = elem_masks_apply<MASKS>(masks, i, r);
        }
    }
};
using EpiNchw = EpiNchwT<kNoMasks>;


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
template <int J, int E, class L>
__device__ __forceinline__ void group_load(const L& l, const typename L::State& s, const typename L::Iter& it,
                                           typename L::Reg (&r)[L::NLD], int k0, int kend)
{
    if constexpr (E < L::NLD) {
        if constexpr (E * (BK / 2) / L::NLD == J) r[E] = l.template elem<E>(s, it, k0, kend);
        group_load<J, E + 1, L>(l, s, it, r, k0, kend);
    }
}

template <int E, class L>
__device__ __forceinline__ void load_all(const L& l, const typename L::State& s, const typename L::Iter& it,
                                         typename L::Reg (&r)[L::NLD], int k0, int kend)
{
    if constexpr (E < L::NLD) {
        r[E] = l.template elem<E>(s, it, k0, kend);
        load_all<E + 1, L>(l, s, it, r, k0, kend);
    }
}

// MFMA operands of the k-steps 2P and 2P+1 out of LDS buffer BUF: lane (r, h) of a wavefront gets
// A[m = 32*i + r][k = 4P + h] and [k = 4P + 2 + h] in one 64-bit read, likewise B.  `a_base` / `b_base` are the
// LDS byte addresses of this lane's pair of buffer 0 at P = 0, i = j = 0; everything else is an immediate offset.
template <class T, int BUF, int P>
__device__ __forceinline__ void request_operands(uint32_t a_base, uint32_t b_base, floatx2 (&af)[T::TM],
                                                 floatx2 (&bf)[T::TN])
{
    constexpr int a_off = (BUF * LdsTile<T::BM>::kFloats + 2 * P * LdsTile<T::BM>::kRowPitch) * 4;
    constexpr int b_off = (BUF * LdsTile<T::BN>::kFloats + 2 * P * LdsTile<T::BN>::kRowPitch) * 4;
    if constexpr (T::TM >= 1) af[0] = lds_read2<a_off>(a_base);
    if constexpr (T::TM >= 2) af[1] = lds_read2<a_off + 256>(a_base);
    if constexpr (T::TM >= 3) af[2] = lds_read2<a_off + 512>(a_base);
    if constexpr (T::TM >= 4) af[3] = lds_read2<a_off + 768>(a_base);
    if constexpr (T::TN >= 1) bf[0] = lds_read2<b_off>(b_base);
    if constexpr (T::TN >= 2) bf[1] = lds_read2<b_off + 256>(b_base);
    if constexpr (T::TN >= 3) bf[2] = lds_read2<b_off + 512>(b_base);
    if constexpr (T::TN >= 4) bf[3] = lds_read2<b_off + 768>(b_base);
    static_assert(T::TM <= 4 && T::TN <= 4, "operand fetch is written for up to 4 blocks per axis");
}

// Everything a step needs besides the accumulators: the register set that receives the loads of the
// tile two steps ahead, and the register set (filled one step earlier) that this step stores into the
// LDS buffer it does not read.
template <class AL, class BL>
struct StepRegs {
    typename AL::Reg (&ra)[AL::NLD];
    typename BL::Reg (&rb)[BL::NLD];
    const typename AL::Reg (&sa)[AL::NLD];
    const typename BL::Reg (&sb)[BL::NLD];
    float* a_store;
    float* b_store;
    int tid;
};

// The LDS stores of a step are spread over its last kStoreGroups MFMA groups.
constexpr int kStoreGroups = 4;

// One MFMA group (k-step J of the LDS tile) and everything scheduled around it: an even group waits for
// the operand pair it shares with the next group, starts the first MFMA and requests the following pair;
// every group issues its share of the global loads, then the remaining MFMAs; the last groups also
// store their share of the tile for the next step into the other LDS buffer, which nobody reads
// between the barrier before this step and the barrier after it.
template <class T, int BUF, int J, class AL, class BL>
__device__ __forceinline__ void mfma_groups(const AL& al, const BL& bl, const typename AL::State& as,
                                            const typename BL::State& bs, const typename AL::Iter& ai,
                                            const typename BL::Iter& bi, const StepRegs<AL, BL>& rg,
                                            uint32_t a_base, uint32_t b_base, floatx16 (&acc)[T::TM][T::TN],
                                            floatx2 (&af)[2][T::TM], floatx2 (&bf)[2][T::TN], int knext, int kend)
{
    constexpr int G = BK / 2;
    if constexpr (J < G) {
        constexpr int P = J / 2, S = P & 1, H = J & 1;
        if constexpr (H == 0) {
            lds_wait(af[S]);
            lds_wait(bf[S]);
        }
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[S][0][H], bf[S][0][H], acc[0][0], 0, 0, 0);
        if constexpr (H == 0 && J + 2 < G) request_operands<T, BUF, P + 1>(a_base, b_base, af[S ^ 1], bf[S ^ 1]);
        group_load<J, 0, AL>(al, as, ai, rg.ra, knext, kend);
        group_load<J, 0, BL>(bl, bs, bi, rg.rb, knext, kend);
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
            for (int j = 0; j < T::TN; ++j)
                if (i + j > 0)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[S][i][H], bf[S][j][H], acc[i][j], 0, 0, 0);
        if constexpr (J >= G - kStoreGroups) {
            al.template store_part<J - (G - kStoreGroups), kStoreGroups>(rg.a_store, rg.sa, rg.tid);
            bl.template store_part<J - (G - kStoreGroups), kStoreGroups>(rg.b_store, rg.sb, rg.tid);
        }
        // keep this group's LDS fetches, global loads and MFMAs together: the instruction scheduler
        // must not sink the loads to the end of the step
        __builtin_amdgcn_sched_barrier(0);
        mfma_groups<T, BUF, J + 1, AL, BL>(al, bl, as, bs, ai, bi, rg, a_base, b_base, acc, af, bf, knext, kend);
    }
}

// Consumes LDS buffer BUF, loads the tile that starts at reduction index knext into (rg.ra, rg.rb)
// and stores (rg.sa, rg.sb) into the other LDS buffer.
template <class T, int BUF, class AL, class BL>
__device__ __forceinline__ void step(const AL& al, const BL& bl, const typename AL::State& as,
                                     const typename BL::State& bs, const StepRegs<AL, BL>& rg,
                                     uint32_t a_base, uint32_t b_base, floatx16 (&acc)[T::TM][T::TN], int knext,
                                     int kend)
{
    typename AL::Iter ai;
    typename BL::Iter bi;
    floatx2 af[2][T::TM], bf[2][T::TN];
    request_operands<T, BUF, 0>(a_base, b_base, af[0], bf[0]);
    al.begin(as, ai, knext, kend);
    bl.begin(bs, bi, knext, kend);
    mfma_groups<T, BUF, 0, AL, BL>(al, bl, as, bs, ai, bi, rg, a_base, b_base, acc, af, bf, knext, kend);
}

// The reduction loop of one tile over [kbeg, kend): adds into `acc`.  Leaves LDS free for reuse
// (every wavefront has passed the barrier that follows the last operand fetch).
template <class T, class AL, class BL>
__device__ __forceinline__ void tile_mainloop(const AL& al, const BL& bl, int m0, int n0, int image, int kbeg,
                                              int kend, float* As0, float* As1, float* Bs0, float* Bs1,
                                              uint32_t a_base, uint32_t b_base, floatx16 (&acc)[T::TM][T::TN], int tid)
{
    typename AL::State as;
    typename BL::State bs;
    al.init(as, m0, image, tid);
    bl.init(bs, n0, image, tid);

    // Register sets: during step s the loads of tile s+2 go to set (s & 1) while set ((s+1) & 1),
    // filled during step s-1 with tile s+1, is stored to the LDS buffer that step s does not read.
    typename AL::Reg ra0[AL::NLD], ra1[AL::NLD];
    typename BL::Reg rb0[BL::NLD], rb1[BL::NLD];
    {   // tiles 0 and 1 (any kend, including an empty range: everything reads as zero)
        typename AL::Iter ai;
        typename BL::Iter bi;
        al.begin(as, ai, kbeg, kend);
        bl.begin(bs, bi, kbeg, kend);
        load_all<0, AL>(al, as, ai, ra0, kbeg, kend);
        load_all<0, BL>(bl, bs, bi, rb0, kbeg, kend);
        al.begin(as, ai, kbeg + BK, kend);
        bl.begin(bs, bi, kbeg + BK, kend);
        load_all<0, AL>(al, as, ai, ra1, kbeg + BK, kend);
        load_all<0, BL>(bl, bs, bi, rb1, kbeg + BK, kend);
    }
    al.store(As0, ra0, tid);
    bl.store(Bs0, rb0, tid);
    __syncthreads();

    // Two steps per trip so that the register sets are named statically.  A reduction range with an
    // odd number of steps runs one extra step on a tile that lies beyond kend and therefore is zero.
    // The stores of a trip's second step fill buffer 0 for the next trip (harmless after the last).
    const StepRegs<AL, BL> even{ra0, rb0, ra1, rb1, As1, Bs1, tid}, odd{ra1, rb1, ra0, rb0, As0, Bs0, tid};
    for (int k0 = kbeg; k0 < kend; k0 += 2 * BK) {
        step<T, 0>(al, bl, as, bs, even, a_base, b_base, acc, k0 + 2 * BK, kend);
        __syncthreads();
        step<T, 1>(al, bl, as, bs, odd, a_base, b_base, acc, k0 + 3 * BK, kend);
        __syncthreads();
    }
}

template <class T>
__device__ __forceinline__ void clear_acc(floatx16 (&acc)[T::TM][T::TN])
{
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
}

// Accumulator layout of v_mfma_f32_32x32x2_f32: register v of lane l holds
// C[8*(v/4) + 4*(l/32) + v%4][l%32] of the 32x32 block.
//
// Generic tile store: one guarded store per element through the epilogue's own store().
template <class T, class EP>
__device__ __forceinline__ void store_tile_generic(const EP& ep, const floatx16 (&acc)[T::TM][T::TN], int m0, int n0,
                                                   int split, int tid)
{
    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;
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

__device__ __forceinline__ rsrc_t make_rsrc_bytes(const void* p, long bytes)
{
    bytes = bytes < 0 ? 0 : (bytes > kMaxSpanBytes ? kMaxSpanBytes : bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// Tile store into an (images, channels, ho*wo) tensor, written as straight-line code: rows of C are
// channels, so the per-channel epilogue parameters are per row; the tile's rows of them are staged in LDS
// once (`lds`: at least 5*BM floats, free at this point) instead of being fetched from memory in front of
// every store; out-of-range rows and columns get a buffer offset beyond the descriptor, which the hardware
// drops, instead of a branch; the gate bytes of a tile are all requested before its first store (loads and
// stores retire in issue order, so a load issued between two stores would wait for the first of them).
// Needs the whole tensor inside one descriptor (fewer than 2^29 elements), which the host guarantees.
template <class T, int MASKS>
__device__ __forceinline__ void store_tile_nchw(const EpiNchwT<MASKS>& ep, const floatx16 (&acc)[T::TM][T::TN], int m0,
                                                int n0, int tid, float* lds)
{
    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;
    const ChanEpilogue ch = ep.chan;
    const bool has_bias = ch.bias != nullptr, has_bn = ch.mean != nullptr;
    if (has_bias || has_bn) {
        if (tid < T::BM) {
            const int m = min(m0 + tid, ep.m_extent - 1);
            if (has_bias) lds[tid] = ch.bias[m];
            if (has_bn) {
                lds[T::BM + tid] = ch.mean[m];
                lds[2 * T::BM + tid] = ch.inv_std[m];
                lds[3 * T::BM + tid] = ch.gamma[m];
                lds[4 * T::BM + tid] = ch.beta[m];
            }
        }
        __syncthreads();
    }
    const long total = ep.p * ep.m_extent;
    const rsrc_t out_rsrc = make_rsrc(ep.out, total);
    // offset of (image, channel 4*frag_k, pixel) of each of this lane's columns, in floats' bytes (col_off4) and
    // in elements (col_off1, for the byte masks), or kOob
    uint32_t col_off4[T::TN];
    [[maybe_unused]] uint32_t col_off1[T::TN];
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
        const int n = n0 + wn0 + j * 32 + frag_r;
        const bool ok = n < ep.p;
        const int nc = ok ? n : 0;
        const int img = nc / ep.howo;
        const int pp = nc - img * ep.howo;
        const uint32_t e = (uint32_t)((img * ep.m_extent + 4 * frag_k) * ep.howo + pp);
        col_off4[j] = ok ? e * 4u : kOob;
        col_off1[j] = ok ? e : kOob;
    }
    const int lane_m0 = m0 + wm0 + 4 * frag_k;  // this lane's first row
    // The gate bytes are requested in batches of up to 64 per lane (all of a 2x2-block tile at once; row blocks
    // of a larger tile one after the other), each batch before the stores it belongs to.
    constexpr int kRowBlocksPerBatch = 16 * T::TN * T::TM <= 64 ? T::TM : 1;
    [[maybe_unused]] float gate[kRowBlocksPerBatch][16][T::TN];
    [[maybe_unused]] rsrc_t gate_rsrc;
    if constexpr (MASKS == kGate) gate_rsrc = make_rsrc_bytes(ep.masks.gate, total);
    [[maybe_unused]] rsrc_t mask_rsrc;
    if constexpr (MASKS == kReluMask) mask_rsrc = make_rsrc_bytes(ep.masks.relu_mask, total);
    if constexpr (MASKS == kResidual) gate_rsrc = make_rsrc(ep.masks.residual, total);
#pragma unroll
    for (int i0 = 0; i0 < T::TM; i0 += kRowBlocksPerBatch) {
        if constexpr (MASKS == kResidual) {  // the residual values of the batch, like the gate bytes below
#pragma unroll
            for (int ib = 0; ib < kRowBlocksPerBatch; ++ib)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = (i0 + ib) * 32 + 8 * (v / 4) + (v % 4);
                    const bool row_ok = lane_m0 + r < ep.m_extent;
                    const uint32_t soff = (uint32_t)(m0 + wm0 + r) * (uint32_t)ep.howo;
#pragma unroll
                    for (int j = 0; j < T::TN; ++j)
                        gate[ib][v][j] = buf_load(gate_rsrc, row_ok ? col_off4[j] : kOob, soff * 4u);
                }
        }
        if constexpr (MASKS == kGate) {
#pragma unroll
            for (int ib = 0; ib < kRowBlocksPerBatch; ++ib)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = (i0 + ib) * 32 + 8 * (v / 4) + (v % 4);
                    const bool row_ok = lane_m0 + r < ep.m_extent;
                    const uint32_t soff = (uint32_t)(m0 + wm0 + r) * (uint32_t)ep.howo;
#pragma unroll
                    for (int j = 0; j < T::TN; ++j)
                        gate[ib][v][j] = (float)(int8_t)__builtin_amdgcn_raw_buffer_load_b8(
                            gate_rsrc, (int)(row_ok ? col_off1[j] : kOob), (int)soff, 0);
                }
        }
#pragma unroll
        for (int ib = 0; ib < kRowBlocksPerBatch; ++ib)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = i0 + ib;
                const int r = i * 32 + 8 * (v / 4) + (v % 4);
                const bool row_ok = lane_m0 + r < ep.m_extent;
                const uint32_t soff = (uint32_t)(m0 + wm0 + r) * (uint32_t)ep.howo;
                const int row = wm0 + 4 * frag_k + r;  // within the tile
                float bias = 0.0f, mean = 0.0f, inv_std = 0.0f, gamma = 0.0f, beta = 0.0f;
                if (has_bias) bias = lds[row];
                if (has_bn) {
                    mean = lds[T::BM + row];
                    inv_std = lds[2 * T::BM + row];
                    gamma = lds[3 * T::BM + row];
                    beta = lds[4 * T::BM + row];
                }
#pragma unroll
                for (int j = 0; j < T::TN; ++j) {
                    float val = acc[i][j][v];
                    if (has_bias) val += bias;
                    if (has_bn) {
                        const float t = (val - mean) * inv_std;
                        val = t * gamma + beta;
                    }
                    if (ch.relu) val = val > 0.0f ? val : 0.0f;
                    if constexpr (MASKS == kGate) val *= gate[ib][v][j];
                    if constexpr (MASKS == kResidual) {
                        val += gate[ib][v][j];
                        if (ep.masks.relu_after_add) val = val > 0.0f ? val : 0.0f;
                    }
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), out_rsrc,
                                                          (int)(row_ok ? col_off4[j] : kOob), (int)(soff * 4u), 0);
                    if constexpr (MASKS == kReluMask)
                        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(val > 0.0f ? 1 : 0), mask_rsrc,
                                                             (int)(row_ok ? col_off1[j] : kOob), (int)soff, 0);
                }
            }
    }
    // the staged parameters are read until here; the caller may refill LDS afterwards
    if (has_bias || has_bn) __syncthreads();
}

// Tile store into a row-major matrix whose columns are the channels, written like store_tile_nchw: raw
// buffer stores whose out-of-range rows / columns carry an offset beyond the descriptor, each column's
// epilogue parameters fetched once, the gate bytes of a column requested before its first store.  Needs the
// destination (all splits) inside one descriptor; larger ones (`span == 0`) take the generic path.
template <class T, int MASKS>
__device__ __forceinline__ void store_tile_plain(const EpiPlainT<MASKS>& ep, const floatx16 (&acc)[T::TM][T::TN],
                                                 int m0, int n0, int split, int tid)
{
    if (ep.span == 0) {
        store_tile_generic<T>(ep, acc, m0, n0, split, tid);
        return;
    }
    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;
    const ChanEpilogue ch = ep.chan;
    const bool has_bias = ch.bias != nullptr, has_bn = ch.mean != nullptr;
    const rsrc_t out_rsrc = make_rsrc(ep.out, ep.span);
    [[maybe_unused]] rsrc_t mask_rsrc;
    if constexpr (MASKS == kGate) mask_rsrc = make_rsrc_bytes(ep.masks.gate, ep.span);
    if constexpr (MASKS == kReluMask) mask_rsrc = make_rsrc_bytes(ep.masks.relu_mask, ep.span);
    if constexpr (MASKS == kResidual) mask_rsrc = make_rsrc(ep.masks.residual, ep.span);
    const int lane_m0 = m0 + wm0 + 4 * frag_k;  // this lane's first row
    const uint32_t ldc = (uint32_t)ep.ldc;
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
        const int n = n0 + wn0 + j * 32 + frag_r;
        const bool col_ok = n < ep.n_extent;
        const int nc = col_ok ? n : 0;
        // element offset of (split, row 4*frag_k, column n); the uniform row offset rides in the scalar operand
        const uint32_t e = (uint32_t)((long)split * ep.split_stride) + (uint32_t)(4 * frag_k) * ldc + (uint32_t)nc;
        const uint32_t off4 = col_ok ? e * 4u : kOob, off1 = col_ok ? e : kOob;
        float bias = 0.0f, mean = 0.0f, inv_std = 0.0f, gamma = 0.0f, beta = 0.0f;
        if (has_bias) bias = ch.bias[nc];
        if (has_bn) {
            mean = ch.mean[nc];
            inv_std = ch.inv_std[nc];
            gamma = ch.gamma[nc];
            beta = ch.beta[nc];
        }
        [[maybe_unused]] float gate[T::TM][16];
        if constexpr (MASKS == kGate) {
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = i * 32 + 8 * (v / 4) + (v % 4);
                    const bool row_ok = lane_m0 + r < ep.m_extent;
                    gate[i][v] = (float)(int8_t)__builtin_amdgcn_raw_buffer_load_b8(
                        mask_rsrc, (int)(row_ok ? off1 : kOob), (int)((uint32_t)(m0 + wm0 + r) * ldc), 0);
                }
        }
        if constexpr (MASKS == kResidual) {
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = i * 32 + 8 * (v / 4) + (v % 4);
                    const bool row_ok = lane_m0 + r < ep.m_extent;
                    gate[i][v] = buf_load(mask_rsrc, row_ok ? off4 : kOob, (uint32_t)(m0 + wm0 + r) * ldc * 4u);
                }
        }
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = i * 32 + 8 * (v / 4) + (v % 4);
                const bool row_ok = lane_m0 + r < ep.m_extent;
                const uint32_t soff = (uint32_t)(m0 + wm0 + r) * ldc;
                float val = acc[i][j][v];
                if (has_bias) val += bias;
                if (has_bn) {
                    const float t = (val - mean) * inv_std;
                    val = t * gamma + beta;
                }
                if (ch.relu) val = val > 0.0f ? val : 0.0f;
                if constexpr (MASKS == kGate) val *= gate[i][v];
                if constexpr (MASKS == kResidual) {
                    val += gate[i][v];
                    if (ep.masks.relu_after_add) val = val > 0.0f ? val : 0.0f;
                }
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, val), out_rsrc,
                                                      (int)(row_ok ? off4 : kOob), (int)(soff * 4u), 0);
                if constexpr (MASKS == kReluMask)
                    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(val > 0.0f ? 1 : 0), mask_rsrc,
                                                         (int)(row_ok ? off1 : kOob), (int)soff, 0);
            }
    }
}

template <class EP>
struct IsEpiNchw { static constexpr bool value = false; };
template <class EP>
struct IsEpiPlain { static constexpr bool value = false; };
template <int MASKS>
struct IsEpiPlain<EpiPlainT<MASKS>> { static constexpr bool value = true; };
template <int MASKS>
struct IsEpiNchw<EpiNchwT<MASKS>> { static constexpr bool value = true; };

// `lds`: at least 5*BM floats that nobody else uses during the call.
template <class T, class EP>
__device__ __forceinline__ void store_tile(const EP& ep, const floatx16 (&acc)[T::TM][T::TN], int m0, int n0,
                                           int split, int tid, float* lds)
{
    if constexpr (IsEpiNchw<EP>::value)
        store_tile_nchw<T>(ep, acc, m0, n0, tid, lds);
    else if constexpr (IsEpiPlain<EP>::value)
        store_tile_plain<T>(ep, acc, m0, n0, split, tid);
    else
        store_tile_generic<T>(ep, acc, m0, n0, split, tid);
}

// LDS byte addresses of this lane's MFMA operand elements of buffer 0 at k-step 0, block (0, 0).
template <class T>
__device__ __forceinline__ void operand_bases(const float* As0, const float* Bs0, int tid, uint32_t* a_base,
                                              uint32_t* b_base)
{
    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;
    *a_base = lds_addr(&As0[LdsTile<T::BM>::index(frag_k, wm0 + frag_r)]);
    *b_base = lds_addr(&Bs0[LdsTile<T::BN>::index(frag_k, wn0 + frag_r)]);
}

template <class T, class AL, class BL, class EP>
__device__ __forceinline__ void gemm_body(const AL& al, const BL& bl, const EP& ep, int tiles_m, const SplitInfo& si)
{
    __shared__ __align__(16) float As[2][BK * (T::BM + kPad)];
    __shared__ __align__(16) float Bs[2][BK * (T::BN + kPad)];

    const int tid = threadIdx.x;
    // all workgroups of the launch in one sequence, tile fastest: the tiles of one reduction chunk, which
    // read the same rows of both operands, run on one XCD
    const int seq = xcd_remap((int)(blockIdx.y * gridDim.x + blockIdx.x), (int)(gridDim.x * gridDim.y));
    const int split = seq / (int)gridDim.x;
    const int tile = seq - split * (int)gridDim.x;
    const int tm_idx = tile % tiles_m, tn_idx = tile / tiles_m;
    const int m0 = tm_idx * T::BM, n0 = tn_idx * T::BN;
    const int group = split / si.cpg;
    const int chunk_idx = split - group * si.cpg;
    const int image = group * si.ips;  // first image of this workgroup's group
    const int k_total = min(si.ips, si.images - image) * si.seg_len;
    const int kbeg = chunk_idx * si.chunk;
    const int kend = min(k_total, kbeg + si.chunk);

    uint32_t a_base, b_base;
    operand_bases<T>(As[0], Bs[0], tid, &a_base, &b_base);
    floatx16 acc[T::TM][T::TN];
    clear_acc<T>(acc);
    tile_mainloop<T>(al, bl, m0, n0, image, kbeg, kend, As[0], As[1], Bs[0], Bs[1], a_base, b_base, acc, tid);
    store_tile<T>(ep, acc, m0, n0, split, tid, As[0]);
}

// Three workgroups per compute unit need at most 168 registers per lane.  The kernels are built under that
// limit unless a loader's per-thread state (precomputed offsets / masks of 16 elements per step) is so large
// that the limit would spill inside the reduction loop (`kLargeState`); those are built without it.  Tiles of
// eight MFMA blocks per wavefront (256x128) hold 128 accumulator registers and are built for two
// workgroups per CU (256 registers).
template <class T, class AL, class BL>
struct WorkgroupsPerCu {
    static constexpr int value = T::TM * T::TN > 4 ? 2 : (AL::kLargeState || BL::kLargeState) ? 0 : 3;  // 0: no limit
};

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3)))
gemm_kernel(AL al, BL bl, EP ep, int tiles_m, SplitInfo si)
{
    gemm_body<T>(al, bl, ep, tiles_m, si);
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_kernel_big_tile(AL al, BL bl, EP ep, int tiles_m, SplitInfo si)
{
    gemm_body<T>(al, bl, ep, tiles_m, si);
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) gemm_kernel_large_state(AL al, BL bl, EP ep, int tiles_m, SplitInfo si)
{
    gemm_body<T>(al, bl, ep, tiles_m, si);
}

template <class T, class AL, class BL, class EP>
inline int launch(const AL& al, const BL& bl, const EP& ep, long m, long n, const SplitInfo& si, int splits,
                  hipStream_t stream)
{
    const long tiles_m = (m + T::BM - 1) / T::BM, tiles_n = (n + T::BN - 1) / T::BN;
    if (tiles_m * tiles_n * splits >= (1l << 31) || splits > 65535 || splits < 1) return PYDTNN_HIP_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)splits);
    constexpr int kPerCu = WorkgroupsPerCu<T, AL, BL>::value;
    if constexpr (kPerCu == 3)
        hipLaunchKernelGGL((gemm_kernel<T, AL, BL, EP>), grid, dim3(kThreads), 0, stream, al, bl, ep, (int)tiles_m, si);
    else if constexpr (kPerCu == 2)
        hipLaunchKernelGGL((gemm_kernel_big_tile<T, AL, BL, EP>), grid, dim3(kThreads), 0, stream, al, bl, ep,
                           (int)tiles_m, si);
    else
        hipLaunchKernelGGL((gemm_kernel_large_state<T, AL, BL, EP>), grid, dim3(kThreads), 0, stream, al, bl, ep,
                           (int)tiles_m, si);
    HIP_RETURN_IF_LAUNCH_FAILED();
    note_launch(kLaunchTiles, T::BM, T::BN, tiles_m * tiles_n * splits, 0, splits);
    return PYDTNN_HIP_OK;
}

// ---------------------------------------------------------------- balanced ("stream-K") form
// A grid of whole tiles leaves compute units idle whenever the tile count is not a multiple of
// what the chip holds at once: 3136 tiles on 256 CUs is 12.25 per CU, so the launch lasts as long
// as 13.  Here the grid is exactly the number of workgroups the chip holds (`gridDim.x`), and
//   * the tiles [0, sk_tiles), sk_tiles = tiles mod gridDim.x, are cut along the reduction axis
//     into units of 2*BK and the units are dealt out evenly: workgroup g takes units
//     [g*U/G, (g+1)*U/G) of the U = sk_tiles*units in all, crossing tile borders as they come;
//   * the remaining tiles, a multiple of the grid, go round-robin, whole.
// A workgroup that holds a tile's whole reduction range stores it through the epilogue; otherwise it
// stores the raw accumulators to one of its two slots of `partial` (a range touches at most two
// tiles partially: slot 0 for the piece that starts at the workgroup's first unit, slot 1 for the
// other), and streamk_fixup_kernel adds a tile's pieces in ascending reduction order and applies
// the epilogue.  No workgroup waits for another, and the result does not depend on timing.
struct StreamK {
    int tiles;      // all tiles of the GEMM
    int sk_tiles;   // tiles cut into units
    int sk_blocks;  // workgroups that take part in the unit phase (each gets at least a few units)
    int units;      // units of 2*BK per tile
    int k;          // reduction length
    float* partial; // 2 * gridDim.x slots of BM*BN floats
};

__host__ __device__ inline long sk_first_unit(int g, long total_units, int sk_blocks)
{
    return (long)g * total_units / sk_blocks;
}

template <class T, class AL, class BL, class EP>
__device__ __forceinline__ void gemm_streamk_body(const AL& al, const BL& bl, const EP& ep, int tiles_m, const StreamK& sk)
{
    __shared__ __align__(16) float As[2][BK * (T::BM + kPad)];
    __shared__ __align__(16) float Bs[2][BK * (T::BN + kPad)];

    const int tid = threadIdx.x;
    const int g = xcd_remap(blockIdx.x, gridDim.x);
    uint32_t a_base, b_base;
    operand_bases<T>(As[0], Bs[0], tid, &a_base, &b_base);

    const long total = (long)sk.sk_tiles * sk.units;
    long u = 0, u_end = 0;
    if (g < sk.sk_blocks) {
        u = sk_first_unit(g, total, sk.sk_blocks);
        u_end = sk_first_unit(g + 1, total, sk.sk_blocks);
    }
    const long u_first = u;
    // Workgroups that share a compute unit would otherwise run in lockstep (all of them in their
    // prologue or their epilogue at once, with the matrix cores idle).  They are launched a third of
    // the grid apart, so each third takes its units after a different number of whole tiles.
    int whole_before_units = (int)((long)blockIdx.x * 3 / gridDim.x);
    int whole_tile = sk.sk_tiles + g;
    for (;;) {
        int tile, kbeg, kend;
        bool whole;
        float* slot = nullptr;
        const bool units_left = u < u_end, tiles_left = whole_tile < sk.tiles;
        if (units_left && (whole_before_units <= 0 || !tiles_left)) {
            tile = (int)(u / sk.units);
            const int ku0 = (int)(u - (long)tile * sk.units);
            const long left = u_end - u;
            const int ku1 = left < sk.units - ku0 ? ku0 + (int)left : sk.units;
            kbeg = ku0 * 2 * BK;
            kend = min(sk.k, ku1 * 2 * BK);
            whole = ku0 == 0 && ku1 == sk.units;
            // slot 0 for the piece that starts at this workgroup's first unit, slot 1 for a piece that
            // starts at a tile border
            slot = sk.partial + (size_t)(2 * g + (u == u_first ? 0 : 1)) * (T::BM * T::BN);
            u += ku1 - ku0;
        } else if (tiles_left) {
            tile = whole_tile;
            kbeg = 0;
            kend = sk.k;
            whole = true;
            whole_tile += gridDim.x;
            --whole_before_units;
        } else {
            break;
        }
        const int tm_idx = tile % tiles_m, tn_idx = tile / tiles_m;
        const int m0 = tm_idx * T::BM, n0 = tn_idx * T::BN;
        floatx16 acc[T::TM][T::TN];
        clear_acc<T>(acc);
        tile_mainloop<T>(al, bl, m0, n0, 0, kbeg, kend, As[0], As[1], Bs[0], Bs[1], a_base, b_base, acc, tid);
        if (whole) {
            store_tile<T>(ep, acc, m0, n0, 0, tid, As[0]);
        } else {
            float* dst = slot + tid;
#pragma unroll
            for (int i = 0; i < T::TM; ++i)
#pragma unroll
                for (int j = 0; j < T::TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) dst[((i * T::TN + j) * 16 + v) * kThreads] = acc[i][j][v];
        }
    }
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3)))
gemm_streamk_kernel(AL al, BL bl, EP ep, int tiles_m, StreamK sk)
{
    gemm_streamk_body<T>(al, bl, ep, tiles_m, sk);
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_streamk_kernel_big_tile(AL al, BL bl, EP ep, int tiles_m, StreamK sk)
{
    gemm_streamk_body<T>(al, bl, ep, tiles_m, sk);
}

template <class T, class AL, class BL, class EP>
__global__ void __launch_bounds__(kThreads) gemm_streamk_kernel_large_state(AL al, BL bl, EP ep, int tiles_m, StreamK sk)
{
    gemm_streamk_body<T>(al, bl, ep, tiles_m, sk);
}

// grid (sk_tiles, TM*TN*4): a workgroup owns four of the 16*TM*TN accumulator registers of one
// tile; if the tile was cut, it adds their pieces in ascending reduction order and stores them.
template <class T, class EP>
__global__ void __launch_bounds__(kThreads) streamk_fixup_kernel(EP ep, int tiles_m, StreamK sk)
{
    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int quad = blockIdx.y;  // registers [4*quad, 4*quad + 4) in (i, j, v) order
    const long total = (long)sk.sk_tiles * sk.units;
    const long a = (long)tile * sk.units, b = a + sk.units;
    // the workgroup whose range holds unit a
    int g = (int)(((a + 1) * sk.sk_blocks - 1) / total);
    while (g > 0 && sk_first_unit(g, total, sk.sk_blocks) > a) --g;
    while (g + 1 < sk.sk_blocks && sk_first_unit(g + 1, total, sk.sk_blocks) <= a) ++g;
    if (sk_first_unit(g + 1, total, sk.sk_blocks) >= b) return;  // it held the whole tile and stored it

    // The ranges of the workgroups are consecutive and none is empty, so the tile's pieces are those of the
    // workgroups g .. g_last, one each; only the first can have begun before the tile did (it then lies in its
    // workgroup's slot 1).  Eight pieces are requested at a time and added in ascending order.
    int g_last = (int)((b * sk.sk_blocks - 1) / total);
    while (g_last > g && sk_first_unit(g_last, total, sk.sk_blocks) >= b) --g_last;
    while (g_last + 1 < sk.sk_blocks && sk_first_unit(g_last + 1, total, sk.sk_blocks) < b) ++g_last;
    const int first_slot = sk_first_unit(g, total, sk.sk_blocks) < a ? 1 : 0;
    const float* lane_base = sk.partial + quad * 4 * kThreads + tid;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int g0 = g; g0 <= g_last; g0 += 8) {
        float v[8][4];
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int gg = g0 + p;
            const float* src = lane_base + (size_t)(2 * gg + (gg == g ? first_slot : 0)) * (T::BM * T::BN);
#pragma unroll
            for (int q = 0; q < 4; ++q) v[p][q] = gg <= g_last ? src[q * kThreads] : 0.0f;
        }
#pragma unroll
        for (int p = 0; p < 8; ++p)
            if (g0 + p <= g_last) {
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[q] += v[p][q];
            }
    }
    const int ij = quad >> 2, i = ij / T::TN, j = ij - i * T::TN, v0 = (quad & 3) * 4;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm0 = (wave % T::WGM) * T::WM, wn0 = (wave / T::WGM) * T::WN;
    const int frag_r = lane & 31, frag_k = lane >> 5;
    const int m0 = (tile % tiles_m) * T::BM, n0 = (tile / tiles_m) * T::BN;
    const typename EP::Col col = ep.column(n0 + wn0 + j * 32 + frag_r, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) ep.store(col, m0 + wm0 + i * 32 + 8 * ((v0 + q) / 4) + 4 * frag_k + ((v0 + q) % 4), acc[q]);
}

// Workgroups of gemm_streamk_kernel<T, ...> the device holds at once, and its compute units.
struct Residency {
    int workgroups;
    int cus;
};

template <class T, class AL, class BL, class EP>
inline hipError_t streamk_blocks_per_cu(int* per_cu)
{
    constexpr int kPerCu = WorkgroupsPerCu<T, AL, BL>::value;
    if constexpr (kPerCu == 3)
        return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, gemm_streamk_kernel<T, AL, BL, EP>, kThreads, 0);
    else if constexpr (kPerCu == 2)
        return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, gemm_streamk_kernel_big_tile<T, AL, BL, EP>,
                                                            kThreads, 0);
    else
        return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, gemm_streamk_kernel_large_state<T, AL, BL, EP>,
                                                            kThreads, 0);
}

// Asked from the runtime once per device and kernel; the answer is two ints, so a race between two first
// callers only repeats the query.
template <class T, class AL, class BL, class EP>
inline Residency resident_workgroups()
{
    constexpr int kDevices = 64;
    static std::atomic<int> workgroups[kDevices], compute_units[kDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kDevices) return Residency{0, 0};
    Residency r = {workgroups[dev].load(std::memory_order_acquire), compute_units[dev].load(std::memory_order_relaxed)};
    if (r.workgroups == 0) {
        int cus = 0, per_cu = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            streamk_blocks_per_cu<T, AL, BL, EP>(&per_cu) != hipSuccess || cus <= 0 || per_cu <= 0)
            return Residency{0, 0};
        r.workgroups = cus * per_cu;
        r.cus = cus;
        compute_units[dev].store(cus, std::memory_order_relaxed);
        workgroups[dev].store(r.workgroups, std::memory_order_release);
    }
    return r;
}

inline size_t streamk_workspace_bytes(int resident, int bm, int bn) { return (size_t)2 * resident * bm * bn * 4; }

// C = A*B over the full reduction range [0, k), balanced as described above when that pays and
// `partial` is large enough; otherwise the plain grid of whole tiles.
// `must_balance`: the caller has no use for the plain grid (few tiles, long reduction); returns
// kNotBalanced without launching when the balanced form is not possible.
constexpr int kNotBalanced = -1;

template <class T, class AL, class BL, class EP>
inline int launch_balanced(const AL& al, const BL& bl, const EP& ep, long m, long n, int k, float* partial,
                           size_t partial_bytes, hipStream_t stream, bool must_balance = false)
{
    const long tiles_m = (m + T::BM - 1) / T::BM, tiles_n = (n + T::BN - 1) / T::BN;
    const long tiles = tiles_m * tiles_n;
    if (tiles >= (1l << 31)) return PYDTNN_HIP_ERR_UNSUPPORTED;
    // The grid, and with it where the reduction ranges are cut, is that of the kernel without byte masks:
    // a masked launch then adds the same pieces in the same order and gives the same bits.
    const Residency res = resident_workgroups<T, AL, BL, typename EP::Unmasked>();
    const int resident = res.workgroups;
    const int units = (k + 2 * BK - 1) / (2 * BK);
    bool balanced = resident > 0 && partial && partial_bytes >= streamk_workspace_bytes(resident, T::BM, T::BN) &&
                    tiles % resident != 0 && units >= 8;
    if (balanced && !must_balance) {
        // A plain grid keeps every compute unit busy for ceil(tiles / CUs) tile times; balancing is
        // worth its partial-tile traffic only when more than a twentieth of that is idle.
        const double per_cu = (double)tiles / res.cus;
        const double rounds = (double)((tiles + res.cus - 1) / res.cus);
        balanced = per_cu / rounds < 0.95;
    }
    if (!balanced) return must_balance ? kNotBalanced : launch<T>(al, bl, ep, m, n, no_split(k), 1, stream);
    StreamK sk;
    sk.tiles = (int)tiles;
    sk.sk_tiles = (int)(tiles % resident);
    sk.units = units;
    sk.k = k;
    sk.partial = partial;
    const long total = (long)sk.sk_tiles * units;
    // at least two units (four reduction steps) per piece: with few cut tiles and a short reduction the pieces
    // of four units that this used to deal added a fifth to the longest workgroup's run
    const long pieces = total / 2;
    sk.sk_blocks = (int)(pieces < resident ? (pieces > 0 ? pieces : 1) : resident);
    constexpr int kPerCu = WorkgroupsPerCu<T, AL, BL>::value;
    if constexpr (kPerCu == 3)
        hipLaunchKernelGGL((gemm_streamk_kernel<T, AL, BL, EP>), dim3((unsigned)resident), dim3(kThreads), 0, stream,
                           al, bl, ep, (int)tiles_m, sk);
    else if constexpr (kPerCu == 2)
        hipLaunchKernelGGL((gemm_streamk_kernel_big_tile<T, AL, BL, EP>), dim3((unsigned)resident), dim3(kThreads), 0,
                           stream, al, bl, ep, (int)tiles_m, sk);
    else
        hipLaunchKernelGGL((gemm_streamk_kernel_large_state<T, AL, BL, EP>), dim3((unsigned)resident),
                           dim3(kThreads), 0, stream, al, bl, ep, (int)tiles_m, sk);
    HIP_RETURN_IF_LAUNCH_FAILED();
    if (sk.sk_tiles > 0) {
        hipLaunchKernelGGL((streamk_fixup_kernel<T, EP>), dim3((unsigned)sk.sk_tiles, T::TM * T::TN * 4), dim3(kThreads), 0,
                           stream, ep, (int)tiles_m, sk);
        HIP_RETURN_IF_LAUNCH_FAILED();
    }
    note_launch(kLaunchBalanced, T::BM, T::BN, resident, sk.sk_tiles, 1);
    return PYDTNN_HIP_OK;
}

}  // namespace gemm

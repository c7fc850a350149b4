// sparse_gather on gfx950: NHWC block stack (row-segment copies) and the fused transpose to [blocks, C, R, S]
// (LDS-staged tiles; workgroups that own whole 128-byte lines of the stack), with the launch configuration.
// Reference semantics: sbnet_tensorflow/sbnet_ops/sparse_gather.cc:67-88.
#include "sbnet_device.h"

namespace sbnet {

// sparse_gather.cc:67-88 with transpose == false.
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_nhwc_wide(const float* __restrict__ x, float* __restrict__ y,
                                                     const int16_t* __restrict__ idx, NhwcArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);  // ib is wave-uniform: scalar load
    const int CV = a.g.C / VEC;
    // columns [slo, shi) of the block lie inside the image
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const vec* __restrict__ xv = reinterpret_cast<const vec*>(x);
    vec* __restrict__ yb = reinterpret_cast<vec*>(y) + (size_t)ib * a.blockV;
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;

    vec v[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        v[u] = vzero<VEC>();
        if (e < a.blockV) {
            const uint32_t r = fdiv(e, a.dRow);
            const int j = (int)(e - r * a.rowV);
            const int hh = o.h0 + (int)r;
            if (o.valid && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi) {
                const int64_t src = (((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0) * CV + j;
                v[u] = ld_stream(xv + src);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        if (e < a.blockV) st_stream(yb + e, v[u]);
    }
}

template <int VEC>
__global__ __launch_bounds__(256) void k_gather_nhwc(const float* __restrict__ x, float* __restrict__ y,
                                                     const int16_t* __restrict__ idx, NhwcArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    const uint32_t ib = fdiv(unit, a.dCpb);
    if (beyond_count(a.g, ib)) return;
    const uint32_t chunk = unit - ib * a.cpb;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const int64_t imgFloats = (int64_t)a.g.H * a.g.W * a.g.C;
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * imgFloats : 0), o.valid ? (uint32_t)imgFloats * 4u : 0u);
    const rsrc_t yr = make_rsrc(y + (int64_t)ib * a.blockV * VEC, a.blockV * (uint32_t)(VEC * 4));
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;
    vec v[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        const uint32_t r = fdiv(e, a.dRow);
        const int j = (int)(e - r * a.rowV);
        const int hh = o.h0 + (int)r;
        const bool ok = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi;
        // (unsigned arithmetic: the value only matters when ok, and then it is the in-range offset)
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0) * (uint32_t)CV + (uint32_t)j) * (uint32_t)(VEC * 4);
        v[u] = buf_load<VEC>(xr, ok ? off : BUF_OOB);
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        buf_store<BUF_NT>(yr, e < a.blockV ? e * (uint32_t)(VEC * 4) : BUF_OOB, v[u]);
    }
}

// sparse_gather.cc:67-88 with transpose == true: y[ib, c, r, s] = x[n, h0+r, w0+s, c] or 0.
template <int VEC>
__device__ __forceinline__ void gather_planar_tile(const float* __restrict__ x, float* __restrict__ y,
                                                   const int16_t* __restrict__ idx, const TileArgs& a, float* lds,
                                                   uint32_t ib, uint32_t rem)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t tid = threadIdx.x, nthr = blockDim.x;
    const uint32_t RS = (uint32_t)(a.g.R * a.g.S);
    TileId t;
    decode_tile<TileRt>(a, t, ib, rem);
    const RawTriple raw = load_triple(idx, t.ib);
    if (beyond_count(a.g, t.ib)) return;
    const BlockOrigin o = origin_of(raw, a.g);
    // a block index outside [0, N) gets an empty descriptor: every load returns 0
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * a.imgFloats : 0), o.valid ? a.imgBytes : 0u);

    vec v[TILE_LD];
    uint32_t pls[TILE_LD];
    nhwc_walk<VEC, TileRt>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t, uint32_t, uint32_t) {
        v[u] = buf_load<VEC>(xr, off);
        pls[u] = pl;
    });

    // registers -> LDS, transposing: this thread's VEC channels go to VEC rows, pixel pl to column pl
    const uint32_t c0l = (tid & ((1u << a.lppLog) - 1u)) * VEC;
#pragma unroll
    for (int u = 0; u < TILE_LD; ++u) {
        if (pls[u] < (uint32_t)t.Pn) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const uint32_t c = c0l + k;
                lds[c * a.Pp + (pls[u] ^ lds_swz(c))] = vget(v[u], k);
            }
        }
    }
    lds_barrier();

    // LDS -> global, planar side.  Full slots in a flat, branch-free loop ...
    const rsrc_t yr = make_rsrc(y + ((int64_t)t.ib * a.g.C + t.c0) * RS + t.p0,
                                ((uint32_t)(t.ctEff - 1) * RS + (uint32_t)t.Pn) * 4u);
    const uint32_t slots = (uint32_t)t.ctEff * a.vpr;
    for (uint32_t base = 0; base < slots; base += 4 * nthr) {
        f4 q[4];
        uint32_t off[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t i = base + u * nthr + tid;
            const uint32_t c = fdiv(i, a.dVpr);
            const uint32_t e0 = 4u * (i - c * a.vpr);
            const bool full = i < slots && e0 + 4u <= (uint32_t)t.Pn;
            q[u] = lds_read4(lds + (full ? c * a.Pp + (e0 ^ lds_swz(c)) : 0u));
            off[u] = full ? (c * RS + e0) * 4u : BUF_OOB;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) buf_store<BUF_NT>(yr, off[u], q[u]);
    }
    // ... then the 1-3 floats that end a run whose length is not a multiple of 4, one row per thread
    const uint32_t tail = (uint32_t)t.Pn & 3u;
    if (tail && tid < (uint32_t)t.ctEff) {
        const uint32_t e0 = (uint32_t)t.Pn - tail;
        const f4 q = lds_read4(lds + tid * a.Pp + (e0 ^ lds_swz(tid)));
        const uint32_t off = (tid * RS + e0) * 4u;
        buf_store<0>(yr, off, q.x);
        if (tail > 1) buf_store<0>(yr, off + 4u, q.y);
        if (tail > 2) buf_store<0>(yr, off + 8u, q.z);
    }
}

template <int VEC>
__global__ __launch_bounds__(512) void k_gather_planar(const float* __restrict__ x, float* __restrict__ y,
                                                       const int16_t* __restrict__ idx, TileArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for_each_block_of_workgroup(a, a.tpb, [&](uint32_t ib, uint32_t rem) {
        gather_planar_tile<VEC>(x, y, idx, a, lds, ib, rem);
    });
}

// ---------------------------------------------------------------------------------------------
// Planar gather whose workgroups own whole, aligned 64-byte pieces ("lines") of the output
// ---------------------------------------------------------------------------------------------
//
// A write-only probe of the tile pattern above (32 runs of 243 floats at 729-float pitch, 4-byte
// aligned, first and last line of every run shared with another workgroup) reaches 3.5 TB/s; the same
// bytes written as whole, 16-byte aligned lines that belong to one workgroup each reach 5.9 TB/s.
// So this kernel cuts the output differently.  The Ct planes of a channel chunk are one contiguous
// piece of y, "the chunk", addressed by a linear float index l = c*RS + p.  Tile (chunk, split) still
// reads the pixels [p0, p1) for all Ct channels, but for row c it writes the lines that START inside
// [c*RS + p0, c*RS + p1): the range [up(c*RS + p0), up(c*RS + p1)), up() rounding to the next line of
// y (the two ends of the chunk stay where they are).  These ranges tile the chunk exactly, every store
// is an aligned dwordx4, and no line is written by two workgroups (except the one line two chunks may
// share).  The price is that a tile needs up to LINE_EXT pixels beyond p1 -- for the last split of a
// plane, where row c's last line runs into row c+1, the first pixels of the plane -- so the tile's pixel
// window is [p0, p1 + LINE_EXT) taken cyclically over the plane; the extra pixels are read by the
// neighbouring tile as well and mostly come from cache.  Used when a plane is split over several tiles;
// a tile of whole planes already writes one contiguous piece.
//
// The unit of ownership is 64 bytes, the granularity of an access to HBM, not the 128 bytes of an L2 line: with
// 16-float units a tile reads 15 extra pixels instead of 31 (6 % instead of 13 % more NHWC reads at 243 pixels
// per tile) and the launch on 312 blocks of 27x27x128 takes 39.05 us instead of 39.6; 32-byte units are no
// faster than 128-byte ones (39.5 us, and 8.8 against 7.5 us on 58 blocks).
//
// LDS: row c at c*Pp, window pixel q at column q + phi(c), phi(c) = (c*RS + p0) & 3, XOR-swizzled as
// above.  The shift phi makes LDS columns congruent to l modulo 4, so every output slot is one
// ds_read_b128.  In the last split the wrapped pixels of channel c (the first pixels of its plane) are
// stored behind the pixels of channel c-1 instead, where l continues: the slots of row c-1's last line
// that cross into plane c are then contiguous in LDS like any other.

constexpr int LINE_FLOATS = 16;
constexpr int LINE_EXT = LINE_FLOATS - 1;

struct LineArgs {
    Geom g;
    int Ct, lppLog;
    int RS;
    int P, Pp, psplit, cchunks;
    int grid2d;         // the launch is (tpb, block rows): see for_each_block_of_workgroup
    uint32_t blocks;    // capacity of the block list (numActive)
    uint32_t tpb, total;
    uint32_t spr;       // bound on the output slots of one row of one tile
    int64_t imgFloats;
    uint32_t imgBytes;
    FastDiv dTpb, dPs, dS;
};

// Geometry of a launch as the kernels see it: either read from the argument struct (any shape) or fixed at compile
// time for the shapes the benchmark configurations use.  With constants the reciprocal divisions, the pitch
// multiplications and the pixel-step bookkeeping fold away (about a third of the vector instructions of a tile),
// LDS accesses take immediate offsets and the unused staging variants are not compiled in.  The host launches a
// fixed-shape instance only when the tile it chose equals the instance's (sbnet_launch.h: Geom::forceGeneric keeps
// tests on the run-time path).
struct LinesRt {
    static constexpr bool FIXED = false;
    __device__ static uint32_t nthr(const LineArgs&) { return blockDim.x; }
    __device__ static uint32_t R(const LineArgs& a) { return (uint32_t)a.g.R; }
    __device__ static uint32_t S(const LineArgs& a) { return (uint32_t)a.g.S; }
    __device__ static uint32_t C(const LineArgs& a) { return (uint32_t)a.g.C; }
    __device__ static uint32_t RS(const LineArgs& a) { return (uint32_t)a.RS; }
    __device__ static uint32_t P(const LineArgs& a) { return (uint32_t)a.P; }
    __device__ static uint32_t Pp(const LineArgs& a) { return (uint32_t)a.Pp; }
    __device__ static uint32_t psplit(const LineArgs& a) { return (uint32_t)a.psplit; }
    __device__ static uint32_t Ct(const LineArgs& a) { return (uint32_t)a.Ct; }
    __device__ static uint32_t lppLog(const LineArgs& a) { return (uint32_t)a.lppLog; }
    __device__ static uint32_t tpb(const LineArgs& a) { return a.tpb; }
    __device__ static uint32_t divS(uint32_t v, const LineArgs& a) { return fdiv(v, a.dS); }
    __device__ static uint32_t divPs(uint32_t v, const LineArgs& a) { return fdiv(v, a.dPs); }
    __device__ static uint32_t divTpb(uint32_t v, const LineArgs& a) { return fdiv(v, a.dTpb); }
};

template <int R_, int S_, int C_, int PSPLIT_, int NTHR_>
struct LinesFixed {
    static constexpr bool FIXED = true;
    static constexpr uint32_t kRS = R_ * S_;
    static constexpr uint32_t kLpp = C_ >= 32 ? 8 : C_ / 4;  // C_ a multiple of 4; Ct = min(C_, 32) rounded to 2^k*4
    static constexpr uint32_t kLppLog = kLpp == 8 ? 3 : kLpp == 4 ? 2 : kLpp == 2 ? 1 : 0;
    static constexpr uint32_t kP = (kRS + PSPLIT_ - 1) / PSPLIT_;
    static constexpr uint32_t kPp = (kP + LINE_EXT + 3 + 31) / 32 * 32;
    static constexpr uint32_t kCchunks = (C_ + 4 * kLpp - 1) / (4 * kLpp);
    static constexpr int kLD = (int)(((kP + LINE_EXT) * kLpp + NTHR_ - 1) / NTHR_) < 4
                                   ? 4 : (int)(((kP + LINE_EXT) * kLpp + NTHR_ - 1) / NTHR_);
    __host__ __device__ static constexpr uint32_t nthr(const LineArgs&) { return NTHR_; }
    __host__ __device__ static constexpr uint32_t R(const LineArgs&) { return R_; }
    __host__ __device__ static constexpr uint32_t S(const LineArgs&) { return S_; }
    __host__ __device__ static constexpr uint32_t C(const LineArgs&) { return C_; }
    __host__ __device__ static constexpr uint32_t RS(const LineArgs&) { return kRS; }
    __host__ __device__ static constexpr uint32_t P(const LineArgs&) { return kP; }
    __host__ __device__ static constexpr uint32_t Pp(const LineArgs&) { return kPp; }
    __host__ __device__ static constexpr uint32_t psplit(const LineArgs&) { return PSPLIT_; }
    __host__ __device__ static constexpr uint32_t Ct(const LineArgs&) { return 4 * kLpp; }
    __host__ __device__ static constexpr uint32_t lppLog(const LineArgs&) { return kLppLog; }
    __host__ __device__ static constexpr uint32_t tpb(const LineArgs&) { return PSPLIT_ * kCchunks; }
    __host__ __device__ static constexpr uint32_t divS(uint32_t v, const LineArgs&) { return v / (uint32_t)S_; }
    __host__ __device__ static constexpr uint32_t divPs(uint32_t v, const LineArgs&) { return v / (uint32_t)PSPLIT_; }
    __host__ __device__ static constexpr uint32_t divTpb(uint32_t v, const LineArgs&) { return v / (PSPLIT_ * kCchunks); }
};

template <int LD, typename G>
__device__ __forceinline__ void gather_lines_tile(const float* __restrict__ x, float* __restrict__ y,
                                                  const int16_t* __restrict__ idx, const LineArgs& a, float* lds,
                                                  uint32_t ib, uint32_t rem)
{
    const uint32_t tid = threadIdx.x, nthr = G::nthr(a);
    const uint32_t RS = G::RS(a), S = G::S(a), R = G::R(a), C = G::C(a), Pp = G::Pp(a);
    const uint32_t lppLog = G::lppLog(a);

    const RawTriple raw = load_triple(idx, ib);
    if (beyond_count(a.g, ib)) return;
    const uint32_t cc = G::divPs(rem, a);
    const uint32_t split = rem - cc * G::psplit(a);
    const uint32_t c0 = cc * G::Ct(a);
    const uint32_t ctEff = min(G::Ct(a), C - c0);
    const uint32_t p0 = split * G::P(a);
    const uint32_t p1 = min(p0 + G::P(a), RS);
    const uint32_t win = p1 - p0 + (uint32_t)LINE_EXT;

    const BlockOrigin o = origin_of(raw, a.g);
    const rsrc_t xr = make_rsrc(x + (o.valid ? (int64_t)o.n * a.imgFloats : 0), o.valid ? a.imgBytes : 0u);

    // NHWC side: lane owns channels [4*cl, 4*cl + 4) of window pixels q0 + u*step.  (r, s) of the pixel is
    // kept by increments; stepping past the end of the plane wraps to its start, which is r -= R.
    const uint32_t cl = tid & ((1u << lppLog) - 1u);
    const uint32_t q0 = tid >> lppLog, step = nthr >> lppLog;
    const uint32_t c = c0 + cl * 4u;
    const bool cok = c < C;
    const uint32_t stepR = G::divS(step, a), stepS = step - stepR * S;
    uint32_t r, sc;
    {
        uint32_t p = p0 + q0;
        if (p >= RS) p -= RS;
        r = G::divS(p, a);
        sc = p - r * S;
    }
    f4 v[LD];
#pragma unroll
    for (int u = 0; u < LD; ++u) {
        const uint32_t q = q0 + (uint32_t)u * step;
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)sc;
        const bool ok = cok && q < win && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww) * C + c) * 4u;
        v[u] = buf_load<4>(xr, ok ? off : BUF_OOB);
        sc += stepS;
        r += stepR;
        if (sc >= S) {
            sc -= S;
            ++r;
        }
        if (r >= R) r -= R;
    }
    // registers -> LDS.  In the last split of a plane the window wraps: its pixels from `wrapStart` on are the
    // first pixels of the plane, which the output needs as the continuation of the PREVIOUS channel's row (the
    // last line of row c-1 runs into row c).  They are stored there, behind row c-1's own pixels, so that every
    // output slot is one aligned 16-byte LDS read; channel 0 of the chunk has no predecessor and drops them.
    const uint32_t wrapStart = (p1 == RS && p0 != 0u) ? RS - p0 : 0xFFFFFFFFu;
    if (wrapStart == 0xFFFFFFFFu) {
        // With a pixel step that is a multiple of 32 the swizzle (bits 2..4 of the column) does not depend on u,
        // and the column of (u, k) is the column of (0, k) plus u*step.
        const uint32_t swz = lds_swz(cl * 4u);
        uint32_t rowAddr[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t phi = ((uint32_t)k * RS + p0) & 3u;  // == ((4*cl + k)*RS + p0) & 3
            rowAddr[k] = (cl * 4u + (uint32_t)k) * Pp + phi;
        }
        if ((step & 31u) == 0) {
#pragma unroll
            for (int k = 0; k < 4; ++k) rowAddr[k] = (rowAddr[k] & ~3u) + (((rowAddr[k] & 3u) + q0) ^ swz);
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                if (q0 + (uint32_t)u * step < win) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) lds[rowAddr[k] + (uint32_t)u * step] = vget(v[u], k);
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                const uint32_t q = q0 + (uint32_t)u * step;
                if (q < win) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        lds[(rowAddr[k] & ~3u) + (((rowAddr[k] & 3u) + q) ^ swz)] = vget(v[u], k);
                }
            }
        }
    } else if ((step & 31u) == 0) {
        // the same with the wrapped pixels one row up: rows 4*cl+k-1 are this thread's own rows 4*cl+k-1 for
        // k >= 1 (same swizzle group), and row 4*cl-1 for k = 0
        const uint32_t swz = lds_swz(cl * 4u);
        uint32_t rowAddr[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t phi = ((uint32_t)k * RS + p0) & 3u;
            rowAddr[k] = (cl * 4u + (uint32_t)k) * Pp + ((phi + q0) ^ swz);
        }
        const uint32_t rowP = cl * 4u - 1u;  // no such row for cl == 0: channel 0 drops its wrapped pixels
        const uint32_t addrP = rowP * Pp + ((((rowP * RS + p0) & 3u) + q0) ^ lds_swz(rowP));
#pragma unroll
        for (int u = 0; u < LD; ++u) {
            const uint32_t q = q0 + (uint32_t)u * step;
            if (q < win) {
                const bool wr = q >= wrapStart;
                if (!(wr && cl == 0u)) lds[(wr ? addrP : rowAddr[0]) + (uint32_t)u * step] = vget(v[u], 0);
#pragma unroll
                for (int k = 1; k < 4; ++k) lds[(wr ? rowAddr[k - 1] : rowAddr[k]) + (uint32_t)u * step] = vget(v[u], k);
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < LD; ++u) {
            const uint32_t q = q0 + (uint32_t)u * step;
            if (q < win) {
                const uint32_t back = q >= wrapStart ? 1u : 0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t row = cl * 4u + (uint32_t)k - back;  // 0xFFFFFFFF for channel 0's wrapped pixels
                    const uint32_t phi = (row * RS + p0) & 3u;
                    if (row != 0xFFFFFFFFu) lds[row * Pp + ((phi + q) ^ lds_swz(row))] = vget(v[u], k);
                }
            }
        }
    }
    lds_barrier();

    // planar side: whole lines of the chunk
    const int64_t chunkBase = ((int64_t)ib * C + c0) * RS;
    const uint32_t chunkFloats = ctEff * RS;
    const uint32_t a0 = (uint32_t)(((reinterpret_cast<uintptr_t>(y) >> 2) + (uint64_t)chunkBase) & (LINE_FLOATS - 1));
    const rsrc_t yr = make_rsrc(y + chunkBase, chunkFloats * 4u);
    {
        // One wave per row, four rows in flight: everything about the row (its range [A, B) of whole lines,
        // its swizzle) is wave-uniform and stays on the scalar unit; a lane only adds 4*k.
        const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
        const uint32_t lane = tid & 63u, nwaves = nthr >> 6;
        for (uint32_t cr0 = wave; cr0 < ctEff; cr0 += 4u * nwaves) {
            for (uint32_t kb = 0; kb < a.spr; kb += 64u) {
                f4 qv[4];
                uint32_t off[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t cr = cr0 + (uint32_t)u * nwaves;
                    const uint32_t lin0 = cr * RS + p0, lin1 = cr * RS + p1;
                    const uint32_t A = (lin0 == 0) ? 0u : ((a0 + lin0 + LINE_EXT) & ~(uint32_t)LINE_EXT) - a0;
                    const uint32_t B = (cr >= ctEff)          ? 0u
                                       : (lin1 == chunkFloats) ? chunkFloats
                                                               : ((a0 + lin1 + LINE_EXT) & ~(uint32_t)LINE_EXT) - a0;
                    const uint32_t colBase = A - lin0 + (lin0 & 3u);  // multiple of 4 less than 36
                    const uint32_t k4 = 4u * (kb + lane);
                    const uint32_t l = A + k4;
                    const bool live = l < B;
                    // (a row's last line may run into the next plane: those pixels sit behind the row in LDS)
                    qv[u] = lds_read4(lds + (live ? cr * Pp + ((colBase + k4) ^ lds_swz(cr)) : 0u));
                    off[u] = live ? l * 4u : BUF_OOB;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) buf_store<BUF_NT>(yr, off[u], qv[u]);
            }
        }
    }
}

template <int LD, typename G>
__global__ __launch_bounds__(512) void k_gather_lines(const float* __restrict__ x, float* __restrict__ y,
                                                      const int16_t* __restrict__ idx, LineArgs a)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for_each_block_of_workgroup(a, G::tpb(a), [&](uint32_t ib, uint32_t rem) {
        gather_lines_tile<LD, G>(x, y, idx, a, lds, ib, rem);
    });
}

// Tile choice of k_gather_lines.  Returns false where the kernel does not apply (the caller then uses
// k_gather_planar): y not 16-byte aligned, a last split shorter than the window extension, LDS.
static bool make_line_args(const Geom& g, int numActive, const float* y, LineArgs& a, int& threads, int& ld,
                           size_t& ldsBytes, unsigned& grid, int maxLd)
{
    if (g.C % 4 != 0 || (reinterpret_cast<uintptr_t>(y) & 15) != 0) return false;
    a.g = g;
    const int64_t RS64 = (int64_t)g.R * g.S;
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (RS64 < 4 || a.imgFloats >= (1ll << 30) || (int64_t)g.C * RS64 >= (1ll << 30)) return false;
    const int RS = (int)RS64;
    a.RS = RS;
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    int lpp = 1;
    while (lpp * 2 * 4 <= 32 && lpp * 4 < g.C) lpp *= 2;
    a.Ct = lpp * 4;
    a.lppLog = ilog2_floor((uint32_t)lpp);
    a.cchunks = (g.C + a.Ct - 1) / a.Ct;
    // The smallest workgroup whose LD vectors per thread cover a whole plane; otherwise 512 threads and as
    // few splits as the window (own pixels + LINE_EXT) allows within maxLd vectors per thread.
    threads = 0;
    a.psplit = 1;
    for (int nthr = 64; nthr <= 512; nthr *= 2) {
        threads = nthr;
        if (4 * nthr / lpp >= RS) break;
    }
    if (4 * threads / lpp < RS) {
        const int cap = maxLd * threads / lpp - LINE_EXT;
        if (cap < 2 * LINE_FLOATS) return false;
        a.psplit = (RS + cap - 1) / cap;
    }
    a.P = (RS + a.psplit - 1) / a.psplit;
    a.psplit = (RS + a.P - 1) / a.P;
    // A tile that takes whole planes writes one contiguous piece of y in k_gather_planar already.
    if (a.psplit == 1) return false;
    if (RS - (a.psplit - 1) * a.P < LINE_FLOATS) return false;  // the last split must hold the extension
    const int win = a.P + LINE_EXT;
    ld = (win * lpp + threads - 1) / threads;
    if (ld < 4) ld = 4;
    if (ld > 8) return false;
    a.Pp = (win + 3 + 31) / 32 * 32;
    ldsBytes = (size_t)a.Ct * a.Pp * sizeof(float);
    if (ldsBytes > 64 * 1024) return false;
    // slots per row: the written range of a row is at most P + LINE_EXT floats; when every chunk starts on a
    // line it is a whole number of lines
    const bool aligned = (reinterpret_cast<uintptr_t>(y) & 127) == 0 && ((int64_t)a.Ct * RS) % LINE_FLOATS == 0 &&
                         ((int64_t)g.C * RS) % LINE_FLOATS == 0;
    a.spr = aligned ? (uint32_t)((a.P + LINE_EXT) / LINE_FLOATS * (LINE_FLOATS / 4)) : (uint32_t)((a.P + LINE_EXT + 3) / 4);
    a.tpb = (uint32_t)(a.psplit * a.cchunks);
    const uint64_t total = (uint64_t)numActive * a.tpb;
    if (total >= (1ull << 31)) return false;
    a.total = (uint32_t)total;
    a.dTpb = make_fastdiv(a.tpb);
    a.dPs = make_fastdiv((uint32_t)a.psplit);
    a.dS = make_fastdiv((uint32_t)g.S);
    grid = a.total;
    a.grid2d = numActive <= GRID_Y_MAX;
    a.blocks = (uint32_t)numActive;
    return true;
}

// 5 vectors per thread (three splits of a 27x27 plane) for launches of many workgroups, up to 7 (two splits, which
// take 6: fewer window pixels read twice, more bytes in flight per workgroup) for launches of few, as for the scatter:
// 8.62 -> 7.76 us at 58 blocks, 21.7 -> 20.8 us at 156, but 31.1 -> 31.6 us at 231 and 40.3 -> 40.6 us at 312.
constexpr int GATHER_FEW_WGS_PER_CU = 9;

static bool choose_line_args(const Geom& g, int numActive, const float* y, LineArgs& a, int& threads, int& ld,
                             size_t& ldsBytes, unsigned& grid)
{
    if (!make_line_args(g, numActive, y, a, threads, ld, ldsBytes, grid, 5)) return false;
    if (a.total < (uint32_t)(GATHER_FEW_WGS_PER_CU * device_cus())) {
        LineArgs b;
        int bt, bld;
        size_t bl;
        unsigned bg;
        if (make_line_args(g, numActive, y, b, bt, bld, bl, bg, 7) && b.psplit < a.psplit) {
            a = b;
            threads = bt;
            ld = bld;
            ldsBytes = bl;
            grid = bg;
        }
    }
    return true;
}

// Fixed-shape instances: launched when the run-time tile choice equals the instance's.
template <typename G>
static bool lines_match(const LineArgs& a, int threads, int ld)
{
    return !a.g.forceGeneric && a.g.R * a.g.S == (int)G::kRS && a.g.S == (int)G::S(a) && a.g.C == (int)G::C(a) &&
           a.psplit == (int)G::psplit(a) && threads == (int)G::nthr(a) && a.P == (int)G::kP && a.Pp == (int)G::kPp &&
           a.Ct == (int)G::Ct(a) && a.lppLog == (int)G::kLppLog && ld == G::kLD && a.tpb == G::tpb(a);
}

template <typename G>
static bool launch_fixed_lines_one(const float* x, float* y, const int16_t* idx, const LineArgs& a, int threads, int ld,
                                   size_t lds, int numActive, hipStream_t stream)
{
    if (!lines_match<G>(a, threads, ld)) return false;
    hipLaunchKernelGGL((k_gather_lines<G::kLD, G>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads), lds,
                       stream, x, y, idx, a);
    return true;
}

static bool launch_fixed_lines(const float* x, float* y, const int16_t* idx, const LineArgs& a, int threads, int ld,
                               size_t lds, int numActive, hipStream_t stream)
{
    // 27x27 blocks of 128 channels (800x800x128 tensor): three and two splits per plane; 18x18 blocks of 64 channels
    return launch_fixed_lines_one<LinesFixed<27, 27, 128, 3, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream) ||
           launch_fixed_lines_one<LinesFixed<27, 27, 128, 2, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream) ||
           launch_fixed_lines_one<LinesFixed<18, 18, 64, 2, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream) ||
           launch_fixed_lines_one<LinesFixed<18, 18, 256, 2, 512>>(x, y, idx, a, threads, ld, lds, numActive, stream);
}

template <int VEC>
static void gather_dispatch(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive,
                            bool transpose, hipStream_t stream, hipError_t& err)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        if (nhwc_fits_buffers(g))
            hipLaunchKernelGGL(k_gather_nhwc<VEC>, dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
        else
            hipLaunchKernelGGL(k_gather_nhwc_wide<VEC>, dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, idx, a);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        if (VEC == 4) {
            LineArgs la;
            int ld;
            if (choose_line_args(g, numActive, y, la, threads, ld, lds, grid)) {
                if (launch_fixed_lines(x, y, idx, la, threads, ld, lds, numActive, stream)) return;
                const dim3 lg = tile_grid(la.grid2d, la.tpb, numActive, la.total, la.g);
                switch (ld) {
                case 4: hipLaunchKernelGGL((k_gather_lines<4, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 5: hipLaunchKernelGGL((k_gather_lines<5, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 6: hipLaunchKernelGGL((k_gather_lines<6, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                case 7: hipLaunchKernelGGL((k_gather_lines<7, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                default: hipLaunchKernelGGL((k_gather_lines<8, LinesRt>), lg, dim3(threads), lds, stream, x, y, idx, la); break;
                }
                return;
            }
        }
        // 32 KB tiles: 46.5 us against 52.7 us with 16 KB tiles on the 800x800x128 workload.
        // Planes of fewer than 4 pixels and images or blocks beyond 32-bit byte offsets take the generic kernel.
        if ((int64_t)g.R * g.S < 4 || !make_tile_args(g, numActive, VEC, a, threads, lds, grid, 32 * 1024)) {
            const int64_t total = (int64_t)numActive * g.C * g.R * g.S;
            const int64_t wgs = (total + 255) / 256;
            hipLaunchKernelGGL((k_planar_small<SCATTER_ASSIGN, true>), dim3((unsigned)(wgs > 65536 ? 65536 : wgs)),
                               dim3(256), 0, stream, x, y, (const float*)y, idx, g, total, (const int32_t*)nullptr);
            return;
        }
        hipLaunchKernelGGL(k_gather_planar<VEC>, tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads), lds,
                           stream, x, y, idx, a);
    }
}

// Test hook (sbnet_test_tile_choice): the tile the planar kernels would use for a geometry, without launching.
// kind 0: k_gather_lines, 1: k_gather_planar, 2: k_scatter_planar.  out = {threads, ldsBytes, P, Pp, psplit, Ct,
// cchunks, vectors or slots per thread needed, vectors or slots per thread available, last split's pixels, fixed
// instance available}.  Returns 0 when that kernel does not apply to the geometry.
int tile_choice(int kind, const Geom& g, int numActive, int vec, int yAlignedTo, int32_t* out)
{
    int threads = 0;
    size_t lds = 0;
    unsigned grid = 0;
    const int RS = g.R * g.S;
    if (kind == 0) {
        LineArgs a;
        int ld = 0;
        // a y pointer with the requested alignment (never dereferenced)
        const float* y = reinterpret_cast<const float*>((uintptr_t)0x10000 + (uintptr_t)yAlignedTo);
        if (vec != 4 || !choose_line_args(g, numActive, y, a, threads, ld, lds, grid)) return 0;
        const int lpp = 1 << a.lppLog;
        out[0] = threads; out[1] = (int32_t)lds; out[2] = a.P; out[3] = a.Pp; out[4] = a.psplit; out[5] = a.Ct;
        out[6] = a.cchunks; out[7] = ((a.P + LINE_EXT) * lpp + threads - 1) / threads; out[8] = ld;
        out[9] = RS - (a.psplit - 1) * a.P;
        out[10] = lines_match<LinesFixed<27, 27, 128, 3, 512>>(a, threads, ld) ||
                  lines_match<LinesFixed<27, 27, 128, 2, 512>>(a, threads, ld) ||
                  lines_match<LinesFixed<18, 18, 64, 2, 512>>(a, threads, ld) ||
                  lines_match<LinesFixed<18, 18, 256, 2, 512>>(a, threads, ld);
        return 1;
    }
    if (kind == 2) return scatter_tile_choice(g, numActive, vec, out);
    TileArgs a;
    if (RS < 4 || !make_tile_args(g, numActive, vec, a, threads, lds, grid, 32 * 1024)) return 0;
    const int lpp = 1 << a.lppLog;
    out[0] = threads; out[1] = (int32_t)lds; out[2] = a.P; out[3] = a.Pp; out[4] = a.psplit; out[5] = a.Ct;
    out[6] = a.cchunks;
    out[7] = (a.P * lpp + threads - 1) / threads;   // the gather's planar side loops, only its NHWC side is bounded
    out[8] = TILE_LD;
    out[9] = RS - (a.psplit - 1) * a.P;
    out[10] = 0;
    return 1;
}

hipError_t launch_gather(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                         bool transpose, hipStream_t stream)
{
    if (numActive == 0) return hipSuccess;
    hipError_t err = hipSuccess;
    // the planar side of the transpose handles its own alignment; only the NHWC pointer matters there
    const int vec = pick_vec(g, x, transpose ? nullptr : y);
    if (vec == 4) gather_dispatch<4>(x, y, idx, g, numActive, transpose, stream, err);
    else if (vec == 2) gather_dispatch<2>(x, y, idx, g, numActive, transpose, stream, err);
    else gather_dispatch<1>(x, y, idx, g, numActive, transpose, stream, err);
    if (err != hipSuccess) return err;
    return hipGetLastError();
}

}  // namespace sbnet

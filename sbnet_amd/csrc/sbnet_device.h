// gfx950 (MI355X, CDNA4, wave64) kernels for reduce_mask, sparse_gather and sparse_scatter.
//
// None of the three ops is a contraction, so there is no MFMA here: they are HBM-bound block
// copies plus one tiny pooling reduction.  What the kernels are built around:
//   * 16-byte (dwordx4) accesses along C on the NHWC side, with 8- and 4-byte variants chosen
//     on the host when C or a base pointer does not allow 16;
//   * for the fused NHWC <-> [blocks, C, R, S] transpose, a tile of Ct channels x P block pixels
//     staged through LDS so that both the NHWC side (runs of Ct floats per pixel) and the planar
//     side (runs of P floats per channel) move in long contiguous pieces; the planar runs start
//     at arbitrary 4-byte alignment (27x27 planes are 729 floats): the scatter reads them as
//     misaligned dwordx4 slots, the gather writes whole, aligned 128-byte lines;
//   * raw buffer addressing with out-of-range offsets instead of branches around loads and stores;
//   * several independent loads in flight per lane before the first use;
//   * no integer division in inner loops (multiply-high reciprocals prepared on the host);
//   * wave64 ballot / popcount for the ordered stream compaction of reduce_mask.
//
// Semantics follow the reference's CPU functors (sbnet_tensorflow/sbnet_ops/reduce_mask.cc:68-96,
// sparse_gather.cc:67-88 and 103-130); each kernel cites the lines it reproduces.
//
// This header holds what the translation units share: the device-side helpers (reciprocal division, vector
// types, block origins, buffer addressing, the LDS tile layout, the walk over a tile's NHWC side), the
// kernels' argument structs, the one kernel both gather and scatter instantiate (k_planar_small), and
// the host-side launch arithmetic common to them.  sbnet_reduce_mask.hip, sbnet_gather.hip and
// sbnet_scatter.hip hold the kernels and launchers of the three ops.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "sbnet_launch.h"

namespace sbnet {

// ---------------------------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------------------------
// Exact unsigned division by a run-time constant: q = (t + ((n - t) >> sh1)) >> sh2 with
// t = mulhi(mul, n).  Valid for every 32-bit n and every d >= 1.
struct FastDiv {
    uint32_t mul, sh1, sh2, d;
};

static FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    uint64_t m = ((1ull << 32) * ((1ull << l) - d)) / d + 1;
    f.mul = (uint32_t)m;
    f.sh1 = l ? 1u : 0u;
    f.sh2 = l ? l - 1u : 0u;
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv& f)
{
    uint32_t t = __umulhi(f.mul, n);
    return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

// Native clang vectors (not HIP's float4 struct): they take the nontemporal builtins and arithmetic.
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

template <int VEC> struct Vec;
template <> struct Vec<4> { typedef f4 type; };
template <> struct Vec<2> { typedef f2 type; };
template <> struct Vec<1> { typedef float type; };

template <int VEC> __device__ __forceinline__ typename Vec<VEC>::type vzero();
template <> __device__ __forceinline__ f4 vzero<4>() { return (f4)(0.f); }
template <> __device__ __forceinline__ f2 vzero<2>() { return (f2)(0.f); }
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }

__device__ __forceinline__ float vget(const f4& v, int k) { return k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w; }
__device__ __forceinline__ float vget(const f2& v, int k) { return k == 0 ? v.x : v.y; }
__device__ __forceinline__ float vget(const float& v, int) { return v; }
__device__ __forceinline__ void vset(f4& v, int k, float f) { if (k == 0) v.x = f; else if (k == 1) v.y = f; else if (k == 2) v.z = f; else v.w = f; }
__device__ __forceinline__ void vset(f2& v, int k, float f) { if (k == 0) v.x = f; else v.y = f; }
__device__ __forceinline__ void vset(float& v, int, float f) { v = f; }

template <typename T> __device__ __forceinline__ T vadd(const T& a, const T& b) { return a + b; }

// 0 + a + b + c + own, with a, b and c taken in ascending order of their list positions pa, pb, pc: what a sequential
// pass over the list leaves in a tensor of zeros.  A term that is absent comes as +0 at any position (a sum that
// started from +0 is never -0, so adding +0 changes nothing).
template <typename T>
__device__ __forceinline__ T sum_in_list_order(int32_t pa, T a, int32_t pb, T b, int32_t pc, T c, const T& own, const T& zero)
{
    auto cx = [](int32_t& p, T& x, int32_t& q, T& y) {
        const bool sw = p > q;
        const int32_t p0 = sw ? q : p, q0 = sw ? p : q;
        const T x0 = sw ? y : x, y0 = sw ? x : y;
        p = p0; q = q0; x = x0; y = y0;
    };
    cx(pa, a, pb, b);
    cx(pb, b, pc, c);
    cx(pa, a, pb, b);
    return vadd(vadd(vadd(vadd(zero, a), b), c), own);
}

// The same where absent terms come with position -1 and value +0.  With at most one term present no order is
// needed, and a + b + c holds two +0 terms, so it is never -0 and equals 0 + that term: the common case (pixels
// under two blocks; only a block's corners lie under more) takes three additions and skips the sort, a wave at a time.
template <typename T>
__device__ __forceinline__ T sum_of_pixel(int32_t pa, const T& a, int32_t pb, const T& b, int32_t pc, const T& c, const T& own,
                                          const T& zero)
{
    const int present = (int)(pa >= 0) + (int)(pb >= 0) + (int)(pc >= 0);
    if (present >= 2) return sum_in_list_order(pa, a, pb, b, pc, c, own, zero);
    return vadd(vadd(vadd(a, b), c), own);
}

// Streaming accesses: every byte of x, of the block stack and of the base tensor is touched once per
// op, so loads and stores carry the nontemporal hint (measured: a plain dwordx4 copy gains ~10 %).
template <typename T> __device__ __forceinline__ T ld_stream(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void st_stream(T* p, const T& v) { __builtin_nontemporal_store(v, p); }

// Hardware fp32 atomic add (global_atomic_add_f32, no return value).
__device__ __forceinline__ void atomic_add_f32(float* p, float v) { unsafeAtomicAdd(p, v); }

// Writes one vector of a block into the base tensor: "=", "+=" or atomic "+="
// (sparse_gather.cc:121-128; the atomic flavour is the GPU-only attribute of the op).
template <int VEC, int MODE>
__device__ __forceinline__ void commit(typename Vec<VEC>::type* dst, const typename Vec<VEC>::type& v)
{
    if (MODE == SCATTER_ASSIGN) {
        st_stream(dst, v);
    } else if (MODE == SCATTER_ADD) {
        st_stream(dst, vadd(ld_stream(dst), v));
    } else {
        float* d = reinterpret_cast<float*>(dst);
#pragma unroll
        for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v, k));
    }
}

// Reads the (n, bh, bw) triple of block ib (wave-uniform) and derives the block origin.
struct BlockOrigin {
    int n, h0, w0;
    int bh, bw;  // the block's grid position
    bool valid;  // n inside [0, N): guards against garbage rows in the index list
};

__device__ __forceinline__ BlockOrigin load_origin(const int16_t* __restrict__ idx, uint32_t ib, const Geom& g)
{
    BlockOrigin o;
    const int16_t* t = idx + (size_t)ib * 3;
    o.n = t[0];
    o.bh = t[1];
    o.bw = t[2];
    o.h0 = g.oh + o.bh * g.U;
    o.w0 = g.ow + o.bw * g.V;
    o.valid = (unsigned)o.n < (unsigned)g.N;
    return o;
}

// The same in two steps, for software pipelines: the loads are issued early and the arithmetic (which
// is what makes a wave wait for them) happens where the origin is first needed.
struct RawTriple {
    uint32_t lo, hi;  // the two aligned dwords that hold the 6-byte triple
    uint32_t shift;   // 0 or 16: where the triple starts inside them
};

// ib is the same for the whole workgroup.  Reading the two aligned dwords around the triple from a uniform
// address lets the compiler use the scalar unit, whose loads are counted apart from vector loads and stores:
// waiting for the triple then does not wait for the stores in flight.  (A triple that ends the list on a
// 4-byte boundary + 2 makes the second dword reach 2 bytes past the list, inside the same aligned dword.)
__device__ __forceinline__ RawTriple load_triple(const int16_t* __restrict__ idx, uint32_t ib)
{
    const uint32_t byteOff = 6u * (uint32_t)__builtin_amdgcn_readfirstlane(ib);
    const uintptr_t base = reinterpret_cast<uintptr_t>(idx) + byteOff;
    // constant address space: a uniform address alone does not make the compiler pick a scalar load, and a
    // triple that arrives in vector registers makes every descriptor built from it "divergent" (each buffer
    // access then sits in a readfirstlane loop).  The list is never written by the kernels that read it.
    typedef const uint32_t __attribute__((address_space(4))) * const_u32_ptr;
    const_u32_ptr w = (const_u32_ptr)(base & ~(uintptr_t)3);
    RawTriple r;
    r.lo = w[0];
    r.hi = w[1];
    r.shift = (uint32_t)(base & 2) * 8u;
    return r;
}

__device__ __forceinline__ BlockOrigin origin_of(const RawTriple& r, const Geom& g)
{
    const uint64_t bits = (((uint64_t)r.hi << 32) | r.lo) >> r.shift;
    BlockOrigin o;
    o.n = (int)(int16_t)(bits & 0xffffu);
    o.bh = (int)(int16_t)((bits >> 16) & 0xffffu);
    o.bw = (int)(int16_t)((bits >> 32) & 0xffffu);
    o.h0 = g.oh + o.bh * g.U;
    o.w0 = g.ow + o.bw * g.V;
    o.valid = (unsigned)o.n < (unsigned)g.N;
    return o;
}

// True for list rows at or beyond the device-resident count (see Geom::countDev); ib is wave-uniform.
__device__ __forceinline__ bool beyond_count(const Geom& g, uint32_t ib)
{
    if (!g.countDev) return false;
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    return ib >= (uint32_t)*(const_i32_ptr)(reinterpret_cast<uintptr_t>(g.countDev));
}

// Overlapping scatter-add in passes ("colours").  Blocks whose grid positions agree modulo
// (Kh, Kw) = (ceil(R/U), ceil(S/V)) cannot overlap, so a launch that handles one residue class can add
// with plain load-add-store; Kh*Kw launches in a row cover the list.  The result is reproducible (the
// order of the adds is the order of the passes) and runs at streaming speed, where hardware atomics reach
// about a tenth of it.  A block listed twice breaks the premise: the map kernel of the pull scatter
// detects that (`dup`), and then pass 0 handles every block with atomics and the other passes do nothing.
constexpr int SCATTER_COLOR = 3;  // kernel-side mode; callers ask for SCATTER_ATOMIC

// Plain writes ("=") of overlapping blocks in the sequential CPU functor's order: that functor visits the
// list front to back (sparse_gather.cc:105), so on a pixel that several blocks cover the one listed last
// wins.  A per-pixel owner map (the highest list position that covers the pixel, built by k_owner_fill and
// k_owner_mark before the launch) lets every block write only the pixels it owns: no pixel is written twice,
// and a block listed twice is handled like any other overlap.
constexpr int SCATTER_OWNED = 4;  // kernel-side mode; callers ask for SCATTER_ASSIGN and give scratch

// The same order without a per-pixel map, for the common case of at most 2x2 blocks over a pixel (bsize <= 2 *
// bstride) and a list short enough to compare every pair of blocks: a block's eight grid neighbours (and any other
// row of the list that names the block itself) are the only blocks that can share pixels with it, and which of
// its pixels a neighbour covers depends only on whether the pixel lies in the block's first R - U rows (shared
// with the row of blocks above), its rows from U on (shared with the row below), or in between, and likewise for
// columns.  k_rank_table leaves nine bits per block: bit 3*rowClass + colClass is set when some block listed
// later covers that class of pixels; the scatter kernels skip those pixels.
constexpr int SCATTER_RANKED = 5;  // kernel-side mode; callers ask for SCATTER_ASSIGN and give scratch

// The same nine bits without a table and without an extra launch: the workgroup that moves a tile of block ib
// compares ib with the rows listed after it while the tile's loads are in flight (a few hundred 6-byte rows from
// L2 against a 16-24 KB tile), so the in-place op needs neither scratch nor a second kernel for the CPU functor's
// order.  Planar tile kernel only: its workgroups are large enough to share the comparison.
constexpr int SCATTER_RANKED_INLINE = 6;  // kernel-side mode; callers ask for SCATTER_ASSIGN
constexpr int RANK_ROWS_PER_THREAD = 2;   // rows of the list fetched per thread ahead of the tile's LDS phase

// "Zeros plus the sum of the blocks" (the gradient of sparse_gather) in one pass over the stack, for at most 2x2
// blocks over a pixel: k_fill_uncovered has written zeros where no block lies; every covered pixel is written once,
// by the block listed last among those that cover it (the owner, as in SCATTER_RANKED), which fetches the other
// blocks' values of that pixel from the stack and adds them up in list order, its own last: 0 + a + b + own, the
// sequential CPU functor's sum (sparse_gather.cc:105-129), bit for bit, without atomics.  The neighbours' list
// positions come from the inverse block map.  A list that names a block twice has no such map: every block then
// adds all of its pixels with hardware atomics onto zeros (k_fill_uncovered clears everything in that case).
constexpr int SCATTER_SUM = 7;  // kernel-side mode of sbnet_sparse_gather_grad

struct ColorArgs {
    int kh, kw, pass;
    const int32_t* dup;
    const int32_t* owner;  // SCATTER_OWNED: [N, H, W] list positions, -1 where no block covers the pixel
    const int32_t* rank;   // SCATTER_RANKED: nine bits per block, see k_rank_table
    // SCATTER_COLOR with `first`: the passes add onto a tensor of which only the pixels that no block covers hold
    // zeros yet (k_fill_uncovered), so a pass reads a pixel only where a block of an earlier pass has written it
    // and stores 0 + v elsewhere.  `map` is the inverse block map [N, nBH, nBW] (list position or -1); SCATTER_SUM
    // reads it too.
    int first;
    const int32_t* map;
    int bhMin, bwMin, nBH, nBW;
    // SCATTER_COLOR: the list sorted by pass (k_color_sort): perm[p * permStride + 0 .. counts[p]) are the list
    // positions of pass p's blocks.  A pass then runs over its own blocks only, and the workgroups beyond them,
    // which leave after one load, come last in the launch instead of in between (where each of them held up a
    // working one).  NULL: every pass walks the whole list.
    const int32_t* perm;
    const int32_t* counts;
    int permStride;
};

// Position `pos` of a colour pass's launch -> position in the block list, false when the pass has no such block.
__device__ __forceinline__ bool color_block(const ColorArgs& col, uint32_t pos, uint32_t& ib)
{
    ib = pos;
    if (!col.perm) return true;
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    // (two independent loads: the pass's count and the slot, which holds garbage beyond the count)
    const int32_t cnt = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.counts + col.pass));
    const int32_t at = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.perm + (int64_t)col.pass * col.permStride + pos));
    if ((int32_t)pos >= cnt) return false;
    ib = (uint32_t)at;
    return true;
}

// Pixel (r, s) of a block against the block's nine bits: true when a block listed later covers it.
__device__ __forceinline__ bool ranked_out(uint32_t bits, uint32_t r, uint32_t s, const Geom& g)
{
    const uint32_t rc = (int)r < g.R - g.U ? 0u : ((int)r >= g.U ? 2u : 1u);
    const uint32_t cc = (int)s < g.S - g.V ? 0u : ((int)s >= g.V ? 2u : 1u);
    return (bits >> (rc * 3u + cc)) & 1u;
}

// Classes of block (n, bh, bw)'s pixels that the block of a later row (n2, bh2, bw2) covers: row classes (0: first
// R-U rows, 1: middle, 2: rows from U on) crossed with the same for columns, bit 3*rowClass + colClass.
__device__ __forceinline__ uint32_t rank_pair_bits(int n, int bh, int bw, int n2, int bh2, int bw2)
{
    const int dh = bh2 - bh, dw = bw2 - bw;
    if (n2 != n || dh < -1 || dh > 1 || dw < -1 || dw > 1) return 0u;
    const uint32_t rows = dh < 0 ? 1u : (dh > 0 ? 4u : 7u), cols = dw < 0 ? 1u : (dw > 0 ? 4u : 7u);
    return ((rows & 1u) ? cols : 0u) | ((rows & 2u) ? cols << 3 : 0u) | ((rows & 4u) ? cols << 6 : 0u);
}

// Length of the block list as the kernels see it: the host's count, capped by the device-resident one.
__device__ __forceinline__ uint32_t list_count(const Geom& g, uint32_t capacity)
{
    if (!g.countDev) return capacity;
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    const int32_t c = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(g.countDev));
    return min(capacity, (uint32_t)max(c, 0));
}

__device__ __forceinline__ uint32_t rank_bits(const ColorArgs& col, uint32_t ib)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;  // ib is wave-uniform: scalar load
    return (uint32_t)*(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.rank + ib));
}

// SCATTER_COLOR with ColorArgs::first (at most 2x2 blocks over a pixel): nine bits like those of SCATTER_RANKED,
// bit 3*rowClass + colClass set when an active block of an earlier pass covers that class of the block's pixels.
// Eight look-ups in the inverse block map, all through the scalar unit (the block is the same for the workgroup).
__device__ __forceinline__ uint32_t earlier_pass_bits(const ColorArgs& col, const BlockOrigin& o)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    // the eight neighbours' entries first (a neighbour beyond the map reads the map's first entry and is masked:
    // the block's own cell may lie beyond the map as well, when the block cannot touch the image),
    // then the arithmetic: eight independent scalar loads instead of a chain
    int32_t other[9];
    bool in[9];
#pragma unroll
    for (int q = 0; q < 9; ++q) {
        const int dh = q / 3 - 1, dw = q % 3 - 1;
        const int ih = o.bh + dh - col.bhMin, iw = o.bw + dw - col.bwMin;
        in[q] = q != 4 && (unsigned)ih < (unsigned)col.nBH && (unsigned)iw < (unsigned)col.nBW;
        const int64_t slot = in[q] ? ((int64_t)o.n * col.nBH + ih) * col.nBW + iw : 0;
        other[q] = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.map + slot));
    }
    uint32_t bits = 0u;
#pragma unroll
    for (int q = 0; q < 9; ++q) {
        const int dh = q / 3 - 1, dw = q % 3 - 1;
        // (kh and kw are 1 or 2 here: the pass of a block is the parity of its position)
        const int pass = (((o.bh + dh) & (col.kh - 1)) * col.kw) + ((o.bw + dw) & (col.kw - 1));
        if (in[q] && other[q] >= 0 && pass < col.pass) {
            const uint32_t rows = dh < 0 ? 1u : (dh > 0 ? 4u : 7u), cols = dw < 0 ? 1u : (dw > 0 ? 4u : 7u);
            bits |= ((rows & 1u) ? cols : 0u) | ((rows & 2u) ? cols << 3 : 0u) | ((rows & 4u) ? cols << 6 : 0u);
        }
    }
    return bits;
}

// SCATTER_SUM: the active neighbours of block ib at (o.bh, o.bw), q = 3 * (dh + 1) + (dw + 1).  `later`: nine bits
// as in SCATTER_RANKED, the classes of the block's pixels that a neighbour listed after it covers (that neighbour,
// or one after it, owns them).  `pos[q]`: list position of a neighbour listed before it, else -1.  All of it
// wave-uniform (scalar loads and ALU).
constexpr int SUM_MAX_BLOCKS = 1 << 30;

struct NeighbourPos {
    uint32_t later;
    int32_t pos[9];
};

__device__ __forceinline__ NeighbourPos neighbour_positions(const ColorArgs& col, const BlockOrigin& o, uint32_t ib)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    int32_t other[9];
    bool in[9];
#pragma unroll
    for (int q = 0; q < 9; ++q) {  // (independent loads; a neighbour beyond the map reads the first entry and is masked)
        const int dh = q / 3 - 1, dw = q % 3 - 1;
        const int ih = o.bh + dh - col.bhMin, iw = o.bw + dw - col.bwMin;
        in[q] = q != 4 && (unsigned)ih < (unsigned)col.nBH && (unsigned)iw < (unsigned)col.nBW;
        const int64_t slot = in[q] ? ((int64_t)o.n * col.nBH + ih) * col.nBW + iw : 0;
        other[q] = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.map + slot));
    }
    NeighbourPos nb;
    nb.later = 0u;
#pragma unroll
    for (int q = 0; q < 9; ++q) {
        const int dh = q / 3 - 1, dw = q % 3 - 1;
        const bool active = in[q] && other[q] >= 0;
        if (active && (uint32_t)other[q] > ib) {
            const uint32_t rows = dh < 0 ? 1u : (dh > 0 ? 4u : 7u), cols = dw < 0 ? 1u : (dw > 0 ? 4u : 7u);
            nb.later |= ((rows & 1u) ? cols : 0u) | ((rows & 2u) ? cols << 3 : 0u) | ((rows & 4u) ? cols << 6 : 0u);
        }
        nb.pos[q] = active && (uint32_t)other[q] < ib ? other[q] : -1;
    }
    return nb;
}

// The up to three other blocks over pixel (r, s) of the block: the vertical neighbour (dh, 0), the horizontal one
// (0, dw) and the diagonal one (dh, dw), as list positions or -1.  In those blocks the pixel lies dh * U rows up and
// dw * V columns left.  Meant for pixels that the block owns: every other block over them is listed before it.
struct PixelNeighbours {
    int32_t pv, ph, pd;
    int dh, dw;
};

__device__ __forceinline__ PixelNeighbours pixel_neighbours(const NeighbourPos& nb, int r, int s, const Geom& g)
{
    PixelNeighbours p;
    p.dh = r < g.R - g.U ? -1 : (r >= g.U ? 1 : 0);
    p.dw = s < g.S - g.V ? -1 : (s >= g.V ? 1 : 0);
    p.pv = p.dh < 0 ? nb.pos[1] : (p.dh > 0 ? nb.pos[7] : -1);
    p.ph = p.dw < 0 ? nb.pos[3] : (p.dw > 0 ? nb.pos[5] : -1);
    const int32_t upper = p.dw < 0 ? nb.pos[0] : nb.pos[2], lower = p.dw < 0 ? nb.pos[6] : nb.pos[8];
    p.pd = p.dh != 0 && p.dw != 0 ? (p.dh < 0 ? upper : lower) : -1;
    return p;
}

// The list names some block twice (k_pull_map's flag, written by an earlier kernel).
__device__ __forceinline__ bool list_has_repeats(const ColorArgs& col)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    return *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.dup)) != 0;
}

// True when this launch has nothing to do for the block; `atomics` tells how to add otherwise.
__device__ __forceinline__ bool color_skip(const ColorArgs& col, const BlockOrigin& o, bool& atomics)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    atomics = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(col.dup)) != 0;  // written by an earlier kernel
    if (atomics) return col.pass != 0;
    int mh = o.bh % col.kh, mw = o.bw % col.kw;
    if (mh < 0) mh += col.kh;
    if (mw < 0) mw += col.kw;
    return mh * col.kw + mw != col.pass;
}

// ---------------------------------------------------------------------------------------------
// NHWC block stack <-> NHWC tensor: row-segment copies
// ---------------------------------------------------------------------------------------------
//
// A block in the stack is R rows of rowV = S*C/VEC vectors, contiguous.  The matching piece of
// the tensor is R row segments of the same length (the in-range part of it).  One wave handles
// one "unit": CHUNK = 64*UNR consecutive vectors of one block; four units per workgroup.

constexpr int NHWC_UNR = 4;  // 4 KB per wave, 16 KB per workgroup (see COPY_UNR)
constexpr int NHWC_CHUNK = 64 * NHWC_UNR;

struct NhwcArgs {
    Geom g;
    uint32_t rowV;    // vectors per block row, S*C/VEC
    uint32_t blockV;  // vectors per block, R*rowV
    uint32_t cpb;     // chunks per block
    uint32_t units;   // numActive * cpb
    FastDiv dCpb, dRow, dCV;  // dCV: by the vectors per pixel, C/VEC
};

// ---------------------------------------------------------------------------------------------
// planar block stack [blocks, C, R, S] <-> NHWC tensor: LDS-staged transpose
// ---------------------------------------------------------------------------------------------
//
// A tile is Ct channels x Pn pixels of one block, pixels numbered p = r*S + s inside the block.
// On the NHWC side a lane moves VEC channels of one pixel (the lanes of a wave cover the Ct/VEC
// vectors of a pixel, then the next pixel).  On the planar side row c of the tile is a contiguous
// run of Pn floats that starts at whatever 4-byte alignment (c*R*S + p0) lands on (27x27 planes hold
// 729 floats).  Runs move as dwordx4 "slots" of 4 consecutive floats from the start of the run, so
// most of these accesses are not 16-byte aligned; gfx950 executes misaligned global dwordx4 accesses
// at the speed of aligned ones (measured with a plain copy), which makes an aligned-body / scalar-
// head-and-tail split unnecessary.  Only the last slot of a run can be partial.
//
// One workgroup moves one tile: all of its global loads are issued back to back into registers (no
// control flow around them: lanes with nothing to fetch use an out-of-range buffer offset, which reads
// as zero), then go through LDS, then leave as stores.  A persistent variant that
// software-pipelined several tiles per workgroup (loads of tile i+1 in flight during the stores of tile
// i) was measured slower the more tiles a workgroup owned (47 -> 52 -> 65 us for 1, 4, 12 tiles per
// workgroup on the 800x800x128 workload): the hardware dispatcher balances one-tile workgroups better
// than a static split, and with 4-5 workgroups resident per CU their phases overlap anyway.  Tiles are
// numbered (block, channel chunk, pixel split) with the pixel split fastest, so the splits of one
// channel chunk, which continue each other's planar runs, are dispatched together.
//
// LDS layout: tile row c at c*Pp floats, Pp a multiple of 32, pixel e at column e.  Columns are
// XOR-swizzled in units of 4 floats by ((c >> 2) & 7): the planar side still sees aligned groups of
// 4 floats (ds_read_b128 / ds_write_b128), and the transposing NHWC side, where 32 lanes touch 4
// consecutive pixels of 8 different channel groups at once, hits 32 distinct banks (LDS has 32
// four-byte banks; a padded, unswizzled layout lost 58 % of its LDS cycles to bank conflicts).

constexpr int TILE_LD = 4;  // vectors (NHWC side) or slots (planar side) held in registers per thread

struct TileArgs {
    Geom g;
    int Ct;             // channels per tile; Ct/VEC is a power of two
    int lppLog;         // log2(Ct/VEC): lanes per pixel on the NHWC side
    int P;              // pixels per tile (the last split of a block may hold fewer)
    int Pp;             // LDS row pitch in floats, multiple of 32, >= P
    int psplit;         // pixel splits per block
    int cchunks;        // channel chunks per block
    uint32_t tpb;       // tiles per block = psplit * cchunks
    uint32_t total;     // numActive * tpb
    int grid2d;         // the launch is (tpb, block rows): see for_each_block_of_workgroup
    uint32_t blocks;    // capacity of the block list (numActive)
    uint32_t vpr;       // slots per planar row: (P + 3) / 4
    int64_t imgFloats;  // H * W * C
    uint32_t imgBytes;  // H * W * C * 4, below 2^32 (the host falls back to k_planar_small otherwise)
    FastDiv dTpb, dPs, dS, dVpr;
};

struct TileId {
    uint32_t ib;
    int c0, ctEff, p0, Pn;
};

// Geometry of a tile launch: read from the argument struct, or fixed at compile time (see LinesRt / LinesFixed
// further down for what that buys).
struct TileRt {
    static constexpr bool FIXED = false;
    __device__ static uint32_t nthr(const TileArgs&) { return blockDim.x; }
    __device__ static uint32_t S(const TileArgs& a) { return (uint32_t)a.g.S; }
    __device__ static uint32_t C(const TileArgs& a) { return (uint32_t)a.g.C; }
    __device__ static uint32_t RS(const TileArgs& a) { return (uint32_t)(a.g.R * a.g.S); }
    __device__ static uint32_t P(const TileArgs& a) { return (uint32_t)a.P; }
    __device__ static uint32_t Pp(const TileArgs& a) { return (uint32_t)a.Pp; }
    __device__ static uint32_t psplit(const TileArgs& a) { return (uint32_t)a.psplit; }
    __device__ static uint32_t Ct(const TileArgs& a) { return (uint32_t)a.Ct; }
    __device__ static uint32_t lppLog(const TileArgs& a) { return (uint32_t)a.lppLog; }
    __device__ static uint32_t tpb(const TileArgs& a) { return a.tpb; }
    __device__ static uint32_t vpr(const TileArgs& a) { return a.vpr; }
    __device__ static uint32_t divS(uint32_t v, const TileArgs& a) { return fdiv(v, a.dS); }
    __device__ static uint32_t divPs(uint32_t v, const TileArgs& a) { return fdiv(v, a.dPs); }
    __device__ static uint32_t divTpb(uint32_t v, const TileArgs& a) { return fdiv(v, a.dTpb); }
    __device__ static uint32_t divVpr(uint32_t v, const TileArgs& a) { return fdiv(v, a.dVpr); }
};

// 4-float channel vectors only (C_ a multiple of 4); P_ pixels per tile.
template <int R_, int S_, int C_, int P_, int NTHR_>
struct TileFixed {
    static constexpr bool FIXED = true;
    static constexpr uint32_t kRS = R_ * S_;
    static constexpr uint32_t kLpp = C_ >= 32 ? 8 : C_ / 4;
    static constexpr uint32_t kLppLog = kLpp == 8 ? 3 : kLpp == 4 ? 2 : kLpp == 2 ? 1 : 0;
    static constexpr uint32_t kPsplit = (kRS + P_ - 1) / P_;
    static constexpr uint32_t kPp = (P_ + 31) / 32 * 32;
    static constexpr uint32_t kVpr = (P_ + 3) / 4;
    static constexpr uint32_t kCchunks = (C_ + 4 * kLpp - 1) / (4 * kLpp);
    static constexpr uint32_t kNthr = NTHR_, kCt = 4 * kLpp;
    __host__ __device__ static constexpr uint32_t nthr(const TileArgs&) { return NTHR_; }
    __host__ __device__ static constexpr uint32_t S(const TileArgs&) { return S_; }
    __host__ __device__ static constexpr uint32_t C(const TileArgs&) { return C_; }
    __host__ __device__ static constexpr uint32_t RS(const TileArgs&) { return kRS; }
    __host__ __device__ static constexpr uint32_t P(const TileArgs&) { return P_; }
    __host__ __device__ static constexpr uint32_t Pp(const TileArgs&) { return kPp; }
    __host__ __device__ static constexpr uint32_t psplit(const TileArgs&) { return kPsplit; }
    __host__ __device__ static constexpr uint32_t Ct(const TileArgs&) { return 4 * kLpp; }
    __host__ __device__ static constexpr uint32_t lppLog(const TileArgs&) { return kLppLog; }
    __host__ __device__ static constexpr uint32_t tpb(const TileArgs&) { return kPsplit * kCchunks; }
    __host__ __device__ static constexpr uint32_t vpr(const TileArgs&) { return kVpr; }
    __host__ __device__ static constexpr uint32_t divS(uint32_t v, const TileArgs&) { return v / (uint32_t)S_; }
    __host__ __device__ static constexpr uint32_t divPs(uint32_t v, const TileArgs&) { return v / kPsplit; }
    __host__ __device__ static constexpr uint32_t divTpb(uint32_t v, const TileArgs&) { return v / (kPsplit * kCchunks); }
    __host__ __device__ static constexpr uint32_t divVpr(uint32_t v, const TileArgs&) { return v / kVpr; }
};

template <typename G>
__device__ __forceinline__ void decode_tile(const TileArgs& a, TileId& t, uint32_t ib, uint32_t rem)
{
    t.ib = ib;
    const uint32_t cc = G::divPs(rem, a);
    const uint32_t pc = rem - cc * G::psplit(a);
    t.c0 = (int)(cc * G::Ct(a));
    t.ctEff = (int)min(G::Ct(a), G::C(a) - (uint32_t)t.c0);
    t.p0 = (int)(pc * G::P(a));
    t.Pn = (int)min(G::P(a), G::RS(a) - (uint32_t)t.p0);
}

__device__ __forceinline__ uint32_t lds_swz(uint32_t c) { return ((c >> 2) & 7u) << 2; }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits until every global store of
// the wave has been acknowledged (vmcnt(0)), which would drain the store queue once per tile.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 16-byte LDS read of 4 consecutive floats.  The promise of alignment has to be explicit: a plain vector
// load through a cast pointer was lowered to two 8-byte-pair reads, which serialise on the LDS banks.
__device__ __forceinline__ f4 lds_read4(const float* p)
{
    return *static_cast<const f4*>(__builtin_assume_aligned(p, 16));
}

// Raw buffer access (V# descriptors): 32-bit byte offsets from a wave-uniform base, and hardware range
// checking: a load whose offset is outside the descriptor returns 0, a store is dropped.  Lanes with
// nothing to do get the offset 0xFFFFFFFF instead of a branch, and the addressing needs no 64-bit
// per-lane arithmetic; the planar kernels spent more cycles computing addresses than waiting for memory.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
constexpr uint32_t BUF_OOB = 0xFFFFFFFFu;
constexpr int BUF_NT = 2;  // cache-policy operand of the buffer builtins: nontemporal

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <int VEC> __device__ __forceinline__ typename Vec<VEC>::type buf_load(rsrc_t r, uint32_t off);
template <> __device__ __forceinline__ f4 buf_load<4>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
}
template <> __device__ __forceinline__ f2 buf_load<2>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(f2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
}
template <> __device__ __forceinline__ float buf_load<1>(rsrc_t r, uint32_t off)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}

// Rows of the block list through a buffer descriptor: row j is 6 bytes at 6*j, fetched as the two aligned dwords
// around it with one 8-byte load (the descriptor starts at the list's address rounded down to 4 bytes and ends
// with the aligned dword that holds the list's last int16, so the load of the last row stays inside it).
struct ListRows {
    rsrc_t r;
    uint32_t mis;  // 0 or 2: the list's own misalignment
};

__device__ __forceinline__ ListRows list_rows(const int16_t* idx, uint32_t count)
{
    const uintptr_t p = reinterpret_cast<uintptr_t>(idx);
    ListRows l;
    l.mis = (uint32_t)(p & 2u);
    l.r = make_rsrc(reinterpret_cast<const void*>(p & ~(uintptr_t)3), (l.mis + count * 6u + 3u) & ~3u);
    return l;
}

struct ListRow {
    u2 w;
    uint32_t shift;  // 0 or 16
};

__device__ __forceinline__ ListRow list_row_load(const ListRows& l, uint32_t j, bool live)
{
    const uint32_t b = j * 6u + l.mis;
    ListRow row;
    row.w = __builtin_bit_cast(u2, __builtin_amdgcn_raw_buffer_load_b64(l.r, live ? (b & ~3u) : BUF_OOB, 0, 0));
    row.shift = (b & 2u) * 8u;
    return row;
}

__device__ __forceinline__ void list_row_unpack(const ListRow& row, int& n, int& bh, int& bw)
{
    const uint32_t nb = __builtin_amdgcn_alignbit(row.w.y, row.w.x, row.shift);  // (hi:lo) >> shift, low dword
    n = (int)(int16_t)(nb & 0xffffu);
    bh = (int)(int16_t)(nb >> 16);
    bw = (int)(int16_t)(row.shift ? row.w.y >> 16 : row.w.y & 0xffffu);
}

template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const f4& v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), r, off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const f2& v)
{
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2, v), r, off, 0, AUX);
}
template <int AUX> __device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, const float& v)
{
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, off, 0, AUX);
}

// ---- NHWC stack <-> NHWC tensor with buffer addressing ------------------------------------------
//
// k_gather_nhwc and k_scatter_nhwc are the row-segment copies for images and blocks below 2^30 floats
// (everything but the largest tensors; the _wide kernels, with 64-bit addresses and branches, remain for
// those): both sides go through range-checked descriptors, lanes
// with nothing to move get an out-of-range offset, and there is no control flow between the first load
// and the last store.  In the branchy version every conditional store was preceded by a full wait for
// outstanding memory operations, stores included, so the four stores of a lane went out one after the
// completion of the other.

// NHWC side of a tile: thread tid owns channel vector cl = tid & (lpp-1) of pixels pl0 + u*step,
// u = 0 .. TILE_LD-1, pl0 = tid >> lppLog, step = nthr >> lppLog.  Walks those pixels keeping (r, s) by
// increments and hands each one's byte offset inside the image (or BUF_OOB), its pixel number h*W + w (only
// meaningful with an in-range offset) and its position (r, s) inside the block to `f(u, pl, off, pix, r, s)`.
template <int VEC, typename G, typename F>
__device__ __forceinline__ void nhwc_walk(const TileArgs& a, const TileId& t, const BlockOrigin& o, uint32_t tid,
                                          uint32_t nthr, F f)
{
    const uint32_t lppLog = G::lppLog(a), S = G::S(a), C = G::C(a);
    const uint32_t lppMask = (1u << lppLog) - 1u;
    const uint32_t step = nthr >> lppLog;
    const uint32_t stepR = G::divS(step, a), stepS = step - stepR * S;
    uint32_t pl = tid >> lppLog;
    const uint32_t c = (uint32_t)t.c0 + (tid & lppMask) * VEC;
    const uint32_t p = (uint32_t)t.p0 + pl;
    uint32_t r = G::divS(p, a), s = p - r * S;
    const bool cok = c < C;
#pragma unroll
    for (int u = 0; u < TILE_LD; ++u) {
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
        const bool ok = cok && pl < (uint32_t)t.Pn && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t off = (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww) * C + c) * 4u;
        f(u, pl, ok ? off : BUF_OOB, (uint32_t)hh * (uint32_t)a.g.W + (uint32_t)ww, r, s);
        pl += step;
        r += stepR;
        s += stepS;
        if (s >= S) {
            s -= S;
            ++r;
        }
    }
}

// Launch shapes of the tile kernels.  (tiles per block, block rows): the block is the workgroup's y id, so its
// index triple can be fetched from preloaded kernel arguments before anything else arrives.  With the block count
// in device memory the launch cannot be sized for it: it covers half of the list's capacity in block rows and a
// workgroup takes block y and, if that is below the count, block y + rows.  Lists are rarely more than half full
// (sparse blocks pay off below that), so a workgroup almost never takes a second block, and the workgroups
// of rows past the count, which leave after one scalar load, are halved (at capacity 1024 and 312 blocks 17 088
// of them cost the scatter 3.6 us).  Beyond 65 535 block rows the launch is linear over the tiles.
template <typename ARGS, typename F>
__device__ __forceinline__ void for_each_block_of_workgroup(const ARGS& a, uint32_t tpb, F tile)
{
    if (a.grid2d) {
        // (two calls, not a loop: around a loop the compiler kept the whole tile's address arithmetic live and
        // tripled the register count)
        tile(blockIdx.y, blockIdx.x);
        const uint32_t ib2 = blockIdx.y + gridDim.y;
        if (ib2 < a.blocks && !beyond_count(a.g, ib2)) {  // (the same for the whole workgroup)
            __syncthreads();                               // LDS is reused
            tile(ib2, blockIdx.x);
        }
    } else {
        const uint32_t ib = blockIdx.x / tpb;
        tile(ib, blockIdx.x - ib * tpb);
    }
}

// Fallback for block planes of fewer than 4 pixels (1x1, 1x2, 1x3 ... blocks), where a dwordx4 slot does
// not fit into a planar run: one thread per stack element.  The channel index varies fastest across
// threads, so the NHWC side stays coalesced.
template <int MODE, bool GATHER>
__global__ __launch_bounds__(256) void k_planar_small(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, Geom g, int64_t total,
                                                      const int32_t* __restrict__ owner)
{
    const int RS = g.R * g.S;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int c = (int)(i % g.C);
        const int p = (int)((i / g.C) % RS);
        const int64_t ib = i / ((int64_t)g.C * RS);
        if (g.countDev && ib >= *g.countDev) continue;
        const int r = p / g.S, s = p - r * g.S;
        const BlockOrigin o = load_origin(idx, (uint32_t)ib, g);
        const int hh = o.h0 + r, ww = o.w0 + s;
        const bool in = o.valid && (unsigned)hh < (unsigned)g.H && (unsigned)ww < (unsigned)g.W;
        const int64_t pix = (((int64_t)o.n * g.H + hh) * g.W + ww) * g.C + c;
        const int64_t st = (ib * g.C + c) * RS + p;
        if (GATHER) {
            y[st] = in ? x[pix] : 0.f;
        } else if (in) {
            if (MODE == SCATTER_OWNED) {
                if (owner[((int64_t)o.n * g.H + hh) * g.W + ww] == (int32_t)ib) y[pix] = x[st];
            } else if (MODE == SCATTER_RANKED) {
                if (!ranked_out((uint32_t)owner[ib], (uint32_t)r, (uint32_t)s, g)) y[pix] = x[st];
            } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED_INLINE) y[pix] = x[st];
            else if (MODE == SCATTER_ADD) y[pix] = ysrc[pix] + x[st];
            else atomic_add_f32(y + pix, x[st]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// host side: launch configuration
// ---------------------------------------------------------------------------------------------

static int ilog2_floor(uint32_t v)
{
    int l = 0;
    while ((2u << l) <= v) ++l;
    return l;
}

constexpr int GRID_Y_MAX = 65535;

// One workgroup per tile, as (tiles per block, block rows) when the block count fits the y dimension of a launch;
// half as many rows as the list holds when the count is only known on the device (for_each_block_of_workgroup).
static dim3 tile_grid(int grid2d, uint32_t tpb, int numActive, uint32_t total, const Geom& g)
{
    if (!grid2d) return dim3(total);
    return dim3(tpb, (unsigned)(g.countDev && numActive > 1 ? (numActive + 1) / 2 : numActive));
}

static int pick_vec(const Geom& g, const void* a, const void* b)
{
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
    if (g.C % 4 == 0 && (bits & 15) == 0) return 4;
    if (g.C % 2 == 0 && (bits & 7) == 0) return 2;
    return 1;
}

static bool make_nhwc_args(const Geom& g, int numActive, int vec, NhwcArgs& a)
{
    a.g = g;
    const uint64_t rowV = (uint64_t)g.S * g.C / vec;
    const uint64_t blockV = rowV * g.R;
    if (blockV >= (1ull << 31)) return false;
    a.rowV = (uint32_t)rowV;
    a.blockV = (uint32_t)blockV;
    a.cpb = (uint32_t)((blockV + NHWC_CHUNK - 1) / NHWC_CHUNK);
    const uint64_t units = (uint64_t)numActive * a.cpb;
    if (units >= (1ull << 31)) return false;
    a.units = (uint32_t)units;
    a.dCpb = make_fastdiv(a.cpb);
    a.dRow = make_fastdiv(a.rowV);
    a.dCV = make_fastdiv((uint32_t)(g.C / vec));
    return true;
}

// 32-bit byte offsets inside one image and inside one block: the buffer-addressed NHWC kernels apply.
static bool nhwc_fits_buffers(const Geom& g)
{
    return (int64_t)g.H * g.W * g.C < (1ll << 30) && (int64_t)g.R * g.S * g.C < (1ll << 30);
}

// Chooses the tile and the workgroup size of the planar kernels; the grid is one workgroup per tile.
static bool make_tile_args(const Geom& g, int numActive, int vec, TileArgs& a, int& threads, size_t& ldsBytes,
                           unsigned& grid, int defaultLdsBudget)
{
    a.g = g;
    const int64_t RS64 = (int64_t)g.R * g.S;
    if (RS64 >= (1ll << 30)) return false;
    const int RS = (int)RS64;
    // channels per tile: 32 floats (one 128-byte line per pixel) unless C is smaller
    const int ctWant = 32;
    int lpp = 1;
    while (lpp * 2 * vec <= ctWant && lpp * vec < g.C) lpp *= 2;
    a.Ct = lpp * vec;
    a.lppLog = ilog2_floor((uint32_t)lpp);
    a.cchunks = (g.C + a.Ct - 1) / a.Ct;
    // Pixels per tile are bounded by the LDS budget and by the TILE_LD registers per thread that hold a
    // tile in flight on either side.  The smallest workgroup that takes a whole block plane wins.
    const int budget = defaultLdsBudget;
    int maxP = 0;
    threads = 0;
    for (int nthr = 64; nthr <= 512; nthr *= 2) {
        const int pLds = (budget / (4 * a.Ct)) / 32 * 32;
        const int pItems = TILE_LD * nthr / lpp;
        const int pSlots = (TILE_LD * nthr / a.Ct) * 4 - 3;
        maxP = pLds < pItems ? pLds : pItems;
        if (pSlots < maxP) maxP = pSlots;
        threads = nthr;
        if (maxP >= RS) break;
    }
    if (maxP < 1) return false;
    a.psplit = (RS + maxP - 1) / maxP;
    a.P = (RS + a.psplit - 1) / a.psplit;
    // whole dwordx4 slots per planar run where the limits allow: only a plane's last split then ends in a
    // partial slot
    if (a.psplit > 1 && ((a.P + 3) & ~3) <= maxP) a.P = (a.P + 3) & ~3;
    a.psplit = (RS + a.P - 1) / a.P;
    a.Pp = (a.P + 31) / 32 * 32;
    a.vpr = (uint32_t)((a.P + 3) / 4);
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (a.imgFloats >= (1ll << 30) || (int64_t)g.C * RS64 >= (1ll << 30)) return false;  // 32-bit byte offsets
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    a.tpb = (uint32_t)(a.psplit * a.cchunks);
    const uint64_t total = (uint64_t)numActive * a.tpb;
    if (total >= (1ull << 31)) return false;
    a.total = (uint32_t)total;
    a.dTpb = make_fastdiv(a.tpb);
    a.dPs = make_fastdiv((uint32_t)a.psplit);
    a.dS = make_fastdiv((uint32_t)g.S);
    a.dVpr = make_fastdiv(a.vpr);
    ldsBytes = (size_t)a.Ct * a.Pp * sizeof(float);
    if (ldsBytes > 64 * 1024) return false;
    grid = a.total;
    a.grid2d = numActive <= GRID_Y_MAX;
    a.blocks = (uint32_t)numActive;
    return true;
}

// Compute units of the current device (256 on MI355X), looked up once per device.
static int device_cus()
{
    static std::mutex mutex;
    static int cus[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return 256;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        cus[dev] = n;
    }
    return cus[dev];
}

// The scatter's half of the tile_choice test hook (sbnet_scatter.hip).
int scatter_tile_choice(const Geom& g, int numActive, int vec, int32_t* out);

}  // namespace sbnet

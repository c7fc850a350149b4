// sparse_scatter / sparse_scatter_var on gfx950: plain write, add and atomic add from either stack layout; the
// owner-computes overlapping add, the add in passes, ordered overlapping writes (rank table, owner map), the
// copying op built in one pass, and the flat copy; with the launch configuration.
// Reference semantics: sbnet_tensorflow/sbnet_ops/sparse_gather.cc:103-130, 135-142, 338-346.
#include "sbnet_device.h"

namespace sbnet {

constexpr int NHWC_RANK_ROWS = 1;  // list rows per thread that the NHWC kernel fetches at once when it ranks its block

// sparse_gather.cc:103-130 with transpose == false.
template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_nhwc_wide(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, NhwcArgs a, ColorArgs col)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    uint32_t ib = fdiv(unit, a.dCpb);
    const uint32_t chunk = unit - ib * a.cpb;
    if (MODE == SCATTER_COLOR && !color_block(col, ib, ib)) return;
    if (beyond_count(a.g, ib)) return;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);  // ib is wave-uniform: scalar load
    if (!o.valid) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, o, atomics)) return;
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const vec* __restrict__ xb = reinterpret_cast<const vec*>(x) + (size_t)ib * a.blockV;
    vec* yv = reinterpret_cast<vec*>(y);
    const vec* ysv = reinterpret_cast<const vec*>(ysrc);  // what an add reads: y itself, or the base y is a copy of
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;

    vec v[NHWC_UNR];
    int64_t dst[NHWC_UNR];
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        dst[u] = -1;
        v[u] = vzero<VEC>();
        if (e < a.blockV) {
            const uint32_t r = fdiv(e, a.dRow);
            const int j = (int)(e - r * a.rowV);
            const int hh = o.h0 + (int)r;
            if ((unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi) {
                dst[u] = (((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0) * CV + j;
                if (MODE == SCATTER_OWNED &&
                    col.owner[((int64_t)o.n * a.g.H + hh) * a.g.W + o.w0 + (int)fdiv((uint32_t)j, a.dCV)] != (int32_t)ib)
                    dst[u] = -1;
                else if (MODE == SCATTER_RANKED && ranked_out(rank_bits(col, ib), r, fdiv((uint32_t)j, a.dCV), a.g))
                    dst[u] = -1;
                else
                    v[u] = ld_stream(xb + e);
            }
        }
    }
    if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
        vec cur[NHWC_UNR];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) cur[u] = ld_stream(ysv + dst[u]);
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) st_stream(yv + dst[u], vadd(cur[u], v[u]));
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_OWNED || MODE == SCATTER_RANKED || MODE == SCATTER_RANKED_INLINE) {
        // (SCATTER_RANKED_INLINE is never launched on this kernel; plain stores if it were)
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) commit<VEC, SCATTER_ASSIGN>(yv + dst[u], v[u]);
    } else {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            if (dst[u] >= 0) commit<VEC, SCATTER_ATOMIC>(yv + dst[u], v[u]);
    }
}

template <int VEC, int MODE>
__global__ __launch_bounds__(256) void k_scatter_nhwc(const float* __restrict__ x, float* y, const float* ysrc,
                                                      const int16_t* __restrict__ idx, NhwcArgs a, ColorArgs col)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t lane = threadIdx.x & 63;
    uint32_t unit = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= a.units) return;
    unit = __builtin_amdgcn_readfirstlane(unit);
    uint32_t ib = fdiv(unit, a.dCpb);
    const uint32_t chunk = unit - ib * a.cpb;
    if (MODE == SCATTER_COLOR && !color_block(col, ib, ib)) return;
    if (beyond_count(a.g, ib)) return;
    const BlockOrigin o = origin_of(load_triple(idx, ib), a.g);
    if (!o.valid) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, o, atomics)) return;
    const int CV = a.g.C / VEC;
    const int slo = max(0, -o.w0), shi = min(a.g.S, a.g.W - o.w0);
    const int lo = slo * CV, hi = shi * CV;
    const int64_t imgFloats = (int64_t)a.g.H * a.g.W * a.g.C;
    float* img = y + (int64_t)o.n * imgFloats;
    const rsrc_t yr = make_rsrc(img, (uint32_t)imgFloats * 4u);
    const rsrc_t sr = make_rsrc(ysrc + (int64_t)o.n * imgFloats, (uint32_t)imgFloats * 4u);  // what an add reads
    const rsrc_t xr = make_rsrc(x + (int64_t)ib * a.blockV * VEC, a.blockV * (uint32_t)(VEC * 4));
    const uint32_t e0 = chunk * NHWC_CHUNK + lane;
    vec v[NHWC_UNR];
    uint32_t dst[NHWC_UNR];
    int32_t own[NHWC_UNR];
    NeighbourPos nb;
    nb.later = 0u;
    const bool repeats = MODE == SCATTER_SUM && list_has_repeats(col);
    if (MODE == SCATTER_SUM && !repeats) nb = neighbour_positions(col, o, ib);
    const rsrc_t wr = make_rsrc(MODE == SCATTER_OWNED ? col.owner + (int64_t)o.n * a.g.H * a.g.W : nullptr,
                                MODE == SCATTER_OWNED ? (uint32_t)(a.g.H * a.g.W) * 4u : 0u);
    // SCATTER_RANKED_INLINE: the block is ranked against the rows listed after it inside the kernel.  The rows are
    // fetched AHEAD of the wave's own loads, so they arrive first and are compared while the data is still on its
    // way (loads return in order): the stores wait no longer than they would anyway.  The four waves of a workgroup
    // mostly move the same block: they then share the comparison, NHWC_RANK_ROWS rows per thread, and meet at one
    // barrier; a workgroup whose waves move two blocks compares per wave.
    __shared__ uint32_t waveBits[4];
    ListRow rows[NHWC_RANK_ROWS];
    ListRows lr;
    uint32_t listCount = 0, me = lane, step = 64u;
    const uint32_t unit0 = blockIdx.x * 4u;
    bool shared = false;
    if (MODE == SCATTER_RANKED_INLINE) {
        listCount = list_count(a.g, fdiv(a.units, a.dCpb));
        lr = list_rows(idx, listCount);
        shared = fdiv(unit0, a.dCpb) == fdiv(min(unit0 + 3u, a.units - 1u), a.dCpb);  // (the same for the whole workgroup)
        if (shared) {
            me = threadIdx.x;
            step = 256u;
        }
#pragma unroll
        for (int u = 0; u < NHWC_RANK_ROWS; ++u) {
            const uint32_t j = ib + 1u + (uint32_t)u * step + me;
            rows[u] = list_row_load(lr, j, j < listCount);
        }
    }
#pragma unroll
    for (int u = 0; u < NHWC_UNR; ++u) {
        const uint32_t e = e0 + u * 64;
        const uint32_t r = fdiv(e, a.dRow);
        const int j = (int)(e - r * a.rowV);
        const int hh = o.h0 + (int)r;
        bool ok = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && j >= lo && j < hi;
        if (MODE == SCATTER_RANKED) ok = ok && !ranked_out(rank_bits(col, ib), r, fdiv((uint32_t)j, a.dCV), a.g);
        if (MODE == SCATTER_SUM) ok = ok && !ranked_out(nb.later, r, fdiv((uint32_t)j, a.dCV), a.g);
        dst[u] = ok ? (((uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0) * (uint32_t)CV + (uint32_t)j) * (uint32_t)(VEC * 4)
                    : BUF_OOB;
        v[u] = buf_load<VEC>(xr, ok ? e * (uint32_t)(VEC * 4) : BUF_OOB);  // off-image parts are not read
        if (MODE == SCATTER_OWNED) {
            const uint32_t pix = (uint32_t)hh * (uint32_t)a.g.W + (uint32_t)o.w0 + fdiv((uint32_t)j, a.dCV);
            own[u] = __builtin_bit_cast(int32_t, buf_load<1>(wr, ok ? pix * 4u : BUF_OOB));
        }
    }
    if (MODE == SCATTER_RANKED_INLINE) {
        // pixels of a class that a later row covers are not stored (their loads were issued for nothing: two rows
        // and columns of a block)
        uint32_t bits = 0u;
#pragma unroll
        for (int u = 0; u < NHWC_RANK_ROWS; ++u) {
            int n2, bh2, bw2;
            list_row_unpack(rows[u], n2, bh2, bw2);
            if (ib + 1u + (uint32_t)u * step + me < listCount) bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        for (uint32_t j = ib + 1u + (uint32_t)NHWC_RANK_ROWS * step + me; j < listCount; j += step) {
            int n2, bh2, bw2;
            list_row_unpack(list_row_load(lr, j, true), n2, bh2, bw2);
            bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        // most waves see none of the few neighbouring rows
        if (__ballot(bits != 0u) != 0ull)
            for (int off = 32; off > 0; off >>= 1) bits |= (uint32_t)__shfl_xor((int)bits, off);
        if (shared) {
            if (lane == 0u) waveBits[threadIdx.x >> 6] = bits;
            lds_barrier();
            // (waves past the last unit have left before the barrier, which waits for the surviving ones only)
            bits = 0u;
#pragma unroll
            for (uint32_t w = 0; w < 4u; ++w)
                if (unit0 + w < a.units) bits |= waveBits[w];
        }
        if (bits != 0u) {
#pragma unroll
            for (int u = 0; u < NHWC_UNR; ++u) {
                const uint32_t e = e0 + u * 64;
                const uint32_t r = fdiv(e, a.dRow);
                if (ranked_out(bits, r, fdiv(e - r * a.rowV, a.dCV), a.g)) dst[u] = BUF_OOB;
            }
        }
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, dst[u], v[u]);
    } else if (MODE == SCATTER_OWNED) {
        // (an out-of-range owner read returns 0, which may equal ib: dst is BUF_OOB there already)
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, own[u] == (int32_t)ib ? dst[u] : BUF_OOB, v[u]);
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED) {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, dst[u], v[u]);
    } else if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
        vec cur[NHWC_UNR];
        // (colour passes onto zeros: a pixel is read only where an earlier pass has written it; an out-of-range
        // read returns 0, and 0 + v is what a pixel's first write stores)
        const uint32_t ebits = MODE == SCATTER_COLOR && col.first ? earlier_pass_bits(col, o) : 0x1ffu;
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) {
            uint32_t src = dst[u];
            if (MODE == SCATTER_COLOR && col.first) {
                const uint32_t e = e0 + u * 64;
                const uint32_t r = fdiv(e, a.dRow);
                if (!ranked_out(ebits, r, fdiv(e - r * a.rowV, a.dCV), a.g)) src = BUF_OOB;
            }
            cur[u] = buf_load<VEC>(sr, src);
        }
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) buf_store<BUF_NT>(yr, dst[u], vadd(cur[u], v[u]));
    } else if (MODE == SCATTER_SUM) {
        if (repeats) {  // (onto zeros everywhere)
#pragma unroll
            for (int u = 0; u < NHWC_UNR; ++u) {
                if (dst[u] != BUF_OOB) {
                    float* d = img + (dst[u] >> 2);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v[u], k));
                }
            }
            return;
        }
        // the owner's sum: 0 + the blocks listed before this one, in list order, + its own value; the other blocks'
        // values of a pixel (three at most) are fetched together
        const rsrc_t sr2 = make_rsrc(x, fdiv(a.units, a.dCpb) * a.blockV * (uint32_t)(VEC * 4));  // the whole stack
        vec nv[NHWC_UNR][3];
        PixelNeighbours pn[NHWC_UNR];
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) {
            const uint32_t e = e0 + u * 64;
            const uint32_t r = fdiv(e, a.dRow);
            const uint32_t j = e - r * a.rowV, sc = fdiv(j, a.dCV);
            pn[u] = pixel_neighbours(nb, (int)r, (int)sc, a.g);
            if (dst[u] == BUF_OOB) pn[u].pv = pn[u].ph = pn[u].pd = -1;
            const int up = pn[u].dh * a.g.U * (int)a.rowV, left = pn[u].dw * a.g.V * CV;
            const uint32_t ev = (uint32_t)((int)e - up), eh = (uint32_t)((int)e - left), ed = (uint32_t)((int)e - up - left);
            // (under branches: a wave without such pixels skips the load)
            nv[u][0] = nv[u][1] = nv[u][2] = vzero<VEC>();
            if (pn[u].pv >= 0) nv[u][0] = buf_load<VEC>(sr2, ((uint32_t)pn[u].pv * a.blockV + ev) * (uint32_t)(VEC * 4));
            if (pn[u].ph >= 0) nv[u][1] = buf_load<VEC>(sr2, ((uint32_t)pn[u].ph * a.blockV + eh) * (uint32_t)(VEC * 4));
            if (pn[u].pd >= 0) nv[u][2] = buf_load<VEC>(sr2, ((uint32_t)pn[u].pd * a.blockV + ed) * (uint32_t)(VEC * 4));
        }
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u)
            buf_store<BUF_NT>(yr, dst[u], sum_of_pixel(pn[u].pv, nv[u][0], pn[u].ph, nv[u][1], pn[u].pd, nv[u][2], v[u],
                                                       vzero<VEC>()));
    } else {
#pragma unroll
        for (int u = 0; u < NHWC_UNR; ++u) {
            if (dst[u] != BUF_OOB) {
                float* d = img + (dst[u] >> 2);
#pragma unroll
                for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(v[u], k));
            }
        }
    }
}

// sparse_gather.cc:103-130 with transpose == true: the block stack is [blocks, C, R, S].
template <int VEC, int MODE, typename G>
__device__ __forceinline__ void scatter_planar_tile(const float* __restrict__ x, float* y, const float* ysrc,
                                                    const int16_t* __restrict__ idx, const TileArgs& a,
                                                    const ColorArgs& col, float* lds, uint32_t* waveBits,
                                                    uint32_t ib, uint32_t rem)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t tid = threadIdx.x, nthr = G::nthr(a);
    const uint32_t RS = G::RS(a), Pp = G::Pp(a), vpr = G::vpr(a);
    TileId t;
    if (MODE == SCATTER_COLOR && !color_block(col, ib, ib)) return;
    decode_tile<G>(a, t, ib, rem);
    const RawTriple raw = load_triple(idx, t.ib);  // scalar load, needed only after the barrier
    if (beyond_count(a.g, t.ib)) return;
    bool atomics = MODE == SCATTER_ATOMIC;
    if (MODE == SCATTER_COLOR && color_skip(col, origin_of(raw, a.g), atomics)) return;  // (here: before the loads)

    // global -> registers, planar side.  The last slot of a run, when partial, is read as the last 4 floats
    // of the run instead (overlapping its neighbour): no load leaves the run, no value needs fixing up.
    const rsrc_t xr = make_rsrc(x + ((int64_t)t.ib * G::C(a) + t.c0) * RS + t.p0,
                                ((uint32_t)(t.ctEff - 1) * RS + (uint32_t)t.Pn) * 4u);
    const uint32_t slots = (uint32_t)t.ctEff * vpr;
    // SCATTER_RANKED_INLINE: the rows listed after this block, RANK_ROWS_PER_THREAD per thread, fetched behind the
    // tile's own loads (loads return in order, so they are there when the tile's data is)
    ListRow rows[RANK_ROWS_PER_THREAD];
    uint32_t listCount = 0;
    ListRows lr;
    // SCATTER_SUM: the other blocks' values of the pixels that this block sums (three per pixel at most) are fetched
    // behind the tile's own loads as well: the neighbours' list positions (scalar loads), the walk over the tile's
    // pixels, then the loads, all before the first wait for the tile's data.
    constexpr int NSUM = MODE == SCATTER_SUM ? TILE_LD : 1;
    typename Vec<VEC>::type nv[NSUM][3];
    PixelNeighbours pn[NSUM];
    uint32_t offs[TILE_LD], pls[TILE_LD];
    NeighbourPos nb;
    nb.later = 0u;
    bool summed = false;  // offs / pls / pn / nv are set
    const uint32_t c0l = (tid & ((1u << G::lppLog(a)) - 1u)) * VEC;
    auto fetch_neighbours = [&]() {
        if (MODE != SCATTER_SUM) return;
        const BlockOrigin o = origin_of(raw, a.g);
        atomics = list_has_repeats(col);
        if (!o.valid || atomics) return;
        nb = neighbour_positions(col, o, t.ib);
        summed = true;
        const rsrc_t sr2 = make_rsrc(x, (uint32_t)a.blocks * G::C(a) * RS * 4u);  // the whole stack
        const int S = (int)G::S(a);
        const uint32_t c = (uint32_t)t.c0 + c0l;
        // (wave-uniform: whole directions without a block listed earlier cost a scalar branch)
        const bool anyV = (nb.pos[1] & nb.pos[7]) >= 0, anyH = (nb.pos[3] & nb.pos[5]) >= 0;
        const bool anyD = (nb.pos[0] & nb.pos[2] & nb.pos[6] & nb.pos[8]) >= 0;
        nhwc_walk<VEC, G>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t, uint32_t r, uint32_t sc) {
            if (ranked_out(nb.later, r, sc, a.g)) off = BUF_OOB;  // (a block listed later owns the pixel)
            offs[u] = off;
            pls[u] = pl;
            const int v = MODE == SCATTER_SUM ? u : 0;
            pn[v].pv = pn[v].ph = pn[v].pd = -1;
            nv[v][0] = nv[v][1] = nv[v][2] = vzero<VEC>();
            if (!(anyV || anyH || anyD)) return;
            const PixelNeighbours q = pixel_neighbours(nb, (int)r, (int)sc, a.g);
            const bool mine = off != BUF_OOB;
            const int p = (int)r * S + (int)sc, up = q.dh * a.g.U * S, left = q.dw * a.g.V;
            // (under branches, not with out-of-range offsets: few pixels have such a block at all, and a wave
            // that has none skips the loads, which would otherwise keep the address units as busy as real ones)
            if (anyV && mine && q.pv >= 0) {
                pn[v].pv = q.pv;
#pragma unroll
                for (int k = 0; k < VEC; ++k)
                    vset(nv[v][0], k, buf_load<1>(sr2, ((((uint32_t)q.pv * G::C(a) + c + k) * RS) + (uint32_t)(p - up)) * 4u));
            }
            if (anyH && mine && q.ph >= 0) {
                pn[v].ph = q.ph;
#pragma unroll
                for (int k = 0; k < VEC; ++k)
                    vset(nv[v][1], k, buf_load<1>(sr2, ((((uint32_t)q.ph * G::C(a) + c + k) * RS) + (uint32_t)(p - left)) * 4u));
            }
            if (anyD && mine && q.pd >= 0) {
                pn[v].pd = q.pd;
#pragma unroll
                for (int k = 0; k < VEC; ++k)
                    vset(nv[v][2], k, buf_load<1>(sr2, ((((uint32_t)q.pd * G::C(a) + c + k) * RS) + (uint32_t)(p - up - left)) * 4u));
            }
        });
    };
    auto fetch_rows = [&]() {
        fetch_neighbours();
        if (MODE != SCATTER_RANKED_INLINE) return;
        listCount = list_count(a.g, a.blocks);
        lr = list_rows(idx, listCount);
#pragma unroll
        for (int u = 0; u < RANK_ROWS_PER_THREAD; ++u) {
            const uint32_t j = t.ib + 1u + (uint32_t)u * nthr + tid;
            rows[u] = list_row_load(lr, j, j < listCount);
        }
    };
    if (t.Pn >= 4) {
        f4 val[TILE_LD];
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            const uint32_t i = u * nthr + tid;
            const uint32_t c = G::divVpr(i, a);
            const int e0 = min(4 * (int)(i - c * vpr), t.Pn - 4);
            val[u] = buf_load<4>(xr, i < slots ? (c * RS + (uint32_t)e0) * 4u : BUF_OOB);
        }
        fetch_rows();
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            const uint32_t i = u * nthr + tid;
            if (i < slots) {
                const uint32_t c = G::divVpr(i, a);
                const int e0 = 4 * (int)(i - c * vpr);
                float* __restrict__ row = lds + c * Pp;
                if (e0 + 4 <= t.Pn) {
                    *reinterpret_cast<f4*>(row + ((uint32_t)e0 ^ lds_swz(c))) = val[u];
                } else if (e0 < t.Pn) {  // partial last slot: holds floats [Pn-4, Pn) of the run
                    const uint32_t t0 = (uint32_t)(t.Pn - 4);
                    row[(t0 + 0) ^ lds_swz(c)] = val[u].x;
                    row[(t0 + 1) ^ lds_swz(c)] = val[u].y;
                    row[(t0 + 2) ^ lds_swz(c)] = val[u].z;
                    row[(t0 + 3) ^ lds_swz(c)] = val[u].w;
                }
            }
        }
    } else {
        // A plane's last split can hold fewer pixels than one slot (the split width is rounded up to whole slots,
        // and 1-3 pixels may remain): one thread per row moves them float by float.
        if (tid < (uint32_t)t.ctEff) {
            for (int k = 0; k < t.Pn; ++k)
                lds[tid * Pp + ((uint32_t)k ^ lds_swz(tid))] = buf_load<1>(xr, (tid * RS + (uint32_t)k) * 4u);
        }
        fetch_rows();
    }
    const BlockOrigin o = origin_of(raw, a.g);
    // (colour passes onto zeros: the neighbours' map entries, fetched while the tile's loads are in flight)
    const uint32_t ebits = MODE == SCATTER_COLOR && col.first && o.valid ? earlier_pass_bits(col, o) : 0x1ffu;
    if (MODE == SCATTER_RANKED_INLINE) {
        // nine bits: classes of this block's pixels that a block listed later covers (the later one wins them)
        uint32_t bits = 0u;
#pragma unroll
        for (int u = 0; u < RANK_ROWS_PER_THREAD; ++u) {
            int n2, bh2, bw2;
            list_row_unpack(rows[u], n2, bh2, bw2);
            if (t.ib + 1u + (uint32_t)u * nthr + tid < listCount) bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        // (lists with more than RANK_ROWS_PER_THREAD * nthr rows after this block)
        for (uint32_t j = t.ib + 1u + (uint32_t)RANK_ROWS_PER_THREAD * nthr + tid; j < listCount; j += nthr) {
            int n2, bh2, bw2;
            list_row_unpack(list_row_load(lr, j, true), n2, bh2, bw2);
            bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        // most waves see none of the few neighbouring rows
        if (__ballot(bits != 0u) != 0ull)
            for (int off = 32; off > 0; off >>= 1) bits |= (uint32_t)__shfl_xor((int)bits, off);
        if ((tid & 63u) == 0u) waveBits[tid >> 6] = bits;
    }
    if (!o.valid) return;  // (the whole workgroup)

    // NHWC side: LDS -> base tensor; pixels outside the image are dropped (sparse_gather.cc:121)
    float* img = y + (int64_t)o.n * a.imgFloats;
    const rsrc_t yr = make_rsrc(img, a.imgBytes);
    const rsrc_t sr = make_rsrc(ysrc + (int64_t)o.n * a.imgFloats, a.imgBytes);  // what an add reads
    vec w[TILE_LD], cur[TILE_LD];
    int32_t own[TILE_LD];
    const rsrc_t wr = make_rsrc(MODE == SCATTER_OWNED ? col.owner + (int64_t)o.n * a.g.H * a.g.W : nullptr,
                                MODE == SCATTER_OWNED ? (uint32_t)(a.g.H * a.g.W) * 4u : 0u);
    uint32_t rbits = MODE == SCATTER_RANKED ? rank_bits(col, t.ib) : 0u;
    // colour passes onto zeros: a pixel is read only where a block of an earlier pass has written it (an out-of-range
    // read returns 0, and 0 + v is what a pixel's first write stores)
    bool rmw[TILE_LD];
    auto walk = [&]() {
        nhwc_walk<VEC, G>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t pix, uint32_t r, uint32_t sc) {
            if ((MODE == SCATTER_RANKED || MODE == SCATTER_RANKED_INLINE) && ranked_out(rbits, r, sc, a.g)) off = BUF_OOB;
            rmw[u] = MODE != SCATTER_COLOR || ranked_out(ebits, r, sc, a.g);
            offs[u] = off;
            pls[u] = pl;
            if (MODE == SCATTER_OWNED) own[u] = __builtin_bit_cast(int32_t, buf_load<1>(wr, off != BUF_OOB ? pix * 4u : BUF_OOB));
        });
    };
    // An add's reads of the base do not depend on the tile: they go out before the barrier, behind the tile's loads.
    constexpr bool EARLY = MODE == SCATTER_ADD || MODE == SCATTER_COLOR;
    if (EARLY) {
        walk();
        if (!atomics) {
#pragma unroll
            for (int u = 0; u < TILE_LD; ++u) cur[u] = buf_load<VEC>(sr, MODE == SCATTER_COLOR && !rmw[u] ? BUF_OOB : offs[u]);
        }
    }
    lds_barrier();
    if (!EARLY) {
        if (MODE == SCATTER_RANKED_INLINE) {
            for (uint32_t wv = 0; wv < (nthr >> 6); ++wv) rbits |= waveBits[wv];
        }
        if (!summed) walk();
    }
#pragma unroll
    for (int u = 0; u < TILE_LD; ++u) {
        w[u] = vzero<VEC>();
        if (offs[u] != BUF_OOB) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const uint32_t c = c0l + k;
                vset(w[u], k, lds[c * Pp + (pls[u] ^ lds_swz(c))]);
            }
        }
    }
    if (MODE == SCATTER_OWNED) {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, own[u] == (int32_t)t.ib ? offs[u] : BUF_OOB, w[u]);
    } else if (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED || MODE == SCATTER_RANKED_INLINE) {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, offs[u], w[u]);
    } else if (MODE == SCATTER_ADD || (MODE == SCATTER_COLOR && !atomics)) {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) buf_store<BUF_NT>(yr, offs[u], vadd(cur[u], w[u]));
    } else if (MODE == SCATTER_SUM && !atomics) {
        // the owner's sum: 0 + the blocks listed before this one, in list order, + its own value
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            const int v = MODE == SCATTER_SUM ? u : 0;
            buf_store<BUF_NT>(yr, offs[u], sum_of_pixel(pn[v].pv, nv[v][0], pn[v].ph, nv[v][1], pn[v].pd, nv[v][2], w[u],
                                                       vzero<VEC>()));
        }
    } else {
#pragma unroll
        for (int u = 0; u < TILE_LD; ++u) {
            if (offs[u] != BUF_OOB) {
                float* d = img + (offs[u] >> 2);
#pragma unroll
                for (int k = 0; k < VEC; ++k) atomic_add_f32(d + k, vget(w[u], k));
            }
        }
    }
}

// The same tile moved in two halves, for launches of so few workgroups that all of them are resident at once: such
// a launch runs in lockstep (every workgroup loads, then every workgroup stores), so its reads and its writes do
// not overlap and it takes the sum of both.  Here a workgroup issues the loads of both halves of its pixels up
// front, and stores the first half (the first 2 of a thread's 4 NHWC pixels: 2 * nthr / 8 tile pixels) while the
// second half's loads are still arriving.  Fixed-shape instances of plain and ordered writes only (4-float channel
// vectors, full channel chunks, every split at least as long as the first half).
template <int MODE, typename G>
__device__ __forceinline__ void scatter_planar_tile_halves(const float* __restrict__ x, float* y,
                                                           const int16_t* __restrict__ idx, const TileArgs& a,
                                                           float* lds, uint32_t* waveBits, uint32_t ib, uint32_t rem)
{
    constexpr uint32_t nthr = G::kNthr, RS = G::kRS, Pp = G::kPp, vpr = G::kVpr;
    constexpr uint32_t PA = 2u * (nthr >> G::kLppLog);  // pixels of the first half
    constexpr uint32_t vprA = PA / 4u, vprB = vpr - vprA;
    constexpr uint32_t CT = G::kCt;
    static_assert(CT * vprA == 2u * nthr, "two loads per thread cover the first half");
    static_assert(CT * vprB <= nthr && vprB > 0, "one load per thread covers the second half");
    const uint32_t tid = threadIdx.x;
    TileId t;
    decode_tile<G>(a, t, ib, rem);
    const RawTriple raw = load_triple(idx, t.ib);
    if (beyond_count(a.g, t.ib)) return;
    const rsrc_t xr = make_rsrc(x + ((int64_t)t.ib * G::C(a) + t.c0) * RS + t.p0,
                                ((uint32_t)(t.ctEff - 1) * RS + (uint32_t)t.Pn) * 4u);
    f4 valA[2], valB;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t i = (uint32_t)u * nthr + tid;
        valA[u] = buf_load<4>(xr, ((i / vprA) * RS + 4u * (i % vprA)) * 4u);
    }
    const uint32_t cB = tid / vprB, eB = vprA + tid % vprB;
    const int e0B = min(4 * (int)eB, t.Pn - 4);  // a partial last slot is read as the run's last 4 floats
    valB = buf_load<4>(xr, cB < CT ? (cB * RS + (uint32_t)e0B) * 4u : BUF_OOB);
    ListRow rows[RANK_ROWS_PER_THREAD];
    uint32_t listCount = 0;
    ListRows lr;
    if (MODE == SCATTER_RANKED_INLINE) {
        listCount = list_count(a.g, a.blocks);
        lr = list_rows(idx, listCount);
#pragma unroll
        for (int u = 0; u < RANK_ROWS_PER_THREAD; ++u) {
            const uint32_t j = t.ib + 1u + (uint32_t)u * nthr + tid;
            rows[u] = list_row_load(lr, j, j < listCount);
        }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t i = (uint32_t)u * nthr + tid;
        const uint32_t c = i / vprA;
        *reinterpret_cast<f4*>(lds + c * Pp + ((4u * (i % vprA)) ^ lds_swz(c))) = valA[u];
    }
    const BlockOrigin o = origin_of(raw, a.g);
    if (MODE == SCATTER_RANKED_INLINE) {
        uint32_t bits = 0u;
#pragma unroll
        for (int u = 0; u < RANK_ROWS_PER_THREAD; ++u) {
            int n2, bh2, bw2;
            list_row_unpack(rows[u], n2, bh2, bw2);
            if (t.ib + 1u + (uint32_t)u * nthr + tid < listCount) bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        for (uint32_t j = t.ib + 1u + (uint32_t)RANK_ROWS_PER_THREAD * nthr + tid; j < listCount; j += nthr) {
            int n2, bh2, bw2;
            list_row_unpack(list_row_load(lr, j, true), n2, bh2, bw2);
            bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
        if (__ballot(bits != 0u) != 0ull)
            for (int off = 32; off > 0; off >>= 1) bits |= (uint32_t)__shfl_xor((int)bits, off);
        if ((tid & 63u) == 0u) waveBits[tid >> 6] = bits;
    }
    lds_barrier();
    if (!o.valid) return;   // (the whole workgroup)
    const rsrc_t yr = make_rsrc(y + (int64_t)o.n * a.imgFloats, a.imgBytes);
    const uint32_t c0l = (tid & ((1u << G::kLppLog) - 1u)) * 4u;
    uint32_t rbits = 0u;
    if (MODE == SCATTER_RANKED_INLINE) {
        for (uint32_t w = 0; w < (nthr >> 6); ++w) rbits |= waveBits[w];
    }
    uint32_t offs[TILE_LD], pls[TILE_LD];
    nhwc_walk<4, G>(a, t, o, tid, nthr, [&](int u, uint32_t pl, uint32_t off, uint32_t, uint32_t r, uint32_t sc) {
        if (MODE == SCATTER_RANKED_INLINE && ranked_out(rbits, r, sc, a.g)) off = BUF_OOB;
        offs[u] = off;
        pls[u] = pl;
    });
    auto store_items = [&](int u0) {
        f4 w[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const int u = u0 + v;
            w[v] = (f4)(0.f);
            if (offs[u] != BUF_OOB) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t c = c0l + (uint32_t)k;
                    vset(w[v], k, lds[c * Pp + (pls[u] ^ lds_swz(c))]);
                }
            }
        }
#pragma unroll
        for (int v = 0; v < 2; ++v) buf_store<BUF_NT>(yr, offs[u0 + v], w[v]);
    };
    store_items(0);
    // second half: its loads were issued before the first half's stores and complete before them
    if (cB < CT) {
        float* __restrict__ row = lds + cB * Pp;
        if (4 * (int)eB + 4 <= t.Pn) {
            *reinterpret_cast<f4*>(row + ((4u * eB) ^ lds_swz(cB))) = valB;
        } else if (4 * (int)eB < t.Pn) {
            const uint32_t t0 = (uint32_t)(t.Pn - 4);
            row[(t0 + 0) ^ lds_swz(cB)] = valB.x;
            row[(t0 + 1) ^ lds_swz(cB)] = valB.y;
            row[(t0 + 2) ^ lds_swz(cB)] = valB.z;
            row[(t0 + 3) ^ lds_swz(cB)] = valB.w;
        }
    }
    lds_barrier();
    store_items(2);
}

// Geometry policy of the tile moved in two halves (same tile as TileFixed).
template <int R_, int S_, int C_, int P_, int NTHR_>
struct TileFixedHalves : TileFixed<R_, S_, C_, P_, NTHR_> {
    static constexpr bool HALVES = true;
};

template <typename G, typename = void>
struct tile_in_halves { static constexpr bool value = false; };
template <typename G>
struct tile_in_halves<G, decltype((void)G::HALVES)> { static constexpr bool value = G::HALVES; };

template <int VEC, int MODE, typename G>
__global__ __launch_bounds__(512) void k_scatter_planar(const float* __restrict__ x, float* y, const float* ysrc,
                                                        const int16_t* __restrict__ idx, TileArgs a, ColorArgs col)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ uint32_t waveBits[8];  // SCATTER_RANKED_INLINE: one word per wave
    for_each_block_of_workgroup(a, G::tpb(a), [&](uint32_t ib, uint32_t rem) {
        if constexpr (tile_in_halves<G>::value)
            scatter_planar_tile_halves<MODE, G>(x, y, idx, a, lds, waveBits, ib, rem);
        else
            scatter_planar_tile<VEC, MODE, G>(x, y, ysrc, idx, a, col, lds, waveBits, ib, rem);
    });
}

// ---------------------------------------------------------------------------------------------
// overlapping scatter-add without atomics: every output pixel is summed by one owner
// ---------------------------------------------------------------------------------------------
//
// With bstride < bsize a pixel is covered by up to ceil(R/U)*ceil(S/V) blocks.  Hardware fp32 atomics
// resolve that at roughly a tenth of the HBM rate (every contribution is a read-modify-write in L2) and
// in arbitrary order.  Given a little scratch memory the add is done by "pulling" instead:
//   1. k_pull_fill / k_pull_map   an inverse map (n, bh, bw) -> position ib in the active list;
//   2. k_pull_table               per active block, the active blocks that overlap it, sorted by ib;
//   3. k_scatter_pull             the workgroup of block ib walks its own pixels; a pixel belongs to the
//                                 lowest-ib block that covers it, and that owner reads the pixel once,
//                                 adds the contributions of all covering blocks in ascending ib order
//                                 and writes it once.
// Ascending ib is the order in which the sequential CPU functor accumulates (sparse_gather.cc:105-129),
// so the result is bit-identical to it and reproducible from run to run.  A block listed twice cannot
// be represented in the map; k_pull_map notices, and k_scatter_pull then falls back to hardware atomics
// for the whole launch (still correct, to rounding).

constexpr int STRIP_ROWS = 4;    // image rows per workgroup of the kernels that walk the output in row order
constexpr int PULL_STEPS = 3;    // 64-vector steps of one wave, all in flight together (1: 223 us, 2: 228, 3: 211, 4: 232
                                 // on the 16x16-at-stride-8, 256-channel workload; 5 and more run out of registers)
constexpr int PULL_CLASSES = 9;  // 3 row classes x 3 column classes of a block's pixels (see below)
constexpr int PULL_COVER = 4;    // at most 2 x 2 blocks cover a pixel
constexpr int PULL_TABLE_STRIDE = PULL_CLASSES * PULL_COVER * 2;  // ints per block

// With at most 2x2 blocks over a pixel, which blocks cover a pixel of block (bh, bw) depends only on the pixel's
// class: its row is among the first R-U rows (shared with the blocks one step up), among the rows from U on (one
// step down) or in between (this row of blocks only), and the same for columns.  The table holds, per block and
// class, the up to four active blocks that cover pixels of the class, sorted by list position, each as (position,
// packed grid offset): the main kernel needs no search, and the first entry names the pixel's owner.

struct PullArgs {
    Geom g;
    int bhMin, bwMin, nBH, nBW;  // extent of the inverse map: blocks that can touch the image
    int kh1, kw1;                // Kh - 1, Kw - 1
    uint32_t CV, rowV, blockV;   // vectors per pixel, per block row, per block
    uint32_t cpb, units;         // wave-units per block, in total
    FastDiv dCpb, dRow, dCV;
};

__global__ __launch_bounds__(256) void k_pull_fill(int32_t* __restrict__ map, int64_t n, int32_t* __restrict__ dup)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) map[i] = -1;
    if (blockIdx.x == 0 && threadIdx.x == 0) *dup = 0;
}

__device__ __forceinline__ int64_t pull_slot(const PullArgs& a, int n, int bh, int bw)
{
    if ((unsigned)n >= (unsigned)a.g.N) return -1;
    const int ih = bh - a.bhMin, iw = bw - a.bwMin;
    if ((unsigned)ih >= (unsigned)a.nBH || (unsigned)iw >= (unsigned)a.nBW) return -1;
    return ((int64_t)n * a.nBH + ih) * a.nBW + iw;
}

__global__ __launch_bounds__(256) void k_pull_map(const int16_t* __restrict__ idx, int numActive, PullArgs a,
                                                  int32_t* __restrict__ map, int32_t* __restrict__ dup)
{
    const int ib = (int)(blockIdx.x * 256 + threadIdx.x);
    if (ib >= numActive || (a.g.countDev && ib >= *a.g.countDev)) return;
    const int64_t slot = pull_slot(a, idx[(size_t)ib * 3], idx[(size_t)ib * 3 + 1], idx[(size_t)ib * 3 + 2]);
    if (slot < 0) return;  // this block cannot touch the image
    if (atomicCAS(map + slot, -1, ib) != -1) *dup = 1;
}

// Both steps by one workgroup, for maps and lists small enough that one workgroup is done in the time a second
// launch takes to start.
constexpr int BLOCK_MAP_ONE_WG = 16384;  // entries of the map, and rows of the list

__global__ __launch_bounds__(1024) void k_pull_map_small(const int16_t* __restrict__ idx, int numActive, PullArgs a,
                                                         int32_t* __restrict__ map, int mapN, int32_t* __restrict__ dup)
{
    const int tid = (int)threadIdx.x;
    for (int i = tid; i < mapN; i += 1024) map[i] = -1;
    if (tid == 0) *dup = 0;
    __syncthreads();  // (the stores above are complete, and visible to this workgroup's atomics, beyond this point)
    int count = numActive;
    if (a.g.countDev) count = min(count, max(*a.g.countDev, 0));
    for (int ib = tid; ib < count; ib += 1024) {
        const int64_t slot = pull_slot(a, idx[(size_t)ib * 3], idx[(size_t)ib * 3 + 1], idx[(size_t)ib * 3 + 2]);
        if (slot >= 0 && atomicCAS(map + slot, -1, ib) != -1) *dup = 1;
    }
}

// The inverse block map of the list and its flag for repeated rows, in one launch or two.
static void launch_block_map(const int16_t* idx, int numActive, const PullArgs& a, int32_t* map, int64_t mapN,
                             int32_t* dup, hipStream_t stream)
{
    if (mapN <= BLOCK_MAP_ONE_WG && numActive <= BLOCK_MAP_ONE_WG) {
        hipLaunchKernelGGL(k_pull_map_small, dim3(1), dim3(1024), 0, stream, idx, numActive, a, map, (int)mapN, dup);
        return;
    }
    int64_t fillWgs = (mapN + 255) / 256;
    if (fillWgs > 4096) fillWgs = 4096;
    if (fillWgs < 1) fillWgs = 1;
    hipLaunchKernelGGL(k_pull_fill, dim3((unsigned)fillWgs), dim3(256), 0, stream, map, mapN, dup);
    hipLaunchKernelGGL(k_pull_map, dim3((unsigned)((numActive + 255) / 256)), dim3(256), 0, stream, idx, numActive, a, map,
                       dup);
}

// One thread per (block, class): the up to four active blocks that cover the class's pixels, sorted by position.
__global__ __launch_bounds__(256) void k_pull_table(const int16_t* __restrict__ idx, int numActive, PullArgs a,
                                                    const int32_t* __restrict__ map, int32_t* __restrict__ table)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    const int ib = (int)(t / PULL_CLASSES), cls = (int)(t % PULL_CLASSES);
    if (ib >= numActive || (a.g.countDev && ib >= *a.g.countDev)) return;
    const int n = idx[(size_t)ib * 3], bh = idx[(size_t)ib * 3 + 1], bw = idx[(size_t)ib * 3 + 2];
    const int rc = cls / 3, cc = cls - rc * 3;
    // a block one step up covers the first R-U rows only (row class 0), one step down the rows from U on (class 2)
    const int dhLo = rc == 0 ? -a.kh1 : 0, dhHi = rc == 2 ? a.kh1 : 0;
    const int dwLo = cc == 0 ? -a.kw1 : 0, dwHi = cc == 2 ? a.kw1 : 0;
    int ids[PULL_COVER], pks[PULL_COVER];
    int cnt = 0;
    if (pull_slot(a, n, bh, bw) >= 0) {
        for (int dh = dhLo; dh <= dhHi; ++dh)
            for (int dw = dwLo; dw <= dwHi; ++dw) {
                const int64_t slot = pull_slot(a, n, bh + dh, bw + dw);
                const int other = slot >= 0 ? map[slot] : -1;
                if (other < 0) continue;
                int k = cnt++;  // insertion sort
                while (k > 0 && ids[k - 1] > other) {
                    ids[k] = ids[k - 1];
                    pks[k] = pks[k - 1];
                    --k;
                }
                ids[k] = other;
                pks[k] = ((dh & 0xffff) << 16) | (dw & 0xffff);
            }
    }
    typedef int i4 __attribute__((ext_vector_type(4)));
    int e[PULL_COVER * 2];
#pragma unroll
    for (int k = 0; k < PULL_COVER; ++k) {
        e[2 * k] = k < cnt ? ids[k] : -1;
        e[2 * k + 1] = k < cnt ? pks[k] : 0;
    }
    i4* q = reinterpret_cast<i4*>(table + (size_t)ib * PULL_TABLE_STRIDE + cls * (PULL_COVER * 2));
    q[0] = (i4){e[0], e[1], e[2], e[3]};
    q[1] = (i4){e[4], e[5], e[6], e[7]};
}

// sparse_gather.cc:103-130 with add == true on overlapping blocks, NHWC stack.
template <int VEC>
__global__ __launch_bounds__(256) void k_scatter_pull(const float* __restrict__ x, float* __restrict__ y,
                                                      const int16_t* __restrict__ idx, PullArgs a,
                                                      const int32_t* __restrict__ table,
                                                      const int32_t* __restrict__ dup)
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
    if (!o.valid) return;
    const vec* __restrict__ xv = reinterpret_cast<const vec*>(x);
    vec* __restrict__ yv = reinterpret_cast<vec*>(y);

    if (*dup != 0) {
        // the list names a block twice: the map cannot represent it; hardware atomics for the whole launch
        for (int step = 0; step < PULL_STEPS; ++step) {
            const uint32_t e = (chunk * PULL_STEPS + step) * 64 + lane;
            if (e >= a.blockV) break;
            const uint32_t r = fdiv(e, a.dRow);
            const uint32_t j = e - r * a.rowV;
            const uint32_t s = fdiv(j, a.dCV);
            const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
            if ((unsigned)hh >= (unsigned)a.g.H || (unsigned)ww >= (unsigned)a.g.W) continue;
            vec* dst = yv + ((((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * a.CV + (j - s * a.CV));
            commit<VEC, SCATTER_ATOMIC>(dst, ld_stream(xv + ((size_t)ib * a.blockV + e)));
        }
        return;
    }

    // Phase 1: per vector, its class's table entries (two 16-byte loads from a table line that the whole block shares).
    const int32_t* __restrict__ t = table + (size_t)ib * PULL_TABLE_STRIDE;
    typedef int i4 __attribute__((ext_vector_type(4)));
    i4 ent[PULL_STEPS][2];
    uint32_t rr[PULL_STEPS], ss[PULL_STEPS], cvv[PULL_STEPS];
    bool in[PULL_STEPS];
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
        const uint32_t e = (chunk * PULL_STEPS + u) * 64 + lane;
        const uint32_t r = fdiv(e, a.dRow);
        const uint32_t j = e - r * a.rowV;
        const uint32_t s = fdiv(j, a.dCV);
        rr[u] = r;
        ss[u] = s;
        cvv[u] = j - s * a.CV;
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)s;
        in[u] = e < a.blockV && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W;
        const uint32_t rc = (int)r < a.g.R - a.g.U ? 0u : ((int)r >= a.g.U ? 2u : 1u);
        const uint32_t cc = (int)s < a.g.S - a.g.V ? 0u : ((int)s >= a.g.V ? 2u : 1u);
        const i4* q = reinterpret_cast<const i4*>(t + (in[u] ? (rc * 3u + cc) * (PULL_COVER * 2) : 0u));
        ent[u][0] = q[0];
        ent[u][1] = q[1];
    }
    // Phase 2: the owner of a pixel (the first of the blocks that cover it) reads the pixel and every contribution.
    vec acc[PULL_STEPS], val[PULL_STEPS][PULL_COVER];
    bool mine[PULL_STEPS], has[PULL_STEPS][PULL_COVER];
    int64_t dstOff[PULL_STEPS];
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
        const int id[PULL_COVER] = {ent[u][0].x, ent[u][0].z, ent[u][1].x, ent[u][1].z};
        const int pk[PULL_COVER] = {ent[u][0].y, ent[u][0].w, ent[u][1].y, ent[u][1].w};
        mine[u] = in[u] && id[0] == (int)ib;
        const int hh = o.h0 + (int)rr[u], ww = o.w0 + (int)ss[u];
        dstOff[u] = (((int64_t)o.n * a.g.H + hh) * a.g.W + ww) * a.CV + cvv[u];
        // (loads under their own conditions: a load that no lane of the wave needs is skipped, and at one block
        // in four active most pixels have one or two contributions, not four)
        acc[u] = vzero<VEC>();
        if (mine[u]) acc[u] = ld_stream(yv + dstOff[u]);
#pragma unroll
        for (int k = 0; k < PULL_COVER; ++k) {
            has[u][k] = mine[u] && id[k] >= 0;
            const int rs = (int)rr[u] - (int)(int16_t)(pk[k] >> 16) * a.g.U;
            const int cs = (int)ss[u] - (int)(int16_t)(pk[k] & 0xffff) * a.g.V;
            const int64_t off = (int64_t)id[k] * a.blockV + (int64_t)rs * a.rowV + (int64_t)cs * a.CV + cvv[u];
            val[u][k] = vzero<VEC>();
            if (has[u][k]) val[u][k] = ld_stream(xv + off);
        }
    }
#pragma unroll
    for (int u = 0; u < PULL_STEPS; ++u) {
#pragma unroll
        for (int k = 0; k < PULL_COVER; ++k)
            if (has[u][k]) acc[u] = vadd(acc[u], val[u][k]);  // ascending list position: the CPU functor's order
        if (mine[u]) st_stream(yv + dstOff[u], acc[u]);
    }
}

// ---------------------------------------------------------------------------------------------
// flat copy (CopyTensorFunctor, sparse_gather.cc:135-142 / sparse_gather.cu:268-276)
// ---------------------------------------------------------------------------------------------

constexpr int COPY_UNR = 4;  // 16 KB per workgroup; 32 KB per workgroup measured 30 % slower

__global__ __launch_bounds__(256) void k_copy_v4(const f4* __restrict__ src, f4* __restrict__ dst, size_t n4)
{
    const size_t base = (size_t)blockIdx.x * (256 * COPY_UNR) + threadIdx.x;
    f4 v[COPY_UNR];
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        v[u] = (f4)(0.f);
        if (i < n4) v[u] = ld_stream(src + i);
    }
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        if (i < n4) st_stream(dst + i, v[u]);
    }
}

__global__ __launch_bounds__(256) void k_copy_scalar(const float* __restrict__ src, float* __restrict__ dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

// Tile of the planar scatter.  16 KB tiles suit a launch that keeps every compute unit busy for several
// rounds of workgroups; a launch of few workgroups finishes in one or two rounds, where the loads and the stores
// of one round do not overlap much, and does better with 24 KB tiles (800x800x128 tensor, 27x27 blocks:
// 9.08 -> 8.87 us at 58 blocks, 20.6 -> 19.9 us at 156, but 40.8 -> 41.4 us at 312).  The 24 KB tile of that tensor
// is moved in two halves (scatter_planar_tile_halves): 8.37 -> 7.64 us at 58 blocks, no change at 156; at 312 the
// 16 KB tile stays ahead of it (38.5 against 40.0 us).
constexpr int SCATTER_FEW_WGS_PER_CU = 22;

// `share`: the launch does work for one block in `share` only (the passes of an overlapping add).
static bool scatter_tile_args(const Geom& g, int numActive, int vec, TileArgs& a, int& threads, size_t& ldsBytes,
                              unsigned& grid, int share = 1)
{
    if (!make_tile_args(g, numActive, vec, a, threads, ldsBytes, grid, 16 * 1024)) return false;
    if (a.psplit > 1 && a.total / (uint32_t)share < (uint32_t)(SCATTER_FEW_WGS_PER_CU * device_cus())) {
        TileArgs b;
        int bt;
        size_t bl;
        unsigned bg;
        if (make_tile_args(g, numActive, vec, b, bt, bl, bg, 24 * 1024) && b.psplit < a.psplit) {
            a = b;
            threads = bt;
            ldsBytes = bl;
            grid = bg;
        }
    }
    return true;
}

template <typename G>
static bool tile_match(const TileArgs& a, int threads)
{
    return !a.g.forceGeneric && a.g.R * a.g.S == (int)G::kRS && a.g.S == (int)G::S(a) && a.g.C == (int)G::C(a) &&
           a.P == (int)G::P(a) && a.psplit == (int)G::kPsplit && threads == (int)G::nthr(a) && a.Pp == (int)G::kPp &&
           a.Ct == (int)G::Ct(a) && a.lppLog == (int)G::kLppLog && a.vpr == G::kVpr && a.tpb == G::tpb(a);
}

template <int VEC, int MODE, typename G>
static bool launch_fixed_scatter_one(const float* x, float* y, const float* ysrc, const int16_t* idx, const TileArgs& a,
                                     int threads, size_t lds, int numActive, const ColorArgs& aux, hipStream_t stream)
{
    if (!tile_match<G>(a, threads)) return false;
    hipLaunchKernelGGL((k_scatter_planar<VEC, MODE, G>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g), dim3(threads),
                       lds, stream, x, y, ysrc, idx, a, aux);
    return true;
}

template <int VEC, int MODE>
static bool launch_fixed_scatter(const float* x, float* y, const float* ysrc, const int16_t* idx, const TileArgs& a,
                                 int threads, size_t lds, int numActive, const ColorArgs& aux, hipStream_t stream)
{
    if constexpr (VEC == 4 && (MODE == SCATTER_ASSIGN || MODE == SCATTER_ADD || MODE == SCATTER_RANKED ||
                               MODE == SCATTER_RANKED_INLINE || MODE == SCATTER_COLOR || MODE == SCATTER_SUM)) {
        // 27x27 blocks of 128 channels with 16 KB and 24 KB tiles; 16x16 blocks of 64 channels
        if constexpr (MODE == SCATTER_ASSIGN || MODE == SCATTER_RANKED_INLINE) {
            // (the 24 KB tile is what launches of few workgroups take: moved in two halves, see above)
            if (y == ysrc &&
                launch_fixed_scatter_one<VEC, MODE, TileFixedHalves<27, 27, 128, 184, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                             numActive, aux, stream))
                return true;
        }
        return launch_fixed_scatter_one<VEC, MODE, TileFixed<27, 27, 128, 124, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                      numActive, aux, stream) ||
               launch_fixed_scatter_one<VEC, MODE, TileFixed<27, 27, 128, 184, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                      numActive, aux, stream) ||
               launch_fixed_scatter_one<VEC, MODE, TileFixed<16, 16, 64, 128, 512>>(x, y, ysrc, idx, a, threads, lds,
                                                                                     numActive, aux, stream);
    }
    return false;
}

// The scatter's half of the tile_choice test hook (kind 2): same `out` fields.
int scatter_tile_choice(const Geom& g, int numActive, int vec, int32_t* out)
{
    int threads = 0;
    size_t lds = 0;
    unsigned grid = 0;
    const int RS = g.R * g.S;
    TileArgs a;
    if (RS < 4 || !scatter_tile_args(g, numActive, vec, a, threads, lds, grid)) return 0;
    const int lpp = 1 << a.lppLog;
    out[0] = threads; out[1] = (int32_t)lds; out[2] = a.P; out[3] = a.Pp; out[4] = a.psplit; out[5] = a.Ct;
    out[6] = a.cchunks;
    // per thread: NHWC items and planar slots of a full tile
    const int items = (a.P * lpp + threads - 1) / threads;
    const int slots = (int)((a.Ct * a.vpr + threads - 1) / threads);
    out[7] = items > slots ? items : slots;
    out[8] = TILE_LD;
    out[9] = RS - (a.psplit - 1) * a.P;
    out[10] = vec == 4 &&
              (tile_match<TileFixed<27, 27, 128, 124, 512>>(a, threads) || tile_match<TileFixed<27, 27, 128, 184, 512>>(a, threads) ||
               tile_match<TileFixed<16, 16, 64, 128, 512>>(a, threads));
    return 1;
}

// `ysrc` is what an add reads: y itself for the in-place op, the base tensor when y is being built as
// "copy of the base + scatter" without copying the covered pixels first.
template <int VEC, int MODE>
static void scatter_dispatch(const float* x, float* y, const float* ysrc, const int16_t* idx, const Geom& g,
                             int numActive, bool transpose, hipStream_t stream, hipError_t& err,
                             const int32_t* order = nullptr)
{
    // `order`: the owner map (SCATTER_OWNED) or the rank table (SCATTER_RANKED)
    const ColorArgs aux{1, 1, 0, nullptr, MODE == SCATTER_OWNED ? order : nullptr,
                        MODE == SCATTER_RANKED ? order : nullptr, 0, nullptr, 0, 0, 0, 0, nullptr, nullptr, 0};
    const int32_t* owner = order;
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) { err = hipErrorInvalidValue; return; }
        if (nhwc_fits_buffers(g))
            hipLaunchKernelGGL((k_scatter_nhwc<VEC, MODE>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y, ysrc,
                               idx, a, aux);
        else
            hipLaunchKernelGGL((k_scatter_nhwc_wide<VEC, MODE>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y,
                               ysrc, idx, a, aux);
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        // 16 KB tiles: 42.6 us against 43.9 us with 32 KB tiles on the same workload
        if ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, VEC, a, threads, lds, grid)) {
            const int64_t total = (int64_t)numActive * g.C * g.R * g.S;
            const int64_t wgs = (total + 255) / 256;
            hipLaunchKernelGGL((k_planar_small<MODE, false>), dim3((unsigned)(wgs > 65536 ? 65536 : wgs)), dim3(256),
                               0, stream, x, y, ysrc, idx, g, total, owner);
            return;
        }
        if (launch_fixed_scatter<VEC, MODE>(x, y, ysrc, idx, a, threads, lds, numActive, aux, stream)) return;
        hipLaunchKernelGGL((k_scatter_planar<VEC, MODE, TileRt>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g),
                           dim3(threads), lds, stream, x, y, ysrc, idx, a, aux);
    }
}

template <int VEC>
static void scatter_mode(const float* x, float* y, const float* ysrc, const int16_t* idx, const Geom& g, int numActive,
                         bool transpose, ScatterMode mode, hipStream_t stream, hipError_t& err, const int32_t* order,
                         bool ranked, bool rankInline)
{
    if (mode == SCATTER_ASSIGN && rankInline)
        scatter_dispatch<VEC, SCATTER_RANKED_INLINE>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
    else if (mode == SCATTER_ASSIGN && order && ranked)
        scatter_dispatch<VEC, SCATTER_RANKED>(x, y, ysrc, idx, g, numActive, transpose, stream, err, order);
    else if (mode == SCATTER_ASSIGN && order)
        scatter_dispatch<VEC, SCATTER_OWNED>(x, y, ysrc, idx, g, numActive, transpose, stream, err, order);
    else if (mode == SCATTER_ASSIGN)
        scatter_dispatch<VEC, SCATTER_ASSIGN>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
    else if (mode == SCATTER_ADD)
        scatter_dispatch<VEC, SCATTER_ADD>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
    else
        scatter_dispatch<VEC, SCATTER_ATOMIC>(x, y, ysrc, idx, g, numActive, transpose, stream, err);
}

static hipError_t scatter_from(const float* x, float* y, const float* ysrc, const int16_t* idx, int numActive,
                               const Geom& g, bool transpose, ScatterMode mode, hipStream_t stream,
                               const int32_t* order = nullptr, bool ranked = false, bool rankInline = false)
{
    if (numActive == 0) return hipSuccess;
    hipError_t err = hipSuccess;
    int vec = pick_vec(g, y, transpose ? nullptr : x);
    const int vsrc = pick_vec(g, ysrc, nullptr);
    if (vsrc < vec) vec = vsrc;
    if (vec == 4) scatter_mode<4>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked, rankInline);
    else if (vec == 2) scatter_mode<2>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked, rankInline);
    else scatter_mode<1>(x, y, ysrc, idx, g, numActive, transpose, mode, stream, err, order, ranked, rankInline);
    if (err != hipSuccess) return err;
    return hipGetLastError();
}

hipError_t launch_scatter(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                          bool transpose, ScatterMode mode, hipStream_t stream)
{
    return scatter_from(x, y, y, idx, numActive, g, transpose, mode, stream);
}

// Extent of the inverse block map (blocks that can touch the image); false when it cannot be built.
static bool make_map_args(const Geom& g, PullArgs& a, int64_t& mapN)
{
    a.g = g;
    // oh + bh*U + R - 1 >= 0 and oh + bh*U <= H - 1 (floor divisions)
    auto floordiv = [](int64_t p, int64_t q) { return p >= 0 ? p / q : -((-p + q - 1) / q); };
    int64_t bhMin = -floordiv((int64_t)g.R - 1 + g.oh, g.U), bhMax = floordiv((int64_t)g.H - 1 - g.oh, g.U);
    int64_t bwMin = -floordiv((int64_t)g.S - 1 + g.ow, g.V), bwMax = floordiv((int64_t)g.W - 1 - g.ow, g.V);
    if (bhMin < -32768) bhMin = -32768;
    if (bwMin < -32768) bwMin = -32768;
    if (bhMax > 32767) bhMax = 32767;
    if (bwMax > 32767) bwMax = 32767;
    if (bhMax < bhMin || bwMax < bwMin) return false;
    a.bhMin = (int)bhMin; a.bwMin = (int)bwMin;
    a.nBH = (int)(bhMax - bhMin + 1); a.nBW = (int)(bwMax - bwMin + 1);
    mapN = (int64_t)g.N * a.nBH * a.nBW;
    return mapN < (1ll << 31);
}

// Geometry of the pull scatter; false when the method does not apply.
static bool make_pull_args(const Geom& g, int numActive, int vec, PullArgs& a, int64_t& mapN)
{
    const int Kh = (g.R + g.U - 1) / g.U, Kw = (g.S + g.V - 1) / g.V;
    if (Kh > 2 || Kw > 2) return false;  // at most 2x2 blocks over a pixel: neighbours one step away only
    if (!make_map_args(g, a, mapN)) return false;
    a.kh1 = Kh - 1;
    a.kw1 = Kw - 1;
    const uint64_t rowV = (uint64_t)g.S * g.C / vec, blockV = rowV * g.R;
    if (blockV >= (1ull << 31)) return false;
    a.CV = (uint32_t)(g.C / vec);
    a.rowV = (uint32_t)rowV;
    a.blockV = (uint32_t)blockV;
    a.cpb = (uint32_t)((blockV + 64 * PULL_STEPS - 1) / (64 * PULL_STEPS));
    const uint64_t units = (uint64_t)numActive * a.cpb;
    if (units >= (1ull << 31)) return false;
    a.units = (uint32_t)units;
    a.dCpb = make_fastdiv(a.cpb);
    a.dRow = make_fastdiv(a.rowV);
    a.dCV = make_fastdiv(a.CV);
    return true;
}

size_t scatter_pull_workspace_bytes(const Geom& g, int numActive)
{
    PullArgs a;
    int64_t mapN = 0;
    if (numActive <= 0 || !make_pull_args(g, numActive, 1, a, mapN)) return 0;
    return (size_t)mapN * 4 + 16 + 16 + (size_t)numActive * PULL_TABLE_STRIDE * 4;  // map, flag, alignment, table
}

hipError_t launch_scatter_pull(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                               void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (numActive == 0) { done = true; return hipSuccess; }
    PullArgs a;
    int64_t mapN = 0;
    const int vec = pick_vec(g, y, x);
    if (!workspace || !make_pull_args(g, numActive, vec, a, mapN)) return hipSuccess;
    if (workspaceBytes < scatter_pull_workspace_bytes(g, numActive) || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return hipSuccess;
    int32_t* map = static_cast<int32_t*>(workspace);
    int32_t* dup = map + mapN;
    // the table is read with 16-byte loads
    int32_t* table = reinterpret_cast<int32_t*>((reinterpret_cast<uintptr_t>(dup + 4) + 15) & ~(uintptr_t)15);
    launch_block_map(idx, numActive, a, map, mapN, dup, stream);
    hipLaunchKernelGGL(k_pull_table, dim3((unsigned)(((int64_t)numActive * PULL_CLASSES + 255) / 256)), dim3(256), 0,
                       stream, idx, numActive, a, map, table);
    const unsigned wgs = (a.units + 3) / 4;
    if (vec == 4) hipLaunchKernelGGL(k_scatter_pull<4>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    else if (vec == 2) hipLaunchKernelGGL(k_scatter_pull<2>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    else hipLaunchKernelGGL(k_scatter_pull<1>, dim3(wgs), dim3(256), 0, stream, x, y, idx, a, table, dup);
    done = true;
    return hipGetLastError();
}

// ---- scatter-add in passes ------------------------------------------------------------------

constexpr int COLOR_MAX_PASSES = 16;
constexpr int COLOR_SORT_MAX_BLOCKS = 1 << 17;  // lists that one workgroup sorts by pass in a few microseconds

// The list sorted by colour pass (see ColorArgs::perm).  One workgroup: counts per pass, offsets, then every row's
// position goes to the next free slot of its pass (the order inside a pass does not matter: its blocks do not
// overlap).  When the list names a block twice the passes fall back to hardware atomics, all in pass 0.
__global__ __launch_bounds__(1024) void k_color_sort(const int16_t* __restrict__ idx, int numActive, Geom g, int kh, int kw,
                                                     const int32_t* __restrict__ dup, int32_t* __restrict__ counts,
                                                     int32_t* __restrict__ perm, int permStride)
{
    __shared__ int next[COLOR_MAX_PASSES];
    const int tid = (int)threadIdx.x;
    int count = numActive;
    if (g.countDev) count = min(count, max(*g.countDev, 0));
    const bool all0 = *dup != 0;
    if (tid < COLOR_MAX_PASSES) next[tid] = 0;
    __syncthreads();
    for (int i = tid; i < count; i += 1024) {
        int p = 0;
        if (!all0) {
            int mh = idx[(size_t)i * 3 + 1] % kh, mw = idx[(size_t)i * 3 + 2] % kw;
            if (mh < 0) mh += kh;
            if (mw < 0) mw += kw;
            p = mh * kw + mw;
        }
        perm[(int64_t)p * permStride + atomicAdd(&next[p], 1)] = i;
    }
    __syncthreads();
    if (tid < COLOR_MAX_PASSES) counts[tid] = next[tid];
}

size_t scatter_color_workspace_bytes(const Geom& g, int numActive)
{
    PullArgs a;
    int64_t mapN = 0;
    const int64_t Kh = ((int64_t)g.R + g.U - 1) / g.U, Kw = ((int64_t)g.S + g.V - 1) / g.V;
    if (numActive <= 0 || Kh * Kw > COLOR_MAX_PASSES || !make_map_args(g, a, mapN)) return 0;
    // the block map, the duplicate flag, the passes' counts, one list of the capacity of the whole list per pass
    const size_t perm = numActive <= COLOR_SORT_MAX_BLOCKS ? (size_t)numActive * (size_t)(Kh * Kw) * 4 : 0;
    return (size_t)mapN * 4 + 16 + COLOR_MAX_PASSES * 4 + perm;
}

template <int VEC>
static bool color_passes(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive, bool transpose,
                         ColorArgs col, int passes, hipStream_t stream)
{
    if (!transpose) {
        NhwcArgs a;
        if (!make_nhwc_args(g, numActive, VEC, a)) return false;
        const bool buf = nhwc_fits_buffers(g);
        for (col.pass = 0; col.pass < passes; ++col.pass) {
            if (buf)
                hipLaunchKernelGGL((k_scatter_nhwc<VEC, SCATTER_COLOR>), dim3((a.units + 3) / 4), dim3(256), 0, stream,
                                   x, y, (const float*)y, idx, a, col);
            else
                hipLaunchKernelGGL((k_scatter_nhwc_wide<VEC, SCATTER_COLOR>), dim3((a.units + 3) / 4), dim3(256), 0,
                                   stream, x, y, (const float*)y, idx, a, col);
        }
    } else {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        if ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, VEC, a, threads, lds, grid, passes)) return false;
        for (col.pass = 0; col.pass < passes; ++col.pass) {
            if (launch_fixed_scatter<VEC, SCATTER_COLOR>(x, y, y, idx, a, threads, lds, numActive, col, stream)) continue;
            hipLaunchKernelGGL((k_scatter_planar<VEC, SCATTER_COLOR, TileRt>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g),
                               dim3(threads), lds, stream, x, y, (const float*)y, idx, a, col);
        }
    }
    return true;
}

// ---- zero-filling for "scatter-add onto zeros" (the gradient of sparse_gather) ------------------------------

__global__ __launch_bounds__(256) void k_fill_zero(f4* __restrict__ y, size_t n4, float* __restrict__ tail, int nTail)
{
    const size_t base = (size_t)blockIdx.x * (256 * COPY_UNR) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < COPY_UNR; ++u) {
        const size_t i = base + (size_t)u * 256;
        if (i < n4) st_stream(y + i, (f4)(0.f));
    }
    if (blockIdx.x == 0 && (int)threadIdx.x < nTail) tail[threadIdx.x] = 0.f;
}

static void launch_fill_zero(float* y, size_t count, hipStream_t stream)
{
    // (16-byte stores from the first aligned float on; the few floats before and after it one by one)
    const uintptr_t p = reinterpret_cast<uintptr_t>(y);
    size_t head = ((16 - (p & 15)) & 15) / 4;
    if (head > count) head = count;
    const size_t n4 = (count - head) / 4, rest = count - head - n4 * 4;
    const size_t per = 256 * COPY_UNR;
    if (n4) hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)((n4 + per - 1) / per)), dim3(256), 0, stream,
                               reinterpret_cast<f4*>(y + head), n4, y + head + n4 * 4, (int)rest);
    else if (rest) hipLaunchKernelGGL(k_fill_zero, dim3(1), dim3(256), 0, stream, reinterpret_cast<f4*>(y + head), (size_t)0,
                                      y + head, (int)rest);
    if (head) hipLaunchKernelGGL(k_fill_zero, dim3(1), dim3(256), 0, stream, reinterpret_cast<f4*>(y), (size_t)0, y, (int)head);
}

// Zeros for the pixels that no active block covers (at most 2x2 blocks over a pixel); the colour passes that follow
// write every covered pixel themselves (ColorArgs::first).  Strips of 4 image rows of one row of stride cells, 256
// channel vectors wide, as in k_scatter_strip; a pixel of cell (bh, bw) can be covered by the blocks (bh, bw),
// (bh, bw-1), (bh-1, bw) and (bh-1, bw-1).  When the list names a block twice the passes fall back to hardware
// atomics, which need zeros everywhere: then every pixel is cleared.
struct FillArgs {
    Geom g;
    int bhMin, bwMin, nBH, nBW;  // extent of the inverse block map
    int cellH0, cellW0;          // first row / column of stride cells that touches the image
    int nBands;                  // rows of cells that touch the image
    uint32_t kPerBand, CV, PX, nPC, imgBytes;
    int64_t imgFloats;
    FastDiv dCV, dV, dK, dPC, dBands;
};

__device__ __forceinline__ bool fill_block_active(const FillArgs& a, const int32_t* __restrict__ map, uint32_t n, int bh,
                                                  int bw)
{
    const int ih = bh - a.bhMin, iw = bw - a.bwMin;
    if ((unsigned)ih >= (unsigned)a.nBH || (unsigned)iw >= (unsigned)a.nBW) return false;
    return map[((int64_t)n * a.nBH + ih) * a.nBW + iw] >= 0;
}

template <int VEC>
__global__ __launch_bounds__(256) void k_fill_uncovered(float* __restrict__ y, const int32_t* __restrict__ map,
                                                        const int32_t* __restrict__ dup, FillArgs a)
{
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    const uint32_t tid = threadIdx.x;
    uint32_t l = blockIdx.x;
    uint32_t t = fdiv(l, a.dPC);
    const uint32_t pc = (uint32_t)__builtin_amdgcn_readfirstlane((int)(l - t * a.nPC));
    l = t; t = fdiv(l, a.dK);
    const int r0 = __builtin_amdgcn_readfirstlane((int)(l - t * a.kPerBand)) * STRIP_ROWS;
    l = t; t = fdiv(l, a.dBands);
    const int bh = __builtin_amdgcn_readfirstlane((int)(l - t * (uint32_t)a.nBands)) + a.cellH0;
    const uint32_t n = (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
    const int hTop = a.g.oh + bh * a.g.U + r0;

    const uint32_t wl = fdiv(tid, a.dCV), cv = tid - wl * a.CV;
    const uint32_t w = pc * a.PX + wl;
    const bool live = wl < a.PX && w < (uint32_t)a.g.W;
    const uint32_t dw = w - (uint32_t)(a.g.ow + a.cellW0 * a.g.V);
    const uint32_t iw = fdiv(dw, a.dV);
    const int sc = (int)(dw - iw * (uint32_t)a.g.V), bw = (int)iw + a.cellW0;

    const bool all = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(dup)) != 0;
    // the block of the pixel's own cell and of the cell to its left, in this row of cells and in the one above
    const bool left = sc + a.g.V < a.g.S, here = sc < a.g.S;
    bool cur = false, up = false;
    if (live && !all) {
        cur = (here && fill_block_active(a, map, n, bh, bw)) || (left && fill_block_active(a, map, n, bh, bw - 1));
        if (r0 + a.g.U < a.g.R)  // (some row of the strip lies under the blocks of the row of cells above)
            up = (here && fill_block_active(a, map, n, bh - 1, bw)) || (left && fill_block_active(a, map, n, bh - 1, bw - 1));
    }
    const rsrc_t yr = make_rsrc(y + (int64_t)n * a.imgFloats, a.imgBytes);
#pragma unroll
    for (int u = 0; u < STRIP_ROWS; ++u) {
        const int r = r0 + u, h = hTop + u;
        const bool covered = (cur && r < a.g.R) || (up && r + a.g.U < a.g.R);
        const bool write = live && r < a.g.U && (unsigned)h < (unsigned)a.g.H && !covered;
        buf_store<BUF_NT>(yr, write ? (((uint32_t)h * (uint32_t)a.g.W + w) * a.CV + cv) * (uint32_t)(VEC * 4) : BUF_OOB,
                          vzero<VEC>());
    }
}

static bool make_fill_args(const Geom& g, int vec, const PullArgs& pa, FillArgs& a, unsigned& grid)
{
    if (g.R > 2 * (int64_t)g.U || g.S > 2 * (int64_t)g.V) return false;  // at most 2x2 blocks over a pixel
    a.g = g;
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (a.imgFloats >= (1ll << 30)) return false;
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    a.bhMin = pa.bhMin; a.bwMin = pa.bwMin; a.nBH = pa.nBH; a.nBW = pa.nBW;
    auto floordiv = [](int64_t p, int64_t q) { return p >= 0 ? p / q : -((-p + q - 1) / q); };
    const int64_t h0 = floordiv(-(int64_t)g.oh, g.U), h1 = floordiv((int64_t)g.H - 1 - g.oh, g.U);
    const int64_t w0 = floordiv(-(int64_t)g.ow, g.V);
    if (h0 < -(1ll << 30) || h1 > (1ll << 30) || w0 < -(1ll << 30) || w0 > (1ll << 30)) return false;
    a.cellH0 = (int)h0; a.cellW0 = (int)w0;
    a.nBands = (int)(h1 - h0 + 1);
    a.kPerBand = (uint32_t)((g.U + STRIP_ROWS - 1) / STRIP_ROWS);
    a.CV = (uint32_t)(g.C / vec);
    if (a.CV > 256u) return false;
    a.PX = 256u / a.CV;
    a.nPC = ((uint32_t)g.W + a.PX - 1u) / a.PX;
    const int64_t tiles = (int64_t)g.N * a.nBands * a.kPerBand * a.nPC;
    if (tiles >= (1ll << 31)) return false;
    grid = (unsigned)tiles;
    a.dCV = make_fastdiv(a.CV);
    a.dV = make_fastdiv((uint32_t)g.V);
    a.dK = make_fastdiv(a.kPerBand);
    a.dPC = make_fastdiv(a.nPC);
    a.dBands = make_fastdiv((uint32_t)a.nBands);
    return true;
}

// ontoZeros: y holds nothing yet and the result is "zeros, plus the blocks" (the gradient of sparse_gather,
// sparse_conv_lib.py:80-107): the zeros are written here, only where they are needed when the geometry allows.
hipError_t launch_scatter_colored(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                  bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream,
                                  bool& done, bool ontoZeros)
{
    done = false;
    if (numActive == 0) {
        if (ontoZeros) launch_fill_zero(y, (size_t)g.N * g.H * g.W * g.C, stream);
        done = true;
        return hipGetLastError();
    }
    const size_t need = scatter_color_workspace_bytes(g, numActive);
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3))
        return hipSuccess;
    PullArgs pa;
    int64_t mapN = 0;
    if (!make_map_args(g, pa, mapN)) return hipSuccess;
    ColorArgs col;
    col.kh = (g.R + g.U - 1) / g.U;
    col.kw = (g.S + g.V - 1) / g.V;
    col.pass = 0;
    col.owner = nullptr;
    col.rank = nullptr;
    int32_t* map = static_cast<int32_t*>(workspace);
    int32_t* dup = map + mapN;
    col.dup = dup;
    col.first = 0;
    col.map = map;
    col.bhMin = pa.bhMin; col.bwMin = pa.bwMin; col.nBH = pa.nBH; col.nBW = pa.nBW;
    int32_t* counts = dup + 4;
    int32_t* perm = counts + COLOR_MAX_PASSES;
    const bool sorted = numActive <= COLOR_SORT_MAX_BLOCKS && col.kh * col.kw > 1;
    col.perm = sorted ? perm : nullptr;
    col.counts = sorted ? counts : nullptr;
    col.permStride = numActive;
    // geometry checks first: nothing is launched unless the passes can run
    const int vec = pick_vec(g, y, transpose ? nullptr : x);
    {
        NhwcArgs na;
        TileArgs ta;
        int threads;
        size_t lds;
        unsigned grid;
        if (!transpose ? !make_nhwc_args(g, numActive, vec, na)
                       : ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, vec, ta, threads, lds, grid, col.kh * col.kw)))
            return hipSuccess;
    }
    FillArgs fa;
    unsigned fillGrid = 0;
    // (the kernels that read only what an earlier pass wrote are the buffer-addressed ones)
    const bool partial = ontoZeros && (transpose || nhwc_fits_buffers(g)) && make_fill_args(g, vec, pa, fa, fillGrid);
    launch_block_map(idx, numActive, pa, map, mapN, dup, stream);
    if (sorted)
        hipLaunchKernelGGL(k_color_sort, dim3(1), dim3(1024), 0, stream, idx, numActive, g, col.kh, col.kw,
                           (const int32_t*)dup, counts, perm, numActive);
    if (partial) {
        col.first = 1;
        const int32_t* cmap = map;
        const int32_t* cdup = dup;
        if (vec == 4) hipLaunchKernelGGL(k_fill_uncovered<4>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
        else if (vec == 2) hipLaunchKernelGGL(k_fill_uncovered<2>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
        else hipLaunchKernelGGL(k_fill_uncovered<1>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
    } else if (ontoZeros) {
        launch_fill_zero(y, (size_t)g.N * g.H * g.W * g.C, stream);
    }
    const int passes = col.kh * col.kw;
    if (vec == 4) color_passes<4>(x, y, idx, g, numActive, transpose, col, passes, stream);
    else if (vec == 2) color_passes<2>(x, y, idx, g, numActive, transpose, col, passes, stream);
    else color_passes<1>(x, y, idx, g, numActive, transpose, col, passes, stream);
    done = true;
    return hipGetLastError();
}

// Fills y with zeros (for callers of the zero-based scatter-add that take another path).
hipError_t launch_zero(float* y, size_t count, hipStream_t stream)
{
    launch_fill_zero(y, count, stream);
    return hipGetLastError();
}

// ---- "copy of the base + scatter" in one pass -------------------------------------------------------
//
// sparse_scatter (not the in-place op) returns a fresh tensor: the base, with the blocks written or added on
// top (sparse_gather.cc:338-346 copies the whole base, then scatters).  Copy-then-scatter moves every covered
// pixel twice more than needed.
//
// Blocks that do not overlap (bstride >= bsize on both axes, which add without atomics requires anyway,
// sparse_gather.cc:322-326): the plane divides into cells of bstride[0] x bstride[1] pixels, cell (bh, bw)
// holds block (bh, bw) in its first bsize rows and columns, and a pixel can only be written by the block of its
// own cell.  With an inverse map "cell -> list position" (k_pull_fill, k_cell_map) ONE streaming kernel
// (k_scatter_strip) walks the output in row order: a workgroup takes a strip of 4 image rows of one row of
// cells, 256 channel vectors wide; a lane looks its cell up once, reads the base where the result needs it (all
// of it for an add, the uncovered pixels for a plain write), reads the block stack where a block covers the
// pixel, and writes the output once.  No flag bytes, no second pass over the covered pixels.
//
// Overlapping plain writes keep the owner map of the ordered scatter as their coverage record (k_copy_uncovered,
// then the ordinary scatter kernels, which read the base where they add).

struct StripArgs {
    Geom g;
    int bhMin, bwMin, nBH, nBW;  // cells that touch the image: bh in [bhMin, bhMin + nBH), likewise bw
    uint32_t kPerBand;           // strips per row of cells: ceil(U / STRIP_ROWS)
    uint32_t CV;                 // channel vectors per pixel
    uint32_t CVT;                // channel vectors per pixel that one strip moves (a chunk of the channels)
    uint32_t CT;                 // the same in floats
    uint32_t nCC;                // channel chunks: ceil(CV / CVT)
    uint32_t PX;                 // pixels per strip: 256 / CVT
    uint32_t imgBytes;
    int64_t imgFloats;
    uint32_t swzMask;            // LDS staging of a planar stack: see strip_lds_index
    uint32_t nPC;                // pixel chunks per image row: ceil(W / PX)
    uint32_t tiles;              // strips in all: N * nBH * kPerBand * nPC * nCC
    uint32_t S4;                 // planar stack: 16-byte slots per block row, S / 4
    uint32_t cellsPerStrip;      // planar stack: PX / V
    FastDiv dCVT, dV, dK, dCC, dPC, dBH, dS4, dCT;
};


// Cell of block (n, bh, bw) in the map, or -1 when the block cannot touch the image.
__device__ __forceinline__ int64_t cell_slot(const StripArgs& a, int n, int bh, int bw)
{
    if ((unsigned)n >= (unsigned)a.g.N) return -1;
    const int ih = bh - a.bhMin, iw = bw - a.bwMin;
    if ((unsigned)ih >= (unsigned)a.nBH || (unsigned)iw >= (unsigned)a.nBW) return -1;
    return ((int64_t)n * a.nBH + ih) * a.nBW + iw;
}

// One thread per list row: the row's position goes into its cell.  A cell named by several rows keeps them as a
// linked list (the map holds the row that arrived last, chain[row] the one it displaced) and raises `dup`; the
// main kernel then walks the lists, so that a plain write still takes the row listed last and an add still sums
// in list order, as the sequential CPU functor does (sparse_gather.cc:105-129).
__global__ __launch_bounds__(256) void k_cell_map(const int16_t* __restrict__ idx, int numActive, StripArgs a,
                                                   int32_t* __restrict__ map, int32_t* __restrict__ chain,
                                                   int32_t* __restrict__ dup)
{
    const int ib = (int)(blockIdx.x * 256 + threadIdx.x);
    if (ib >= numActive || (a.g.countDev && ib >= *a.g.countDev)) return;
    const int64_t slot = cell_slot(a, idx[(size_t)ib * 3], idx[(size_t)ib * 3 + 1], idx[(size_t)ib * 3 + 2]);
    int32_t prev = -1;
    if (slot >= 0) {
        prev = atomicExch(map + slot, ib);
        if (prev >= 0) *dup = 1;
    }
    chain[ib] = prev;
}

// The cleared map and the list's rows in it by one workgroup, for maps and lists small enough that one workgroup
// is done in the time a second launch takes to start.
__global__ __launch_bounds__(1024) void k_cell_map_small(const int16_t* __restrict__ idx, int numActive, StripArgs a,
                                                          int32_t* __restrict__ map, int mapN,
                                                          int32_t* __restrict__ chain, int32_t* __restrict__ dup)
{
    const int tid = (int)threadIdx.x;
    for (int i = tid; i < mapN; i += 1024) map[i] = -1;
    if (tid == 0) *dup = 0;
    __syncthreads();  // (the stores above are complete, and visible to this workgroup's atomics, beyond this point)
    int count = numActive;
    if (a.g.countDev) count = min(count, max(*a.g.countDev, 0));
    for (int ib = tid; ib < count; ib += 1024) {
        const int64_t slot = cell_slot(a, idx[(size_t)ib * 3], idx[(size_t)ib * 3 + 1], idx[(size_t)ib * 3 + 2]);
        int32_t prev = -1;
        if (slot >= 0) {
            prev = atomicExch(map + slot, ib);
            if (prev >= 0) *dup = 1;
        }
        chain[ib] = prev;
    }
}

// VEC channels of block ib at block pixel (r, s), channel vector cv.
template <int VEC, bool PLANAR>
__device__ __forceinline__ typename Vec<VEC>::type strip_stack_load(const float* __restrict__ x, int ib, int r,
                                                                    uint32_t s, uint32_t cv, const StripArgs& a)
{
    typedef typename Vec<VEC>::type vec;
    if (!PLANAR) {
        const int64_t e = (((int64_t)ib * a.g.R + r) * a.g.S + s) * a.CV + cv;
        return ld_stream(reinterpret_cast<const vec*>(x) + e);
    }
    vec v = vzero<VEC>();
    const int64_t plane = (int64_t)a.g.R * a.g.S;
    const float* __restrict__ p = x + ((int64_t)ib * a.g.C + cv * VEC) * plane + (int64_t)r * a.g.S + s;
#pragma unroll
    for (int k = 0; k < VEC; ++k) vset(v, k, ld_stream(p + k * plane));
    return v;
}

// Planar stack [blocks, C, R, S]: the strip's part of it goes through LDS, for geometries in which the strips line
// up with the cells and the planar rows with 16-byte vectors (bsize[1], bstride[1] multiples of 4, bstride[1]
// dividing the strip's width, boffset[1] a multiple of bstride[1]: the usual output geometry of a convolution over
// the gathered blocks).  LDS holds the strip as [row][pixel][channel of the chunk], the order in which the NHWC side
// consumes it (one 16-byte read per lane).  The loading side deals 16-byte slots to the threads in the stack's own
// memory order (4 pixels of a planar row, then the strip's rows of that channel, then the channels, then the
// cells), so that a wave reads long contiguous pieces: a whole block when the plane is 4x4.  Channels are
// XOR-swizzled in units of 4 by the pixel group's number, which spreads the transposing writes over the banks and
// keeps every pixel's 4-channel vectors whole.
__device__ __forceinline__ uint32_t strip_lds_index(const StripArgs& a, uint32_t u, uint32_t px, uint32_t c)
{
    return (u * a.PX + px) * a.CT + (c ^ (((px >> 2) & a.swzMask) << 2));  // c: channel inside the strip's chunk
}

constexpr int STRIP_SLOTS = 4;  // 16-byte slots per thread: 256 threads x 4 x 16 B = the strip's 16 KB

__device__ __forceinline__ void strip_stage_planar(const float* __restrict__ x, const int32_t* __restrict__ mapRow,
                                                   const StripArgs& a, float* lds, uint32_t pc, uint32_t c0, int r0,
                                                   int hTop)
{
    const uint32_t C = (uint32_t)a.g.C, S = (uint32_t)a.g.S;
    const int64_t plane = (int64_t)a.g.R * a.g.S;
    const uint32_t iw0 = pc * a.cellsPerStrip;  // the strip's first cell
    int ib[STRIP_SLOTS];
    uint32_t cl[STRIP_SLOTS], uu[STRIP_SLOTS], px[STRIP_SLOTS], col[STRIP_SLOTS];
    bool use[STRIP_SLOTS];
#pragma unroll
    for (int k = 0; k < STRIP_SLOTS; ++k) {
        const uint32_t p = threadIdx.x + (uint32_t)k * 256u;
        // p = ((cell * CT + cl) * 4 + u) * S4 + q
        uint32_t t = fdiv(p, a.dS4);
        const uint32_t q = p - t * a.S4;
        uu[k] = t & 3u;
        t >>= 2;
        const uint32_t cell = fdiv(t, a.dCT);
        cl[k] = t - cell * a.CT;
        col[k] = 4u * q;
        px[k] = cell * (uint32_t)a.g.V + col[k];
        const int r = r0 + (int)uu[k];
        use[k] = cell < a.cellsPerStrip && iw0 + cell < (uint32_t)a.nBW && c0 + cl[k] < C && r < a.g.R &&
                 (unsigned)(hTop + (int)uu[k]) < (unsigned)a.g.H && pc * a.PX + px[k] < (uint32_t)a.g.W;
        ib[k] = use[k] ? mapRow[iw0 + cell] : -1;
    }
    f4 val[STRIP_SLOTS];
#pragma unroll
    for (int k = 0; k < STRIP_SLOTS; ++k) {
        if (ib[k] >= 0) {
            const float* __restrict__ src = x + ((int64_t)ib[k] * C + c0 + cl[k]) * plane + (int64_t)(r0 + (int)uu[k]) * S + col[k];
            val[k] = ld_stream(reinterpret_cast<const f4*>(src));
        }
    }
#pragma unroll
    for (int k = 0; k < STRIP_SLOTS; ++k) {
        if (ib[k] >= 0) {
            // (a block's last columns may lie beyond the image: those pixels are not consumed)
            const uint32_t at = strip_lds_index(a, uu[k], px[k], cl[k]);
            lds[at] = val[k].x;
            lds[at + a.CT] = val[k].y;
            lds[at + 2u * a.CT] = val[k].z;
            lds[at + 3u * a.CT] = val[k].w;
        }
    }
}

// sparse_gather.cc:103-130 on top of a copy of ybase (sparse_gather.cc:338-346), non-overlapping blocks.
// OP: STRIP_ASSIGN / STRIP_ADD write the whole output; STRIP_COPY writes only the pixels that no block covers and
// leaves the covered ones to a scatter kernel that follows (planar stacks whose geometry the staging above does
// not take).
constexpr int STRIP_ASSIGN = 0, STRIP_ADD = 1, STRIP_COPY = 2;

template <int VEC, int OP, bool PLANAR>
__global__ __launch_bounds__(256) void k_scatter_strip(const float* __restrict__ x, const float* __restrict__ ybase,
                                                       float* __restrict__ y, const int32_t* __restrict__ map,
                                                       const int32_t* __restrict__ chain,
                                                       const int32_t* __restrict__ dup, StripArgs a)
{
    typedef typename Vec<VEC>::type vec;
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    constexpr bool ADD = OP == STRIP_ADD;
    const uint32_t tid = threadIdx.x;
    // Which strip: channel chunk, pixel chunk, strip of the row of cells, row of cells, image, the first fastest:
    // neighbouring workgroups write neighbouring pieces of the same image rows.
    uint32_t l = blockIdx.x;
    uint32_t t = fdiv(l, a.dCC);
    const uint32_t cc = (uint32_t)__builtin_amdgcn_readfirstlane((int)(l - t * a.nCC));
    l = t; t = fdiv(l, a.dPC);
    const uint32_t pc = (uint32_t)__builtin_amdgcn_readfirstlane((int)(l - t * a.nPC));
    l = t; t = fdiv(l, a.dK);
    const int r0 = __builtin_amdgcn_readfirstlane((int)(l - t * a.kPerBand)) * STRIP_ROWS;  // first block row of the strip
    l = t; t = fdiv(l, a.dBH);
    const uint32_t band = (uint32_t)__builtin_amdgcn_readfirstlane((int)(l - t * (uint32_t)a.nBH));
    const uint32_t n = (uint32_t)__builtin_amdgcn_readfirstlane((int)t);
    const int hTop = a.g.oh + ((int)band + a.bhMin) * a.g.U + r0;  // the strip's first image row

    const uint32_t wl = fdiv(tid, a.dCVT), cvl = tid - wl * a.CVT;
    const uint32_t cv = cc * a.CVT + cvl;
    const uint32_t w = pc * a.PX + wl;
    const bool live = wl < a.PX && w < (uint32_t)a.g.W && cv < a.CV;

    // the lane's cell: one look-up for the strip's rows (they lie in one row of cells)
    const int32_t* __restrict__ mapRow = map + ((int64_t)n * a.nBH + band) * a.nBW;
    const uint32_t dw = w - (uint32_t)(a.g.ow + a.bwMin * a.g.V);  // >= 0 for every pixel of the image
    const uint32_t iw = fdiv(dw, a.dV), s = dw - iw * (uint32_t)a.g.V;
    int ib = -1;
    if (live && s < (uint32_t)a.g.S && r0 < a.g.R) ib = mapRow[iw];

    const rsrc_t br = make_rsrc(ybase + (int64_t)n * a.imgFloats, a.imgBytes);
    const rsrc_t yr = make_rsrc(y + (int64_t)n * a.imgFloats, a.imgBytes);
    uint32_t off[STRIP_ROWS];
    bool inBlock[STRIP_ROWS];  // (the same for the whole workgroup)
#pragma unroll
    for (int u = 0; u < STRIP_ROWS; ++u) {
        const int h = hTop + u;
        const bool rowLive = r0 + u < a.g.U && (unsigned)h < (unsigned)a.g.H;
        inBlock[u] = r0 + u < a.g.R;
        off[u] = live && rowLive ? (((uint32_t)h * (uint32_t)a.g.W + w) * a.CV + cv) * (uint32_t)(VEC * 4) : BUF_OOB;
    }
    vec b[STRIP_ROWS], v[STRIP_ROWS];
    if (ADD) {
        // an add reads the base everywhere: these loads do not wait for the look-up
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) b[u] = buf_load<VEC>(br, off[u]);
    }
    if (OP == STRIP_COPY) {
        // covered pixels (whichever rows of the list cover them) belong to the scatter kernel that follows
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) {
            if (ib >= 0 && inBlock[u]) off[u] = BUF_OOB;
            b[u] = buf_load<VEC>(br, off[u]);
        }
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) buf_store<BUF_NT>(yr, off[u], b[u]);
        return;
    }
    const bool dups = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(dup)) != 0;
    if (!dups) {
        const bool cov = ib >= 0;
        if (!ADD) {
#pragma unroll
            for (int u = 0; u < STRIP_ROWS; ++u) b[u] = buf_load<VEC>(br, cov && inBlock[u] ? BUF_OOB : off[u]);  // covered pixels are not read
        }
        if (PLANAR && r0 < a.g.R) {
            extern __shared__ __attribute__((aligned(16))) float lds[];
            strip_stage_planar(x, mapRow, a, lds, pc, cc * a.CT, r0, hTop);
            lds_barrier();
#pragma unroll
            for (int u = 0; u < STRIP_ROWS; ++u) {
                v[u] = vzero<VEC>();
                if (cov && inBlock[u] && off[u] != BUF_OOB) {
                    if (VEC == 4) {
                        const f4 q = lds_read4(lds + strip_lds_index(a, (uint32_t)u, wl, cvl * 4u));
#pragma unroll
                        for (int k = 0; k < VEC; ++k) vset(v[u], k, vget(q, k));
                    } else {
#pragma unroll
                        for (int k = 0; k < VEC; ++k) vset(v[u], k, lds[strip_lds_index(a, (uint32_t)u, wl, cvl * VEC + k)]);
                    }
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < STRIP_ROWS; ++u) {
                v[u] = vzero<VEC>();
                if (cov && inBlock[u] && off[u] != BUF_OOB) v[u] = strip_stack_load<VEC, false>(x, ib, r0 + u, s, cv, a);
            }
        }
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) {
            const bool hit = cov && inBlock[u];
            buf_store<BUF_NT>(yr, off[u], hit ? (ADD ? vadd(b[u], v[u]) : v[u]) : b[u]);
        }
        return;
    }
    // Some cell is named by several rows of the list (rare; reduce_mask never produces such a list): the rows of a
    // cell form a linked list.  A plain write takes the row listed last; an add sums the rows in list order.
    if (!ADD) {
        for (int c = ib; c >= 0; c = chain[c]) ib = max(ib, c);
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) {
            const bool hit = ib >= 0 && inBlock[u];
            vec out;
            if (hit && off[u] != BUF_OOB) out = strip_stack_load<VEC, PLANAR>(x, ib, r0 + u, s, cv, a);
            else out = buf_load<VEC>(br, hit ? BUF_OOB : off[u]);
            buf_store<BUF_NT>(yr, off[u], out);
        }
    } else {
        int prev = -1;
        while (ib >= 0) {
            int cur = 0x7fffffff;
            for (int c = ib; c >= 0; c = chain[c])
                if (c > prev && c < cur) cur = c;
            if (cur == 0x7fffffff) break;
#pragma unroll
            for (int u = 0; u < STRIP_ROWS; ++u)
                if (inBlock[u] && off[u] != BUF_OOB) b[u] = vadd(b[u], strip_stack_load<VEC, PLANAR>(x, cur, r0 + u, s, cv, a));
            prev = cur;
        }
#pragma unroll
        for (int u = 0; u < STRIP_ROWS; ++u) buf_store<BUF_NT>(yr, off[u], b[u]);
    }
}

// ---- planar stack, blocks that tile the plane (bsize == bstride): one launch over the cells --------------------
//
// A planar stack whose rows the strips above cannot stage (18x18 blocks at an odd offset: 72-byte pieces at 8-byte
// alignment) wants to be read along its planes, by the tile kernel.  With bsize == bstride a cell is exactly its
// block, so the launch runs over the CELLS of the grid instead of the list: a workgroup looks its cell up in the
// map; an active cell is scattered as one tile of scatter_planar_tile (which reads the base where it adds), an
// empty cell is copied from the base, tile number `rem` of its `tpb` taking every tpb-th part of the cell's row
// segments.  Every byte of the output is written once and nothing is read twice.  A cell that several rows of the
// list name (rare) is built element by element: the row listed last for a plain write, every row in list order
// for an add (sparse_gather.cc:105-129).
struct CellArgs {
    int bhMin, bwMin, nBH, nBW;
    uint32_t CV;  // channel vectors per pixel
    FastDiv dBW, dBHW;
};

constexpr int CELL_UNR = 4;

template <int VEC, int MODE>
__device__ __forceinline__ void cell_by_elements(const float* __restrict__ x, const float* __restrict__ ybase,
                                                 float* __restrict__ y, const int32_t* __restrict__ chain,
                                                 const TileArgs& a, const CellArgs& c, int head, uint32_t cell,
                                                 uint32_t rem)
{
    typedef typename Vec<VEC>::type vec;
    const Geom& g = a.g;
    const uint32_t n = fdiv(cell, c.dBHW);
    const uint32_t inImg = cell - n * (uint32_t)(c.nBH * c.nBW);
    const uint32_t ih = fdiv(inImg, c.dBW), iw = inImg - ih * (uint32_t)c.nBW;
    const int h0 = g.oh + ((int)ih + c.bhMin) * g.U, w0 = g.ow + ((int)iw + c.bwMin) * g.V;
    const int hlo = max(0, h0), hhi = min(g.H, h0 + g.U), wlo = max(0, w0), whi = min(g.W, w0 + g.V);
    if (hhi <= hlo || whi <= wlo) return;
    const uint32_t segV = (uint32_t)(whi - wlo) * c.CV;  // vectors per row segment: contiguous in the tensor
    const uint32_t total = (uint32_t)(hhi - hlo) * segV;
    const uint32_t nthr = blockDim.x, stride = a.tpb * nthr;
    const rsrc_t br = make_rsrc(ybase + (int64_t)n * a.imgFloats, a.imgBytes);
    const rsrc_t yr = make_rsrc(y + (int64_t)n * a.imgFloats, a.imgBytes);
    if (head < 0) {
        for (uint32_t e0 = rem * nthr + threadIdx.x; e0 < total; e0 += CELL_UNR * stride) {
            uint32_t off[CELL_UNR];
            vec v[CELL_UNR];
#pragma unroll
            for (int u = 0; u < CELL_UNR; ++u) {
                const uint32_t e = e0 + (uint32_t)u * stride;
                const uint32_t r = e / segV, j = e - r * segV;
                off[u] = e < total ? ((((uint32_t)hlo + r) * (uint32_t)g.W + (uint32_t)wlo) * c.CV + j) * (uint32_t)(VEC * 4)
                                   : BUF_OOB;
                v[u] = buf_load<VEC>(br, off[u]);
            }
#pragma unroll
            for (int u = 0; u < CELL_UNR; ++u) buf_store<BUF_NT>(yr, off[u], v[u]);
        }
        return;
    }
    // several rows of the list name this cell
    const int64_t plane = (int64_t)g.R * g.S;
    int last = head;
    for (int q = head; q >= 0; q = chain[q]) last = max(last, q);
    for (uint32_t e = rem * nthr + threadIdx.x; e < total; e += stride) {
        const uint32_t r = e / segV, j = e - r * segV;
        const uint32_t px = j / c.CV, cv = j - px * c.CV;
        const uint32_t off = ((((uint32_t)hlo + r) * (uint32_t)g.W + (uint32_t)wlo) * c.CV + j) * (uint32_t)(VEC * 4);
        const int64_t at = ((int64_t)hlo + r - h0) * g.S + ((int64_t)wlo + px - w0);  // the pixel inside the block's plane
        vec out;
        if (MODE == SCATTER_ADD) {
            out = buf_load<VEC>(br, off);
            int prev = -1;
            for (;;) {
                int cur = 0x7fffffff;
                for (int q = head; q >= 0; q = chain[q])
                    if (q > prev && q < cur) cur = q;
                if (cur == 0x7fffffff) break;
                const float* __restrict__ src = x + ((int64_t)cur * g.C + cv * VEC) * plane + at;
#pragma unroll
                for (int k = 0; k < VEC; ++k) vset(out, k, vget(out, k) + src[k * plane]);
                prev = cur;
            }
        } else {
            const float* __restrict__ src = x + ((int64_t)last * g.C + cv * VEC) * plane + at;
#pragma unroll
            for (int k = 0; k < VEC; ++k) vset(out, k, src[k * plane]);
        }
        buf_store<BUF_NT>(yr, off, out);
    }
}

template <int VEC, int MODE>
__global__ __launch_bounds__(512) void k_scatter_cells(const float* __restrict__ x, const float* ybase, float* y,
                                                       const int16_t* __restrict__ idx,
                                                       const int32_t* __restrict__ map,
                                                       const int32_t* __restrict__ chain,
                                                       const int32_t* __restrict__ dup, TileArgs a, ColorArgs col,
                                                       CellArgs c)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ uint32_t waveBits[8];
    typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
    uint32_t cell, rem;
    if (a.grid2d) {
        cell = blockIdx.y;
        rem = blockIdx.x;
    } else {
        cell = blockIdx.x / a.tpb;
        rem = blockIdx.x - cell * a.tpb;
    }
    // (scalar loads: the map was written by an earlier launch and is not written here)
    const int head = ((const_i32_ptr)(reinterpret_cast<uintptr_t>(map)))[cell];
    const bool dups = *(const_i32_ptr)(reinterpret_cast<uintptr_t>(dup)) != 0;
    bool several = false;
    if (dups && head >= 0) several = ((const_i32_ptr)(reinterpret_cast<uintptr_t>(chain)))[head] >= 0;
    if (head >= 0 && !several) {
        scatter_planar_tile<VEC, MODE, TileRt>(x, y, ybase, idx, a, col, lds, waveBits, (uint32_t)head, rem);
        return;
    }
    cell_by_elements<VEC, MODE>(x, ybase, y, chain, a, c, head, cell, rem);
}

struct CoverArgs {
    Geom g;
    uint32_t RS;
    uint32_t imgV;      // vectors per image
    uint32_t imgBytes;
    int64_t imgFloats, imgPixels;
    FastDiv dCV, dS;
};

constexpr int COVER_UNR = 4;

// Owner map of the ordered plain scatter (SCATTER_OWNED): -1 everywhere, then the highest list position among the
// blocks that cover each pixel.  Rows past the device-resident count and rows that name no image mark nothing.
__global__ __launch_bounds__(256) void k_owner_fill(int32_t* __restrict__ owner, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) owner[i] = -1;
}

__global__ __launch_bounds__(256) void k_owner_mark(const int16_t* __restrict__ idx, int numActive, CoverArgs a,
                                                    int32_t* __restrict__ owner)
{
    const int64_t total = (int64_t)numActive * a.RS;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const uint32_t ib = (uint32_t)(i / a.RS);
        if (a.g.countDev && ib >= (uint32_t)*a.g.countDev) return;
        const uint32_t p = (uint32_t)(i - (int64_t)ib * a.RS);
        const uint32_t r = fdiv(p, a.dS), sc = p - r * (uint32_t)a.g.S;
        const BlockOrigin o = load_origin(idx, ib, a.g);
        const int hh = o.h0 + (int)r, ww = o.w0 + (int)sc;
        if (o.valid && (unsigned)hh < (unsigned)a.g.H && (unsigned)ww < (unsigned)a.g.W)
            atomicMax(owner + ((int64_t)o.n * a.imgPixels + (int64_t)hh * a.g.W + ww), (int32_t)ib);
    }
}

// Copies the pixels that no block covers (owner map entry below 0); the ordered scatter writes the others.
template <int VEC>
__global__ __launch_bounds__(256) void k_copy_uncovered(const float* __restrict__ src, float* __restrict__ dst,
                                                        const int32_t* __restrict__ owner, CoverArgs a)
{
    typedef typename Vec<VEC>::type vec;
    const uint32_t n = blockIdx.y;
    const rsrc_t sr = make_rsrc(src + (int64_t)n * a.imgFloats, a.imgBytes);
    const rsrc_t dr = make_rsrc(dst + (int64_t)n * a.imgFloats, a.imgBytes);
    const int32_t* __restrict__ fl = owner + (int64_t)n * a.imgPixels;
    const uint32_t e0 = blockIdx.x * (256u * COVER_UNR) + threadIdx.x;
    bool cov[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) {
        const uint32_t e = min(e0 + (uint32_t)u * 256u, a.imgV - 1u);
        cov[u] = fl[fdiv(e, a.dCV)] >= 0;
    }
    uint32_t off[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) {
        const uint32_t e = e0 + (uint32_t)u * 256u;
        off[u] = (e >= a.imgV || cov[u]) ? BUF_OOB : e * (uint32_t)(VEC * 4);
    }
    vec v[COVER_UNR];
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) v[u] = buf_load<VEC>(sr, off[u]);
#pragma unroll
    for (int u = 0; u < COVER_UNR; ++u) buf_store<BUF_NT>(dr, off[u], v[u]);
}

// Cells that touch the image and the strip geometry; false where k_scatter_strip does not apply.
// `planar`: the strips also stage a planar stack through LDS (strip_stage_planar); false where that does not apply.
static bool make_strip_args(const Geom& g, int vec, bool planar, const float* x, StripArgs& a, int64_t& mapN)
{
    if (g.U < g.R || g.V < g.S) return false;  // overlapping blocks: a pixel may belong to several
    a.g = g;
    a.imgFloats = (int64_t)g.H * g.W * g.C;
    if (a.imgFloats >= (1ll << 30)) return false;  // 32-bit byte offsets inside one image
    if ((int64_t)g.R * g.S >= (1ll << 31)) return false;
    auto floordiv = [](int64_t p, int64_t q) { return p >= 0 ? p / q : -((-p + q - 1) / q); };
    int64_t bhMin = floordiv(-(int64_t)g.oh, g.U), bhMax = floordiv((int64_t)g.H - 1 - g.oh, g.U);
    int64_t bwMin = floordiv(-(int64_t)g.ow, g.V), bwMax = floordiv((int64_t)g.W - 1 - g.ow, g.V);
    // (cells beyond the int16 range of the list can hold no block: they stay -1 in the map)
    if (bhMin < -(1ll << 30) || bwMin < -(1ll << 30) || bhMax > (1ll << 30) || bwMax > (1ll << 30)) return false;
    a.bhMin = (int)bhMin; a.bwMin = (int)bwMin;
    a.nBH = (int)(bhMax - bhMin + 1); a.nBW = (int)(bwMax - bwMin + 1);
    mapN = (int64_t)g.N * a.nBH * a.nBW;
    if (mapN >= (1ll << 31)) return false;
    if ((int64_t)g.ow + (int64_t)a.bwMin * g.V < -(1ll << 31)) return false;
    a.kPerBand = (uint32_t)((g.U + STRIP_ROWS - 1) / STRIP_ROWS);
    a.CV = (uint32_t)(g.C / vec);
    // NHWC stack: all channels of a pixel in one strip (both sides move whole pixels).  Planar stack: chunks of 32
    // channels, so that a strip is wide enough in pixels to take whole cells.
    a.CVT = planar && a.CV * (uint32_t)vec > 32u ? 32u / (uint32_t)vec : a.CV;
    if (a.CVT > 256u) return false;
    a.CT = a.CVT * (uint32_t)vec;
    a.nCC = (a.CV + a.CVT - 1u) / a.CVT;
    a.PX = 256u / a.CVT;
    a.imgBytes = (uint32_t)(a.imgFloats * 4);
    a.nPC = ((uint32_t)g.W + a.PX - 1u) / a.PX;
    const int64_t tiles = (int64_t)g.N * a.nBH * a.kPerBand * a.nPC * a.nCC;
    if (tiles >= (1ll << 31)) return false;
    a.tiles = (uint32_t)tiles;
    a.swzMask = 0;
    a.S4 = 1;
    a.cellsPerStrip = 1;
    if (planar) {
        // strips that line up with the cells, planar rows that are whole 16-byte vectors (see strip_stage_planar)
        if (g.S % 4 != 0 || g.V % 4 != 0 || (uint32_t)g.V > a.PX || a.PX % (uint32_t)g.V != 0) return false;
        if (g.ow + a.bwMin * g.V != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0) return false;
        a.S4 = (uint32_t)g.S / 4u;
        a.cellsPerStrip = a.PX / (uint32_t)g.V;
        if (a.CT % 4u == 0) {
            const uint32_t c4 = a.CT / 4u, low = c4 & (~c4 + 1u);  // largest power of two that divides CT/4
            a.swzMask = (low > 8u ? 8u : low) - 1u;
        }
    }
    a.dCVT = make_fastdiv(a.CVT);
    a.dCC = make_fastdiv(a.nCC);
    a.dV = make_fastdiv((uint32_t)g.V);
    a.dK = make_fastdiv(a.kPerBand);
    a.dPC = make_fastdiv(a.nPC);
    a.dBH = make_fastdiv((uint32_t)a.nBH);
    a.dS4 = make_fastdiv(a.S4);
    a.dCT = make_fastdiv(a.CT);
    return true;
}

// Scratch of the one-pass copying scatter: the cell map, the duplicate flag, one chain entry per list row.
size_t scatter_cover_workspace_bytes(const Geom& g, int numActive)
{
    if (numActive <= 0) return 0;
    StripArgs a;
    int64_t mapN = 0;
    // (with the widest channel vectors C allows; a call whose pointers force narrower ones checks again)
    if (make_strip_args(g, g.C % 4 == 0 ? 4 : (g.C % 2 == 0 ? 2 : 1), false, nullptr, a, mapN))
        return (size_t)mapN * 4 + 16 + (size_t)numActive * 4 + 16;
    return 0;
}

static void make_cover_args(const Geom& g, int vec, CoverArgs& c)
{
    c.g = g;
    c.RS = (uint32_t)(g.R * g.S);
    c.imgFloats = (int64_t)g.H * g.W * g.C;
    c.imgPixels = (int64_t)g.H * g.W;
    c.imgV = (uint32_t)(c.imgFloats / vec);
    c.imgBytes = (uint32_t)(c.imgFloats * 4);
    c.dCV = make_fastdiv((uint32_t)(g.C / vec));
    c.dS = make_fastdiv((uint32_t)g.S);
}

// Nine bits per block for SCATTER_RANKED.  One wave per block: the lanes compare the block with every row of the
// list; a later row that names the same image and a grid position within one step in both directions sets the
// classes of pixels it shares with the block (itself included: a block listed twice loses all its pixels to the
// later row).
constexpr int RANK_MAX_BLOCKS = 4096;   // rows compared pairwise: 16.8 M comparisons at most

__global__ __launch_bounds__(256) void k_rank_table(const int16_t* __restrict__ idx, int numActive, Geom g,
                                                    int32_t* __restrict__ table)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t ib = (uint32_t)__builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4u + (threadIdx.x >> 6)));
    const uint32_t count = list_count(g, (uint32_t)numActive);
    if (ib >= count) return;
    const RawTriple raw = load_triple(idx, ib);
    const ListRows lr = list_rows(idx, count);
    uint32_t bits = 0u;
    // eight rows per lane in flight (one 8-byte load each): the kernel is a chain of load latencies and nothing else
    constexpr int UNR = 8;
    for (uint32_t j0 = ib + 1u; j0 < count; j0 += 64u * UNR) {
        ListRow rows[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const uint32_t j = j0 + (uint32_t)u * 64u + lane;
            rows[u] = list_row_load(lr, j, j < count);
        }
        const BlockOrigin o = origin_of(raw, g);
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            int n2, bh2, bw2;
            list_row_unpack(rows[u], n2, bh2, bw2);
            if (j0 + (uint32_t)u * 64u + lane < count) bits |= rank_pair_bits(o.n, o.bh, o.bw, n2, bh2, bw2);
        }
    }
    for (int off = 32; off > 0; off >>= 1) bits |= (uint32_t)__shfl_xor((int)bits, off);
    if (lane == 0) table[ib] = (int32_t)bits;
}

// The rank table applies when at most 2x2 blocks share a pixel and the list is short enough for pairwise comparison.
static bool rank_table_applies(const Geom& g, int numActive)
{
    return numActive <= RANK_MAX_BLOCKS && g.R <= 2 * (int64_t)g.U && g.S <= 2 * (int64_t)g.V;
}

size_t scatter_owner_workspace_bytes(const Geom& g, int numActive)
{
    if (numActive <= 0 || !(g.U < g.R || g.V < g.S)) return 0;  // only overlapping blocks need an order
    if ((int64_t)g.R * g.S >= (1ll << 31)) return 0;
    // (the owner map; the rank table of the in-place op needs less, but the copying op always takes the map)
    const size_t map = (size_t)g.N * g.H * g.W * 4 + 16, table = (size_t)numActive * 4 + 16;
    return map > table ? map : table;
}

// Builds the owner map in `workspace`; false (nothing launched) when the ordered scatter does not apply.
static bool build_owner_map(const int16_t* idx, int numActive, const Geom& g, void* workspace, size_t workspaceBytes,
                            hipStream_t stream, int32_t*& owner)
{
    const size_t need = scatter_owner_workspace_bytes(g, numActive);
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3)) return false;
    owner = static_cast<int32_t*>(workspace);
    CoverArgs c;
    make_cover_args(g, 1, c);
    const int64_t n = (int64_t)g.N * g.H * g.W;
    int64_t wgs = (n + 1023) / 1024;
    if (wgs > 8192) wgs = 8192;
    hipLaunchKernelGGL(k_owner_fill, dim3((unsigned)wgs), dim3(256), 0, stream, owner, n);
    int64_t markWgs = ((int64_t)numActive * c.RS + 255) / 256;
    if (markWgs > 65536) markWgs = 65536;
    hipLaunchKernelGGL(k_owner_mark, dim3((unsigned)markWgs), dim3(256), 0, stream, idx, numActive, c, owner);
    return true;
}

// The kernels can rank the blocks themselves (SCATTER_RANKED_INLINE): at most 2x2 blocks over a pixel, a list short
// enough that the comparison stays small against the data moved: a workgroup of the planar tile kernel compares
// once per 16-24 KB tile; a wave of the NHWC kernel moves 4 KB and is slowed by every instruction on its way (with 312
// blocks that kernel takes 39 us against 34), which is worth it while the launch of k_rank_table (3-5 us) costs
// more: up to about 200 blocks of the 800x800x128 workload.
constexpr int RANK_INLINE_MAX_BLOCKS = 2048;
constexpr int RANK_INLINE_MAX_BLOCKS_NHWC = 192;

static bool rank_inline_applies(const Geom& g, int numActive, bool transpose, int vec)
{
    if (numActive > RANK_INLINE_MAX_BLOCKS || !(g.U < g.R || g.V < g.S)) return false;
    if (g.R > 2 * (int64_t)g.U || g.S > 2 * (int64_t)g.V || (int64_t)g.R * g.S < 4) return false;
    // (the wide NHWC kernel, for images beyond 32-bit offsets, does not rank)
    if (!transpose) return numActive <= RANK_INLINE_MAX_BLOCKS_NHWC && nhwc_fits_buffers(g);
    TileArgs a;
    int threads;
    size_t lds;
    unsigned grid;
    return scatter_tile_args(g, numActive, vec, a, threads, lds, grid);  // else k_planar_small would run
}

hipError_t launch_scatter_owned(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (numActive == 0) { done = true; return hipSuccess; }
    if (rank_inline_applies(g, numActive, transpose, pick_vec(g, y, nullptr))) {
        done = true;
        return scatter_from(x, y, y, idx, numActive, g, transpose, SCATTER_ASSIGN, stream, nullptr, false, true);
    }
    if (rank_table_applies(g, numActive) && scatter_owner_workspace_bytes(g, numActive) != 0 && workspace &&
        workspaceBytes >= (size_t)numActive * 4 + 16 && (reinterpret_cast<uintptr_t>(workspace) & 3) == 0) {
        int32_t* table = static_cast<int32_t*>(workspace);
        hipLaunchKernelGGL(k_rank_table, dim3((unsigned)((numActive + 3) / 4)), dim3(256), 0, stream, idx, numActive, g,
                           table);
        done = true;
        return scatter_from(x, y, y, idx, numActive, g, transpose, SCATTER_ASSIGN, stream, table, true);
    }
    int32_t* owner = nullptr;
    if (!build_owner_map(idx, numActive, g, workspace, workspaceBytes, stream, owner)) return hipSuccess;
    done = true;
    return scatter_from(x, y, y, idx, numActive, g, transpose, SCATTER_ASSIGN, stream, owner);
}

// y = zeros, plus the sum of the blocks (the gradient of sparse_gather), for overlapping blocks of which at most 2x2
// cover a pixel, in one pass over the stack: zeros where no block lies (k_fill_uncovered), then SCATTER_SUM.
// `done` is false, and nothing launched, where this does not apply; the caller then takes the colour passes.
template <int VEC>
static void launch_sum(const float* x, float* y, const int16_t* idx, const Geom& g, int numActive, bool transpose,
                          const ColorArgs& col, hipStream_t stream)
{
    if (!transpose) {
        NhwcArgs a;
        make_nhwc_args(g, numActive, VEC, a);
        hipLaunchKernelGGL((k_scatter_nhwc<VEC, SCATTER_SUM>), dim3((a.units + 3) / 4), dim3(256), 0, stream, x, y,
                           (const float*)y, idx, a, col);
        return;
    }
    TileArgs a;
    int threads;
    size_t lds;
    unsigned grid;
    scatter_tile_args(g, numActive, VEC, a, threads, lds, grid);
    if (launch_fixed_scatter<VEC, SCATTER_SUM>(x, y, y, idx, a, threads, lds, numActive, col, stream)) return;
    hipLaunchKernelGGL((k_scatter_planar<VEC, SCATTER_SUM, TileRt>), tile_grid(a.grid2d, a.tpb, numActive, a.total, a.g),
                       dim3(threads), lds, stream, x, y, (const float*)y, idx, a, col);
}

hipError_t launch_scatter_onto_zeros(const float* x, float* y, const int16_t* idx, int numActive, const Geom& g,
                                     bool transpose, void* workspace, size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (numActive <= 0 || numActive > SUM_MAX_BLOCKS || g.countDev || !(g.U < g.R || g.V < g.S)) return hipSuccess;
    // (the other blocks' values are read through one buffer over the whole stack: 32-bit byte offsets)
    if ((int64_t)numActive * g.C * g.R * g.S * 4 >= (1ll << 32) - 16) return hipSuccess;
    const size_t need = scatter_color_workspace_bytes(g, numActive);  // (the map and the flag are its first part)
    if (!workspace || need == 0 || workspaceBytes < need || (reinterpret_cast<uintptr_t>(workspace) & 3)) return hipSuccess;
    PullArgs pa;
    int64_t mapN = 0;
    if (!make_map_args(g, pa, mapN)) return hipSuccess;
    const int vec = pick_vec(g, y, transpose ? nullptr : x);
    FillArgs fa;
    unsigned fillGrid = 0;
    if (!make_fill_args(g, vec, pa, fa, fillGrid)) return hipSuccess;  // (more than 2x2 blocks over a pixel)
    if (transpose) {
        TileArgs a;
        int threads;
        size_t lds;
        unsigned grid;
        if ((int64_t)g.R * g.S < 4 || !scatter_tile_args(g, numActive, vec, a, threads, lds, grid)) return hipSuccess;
    } else {
        NhwcArgs na;
        if (!nhwc_fits_buffers(g) || !make_nhwc_args(g, numActive, vec, na)) return hipSuccess;
    }
    int32_t* map = static_cast<int32_t*>(workspace);
    int32_t* dup = map + mapN;
    launch_block_map(idx, numActive, pa, map, mapN, dup, stream);
    const int32_t* cmap = map;
    const int32_t* cdup = dup;
    if (vec == 4) hipLaunchKernelGGL(k_fill_uncovered<4>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
    else if (vec == 2) hipLaunchKernelGGL(k_fill_uncovered<2>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
    else hipLaunchKernelGGL(k_fill_uncovered<1>, dim3(fillGrid), dim3(256), 0, stream, y, cmap, cdup, fa);
    ColorArgs col;
    col.kh = 2; col.kw = 2; col.pass = 0;  // (unused by this mode, like the fields of the other orders)
    col.dup = cdup; col.owner = nullptr; col.rank = nullptr; col.first = 0; col.map = cmap;
    col.bhMin = pa.bhMin; col.bwMin = pa.bwMin; col.nBH = pa.nBH; col.nBW = pa.nBW;
    col.perm = nullptr; col.counts = nullptr; col.permStride = 0;
    if (vec == 4) launch_sum<4>(x, y, idx, g, numActive, transpose, col, stream);
    else if (vec == 2) launch_sum<2>(x, y, idx, g, numActive, transpose, col, stream);
    else launch_sum<1>(x, y, idx, g, numActive, transpose, col, stream);
    done = true;
    return hipGetLastError();
}

template <int VEC>
static void launch_strip(const float* x, const float* ybase, float* y, bool planar, int op, const int32_t* map,
                         const int32_t* chain, const int32_t* dup, const StripArgs& a, hipStream_t stream)
{
    const dim3 grid(a.tiles);
    const size_t lds = planar ? (size_t)STRIP_ROWS * a.PX * a.CT * sizeof(float) : 0;  // 16 KB with 16-byte vectors
#define SBNET_STRIP(OP, PL) \
    hipLaunchKernelGGL((k_scatter_strip<VEC, OP, PL>), grid, dim3(256), lds, stream, x, ybase, y, map, chain, dup, a)
    if (op == STRIP_COPY) SBNET_STRIP(STRIP_COPY, false);
    else if (op == STRIP_ADD && planar) SBNET_STRIP(STRIP_ADD, true);
    else if (op == STRIP_ADD) SBNET_STRIP(STRIP_ADD, false);
    else if (planar) SBNET_STRIP(STRIP_ASSIGN, true);
    else SBNET_STRIP(STRIP_ASSIGN, false);
#undef SBNET_STRIP
}

// The copying scatter of a planar stack as one launch over the cells (k_scatter_cells); false, with nothing
// launched, where that does not apply: blocks that do not tile the plane, cells too small to be copied one by one.
template <int VEC>
static bool launch_cells(const float* x, const float* ybase, float* y, const int16_t* idx, int numActive, const Geom& g,
                         ScatterMode mode, const StripArgs& sa, int64_t mapN, const int32_t* map, const int32_t* chain,
                         const int32_t* dup, hipStream_t stream, bool dry)
{
    if (g.R != g.U || g.S != g.V || (int64_t)g.R * g.S < 4) return false;
    if ((int64_t)g.U * g.V * g.C * 4 < 4096 || mapN > 0x7fffffffll) return false;
    TileArgs a;
    int threads;
    size_t lds;
    unsigned grid;
    if (!scatter_tile_args(g, (int)mapN, VEC, a, threads, lds, grid)) return false;
    if (mapN * (int64_t)a.tpb >= (1ll << 31)) return false;
    if (dry) return true;
    a.grid2d = mapN <= GRID_Y_MAX;
    CellArgs c;
    c.bhMin = sa.bhMin; c.bwMin = sa.bwMin; c.nBH = sa.nBH; c.nBW = sa.nBW;
    c.CV = (uint32_t)(g.C / VEC);
    c.dBW = make_fastdiv((uint32_t)sa.nBW);
    c.dBHW = make_fastdiv((uint32_t)(sa.nBH * sa.nBW));
    const ColorArgs aux{1, 1, 0, nullptr, nullptr, nullptr, 0, nullptr, 0, 0, 0, 0, nullptr, nullptr, 0};
    const dim3 gr = a.grid2d ? dim3(a.tpb, (unsigned)mapN) : dim3((unsigned)(mapN * a.tpb));
    (void)numActive;
    if (mode == SCATTER_ADD)
        hipLaunchKernelGGL((k_scatter_cells<VEC, SCATTER_ADD>), gr, dim3(threads), lds, stream, x, ybase, y, idx, map, chain,
                           dup, a, aux, c);
    else
        hipLaunchKernelGGL((k_scatter_cells<VEC, SCATTER_ASSIGN>), gr, dim3(threads), lds, stream, x, ybase, y, idx, map,
                           chain, dup, a, aux, c);
    return true;
}

hipError_t launch_scatter_over_base(const float* x, const float* ybase, float* y, const int16_t* idx, int numActive,
                                    const Geom& g, bool transpose, ScatterMode mode, void* workspace,
                                    size_t workspaceBytes, hipStream_t stream, bool& done)
{
    done = false;
    if (mode == SCATTER_ATOMIC || numActive <= 0) return hipSuccess;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 3)) return hipSuccess;

    // Blocks that do not overlap: one streaming pass over the output (k_scatter_strip).  A planar stack whose
    // geometry the strips do not stage is scattered by the tile kernel after a pass that copies the rest.
    {
        StripArgs a;
        int64_t mapN = 0;
        const int vb = pick_vec(g, ybase, y), vx = pick_vec(g, transpose ? nullptr : x, nullptr);
        const int vec = vb < vx ? vb : vx;
        const size_t need = scatter_cover_workspace_bytes(g, numActive);
        bool planar = transpose;
        bool ok = need != 0 && workspaceBytes >= need;
        bool cells = false;  // one launch over the cells of the block grid instead of the strips
        if (ok && !make_strip_args(g, vec, planar, x, a, mapN)) {
            planar = false;
            ok = transpose && make_strip_args(g, vec, false, x, a, mapN);
            if (ok) {
                cells = vec == 4 ? launch_cells<4>(x, ybase, y, idx, numActive, g, mode, a, mapN, nullptr, nullptr, nullptr, stream, true)
                      : vec == 2 ? launch_cells<2>(x, ybase, y, idx, numActive, g, mode, a, mapN, nullptr, nullptr, nullptr, stream, true)
                                 : launch_cells<1>(x, ybase, y, idx, numActive, g, mode, a, mapN, nullptr, nullptr, nullptr, stream, true);
                // (else two passes and four launches: worth it once the blocks cover enough of the tensor)
                if (!cells) ok = (int64_t)numActive * g.R * g.S * g.C * 4 >= (16ll << 20);
            }
        }
        if (ok) {
            a.g = g;
            int32_t* map = static_cast<int32_t*>(workspace);
            int32_t* dup = map + mapN;
            int32_t* chain = dup + 4;
            if (mapN <= BLOCK_MAP_ONE_WG && numActive <= BLOCK_MAP_ONE_WG) {
                hipLaunchKernelGGL(k_cell_map_small, dim3(1), dim3(1024), 0, stream, idx, numActive, a, map, (int)mapN,
                                   chain, dup);
            } else {
                int64_t fillWgs = (mapN + 255) / 256;
                if (fillWgs > 4096) fillWgs = 4096;
                hipLaunchKernelGGL(k_pull_fill, dim3((unsigned)fillWgs), dim3(256), 0, stream, map, mapN, dup);
                hipLaunchKernelGGL(k_cell_map, dim3((unsigned)((numActive + 255) / 256)), dim3(256), 0, stream, idx,
                                   numActive, a, map, chain, dup);
            }
            if (cells) {
                if (vec == 4) launch_cells<4>(x, ybase, y, idx, numActive, g, mode, a, mapN, map, chain, dup, stream, false);
                else if (vec == 2) launch_cells<2>(x, ybase, y, idx, numActive, g, mode, a, mapN, map, chain, dup, stream, false);
                else launch_cells<1>(x, ybase, y, idx, numActive, g, mode, a, mapN, map, chain, dup, stream, false);
                done = true;
                return hipGetLastError();
            }
            const int op = transpose && !planar ? STRIP_COPY : (mode == SCATTER_ADD ? STRIP_ADD : STRIP_ASSIGN);
            if (vec == 4) launch_strip<4>(x, ybase, y, planar, op, map, chain, dup, a, stream);
            else if (vec == 2) launch_strip<2>(x, ybase, y, planar, op, map, chain, dup, a, stream);
            else launch_strip<1>(x, ybase, y, planar, op, map, chain, dup, a, stream);
            done = true;
            if (op == STRIP_COPY) return scatter_from(x, y, ybase, idx, numActive, g, transpose, mode, stream);
            return hipGetLastError();
        }
    }

    // Plain writes of overlapping blocks: the owner map of the ordered scatter also tells which pixels are covered.
    // Two small launches prepare it: worth it once the blocks cover enough of the tensor to pay for them (each
    // covered byte saves one read and one write of the copy).
    if (mode != SCATTER_ASSIGN || scatter_owner_workspace_bytes(g, numActive) == 0) return hipSuccess;
    if ((int64_t)numActive * g.R * g.S * g.C * 4 < (16ll << 20)) return hipSuccess;
    if ((int64_t)g.H * g.W * g.C >= (1ll << 30)) return hipSuccess;  // 32-bit byte offsets inside one image
    CoverArgs c;
    const int vec = pick_vec(g, ybase, y);
    make_cover_args(g, vec, c);
    const dim3 grid((c.imgV + 256u * COVER_UNR - 1) / (256u * COVER_UNR), (unsigned)g.N);
    int32_t* owner = nullptr;
    if (!build_owner_map(idx, numActive, g, workspace, workspaceBytes, stream, owner)) return hipSuccess;
    if (vec == 4) hipLaunchKernelGGL((k_copy_uncovered<4>), grid, dim3(256), 0, stream, ybase, y, owner, c);
    else if (vec == 2) hipLaunchKernelGGL((k_copy_uncovered<2>), grid, dim3(256), 0, stream, ybase, y, owner, c);
    else hipLaunchKernelGGL((k_copy_uncovered<1>), grid, dim3(256), 0, stream, ybase, y, owner, c);
    done = true;
    return scatter_from(x, y, ybase, idx, numActive, g, transpose, mode, stream, owner);
}

hipError_t launch_copy(float* dst, const float* src, size_t count, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
    if ((bits & 15) == 0) {
        const size_t n4 = count / 4;
        if (n4) {
            const size_t per = 256 * COPY_UNR;
            hipLaunchKernelGGL(k_copy_v4, dim3((unsigned)((n4 + per - 1) / per)), dim3(256), 0, stream,
                               reinterpret_cast<const f4*>(src), reinterpret_cast<f4*>(dst), n4);
        }
        const size_t rem = count - n4 * 4;
        if (rem) hipLaunchKernelGGL(k_copy_scalar, dim3(1), dim3(256), 0, stream, src + n4 * 4, dst + n4 * 4, rem);
    } else {
        size_t wgs = (count + 255) / 256;
        if (wgs > 65536) wgs = 65536;
        hipLaunchKernelGGL(k_copy_scalar, dim3((unsigned)wgs), dim3(256), 0, stream, src, dst, count);
    }
    return hipGetLastError();
}

}  // namespace sbnet

/*
 * CPU oracle for the reduce_mask -> sparse_gather -> sparse_scatter path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a plain-C restatement of the reference's CPU functors
 * and of the host-visible behaviour of the ops that wrap them.  It exists so the parity tests,
 * the smoke check and the bench's cpu_baseline leg have something to compare the HIP kernels
 * against.  Nothing in the product library links, loads or calls it.
 *
 * Reference lines each function follows (paths relative to the reference checkout,
 * sbnet_tensorflow/sbnet_ops/):
 *   oracle_reduce_mask          reduce_mask.cc:68-96   (functor loop nest, lexicographic order)
 *                               reduce_mask.cc:206-218 (zero-count fix-up done by the op)
 *   oracle_sparse_gather        sparse_gather.cc:67-88
 *   oracle_sparse_scatter       sparse_gather.cc:103-130 (sequential in ib; the reference Makefile
 *                               builds the .cc files without -fopenmp, Makefile:53-59, so its
 *                               "#pragma omp parallel for" lines are inert)
 *   oracle_sparse_scatter_op    sparse_gather.cc:322-346 (validation, copy-then-scatter)
 *   oracle_copy_tensor          sparse_gather.cc:135-142
 *
 * Pinning status (what checks each function against something other than itself):
 *   oracle_reduce_mask     pinned: the two hand-written masks of benchmark/reduce_mask_tests.py:54-81
 *                          with index sets derived from max-pool + where on the padded mask; the
 *                          zero-count case of tests/test_sparse_blocks.py:303-306; torch
 *                          max_pool2d / avg_pool2d on explicitly padded masks for random shapes.
 *   oracle_sparse_gather   pinned: numpy slicing of the zero-padded tensor (README.md:86-92),
 *                          arange inputs of benchmark/sparse_gather_tests.py:96-97,119-120,
 *                          transposed == transpose(untransposed) (test_sparse_blocks.py:325-342).
 *   oracle_sparse_scatter  pinned: README.md:119-125 slice assignment in numpy, torch fold for
 *                          overlapping add, the known-answer y_exp tables of
 *                          benchmark/sparse_conv_tests.py:211-320,451-459 through the full pipeline.
 *   oracle_copy_tensor     pinned: numpy copy.
 *
 * The *_omp variants are the "best effort" CPU rows of the benchmark (OpenMP over active blocks
 * where blocks do not overlap); they are checked against the sequential functions in the tests.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_OK 0
#define ORACLE_EINVAL_OVERLAP 1 /* add && !atomic with overlapping blocks */
#define ORACLE_EINVAL_RANK 2    /* ybase is not rank 4 */

/* reduce_mask.cc:68-96.  mask is [N,H,W,1] fp32.  Returns the raw count (may be 0). */
int oracle_reduce_mask_functor(const float* mask, int N, int H, int W, float threshold,
                               int bOffsH0, int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW,
                               int bCntH, int bCntW, int16_t* activeBlockIndices, int avgPool)
{
    int count = 0;
    for (int n = 0; n < N; ++n)
        for (int bh = 0; bh < bCntH; ++bh)
            for (int bw = 0; bw < bCntW; ++bw) {
                int h0 = bOffsH0 + bh * bStrH;
                int w0 = bOffsW0 + bw * bStrW;
                int active = 0;
                float sum = 0.0f;
                for (int hh = h0 > 0 ? h0 : 0; hh < h0 + bSzH && hh < H; ++hh)
                    for (int ww = w0 > 0 ? w0 : 0; ww < w0 + bSzW && ww < W; ++ww) {
                        float val = mask[((size_t)n * H + hh) * W + ww];
                        if (avgPool)
                            sum += val;
                        else
                            active |= (val > threshold);
                    }
                if (avgPool)
                    active = ((sum / (bSzH * bSzW)) > threshold);
                if (active) {
                    activeBlockIndices[(size_t)count * 3 + 0] = (int16_t)n;
                    activeBlockIndices[(size_t)count * 3 + 1] = (int16_t)bh;
                    activeBlockIndices[(size_t)count * 3 + 2] = (int16_t)bw;
                    count++;
                }
            }
    return count;
}

/* Op-level behaviour, reduce_mask.cc:141-220: the functor, then "count 0 becomes one block
 * (0,0,0)".  bin_counts[0] receives the reported count. */
int oracle_reduce_mask(const float* mask, int N, int H, int W, float threshold,
                       const int32_t* bcount, const int32_t* bsize, const int32_t* bstride,
                       const int32_t* boffset, int avgPool,
                       int16_t* activeBlockIndices, int32_t* bin_counts)
{
    int count = oracle_reduce_mask_functor(mask, N, H, W, threshold, boffset[0], boffset[1],
                                           bsize[0], bsize[1], bstride[0], bstride[1],
                                           bcount[0], bcount[1], activeBlockIndices, avgPool);
    if (count == 0) {
        activeBlockIndices[0] = 0;
        activeBlockIndices[1] = 0;
        activeBlockIndices[2] = 0;
        count = 1;
    }
    bin_counts[0] = count;
    return ORACLE_OK;
}

/* One block of sparse_gather.cc:69-88. */
static void gather_block(const float* x, int H, int W, int C, float* y, int bOffsH0, int bOffsW0,
                         int R, int S, int bStrH, int bStrW, int ib, const int16_t* idx,
                         int transpose)
{
    int biN = idx[(size_t)ib * 3 + 0];
    int biH = idx[(size_t)ib * 3 + 1];
    int biW = idx[(size_t)ib * 3 + 2];
    int h0 = bOffsH0 + biH * bStrH;
    int w0 = bOffsW0 + biW * bStrW;
    float* yb = y + (size_t)ib * R * S * C;
    for (int r = 0; r < R; ++r)
        for (int s = 0; s < S; ++s) {
            int hh = h0 + r, ww = w0 + s;
            int inside = (hh >= 0 && ww >= 0 && hh < H && ww < W);
            const float* px = inside ? x + (((size_t)biN * H + hh) * W + ww) * C : x;
            for (int cc = 0; cc < C; ++cc) {
                float v = inside ? px[cc] : 0.0f;
                if (transpose)
                    yb[((size_t)cc * R + r) * S + s] = v;
                else
                    yb[((size_t)r * S + s) * C + cc] = v;
            }
        }
}

/* sparse_gather.cc:67-88. */
void oracle_sparse_gather(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                          int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int numActive,
                          const int16_t* activeBlockIndices, int transpose)
{
    (void)N;
    for (int ib = 0; ib < numActive; ++ib)
        gather_block(x, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH, bStrW, ib,
                     activeBlockIndices, transpose);
}

void oracle_sparse_gather_omp(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                              int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW,
                              int numActive, const int16_t* activeBlockIndices, int transpose)
{
    (void)N;
#pragma omp parallel for schedule(dynamic, 1)
    for (int ib = 0; ib < numActive; ++ib)
        gather_block(x, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH, bStrW, ib,
                     activeBlockIndices, transpose);
}

/* One block of sparse_gather.cc:105-129.  "atomic" has no effect on the CPU. */
static void scatter_block(const float* x, int H, int W, int C, float* y, int bOffsH0, int bOffsW0,
                          int R, int S, int bStrH, int bStrW, int ib, const int16_t* idx, int add,
                          int transpose)
{
    int biN = idx[(size_t)ib * 3 + 0];
    int biH = idx[(size_t)ib * 3 + 1];
    int biW = idx[(size_t)ib * 3 + 2];
    int h0 = bOffsH0 + biH * bStrH;
    int w0 = bOffsW0 + biW * bStrW;
    const float* xb = x + (size_t)ib * R * S * C;
    for (int r = 0; r < R; ++r)
        for (int s = 0; s < S; ++s) {
            int hh = h0 + r, ww = w0 + s;
            if (!(hh >= 0 && ww >= 0 && hh < H && ww < W))
                continue;
            float* py = y + (((size_t)biN * H + hh) * W + ww) * C;
            for (int cc = 0; cc < C; ++cc) {
                float v = transpose ? xb[((size_t)cc * R + r) * S + s]
                                    : xb[((size_t)r * S + s) * C + cc];
                if (add)
                    py[cc] += v;
                else
                    py[cc] = v;
            }
        }
}

/* sparse_gather.cc:103-130, sequential in ib: adds accumulate in ib-major order and, without add,
 * the highest ib covering a pixel wins. */
void oracle_sparse_scatter(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                           int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int numActive,
                           const int16_t* activeBlockIndices, int add, int transpose, int atomic)
{
    (void)N;
    (void)atomic;
    for (int ib = 0; ib < numActive; ++ib)
        scatter_block(x, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH, bStrW, ib,
                      activeBlockIndices, add, transpose);
}

/* OpenMP over blocks; only valid (race-free, order-free) when blocks do not overlap or when
 * overlapping writes carry identical values.  The caller decides. */
void oracle_sparse_scatter_omp(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                               int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW,
                               int numActive, const int16_t* activeBlockIndices, int add,
                               int transpose, int atomic)
{
    (void)N;
    (void)atomic;
#pragma omp parallel for schedule(dynamic, 1)
    for (int ib = 0; ib < numActive; ++ib)
        scatter_block(x, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH, bStrW, ib,
                      activeBlockIndices, add, transpose);
}

/* sparse_gather.cc:135-142. */
void oracle_copy_tensor(float* dst, const float* src, size_t count)
{
    memcpy(dst, src, count * sizeof(float));
}

/* Op-level scatter, sparse_gather.cc:286-357.  ybase_rank models the rank check at :327.
 * use_var != 0: scatter in place into ybase (y is ignored, the result aliases ybase).
 * use_var == 0: y = copy(ybase), then scatter on top of y. */
int oracle_sparse_scatter_op(const float* x, int numActive, const int16_t* activeBlockIndices,
                             float* ybase, int ybase_rank, int N, int H, int W, int C,
                             const int32_t* bsize, const int32_t* bstride, const int32_t* boffset,
                             int add, int atomic, int transpose, int use_var, float* y)
{
    if (!atomic && add) {
        if (!(bstride[0] >= bsize[0] && bstride[1] >= bsize[1]))
            return ORACLE_EINVAL_OVERLAP;
    }
    if (ybase_rank != 4)
        return ORACLE_EINVAL_RANK;
    float* out = ybase;
    if (!use_var) {
        oracle_copy_tensor(y, ybase, (size_t)N * H * W * C);
        out = y;
    }
    oracle_sparse_scatter(x, N, H, W, C, out, boffset[0], boffset[1], bsize[0], bsize[1],
                          bstride[0], bstride[1], numActive, activeBlockIndices, add, transpose,
                          atomic);
    return ORACLE_OK;
}

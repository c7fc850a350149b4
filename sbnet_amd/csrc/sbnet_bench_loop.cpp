// Timed host loops over the public C ABI (include/sbnet_amd.h), for bench.py: the same
// reduce_mask -> sparse_gather -> sparse_scatter_var step that bench.py drives from Python, driven from C++
// as a caller written in the reference's host language would (the reference's ops are C++ TensorFlow kernels,
// reduce_mask.cc:123-221, sparse_gather.cc:160-218, 286-357).  Nothing here is part of libsbnet_amd.so.
#include <hip/hip_runtime_api.h>

#include <chrono>

#include "../../include/sbnet_amd.h"

extern "C" {

// One buffer set of the pipeline; every pointer is device memory except where noted.
struct sbnet_bench_set {
    const float* mask;          // [N,H,W,1], or NULL: the block list is given, fixed_count rows, no reduce_mask
    const float* x;             // [N,H,W,C], or NULL: no gather
    float* base;                // [N,H,W,C]: scattered into in place, or the copying scatter's base
    float* stack;               // block stack, capacity max_active blocks
    int16_t* idx;               // [max_active, 3]
    int32_t* count_dev;         // [1]
    void* reduce_ws;
    size_t reduce_ws_bytes;
    void* scatter_ws;           // scratch of sbnet_sparse_scatter_workspace_bytes() for max_active blocks, or NULL
    size_t scatter_ws_bytes;
    const float* scatter_stack; // what the scatter reads (the gathered stack itself, or a stack of the scatter's block size)
    float* out;                 // [N,H,W,C]: output of the copying op sparse_scatter, or NULL: sparse_scatter_var on base
};

struct sbnet_bench_geom {
    int N, H, W, C;
    int32_t bcount[2], bsize[2], bstride[2], boffset[2];        // reduce_mask / gather
    int32_t s_bsize[2], s_bstride[2], s_boffset[2];             // scatter
    float tol;
    int avgpool, transpose, add, atomic;
    int32_t max_active;
    int32_t fixed_count;        // length of the given block list (sets without a mask)
};

// sizeof of the two structs above (0: set, 1: geometry), for a caller that mirrors them in another language to
// check its layout before passing pointers.
size_t sbnet_bench_struct_bytes(int which)
{
    return which == 0 ? sizeof(sbnet_bench_set) : which == 1 ? sizeof(sbnet_bench_geom) : 0;
}

// Runs `steps` steps on `stream`, rotating over the sets, between two stream synchronisations; writes the elapsed
// wall time in seconds and the count of the last step.  mode 0: the reference's contract (reduce_mask returns
// with the count on the host, which sizes gather and scatter; sets without a mask or without x skip those ops, sets
// with `out` run the copying sparse_scatter); mode 1: the count stays on the device (mask, x and in-place scatter).
int sbnet_bench_pipeline(const sbnet_bench_set* sets, int nsets, const sbnet_bench_geom* g, int steps, int mode,
                         void* stream, double* seconds, int32_t* last_count)
{
    const int64_t dims[4] = {g->N, g->H, g->W, g->C};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (hipStreamSynchronize(s) != hipSuccess) return SBNET_EHIP;
    int32_t count = 0;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) {
        const sbnet_bench_set& b = sets[i % nsets];
        int rc;
        if (mode == 0) {
            count = g->fixed_count;
            if (b.mask) {
                rc = sbnet_reduce_mask(b.mask, g->N, g->H, g->W, g->bcount, 2, g->bsize, 2, g->bstride, 2, g->boffset,
                                       2, g->tol, g->avgpool, b.idx, &count, b.count_dev, b.reduce_ws,
                                       b.reduce_ws_bytes, stream);
                if (rc) return rc;
            }
            if (b.x) {
                rc = sbnet_sparse_gather(b.x, dims, 4, count, b.idx, g->bsize, 2, g->bstride, 2, g->boffset, 2,
                                         g->transpose, b.stack, stream);
                if (rc) return rc;
            }
            if (b.out)
                rc = sbnet_sparse_scatter(b.scatter_stack, count, b.idx, b.base, dims, 4, g->s_bsize, 2, g->s_bstride, 2,
                                          g->s_boffset, 2, g->add, g->atomic, g->transpose, b.out, b.scatter_ws,
                                          b.scatter_ws_bytes, stream);
            else
                rc = sbnet_sparse_scatter_var(b.scatter_stack, count, b.idx, b.base, dims, 4, g->s_bsize, 2, g->s_bstride,
                                              2, g->s_boffset, 2, g->add, g->atomic, g->transpose, b.scatter_ws,
                                              b.scatter_ws_bytes, stream);
            if (rc) return rc;
        } else {
            rc = sbnet_reduce_mask(b.mask, g->N, g->H, g->W, g->bcount, 2, g->bsize, 2, g->bstride, 2, g->boffset, 2,
                                   g->tol, g->avgpool, b.idx, nullptr, b.count_dev, b.reduce_ws, b.reduce_ws_bytes,
                                   stream);
            if (rc) return rc;
            rc = sbnet_sparse_gather_device_count(b.x, dims, 4, b.count_dev, g->max_active, b.idx, g->bsize, 2,
                                                  g->bstride, 2, g->boffset, 2, g->transpose, b.stack, stream);
            if (rc) return rc;
            rc = sbnet_sparse_scatter_var_device_count(b.stack, b.count_dev, g->max_active, b.idx, b.base, dims, 4,
                                                       g->s_bsize, 2, g->s_bstride, 2, g->s_boffset, 2, g->add,
                                                       g->atomic, g->transpose, b.scatter_ws, b.scatter_ws_bytes,
                                                       stream);
            if (rc) return rc;
        }
    }
    if (hipStreamSynchronize(s) != hipSuccess) return SBNET_EHIP;
    *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (mode != 0 && hipMemcpy(&count, sets[(steps - 1) % nsets].count_dev, 4, hipMemcpyDeviceToHost) != hipSuccess)
        return SBNET_EHIP;
    *last_count = count;
    return SBNET_OK;
}

}  // extern "C"

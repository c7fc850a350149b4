// C ABI of libsbnet_amd.so (declared in include/sbnet_amd.h): argument validation that mirrors
// the reference ops' OP_REQUIRES checks, then the kernel launches of sbnet_reduce_mask.hip, sbnet_gather.hip and sbnet_scatter.hip.
//
// Reference behaviour reproduced here (sbnet_tensorflow/sbnet_ops/):
//   reduce_mask.cc:132-138, 141-220   parameter shape check, host-visible count, zero-count fix-up
//   sparse_gather.cc:164-175, 190-207 rank / parameter checks, count taken from the host
//   sparse_gather.cc:307-346          parameter checks, add/atomic/overlap rule, rank check,
//                                     in place (Var) versus copy-then-scatter
#include "../../include/sbnet_amd.h"

#include <hip/hip_runtime_api.h>
#include <sched.h>

#include <mutex>
#include <vector>

#include "sbnet_launch.h"

namespace {

thread_local int g_lastHipError = 0;
thread_local int t_forceGeneric = 0;  // test hook, see sbnet_test_force_generic

int hip_fail(hipError_t e)
{
    g_lastHipError = (int)e;
    return SBNET_EHIP;
}

#define SBNET_HIP(call)                                  \
    do {                                                 \
        hipError_t e_ = (call);                          \
        if (e_ != hipSuccess) return hip_fail(e_);       \
    } while (0)

bool pair_ok(const int32_t* p, int len) { return p != nullptr && len == 2; }

// The host-visible count of reduce_mask (reduce_mask.cc:198-204: a HostMemory output filled by a blocking
// cudaMemcpy).  Instead of a device-to-host copy and a stream synchronisation (about 17 us of a 113 us
// pipeline step), the kernel that knows the count stores it, tagged with a sequence number, into one word
// of pinned host memory and the calling thread polls that word.  One word per thread and device, allocated
// on first use and kept until the process ends.
constexpr int MAX_SIGNAL_DEVICES = 64;
struct HostSignal {
    unsigned long long* host = nullptr;  // pinned, device-visible (same address on both sides)
    uint32_t seq = 0;
    bool failed = false;                 // allocation refused once: do not try again
};

// Words are handed out per thread and device; a thread that ends returns its words to a free list, so the
// number of words is bounded by the largest number of threads alive at once, and sbnet_shutdown() frees
// them.  Nothing is freed from a static destructor: the HIP runtime may already be gone by then.
std::mutex g_signalMutex;
std::vector<unsigned long long*> g_signalFree[MAX_SIGNAL_DEVICES];
std::vector<unsigned long long*> g_signalAll;

struct ThreadSignals {
    HostSignal dev[MAX_SIGNAL_DEVICES];
    ~ThreadSignals()
    {
        std::lock_guard<std::mutex> lock(g_signalMutex);
        for (int d = 0; d < MAX_SIGNAL_DEVICES; ++d)
            if (dev[d].host) g_signalFree[d].push_back(dev[d].host);
    }
};
thread_local ThreadSignals t_signal;

HostSignal* host_signal()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_SIGNAL_DEVICES) return nullptr;
    HostSignal& s = t_signal.dev[dev];
    if (!s.host && !s.failed) {
        std::lock_guard<std::mutex> lock(g_signalMutex);
        if (!g_signalFree[dev].empty()) {
            s.host = g_signalFree[dev].back();
            g_signalFree[dev].pop_back();
            // the word keeps the last tag its previous owner saw: continue from there, never reuse a tag
            s.seq = (uint32_t)(__atomic_load_n(s.host, __ATOMIC_ACQUIRE) >> 32);
        } else {
            void* p = nullptr;
            if (hipHostMalloc(&p, 64, hipHostMallocMapped | hipHostMallocPortable) != hipSuccess || !p) {
                (void)hipGetLastError();
                s.failed = true;
            } else {
                s.host = static_cast<unsigned long long*>(p);
                *s.host = 0;
                g_signalAll.push_back(s.host);
            }
        }
    }
    return s.host ? &s : nullptr;
}

inline void cpu_relax()
{
#if defined(__x86_64__) || defined(__i386__)
    __builtin_ia32_pause();
#endif
}

// Waits until the word carries `seq` and returns the count; gives up (false) as soon as the stream has
// drained without the word arriving or reports an error, so the wait always ends with the stream.
bool poll_host_signal(const HostSignal& s, uint32_t seq, hipStream_t stream, int32_t* count, hipError_t* err)
{
    *err = hipSuccess;
    // Back-off: the count normally arrives within a few microseconds, so the first reads only pause the core;
    // behind a long queue the thread yields between reads instead of burning its core.
    for (uint32_t spins = 1;; ++spins) {
        const unsigned long long v = __atomic_load_n(s.host, __ATOMIC_ACQUIRE);
        if ((uint32_t)(v >> 32) == seq) {
            *count = (int32_t)(uint32_t)v;
            return true;
        }
        if (spins < 4096u) cpu_relax();
        else sched_yield();
        if ((spins & 255u) == 0) {
            const hipError_t q = hipStreamQuery(stream);
            if (q == hipErrorNotReady) {
                (void)hipGetLastError();
                continue;
            }
            if (q != hipSuccess) {
                *err = q;
                return false;
            }
            // the stream is idle: the store has been issued; look once more, then leave it to a copy
            const unsigned long long w = __atomic_load_n(s.host, __ATOMIC_ACQUIRE);
            if ((uint32_t)(w >> 32) == seq) {
                *count = (int32_t)(uint32_t)w;
                return true;
            }
            return false;
        }
    }
}

// Limits the reference leaves unchecked.  Indices are int16 triples, so n, bh and bw must fit.
bool geom_ok(int N, int H, int W, int C, const int32_t* bsize, const int32_t* bstride)
{
    return N > 0 && H > 0 && W > 0 && C > 0 && bsize[0] > 0 && bsize[1] > 0 && bstride[0] > 0 &&
           bstride[1] > 0 && (int64_t)N * H * W * C < (1ll << 40);
}

sbnet::Geom make_geom(int N, int H, int W, int C, const int32_t* bsize, const int32_t* bstride,
                      const int32_t* boffset)
{
    sbnet::Geom g;
    g.N = N; g.H = H; g.W = W; g.C = C;
    g.R = bsize[0]; g.S = bsize[1];
    g.U = bstride[0]; g.V = bstride[1];
    g.oh = boffset[0]; g.ow = boffset[1];
    g.countDev = nullptr;
    g.forceGeneric = t_forceGeneric;
    return g;
}

bool dims_fit_int(const int64_t* d)
{
    for (int i = 0; i < 4; ++i)
        if (d[i] < 0 || d[i] > 0x7fffffffll) return false;
    return true;
}

int reduce_mask_impl(const float* mask, int N, int H, int W, const int32_t* bcount,
                     const int32_t* bsize, const int32_t* bstride, const int32_t* boffset, float tol,
                     int avgpool, bool fixup, int16_t* idx, int32_t* countHost, int32_t* countDev,
                     void* workspace, size_t workspaceBytes, hipStream_t stream)
{
    if (!mask || !idx || (!countHost && !countDev)) return SBNET_EINVAL_ARG;
    if (!geom_ok(N, H, W, 1, bsize, bstride)) return SBNET_EINVAL_ARG;
    if (bcount[0] <= 0 || bcount[1] <= 0) return SBNET_EINVAL_ARG;
    // (n, bh, bw) are stored as int16
    if (N > 32768 || bcount[0] > 32768 || bcount[1] > 32768) return SBNET_EINVAL_ARG;
    const int64_t T = (int64_t)N * bcount[0] * bcount[1];
    if (T >= (1ll << 31)) return SBNET_EINVAL_ARG;
    // block origins and ends must stay inside int arithmetic
    const int64_t hEnd = (int64_t)boffset[0] + (int64_t)bstride[0] * (bcount[0] - 1) + bsize[0];
    const int64_t wEnd = (int64_t)boffset[1] + (int64_t)bstride[1] * (bcount[1] - 1) + bsize[1];
    if (hEnd > 0x7fffffffll || wEnd > 0x7fffffffll || (int64_t)bsize[0] * bsize[1] > 0x7fffffffll)
        return SBNET_EINVAL_ARG;

    const size_t need = sbnet::reduce_mask_workspace_bytes(T);
    void* ws = workspace;
    bool ownWs = false;
    if (ws && (workspaceBytes < need || (reinterpret_cast<uintptr_t>(ws) & 15))) return SBNET_EINVAL_ARG;
    // Neither a host-visible count (nothing runs during capture) nor a scratch buffer of the library's own
    // (allocating and freeing it synchronises) can be had while the stream is being captured: refuse before
    // anything is allocated or enqueued, so the capture stays valid.
    bool capturing = false;
    if (countHost || !ws) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();  // (cannot be asked: not capturing)
        else capturing = cap != hipStreamCaptureStatusNone;
        if (capturing) return hip_fail(hipErrorStreamCaptureUnsupported);
    }
    if (!ws) {
        SBNET_HIP(hipMalloc(&ws, need));
        ownWs = true;
    }
    const sbnet::Geom g = make_geom(N, H, W, 1, bsize, bstride, boffset);
    HostSignal* sig = nullptr;
    uint32_t seq = 0;
    if (countHost) {
        sig = host_signal();
        if (sig) {
            seq = ++sig->seq;
            if (seq == 0) seq = ++sig->seq;  // 0 is the word's initial tag
        }
    }
    hipError_t e = sbnet::launch_reduce_mask(mask, g, bcount[0], bcount[1], tol, avgpool != 0, fixup, idx,
                                             countDev, ws, stream, sig ? sig->host : nullptr, seq);
    bool haveCount = false;
    if (e == hipSuccess && sig) haveCount = poll_host_signal(*sig, seq, stream, countHost, &e);
    if (e == hipSuccess && countHost && !haveCount) {
        // the count sits in countDev, or in the workspace
        const int32_t* src = countDev ? countDev : sbnet::reduce_mask_count_slot(ws, T);
        e = hipMemcpyAsync(countHost, src, sizeof(int32_t), hipMemcpyDeviceToHost, stream);
        if (e == hipSuccess) e = hipStreamSynchronize(stream);
    }
    if (ownWs) {
        hipError_t e2 = hipStreamSynchronize(stream);
        hipError_t e3 = hipFree(ws);
        if (e == hipSuccess) e = e2 != hipSuccess ? e2 : e3;
    }
    if (e != hipSuccess) return hip_fail(e);
    return SBNET_OK;
}

int gather_impl(const float* x, int N, int H, int W, int C, float* y, const int32_t* bsize, const int32_t* bstride,
                const int32_t* boffset, int numActive, const int32_t* countDev, const int16_t* idx, int transpose,
                hipStream_t stream)
{
    if (numActive < 0) return SBNET_EINVAL_ARG;
    if (numActive > 0 && (!x || !y || !idx)) return SBNET_EINVAL_ARG;
    if (!geom_ok(N, H, W, C, bsize, bstride)) return SBNET_EINVAL_ARG;
    sbnet::Geom g = make_geom(N, H, W, C, bsize, bstride, boffset);
    g.countDev = countDev;
    SBNET_HIP(sbnet::launch_gather(x, y, idx, numActive, g, transpose != 0, stream));
    return SBNET_OK;
}

int scatter_impl(const float* x, int32_t numActive, const int32_t* countDev, const int16_t* idx, float* out,
                 const int64_t* dims, const int32_t* bsize, const int32_t* bstride,
                 const int32_t* boffset, int add, int atomic, int transpose, void* workspace,
                 size_t workspaceBytes, hipStream_t stream)
{
    if (numActive < 0) return SBNET_EINVAL_ARG;
    if (numActive > 0 && (!x || !idx)) return SBNET_EINVAL_ARG;
    if (!out || !dims_fit_int(dims)) return SBNET_EINVAL_ARG;
    if (!geom_ok((int)dims[0], (int)dims[1], (int)dims[2], (int)dims[3], bsize, bstride))
        return SBNET_EINVAL_ARG;
    sbnet::Geom g = make_geom((int)dims[0], (int)dims[1], (int)dims[2], (int)dims[3], bsize, bstride, boffset);
    g.countDev = countDev;
    const sbnet::ScatterMode mode =
        !add ? sbnet::SCATTER_ASSIGN : (atomic ? sbnet::SCATTER_ATOMIC : sbnet::SCATTER_ADD);
    if (mode == sbnet::SCATTER_ATOMIC && workspace) {
        // with scratch an "atomic" add needs no atomics: the owner-computes kernel where it applies (NHWC stack,
        // at most 2x2 blocks per pixel; exact sequential order), else passes of plain adds over non-overlapping
        // classes of blocks
        bool done = false;
        if (!transpose)
            SBNET_HIP(sbnet::launch_scatter_pull(x, out, idx, numActive, g, workspace, workspaceBytes, stream, done));
        if (done) return SBNET_OK;
        SBNET_HIP(sbnet::launch_scatter_colored(x, out, idx, numActive, g, transpose != 0, workspace, workspaceBytes,
                                                stream, done));
        if (done) return SBNET_OK;
    }
    if (mode == sbnet::SCATTER_ASSIGN) {
        // overlapping plain writes land in the CPU functor's order (the block listed last wins): decided inside the
        // planar kernel where that applies, else with scratch (nothing is done here without scratch then)
        bool done = false;
        SBNET_HIP(sbnet::launch_scatter_owned(x, out, idx, numActive, g, transpose != 0, workspace, workspaceBytes,
                                              stream, done));
        if (done) return SBNET_OK;
    }
    SBNET_HIP(sbnet::launch_scatter(x, out, idx, numActive, g, transpose != 0, mode, stream));
    return SBNET_OK;
}

// Library-managed scratch for callers without an allocator at hand (sbnet_scratch_acquire): one grow-only buffer
// per (device, stream).  Work on one stream runs in order, so consecutive calls on that stream may share it.
struct ScratchSlot {
    int dev;
    hipStream_t stream;
    void* ptr;
    size_t bytes;
};
std::mutex g_scratchMutex;
std::vector<ScratchSlot> g_scratch;
// Buffers that a slot has outgrown.  A caller may still hold such a pointer (it asked before another thread's
// larger request on the same stream) and work that uses it may still be queued, so nothing is freed before
// sbnet_shutdown.
std::vector<ScratchSlot> g_scratchRetired;

}  // namespace

extern "C" {

const char* sbnet_version(void) { return "sbnet_amd 0.1 (gfx950)"; }

int sbnet_last_hip_error(void) { return g_lastHipError; }

const char* sbnet_status_string(int status)
{
    switch (status) {
    case SBNET_OK: return "OK";
    case SBNET_EINVAL_PARAM_SHAPE:
        return "InvalidArgument: dynamic_b<count, size, stride, offset> should be one-dimensional with shape[0] == 2.";
    case SBNET_EINVAL_RANK: return "InvalidArgument: x / ybase must be rank 4";
    case SBNET_EINVAL_OVERLAP:
        return "InvalidArgument: Only non-overlapping blocks are supported with add=True, atomic=False";
    case SBNET_EINVAL_ARG: return "InvalidArgument: null pointer, size out of range or workspace too small";
    case SBNET_EHIP: return "HIP runtime error (see sbnet_last_hip_error)";
    case SBNET_ETOOBIG:
        return "InvalidArgument: more blocks than the library's own scratch holds (sbnet_reduce_mask_static_max_indices); "
               "use sbnet_reduce_mask with a workspace";
    default: return "unknown sbnet status";
    }
}

int64_t sbnet_reduce_mask_max_indices(int N, const int32_t* bcount, int bcount_len)
{
    if (!pair_ok(bcount, bcount_len) || N < 0 || bcount[0] < 0 || bcount[1] < 0) return -1;
    return (int64_t)N * bcount[0] * bcount[1];
}

size_t sbnet_reduce_mask_workspace_bytes(int N, const int32_t* bcount, int bcount_len)
{
    const int64_t T = sbnet_reduce_mask_max_indices(N, bcount, bcount_len);
    if (T < 0) return 0;
    return sbnet::reduce_mask_workspace_bytes(T);
}

int sbnet_reduce_mask(const float* mask, int N, int H, int W, const int32_t* bcount, int bcount_len,
                      const int32_t* bsize, int bsize_len, const int32_t* bstride, int bstride_len,
                      const int32_t* boffset, int boffset_len, float tol, int avgpool,
                      int16_t* active_block_indices, int32_t* bin_counts_host,
                      int32_t* bin_counts_device, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!pair_ok(bcount, bcount_len) || !pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) ||
        !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    return reduce_mask_impl(mask, N, H, W, bcount, bsize, bstride, boffset, tol, avgpool, true,
                            active_block_indices, bin_counts_host, bin_counts_device, workspace,
                            workspace_bytes, static_cast<hipStream_t>(stream));
}

int sbnet_reduce_mask_static(const float* mask, int N, int H, int W, const int32_t* bcount, int bcount_len,
                             const int32_t* bsize, int bsize_len, const int32_t* bstride, int bstride_len,
                             const int32_t* boffset, int boffset_len, float tol, int avgpool,
                             int16_t* active_block_indices, int32_t* bin_counts_device, void* stream)
{
    if (!pair_ok(bcount, bcount_len) || !pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) ||
        !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    if (!bin_counts_device) return SBNET_EINVAL_ARG;
    // what sbnet_reduce_mask rejects as an argument error is one here too; SBNET_ETOOBIG is for valid sizes only
    if (N <= 0 || bcount[0] <= 0 || bcount[1] <= 0 || N > 32768 || bcount[0] > 32768 || bcount[1] > 32768)
        return SBNET_EINVAL_ARG;
    const int64_t T = (int64_t)N * bcount[0] * bcount[1];
    if (T >= (1ll << 31)) return SBNET_EINVAL_ARG;
    if (sbnet::reduce_mask_workspace_bytes(T) > sbnet::STATIC_SCRATCH_BYTES) return SBNET_ETOOBIG;
    void* ws = nullptr;
    SBNET_HIP(sbnet::static_scratch(&ws));
    return reduce_mask_impl(mask, N, H, W, bcount, bsize, bstride, boffset, tol, avgpool, true, active_block_indices,
                            nullptr, bin_counts_device, ws, sbnet::STATIC_SCRATCH_BYTES,
                            static_cast<hipStream_t>(stream));
}

int64_t sbnet_reduce_mask_static_max_indices(void)
{
    // the largest T with reduce_mask_workspace_bytes(T) <= STATIC_SCRATCH_BYTES
    int64_t lo = 0, hi = (int64_t)sbnet::STATIC_SCRATCH_BYTES;
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) / 2;
        if (sbnet::reduce_mask_workspace_bytes(mid) <= sbnet::STATIC_SCRATCH_BYTES) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

int sbnet_reduce_mask_functor(const float* mask, int N, int H, int W, float threshold, int bOffsH0,
                              int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int bCntH,
                              int bCntW, unsigned int numBins, unsigned int binSize,
                              int16_t* activeBlockIndices, int32_t* binCounts, int avgPool,
                              void* workspace, size_t workspace_bytes, void* stream)
{
    (void)binSize;
    if (numBins != 1 || !binCounts) return SBNET_EINVAL_ARG;  // reduce_mask.cc:69 asserts numBins == 1
    const int32_t bcount[2] = {bCntH, bCntW}, bsize[2] = {bSzH, bSzW}, bstride[2] = {bStrH, bStrW},
                  boffset[2] = {bOffsH0, bOffsW0};
    return reduce_mask_impl(mask, N, H, W, bcount, bsize, bstride, boffset, threshold, avgPool, false,
                            activeBlockIndices, nullptr, binCounts, workspace, workspace_bytes,
                            static_cast<hipStream_t>(stream));
}

int sbnet_sparse_gather(const float* x, const int64_t* x_dims, int x_rank, int32_t num_active,
                        const int16_t* active_block_indices, const int32_t* bsize, int bsize_len,
                        const int32_t* bstride, int bstride_len, const int32_t* boffset,
                        int boffset_len, int transpose, float* y, void* stream)
{
    if (x_rank != 4) return SBNET_EINVAL_RANK;  // sparse_gather.cc:164
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;  // sparse_gather.cc:169-175
    if (!x_dims || !dims_fit_int(x_dims)) return SBNET_EINVAL_ARG;
    return sbnet_sparse_gather_functor(x, (int)x_dims[0], (int)x_dims[1], (int)x_dims[2], (int)x_dims[3], y,
                                       boffset[0], boffset[1], bsize[0], bsize[1], bstride[0], bstride[1],
                                       num_active, active_block_indices, transpose, stream);
}

int sbnet_sparse_gather_functor(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                                int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int numActive,
                                const int16_t* activeBlockIndices, int transpose, void* stream)
{
    const int32_t bsize[2] = {bSzH, bSzW}, bstride[2] = {bStrH, bStrW}, boffset[2] = {bOffsH0, bOffsW0};
    return gather_impl(x, N, H, W, C, y, bsize, bstride, boffset, numActive, nullptr, activeBlockIndices, transpose,
                       static_cast<hipStream_t>(stream));
}

int sbnet_sparse_gather_device_count(const float* x, const int64_t* x_dims, int x_rank,
                                     const int32_t* bin_counts_device, int32_t max_active,
                                     const int16_t* active_block_indices, const int32_t* bsize, int bsize_len,
                                     const int32_t* bstride, int bstride_len, const int32_t* boffset,
                                     int boffset_len, int transpose, float* y, void* stream)
{
    if (x_rank != 4) return SBNET_EINVAL_RANK;
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    if (!x_dims || !dims_fit_int(x_dims) || !bin_counts_device) return SBNET_EINVAL_ARG;
    return gather_impl(x, (int)x_dims[0], (int)x_dims[1], (int)x_dims[2], (int)x_dims[3], y, bsize, bstride, boffset,
                       max_active, bin_counts_device, active_block_indices, transpose,
                       static_cast<hipStream_t>(stream));
}

size_t sbnet_sparse_scatter_workspace_bytes(int32_t num_active, const int64_t* ybase_dims, int ybase_rank,
                                            const int32_t* bsize, int bsize_len, const int32_t* bstride,
                                            int bstride_len, const int32_t* boffset, int boffset_len)
{
    if (ybase_rank != 4 || !ybase_dims || !dims_fit_int(ybase_dims) || num_active <= 0) return 0;
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len)) return 0;
    if (!geom_ok((int)ybase_dims[0], (int)ybase_dims[1], (int)ybase_dims[2], (int)ybase_dims[3], bsize, bstride))
        return 0;
    const sbnet::Geom g = make_geom((int)ybase_dims[0], (int)ybase_dims[1], (int)ybase_dims[2], (int)ybase_dims[3],
                                    bsize, bstride, boffset);
    const size_t pull = sbnet::scatter_pull_workspace_bytes(g, num_active);
    const size_t color = sbnet::scatter_color_workspace_bytes(g, num_active);
    const size_t cover = sbnet::scatter_cover_workspace_bytes(g, num_active);
    const size_t owner = sbnet::scatter_owner_workspace_bytes(g, num_active);
    size_t m = pull > color ? pull : color;
    if (cover > m) m = cover;
    return owner > m ? owner : m;
}

static int scatter_op(const float* x, int32_t num_active, const int32_t* bin_counts_device,
                      const int16_t* active_block_indices, const float* ybase, const int64_t* ybase_dims,
                      int ybase_rank, const int32_t* bsize, int bsize_len, const int32_t* bstride, int bstride_len,
                      const int32_t* boffset, int boffset_len, int add, int atomic, int transpose, float* y,
                      void* workspace, size_t workspace_bytes, void* stream)
{
    // order of checks as in sparse_gather.cc:307-327
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    if (!atomic && add && !(bstride[0] >= bsize[0] && bstride[1] >= bsize[1])) return SBNET_EINVAL_OVERLAP;
    if (ybase_rank != 4) return SBNET_EINVAL_RANK;
    if (!ybase || !y || !ybase_dims || !dims_fit_int(ybase_dims)) return SBNET_EINVAL_ARG;
    const size_t count = (size_t)ybase_dims[0] * ybase_dims[1] * ybase_dims[2] * ybase_dims[3];
    {
        const uintptr_t a = reinterpret_cast<uintptr_t>(ybase), b = reinterpret_cast<uintptr_t>(y);
        const uintptr_t bytes = count * sizeof(float);
        if (a < b + bytes && b < a + bytes) return SBNET_EINVAL_ARG;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!geom_ok((int)ybase_dims[0], (int)ybase_dims[1], (int)ybase_dims[2], (int)ybase_dims[3], bsize, bstride))
        return SBNET_EINVAL_ARG;
    // With scratch for one flag byte per pixel the output is built in one pass over its bytes: uncovered pixels
    // are copied, covered ones written by the scatter (which reads ybase where it adds).
    if (num_active > 0 && x && active_block_indices && !(add && atomic)) {
        sbnet::Geom g = make_geom((int)ybase_dims[0], (int)ybase_dims[1], (int)ybase_dims[2], (int)ybase_dims[3], bsize,
                                  bstride, boffset);
        g.countDev = bin_counts_device;
        bool done = false;
        SBNET_HIP(sbnet::launch_scatter_over_base(x, ybase, y, active_block_indices, num_active, g, transpose != 0,
                                                  add ? sbnet::SCATTER_ADD : sbnet::SCATTER_ASSIGN, workspace,
                                                  workspace_bytes, s, done));
        if (done) return SBNET_OK;
    }
    SBNET_HIP(sbnet::launch_copy(y, ybase, count, s));  // sparse_gather.cc:338-346, no stream sync
    return scatter_impl(x, num_active, bin_counts_device, active_block_indices, y, ybase_dims, bsize, bstride, boffset,
                        add, atomic, transpose, workspace, workspace_bytes, s);
}

int sbnet_sparse_scatter(const float* x, int32_t num_active, const int16_t* active_block_indices,
                         const float* ybase, const int64_t* ybase_dims, int ybase_rank,
                         const int32_t* bsize, int bsize_len, const int32_t* bstride, int bstride_len,
                         const int32_t* boffset, int boffset_len, int add, int atomic, int transpose,
                         float* y, void* workspace, size_t workspace_bytes, void* stream)
{
    return scatter_op(x, num_active, nullptr, active_block_indices, ybase, ybase_dims, ybase_rank, bsize, bsize_len,
                      bstride, bstride_len, boffset, boffset_len, add, atomic, transpose, y, workspace,
                      workspace_bytes, stream);
}

int sbnet_sparse_scatter_device_count(const float* x, const int32_t* bin_counts_device, int32_t max_active,
                                      const int16_t* active_block_indices, const float* ybase,
                                      const int64_t* ybase_dims, int ybase_rank, const int32_t* bsize, int bsize_len,
                                      const int32_t* bstride, int bstride_len, const int32_t* boffset,
                                      int boffset_len, int add, int atomic, int transpose, float* y,
                                      void* workspace, size_t workspace_bytes, void* stream)
{
    if (!bin_counts_device) return SBNET_EINVAL_ARG;
    return scatter_op(x, max_active, bin_counts_device, active_block_indices, ybase, ybase_dims, ybase_rank, bsize,
                      bsize_len, bstride, bstride_len, boffset, boffset_len, add, atomic, transpose, y, workspace,
                      workspace_bytes, stream);
}

static int scatter_var_op(const float* x, int32_t num_active, const int32_t* bin_counts_device,
                          const int16_t* active_block_indices, float* ybase, const int64_t* ybase_dims,
                          int ybase_rank, const int32_t* bsize, int bsize_len, const int32_t* bstride,
                          int bstride_len, const int32_t* boffset, int boffset_len, int add, int atomic,
                          int transpose, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    if (!atomic && add && !(bstride[0] >= bsize[0] && bstride[1] >= bsize[1])) return SBNET_EINVAL_OVERLAP;
    if (ybase_rank != 4) return SBNET_EINVAL_RANK;
    if (!ybase || !ybase_dims) return SBNET_EINVAL_ARG;
    return scatter_impl(x, num_active, bin_counts_device, active_block_indices, ybase, ybase_dims, bsize, bstride,
                        boffset, add, atomic, transpose, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int sbnet_sparse_scatter_var(const float* x, int32_t num_active, const int16_t* active_block_indices,
                             float* ybase, const int64_t* ybase_dims, int ybase_rank,
                             const int32_t* bsize, int bsize_len, const int32_t* bstride,
                             int bstride_len, const int32_t* boffset, int boffset_len, int add,
                             int atomic, int transpose, void* workspace, size_t workspace_bytes,
                             void* stream)
{
    return scatter_var_op(x, num_active, nullptr, active_block_indices, ybase, ybase_dims, ybase_rank, bsize,
                          bsize_len, bstride, bstride_len, boffset, boffset_len, add, atomic, transpose, workspace,
                          workspace_bytes, stream);
}

int sbnet_sparse_scatter_var_device_count(const float* x, const int32_t* bin_counts_device, int32_t max_active,
                                          const int16_t* active_block_indices, float* ybase,
                                          const int64_t* ybase_dims, int ybase_rank, const int32_t* bsize,
                                          int bsize_len, const int32_t* bstride, int bstride_len,
                                          const int32_t* boffset, int boffset_len, int add, int atomic,
                                          int transpose, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!bin_counts_device) return SBNET_EINVAL_ARG;
    return scatter_var_op(x, max_active, bin_counts_device, active_block_indices, ybase, ybase_dims, ybase_rank,
                          bsize, bsize_len, bstride, bstride_len, boffset, boffset_len, add, atomic, transpose,
                          workspace, workspace_bytes, stream);
}

int sbnet_sparse_gather_grad(const float* dy, int32_t num_active, const int16_t* active_block_indices, float* dx,
                             const int64_t* x_dims, int x_rank, const int32_t* bsize, int bsize_len,
                             const int32_t* bstride, int bstride_len, const int32_t* boffset, int boffset_len,
                             int transpose, void* workspace, size_t workspace_bytes, void* stream)
{
    if (x_rank != 4) return SBNET_EINVAL_RANK;
    if (!pair_ok(bsize, bsize_len) || !pair_ok(bstride, bstride_len) || !pair_ok(boffset, boffset_len))
        return SBNET_EINVAL_PARAM_SHAPE;
    if (!dx || !x_dims || !dims_fit_int(x_dims) || num_active < 0) return SBNET_EINVAL_ARG;
    if (num_active > 0 && (!dy || !active_block_indices)) return SBNET_EINVAL_ARG;
    if (!geom_ok((int)x_dims[0], (int)x_dims[1], (int)x_dims[2], (int)x_dims[3], bsize, bstride)) return SBNET_EINVAL_ARG;
    const sbnet::Geom g = make_geom((int)x_dims[0], (int)x_dims[1], (int)x_dims[2], (int)x_dims[3], bsize, bstride, boffset);
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool done = false;
    SBNET_HIP(sbnet::launch_scatter_onto_zeros(dy, dx, active_block_indices, num_active, g, transpose != 0, workspace,
                                               workspace_bytes, s, done));
    if (done) return SBNET_OK;
    SBNET_HIP(sbnet::launch_scatter_colored(dy, dx, active_block_indices, num_active, g, transpose != 0, workspace,
                                            workspace_bytes, s, done, true));
    if (done) return SBNET_OK;
    // no scratch, or a geometry the passes do not take: zeros everywhere, then the atomic scatter-add
    SBNET_HIP(sbnet::launch_zero(dx, (size_t)x_dims[0] * x_dims[1] * x_dims[2] * x_dims[3], s));
    return scatter_impl(dy, num_active, nullptr, active_block_indices, dx, x_dims, bsize, bstride, boffset, 1, 1, transpose,
                        workspace, workspace_bytes, s);
}

int sbnet_sparse_scatter_functor(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                                 int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int numActive,
                                 const int16_t* activeBlockIndices, int add, int transpose, int atomic,
                                 void* stream)
{
    return sbnet_sparse_scatter_functor_ws(x, N, H, W, C, y, bOffsH0, bOffsW0, bSzH, bSzW, bStrH, bStrW, numActive,
                                           activeBlockIndices, add, transpose, atomic, nullptr, 0, stream);
}

int sbnet_sparse_scatter_functor_ws(const float* x, int N, int H, int W, int C, float* y, int bOffsH0,
                                    int bOffsW0, int bSzH, int bSzW, int bStrH, int bStrW, int numActive,
                                    const int16_t* activeBlockIndices, int add, int transpose, int atomic,
                                    void* workspace, size_t workspace_bytes, void* stream)
{
    const int32_t bsize[2] = {bSzH, bSzW}, bstride[2] = {bStrH, bStrW}, boffset[2] = {bOffsH0, bOffsW0};
    const int64_t dims[4] = {N, H, W, C};
    return scatter_impl(x, numActive, nullptr, activeBlockIndices, y, dims, bsize, bstride, boffset, add, atomic,
                        transpose, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

void* sbnet_scratch_acquire(size_t bytes, void* stream)
{
    if (bytes == 0) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    ScratchSlot* slot = nullptr;
    for (ScratchSlot& c : g_scratch)
        if (c.dev == dev && c.stream == s) slot = &c;
    if (slot && slot->bytes >= bytes) return slot->ptr;
    // growing allocates, which a stream under capture must not do
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
        (void)hipGetLastError();  // a stream that cannot be asked is not being captured
        cap = hipStreamCaptureStatusNone;
    }
    if (cap != hipStreamCaptureStatusNone) return nullptr;
    size_t want = (size_t)1 << 20;
    while (want < bytes) want <<= 1;
    void* p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess || !p) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (slot) {
        g_scratchRetired.push_back(*slot);  // may still be handed out or in use by queued work: kept until shutdown
        slot->ptr = p;
        slot->bytes = want;
    } else {
        g_scratch.push_back(ScratchSlot{dev, s, p, want});
    }
    return p;
}

int sbnet_shutdown(void)
{
    hipError_t first = hipSuccess;
    {
        std::lock_guard<std::mutex> lock(g_scratchMutex);
        for (std::vector<ScratchSlot>* list : {&g_scratch, &g_scratchRetired}) {
            for (ScratchSlot& c : *list) {
                int cur = 0;
                (void)hipGetDevice(&cur);
                (void)hipSetDevice(c.dev);
                hipError_t e = hipFree(c.ptr);  // waits for the device
                (void)hipSetDevice(cur);
                if (e != hipSuccess && first == hipSuccess) first = e;
            }
            list->clear();
        }
    }
    {
        // only the words no thread holds; a live thread keeps its own until it ends
        std::lock_guard<std::mutex> lock(g_signalMutex);
        for (int d = 0; d < MAX_SIGNAL_DEVICES; ++d) {
            for (unsigned long long* w : g_signalFree[d]) {
                hipError_t e = hipHostFree(w);
                if (e != hipSuccess && first == hipSuccess) first = e;
                for (size_t i = 0; i < g_signalAll.size(); ++i)
                    if (g_signalAll[i] == w) {
                        g_signalAll[i] = g_signalAll.back();
                        g_signalAll.pop_back();
                        break;
                    }
            }
            g_signalFree[d].clear();
        }
    }
    if (first != hipSuccess) return hip_fail(first);
    return SBNET_OK;
}

// Test hook, not part of the public header: while on (per calling thread), gather and scatter never take a
// kernel instance compiled for one block shape, so the tests cover the run-time-geometry kernels on the
// benchmark shapes as well.  Returns the previous setting.
int sbnet_test_force_generic(int on)
{
    const int prev = t_forceGeneric;
    t_forceGeneric = on ? 1 : 0;
    return prev;
}

// Test hook, not part of the public header: the tile the planar kernels would choose (no device work, so the
// choice can be checked on a machine without a GPU).  out must hold 11 int32; see sbnet::tile_choice.
int sbnet_test_tile_choice(int kind, int N, int H, int W, int C, int R, int S, int U, int V, int num_active, int vec,
                           int y_aligned_to, int32_t* out)
{
    const int32_t bsize[2] = {R, S}, bstride[2] = {U, V}, boffset[2] = {0, 0};
    if (!out || !geom_ok(N, H, W, C, bsize, bstride)) return -1;
    return sbnet::tile_choice(kind, make_geom(N, H, W, C, bsize, bstride, boffset), num_active, vec, y_aligned_to, out);
}

int sbnet_copy_tensor(float* dst, const float* src, size_t count, void* stream)
{
    if (count && (!dst || !src)) return SBNET_EINVAL_ARG;
    SBNET_HIP(sbnet::launch_copy(dst, src, count, static_cast<hipStream_t>(stream)));
    return SBNET_OK;
}

int sbnet_timer_start(void* stream, int64_t* start_event)
{
    if (!start_event) return SBNET_EINVAL_ARG;
    hipEvent_t ev;
    SBNET_HIP(hipEventCreate(&ev));
    hipError_t e = hipEventRecord(ev, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) {
        (void)hipEventDestroy(ev);
        return hip_fail(e);
    }
    *start_event = (int64_t)reinterpret_cast<intptr_t>(ev);
    return SBNET_OK;
}

int sbnet_timer_end(int64_t start_event, void* stream, float* dt_ms)
{
    if (!start_event || !dt_ms) return SBNET_EINVAL_ARG;
    hipEvent_t start = reinterpret_cast<hipEvent_t>((intptr_t)start_event);
    hipEvent_t end;
    SBNET_HIP(hipEventCreate(&end));
    hipError_t e = hipEventRecord(end, static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipEventSynchronize(end);
    if (e == hipSuccess) e = hipEventElapsedTime(dt_ms, start, end);
    (void)hipEventDestroy(end);
    (void)hipEventDestroy(start);
    if (e != hipSuccess) return hip_fail(e);
    return SBNET_OK;
}

}  // extern "C"

// Internal runtime helpers shared by the .hip translation units: error capture, the caching
// device allocator behind zk_malloc/zk_free, and a pinned staging area for small results.
#pragma once
#include <memory>
#include <vector>
#include <cstddef>
#include <cstdint>
#include <string>
#include <hip/hip_runtime.h>

namespace zk {

enum : int {
    ZK_OK = 0,
    ZK_ERR_ARG = 10001,      // bad argument (shape mismatch, null pointer, size over a stated limit)
    ZK_ERR_NO_DEVICE = 10002,
    ZK_ERR_BLAS = 10003      // a rocBLAS call failed (the integer GEMMs of large matrix products)
};

void set_error(int code, const std::string& msg);
int hip_fail(hipError_t e, const char* what, const char* file, int line);

#define ZK_HIP(call)                                                        \
    do {                                                                    \
        hipError_t e__ = (call);                                            \
        if (e__ != hipSuccess) return zk::hip_fail(e__, #call, __FILE__, __LINE__); \
    } while (0)

#define ZK_ARG(cond, msg)                                                   \
    do {                                                                    \
        if (!(cond)) { zk::set_error(zk::ZK_ERR_ARG, msg); return zk::ZK_ERR_ARG; } \
    } while (0)

#define ZK_LAUNCH_CHECK() ZK_HIP(hipGetLastError())

// Caching allocator: blocks are kept on per-size free lists and reused; all work is assumed to
// run on one stream, so a block handed out again is ordered after its previous user.
int pool_alloc(void** out, size_t bytes);
int pool_free(void* p);
int pool_trim();

// RAII scratch from the pool for use inside one entry point.
struct Scratch {
    void* p = nullptr;
    int rc = 0;
    explicit Scratch(size_t bytes) { rc = pool_alloc(&p, bytes ? bytes : 1); }
    ~Scratch() { if (p) pool_free(p); }
    template <class T> T* as() const { return reinterpret_cast<T*>(p); }
    Scratch(const Scratch&) = delete;
    Scratch& operator=(const Scratch&) = delete;
};

// Device buffers of one job that may run on a stream of its own: all released together once that stream has drained,
// so none of them returns to the allocator while the job's kernels are pending.
struct Arena {
    std::vector<std::unique_ptr<Scratch>> v;
    Scratch& add(size_t bytes) { v.emplace_back(new Scratch(bytes)); return *v.back(); }
};
// One of the library's own streams (non-blocking, default priority), handed out round-robin; null on failure.
// Two pools, so that a short job (pool 1: sumchecks) never queues behind a long one (pool 0: openings).
hipStream_t side_stream(int pool);

// Pinned host buffers of 64 KiB for results that a job on a side stream copies out behind its last kernel, so that
// fetching them waits for that job alone (an event) and not for whatever was queued on the stream after it.
int pinned_acquire(void** host_ptr);
void pinned_release(void* host_ptr);

// Pinned host buffer (64 KiB) for device->host results of reductions.
int staging(void** host_ptr, size_t bytes);

// Looks up, for the current device, the address of the device array behind zk_fr_sum_static (fr_kernels.hip); called
// by zk_init so that the entry point itself has nothing left to set up.
int fr_static_scratch_setup();

static inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace zk

// Internal runtime helpers shared by the .hip translation units: error capture, the caching
// device allocator behind zk_malloc/zk_free, and a pinned staging area for small results.
#pragma once
#include <functional>
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
    ZK_ERR_NO_DEVICE = 10002
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

// Caching allocator: blocks are kept on per-size free lists and reused.  Every block remembers the stream its last user
// named when it was freed.  A block handed out for another stream makes that stream wait (an event recorded on the old
// stream at that moment covers everything queued there before the free) -- so reuse is ordered behind the previous user
// whatever streams the two run on.  Blocks freed as `idle` (their stream is known to have drained) need no wait.
// `also`: a second stream whose kernels will touch the block too (a job that runs on two streams); it is ordered as well.
int pool_alloc(void** out, size_t bytes, hipStream_t stream, const hipStream_t* also = nullptr);
int pool_free(void* p, hipStream_t stream, bool idle = false);
int pool_trim();

// RAII scratch from the pool for use inside one entry point; `stream` is the stream the entry point's kernels run on.
struct Scratch {
    void* p = nullptr;
    int rc = 0;
    hipStream_t st = nullptr;
    bool idle_on_free = false;      // set when the owner has synchronised the stream before releasing
    Scratch(size_t bytes, hipStream_t stream, const hipStream_t* also = nullptr) : st(stream) { rc = pool_alloc(&p, bytes ? bytes : 1, stream, also); }
    ~Scratch() { if (p) pool_free(p, st, idle_on_free); }
    template <class T> T* as() const { return reinterpret_cast<T*>(p); }
    Scratch(const Scratch&) = delete;
    Scratch& operator=(const Scratch&) = delete;
};

// Device buffers of one job that may run on a stream of its own: all released together, tagged with the job's stream (or
// as idle once the owner has waited for that stream), so none of them reaches another stream's kernels early.
struct Arena {
    hipStream_t st = nullptr;       // set before the first add(); blocks are released as last used on this stream
    hipStream_t st2 = nullptr;      // a job's second stream, when it has one: its work must have joined `st` before release
    bool two = false;
    std::vector<std::unique_ptr<Scratch>> v;
    Arena() = default;
    explicit Arena(hipStream_t stream) : st(stream) {}
    void streams(hipStream_t a, hipStream_t b) { st = a; st2 = b; two = (a != b); }
    Scratch& add(size_t bytes) { v.emplace_back(new Scratch(bytes, st, two ? &st2 : nullptr)); return *v.back(); }
    void mark_idle() { for (auto& s : v) s->idle_on_free = true; }
};
// One of the library's own streams (non-blocking, default priority), handed out round-robin; null on failure.
// Two pools, so that a short job (pool 1: sumchecks) never queues behind a long one (pool 0: openings).
hipStream_t side_stream(int pool);

// Pinned host buffers of 64 KiB for results that a job on a side stream copies out behind its last kernel, so that
// fetching them waits for that job alone (an event) and not for whatever was queued on the stream after it.
int pinned_acquire(void** host_ptr);
void pinned_release(void* host_ptr);

// Pinned host buffer (64 KiB, one per host thread) for device->host results of reductions.
int staging(void** host_ptr, size_t bytes);

// Small results of an entry point (a few field elements: sums, round polynomials) on their way to the host.
// Normally: copied through the staging buffer, the stream waited for, host_dst filled; the first n_mont elements multiplied by
// 2^256 mod r there (sums that left the device with a factor R^-1).  While the calling thread has a batch of deferred results
// open (zk_defer_begin): the copy goes into the batch's pinned buffer behind what is queued on the stream, nothing is waited for,
// host_dst is NOT written, and zk_defer_wait hands the values out later, in the order of the deliver calls.
int deliver(hipStream_t st, const void* dev_src, void* host_dst, size_t count_fr, int n_mont);

// Looks up, for the current device, the address of the device array behind zk_fr_sum_static (fr_kernels.hip); called
// by zk_init so that the entry point itself has nothing left to set up.
int fr_static_scratch_setup();

// fn is called by zk_shutdown (device idle, before the cached blocks are given back): a file drops the events and cached
// buffers it holds in static objects
void at_shutdown(void (*fn)());

// The allocator is told that `to` now waits for everything queued on `from` so far (the caller has just recorded an event on
// `from` and made `to` wait for it): blocks that `from` let go before this call need no further wait when `to` takes them.
void pool_note_wait(hipStream_t from, hipStream_t to);

// The library's launch thread: closures run there one after the other, in the order of their submission, with the
// submitting thread's device current.  A job that is a long sequence of launches on a stream of its own hands that sequence
// over and returns to its caller at once; whoever collects the job waits for its ticket first.  Off with ZKLLM_ASYNC_JOBS=0
// (launcher_enabled() is false then and the caller runs the closure itself).  Error text set inside a closure belongs to the
// launch thread: a closure that can fail takes it along with last_error_text().
bool launcher_enabled();
void launcher_set_enabled(bool on);
uint64_t launcher_submit(std::function<void()> fn);
void launcher_wait(uint64_t ticket);      // 0: nothing to wait for
void launcher_stop();                     // runs what is queued, then ends the thread (it starts again on demand)
std::string last_error_text();

static inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace zk
